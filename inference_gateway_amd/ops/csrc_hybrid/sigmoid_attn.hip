// Windowed sigmoid attention over paged K/V caches (gfx950).  Keys are
// cached as [blocks, G, block, dk]; values transposed inside the page,
// [blocks, G, dv, block].
//
// For query row t (position p, sequence s), query head g (key/value head
// c = g / (H/G)) and key j, max(0, p - window + 1) <= j <= p (window 0: from
// 0):
//
//   w_g(j)  = sigmoid((q[t,g] . k_c(j)) * scale + dist_bias[min(p-j, ND-1), g])
//   m_h(j)  = sum_g talk[h, g] * w_g(j)                 (weights mixed
//                                                        across heads)
//   out[t,h] = sigmoid(gate[t,h]) * sum_j m_h(j) v_c'(j),  c' = h / (H/G)
//
// There is no normalisation over keys, so there is no running maximum and
// key tiles simply accumulate.  Scores, weights, the mixing and the
// accumulator are fp32.
//
// sigmoid_attention_rows: one 256-thread block per query row, keys in tiles
// of 32 — the threads first share the (head, key) scores, then the mixing,
// then own the output entries.  Works for any sizes and both activation
// types; rows of a prompt portion and decoded rows look the same to it
// (each row carries its own position and sequence, and reads its keys from
// the paged cache).
#include "act_types.h"

namespace igw {

constexpr int SA_BLOCK = 256;
constexpr int SA_KT = 32;

template <typename T, int NACC>
__global__ __launch_bounds__(SA_BLOCK) void sigmoid_attention_rows_kernel(
    T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ kcache,
    const T* __restrict__ vcache, const int32_t* __restrict__ block_table,
    int max_blocks, const int32_t* __restrict__ row_seq,
    const int32_t* __restrict__ positions, const float* __restrict__ dist_bias,
    int ND, const float* __restrict__ talk, const T* __restrict__ gate,
    int64_t gate_stride, float scale, int window, int H, int G, int DK, int DV,
    int block_size) {
  extern __shared__ float lds[];
  float* q_lds = lds;                        // [H*DK]
  float* talk_lds = q_lds + H * DK;          // [H*H]
  float* w_lds = talk_lds + H * H;           // [H][KT]
  float* m_lds = w_lds + H * SA_KT;          // [H][KT]
  int32_t* blk_lds = (int32_t*)(m_lds + H * SA_KT);  // [KT] page of a key
  int32_t* off_lds = blk_lds + SA_KT;                // [KT] row in the page
  const int t = blockIdx.x, tid = threadIdx.x;
  const int per = H / G;
  const int pos = positions[t];
  const int32_t* bt = block_table + (int64_t)row_seq[t] * max_blocks;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  for (int d = tid; d < H * DK; d += SA_BLOCK)
    q_lds[d] = Act<T>::ld(q + (int64_t)t * H * DK + d);
  for (int d = tid; d < H * H; d += SA_BLOCK) talk_lds[d] = talk[d];
  float acc[NACC];
#pragma unroll
  for (int i = 0; i < NACC; ++i) acc[i] = 0.0f;
  for (int j0 = lo; j0 <= pos; j0 += SA_KT) {
    const int n = min(SA_KT, pos - j0 + 1);
    __syncthreads();   // previous tile's readers are done (and q is there)
    if (tid < SA_KT) {
      const int j = j0 + tid;
      blk_lds[tid] = tid < n ? bt[j / block_size] : 0;
      off_lds[tid] = j % block_size;
    }
    __syncthreads();
    for (int idx = tid; idx < H * SA_KT; idx += SA_BLOCK) {
      const int g = idx / SA_KT, jj = idx % SA_KT;
      float w = 0.0f;
      if (jj < n) {
        const T* kr = kcache + (((int64_t)blk_lds[jj] * G + g / per) *
                                    block_size + off_lds[jj]) * DK;
        const float* qr = q_lds + g * DK;
        float a = 0.0f;
        for (int d = 0; d < DK; ++d) a += qr[d] * Act<T>::ld(kr + d);
        const int dist = min(pos - (j0 + jj), ND - 1);
        w = sigmoid_for<T>(a * scale + dist_bias[dist * H + g]);
      }
      w_lds[idx] = w;
    }
    __syncthreads();
    for (int idx = tid; idx < H * SA_KT; idx += SA_BLOCK) {
      const int h = idx / SA_KT, jj = idx % SA_KT;
      float m = 0.0f;
      for (int g = 0; g < H; ++g) m += talk_lds[h * H + g] * w_lds[g * SA_KT + jj];
      m_lds[idx] = m;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NACC; ++i) {
      const int o = tid + SA_BLOCK * i;
      if (o < H * DV) {
        const int h = o / DV, d = o % DV, c = h / per;
        float a = acc[i];
        for (int jj = 0; jj < n; ++jj) {
          const T* vr = vcache + (((int64_t)blk_lds[jj] * G + c) * DV + d) *
                                     block_size + off_lds[jj];
          a += m_lds[h * SA_KT + jj] * Act<T>::ld(vr);
        }
        acc[i] = a;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < NACC; ++i) {
    const int o = tid + SA_BLOCK * i;
    if (o < H * DV)
      Act<T>::st(out + (int64_t)t * H * DV + o,
                 acc[i] * sigmoid_for<T>(Act<T>::ld(gate + t * gate_stride + o)));
  }
}

void sigmoid_attention_check(torch::Tensor out, torch::Tensor q,
                             torch::Tensor kcache, torch::Tensor vcache,
                             torch::Tensor block_table, torch::Tensor row_seq,
                             torch::Tensor positions, torch::Tensor dist_bias,
                             torch::Tensor talk, torch::Tensor gate) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 2 && q.is_contiguous());
  TORCH_CHECK(talk.dim() == 2 && talk.size(0) == talk.size(1) &&
              talk.dtype() == torch::kFloat32 && talk.is_contiguous());
  TORCH_CHECK(kcache.is_contiguous() && kcache.dim() == 4 &&
              vcache.is_contiguous() && vcache.dim() == 4);
  const int64_t T = q.size(0), H = talk.size(0), G = kcache.size(1);
  const int64_t DK = kcache.size(3), DV = vcache.size(2);
  TORCH_CHECK(G >= 1 && H % G == 0 && q.size(1) == H * DK);
  TORCH_CHECK(vcache.size(0) == kcache.size(0) && vcache.size(1) == G &&
              vcache.size(3) == kcache.size(2));
  TORCH_CHECK(kcache.dtype() == q.dtype() && vcache.dtype() == q.dtype());
  TORCH_CHECK(out.is_contiguous() && out.dtype() == q.dtype() &&
              out.dim() == 2 && out.size(0) == T && out.size(1) == H * DV);
  TORCH_CHECK(gate.dim() == 2 && gate.stride(1) == 1 && gate.size(0) == T &&
              gate.size(1) == H * DV && gate.dtype() == q.dtype());
  TORCH_CHECK(dist_bias.dtype() == torch::kFloat32 &&
              dist_bias.is_contiguous() && dist_bias.dim() == 2 &&
              dist_bias.size(0) >= 1 && dist_bias.size(1) == H);
  TORCH_CHECK(block_table.dtype() == torch::kInt32 &&
              block_table.is_contiguous() && block_table.dim() == 2);
  TORCH_CHECK(row_seq.dtype() == torch::kInt32 && row_seq.numel() == T);
  TORCH_CHECK(positions.dtype() == torch::kInt32 && positions.numel() == T);
}

void sigmoid_attention(torch::Tensor out, torch::Tensor q,
                       torch::Tensor kcache, torch::Tensor vcache,
                       torch::Tensor block_table, torch::Tensor row_seq,
                       torch::Tensor positions, torch::Tensor dist_bias,
                       torch::Tensor talk, torch::Tensor gate, double scale,
                       int64_t window) {
  sigmoid_attention_check(out, q, kcache, vcache, block_table, row_seq,
                          positions, dist_bias, talk, gate);
  const int T = q.size(0), H = talk.size(0), G = kcache.size(1);
  const int DK = kcache.size(3), DV = vcache.size(2);
  TORCH_CHECK(H * DV <= SA_BLOCK * 32,
              "sigmoid_attention: heads * vdim above 8192");
  const size_t shmem =
      ((size_t)H * DK + (size_t)H * H + 2 * (size_t)H * SA_KT + 2 * SA_KT) *
      sizeof(float);
  TORCH_CHECK(shmem <= 64 * 1024, "sigmoid_attention: heads * dim too large");
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  const int nacc = (H * DV + SA_BLOCK - 1) / SA_BLOCK;
#define LAUNCH_SA(NA)                                                         \
  hipLaunchKernelGGL(                                                         \
      (sigmoid_attention_rows_kernel<act_t, NA>), dim3(T), dim3(SA_BLOCK),    \
      shmem, stream, (act_t*)out.data_ptr(), (const act_t*)q.data_ptr(),      \
      (const act_t*)kcache.data_ptr(), (const act_t*)vcache.data_ptr(),       \
      (const int32_t*)block_table.data_ptr(), (int)block_table.size(1),       \
      (const int32_t*)row_seq.data_ptr(),                                     \
      (const int32_t*)positions.data_ptr(),                                   \
      (const float*)dist_bias.data_ptr(), (int)dist_bias.size(0),             \
      (const float*)talk.data_ptr(), (const act_t*)gate.data_ptr(),           \
      (int64_t)gate.stride(0), (float)scale, (int)window, H, G, DK, DV,       \
      (int)kcache.size(2))
  IGW_DISPATCH_ACT(q, {
    if (nacc <= 1) LAUNCH_SA(1);
    else if (nacc <= 2) LAUNCH_SA(2);
    else if (nacc <= 4) LAUNCH_SA(4);
    else if (nacc <= 8) LAUNCH_SA(8);
    else if (nacc <= 16) LAUNCH_SA(16);
    else LAUNCH_SA(32);
  });
#undef LAUNCH_SA
  HIP_CHECK_KERNEL();
}

}  // namespace igw
