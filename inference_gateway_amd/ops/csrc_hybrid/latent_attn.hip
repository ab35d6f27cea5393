// Absorbed latent attention over a paged cache (gfx950).
//
// Each cached token is ONE row (latent c_j [R] | rotated shared key kr_j
// [RD]) read by every head.  For query row t (position p, sequence s) and
// head h:
//
//   score_j = (q_abs[t,h] . c_j + q_rot[t,h] . kr_j) * scale,
//             max(0, p - window + 1) <= j <= p        (window 0: from 0)
//   out[t,h] = sum_j softmax_j(score ; sink_h) c_j    [R]
//
// where the softmax denominator additionally holds exp(sink_h): the sink is
// folded in as the INITIAL state of the online softmax (running max =
// sink, running sum = 1, accumulator = 0), i.e. a key with no value.
// Scores, probabilities and the accumulator are fp32.
//
// latent_attention_rows: one wave per (row, head); lanes are keys for the
// scores and latent entries for the weighted sum.  Works for any sizes;
// rows of a prompt portion and decoded rows look the same to it (each row
// carries its own position and sequence).
#include "act_types.h"

namespace igw {

template <typename T, int NACC>
__global__ __launch_bounds__(64) void latent_attention_rows_kernel(
    T* __restrict__ out, const T* __restrict__ q_abs, int64_t qa_s0,
    int64_t qa_s1, const T* __restrict__ q_rot, int64_t qr_s0, int64_t qr_s1,
    const T* __restrict__ cache, const int32_t* __restrict__ block_table,
    int max_blocks, const int32_t* __restrict__ row_seq,
    const int32_t* __restrict__ positions, const float* __restrict__ sink,
    float scale, int window, int H, int R, int RD, int block_size) {
  extern __shared__ float lds[];
  float* q = lds;                      // [R + RD], pre-scaled
  float* p_lds = lds + R + RD;         // [64]
  int32_t* row_lds = (int32_t*)(p_lds + 64);  // [64] physical cache rows
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int CW = R + RD;
  const int pos = positions[t];
  const int32_t* bt = block_table + (int64_t)row_seq[t] * max_blocks;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  for (int d = lane; d < R; d += 64)
    q[d] = Act<T>::ld(q_abs + t * qa_s0 + h * qa_s1 + d) * scale;
  for (int d = lane; d < RD; d += 64)
    q[R + d] = Act<T>::ld(q_rot + t * qr_s0 + h * qr_s1 + d) * scale;
  __syncthreads();
  float m = sink[h], l = 1.0f;
  float acc[NACC];
#pragma unroll
  for (int i = 0; i < NACC; ++i) acc[i] = 0.0f;
  for (int j0 = lo; j0 <= pos; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j <= pos;
    float s = -INFINITY;
    int32_t prow = 0;
    if (valid) {
      prow = bt[j / block_size] * block_size + j % block_size;
      const T* row = cache + (int64_t)prow * CW;
      float a = 0.0f;
      for (int d = 0; d < CW; ++d) a += q[d] * Act<T>::ld(row + d);
      s = a;
    }
    const float m_new = fmaxf(m, wave_reduce_max(s));
    const float corr = expf(m - m_new);
    const float p = valid ? expf(s - m_new) : 0.0f;
    l = l * corr + wave_reduce_sum(p);
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] *= corr;
    m = m_new;
    __syncthreads();
    p_lds[lane] = p;
    row_lds[lane] = prow;
    __syncthreads();
    const int n = min(64, pos - j0 + 1);
    for (int k = 0; k < n; ++k) {
      const float pk = p_lds[k];
      const T* row = cache + (int64_t)row_lds[k] * CW;
#pragma unroll
      for (int i = 0; i < NACC; ++i) {
        const int d = lane + 64 * i;
        if (d < R) acc[i] += pk * Act<T>::ld(row + d);
      }
    }
  }
  const float inv = 1.0f / l;
  T* o = out + ((int64_t)t * H + h) * R;
#pragma unroll
  for (int i = 0; i < NACC; ++i) {
    const int d = lane + 64 * i;
    if (d < R) Act<T>::st(o + d, acc[i] * inv);
  }
}

void latent_attention(torch::Tensor out, torch::Tensor q_abs,
                      torch::Tensor q_rot, torch::Tensor cache,
                      torch::Tensor block_table, torch::Tensor row_seq,
                      torch::Tensor positions, torch::Tensor sink,
                      double scale, int64_t window) {
  TORCH_CHECK(q_abs.is_cuda() && q_abs.dim() == 3 && q_abs.stride(2) == 1);
  TORCH_CHECK(q_rot.dim() == 3 && q_rot.stride(2) == 1 &&
              q_rot.dtype() == q_abs.dtype());
  const int T = q_abs.size(0), H = q_abs.size(1), R = q_abs.size(2);
  const int RD = q_rot.size(2);
  TORCH_CHECK(q_rot.size(0) == T && q_rot.size(1) == H);
  TORCH_CHECK(cache.is_contiguous() && cache.dim() == 3 &&
              cache.size(2) == R + RD && cache.dtype() == q_abs.dtype());
  TORCH_CHECK(out.is_contiguous() && out.dtype() == q_abs.dtype() &&
              out.numel() == (int64_t)T * H * R);
  TORCH_CHECK(block_table.dtype() == torch::kInt32 &&
              block_table.is_contiguous() && block_table.dim() == 2);
  TORCH_CHECK(row_seq.dtype() == torch::kInt32 && row_seq.numel() == T);
  TORCH_CHECK(positions.dtype() == torch::kInt32 && positions.numel() == T);
  TORCH_CHECK(sink.dtype() == torch::kFloat32 && sink.numel() == H);
  TORCH_CHECK(R <= 1024, "latent width above 1024 is not supported");
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  const size_t shmem = (size_t)(R + RD + 128) * sizeof(float);
  const int nacc = (R + 63) / 64;
#define LAUNCH_ROWS(NA)                                                       \
  hipLaunchKernelGGL(                                                         \
      (latent_attention_rows_kernel<act_t, NA>), dim3(T, H), dim3(64), shmem, \
      stream, (act_t*)out.data_ptr(), (const act_t*)q_abs.data_ptr(),         \
      (int64_t)q_abs.stride(0), (int64_t)q_abs.stride(1),                     \
      (const act_t*)q_rot.data_ptr(), (int64_t)q_rot.stride(0),               \
      (int64_t)q_rot.stride(1), (const act_t*)cache.data_ptr(),               \
      (const int32_t*)block_table.data_ptr(), (int)block_table.size(1),       \
      (const int32_t*)row_seq.data_ptr(),                                     \
      (const int32_t*)positions.data_ptr(), (const float*)sink.data_ptr(),    \
      (float)scale, (int)window, H, R, RD, (int)cache.size(1))
  IGW_DISPATCH_ACT(q_abs, {
    if (nacc <= 1) LAUNCH_ROWS(1);
    else if (nacc <= 2) LAUNCH_ROWS(2);
    else if (nacc <= 4) LAUNCH_ROWS(4);
    else if (nacc <= 8) LAUNCH_ROWS(8);
    else LAUNCH_ROWS(16);
  });
#undef LAUNCH_ROWS
  HIP_CHECK_KERNEL();
}

}  // namespace igw
