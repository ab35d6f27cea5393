// Absorbed latent attention on the matrix cores (gfx950, bf16).
//
// Same contract as latent_attention_rows (latent_attn.hip); this kernel is
// the serving path for bf16.  Because every head reads the SAME cached row
// (latent | rotated key), heads are stacked into the M dimension of the MFMA
// tiles: a workgroup owns 64 (token row, head) pairs — TQ consecutive rows
// of one sequence times HB heads — and streams the keys those rows can see
// through LDS once, 32 keys at a time.  Prompt portions and single decoded
// tokens use the same kernel (a decoded token is a tile with one row).
//
// Per key tile, per wave (16 of the 64 pairs):
//   S  = Q . K^T        mfma 16x16x32 bf16, Q fragments held in registers,
//                       K tile row-major in LDS
//   online softmax in fp32 registers; the running max starts at the head's
//   sink and the running sum at 1 (the sink is a key without a value)
//   O += P . C          P through a per-wave LDS tile (C layout -> A
//                       layout), latents staged TRANSPOSED in LDS
// Sizes are runtime values; the register tiles are sized by the template
// (KS = 32-wide steps over latent+key width, NT = 16-wide output tiles) and
// loops are predicated on the runtime counts.
#include "act_types.h"

namespace igw {

typedef __attribute__((ext_vector_type(8))) short short8v;
typedef __attribute__((ext_vector_type(4))) float float4v;

constexpr int LA_BN = 32;        // keys per tile
constexpr int LA_PAD = 8;        // bf16 elements of row padding in LDS

template <int KS, int NT>
__global__ __launch_bounds__(256) void latent_attention_mfma_kernel(
    uint16_t* __restrict__ out, const uint16_t* __restrict__ q_abs,
    int64_t qa_s0, int64_t qa_s1, const uint16_t* __restrict__ q_rot,
    int64_t qr_s0, int64_t qr_s1, const uint16_t* __restrict__ cache,
    const int32_t* __restrict__ block_table, int max_blocks,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ tile_row0,
    const int32_t* __restrict__ tile_nrows, const float* __restrict__ sink,
    float scale, int window, int H, int R, int RD, int block_size, int HB) {
  extern __shared__ __attribute__((aligned(16))) uint16_t la_smem[];
  const int CW = R + RD;
  const int ks_n = (CW + 31) / 32;          // 32-wide steps actually used
  const int nt_n = (R + 15) / 16;           // 16-wide output tiles used
  const int krs = ks_n * 32 + LA_PAD;       // K tile row stride (elements)
  constexpr int crs = LA_BN + LA_PAD;       // CT / P row stride
  uint16_t* k_s = la_smem;                          // [32][krs]
  uint16_t* ct_s = k_s + LA_BN * krs;               // [nt_n*16][crs]
  uint16_t* p_s = ct_s + nt_n * 16 * crs;           // [4][16][crs]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint16_t* pw_s = p_s + wave * 16 * crs;
  const int row0 = tile_row0[blockIdx.x];
  const int nrows = tile_nrows[blockIdx.x];
  const int h0 = blockIdx.y * HB;
  const int p0 = positions[row0];
  const int32_t* bt = block_table + (int64_t)row_seq[row0] * max_blocks;
  const int hi = p0 + nrows - 1;
  const int lo = window > 0 ? max(0, p0 - window + 1) : 0;

  const int frag_m = lane & 15, frag_k8 = (lane >> 4) * 8;
  const int crow0 = (lane >> 4) * 4, ccol = lane & 15;

  // zero the LDS columns/rows that staging never writes (they meet zero
  // query padding, but stale bits could be NaN patterns)
  for (int i = tid; i < LA_BN * krs; i += 256)
    if (i % krs >= CW) k_s[i] = 0;
  for (int i = tid; i < (nt_n * 16 - R) * crs; i += 256)
    ct_s[R * crs + i] = 0;

  // ---- Q fragments: A operand, row = pair (r, head), 8 entries of the
  //      concatenated (q_abs | q_rot) vector per lane per step ----
  short8v qfrag[KS];
  {
    const int m = wave * 16 + frag_m;
    const int r = m / HB, hh = m % HB;
    const bool ok = r < nrows && h0 + hh < H;
    const uint16_t* qa = q_abs + (int64_t)(row0 + r) * qa_s0 + (h0 + hh) * qa_s1;
    const uint16_t* qr = q_rot + (int64_t)(row0 + r) * qr_s0 + (h0 + hh) * qr_s1;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) {
      short8v f = {0, 0, 0, 0, 0, 0, 0, 0};
      if (ok && kk < ks_n) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int d = kk * 32 + frag_k8 + e;
          uint16_t v = 0;
          if (d < R) v = qa[d];
          else if (d < CW) v = qr[d - R];
          f[e] = (short)v;
        }
      }
      qfrag[kk] = f;
    }
  }

  // ---- per-lane row bookkeeping for the 4 C rows this lane holds ----
  int rpos[4];
  float m_run[4], l_run[4];
#pragma unroll
  for (int r4 = 0; r4 < 4; ++r4) {
    const int m = wave * 16 + crow0 + r4;
    const int r = m / HB, hh = m % HB;
    const bool ok = r < nrows && h0 + hh < H;
    rpos[r4] = ok ? p0 + r : -1;           // -1: sees no key
    m_run[r4] = ok ? sink[h0 + hh] : 0.0f;
    l_run[r4] = 1.0f;
  }
  float4v acc_o[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) acc_o[nt] = {0.f, 0.f, 0.f, 0.f};

  const bool vec = (CW % 8 == 0) && (R % 8 == 0);
  for (int j0 = lo; j0 <= hi; j0 += LA_BN) {
    __syncthreads();   // previous tile consumed (and the zero fill landed)
    // ---- stage 32 cached rows: row-major for S, transposed for O ----
    if (vec) {
      const int c8n = CW / 8;
      for (int idx = tid; idx < LA_BN * c8n; idx += 256) {
        const int key = idx / c8n, d8 = (idx % c8n) * 8;
        const int j = min(j0 + key, hi);
        const int64_t prow = (int64_t)bt[j / block_size] * block_size +
                             j % block_size;
        const ushort8 val =
            *reinterpret_cast<const ushort8*>(cache + prow * CW + d8);
        *reinterpret_cast<ushort8*>(k_s + key * krs + d8) = val;
        if (d8 < R) {
#pragma unroll
          for (int e = 0; e < 8; ++e) ct_s[(d8 + e) * crs + key] = val.v[e];
        }
      }
    } else {
      for (int idx = tid; idx < LA_BN * CW; idx += 256) {
        const int key = idx / CW, d = idx % CW;
        const int j = min(j0 + key, hi);
        const int64_t prow = (int64_t)bt[j / block_size] * block_size +
                             j % block_size;
        const uint16_t val = cache[prow * CW + d];
        k_s[key * krs + d] = val;
        if (d < R) ct_s[d * crs + key] = val;
      }
    }
    __syncthreads();

    // ---- S = Q . K^T : two 16-key sub-tiles ----
    float4v acc_s[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      acc_s[nt] = {0.f, 0.f, 0.f, 0.f};
      const uint16_t* krow = k_s + (nt * 16 + frag_m) * krs + frag_k8;
#pragma unroll
      for (int kk = 0; kk < KS; ++kk) {
        if (kk < ks_n) {
          const short8v bfrag =
              *reinterpret_cast<const short8v*>(krow + kk * 32);
          acc_s[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              qfrag[kk], bfrag, acc_s[nt], 0, 0, 0);
        }
      }
    }

    // ---- mask + online softmax (fp32) ----
    float alpha[4];
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      const int pr = rpos[r4];
      float mx = -INFINITY;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        const int j = j0 + nt * 16 + ccol;
        float s = acc_s[nt][r4] * scale;
        if (j > pr || (window > 0 && j <= pr - window)) s = -INFINITY;
        acc_s[nt][r4] = s;
        mx = fmaxf(mx, s);
      }
      const float mn = fmaxf(m_run[r4], group_reduce_max<16>(mx));
      alpha[r4] = expf(m_run[r4] - mn);
      m_run[r4] = mn;
      float rowsum = 0.0f;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        const float p = expf(acc_s[nt][r4] - mn);   // exp(-inf) = 0
        rowsum += p;
        pw_s[(crow0 + r4) * crs + nt * 16 + ccol] = f32_to_bf16(p);
      }
      l_run[r4] = l_run[r4] * alpha[r4] + group_reduce_sum<16>(rowsum);
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) acc_o[nt][r4] *= alpha[r4];
    }

    // ---- O += P . C : one 32-key step per 16-wide output tile ----
    const short8v pfrag =
        *reinterpret_cast<const short8v*>(pw_s + frag_m * crs + frag_k8);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      if (nt < nt_n) {
        const short8v cfrag = *reinterpret_cast<const short8v*>(
            ct_s + (nt * 16 + frag_m) * crs + frag_k8);
        acc_o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            pfrag, cfrag, acc_o[nt], 0, 0, 0);
      }
    }
  }

  // ---- normalise and store the valid pairs ----
#pragma unroll
  for (int r4 = 0; r4 < 4; ++r4) {
    if (rpos[r4] < 0) continue;
    const int m = wave * 16 + crow0 + r4;
    const int r = m / HB, hh = m % HB;
    const float inv = 1.0f / l_run[r4];
    uint16_t* o = out + ((int64_t)(row0 + r) * H + h0 + hh) * R;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int d = nt * 16 + ccol;
      if (nt < nt_n && d < R) o[d] = f32_to_bf16(acc_o[nt][r4] * inv);
    }
  }
}

// heads per workgroup and rows per tile for a head count
static inline int la_heads_per_block(int H) { return H < 64 ? H : 64; }

int64_t latent_attention_tile_rows(int64_t H) {
  const int HB = la_heads_per_block((int)H);
  return 64 / HB > 0 ? 64 / HB : 1;
}

// returns false when the sizes do not fit this kernel (the caller then
// runs latent_attention_rows)
bool latent_attention_mfma(torch::Tensor out, torch::Tensor q_abs,
                           torch::Tensor q_rot, torch::Tensor cache,
                           torch::Tensor block_table, torch::Tensor row_seq,
                           torch::Tensor positions, torch::Tensor tile_row0,
                           torch::Tensor tile_nrows, torch::Tensor sink,
                           double scale, int64_t window) {
  TORCH_CHECK(q_abs.is_cuda() && q_abs.dim() == 3 && q_abs.stride(2) == 1 &&
              q_abs.dtype() == torch::kBFloat16);
  TORCH_CHECK(q_rot.dim() == 3 && q_rot.stride(2) == 1 &&
              q_rot.dtype() == torch::kBFloat16);
  const int T = q_abs.size(0), H = q_abs.size(1), R = q_abs.size(2);
  const int RD = q_rot.size(2);
  TORCH_CHECK(q_rot.size(0) == T && q_rot.size(1) == H);
  TORCH_CHECK(cache.is_contiguous() && cache.dim() == 3 &&
              cache.size(2) == R + RD && cache.dtype() == torch::kBFloat16);
  TORCH_CHECK(out.is_contiguous() && out.dtype() == torch::kBFloat16 &&
              out.numel() == (int64_t)T * H * R);
  TORCH_CHECK(block_table.dtype() == torch::kInt32 &&
              block_table.is_contiguous() && block_table.dim() == 2);
  TORCH_CHECK(row_seq.dtype() == torch::kInt32 && row_seq.numel() == T);
  TORCH_CHECK(positions.dtype() == torch::kInt32 && positions.numel() == T);
  TORCH_CHECK(sink.dtype() == torch::kFloat32 && sink.numel() == H);
  const int ntiles = tile_row0.numel();
  TORCH_CHECK(tile_row0.dtype() == torch::kInt32 &&
              tile_nrows.dtype() == torch::kInt32 &&
              tile_nrows.numel() == ntiles);
  if (T == 0 || ntiles == 0) return true;
  const int CW = R + RD;
  const int ks_n = (CW + 31) / 32, nt_n = (R + 15) / 16;
  if (ks_n > 18 || nt_n > 32) return false;
  const int HB = la_heads_per_block(H);
  const size_t shmem =
      sizeof(uint16_t) * ((size_t)LA_BN * (ks_n * 32 + LA_PAD) +
                          (size_t)nt_n * 16 * (LA_BN + LA_PAD) +
                          (size_t)4 * 16 * (LA_BN + LA_PAD));
  int dev = 0;
  hipGetDevice(&dev);
  int lds_max = 0;
  hipDeviceGetAttribute(&lds_max, hipDeviceAttributeMaxSharedMemoryPerBlock,
                        dev);
  if ((int64_t)shmem > (int64_t)lds_max) return false;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  dim3 grid(ntiles, (H + HB - 1) / HB);
#define LAUNCH_LA(KSV, NTV)                                                   \
  do {                                                                        \
    auto kern = latent_attention_mfma_kernel<KSV, NTV>;                       \
    if (shmem > 64 * 1024)                                                    \
      (void)hipFuncSetAttribute((const void*)kern,                            \
                                hipFuncAttributeMaxDynamicSharedMemorySize,   \
                                (int)shmem);                                  \
    hipLaunchKernelGGL(                                                       \
        kern, grid, dim3(256), shmem, stream, (uint16_t*)out.data_ptr(),      \
        (const uint16_t*)q_abs.data_ptr(), (int64_t)q_abs.stride(0),          \
        (int64_t)q_abs.stride(1), (const uint16_t*)q_rot.data_ptr(),          \
        (int64_t)q_rot.stride(0), (int64_t)q_rot.stride(1),                   \
        (const uint16_t*)cache.data_ptr(),                                    \
        (const int32_t*)block_table.data_ptr(), (int)block_table.size(1),     \
        (const int32_t*)row_seq.data_ptr(),                                   \
        (const int32_t*)positions.data_ptr(),                                 \
        (const int32_t*)tile_row0.data_ptr(),                                 \
        (const int32_t*)tile_nrows.data_ptr(), (const float*)sink.data_ptr(), \
        (float)scale, (int)window, H, R, RD, (int)cache.size(1), HB);         \
  } while (0)
  if (ks_n <= 4 && nt_n <= 4) LAUNCH_LA(4, 4);
  else if (ks_n <= 10 && nt_n <= 16) LAUNCH_LA(10, 16);
  else LAUNCH_LA(18, 32);
#undef LAUNCH_LA
  (void)hipGetLastError();   // a refused attribute must not poison the check
  HIP_CHECK_KERNEL();
  return true;
}

}  // namespace igw
