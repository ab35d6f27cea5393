// Absorbed latent attention on the matrix cores (gfx950, bf16).
//
// Same interface as latent_attention_rows (latent_attn.hip); this kernel is
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
// Two workgroups per compute unit are requested for the smaller register
// tiles (measured: 160 -> 104 VGPRs, prompt portions 1.9x faster; three
// would spill).
// Sizes are runtime values; the register tiles are sized by the template
// (KS = 32-wide steps over latent+key width, NT = 16-wide output tiles) and
// loops are predicated on the runtime counts.
#include "act_types.h"

namespace igw {

typedef __attribute__((ext_vector_type(8))) short short8v;
typedef __attribute__((ext_vector_type(4))) float float4v;

constexpr int LA_BN = 32;        // keys per tile
constexpr int LA_PAD = 8;        // bf16 elements of row padding in LDS

template <int KS, int NT, bool PIPE, int NW>
__global__ __launch_bounds__(NW * 64, ((NW == 4 && KS <= 10) ? 2 : 1)) void latent_attention_mfma_kernel(
    uint16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, int nsplit, int T, const uint16_t* __restrict__ q_abs,
    int64_t qa_s0, int64_t qa_s1, const uint16_t* __restrict__ q_rot,
    int64_t qr_s0, int64_t qr_s1, const uint16_t* __restrict__ cache,
    const int32_t* __restrict__ block_table, int max_blocks,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ tile_row0,
    const int32_t* __restrict__ tile_nrows, const float* __restrict__ sink,
    float scale, int window, int H, int R, int RD, int block_size, int HB,
    bool qvec) {
  extern __shared__ __attribute__((aligned(16))) uint16_t la_smem[];
  const int CW = R + RD;
  const int ks_n = (CW + 31) / 32;          // 32-wide steps actually used
  const int nt_n = (R + 15) / 16;           // 16-wide output tiles used
  const int krs = ks_n * 32 + LA_PAD;       // K tile row stride (elements)
  constexpr int crs = LA_BN + LA_PAD;       // CT / P row stride
  uint16_t* k_s = la_smem;                          // [32][krs]
  uint16_t* ct_s = k_s + LA_BN * krs;               // [nt_n*16][crs]
  uint16_t* p_s = ct_s + nt_n * 16 * crs;           // [NW][16][crs]
  constexpr int NTHR = NW * 64;   // NW = 4: 64 pairs per workgroup; NW = 1:
                                  // one wave owns its 16 pairs and its key
                                  // tiles alone (decode launches, few heads)

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint16_t* pw_s = p_s + wave * 16 * crs;
  const int row0 = tile_row0[blockIdx.x];
  const int nrows = tile_nrows[blockIdx.x];
  const int h0 = blockIdx.y * HB;
  const int p0 = positions[row0];
  const int32_t* bt = block_table + (int64_t)row_seq[row0] * max_blocks;
  const int hi_all = p0 + nrows - 1;
  const int lo_all = window > 0 ? max(0, p0 - window + 1) : 0;
  // key splits (gridDim.z): each takes a contiguous run of whole key tiles;
  // split 0 carries the sink
  const int split = blockIdx.z;
  const int ntile_all = (hi_all - lo_all) / LA_BN + 1;
  const int per = (ntile_all + nsplit - 1) / nsplit;
  const int lo = lo_all + split * per * LA_BN;
  const int hi = min(hi_all, lo + per * LA_BN - 1);

  const int frag_m = lane & 15, frag_k8 = (lane >> 4) * 8;
  const int crow0 = (lane >> 4) * 4, ccol = lane & 15;

  // zero the LDS columns/rows that staging never writes (they meet zero
  // query padding, but stale bits could be NaN patterns)
  for (int i = tid; i < LA_BN * krs; i += NTHR)
    if (i % krs >= CW) k_s[i] = 0;
  for (int i = tid; i < (nt_n * 16 - R) * crs; i += NTHR)
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
      if (qvec) {
        // 8 entries never straddle q_abs | q_rot when R % 8 == 0: one
        // 16-byte load per step, all steps in flight together
        const int d = kk * 32 + frag_k8;
        if (ok && d < CW)
          f = *reinterpret_cast<const short8v*>(d < R ? qa + d : qr + (d - R));
      } else if (ok && kk < ks_n) {
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
    // later splits start empty: a finite "minus infinity" keeps the
    // rescaling factors well defined
    m_run[r4] = !ok ? 0.0f : split == 0 ? sink[h0 + hh] : -1e30f;
    l_run[r4] = split == 0 ? 1.0f : 0.0f;
  }
  float4v acc_o[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) acc_o[nt] = {0.f, 0.f, 0.f, 0.f};
  // pairs are numbered rows-major, so a wave is live iff its first pair is
  const bool wave_live =
      (wave * 16) / HB < nrows && h0 + (wave * 16) % HB < H;

  // Staging.  256 % LA_BN == 0, so a thread stages the SAME key of every
  // tile (key = tid % 32) and walks the row in 16-byte pieces 8 keys' worth
  // of threads apart: one block-table lookup per tile per thread, and all of
  // a tile's loads are issued together into registers.  The next tile's
  // loads are issued BEFORE the current tile's matrix work, so memory
  // latency hides behind the MFMAs (register double buffering).
  const bool vec = (CW % 8 == 0) && (R % 8 == 0);
  constexpr int PSTEP = NTHR / LA_BN;    // pieces covered per pass
  constexpr int NCH = (KS * 4 + PSTEP - 1) / PSTEP;   // pieces per thread
  const int skey = tid % LA_BN, spiece = tid / LA_BN;
  const int c8n = CW / 8;
  ushort8 stage[NCH];
  auto cached_row = [&](int j0) -> int64_t {
    const int j = min(j0 + skey, hi);
    return (int64_t)bt[j / block_size] * block_size + j % block_size;
  };
  auto issue_loads = [&](int j0) {
    const uint16_t* row = cache + cached_row(j0) * CW;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int piece = i * PSTEP + spiece;
      if (piece < c8n)
        stage[i] = *reinterpret_cast<const ushort8*>(row + piece * 8);
    }
  };
  if (PIPE && vec && lo <= hi) issue_loads(lo);

  for (int j0 = lo; j0 <= hi; j0 += LA_BN) {
    if (!PIPE && vec) issue_loads(j0);
    __syncthreads();   // previous tile consumed (and the zero fill landed)
    // ---- stage 32 cached rows: row-major for S, transposed for O ----
    if (vec) {
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int d8 = (i * PSTEP + spiece) * 8;
        if (d8 < CW) {
          *reinterpret_cast<ushort8*>(k_s + skey * krs + d8) = stage[i];
          if (d8 < R) {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              ct_s[(d8 + e) * crs + skey] = stage[i].v[e];
          }
        }
      }
    } else {
      const uint16_t* row = cache + cached_row(j0) * CW;
      for (int d = spiece; d < CW; d += PSTEP) {
        const uint16_t val = row[d];
        k_s[skey * krs + d] = val;
        if (d < R) ct_s[d * crs + skey] = val;
      }
    }
    __syncthreads();
    if (PIPE && vec && j0 + LA_BN <= hi) issue_loads(j0 + LA_BN);

    if (!wave_live) continue;   // no valid pair in this wave: stage only

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
      alpha[r4] = __expf(m_run[r4] - mn);
      m_run[r4] = mn;
      float rowsum = 0.0f;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        // hardware exponential: the result is rounded to bf16 for the
        // P.C product anyway, and this loop is VALU-bound; exp(-inf) = 0
        const float p = __expf(acc_s[nt][r4] - mn);
        rowsum += p;
        pw_s[(crow0 + r4) * crs + nt * 16 + ccol] = f32_to_bf16(p);
      }
      l_run[r4] = l_run[r4] * alpha[r4] + group_reduce_sum<16>(rowsum);
    }
    // the running maxima settle after the first tiles: skip the rescale
    // of the whole accumulator when no row of this wave moved
    const bool moved = alpha[0] != 1.0f || alpha[1] != 1.0f ||
                       alpha[2] != 1.0f || alpha[3] != 1.0f;
    if (__any(moved)) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) acc_o[nt][r4] *= alpha[r4];
      }
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

  // ---- store the valid pairs: normalised, or as a partial to merge ----
#pragma unroll
  for (int r4 = 0; r4 < 4; ++r4) {
    if (rpos[r4] < 0) continue;
    const int m = wave * 16 + crow0 + r4;
    const int r = m / HB, hh = m % HB;
    const int64_t pair = (int64_t)(row0 + r) * H + h0 + hh;
    if (nsplit == 1) {
      const float inv = 1.0f / l_run[r4];
      uint16_t* o = out + pair * R;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const int d = nt * 16 + ccol;
        if (nt < nt_n && d < R) o[d] = f32_to_bf16(acc_o[nt][r4] * inv);
      }
    } else {
      const int64_t slot = (int64_t)split * T * H + pair;
      float* o = part_o + slot * R;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const int d = nt * 16 + ccol;
        if (nt < nt_n && d < R) o[d] = acc_o[nt][r4];
      }
      if (ccol == 0) {
        part_ml[2 * slot] = m_run[r4];
        part_ml[2 * slot + 1] = l_run[r4];
      }
    }
  }
}

// merge the key splits of one (row, head): out = sum_z acc_z e^(m_z - M) /
// sum_z l_z e^(m_z - M)
__global__ __launch_bounds__(64) void latent_attention_merge_kernel(
    uint16_t* __restrict__ out, const float* __restrict__ part_o,
    const float* __restrict__ part_ml, int nsplit, int64_t pairs, int R) {
  const int64_t pair = blockIdx.x;
  float M = -INFINITY;
  for (int z = 0; z < nsplit; ++z)
    M = fmaxf(M, part_ml[2 * (z * pairs + pair)]);
  float den = 0.0f;
  for (int z = 0; z < nsplit; ++z)
    den += part_ml[2 * (z * pairs + pair) + 1] *
           expf(part_ml[2 * (z * pairs + pair)] - M);
  const float inv = 1.0f / den;
  for (int d = threadIdx.x; d < R; d += 64) {
    float acc = 0.0f;
    for (int z = 0; z < nsplit; ++z)
      acc += part_o[(z * pairs + pair) * R + d] *
             expf(part_ml[2 * (z * pairs + pair)] - M);
    out[pair * R + d] = f32_to_bf16(acc * inv);
  }
}

// heads per workgroup and rows per tile for a head count
static inline int la_heads_per_block(int H, int nw = 4) {
  return H < nw * 16 ? H : nw * 16;
}

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
                           double scale, int64_t window, int64_t max_keys) {
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
  // decode-only launches with few heads: single-wave workgroups (no idle
  // waves, no cross-wave barriers, three per compute unit by LDS)
  const int nw =
      (ntiles == T && H <= 32 && ks_n <= 10 && nt_n <= 16) ? 1 : 4;
  const int HB = la_heads_per_block(H, nw);
  const size_t shmem =
      sizeof(uint16_t) * ((size_t)LA_BN * (ks_n * 32 + LA_PAD) +
                          (size_t)nt_n * 16 * (LA_BN + LA_PAD) +
                          (size_t)nw * 16 * (LA_BN + LA_PAD));
  int dev = 0;
  hipGetDevice(&dev);
  int lds_max = 0;
  hipDeviceGetAttribute(&lds_max, hipDeviceAttributeMaxSharedMemoryPerBlock,
                        dev);
  if ((int64_t)shmem > (int64_t)lds_max) return false;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  const int hgroups = (H + HB - 1) / HB;
  // Fewer workgroups than compute units (small decode batches): cut the
  // keys into splits so the chip fills, at least 4 key tiles per split.
  // Launches of up to a few workgroups per unit also prefetch the next key
  // tile through registers; larger ones hide latency by themselves.
  hipDeviceProp_t* prop = at::cuda::getCurrentDeviceProperties();
  const int64_t cus = prop->multiProcessorCount;
  const int64_t blocks = (int64_t)ntiles * hgroups;
  int nsplit = 1;
  const int64_t want_blocks = cus * (nw == 1 ? 4 : 1);
  if (blocks < want_blocks) {
    const int64_t key_tiles = std::max<int64_t>(1, max_keys / LA_BN);
    nsplit = (int)std::min<int64_t>(
        std::min<int64_t>(8, (want_blocks + blocks - 1) / blocks),
        std::max<int64_t>(1, key_tiles / 4));
  }
  const bool pipe = blocks * nsplit < 2048;
  torch::Tensor part_o, part_ml;
  if (nsplit > 1) {
    auto f32 = q_abs.options().dtype(torch::kFloat32);
    part_o = torch::empty({nsplit, (int64_t)T * H, R}, f32);
    part_ml = torch::empty({nsplit, (int64_t)T * H, 2}, f32);
  }
  dim3 grid(ntiles, hgroups, nsplit);
  // 16-byte query loads need aligned rows on both query tensors
  const bool qvec =
      R % 8 == 0 && RD % 8 == 0 && q_abs.stride(0) % 8 == 0 &&
      q_abs.stride(1) % 8 == 0 && q_rot.stride(0) % 8 == 0 &&
      q_rot.stride(1) % 8 == 0 &&
      reinterpret_cast<uintptr_t>(q_abs.data_ptr()) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(q_rot.data_ptr()) % 16 == 0;
#define LAUNCH_LA2(KSV, NTV, PIPEV, NWV)                                      \
  do {                                                                        \
    auto kern = latent_attention_mfma_kernel<KSV, NTV, PIPEV, NWV>;           \
    if (shmem > 64 * 1024)                                                    \
      (void)hipFuncSetAttribute((const void*)kern,                            \
                                hipFuncAttributeMaxDynamicSharedMemorySize,   \
                                (int)shmem);                                  \
    hipLaunchKernelGGL(                                                       \
        kern, grid, dim3(NWV * 64), shmem, stream, (uint16_t*)out.data_ptr(), \
        nsplit > 1 ? (float*)part_o.data_ptr() : nullptr,                     \
        nsplit > 1 ? (float*)part_ml.data_ptr() : nullptr, nsplit, T,         \
        (const uint16_t*)q_abs.data_ptr(), (int64_t)q_abs.stride(0),          \
        (int64_t)q_abs.stride(1), (const uint16_t*)q_rot.data_ptr(),          \
        (int64_t)q_rot.stride(0), (int64_t)q_rot.stride(1),                   \
        (const uint16_t*)cache.data_ptr(),                                    \
        (const int32_t*)block_table.data_ptr(), (int)block_table.size(1),     \
        (const int32_t*)row_seq.data_ptr(),                                   \
        (const int32_t*)positions.data_ptr(),                                 \
        (const int32_t*)tile_row0.data_ptr(),                                 \
        (const int32_t*)tile_nrows.data_ptr(), (const float*)sink.data_ptr(), \
        (float)scale, (int)window, H, R, RD, (int)cache.size(1), HB, qvec);   \
  } while (0)
#define LAUNCH_LA(KSV, NTV)                                                   \
  do {                                                                        \
    if (pipe) LAUNCH_LA2(KSV, NTV, true, 4);                                  \
    else LAUNCH_LA2(KSV, NTV, false, 4);                                      \
  } while (0)
  if (nw == 1) {
    // single-wave workgroups always prefetch (they have nobody to overlap
    // with); many more of them fit, so the split target is per wave slot
    if (ks_n <= 4 && nt_n <= 4) LAUNCH_LA2(4, 4, true, 1);
    else LAUNCH_LA2(10, 16, true, 1);
  } else if (ks_n <= 4 && nt_n <= 4) LAUNCH_LA(4, 4);
  else if (ks_n <= 10 && nt_n <= 16) LAUNCH_LA(10, 16);
  else LAUNCH_LA(18, 32);
#undef LAUNCH_LA
#undef LAUNCH_LA2
  (void)hipGetLastError();   // a refused attribute must not poison the check
  HIP_CHECK_KERNEL();
  if (nsplit > 1) {
    hipLaunchKernelGGL(latent_attention_merge_kernel, dim3((int64_t)T * H),
                       dim3(64), 0, stream, (uint16_t*)out.data_ptr(),
                       (const float*)part_o.data_ptr(),
                       (const float*)part_ml.data_ptr(), nsplit,
                       (int64_t)T * H, R);
    HIP_CHECK_KERNEL();
  }
  return true;
}

}  // namespace igw
