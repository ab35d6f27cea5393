// Windowed sigmoid attention on the matrix cores (gfx950, bf16).
//
// Same mathematics and interface as sigmoid_attention_rows
// (sigmoid_attn.hip); this kernel is the serving path for bf16.  The weights
// of ALL heads at one (query, key) pair are mixed before they meet the
// values, so a workgroup owns 16 consecutive query rows of one sequence and
// EVERY head, and walks the keys those rows can see in tiles of 32 (aligned
// to multiples of 32, so a tile never straddles an 8-key group of a page).
// Prompt portions and single decoded tokens use the same kernel (a decoded
// token is a tile with one row).
//
// 8 waves; wave w owns heads [w*hw, w*hw + hw), hw = ceil(H / 8).  Per key
// tile:
//   S_g = Q_g . K_c^T     mfma 16x16x32 bf16; Q fragments live in registers,
//                         K fragments are loaded STRAIGHT from the paged
//                         cache (a key row is the B operand's k-contiguous
//                         layout already) — no LDS staging
//   w_g = sigmoid(S_g * scale + bias[distance, g]), 0 for masked keys, fp32;
//         rounded to bf16 into LDS as [(row, key)][head]
//   M   = talk . W        the head mixing as a matrix product: A = talk
//                         [H x H], B = the LDS tile, 32 column tiles shared
//                         by the 8 waves; result to LDS as [head][row][key]
//   O_h += M_h . V_c      A = LDS tile, B = value fragments straight from
//                         the cache: values are stored transposed inside
//                         the page ([dv][key]), 8 consecutive keys = 16 bytes
// There is no normalisation over keys, hence no running maximum: tiles just
// accumulate, and key splits (gridDim.z) are summed by a small merge kernel
// that also applies the output gate.  The value width can be split over
// gridDim.y when heads * value tiles would not fit the register file.
#include "act_types.h"

namespace igw {

typedef __attribute__((ext_vector_type(8))) short short8v;
typedef __attribute__((ext_vector_type(4))) float float4v;

// round-to-nearest-even fp32 -> bf16 on the conversion unit
DEVINLINE uint16_t sm_bf16(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}

constexpr int SM_TQ = 16;        // query rows per workgroup
constexpr int SM_BN = 32;        // keys per tile
constexpr int SM_NW = 8;         // waves per workgroup
constexpr int SM_WS = 32 + 8;    // LDS row stride (bf16 elements)

// UNI: all heads of a wave read one key/value head (heads per wave divides
// heads per group).  The K/V prefetches are compiled in where the register
// file has room for them next to the Q fragments and the accumulators.
template <int HW, int NT, int KS, bool UNI>
__global__ __launch_bounds__(SM_NW * 64) void sigmoid_attention_mfma_kernel(
    uint16_t* __restrict__ out, float* __restrict__ part, int nsplit, int T,
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ kcache,
    const uint16_t* __restrict__ vcache,
    const int32_t* __restrict__ block_table, int max_blocks,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ tile_row0,
    const int32_t* __restrict__ tile_nrows,
    const float* __restrict__ dist_bias, int ND,
    const float* __restrict__ talk, const uint16_t* __restrict__ gate,
    int64_t gate_stride, float scale, int window, int H, int G, int DK, int DV,
    int block_size, int hw_n, int nt_n) {
  extern __shared__ __attribute__((aligned(16))) uint16_t sm_smem[];
  uint16_t* w_s = sm_smem;                               // [16*32][SM_WS]
  uint16_t* m_s = w_s + SM_TQ * SM_BN * SM_WS;           // [H][16][SM_WS]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int frag_m = lane & 15, frag_k8 = (lane >> 4) * 8;
  const int crow0 = (lane >> 4) * 4, ccol = lane & 15;
  const int per = H / G;
  const int row0 = tile_row0[blockIdx.x];
  const int nrows = tile_nrows[blockIdx.x];
  const int p0 = positions[row0];
  const int32_t* bt = block_table + (int64_t)row_seq[row0] * max_blocks;
  const int hi_all = p0 + nrows - 1;
  const int lo_all = window > 0 ? max(0, p0 - window + 1) : 0;
  // key splits: each takes a contiguous run of whole (aligned) key tiles
  const int t_lo = lo_all / SM_BN, t_hi = hi_all / SM_BN;
  const int t_per = (t_hi - t_lo + nsplit) / nsplit;
  const int t_a = t_lo + (int)blockIdx.z * t_per;
  const int t_b = min(t_hi, t_a + t_per - 1);
  const int d_base = (int)blockIdx.y * nt_n * 16;   // first value entry here
  // keys a row sees: 0 <= distance < wlim
  const unsigned wlim = window > 0 ? (unsigned)window : 0x7fffffffu;
  const int last_page = hi_all / block_size;

  // head columns past H of the weight tile are never written: clear them
  // once (they meet zero entries of talk, but stale bits could be NaNs)
  for (int i = tid; i < SM_TQ * SM_BN * SM_WS; i += SM_NW * 64) w_s[i] = 0;

  // ---- Q fragments (A operand: row = query row, 8 entries per lane) ----
  short8v qfrag[HW][KS];
#pragma unroll
  for (int hw = 0; hw < HW; ++hw) {
    const int g = wave * hw_n + hw;
    const bool ok = hw < hw_n && g < H && frag_m < nrows;
    const uint16_t* qr = q + ((int64_t)(row0 + frag_m) * H + g) * DK;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) {
      short8v f = {0, 0, 0, 0, 0, 0, 0, 0};
      const int d = kk * 32 + frag_k8;
      if (ok && d < DK) f = *reinterpret_cast<const short8v*>(qr + d);
      qfrag[hw][kk] = f;
    }
  }
  // ---- talk fragments (A operand of the mixing: row = h, k = g) ----
  short8v tfrag[2];
#pragma unroll
  for (int mt = 0; mt < 2; ++mt) {
    short8v f = {0, 0, 0, 0, 0, 0, 0, 0};
    const int h = mt * 16 + frag_m;
    if (h < H) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int g = frag_k8 + e;
        if (g < H) f[e] = (short)f32_to_bf16(talk[h * H + g]);
      }
    }
    tfrag[mt] = f;
  }
  const int mt_n = (H + 15) / 16;

  float4v acc[HW][NT];
#pragma unroll
  for (int hw = 0; hw < HW; ++hw)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[hw][nt] = {0.f, 0.f, 0.f, 0.f};

  __syncthreads();

  // UNI: the wave's K and V fragments are loaded once per tile and shared
  // by its heads; the V fragments are requested at the top of the tile
  // (PFV) and the NEXT tile's K fragments right after the scores (PFK), so
  // both loads fly during the barriers and the mixing.
  constexpr int REG_QA = 4 * HW * KS + 4 * HW * NT;
  constexpr bool PFK = UNI && (REG_QA + 8 * KS + 4 * NT <= 112);
  constexpr bool PFV =
      UNI && (REG_QA + 4 * NT <= 128) && !(HW == 4 && KS == 4);
  const int g0 = wave * hw_n;
  const bool wave_on = g0 < H;
  const bool pair_ok = hw_n % 2 == 0 && per % 2 == 0;
  const int c0 = wave_on ? g0 / per : 0;
  short8v kfrag[PFK ? 2 : 1][KS];
  auto load_k = [&](int jt, int nt, int slot) {
    const int j = min(jt * SM_BN + nt * 16 + frag_m, hi_all);
    const uint16_t* kr =
        kcache + (((int64_t)bt[j / block_size] * G + c0) * block_size +
                  j % block_size) * DK + frag_k8;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) {
      short8v b = {0, 0, 0, 0, 0, 0, 0, 0};
      if (wave_on && kk * 32 + frag_k8 < DK)
        b = *reinterpret_cast<const short8v*>(kr + kk * 32);
      kfrag[slot][kk] = b;
    }
  };
  if (PFK && t_a <= t_b) {
    load_k(t_a, 0, 0);
    load_k(t_a, 1, PFK ? 1 : 0);
  }

  for (int jt = t_a; jt <= t_b; ++jt) {
    const int j0 = jt * SM_BN;
    const int jk = j0 + frag_k8;
    const int64_t vbase =
        (int64_t)bt[min(jk / block_size, last_page)] * G * DV * block_size +
        jk % block_size;
    short8v vfrag[PFV ? NT : 1];
    if (PFV) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const int d = d_base + nt * 16 + frag_m;
        short8v b = {0, 0, 0, 0, 0, 0, 0, 0};
        if (wave_on && nt < nt_n && d < DV)
          b = *reinterpret_cast<const short8v*>(
              vcache + vbase + ((int64_t)c0 * DV + d) * block_size);
        vfrag[PFV ? nt : 0] = b;
      }
    }
    // ---- scores and weights of the owned heads ----
    // rows past the tile's last one are skipped as a whole (r4 >= nrows
    // means every lane's row is): a decoded token pays for one row, not 16.
    // Their LDS entries keep whatever they held — each query row only ever
    // meets its own entries, and those rows are never stored.
    auto emit = [&](int g, int nt, const float4v& sc) {
      const int dist0 = p0 + crow0 - (j0 + nt * 16 + ccol);
      uint16_t* wp = w_s + ((crow0 * SM_BN) + nt * 16 + ccol) * SM_WS + g;
      const float* bp = dist_bias + g;
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        if (r4 < nrows) {
          const int dist = dist0 + r4;
          float w = 0.0f;
          if (crow0 + r4 < nrows && (unsigned)dist < wlim)
            w = sigmoid_fast(sc[r4] * scale + bp[min(dist, ND - 1) * H]);
          wp[r4 * SM_BN * SM_WS] = sm_bf16(w);
        }
      }
    };
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      if (UNI) {
        float4v sacc[HW];
#pragma unroll
        for (int hw = 0; hw < HW; ++hw) sacc[hw] = {0.f, 0.f, 0.f, 0.f};
        if (!PFK) load_k(jt, nt, 0);
#pragma unroll
        for (int kk = 0; kk < KS; ++kk)
#pragma unroll
          for (int hw = 0; hw < HW; ++hw)
            if (hw < hw_n)
              sacc[hw] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                  qfrag[hw][kk], kfrag[PFK ? nt : 0][kk], sacc[hw], 0, 0, 0);
        if (PFK && jt < t_b) load_k(jt + 1, nt, PFK ? nt : 0);
#pragma unroll
        for (int hw = 0; hw < HW; ++hw)
          if (hw < hw_n && g0 + hw < H) emit(g0 + hw, nt, sacc[hw]);
      } else {
        // heads of a wave on different key/value heads (or no room for
        // shared fragments): load per head; the lane's key is clamped into
        // the sequence for the ADDRESS only
        const int j = min(j0 + nt * 16 + frag_m, hi_all);
        const int64_t kbase = ((int64_t)bt[j / block_size] * G * block_size +
                               j % block_size) * DK + frag_k8;
        if (HW >= 2 && pair_ok) {
          // two neighbouring heads of one key/value head share each K
          // fragment
#pragma unroll
          for (int hw = 0; hw + 1 < HW; hw += 2) {
            const int g = g0 + hw;
            if (hw < hw_n && g < H) {
              const uint16_t* kr =
                  kcache + kbase + (int64_t)(g / per) * block_size * DK;
              float4v s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
              for (int kk = 0; kk < KS; ++kk) {
                short8v bq = {0, 0, 0, 0, 0, 0, 0, 0};
                if (kk * 32 + frag_k8 < DK)
                  bq = *reinterpret_cast<const short8v*>(kr + kk * 32);
                s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qfrag[hw][kk], bq,
                                                             s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    qfrag[hw + 1][kk], bq, s1, 0, 0, 0);
              }
              emit(g, nt, s0);
              emit(g + 1, nt, s1);
            }
          }
        } else {
#pragma unroll
          for (int hw = 0; hw < HW; ++hw) {
            const int g = g0 + hw;
            if (hw < hw_n && g < H) {
              const uint16_t* kr =
                  kcache + kbase + (int64_t)(g / per) * block_size * DK;
              float4v sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
              for (int kk = 0; kk < KS; ++kk) {
                short8v bq = {0, 0, 0, 0, 0, 0, 0, 0};
                if (kk * 32 + frag_k8 < DK)
                  bq = *reinterpret_cast<const short8v*>(kr + kk * 32);
                sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qfrag[hw][kk], bq,
                                                             sc, 0, 0, 0);
              }
              emit(g, nt, sc);
            }
          }
        }
      }
    }
    __syncthreads();
    // ---- mix the heads: 32 column tiles of 16 (row i, 16 keys) ----
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const int nti = wave * 4 + q4;
      const int i = nti >> 1, jh = (nti & 1) * 16;
      if (i >= nrows) continue;
      const short8v b = *reinterpret_cast<const short8v*>(
          w_s + (nti * 16 + frag_m) * SM_WS + frag_k8);
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        if (mt < mt_n) {
          float4v m = {0.f, 0.f, 0.f, 0.f};
          m = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tfrag[mt], b, m, 0, 0, 0);
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4) {
            const int h = mt * 16 + crow0 + r4;
            if (h < H)
              m_s[(h * SM_TQ + i) * SM_WS + jh + ccol] = sm_bf16(m[r4]);
          }
        }
      }
    }
    __syncthreads();
    // ---- O_h += M_h . V_c : B fragments are 8 consecutive keys of one
    //      value entry, contiguous in the page-transposed cache ----
    if (!PFV && HW >= 2 && REG_QA <= 96 && pair_ok) {
      // two neighbouring heads of one key/value head share each V fragment
#pragma unroll
      for (int hw = 0; hw + 1 < HW; hw += 2) {
        const int h = g0 + hw;
        if (hw < hw_n && h < H) {
          const int c = h / per;
          const short8v a0 = *reinterpret_cast<const short8v*>(
              m_s + (h * SM_TQ + frag_m) * SM_WS + frag_k8);
          const short8v a1 = *reinterpret_cast<const short8v*>(
              m_s + ((h + 1) * SM_TQ + frag_m) * SM_WS + frag_k8);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            const int d = d_base + nt * 16 + frag_m;
            short8v bv = {0, 0, 0, 0, 0, 0, 0, 0};
            if (nt < nt_n && d < DV)
              bv = *reinterpret_cast<const short8v*>(
                  vcache + vbase + ((int64_t)c * DV + d) * block_size);
            acc[hw][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                a0, bv, acc[hw][nt], 0, 0, 0);
            acc[hw + 1][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                a1, bv, acc[hw + 1][nt], 0, 0, 0);
          }
        }
      }
    } else {
#pragma unroll
      for (int hw = 0; hw < HW; ++hw) {
        const int h = g0 + hw;
        if (hw < hw_n && h < H) {
          const int c = h / per;
          const short8v a = *reinterpret_cast<const short8v*>(
              m_s + (h * SM_TQ + frag_m) * SM_WS + frag_k8);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            short8v bv = {0, 0, 0, 0, 0, 0, 0, 0};
            if (PFV) {
              bv = vfrag[PFV ? nt : 0];
            } else {
              const int d = d_base + nt * 16 + frag_m;
              if (nt < nt_n && d < DV)
                bv = *reinterpret_cast<const short8v*>(
                    vcache + vbase + ((int64_t)c * DV + d) * block_size);
            }
            acc[hw][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                a, bv, acc[hw][nt], 0, 0, 0);
          }
        }
      }
    }
    // the next tile's weight writes wait on nothing here: w_s was last
    // read before the barrier above, and m_s is rewritten only after the
    // next tile's first barrier, which every wave reaches after this loop
  }

  // ---- store: gated bf16, or fp32 partials for the merge ----
  const int64_t HD = (int64_t)H * DV;
#pragma unroll
  for (int hw = 0; hw < HW; ++hw) {
    const int h = wave * hw_n + hw;
    if (hw >= hw_n || h >= H) continue;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int d = d_base + nt * 16 + ccol;
      if (nt >= nt_n || d >= DV) continue;
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const int i = crow0 + r4;
        if (i >= nrows) continue;
        const int64_t o = (int64_t)(row0 + i) * HD + h * DV + d;
        if (nsplit == 1) {
          const float gt = bf16_to_f32(
              gate[(int64_t)(row0 + i) * gate_stride + h * DV + d]);
          out[o] = f32_to_bf16(acc[hw][nt][r4] * sigmoid_fast(gt));
        } else {
          part[(int64_t)blockIdx.z * T * HD + o] = acc[hw][nt][r4];
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Single decoded rows: the matrix tiles are turned so that the M dimension
// holds the HEADS of one key/value group instead of 16 query rows.  One
// workgroup per (row, key split); wave c owns key/value head c: one K
// fragment set scores all heads of the group, one V fragment set serves
// them all, nothing is loaded twice and the register tiles are small enough
// for several workgroups per compute unit.  The head mixing in the middle is
// the same matrix product, over 32 keys.  For at most 8 key/value heads of
// at most 16 query heads each and value widths up to 128.
template <int NT, int KS>
__global__ __launch_bounds__(SM_NW * 64) void sigmoid_attention_decode_mfma_kernel(
    uint16_t* __restrict__ out, float* __restrict__ part, int nsplit, int T,
    int row_first, const uint16_t* __restrict__ q,
    const uint16_t* __restrict__ kcache, const uint16_t* __restrict__ vcache,
    const int32_t* __restrict__ block_table, int max_blocks,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ positions,
    const float* __restrict__ dist_bias, int ND,
    const float* __restrict__ talk, const uint16_t* __restrict__ gate,
    int64_t gate_stride, float scale, int window, int H, int G, int DK, int DV,
    int block_size) {
  __shared__ __attribute__((aligned(16))) uint16_t w_s[SM_BN * SM_WS];
  __shared__ __attribute__((aligned(16))) uint16_t m_s[(32 + 16) * SM_WS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int frag_m = lane & 15, frag_k8 = (lane >> 4) * 8;
  const int crow0 = (lane >> 4) * 4, ccol = lane & 15;
  const int per = H / G;
  const int t = row_first + blockIdx.x;
  const int pos = positions[t];
  const int32_t* bt = block_table + (int64_t)row_seq[t] * max_blocks;
  const int lo_all = window > 0 ? max(0, pos - window + 1) : 0;
  const unsigned wlim = window > 0 ? (unsigned)window : 0x7fffffffu;
  const int t_lo = lo_all / SM_BN, t_hi = pos / SM_BN;
  const int t_per = (t_hi - t_lo + nsplit) / nsplit;
  const int t_a = t_lo + (int)blockIdx.z * t_per;
  const int t_b = min(t_hi, t_a + t_per - 1);
  const int last_page = pos / block_size;
  const int c = wave;                    // this wave's key/value head
  const bool wave_on = c < G;
  const int nt_n = (DV + 15) / 16;
  const int mt_n = (H + 15) / 16;

  for (int i = tid; i < SM_BN * SM_WS; i += SM_NW * 64) w_s[i] = 0;
  for (int i = tid; i < (32 + 16) * SM_WS; i += SM_NW * 64) m_s[i] = 0;

  // Q fragments: row = head of the group
  short8v qfrag[KS];
#pragma unroll
  for (int kk = 0; kk < KS; ++kk) {
    short8v f = {0, 0, 0, 0, 0, 0, 0, 0};
    const int d = kk * 32 + frag_k8;
    if (wave_on && frag_m < per && d < DK)
      f = *reinterpret_cast<const short8v*>(
          q + ((int64_t)t * H + c * per + frag_m) * DK + d);
    qfrag[kk] = f;
  }
  // mixing jobs: (key half, head tile) pairs on the first waves
  const int mix_nt = wave & 1, mix_mt = wave >> 1;
  short8v tfrag = {0, 0, 0, 0, 0, 0, 0, 0};
  if (mix_mt < mt_n) {
    const int h = mix_mt * 16 + frag_m;
    if (h < H) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int g = frag_k8 + e;
        if (g < H) tfrag[e] = (short)f32_to_bf16(talk[h * H + g]);
      }
    }
  }
  float4v acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) acc[nt] = {0.f, 0.f, 0.f, 0.f};
  short8v kfrag[2][KS];
  auto load_k = [&](int jt) {
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const int j = min(jt * SM_BN + nt * 16 + frag_m, pos);
      const uint16_t* kr =
          kcache + (((int64_t)bt[j / block_size] * G + c) * block_size +
                    j % block_size) * DK + frag_k8;
#pragma unroll
      for (int kk = 0; kk < KS; ++kk) {
        short8v b = {0, 0, 0, 0, 0, 0, 0, 0};
        if (wave_on && kk * 32 + frag_k8 < DK)
          b = *reinterpret_cast<const short8v*>(kr + kk * 32);
        kfrag[nt][kk] = b;
      }
    }
  };
  if (t_a <= t_b) load_k(t_a);
  __syncthreads();

  for (int jt = t_a; jt <= t_b; ++jt) {
    const int j0 = jt * SM_BN;
    const int jk = j0 + frag_k8;
    short8v vfrag[NT];
    {
      const int64_t vbase =
          ((int64_t)bt[min(jk / block_size, last_page)] * G + c) * DV *
              block_size + jk % block_size;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const int d = nt * 16 + frag_m;
        short8v b = {0, 0, 0, 0, 0, 0, 0, 0};
        if (wave_on && nt < nt_n && d < DV)
          b = *reinterpret_cast<const short8v*>(vcache + vbase +
                                                (int64_t)d * block_size);
        vfrag[nt] = b;
      }
    }
    float4v sacc[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      sacc[nt] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < KS; ++kk)
        sacc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            qfrag[kk], kfrag[nt][kk], sacc[nt], 0, 0, 0);
    }
    if (jt < t_b) load_k(jt + 1);
    if (wave_on) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        const int dist = pos - (j0 + nt * 16 + ccol);
        const bool seen = (unsigned)dist < wlim;
        const float* bp = dist_bias + min(max(dist, 0), ND - 1) * H + c * per;
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          const int pp = crow0 + r4;
          if (pp < per) {
            float w = 0.0f;
            if (seen) w = sigmoid_fast(sacc[nt][r4] * scale + bp[pp]);
            w_s[(nt * 16 + ccol) * SM_WS + c * per + pp] = sm_bf16(w);
          }
        }
      }
    }
    __syncthreads();
    if (mix_mt < mt_n) {
      const short8v b = *reinterpret_cast<const short8v*>(
          w_s + (mix_nt * 16 + frag_m) * SM_WS + frag_k8);
      float4v m = {0.f, 0.f, 0.f, 0.f};
      m = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tfrag, b, m, 0, 0, 0);
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const int h = mix_mt * 16 + crow0 + r4;
        if (h < H) m_s[h * SM_WS + mix_nt * 16 + ccol] = sm_bf16(m[r4]);
      }
    }
    __syncthreads();
    if (wave_on) {
      // rows past the group's heads read other heads' (finite) entries or
      // the zero tail; their results are never stored
      const short8v a = *reinterpret_cast<const short8v*>(
          m_s + (c * per + frag_m) * SM_WS + frag_k8);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        if (nt < nt_n)
          acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, vfrag[nt],
                                                            acc[nt], 0, 0, 0);
    }
  }

  if (!wave_on) return;
  const int64_t HD = (int64_t)H * DV;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int d = nt * 16 + ccol;
    if (nt >= nt_n || d >= DV) continue;
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      const int pp = crow0 + r4;
      if (pp >= per) continue;
      const int64_t col = (int64_t)(c * per + pp) * DV + d;
      if (nsplit == 1) {
        const float gt = bf16_to_f32(gate[(int64_t)t * gate_stride + col]);
        out[(int64_t)t * HD + col] =
            f32_to_bf16(acc[nt][r4] * sigmoid_fast(gt));
      } else {
        part[((int64_t)blockIdx.z * T + t) * HD + col] = acc[nt][r4];
      }
    }
  }
}

// out = sigmoid(gate) * sum over key splits
// (rows [row_a, row_b) of T)
__global__ void sigmoid_attention_merge_kernel(
    uint16_t* __restrict__ out, const float* __restrict__ part, int nsplit,
    int64_t T, int64_t row_a, int64_t row_b, int64_t HD,
    const uint16_t* __restrict__ gate, int64_t gate_stride) {
  const int64_t total = T * HD;
  for (int64_t i = row_a * HD + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
       i < row_b * HD; i += (int64_t)gridDim.x * blockDim.x) {
    float a = 0.0f;
    for (int z = 0; z < nsplit; ++z) a += part[z * total + i];
    const int64_t t = i / HD, c = i % HD;
    out[i] = f32_to_bf16(a * sigmoid_fast(bf16_to_f32(gate[t * gate_stride + c])));
  }
}

int64_t sigmoid_attention_tile_rows() { return SM_TQ; }

void sigmoid_attention_check(torch::Tensor out, torch::Tensor q,
                             torch::Tensor kcache, torch::Tensor vcache,
                             torch::Tensor block_table, torch::Tensor row_seq,
                             torch::Tensor positions, torch::Tensor dist_bias,
                             torch::Tensor talk, torch::Tensor gate);

bool sigmoid_attention_mfma(torch::Tensor out, torch::Tensor q,
                            torch::Tensor kcache, torch::Tensor vcache,
                            torch::Tensor block_table, torch::Tensor row_seq,
                            torch::Tensor positions, torch::Tensor tile_row0,
                            torch::Tensor tile_nrows, torch::Tensor dist_bias,
                            torch::Tensor talk, torch::Tensor gate,
                            double scale, int64_t window, int64_t max_keys,
                            int64_t num_prefill_rows) {
  sigmoid_attention_check(out, q, kcache, vcache, block_table, row_seq,
                          positions, dist_bias, talk, gate);
  TORCH_CHECK(q.scalar_type() == torch::kBFloat16);
  const int T = q.size(0), H = talk.size(0), G = kcache.size(1);
  const int DK = kcache.size(3), DV = vcache.size(2);
  const int bs = kcache.size(2);
  const int ntiles_all = tile_row0.numel();
  TORCH_CHECK(tile_row0.dtype() == torch::kInt32 &&
              tile_nrows.dtype() == torch::kInt32 &&
              tile_nrows.numel() == ntiles_all);
  TORCH_CHECK(num_prefill_rows >= 0 && num_prefill_rows <= T &&
              T - num_prefill_rows <= ntiles_all);
  // shapes this kernel is built for; everything else takes the row kernel
  if (H > 4 * SM_NW || DK % 8 != 0 || DK > 128 || bs % 8 != 0) return false;
  const int hw_n = (H + SM_NW - 1) / SM_NW;           // heads per wave
  // shared fragments need registers the largest tiles do not have left
  const bool uni = (H / G) % hw_n == 0 && !(hw_n > 2 && DK > 64);
  const int nt_all = (DV + 15) / 16;
  // at most 16 accumulator tiles per wave: split the value width over
  // gridDim.y beyond that (which repeats the scores and the mixing)
  const int nt_max = hw_n <= 2 ? 8 : 4;
  const int dsplit = (nt_all + nt_max - 1) / nt_max;
  const int nt_n = (nt_all + dsplit - 1) / dsplit;
  if (nt_n > nt_max) return false;
  const size_t shmem =
      ((size_t)SM_TQ * SM_BN + (size_t)H * SM_TQ) * SM_WS * sizeof(uint16_t);
  if (T == 0 || ntiles_all == 0) return true;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  const int64_t HD = (int64_t)H * DV;
  const int key_tiles = std::max<int64_t>(1, (max_keys + SM_TQ) / SM_BN + 1);
  auto splits_for = [&](int64_t groups, int64_t want) {
    // key splits: fill the chip when there are few workgroups
    int64_t n = 1;
    if (groups < want) n = std::min<int64_t>(key_tiles, (want + groups - 1) / groups);
    return (int)std::max<int64_t>(1, std::min<int64_t>(n, 64));
  };
  auto merge = [&](const torch::Tensor& part, int nsplit, int64_t ra,
                   int64_t rb) {
    const int64_t total = (rb - ra) * HD;
    const int blocks = (int)std::min<int64_t>((total + 255) / 256, 8192);
    hipLaunchKernelGGL(sigmoid_attention_merge_kernel, dim3(blocks), dim3(256),
                       0, stream, (uint16_t*)out.data_ptr(),
                       (const float*)part.data_ptr(), nsplit, (int64_t)T, ra,
                       rb, HD, (const uint16_t*)gate.data_ptr(),
                       (int64_t)gate.stride(0));
  };

  // single decoded rows go to the heads-as-rows kernel when its shape
  // limits hold; prompt portions (and everything otherwise) to the
  // rows-as-rows kernel
  const int per = H / G;
  const bool dec_ok = G <= SM_NW && per <= 16 && nt_all <= 8;
  const int n_dec = dec_ok ? T - (int)num_prefill_rows : 0;
  const int ntiles = ntiles_all - n_dec;

  if (ntiles > 0) {
    const int nsplit = splits_for((int64_t)ntiles * dsplit, 512);
    torch::Tensor part;
    if (nsplit > 1)
      part = torch::empty({nsplit, T, HD}, q.options().dtype(torch::kFloat32));
#define LAUNCH_SM(HWT, NTT, KST)                       \
  do {                                                 \
    if (uni) LAUNCH_SM_U(HWT, NTT, KST, true);         \
    else LAUNCH_SM_U(HWT, NTT, KST, false);            \
  } while (0)
#define LAUNCH_SM_U(HWT, NTT, KST, UNIT)                                      \
  do {                                                                        \
    auto kern = sigmoid_attention_mfma_kernel<HWT, NTT, KST, UNIT>;           \
    static size_t lds_granted = 48 * 1024;                                    \
    if (shmem > lds_granted) {                                                \
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),            \
                              hipFuncAttributeMaxDynamicSharedMemorySize,     \
                              (int)shmem) != hipSuccess) {                    \
        (void)hipGetLastError();                                              \
        return false;                                                         \
      }                                                                       \
      lds_granted = shmem;                                                    \
    }                                                                         \
    hipLaunchKernelGGL(                                                       \
        kern, dim3(ntiles, dsplit, nsplit), dim3(SM_NW * 64), shmem, stream,  \
        (uint16_t*)out.data_ptr(),                                            \
        nsplit > 1 ? (float*)part.data_ptr() : nullptr, nsplit, T,            \
        (const uint16_t*)q.data_ptr(), (const uint16_t*)kcache.data_ptr(),    \
        (const uint16_t*)vcache.data_ptr(),                                   \
        (const int32_t*)block_table.data_ptr(), (int)block_table.size(1),     \
        (const int32_t*)row_seq.data_ptr(),                                   \
        (const int32_t*)positions.data_ptr(),                                 \
        (const int32_t*)tile_row0.data_ptr(),                                 \
        (const int32_t*)tile_nrows.data_ptr(),                                \
        (const float*)dist_bias.data_ptr(), (int)dist_bias.size(0),           \
        (const float*)talk.data_ptr(), (const uint16_t*)gate.data_ptr(),      \
        (int64_t)gate.stride(0), (float)scale, (int)window, H, G, DK, DV, bs, \
        hw_n, nt_n);                                                          \
  } while (0)
#define LAUNCH_SM_KS(HWT, NTT)                \
  do {                                        \
    if (DK <= 64) LAUNCH_SM(HWT, NTT, 2);     \
    else LAUNCH_SM(HWT, NTT, 4);              \
  } while (0)
    if (hw_n <= 1) {
      if (nt_n <= 2) LAUNCH_SM_KS(1, 2);
      else if (nt_n <= 4) LAUNCH_SM_KS(1, 4);
      else LAUNCH_SM_KS(1, 8);
    } else if (hw_n <= 2) {
      if (nt_n <= 2) LAUNCH_SM_KS(2, 2);
      else if (nt_n <= 4) LAUNCH_SM_KS(2, 4);
      else LAUNCH_SM_KS(2, 8);
    } else {
      if (nt_n <= 2) LAUNCH_SM_KS(4, 2);
      else LAUNCH_SM_KS(4, 4);
    }
#undef LAUNCH_SM_KS
#undef LAUNCH_SM
#undef LAUNCH_SM_U
    HIP_CHECK_KERNEL();
    if (nsplit > 1) {
      // rows of the launched tiles: [0, first decoded row) or all rows
      merge(part, nsplit, 0, n_dec > 0 ? num_prefill_rows : (int64_t)T);
      HIP_CHECK_KERNEL();
    }
  }

  if (n_dec > 0) {
    const int row_first = (int)num_prefill_rows;
    const int nsplit = splits_for(n_dec, 1024);
    torch::Tensor part;
    if (nsplit > 1)
      part = torch::empty({nsplit, T, HD}, q.options().dtype(torch::kFloat32));
#define LAUNCH_DEC(NTT, KST)                                                  \
  hipLaunchKernelGGL(                                                         \
      (sigmoid_attention_decode_mfma_kernel<NTT, KST>), dim3(n_dec, 1, nsplit), \
      dim3(SM_NW * 64), 0, stream, (uint16_t*)out.data_ptr(),                 \
      nsplit > 1 ? (float*)part.data_ptr() : nullptr, nsplit, T, row_first,   \
      (const uint16_t*)q.data_ptr(), (const uint16_t*)kcache.data_ptr(),      \
      (const uint16_t*)vcache.data_ptr(),                                     \
      (const int32_t*)block_table.data_ptr(), (int)block_table.size(1),       \
      (const int32_t*)row_seq.data_ptr(),                                     \
      (const int32_t*)positions.data_ptr(),                                   \
      (const float*)dist_bias.data_ptr(), (int)dist_bias.size(0),             \
      (const float*)talk.data_ptr(), (const uint16_t*)gate.data_ptr(),        \
      (int64_t)gate.stride(0), (float)scale, (int)window, H, G, DK, DV, bs)
    if (nt_all <= 2) {
      if (DK <= 64) LAUNCH_DEC(2, 2);
      else LAUNCH_DEC(2, 4);
    } else if (nt_all <= 4) {
      if (DK <= 64) LAUNCH_DEC(4, 2);
      else LAUNCH_DEC(4, 4);
    } else {
      if (DK <= 64) LAUNCH_DEC(8, 2);
      else LAUNCH_DEC(8, 4);
    }
#undef LAUNCH_DEC
    HIP_CHECK_KERNEL();
    if (nsplit > 1) {
      merge(part, nsplit, row_first, T);
      HIP_CHECK_KERNEL();
    }
  }
  return true;
}

}  // namespace igw
