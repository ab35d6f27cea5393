// Row-wise and element-wise kernels of the parallel-block decoder (gfx950):
//
//   add_rmsnorm_pair  residual(fp32) += delta_a + delta_b; ONE RMS statistic,
//                     two weighted outputs (the mixer's and the
//                     feed-forward's norm read the same stream)
//   qk_norm_append    RMS norm over the WHOLE query block and the whole key
//                     block of a fused projection, value blend with another
//                     layer's values, paged append of keys and values
//   gated_act         (gate | up) -> silu(g) u, or the clamped unit
//                     g' sigmoid(alpha g') (u' + 1)
//
// One 256-thread block (4 waves) per token row for the row-wise kernels;
// all arithmetic fp32, loads/stores in the activation type.
#include "act_types.h"

namespace igw {

constexpr int PROW_BLOCK = 256;

DEVINLINE float prow_block_sum(float x, float* lds) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  x = wave_reduce_sum(x);
  if (lane == 0) lds[wave] = x;
  __syncthreads();
  float r = 0.0f;
#pragma unroll
  for (int w = 0; w < PROW_BLOCK / 64; ++w) r += lds[w];
  return r;
}

// 4 consecutive activations <-> 4 floats
template <typename T>
struct Act4;
template <>
struct Act4<float> {
  static DEVINLINE float4 ld(const float* p) { return *(const float4*)p; }
  static DEVINLINE void st(float* p, float4 v) { *(float4*)p = v; }
};
template <>
struct Act4<uint16_t> {
  static DEVINLINE float4 ld(const uint16_t* p) {
    const ushort4x r = *(const ushort4x*)p;
    return make_float4(bf16_to_f32(r.v[0]), bf16_to_f32(r.v[1]),
                       bf16_to_f32(r.v[2]), bf16_to_f32(r.v[3]));
  }
  static DEVINLINE void st(uint16_t* p, float4 v) {
    ushort4x r;
    r.v[0] = f32_to_bf16(v.x);
    r.v[1] = f32_to_bf16(v.y);
    r.v[2] = f32_to_bf16(v.z);
    r.v[3] = f32_to_bf16(v.w);
    *(ushort4x*)p = r;
  }
};

// VEC = 4: D % 4 == 0 and every row 16-byte aligned; VEC = 1 otherwise.
template <typename T, int VEC>
__global__ __launch_bounds__(PROW_BLOCK) void add_rmsnorm_pair_kernel(
    T* __restrict__ out1, T* __restrict__ out2, float* __restrict__ res,
    const T* __restrict__ da, const T* __restrict__ db,
    const float* __restrict__ w1, const float* __restrict__ w2, int D,
    float eps) {
  __shared__ float lds[PROW_BLOCK / 64];
  const int64_t row = blockIdx.x;
  float* r = res + row * D;
  const T* a = da ? da + row * D : nullptr;
  const T* b = db ? db + row * D : nullptr;
  float sq = 0.0f;
  if constexpr (VEC == 4) {
    for (int d = threadIdx.x * 4; d < D; d += PROW_BLOCK * 4) {
      float4 v = *(float4*)(r + d);
      if (a != nullptr || b != nullptr) {
        float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
        if (a != nullptr) s = Act4<T>::ld(a + d);
        if (b != nullptr) {
          const float4 y = Act4<T>::ld(b + d);
          s.x += y.x; s.y += y.y; s.z += y.z; s.w += y.w;
        }
        v.x += s.x; v.y += s.y; v.z += s.z; v.w += s.w;
        *(float4*)(r + d) = v;
      }
      sq += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
  } else {
    for (int d = threadIdx.x; d < D; d += PROW_BLOCK) {
      float v = r[d];
      if (a != nullptr || b != nullptr) {
        float s = 0.0f;
        if (a != nullptr) s = Act<T>::ld(a + d);
        if (b != nullptr) s += Act<T>::ld(b + d);
        v += s;
        r[d] = v;
      }
      sq += v * v;
    }
  }
  const float rstd = 1.0f / sqrtf(prow_block_sum(sq, lds) / (float)D + eps);
  T* o1 = out1 + row * D;
  T* o2 = out2 ? out2 + row * D : nullptr;
  // each thread re-reads exactly the elements it wrote
  if constexpr (VEC == 4) {
    for (int d = threadIdx.x * 4; d < D; d += PROW_BLOCK * 4) {
      const float4 v = *(const float4*)(r + d);
      const float4 g1 = *(const float4*)(w1 + d);
      Act4<T>::st(o1 + d, make_float4(v.x * rstd * g1.x, v.y * rstd * g1.y,
                                      v.z * rstd * g1.z, v.w * rstd * g1.w));
      if (o2 != nullptr) {
        const float4 g2 = *(const float4*)(w2 + d);
        Act4<T>::st(o2 + d, make_float4(v.x * rstd * g2.x, v.y * rstd * g2.y,
                                        v.z * rstd * g2.z, v.w * rstd * g2.w));
      }
    }
  } else {
    for (int d = threadIdx.x; d < D; d += PROW_BLOCK) {
      const float v = r[d] * rstd;
      Act<T>::st(o1 + d, v * w1[d]);
      if (o2 != nullptr) Act<T>::st(o2 + d, v * w2[d]);
    }
  }
}

void add_rmsnorm_pair(torch::Tensor out1, c10::optional<torch::Tensor> out2,
                      torch::Tensor residual,
                      c10::optional<torch::Tensor> delta_a,
                      c10::optional<torch::Tensor> delta_b, torch::Tensor w1,
                      c10::optional<torch::Tensor> w2, double eps) {
  TORCH_CHECK(residual.is_cuda() && residual.dtype() == torch::kFloat32 &&
              residual.is_contiguous() && residual.dim() == 2);
  const int T = residual.size(0), D = residual.size(1);
  TORCH_CHECK(out1.is_contiguous() && out1.size(0) == T && out1.size(1) == D);
  TORCH_CHECK(w1.dtype() == torch::kFloat32 && w1.numel() == D &&
              w1.is_contiguous());
  TORCH_CHECK(out2.has_value() == w2.has_value());
  if (out2.has_value()) {
    TORCH_CHECK(out2->is_contiguous() && out2->dtype() == out1.dtype() &&
                out2->size(0) == T && out2->size(1) == D);
    TORCH_CHECK(w2->dtype() == torch::kFloat32 && w2->numel() == D &&
                w2->is_contiguous());
  }
  for (const auto* dl : {&delta_a, &delta_b}) {
    if (dl->has_value()) {
      TORCH_CHECK((*dl)->is_contiguous() && (*dl)->size(0) == T &&
                  (*dl)->size(1) == D && (*dl)->dtype() == out1.dtype());
    }
  }
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
#define LAUNCH_PAIR(VEC)                                                     \
  hipLaunchKernelGGL(                                                        \
      (add_rmsnorm_pair_kernel<act_t, VEC>), dim3(T), dim3(PROW_BLOCK), 0,   \
      stream, (act_t*)out1.data_ptr(),                                       \
      out2.has_value() ? (act_t*)out2->data_ptr() : nullptr,                 \
      (float*)residual.data_ptr(),                                           \
      delta_a.has_value() ? (const act_t*)delta_a->data_ptr() : nullptr,     \
      delta_b.has_value() ? (const act_t*)delta_b->data_ptr() : nullptr,     \
      (const float*)w1.data_ptr(),                                           \
      w2.has_value() ? (const float*)w2->data_ptr() : nullptr, D, (float)eps)
  IGW_DISPATCH_ACT(out1, {
    if (D % 4 == 0) LAUNCH_PAIR(4);
    else LAUNCH_PAIR(1);
  });
#undef LAUNCH_PAIR
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
// proj row: [ q (H*dk) | k (G*dk) | v (G*dv) | ... ].  Keys are cached as
// [blocks, G, block, dk], values transposed inside the page as
// [blocks, G, dv, block]; slot = block * block_size + offset.
// VEC = 4: NQ, NK, DK % 4 == 0 and 16-byte aligned projection rows.
// R rows per block: with R = 8 the blended values of 8 consecutive batch
// rows wait in LDS, and when those rows are 8 consecutive, 8-aligned slots
// of one page (the usual case inside a prompt portion) each value entry's 8
// tokens leave as ONE contiguous store into the page-transposed cache
// instead of eight 2-byte stores 2 * block_size bytes apart.
template <typename T>
struct alignas(sizeof(T) * 8) Pack8 {
  T v[8];
};

template <typename T, int VEC, int R>
__global__ __launch_bounds__(PROW_BLOCK) void qk_norm_append_kernel(
    T* __restrict__ q_out, const T* __restrict__ proj, int64_t proj_stride,
    const int32_t* __restrict__ slot_mapping, T* __restrict__ kcache,
    T* __restrict__ vcache, const float* __restrict__ wq,
    const float* __restrict__ wk, const T* __restrict__ v_first,
    int64_t vf_stride, float lam, float eps, int NQ, int G, int DK, int DV,
    int block_size, int T_rows) {
  __shared__ float lds_a[PROW_BLOCK / 64], lds_b[PROW_BLOCK / 64];
  extern __shared__ __attribute__((aligned(16))) unsigned char qkn_smem[];
  T* v_lds = reinterpret_cast<T*>(qkn_smem);          // [R][NV], R > 1 only
  const int NK = G * DK, NV = G * DV;
  const int64_t t0 = (int64_t)blockIdx.x * R;
  const int nr = (int)min((int64_t)R, (int64_t)T_rows - t0);
  for (int r = 0; r < nr; ++r) {
    const int64_t t = t0 + r;
    const T* x = proj + t * proj_stride;
    float sq = 0.0f, sk = 0.0f;
    if constexpr (VEC == 4) {
      for (int d = threadIdx.x * 4; d < NQ; d += PROW_BLOCK * 4) {
        const float4 v = Act4<T>::ld(x + d);
        sq += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
      }
      for (int d = threadIdx.x * 4; d < NK; d += PROW_BLOCK * 4) {
        const float4 v = Act4<T>::ld(x + NQ + d);
        sk += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
      }
    } else {
      for (int d = threadIdx.x; d < NQ; d += PROW_BLOCK) {
        const float v = Act<T>::ld(x + d);
        sq += v * v;
      }
      for (int d = threadIdx.x; d < NK; d += PROW_BLOCK) {
        const float v = Act<T>::ld(x + NQ + d);
        sk += v * v;
      }
    }
    // (the two reductions use different LDS words, and each one's barrier
    // separates the other's reads from its next writes)
    const float rq = 1.0f / sqrtf(prow_block_sum(sq, lds_a) / (float)NQ + eps);
    const float rk = 1.0f / sqrtf(prow_block_sum(sk, lds_b) / (float)NK + eps);
    const int slot = slot_mapping[t];
    const int64_t blk = slot / block_size, off = slot % block_size;
    if constexpr (VEC == 4) {
      for (int d = threadIdx.x * 4; d < NQ; d += PROW_BLOCK * 4) {
        const float4 v = Act4<T>::ld(x + d);
        const float4 g = *(const float4*)(wq + d);
        Act4<T>::st(q_out + t * NQ + d,
                    make_float4(v.x * rq * g.x, v.y * rq * g.y, v.z * rq * g.z,
                                v.w * rq * g.w));
      }
      for (int d = threadIdx.x * 4; d < NK; d += PROW_BLOCK * 4) {
        const int g = d / DK, e = d % DK;
        const float4 v = Act4<T>::ld(x + NQ + d);
        const float4 w = *(const float4*)(wk + d);
        Act4<T>::st(kcache + ((blk * G + g) * block_size + off) * DK + e,
                    make_float4(v.x * rk * w.x, v.y * rk * w.y, v.z * rk * w.z,
                                v.w * rk * w.w));
      }
    } else {
      for (int d = threadIdx.x; d < NQ; d += PROW_BLOCK)
        Act<T>::st(q_out + t * NQ + d, Act<T>::ld(x + d) * rq * wq[d]);
      for (int d = threadIdx.x; d < NK; d += PROW_BLOCK) {
        const int g = d / DK, e = d % DK;
        Act<T>::st(kcache + ((blk * G + g) * block_size + off) * DK + e,
                   Act<T>::ld(x + NQ + d) * rk * wk[d]);
      }
    }
    // values go in transposed (one entry per page row)
    const T* vf = v_first ? v_first + t * vf_stride : nullptr;
    for (int d = threadIdx.x; d < NV; d += PROW_BLOCK) {
      float v = Act<T>::ld(x + NQ + NK + d);
      if (vf != nullptr) v = (1.0f - lam) * v + lam * Act<T>::ld(vf + d);
      if constexpr (R > 1) {
        Act<T>::st(v_lds + r * NV + d, v);
      } else {
        const int g = d / DV, e = d % DV;
        Act<T>::st(vcache + ((blk * G + g) * DV + e) * block_size + off, v);
      }
    }
  }
  if constexpr (R > 1) {
    __syncthreads();
    const int s0 = slot_mapping[t0];
    bool run = nr == R && block_size % R == 0 && (s0 % block_size) % R == 0;
    for (int r = 1; r < nr; ++r)
      run = run && slot_mapping[t0 + r] == s0 + r;
    if (run) {
      const int64_t blk = s0 / block_size, off = s0 % block_size;
      for (int d = threadIdx.x; d < NV; d += PROW_BLOCK) {
        const int g = d / DV, e = d % DV;
        Pack8<T> p;
#pragma unroll
        for (int r = 0; r < 8; ++r) p.v[r] = v_lds[r * NV + d];
        *reinterpret_cast<Pack8<T>*>(
            vcache + ((blk * G + g) * DV + e) * block_size + off) = p;
      }
    } else {
      for (int r = 0; r < nr; ++r) {
        const int slot = slot_mapping[t0 + r];
        const int64_t blk = slot / block_size, off = slot % block_size;
        for (int d = threadIdx.x; d < NV; d += PROW_BLOCK) {
          const int g = d / DV, e = d % DV;
          vcache[((blk * G + g) * DV + e) * block_size + off] =
              v_lds[r * NV + d];
        }
      }
    }
  }
}

void qk_norm_append(torch::Tensor q_out, torch::Tensor proj,
                    torch::Tensor slot_mapping, torch::Tensor kcache,
                    torch::Tensor vcache, torch::Tensor qnorm_w,
                    torch::Tensor knorm_w,
                    c10::optional<torch::Tensor> v_first, double lam,
                    double eps, int64_t heads, int64_t kv_heads, int64_t dim,
                    int64_t vdim) {
  TORCH_CHECK(proj.is_cuda() && proj.dim() == 2 && proj.stride(1) == 1);
  const int T = proj.size(0);
  const int NQ = heads * dim, NK = kv_heads * dim, NV = kv_heads * vdim;
  TORCH_CHECK(proj.size(1) >= NQ + NK + NV);
  TORCH_CHECK(q_out.is_contiguous() && q_out.dtype() == proj.dtype() &&
              q_out.size(0) == T && q_out.size(1) == NQ);
  TORCH_CHECK(kcache.is_contiguous() && kcache.dim() == 4 &&
              kcache.size(1) == kv_heads && kcache.size(3) == dim &&
              kcache.dtype() == proj.dtype());
  TORCH_CHECK(vcache.is_contiguous() && vcache.dim() == 4 &&
              vcache.size(0) == kcache.size(0) && vcache.size(1) == kv_heads &&
              vcache.size(3) == kcache.size(2) && vcache.size(2) == vdim &&
              vcache.dtype() == proj.dtype());
  TORCH_CHECK(slot_mapping.dtype() == torch::kInt32 &&
              slot_mapping.numel() == T);
  TORCH_CHECK(qnorm_w.dtype() == torch::kFloat32 && qnorm_w.numel() == NQ);
  TORCH_CHECK(knorm_w.dtype() == torch::kFloat32 && knorm_w.numel() == NK);
  if (v_first.has_value()) {
    TORCH_CHECK(v_first->dim() == 2 && v_first->stride(1) == 1 &&
                v_first->size(0) == T && v_first->size(1) == NV &&
                v_first->dtype() == proj.dtype());
  }
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  const bool vec4 = NQ % 4 == 0 && dim % 4 == 0 && proj.stride(0) % 4 == 0 &&
                    (uintptr_t)proj.data_ptr() % 16 == 0;
  // prompt-sized batches with wide values: 8 rows per block, values staged
  // in LDS (measured: ahead from about 1024 value entries per token, where
  // the scattered stores outweigh the rows' serialised reductions)
  const size_t stage = (size_t)8 * NV * proj.element_size();
  const bool rows8 = T >= 1024 && NV >= 1024 && stage <= 48 * 1024;
#define LAUNCH_QKN(VEC)                                  \
  do {                                                   \
    if (rows8) LAUNCH_QKN_R(VEC, 8, (T + 7) / 8, stage); \
    else LAUNCH_QKN_R(VEC, 1, T, 0);                     \
  } while (0)
#define LAUNCH_QKN_R(VEC, RR, BLOCKS, SHMEM)                                  \
  hipLaunchKernelGGL(                                                         \
      (qk_norm_append_kernel<act_t, VEC, RR>), dim3(BLOCKS),                  \
      dim3(PROW_BLOCK), SHMEM, stream, (act_t*)q_out.data_ptr(),              \
      (const act_t*)proj.data_ptr(),                                          \
      (int64_t)proj.stride(0), (const int32_t*)slot_mapping.data_ptr(),       \
      (act_t*)kcache.data_ptr(), (act_t*)vcache.data_ptr(),                   \
      (const float*)qnorm_w.data_ptr(), (const float*)knorm_w.data_ptr(),     \
      v_first.has_value() ? (const act_t*)v_first->data_ptr() : nullptr,      \
      v_first.has_value() ? (int64_t)v_first->stride(0) : (int64_t)0,         \
      (float)lam, (float)eps, NQ, (int)kv_heads, (int)dim, (int)vdim,         \
      (int)kcache.size(2), T)
  IGW_DISPATCH_ACT(proj, {
    if (vec4) LAUNCH_QKN(4);
    else LAUNCH_QKN(1);
  });
#undef LAUNCH_QKN
#undef LAUNCH_QKN_R
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
// MODE 0: silu(g) * u.  MODE 1: g' = min(g, L), u' = clamp(u, -L, L):
// g' * sigmoid(alpha * g') * (u' + 1).
template <typename T, int MODE>
DEVINLINE float gated_one(float g, float u, float limit, float alpha) {
  if constexpr (MODE == 0) {
    return g * sigmoid_for<T>(g) * u;
  } else {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g * sigmoid_for<T>(alpha * g) * (u + 1.0f);
  }
}

template <typename T, int MODE, int VEC>
__global__ void gated_act_kernel(T* __restrict__ out, const T* __restrict__ in,
                                 int64_t rows, int F, float limit,
                                 float alpha) {
  const int64_t per_row = F / VEC;
  const int64_t total = rows * per_row;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / per_row;
    const int c = (int)(i % per_row) * VEC;
    const T* g = in + r * 2 * F + c;
    T* o = out + r * F + c;
    if constexpr (VEC == 4) {
      const float4 a = Act4<T>::ld(g), b = Act4<T>::ld(g + F);
      Act4<T>::st(o, make_float4(gated_one<T, MODE>(a.x, b.x, limit, alpha),
                                 gated_one<T, MODE>(a.y, b.y, limit, alpha),
                                 gated_one<T, MODE>(a.z, b.z, limit, alpha),
                                 gated_one<T, MODE>(a.w, b.w, limit, alpha)));
    } else {
      Act<T>::st(o, gated_one<T, MODE>(Act<T>::ld(g), Act<T>::ld(g + F), limit,
                                       alpha));
    }
  }
}

void gated_act(torch::Tensor out, torch::Tensor in, int64_t mode, double limit,
               double alpha) {
  TORCH_CHECK(in.is_cuda() && in.is_contiguous() && out.is_contiguous() &&
              out.dtype() == in.dtype());
  TORCH_CHECK(mode == 0 || mode == 1, "gated_act: unknown mode");
  const int F = in.size(-1) / 2;
  TORCH_CHECK(in.size(-1) == 2 * F && out.size(-1) == F &&
              out.numel() * 2 == in.numel());
  const int64_t rows = F ? out.numel() / F : 0;
  if (rows == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  const int vec = F % 4 == 0 ? 4 : 1;
  const int64_t total = rows * (F / vec);
  const int blocks = (int)std::min<int64_t>((total + 255) / 256, 256 * 32);
#define LAUNCH_GATED(MODE, VEC)                                              \
  hipLaunchKernelGGL((gated_act_kernel<act_t, MODE, VEC>), dim3(blocks),     \
                     dim3(256), 0, stream, (act_t*)out.data_ptr(),           \
                     (const act_t*)in.data_ptr(), rows, F, (float)limit,     \
                     (float)alpha)
  IGW_DISPATCH_ACT(in, {
    if (mode == 0) {
      if (vec == 4) LAUNCH_GATED(0, 4);
      else LAUNCH_GATED(0, 1);
    } else {
      if (vec == 4) LAUNCH_GATED(1, 4);
      else LAUNCH_GATED(1, 1);
    }
  });
#undef LAUNCH_GATED
  HIP_CHECK_KERNEL();
}

}  // namespace igw
