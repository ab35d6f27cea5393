// Row-wise and element-wise kernels of the hybrid decoder (gfx950):
//
//   add_layernorm     residual(fp32) += delta; out = LayerNorm(residual)
//   latent_down_post  RMS-norm the two latents of a fused down projection,
//                     rotate the shared key, append (latent | key) to the
//                     paged cache, squash the head gates
//   rope_pairs        in-place interleaved-pair rotation of a slice of
//                     every head
//   xielu / relu2     feed-forward activations
//   gate_heads        [H, T, vd] * gate[T, H] -> [T, H*vd]
//   moe_topk_route    top-k experts + softmax over the chosen logits (times
//                     a constant)
//
// One 256-thread block (4 waves) per token row for the row-wise kernels;
// all arithmetic fp32, loads/stores in the activation type.
#include "act_types.h"

namespace igw {

constexpr int ROW_BLOCK = 256;

// block-wide sum; `lds` holds ROW_BLOCK/64 + 1 floats and must not be
// shared between two reductions without a barrier in between
DEVINLINE float row_block_sum(float x, float* lds) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  x = wave_reduce_sum(x);
  if (lane == 0) lds[wave] = x;
  __syncthreads();
  float r = 0.0f;
#pragma unroll
  for (int w = 0; w < ROW_BLOCK / 64; ++w) r += lds[w];
  return r;
}

template <typename T>
__global__ __launch_bounds__(ROW_BLOCK) void add_layernorm_kernel(
    T* __restrict__ out, float* __restrict__ res, const T* __restrict__ delta,
    const float* __restrict__ w, const float* __restrict__ b, int D,
    float eps) {
  __shared__ float lds_a[ROW_BLOCK / 64], lds_b[ROW_BLOCK / 64];
  const int64_t row = blockIdx.x;
  float* r = res + row * D;
  float sum = 0.0f;
  if (delta != nullptr) {
    const T* dl = delta + row * D;
    for (int d = threadIdx.x; d < D; d += ROW_BLOCK) {
      const float v = r[d] + Act<T>::ld(dl + d);
      r[d] = v;
      sum += v;
    }
  } else {
    for (int d = threadIdx.x; d < D; d += ROW_BLOCK) sum += r[d];
  }
  const float mean = row_block_sum(sum, lds_a) / (float)D;
  // second pass over the thread's own elements: mean squared deviation
  float sq = 0.0f;
  for (int d = threadIdx.x; d < D; d += ROW_BLOCK) {
    const float dv = r[d] - mean;
    sq += dv * dv;
  }
  const float var = row_block_sum(sq, lds_b) / (float)D;
  const float rstd = 1.0f / sqrtf(var + eps);
  T* o = out + row * D;
  for (int d = threadIdx.x; d < D; d += ROW_BLOCK)
    Act<T>::st(o + d, (r[d] - mean) * rstd * w[d] + b[d]);
}

void add_layernorm(torch::Tensor out, torch::Tensor residual,
                   c10::optional<torch::Tensor> delta, torch::Tensor weight,
                   torch::Tensor bias, double eps) {
  TORCH_CHECK(residual.is_cuda() && residual.dtype() == torch::kFloat32 &&
              residual.is_contiguous() && residual.dim() == 2);
  TORCH_CHECK(weight.dtype() == torch::kFloat32 &&
              bias.dtype() == torch::kFloat32);
  const int T = residual.size(0), D = residual.size(1);
  TORCH_CHECK(out.is_contiguous() && out.size(0) == T && out.size(1) == D);
  TORCH_CHECK(weight.numel() == D && bias.numel() == D);
  if (delta.has_value()) {
    TORCH_CHECK(delta->is_contiguous() && delta->size(0) == T &&
                delta->size(1) == D && delta->dtype() == out.dtype());
  }
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  IGW_DISPATCH_ACT(out, {
    hipLaunchKernelGGL(
        (add_layernorm_kernel<act_t>), dim3(T), dim3(ROW_BLOCK), 0, stream,
        (act_t*)out.data_ptr(), (float*)residual.data_ptr(),
        delta.has_value() ? (const act_t*)delta->data_ptr() : nullptr,
        (const float*)weight.data_ptr(), (const float*)bias.data_ptr(), D,
        (float)eps);
  });
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(ROW_BLOCK) void latent_down_post_kernel(
    T* __restrict__ cq, float* __restrict__ gate, const T* __restrict__ down,
    int64_t down_stride, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ slot_mapping, T* __restrict__ cache,
    const float* __restrict__ wq, const float* __restrict__ wc,
    const float* __restrict__ inv_freq, int n_pairs, float eps, int QR, int R,
    int RD, int H) {
  __shared__ float lds_a[ROW_BLOCK / 64], lds_b[ROW_BLOCK / 64];
  const int64_t t = blockIdx.x;
  const T* x = down + t * down_stride;
  float sq = 0.0f, sc = 0.0f;
  for (int d = threadIdx.x; d < QR; d += ROW_BLOCK) {
    const float v = Act<T>::ld(x + d);
    sq += v * v;
  }
  for (int d = threadIdx.x; d < R; d += ROW_BLOCK) {
    const float v = Act<T>::ld(x + QR + d);
    sc += v * v;
  }
  const float rq = 1.0f / sqrtf(row_block_sum(sq, lds_a) / (float)QR + eps);
  const float rc = 1.0f / sqrtf(row_block_sum(sc, lds_b) / (float)R + eps);
  for (int d = threadIdx.x; d < QR; d += ROW_BLOCK)
    Act<T>::st(cq + t * QR + d, Act<T>::ld(x + d) * rq * wq[d]);
  T* crow = cache + (int64_t)slot_mapping[t] * (R + RD);
  for (int d = threadIdx.x; d < R; d += ROW_BLOCK)
    Act<T>::st(crow + d, Act<T>::ld(x + QR + d) * rc * wc[d]);
  const float pos = (float)positions[t];
  const T* kr = x + QR + R;
  for (int i = threadIdx.x; i < n_pairs; i += ROW_BLOCK) {
    const float u = Act<T>::ld(kr + 2 * i), v = Act<T>::ld(kr + 2 * i + 1);
    float s, c;
    sincosf(pos * inv_freq[i], &s, &c);
    Act<T>::st(crow + R + 2 * i, u * c - v * s);
    Act<T>::st(crow + R + 2 * i + 1, v * c + u * s);
  }
  for (int d = 2 * n_pairs + threadIdx.x; d < RD; d += ROW_BLOCK)
    crow[R + d] = kr[d];
  for (int h = threadIdx.x; h < H; h += ROW_BLOCK)
    gate[t * H + h] = sigmoid_f32(Act<T>::ld(x + QR + R + RD + h));
}

void latent_down_post(torch::Tensor cq, torch::Tensor gate, torch::Tensor down,
                      torch::Tensor positions, torch::Tensor slot_mapping,
                      torch::Tensor cache, torch::Tensor qnorm_w,
                      torch::Tensor kvnorm_w, torch::Tensor inv_freq,
                      double eps, int64_t q_rank, int64_t kv_rank,
                      int64_t rot_dim, int64_t heads) {
  const int T = down.size(0);
  TORCH_CHECK(down.is_cuda() && down.dim() == 2 && down.stride(1) == 1);
  TORCH_CHECK(down.size(1) == q_rank + kv_rank + rot_dim + heads);
  TORCH_CHECK(cache.is_contiguous() && cache.dim() == 3 &&
              cache.size(2) == kv_rank + rot_dim &&
              cache.dtype() == down.dtype());
  TORCH_CHECK(cq.is_contiguous() && cq.dtype() == down.dtype() &&
              cq.size(0) == T && cq.size(1) == q_rank);
  TORCH_CHECK(gate.is_contiguous() && gate.dtype() == torch::kFloat32 &&
              gate.size(0) == T && gate.size(1) == heads);
  TORCH_CHECK(positions.dtype() == torch::kInt32 && positions.numel() == T);
  TORCH_CHECK(slot_mapping.dtype() == torch::kInt32 &&
              slot_mapping.numel() == T);
  TORCH_CHECK(qnorm_w.dtype() == torch::kFloat32 &&
              qnorm_w.numel() == q_rank);
  TORCH_CHECK(kvnorm_w.dtype() == torch::kFloat32 &&
              kvnorm_w.numel() == kv_rank);
  TORCH_CHECK(inv_freq.dtype() == torch::kFloat32 &&
              2 * inv_freq.numel() <= rot_dim);
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  IGW_DISPATCH_ACT(down, {
    hipLaunchKernelGGL(
        (latent_down_post_kernel<act_t>), dim3(T), dim3(ROW_BLOCK), 0, stream,
        (act_t*)cq.data_ptr(), (float*)gate.data_ptr(),
        (const act_t*)down.data_ptr(), (int64_t)down.stride(0),
        (const int32_t*)positions.data_ptr(),
        (const int32_t*)slot_mapping.data_ptr(), (act_t*)cache.data_ptr(),
        (const float*)qnorm_w.data_ptr(), (const float*)kvnorm_w.data_ptr(),
        (const float*)inv_freq.data_ptr(), (int)inv_freq.numel(), (float)eps,
        (int)q_rank, (int)kv_rank, (int)rot_dim, (int)heads);
  });
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
template <typename T>
__global__ void rope_pairs_kernel(T* __restrict__ x, int64_t s0, int64_t s1,
                                  const int32_t* __restrict__ positions,
                                  const float* __restrict__ inv_freq,
                                  int n_pairs, int H, int offset,
                                  int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int p = (int)(i % n_pairs);
  const int h = (int)((i / n_pairs) % H);
  const int64_t t = i / ((int64_t)n_pairs * H);
  T* e = x + t * s0 + h * s1 + offset + 2 * p;
  const float u = Act<T>::ld(e), v = Act<T>::ld(e + 1);
  float s, c;
  sincosf((float)positions[t] * inv_freq[p], &s, &c);
  Act<T>::st(e, u * c - v * s);
  Act<T>::st(e + 1, v * c + u * s);
}

void rope_pairs(torch::Tensor x, torch::Tensor positions,
                torch::Tensor inv_freq, int64_t offset) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 3 && x.stride(2) == 1);
  const int T = x.size(0), H = x.size(1);
  const int n_pairs = inv_freq.numel();
  TORCH_CHECK(offset >= 0 && offset + 2 * n_pairs <= x.size(2));
  TORCH_CHECK(positions.dtype() == torch::kInt32 && positions.numel() == T);
  TORCH_CHECK(inv_freq.dtype() == torch::kFloat32);
  const int64_t total = (int64_t)T * H * n_pairs;
  if (total == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  IGW_DISPATCH_ACT(x, {
    hipLaunchKernelGGL((rope_pairs_kernel<act_t>),
                       dim3((total + 255) / 256), dim3(256), 0, stream,
                       (act_t*)x.data_ptr(), (int64_t)x.stride(0),
                       (int64_t)x.stride(1),
                       (const int32_t*)positions.data_ptr(),
                       (const float*)inv_freq.data_ptr(), n_pairs, H,
                       (int)offset, total);
  });
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
DEVINLINE float softplus_f32(float x) {
  return x > 20.0f ? x : log1pf(expf(x));
}

template <typename T>
__global__ void xielu_kernel(T* __restrict__ out, const T* __restrict__ in,
                             const float* __restrict__ pq, int64_t n) {
  const float ap = softplus_f32(pq[0]);
  const float an = 0.5f + softplus_f32(pq[1]);
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const float z = Act<T>::ld(in + i);
    const float y = z > 0.0f ? ap * z * z + 0.5f * z
                             : an * (expm1f(z) - z) + 0.5f * z;
    Act<T>::st(out + i, y);
  }
}

template <typename T>
__global__ void relu2_kernel(T* __restrict__ out, const T* __restrict__ in,
                             int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const float z = fmaxf(Act<T>::ld(in + i), 0.0f);
    Act<T>::st(out + i, z * z);
  }
}

static inline int ew_blocks(int64_t n) {
  return (int)std::min<int64_t>((n + 255) / 256, 256 * 32);
}

void xielu(torch::Tensor out, torch::Tensor in, torch::Tensor pq) {
  TORCH_CHECK(in.is_cuda() && in.is_contiguous() && out.is_contiguous() &&
              out.dtype() == in.dtype() && out.numel() == in.numel());
  TORCH_CHECK(pq.dtype() == torch::kFloat32 && pq.numel() == 2);
  const int64_t n = in.numel();
  if (n == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  IGW_DISPATCH_ACT(in, {
    hipLaunchKernelGGL((xielu_kernel<act_t>), dim3(ew_blocks(n)), dim3(256), 0,
                       stream, (act_t*)out.data_ptr(),
                       (const act_t*)in.data_ptr(),
                       (const float*)pq.data_ptr(), n);
  });
  HIP_CHECK_KERNEL();
}

void relu2(torch::Tensor out, torch::Tensor in) {
  TORCH_CHECK(in.is_cuda() && in.is_contiguous() && out.is_contiguous() &&
              out.dtype() == in.dtype() && out.numel() == in.numel());
  const int64_t n = in.numel();
  if (n == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  IGW_DISPATCH_ACT(in, {
    hipLaunchKernelGGL((relu2_kernel<act_t>), dim3(ew_blocks(n)), dim3(256), 0,
                       stream, (act_t*)out.data_ptr(),
                       (const act_t*)in.data_ptr(), n);
  });
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
template <typename T>
__global__ void gate_heads_kernel(T* __restrict__ out, const T* __restrict__ v,
                                  int64_t sh, int64_t st_,
                                  const float* __restrict__ gate, int H,
                                  int VD, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int d = (int)(i % VD);
  const int h = (int)((i / VD) % H);
  const int64_t t = i / ((int64_t)VD * H);
  Act<T>::st(out + i, Act<T>::ld(v + h * sh + t * st_ + d) * gate[t * H + h]);
}

void gate_heads(torch::Tensor out, torch::Tensor v, torch::Tensor gate) {
  TORCH_CHECK(v.is_cuda() && v.dim() == 3 && v.stride(2) == 1);
  const int H = v.size(0), T = v.size(1), VD = v.size(2);
  TORCH_CHECK(out.is_contiguous() && out.dtype() == v.dtype() &&
              out.numel() == (int64_t)H * T * VD);
  TORCH_CHECK(gate.is_contiguous() && gate.dtype() == torch::kFloat32 &&
              gate.size(0) == T && gate.size(1) == H);
  const int64_t total = (int64_t)H * T * VD;
  if (total == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  IGW_DISPATCH_ACT(v, {
    hipLaunchKernelGGL((gate_heads_kernel<act_t>), dim3((total + 255) / 256),
                       dim3(256), 0, stream, (act_t*)out.data_ptr(),
                       (const act_t*)v.data_ptr(), (int64_t)v.stride(0),
                       (int64_t)v.stride(1), (const float*)gate.data_ptr(), H,
                       VD, total);
  });
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
// One thread per token; the chosen set is a 64-bit mask, so any top-k up to
// the expert count works without per-k template instances.  Ties go to the
// lower expert id.
__global__ void moe_topk_route_kernel(float* __restrict__ weights,
                                      int32_t* __restrict__ idx,
                                      int64_t* __restrict__ dst,
                                      int32_t* __restrict__ counts,
                                      const float* __restrict__ logits, int T,
                                      int E, int K, int capacity,
                                      float scale) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const float* row = logits + (int64_t)t * E;
  float* w = weights + (int64_t)t * K;
  int32_t* id = idx + (int64_t)t * K;
  uint64_t taken = 0;
  float m = 0.0f;
  for (int k = 0; k < K; ++k) {
    int best = -1;
    float bv = 0.0f;
    for (int e = 0; e < E; ++e) {
      const float v = row[e];
      if (!((taken >> e) & 1ull) && (best < 0 || v > bv)) {
        bv = v;
        best = e;
      }
    }
    taken |= 1ull << best;
    id[k] = best;
    w[k] = bv;
    if (k == 0) m = bv;
  }
  float z = 0.0f;
  for (int k = 0; k < K; ++k) {
    const float e = expf(w[k] - m);
    w[k] = e;
    z += e;
  }
  for (int k = 0; k < K; ++k) w[k] = w[k] / z * scale;
  // optional padded dispatch: row = expert * capacity + arrival rank (the
  // order inside an expert's segment carries no meaning: the gather back
  // uses the same rows)
  if (dst != nullptr) {
    for (int k = 0; k < K; ++k) {
      const int e = id[k];
      const int r = atomicAdd(counts + e, 1);
      dst[(int64_t)t * K + k] = (int64_t)e * capacity + r;
    }
  }
}

void moe_topk_route(torch::Tensor weights, torch::Tensor idx,
                    torch::Tensor logits, c10::optional<torch::Tensor> dst,
                    c10::optional<torch::Tensor> counts, int64_t capacity,
                    double scale) {
  TORCH_CHECK(logits.is_cuda() && logits.dtype() == torch::kFloat32 &&
              logits.is_contiguous() && logits.dim() == 2);
  const int T = logits.size(0), E = logits.size(1), K = weights.size(1);
  TORCH_CHECK(E <= 64 && K >= 1 && K <= E, "moe_topk_route: 1 <= k <= E <= 64");
  TORCH_CHECK(weights.is_contiguous() && weights.dtype() == torch::kFloat32 &&
              weights.size(0) == T);
  TORCH_CHECK(idx.is_contiguous() && idx.dtype() == torch::kInt32 &&
              idx.size(0) == T && idx.size(1) == K);
  if (dst.has_value()) {
    TORCH_CHECK(counts.has_value() && capacity >= T);
    TORCH_CHECK(dst->is_contiguous() && dst->dtype() == torch::kInt64 &&
                dst->numel() == (int64_t)T * K);
    TORCH_CHECK(counts->is_contiguous() && counts->dtype() == torch::kInt32 &&
                counts->numel() == E);   // zeroed by the caller
  }
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  hipLaunchKernelGGL(moe_topk_route_kernel, dim3((T + 63) / 64), dim3(64), 0,
                     stream, (float*)weights.data_ptr(),
                     (int32_t*)idx.data_ptr(),
                     dst.has_value() ? (int64_t*)dst->data_ptr() : nullptr,
                     dst.has_value() ? (int32_t*)counts->data_ptr() : nullptr,
                     (const float*)logits.data_ptr(), T, E, K, (int)capacity,
                     (float)scale);
  HIP_CHECK_KERNEL();
}

}  // namespace igw
