// minGRU recurrence + output gate for a ragged batch (gfx950).
//
//   z = sigmoid(zp)        cand = u + 1/2 (u >= 0) | sigmoid(u)
//   S_t = (1 - z_t) S_{t-1} + z_t cand_t        y_t = S_t * silu(g_t)
//
// with (zp | u | g) the three thirds of a fused projection row.  The state
// S is fp32, one vector per sequence slot; a sequence whose first row is
// position 0 starts from zero (the slot's old content is ignored), any
// other continues from its slot.  The slot is always written back.
//
// Two schedules:
//  * sequential: one thread per (sequence, channel) walks the sequence's
//    rows.  Decode batches and short portions.
//  * chunked scan: the recurrence is linear in S (S_t = a_t S_{t-1} + b_t),
//    so rows are cut into chunks of CHUNK; pass 1 reduces every chunk to
//    (prod a, local end state) in parallel, pass 2 carries the state across
//    a sequence's chunks, pass 3 replays every chunk from its true start
//    state and writes y.  Long prompt portions, where one thread per
//    channel would leave the chip idle.
#include "act_types.h"

namespace igw {

constexpr int GRU_BLOCK = 64;

// V consecutive channels per thread (V = 4 when the width and the row
// stride allow 8/16-byte loads, else 1)
template <typename T, int V>
DEVINLINE void load_v(const T* p, float* o);
template <>
DEVINLINE void load_v<float, 1>(const float* p, float* o) { o[0] = *p; }
template <>
DEVINLINE void load_v<uint16_t, 1>(const uint16_t* p, float* o) {
  o[0] = bf16_to_f32(*p);
}
template <>
DEVINLINE void load_v<float, 4>(const float* p, float* o) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}
template <>
DEVINLINE void load_v<uint16_t, 4>(const uint16_t* p, float* o) {
  const ushort4x v = *reinterpret_cast<const ushort4x*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = bf16_to_f32(v.v[i]);
}
template <typename T, int V>
DEVINLINE void store_v(T* p, const float* o);
template <>
DEVINLINE void store_v<float, 1>(float* p, const float* o) { *p = o[0]; }
template <>
DEVINLINE void store_v<uint16_t, 1>(uint16_t* p, const float* o) {
  *p = f32_to_bf16(o[0]);
}
template <>
DEVINLINE void store_v<float, 4>(float* p, const float* o) {
  *reinterpret_cast<float4*>(p) = make_float4(o[0], o[1], o[2], o[3]);
}
template <>
DEVINLINE void store_v<uint16_t, 4>(uint16_t* p, const float* o) {
  ushort4x v;
#pragma unroll
  for (int i = 0; i < 4; ++i) v.v[i] = f32_to_bf16(o[i]);
  *reinterpret_cast<ushort4x*>(p) = v;
}

template <typename T, int V>
DEVINLINE void gru_coeffs(const T* row, int W, int c, float* a, float* b) {
  float zp[V], u[V];
  load_v<T, V>(row + c, zp);
  load_v<T, V>(row + W + c, u);
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const float z = sigmoid_for<T>(zp[i]);
    const float cand = u[i] >= 0.0f ? u[i] + 0.5f : sigmoid_for<T>(u[i]);
    a[i] = 1.0f - z;
    b[i] = z * cand;
  }
}

// one step of the recurrence for V channels; writes y = S * silu(g)
template <typename T, int V>
DEVINLINE void gru_step(const T* row, T* yrow, int W, int c, float* S) {
  float a[V], b[V], g[V], y[V];
  gru_coeffs<T, V>(row, W, c, a, b);
  load_v<T, V>(row + 2 * W + c, g);
#pragma unroll
  for (int i = 0; i < V; ++i) {
    S[i] = a[i] * S[i] + b[i];
    y[i] = S[i] * (g[i] * sigmoid_for<T>(g[i]));
  }
  store_v<T, V>(yrow + c, y);
}

template <typename T, int V>
__global__ __launch_bounds__(GRU_BLOCK) void mingru_seq_kernel(
    T* __restrict__ y, const T* __restrict__ zug, int64_t zs,
    float* __restrict__ state, const int32_t* __restrict__ cu,
    const int32_t* __restrict__ start, const int32_t* __restrict__ slots,
    int W) {
  const int s = blockIdx.y;
  const int c = (blockIdx.x * GRU_BLOCK + threadIdx.x) * V;
  if (c >= W) return;
  const int r0 = cu[s], r1 = cu[s + 1];
  float* st = state + (int64_t)slots[s] * W + c;
  float S[V];
#pragma unroll
  for (int i = 0; i < V; ++i) S[i] = start[s] > 0 ? st[i] : 0.0f;
#pragma unroll 4
  for (int r = r0; r < r1; ++r)
    gru_step<T, V>(zug + (int64_t)r * zs, y + (int64_t)r * W, W, c, S);
#pragma unroll
  for (int i = 0; i < V; ++i) st[i] = S[i];
}

// pass 1: per chunk, P = prod a and Q = end state from a zero start
template <typename T, int V>
__global__ __launch_bounds__(GRU_BLOCK) void mingru_chunk_reduce_kernel(
    float* __restrict__ P, float* __restrict__ Q, const T* __restrict__ zug,
    int64_t zs, const int32_t* __restrict__ chunk_r0,
    const int32_t* __restrict__ chunk_r1, int W) {
  const int k = blockIdx.y;
  const int c = (blockIdx.x * GRU_BLOCK + threadIdx.x) * V;
  if (c >= W) return;
  float p[V], q[V];
#pragma unroll
  for (int i = 0; i < V; ++i) { p[i] = 1.0f; q[i] = 0.0f; }
  const int r1 = chunk_r1[k];
#pragma unroll 4
  for (int r = chunk_r0[k]; r < r1; ++r) {
    float a[V], b[V];
    gru_coeffs<T, V>(zug + (int64_t)r * zs, W, c, a, b);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      p[i] *= a[i];
      q[i] = a[i] * q[i] + b[i];
    }
  }
#pragma unroll
  for (int i = 0; i < V; ++i) {
    P[(int64_t)k * W + c + i] = p[i];
    Q[(int64_t)k * W + c + i] = q[i];
  }
}

// pass 2: carry the state across each sequence's chunks; Q[k] becomes the
// state ENTERING chunk k
__global__ __launch_bounds__(GRU_BLOCK) void mingru_chunk_carry_kernel(
    const float* __restrict__ P, float* __restrict__ Q,
    float* __restrict__ state, const int32_t* __restrict__ seq_chunk_cu,
    const int32_t* __restrict__ start, const int32_t* __restrict__ slots,
    int W) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * GRU_BLOCK + threadIdx.x;
  if (c >= W) return;
  float* st = state + (int64_t)slots[s] * W + c;
  float S = start[s] > 0 ? *st : 0.0f;
  for (int k = seq_chunk_cu[s]; k < seq_chunk_cu[s + 1]; ++k) {
    const int64_t i = (int64_t)k * W + c;
    const float q = Q[i];
    Q[i] = S;
    S = P[i] * S + q;
  }
  *st = S;
}

// pass 3: replay each chunk from its entering state and write y
template <typename T, int V>
__global__ __launch_bounds__(GRU_BLOCK) void mingru_chunk_apply_kernel(
    T* __restrict__ y, const float* __restrict__ Sin,
    const T* __restrict__ zug, int64_t zs,
    const int32_t* __restrict__ chunk_r0,
    const int32_t* __restrict__ chunk_r1, int W) {
  const int k = blockIdx.y;
  const int c = (blockIdx.x * GRU_BLOCK + threadIdx.x) * V;
  if (c >= W) return;
  float S[V];
#pragma unroll
  for (int i = 0; i < V; ++i) S[i] = Sin[(int64_t)k * W + c + i];
  const int r1 = chunk_r1[k];
#pragma unroll 4
  for (int r = chunk_r0[k]; r < r1; ++r)
    gru_step<T, V>(zug + (int64_t)r * zs, y + (int64_t)r * W, W, c, S);
}

static void check_scan_args(torch::Tensor y, torch::Tensor zug,
                            torch::Tensor state, torch::Tensor seq_cu,
                            torch::Tensor seq_start, torch::Tensor seq_slots) {
  TORCH_CHECK(zug.is_cuda() && zug.dim() == 2 && zug.stride(1) == 1 &&
              zug.size(1) % 3 == 0);
  const int T = zug.size(0), W = zug.size(1) / 3;
  TORCH_CHECK(y.is_contiguous() && y.dtype() == zug.dtype() &&
              y.size(0) == T && y.size(1) == W);
  TORCH_CHECK(state.is_contiguous() && state.dtype() == torch::kFloat32 &&
              state.dim() == 2 && state.size(1) == W);
  const int S = seq_slots.numel();
  TORCH_CHECK(seq_cu.dtype() == torch::kInt32 && seq_cu.numel() == S + 1);
  TORCH_CHECK(seq_start.dtype() == torch::kInt32 && seq_start.numel() == S);
  TORCH_CHECK(seq_slots.dtype() == torch::kInt32);
}

void mingru_scan(torch::Tensor y, torch::Tensor zug, torch::Tensor state,
                 torch::Tensor seq_cu, torch::Tensor seq_start,
                 torch::Tensor seq_slots) {
  check_scan_args(y, zug, state, seq_cu, seq_start, seq_slots);
  const int W = zug.size(1) / 3, S = seq_slots.numel();
  if (S == 0 || zug.size(0) == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  const bool v4 = W % 4 == 0 && zug.stride(0) % 4 == 0;
#define LAUNCH_SEQ(V)                                                        \
  hipLaunchKernelGGL((mingru_seq_kernel<act_t, V>),                          \
                     dim3((W / V + GRU_BLOCK - 1) / GRU_BLOCK, S),           \
                     dim3(GRU_BLOCK), 0, stream, (act_t*)y.data_ptr(),       \
                     (const act_t*)zug.data_ptr(), (int64_t)zug.stride(0),   \
                     (float*)state.data_ptr(),                               \
                     (const int32_t*)seq_cu.data_ptr(),                      \
                     (const int32_t*)seq_start.data_ptr(),                   \
                     (const int32_t*)seq_slots.data_ptr(), W)
  IGW_DISPATCH_ACT(zug, {
    if (v4) LAUNCH_SEQ(4);
    else LAUNCH_SEQ(1);
  });
#undef LAUNCH_SEQ
  HIP_CHECK_KERNEL();
}

// chunk_r0/chunk_r1 [NC]: row ranges, sequence by sequence, in order;
// seq_chunk_cu [S+1]: each sequence's range of chunks; work [2, NC, W] fp32.
void mingru_scan_chunked(torch::Tensor y, torch::Tensor zug,
                         torch::Tensor state, torch::Tensor seq_start,
                         torch::Tensor seq_slots, torch::Tensor chunk_r0,
                         torch::Tensor chunk_r1, torch::Tensor seq_chunk_cu,
                         torch::Tensor work) {
  check_scan_args(y, zug, state, seq_chunk_cu, seq_start, seq_slots);
  const int W = zug.size(1) / 3, S = seq_slots.numel();
  const int NC = chunk_r0.numel();
  TORCH_CHECK(chunk_r0.dtype() == torch::kInt32 &&
              chunk_r1.dtype() == torch::kInt32 && chunk_r1.numel() == NC);
  TORCH_CHECK(work.is_contiguous() && work.dtype() == torch::kFloat32 &&
              work.numel() == (int64_t)2 * NC * W);
  if (S == 0 || NC == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  float* P = (float*)work.data_ptr();
  float* Q = P + (int64_t)NC * W;
  const bool v4 = W % 4 == 0 && zug.stride(0) % 4 == 0;
  const int cb1 = (W + GRU_BLOCK - 1) / GRU_BLOCK;
#define LAUNCH_CHUNKED(V)                                                    \
  do {                                                                       \
    const int cb = (W / V + GRU_BLOCK - 1) / GRU_BLOCK;                      \
    hipLaunchKernelGGL((mingru_chunk_reduce_kernel<act_t, V>), dim3(cb, NC), \
                       dim3(GRU_BLOCK), 0, stream, P, Q,                     \
                       (const act_t*)zug.data_ptr(), (int64_t)zug.stride(0), \
                       (const int32_t*)chunk_r0.data_ptr(),                  \
                       (const int32_t*)chunk_r1.data_ptr(), W);              \
    hipLaunchKernelGGL(mingru_chunk_carry_kernel, dim3(cb1, S),              \
                       dim3(GRU_BLOCK), 0, stream, P, Q,                     \
                       (float*)state.data_ptr(),                             \
                       (const int32_t*)seq_chunk_cu.data_ptr(),              \
                       (const int32_t*)seq_start.data_ptr(),                 \
                       (const int32_t*)seq_slots.data_ptr(), W);             \
    hipLaunchKernelGGL((mingru_chunk_apply_kernel<act_t, V>), dim3(cb, NC),  \
                       dim3(GRU_BLOCK), 0, stream, (act_t*)y.data_ptr(), Q,  \
                       (const act_t*)zug.data_ptr(), (int64_t)zug.stride(0), \
                       (const int32_t*)chunk_r0.data_ptr(),                  \
                       (const int32_t*)chunk_r1.data_ptr(), W);              \
  } while (0)
  IGW_DISPATCH_ACT(zug, {
    if (v4) LAUNCH_CHUNKED(4);
    else LAUNCH_CHUNKED(1);
  });
#undef LAUNCH_CHUNKED
  HIP_CHECK_KERNEL();
}

}  // namespace igw
