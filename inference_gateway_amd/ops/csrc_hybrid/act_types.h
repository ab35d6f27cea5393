// Activation-type plumbing for the hybrid-decoder kernels (gfx950).
//
// Every kernel here is templated on the ACTIVATION storage type: bf16
// (held as uint16_t) for serving, float for true 32-bit runs.  All
// arithmetic is fp32 either way; only loads and stores differ.
#pragma once

#include <ATen/cuda/CUDAContext.h>
#include <torch/extension.h>

#include "../csrc/common.h"

namespace igw {

template <typename T>
struct Act;

template <>
struct Act<float> {
  static DEVINLINE float ld(const float* p) { return *p; }
  static DEVINLINE void st(float* p, float v) { *p = v; }
};

template <>
struct Act<uint16_t> {
  static DEVINLINE float ld(const uint16_t* p) { return bf16_to_f32(*p); }
  static DEVINLINE void st(uint16_t* p, float v) { *p = f32_to_bf16(v); }
};

// fp32 logistic with the full-precision exponential (the recurrence and
// gates are specified in 32-bit; the fast __expf is ~2 ulp worse)
DEVINLINE float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }

// fp32 logistic on the hardware exp/rcp units (a few ulp): used where the
// activations around it are bf16 and the exact version is the bottleneck
DEVINLINE float sigmoid_fast(float x) {
  return __frcp_rn(1.0f + __expf(-x));
}

template <typename T>
DEVINLINE float sigmoid_for(float x);
template <>
DEVINLINE float sigmoid_for<float>(float x) { return sigmoid_f32(x); }
template <>
DEVINLINE float sigmoid_for<uint16_t>(float x) { return sigmoid_fast(x); }

#define IGW_DISPATCH_ACT(TENSOR, ...)                                   \
  do {                                                                  \
    if ((TENSOR).scalar_type() == torch::kBFloat16) {                   \
      using act_t = uint16_t;                                           \
      __VA_ARGS__                                                       \
    } else if ((TENSOR).scalar_type() == torch::kFloat32) {             \
      using act_t = float;                                              \
      __VA_ARGS__                                                       \
    } else {                                                            \
      TORCH_CHECK(false, "activations must be bfloat16 or float32");    \
    }                                                                   \
  } while (0)

}  // namespace igw
