// Shared helpers for the stateful sequence-mixer kernels (group "mix").
//
// Activations are bf16 or f32 (one dtype per call); every kernel widens
// to f32 on load and computes in f32. States and small per-channel
// parameters are f32 tensors.
#pragma once

#include "common.h"
#include <torch/library.h>
#include <ATen/ATen.h>
#include <ATen/hip/HIPContext.h>

namespace kaito {

struct bf16_act { short v; };

template <typename T> KAITO_DEV float act_ld(const T* p);
template <> KAITO_DEV float act_ld<float>(const float* p) { return *p; }
template <> KAITO_DEV float act_ld<bf16_act>(const bf16_act* p) {
  return bf16_to_f32(p->v);
}
template <typename T> KAITO_DEV void act_st(T* p, float v);
template <> KAITO_DEV void act_st<float>(float* p, float v) { *p = v; }
template <> KAITO_DEV void act_st<bf16_act>(bf16_act* p, float v) {
  p->v = f32_to_bf16(v);
}

KAITO_DEV float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
KAITO_DEV float silu_f(float x) { return x / (1.0f + expf(-x)); }
KAITO_DEV float softplus_f(float x) {
  return x > 20.0f ? x : log1pf(expf(x));
}
KAITO_DEV float gelu_tanh_f(float z) {
  const float c = 0.7978845608028654f;   // sqrt(2/pi)
  return 0.5f * z * (1.0f + tanhf(c * (z + 0.044715f * z * z * z)));
}

inline bool is_act_dtype(const at::Tensor& t) {
  return t.dtype() == at::kBFloat16 || t.dtype() == at::kFloat;
}

#define KAITO_CHECK_I32(t) \
  TORCH_CHECK((t).is_cuda() && (t).dtype() == at::kInt && (t).is_contiguous(), #t " must be a contiguous int32 device tensor")
#define KAITO_CHECK_F32(t) \
  TORCH_CHECK((t).is_cuda() && (t).dtype() == at::kFloat && (t).is_contiguous(), #t " must be a contiguous f32 device tensor")

// Run `body` with `act_t` bound to the element type of an activation tensor.
#define KAITO_DISPATCH_ACT(tensor, ...)                          \
  do {                                                           \
    if ((tensor).dtype() == at::kBFloat16) {                     \
      using act_t = bf16_act;                                    \
      __VA_ARGS__                                                \
    } else if ((tensor).dtype() == at::kFloat) {                 \
      using act_t = float;                                       \
      __VA_ARGS__                                                \
    } else {                                                     \
      TORCH_CHECK(false, "activation dtype must be bf16 or f32"); \
    }                                                            \
  } while (0)

}  // namespace kaito
