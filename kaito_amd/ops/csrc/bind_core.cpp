// torch op registration for the "core" kernel group of kaito_amd's gfx950
// extension (one shared library per group, loaded on first use).
#include <torch/library.h>
#include <ATen/ATen.h>

namespace kaito {
void rms_norm(at::Tensor out, at::Tensor input, at::Tensor weight, double eps);
void fused_add_rms_norm(at::Tensor out, at::Tensor input, at::Tensor residual,
                        at::Tensor weight, double eps);
void rotary_embedding(at::Tensor positions, at::Tensor q, at::Tensor k,
                      int64_t head_dim, at::Tensor cos_sin_cache);
void silu_and_mul(at::Tensor out, at::Tensor x);
void gelu_and_mul(at::Tensor out, at::Tensor x);
void gelu(at::Tensor out, at::Tensor x);
void layer_norm(at::Tensor out, at::Tensor input, at::Tensor weight,
                at::Tensor bias, double eps);
void fused_add_layer_norm(at::Tensor out, at::Tensor input,
                          at::Tensor residual, at::Tensor weight,
                          at::Tensor bias, double eps);
void reshape_and_cache(at::Tensor k, at::Tensor v, at::Tensor k_cache,
                       at::Tensor v_cache, at::Tensor slot_mapping);
void topk(at::Tensor out_vals, at::Tensor out_idx, at::Tensor scores,
          int64_t k);
}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("rms_norm(Tensor(a!) out, Tensor input, Tensor weight, float eps) -> ()");
  m.def("fused_add_rms_norm(Tensor(a!) out, Tensor input, Tensor(b!) residual, Tensor weight, float eps) -> ()");
  m.def("rotary_embedding(Tensor positions, Tensor(a!) q, Tensor(b!) k, int head_dim, Tensor cos_sin_cache) -> ()");
  m.def("silu_and_mul(Tensor(a!) out, Tensor x) -> ()");
  m.def("gelu_and_mul(Tensor(a!) out, Tensor x) -> ()");
  m.def("gelu(Tensor(a!) out, Tensor x) -> ()");
  m.def("layer_norm(Tensor(a!) out, Tensor input, Tensor weight, Tensor bias, float eps) -> ()");
  m.def("fused_add_layer_norm(Tensor(a!) out, Tensor input, Tensor(b!) residual, Tensor weight, Tensor bias, float eps) -> ()");
  m.def("reshape_and_cache(Tensor k, Tensor v, Tensor(a!) k_cache, Tensor(b!) v_cache, Tensor slot_mapping) -> ()");
  m.def("topk(Tensor(a!) out_vals, Tensor(b!) out_idx, Tensor scores, int k) -> ()");
}

TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("rms_norm", &kaito::rms_norm);
  m.impl("fused_add_rms_norm", &kaito::fused_add_rms_norm);
  m.impl("rotary_embedding", &kaito::rotary_embedding);
  m.impl("silu_and_mul", &kaito::silu_and_mul);
  m.impl("gelu_and_mul", &kaito::gelu_and_mul);
  m.impl("gelu", &kaito::gelu);
  m.impl("layer_norm", &kaito::layer_norm);
  m.impl("fused_add_layer_norm", &kaito::fused_add_layer_norm);
  m.impl("reshape_and_cache", &kaito::reshape_and_cache);
  m.impl("topk", &kaito::topk);
}
