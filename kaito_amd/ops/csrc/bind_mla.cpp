// torch op registration for the "mla" kernel group of kaito_amd's gfx950
// extension (one shared library per group, loaded on first use).
#include <torch/library.h>
#include <ATen/ATen.h>

namespace kaito {
void mla_decode(at::Tensor out, at::Tensor q, at::Tensor cache,
                at::Tensor block_tables, at::Tensor seq_lens, double scale);
void mla_cache_write(at::Tensor cache, at::Tensor c_kv, at::Tensor k_pe,
                     at::Tensor slots);
}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("mla_decode(Tensor(a!) out, Tensor q, Tensor cache, Tensor block_tables, Tensor seq_lens, float scale) -> ()");
  m.def("mla_cache_write(Tensor(a!) cache, Tensor c_kv, Tensor k_pe, Tensor slots) -> ()");
}

TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("mla_decode", &kaito::mla_decode);
  m.impl("mla_cache_write", &kaito::mla_cache_write);
}
