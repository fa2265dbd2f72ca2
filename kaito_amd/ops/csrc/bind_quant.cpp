// torch op registration for the "quant" kernel group of kaito_amd's gfx950
// extension (one shared library per group, loaded on first use).
#include <torch/library.h>
#include <ATen/ATen.h>

namespace kaito {
void w4a16_gemv(at::Tensor out, at::Tensor x, at::Tensor qweight,
                at::Tensor scales, at::Tensor zeros, int64_t group);
void w4a16_dequant(at::Tensor out, at::Tensor qweight, at::Tensor scales,
                   at::Tensor zeros, int64_t group);
void w4a16_gemm(at::Tensor out, at::Tensor x, at::Tensor qweight,
                at::Tensor scales, at::Tensor zeros, int64_t group);
void lora_shrink(at::Tensor tmp, at::Tensor x, at::Tensor A, at::Tensor idx,
                 double scale);
void lora_expand(at::Tensor y, at::Tensor tmp, at::Tensor B, at::Tensor idx);
}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("w4a16_gemv(Tensor(a!) out, Tensor x, Tensor qweight, Tensor scales, Tensor zeros, int group) -> ()");
  m.def("w4a16_dequant(Tensor(a!) out, Tensor qweight, Tensor scales, Tensor zeros, int group) -> ()");
  m.def("w4a16_gemm(Tensor(a!) out, Tensor x, Tensor qweight, Tensor scales, Tensor zeros, int group) -> ()");
  m.def("lora_shrink(Tensor(a!) tmp, Tensor x, Tensor A, Tensor idx, float scale) -> ()");
  m.def("lora_expand(Tensor(a!) y, Tensor tmp, Tensor B, Tensor idx) -> ()");
}

TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("w4a16_gemv", &kaito::w4a16_gemv);
  m.impl("w4a16_dequant", &kaito::w4a16_dequant);
  m.impl("w4a16_gemm", &kaito::w4a16_gemm);
  m.impl("lora_shrink", &kaito::lora_shrink);
  m.impl("lora_expand", &kaito::lora_expand);
}
