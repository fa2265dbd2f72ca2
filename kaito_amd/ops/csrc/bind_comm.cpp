// torch op registration for the "comm" kernel group of kaito_amd's gfx950
// extension (one shared library per group, loaded on first use).
#include <torch/library.h>
#include <ATen/ATen.h>

namespace kaito {
void allreduce_rmsnorm(at::Tensor out, at::Tensor ptrs, at::Tensor weight,
                       double eps);
void one_shot_ar_rmsnorm(at::Tensor out, at::Tensor residual, at::Tensor ptrs,
                         at::Tensor sig_ptrs, at::Tensor counter,
                         at::Tensor weight, double eps, int64_t rank);
at::Tensor ipc_handle(at::Tensor t);
int64_t ipc_open(at::Tensor handle_bytes);
void ipc_close(int64_t ptr);
}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("allreduce_rmsnorm(Tensor(a!) out, Tensor ptrs, Tensor weight, float eps) -> ()");
  m.def("one_shot_ar_rmsnorm(Tensor(a!) out, Tensor(b!) residual, Tensor ptrs, Tensor sig_ptrs, Tensor(c!) counter, Tensor weight, float eps, int rank) -> ()");
  m.def("ipc_handle(Tensor t) -> Tensor");
  m.def("ipc_open(Tensor handle_bytes) -> int");
  m.def("ipc_close(int ptr) -> ()");
}

TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("allreduce_rmsnorm", &kaito::allreduce_rmsnorm);
  m.impl("one_shot_ar_rmsnorm", &kaito::one_shot_ar_rmsnorm);
  m.impl("ipc_handle", &kaito::ipc_handle);
  m.impl("ipc_open", &kaito::ipc_open);
  m.impl("ipc_close", &kaito::ipc_close);
}
