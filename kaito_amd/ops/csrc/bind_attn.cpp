// torch op registration for the "attn" kernel group of kaito_amd's gfx950
// extension (one shared library per group, loaded on first use).
#include <torch/library.h>
#include <ATen/ATen.h>

namespace kaito {
void paged_attention(at::Tensor out, at::Tensor query, at::Tensor k_cache,
                     at::Tensor v_cache, at::Tensor block_tables,
                     at::Tensor seq_lens, double scale);
void paged_attention_sp(at::Tensor out, at::Tensor query, at::Tensor k_cache,
                        at::Tensor v_cache, at::Tensor block_tables,
                        at::Tensor seq_lens, double scale, int64_t window,
                        at::Tensor sinks);
void prefill_attention(at::Tensor out, at::Tensor q, at::Tensor k, at::Tensor v,
                       at::Tensor tile_seq, at::Tensor tile_qbase,
                       at::Tensor cu_seqlens, double scale, int64_t window,
                       at::Tensor sinks);
void context_attention(at::Tensor out, at::Tensor q, at::Tensor k_cache,
                       at::Tensor v_cache, at::Tensor tile_seq,
                       at::Tensor tile_qbase, at::Tensor cu_seqlens_q,
                       at::Tensor kv_lens, at::Tensor block_tables,
                       double scale, int64_t window, at::Tensor sinks);
at::Tensor mfma_tile_gemm(at::Tensor a, at::Tensor b);
void paged_read_bw(at::Tensor out, at::Tensor k_cache, at::Tensor v_cache,
                   at::Tensor block_tables, at::Tensor seq_lens,
                   int64_t mode);
}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("paged_attention(Tensor(a!) out, Tensor query, Tensor k_cache, Tensor v_cache, Tensor block_tables, Tensor seq_lens, float scale) -> ()");
  m.def("paged_attention_sp(Tensor(a!) out, Tensor query, Tensor k_cache, Tensor v_cache, Tensor block_tables, Tensor seq_lens, float scale, int window, Tensor sinks) -> ()");
  m.def("prefill_attention(Tensor(a!) out, Tensor q, Tensor k, Tensor v, Tensor tile_seq, Tensor tile_qbase, Tensor cu_seqlens, float scale, int window, Tensor sinks) -> ()");
  m.def("context_attention(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, Tensor tile_seq, Tensor tile_qbase, Tensor cu_seqlens_q, Tensor kv_lens, Tensor block_tables, float scale, int window, Tensor sinks) -> ()");
  m.def("mfma_tile_gemm(Tensor a, Tensor b) -> Tensor");
  m.def("paged_read_bw(Tensor(a!) out, Tensor k_cache, Tensor v_cache, Tensor block_tables, Tensor seq_lens, int mode) -> ()");
}

TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("paged_attention", &kaito::paged_attention);
  m.impl("paged_attention_sp", &kaito::paged_attention_sp);
  m.impl("prefill_attention", &kaito::prefill_attention);
  m.impl("context_attention", &kaito::context_attention);
  m.impl("mfma_tile_gemm", &kaito::mfma_tile_gemm);
  m.impl("paged_read_bw", &kaito::paged_read_bw);
}
