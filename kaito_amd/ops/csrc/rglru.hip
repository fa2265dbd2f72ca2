// Real-gated linear recurrent unit for batches of chunks.
//
// Per channel c (block blk = c / bw of the block-diagonal gates):
//     r = sigmoid(gates[blk, t, c % bw])        recurrence gate
//     i = sigmoid(gates[blk, t, bw + c % bw])   input gate
//     log a = -r * decay_rate[c];  a = exp(log a)
//     S <- a * S + sqrt(1 - a^2) * i * u[t, c]
//     out[t, c] = S * gelu_tanh(y[t, c])
// The gate pre-activations come from a batched f32 matrix product; the
// recurrence is diagonal, so one thread owns one channel of one chunk and
// walks its tokens in order (loads of later tokens do not depend on S and
// pipeline freely). sqrt(1 - a^2) is evaluated as sqrt(-expm1(2 log a)),
// which keeps its precision when a is close to 1. S is f32 in the state
// slot; a chunk starting at position 0 starts from S = 0.
#include "mix_common.h"

namespace kaito {

namespace {

template <typename T>
__global__ void rglru_scan_kernel(
    T* __restrict__ out, const T* __restrict__ u, const int64_t u_s0,
    const float* __restrict__ gates,        // [NB, T, 2*bw]
    const T* __restrict__ y, const int64_t y_s0,
    const float* __restrict__ decay_rate, float* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ starts, const int T_total, const int W,
    const int bw) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int slot = slots[b];
  const int r0 = cu[b], r1 = cu[b + 1];
  if (slot < 0 || r1 <= r0) return;
  const int blk = c / bw, cc = c % bw;
  const float rate = decay_rate[c];
  float S = starts[b] > 0 ? state[(int64_t)slot * W + c] : 0.0f;
  const float* gp = gates + ((int64_t)blk * T_total) * (2 * bw) + cc;
#pragma unroll 4
  for (int t = r0; t < r1; t++) {
    const float rg = sigmoid_f(gp[(int64_t)t * (2 * bw)]);
    const float ig = sigmoid_f(gp[(int64_t)t * (2 * bw) + bw]);
    const float log_a = -rg * rate;
    const float a = expf(log_a);
    const float mult = sqrtf(-expm1f(2.0f * log_a));
    const float uv = act_ld(u + (int64_t)t * u_s0 + c);
    S = a * S + mult * ig * uv;
    act_st(out + (int64_t)t * W + c,
           S * gelu_tanh_f(act_ld(y + (int64_t)t * y_s0 + c)));
  }
  state[(int64_t)slot * W + c] = S;
}

}  // namespace

void rglru_scan(at::Tensor out, at::Tensor u, at::Tensor gates, at::Tensor y,
                at::Tensor decay_rate, at::Tensor state,
                at::Tensor cu_seqlens, at::Tensor state_slots,
                at::Tensor seq_starts) {
  TORCH_CHECK(u.is_cuda() && u.dim() == 2 && y.dim() == 2 &&
              u.stride(1) == 1 && y.stride(1) == 1 && u.dtype() == y.dtype());
  const int T = u.size(0), W = u.size(1);
  TORCH_CHECK(y.size(0) == T && y.size(1) == W);
  TORCH_CHECK(out.is_contiguous() && out.dtype() == u.dtype() &&
              out.size(0) == T && out.size(1) == W);
  KAITO_CHECK_F32(gates); KAITO_CHECK_F32(decay_rate); KAITO_CHECK_F32(state);
  TORCH_CHECK(gates.dim() == 3 && gates.size(1) == T);
  const int NB = gates.size(0);
  TORCH_CHECK(NB > 0 && W % NB == 0 && gates.size(2) == 2 * (W / NB));
  TORCH_CHECK(decay_rate.numel() == W && state.dim() == 2 &&
              state.size(1) == W);
  KAITO_CHECK_I32(cu_seqlens); KAITO_CHECK_I32(state_slots);
  KAITO_CHECK_I32(seq_starts);
  const int B = state_slots.size(0);
  TORCH_CHECK(cu_seqlens.size(0) == B + 1 && seq_starts.size(0) == B);
  if (T == 0 || B == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const int threads = W >= 256 ? 256 : 64;
  KAITO_DISPATCH_ACT(u, {
    hipLaunchKernelGGL((rglru_scan_kernel<act_t>),
        dim3(B, (W + threads - 1) / threads), dim3(threads), 0, stream,
        (act_t*)out.data_ptr(), (const act_t*)u.data_ptr(), u.stride(0),
        gates.data_ptr<float>(), (const act_t*)y.data_ptr(), y.stride(0),
        decay_rate.data_ptr<float>(), state.data_ptr<float>(),
        cu_seqlens.data_ptr<int>(), state_slots.data_ptr<int>(),
        seq_starts.data_ptr<int>(), T, W, W / NB);
  });
}

}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("rglru_scan(Tensor(a!) out, Tensor u, Tensor gates, Tensor y, Tensor decay_rate, Tensor(b!) state, Tensor cu_seqlens, Tensor state_slots, Tensor seq_starts) -> ()");
}
TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("rglru_scan", &kaito::rglru_scan);
}
