// Depthwise causal short convolution over time with a carried tail, for
// batches of chunks (prompt portions and single decode tokens alike).
//
//   out[t, c] = act( bias[c] + sum_j w[c, j] * in(t - (taps-1-j), c) )
//
// where in(.) is the chunk's own rows, the sequence's last taps-1 inputs
// kept in its state slot for offsets before the chunk, and zero before
// the start of the sequence. Token-parallel: one thread per (row,
// channel); the tail is advanced by a second launch (stream order puts it
// after every read of the old tail).
#include "mix_common.h"

namespace kaito {

namespace {

template <typename T>
__global__ void causal_conv_out_kernel(
    T* __restrict__ out, const T* __restrict__ x, const int64_t x_stride,
    const float* __restrict__ w, const float* __restrict__ bias,
    const T* __restrict__ state, const int* __restrict__ cu,
    const int* __restrict__ slots, const int* __restrict__ starts,
    const int* __restrict__ token_seq, const int C, const int taps,
    const int tail, const int act) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int b = token_seq[t];
  if (b < 0) return;
  const int slot = slots[b];
  if (slot < 0) return;
  const int r0 = cu[b];
  const int off = t - r0;
  const bool carried = starts[b] > 0;
  float acc = bias ? bias[c] : 0.0f;
  for (int j = 0; j < taps; j++) {
    const int o = off - (taps - 1 - j);
    float xv = 0.0f;
    if (o >= 0) {
      xv = act_ld(x + (int64_t)(r0 + o) * x_stride + c);
    } else if (carried) {
      // the tail keeps inputs at offsets -(taps-1) .. -1 in rows 0 .. taps-2
      xv = act_ld(state + ((int64_t)slot * tail + (taps - 1 + o)) * C + c);
    }
    acc += w[c * taps + j] * xv;
  }
  if (act == 1) acc = silu_f(acc);
  act_st(out + (int64_t)t * C + c, acc);
}

template <typename T>
__global__ void causal_conv_tail_kernel(
    const T* __restrict__ x, const int64_t x_stride, T* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ starts, const int C, const int taps,
    const int tail) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int slot = slots[b];
  const int r0 = cu[b];
  const int n = cu[b + 1] - r0;
  if (slot < 0 || n <= 0) return;
  const bool carried = starts[b] > 0;
  T* st = state + (int64_t)slot * tail * C + c;
  // ascending s reads row s+n (> s) of the old tail before it is overwritten
  for (int s = 0; s < taps - 1; s++) {
    const int o = n - (taps - 1) + s;
    float v = 0.0f;
    if (o >= 0) v = act_ld(x + (int64_t)(r0 + o) * x_stride + c);
    else if (carried) v = act_ld(st + (int64_t)(taps - 1 + o) * C);
    act_st(st + (int64_t)s * C, v);
  }
}

}  // namespace

void causal_conv_update(at::Tensor out, at::Tensor x, at::Tensor weight,
                        at::Tensor bias, at::Tensor conv_state,
                        at::Tensor cu_seqlens, at::Tensor state_slots,
                        at::Tensor seq_starts, at::Tensor token_seq,
                        int64_t act) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.stride(1) == 1);
  TORCH_CHECK(out.is_contiguous() && out.sizes() == x.sizes() &&
              out.dtype() == x.dtype());
  const int T = x.size(0), C = x.size(1);
  KAITO_CHECK_F32(weight);
  TORCH_CHECK(weight.dim() == 2 && weight.size(0) == C);
  const int taps = weight.size(1);
  TORCH_CHECK(taps >= 1);
  const bool has_bias = bias.numel() > 0;
  if (has_bias) { KAITO_CHECK_F32(bias); TORCH_CHECK(bias.numel() == C); }
  TORCH_CHECK(conv_state.is_contiguous() && conv_state.dim() == 3 &&
              conv_state.dtype() == x.dtype() && conv_state.size(2) == C &&
              conv_state.size(1) >= std::max(taps - 1, 1));
  const int tail = conv_state.size(1);
  KAITO_CHECK_I32(cu_seqlens); KAITO_CHECK_I32(state_slots);
  KAITO_CHECK_I32(seq_starts); KAITO_CHECK_I32(token_seq);
  const int B = state_slots.size(0);
  TORCH_CHECK(cu_seqlens.size(0) == B + 1 && seq_starts.size(0) == B &&
              token_seq.size(0) == T);
  if (T == 0 || B == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const int threads = 256;
  const dim3 gc((C + threads - 1) / threads);
  KAITO_DISPATCH_ACT(x, {
    hipLaunchKernelGGL((causal_conv_out_kernel<act_t>),
        dim3(T, gc.x), dim3(threads), 0, stream,
        (act_t*)out.data_ptr(), (const act_t*)x.data_ptr(), x.stride(0),
        weight.data_ptr<float>(),
        has_bias ? bias.data_ptr<float>() : nullptr,
        (const act_t*)conv_state.data_ptr(), cu_seqlens.data_ptr<int>(),
        state_slots.data_ptr<int>(), seq_starts.data_ptr<int>(),
        token_seq.data_ptr<int>(), C, taps, tail, (int)act);
    if (taps > 1) {
      hipLaunchKernelGGL((causal_conv_tail_kernel<act_t>),
          dim3(B, gc.x), dim3(threads), 0, stream,
          (const act_t*)x.data_ptr(), x.stride(0),
          (act_t*)conv_state.data_ptr(), cu_seqlens.data_ptr<int>(),
          state_slots.data_ptr<int>(), seq_starts.data_ptr<int>(), C, taps,
          tail);
    }
  });
}

}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("causal_conv_update(Tensor(a!) out, Tensor x, Tensor weight, Tensor bias, Tensor(b!) conv_state, Tensor cu_seqlens, Tensor state_slots, Tensor seq_starts, Tensor token_seq, int act) -> ()");
}
TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("causal_conv_update", &kaito::causal_conv_update);
}
