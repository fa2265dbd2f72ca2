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

// ---- segment-parallel scan for prompt-sized steps --------------------------
// The recurrence is linear, S_t = a_t S_(t-1) + b_t, so the rows of a step
// are cut into fixed segments of SEG rows (chunk borders may fall anywhere
// inside one) and scanned in three launches:
//   1. per (segment, channel): walk the rows from a zero carry with the
//      running product P of a's; a row that starts a chunk replaces the
//      running state by that chunk's initial state and sets P = 0 (nothing
//      before it can reach past it). Emit (P, E = state at segment end).
//   2. per channel: fold the segments in order, S_in[s+1] = P[s] S_in[s] + E[s].
//   3. per (segment, channel): walk again from the true S_in, write the
//      outputs, and store the state at every chunk's last row.
constexpr int SEG = 64;

template <typename T>
KAITO_DEV void rglru_coeffs(const float* __restrict__ gp, const int64_t t,
                            const int bw, const float rate,
                            const T* __restrict__ u, const int64_t u_s0,
                            const int c, float& a, float& drive) {
  const float rg = sigmoid_f(gp[t * (2 * bw)]);
  const float ig = sigmoid_f(gp[t * (2 * bw) + bw]);
  const float log_a = -rg * rate;
  a = expf(log_a);
  drive = sqrtf(-expm1f(2.0f * log_a)) * ig * act_ld(u + t * u_s0 + c);
}

template <typename T, int PHASE>
__global__ void rglru_segment_kernel(
    T* __restrict__ out, const T* __restrict__ u, const int64_t u_s0,
    const float* __restrict__ gates, const T* __restrict__ y,
    const int64_t y_s0, const float* __restrict__ decay_rate,
    float* __restrict__ state, float* __restrict__ seg_p,
    float* __restrict__ seg_e, const float* __restrict__ seg_in,
    const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ starts, const int* __restrict__ token_seq,
    const int T_total, const int W, const int bw) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int blk = c / bw, cc = c % bw;
  const float rate = decay_rate[c];
  const float* gp = gates + ((int64_t)blk * T_total) * (2 * bw) + cc;
  const int t0 = s * SEG, t1 = min(T_total, t0 + SEG);
  float S = PHASE == 3 ? seg_in[(int64_t)s * W + c] : 0.0f;
  float P = 1.0f;
  for (int t = t0; t < t1; t++) {
    const int b = token_seq[t];
    const int slot = b >= 0 ? slots[b] : -1;
    if (slot < 0) { S = 0.0f; P = 0.0f; continue; }   // padding row
    if (t == cu[b]) {                                  // chunk starts here
      S = starts[b] > 0 ? state[(int64_t)slot * W + c] : 0.0f;
      P = 0.0f;
    }
    float a, drive;
    rglru_coeffs<T>(gp, t, bw, rate, u, u_s0, c, a, drive);
    S = a * S + drive;
    if (PHASE == 1) {
      P *= a;
    } else {
      act_st(out + (int64_t)t * W + c,
             S * gelu_tanh_f(act_ld(y + (int64_t)t * y_s0 + c)));
    }
  }
  if (PHASE == 1) {
    seg_p[(int64_t)s * W + c] = P;
    seg_e[(int64_t)s * W + c] = S;
  }
}

// phase 3 still reads the slots' OLD states at chunk starts, so the new
// states are written by a launch of their own after it
__global__ void rglru_fold_kernel(
    float* __restrict__ seg_in, const float* __restrict__ seg_p,
    const float* __restrict__ seg_e, const int nseg, const int W) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  float S = 0.0f;
  for (int s = 0; s < nseg; s++) {
    seg_in[(int64_t)s * W + c] = S;
    S = seg_p[(int64_t)s * W + c] * S + seg_e[(int64_t)s * W + c];
  }
}

// state at the last row of every chunk = state entering the next row's
// segment position; recomputed from seg_in by walking the chunk's final
// segment up to its last row
template <typename T>
__global__ void rglru_final_state_kernel(
    const T* __restrict__ u, const int64_t u_s0,
    const float* __restrict__ gates, const float* __restrict__ decay_rate,
    float* state, const float* old_state,
    const float* __restrict__ seg_in, const int* __restrict__ cu,
    const int* __restrict__ slots, const int* __restrict__ starts,
    const int* __restrict__ token_seq, const int T_total, const int W,
    const int bw) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int slot = slots[b];
  const int r0 = cu[b], r1 = cu[b + 1];
  if (slot < 0 || r1 <= r0) return;
  const int blk = c / bw, cc = c % bw;
  const float rate = decay_rate[c];
  const float* gp = gates + ((int64_t)blk * T_total) * (2 * bw) + cc;
  const int s = (r1 - 1) / SEG;
  int t = s * SEG;
  float S = seg_in[(int64_t)s * W + c];
  // a chunk start inside the segment cuts the carry; the last one at or
  // before row r1-1 that matters is this chunk's own start
  if (r0 >= t) {
    t = r0;
    S = starts[b] > 0 ? old_state[(int64_t)slot * W + c] : 0.0f;
  }
  for (; t < r1; t++) {
    float a, drive;
    rglru_coeffs<T>(gp, t, bw, rate, u, u_s0, c, a, drive);
    S = a * S + drive;
  }
  state[(int64_t)slot * W + c] = S;
}

template <typename T>
void run_rglru_segments(hipStream_t stream, at::Tensor& out,
                        const at::Tensor& u, const at::Tensor& gates,
                        const at::Tensor& y, const at::Tensor& decay_rate,
                        at::Tensor& state, at::Tensor& seg_p,
                        at::Tensor& seg_e, at::Tensor& seg_in,
                        const at::Tensor& cu, const at::Tensor& slots,
                        const at::Tensor& starts, const at::Tensor& token_seq,
                        int nseg, int cblocks, int threads, int bw) {
  const int T_total = u.size(0), W = u.size(1), B = slots.size(0);
#define KAITO_RGLRU_SEG(PHASE_)                                              \
  hipLaunchKernelGGL((rglru_segment_kernel<T, PHASE_>),                      \
      dim3(nseg, cblocks), dim3(threads), 0, stream, (T*)out.data_ptr(),     \
      (const T*)u.data_ptr(), u.stride(0), gates.data_ptr<float>(),          \
      (const T*)y.data_ptr(), y.stride(0), decay_rate.data_ptr<float>(),     \
      state.data_ptr<float>(), seg_p.data_ptr<float>(),                      \
      seg_e.data_ptr<float>(), seg_in.data_ptr<float>(),                     \
      cu.data_ptr<int>(), slots.data_ptr<int>(), starts.data_ptr<int>(),     \
      token_seq.data_ptr<int>(), T_total, W, bw)
  KAITO_RGLRU_SEG(1);
  hipLaunchKernelGGL(rglru_fold_kernel, dim3(cblocks), dim3(threads), 0,
      stream, seg_in.data_ptr<float>(), seg_p.data_ptr<float>(),
      seg_e.data_ptr<float>(), nseg, W);
  KAITO_RGLRU_SEG(3);
#undef KAITO_RGLRU_SEG
  // each (chunk, channel) thread reads its slot's old value before it
  // overwrites it, and nobody else touches that element in this launch
  hipLaunchKernelGGL((rglru_final_state_kernel<T>), dim3(B, cblocks),
      dim3(threads), 0, stream, (const T*)u.data_ptr(), u.stride(0),
      gates.data_ptr<float>(), decay_rate.data_ptr<float>(),
      state.data_ptr<float>(), state.data_ptr<float>(),
      seg_in.data_ptr<float>(), cu.data_ptr<int>(), slots.data_ptr<int>(),
      starts.data_ptr<int>(), token_seq.data_ptr<int>(), T_total, W, bw);
}

}  // namespace

void rglru_scan(at::Tensor out, at::Tensor u, at::Tensor gates, at::Tensor y,
                at::Tensor decay_rate, at::Tensor state,
                at::Tensor cu_seqlens, at::Tensor state_slots,
                at::Tensor seq_starts, at::Tensor token_seq) {
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
  const int cblocks = (W + threads - 1) / threads;
  if (token_seq.numel() > 0 && T >= 4 * B && T >= 2 * SEG) {
    // prompt-sized step: segment-parallel scan
    KAITO_CHECK_I32(token_seq);
    TORCH_CHECK(token_seq.size(0) == T);
    const int nseg = (T + SEG - 1) / SEG;
    auto f32 = state.options();
    at::Tensor seg_p = at::empty({nseg, W}, f32);
    at::Tensor seg_e = at::empty({nseg, W}, f32);
    at::Tensor seg_in = at::empty({nseg, W}, f32);
    KAITO_DISPATCH_ACT(u, {
      run_rglru_segments<act_t>(stream, out, u, gates, y, decay_rate, state,
                                seg_p, seg_e, seg_in, cu_seqlens, state_slots,
                                seq_starts, token_seq, nseg, cblocks, threads,
                                W / NB);
    });
    return;
  }
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
  m.def("rglru_scan(Tensor(a!) out, Tensor u, Tensor gates, Tensor y, Tensor decay_rate, Tensor(b!) state, Tensor cu_seqlens, Tensor state_slots, Tensor seq_starts, Tensor token_seq) -> ()");
}
TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("rglru_scan", &kaito::rglru_scan);
}
