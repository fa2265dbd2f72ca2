// Gated delta rule (linear attention with a matrix state per head) for
// batches of chunks.
//
// Per head h (query/key head g = h / (H/G)) the state S is [D, V] f32.
// For each token, in order:
//     S <- decay * S
//     u  = beta * (v - S^T k)
//     S <- S + k u^T
//     o  = S^T q
// with k, q unit-normalised (q also scaled by D^-1/2),
// decay = exp(-exp(a_log) * softplus(a + dt_bias)), beta = sigmoid(b).
// The read-out is RMS-normed over V, weighted and gated by silu(gate).
//
// Three launches:
//   1. prep (token-parallel): unit-norm q/k, decay and beta → f32 scratch
//   2. recurrence: thread (j, part) owns rows [part*DP, part*DP+DP) of
//      column j of S in registers; tokens are staged through LDS eight at
//      a time, so the token loop itself has no barrier and the only
//      cross-lane traffic is the PARTS-wide butterfly. Fast path: one
//      single-wave workgroup per (chunk, head, group of columns); other
//      sizes: one workgroup per (chunk, head)
//   3. epilogue (token-parallel): RMS norm, weight, silu gate, store
// A chunk that starts at position 0 starts from S = 0 whatever its slot
// held; slots < 0 are padding and skipped.
#include "mix_common.h"
#include <cstdlib>

namespace kaito {

namespace {

constexpr int TOK_TILE = 8;

template <typename T>
__global__ void delta_prep_kernel(
    float* __restrict__ qn, float* __restrict__ kn,      // [T, G, D]
    float* __restrict__ kq,                               // [T, G] = qn . kn
    float* __restrict__ decay, float* __restrict__ beta,  // [T, H]
    const T* __restrict__ q, const int64_t q_s0, const int64_t q_s1,
    const T* __restrict__ k, const int64_t k_s0, const int64_t k_s1,
    const T* __restrict__ a, const int64_t a_s0,
    const T* __restrict__ b, const int64_t b_s0,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    const int G, const int D, const int H, const float qk_eps) {
  // one wave per (token, qk head); wave 0 of head 0 also does decay/beta
  const int t = blockIdx.x;
  const int g = blockIdx.y;
  const int lane = threadIdx.x;
  const T* qr = q + (int64_t)t * q_s0 + (int64_t)g * q_s1;
  const T* kr = k + (int64_t)t * k_s0 + (int64_t)g * k_s1;
  float sq = 0.f, sk = 0.f, sqk = 0.f;
  for (int d = lane; d < D; d += 64) {
    const float qv = act_ld(qr + d), kv = act_ld(kr + d);
    sq += qv * qv;
    sk += kv * kv;
    sqk += qv * kv;
  }
  sq = wave_reduce_sum(sq);
  sk = wave_reduce_sum(sk);
  sqk = wave_reduce_sum(sqk);
  const float iq = (1.0f / sqrtf(sq + qk_eps)) * (1.0f / sqrtf((float)D));
  const float ik = 1.0f / sqrtf(sk + qk_eps);
  float* qo = qn + ((int64_t)t * G + g) * D;
  float* ko = kn + ((int64_t)t * G + g) * D;
  for (int d = lane; d < D; d += 64) {
    qo[d] = act_ld(qr + d) * iq;
    ko[d] = act_ld(kr + d) * ik;
  }
  if (lane == 0) kq[(int64_t)t * G + g] = sqk * iq * ik;
  if (g == 0) {
    for (int h = lane; h < H; h += 64) {
      const float av = act_ld(a + (int64_t)t * a_s0 + h);
      const float bv = act_ld(b + (int64_t)t * b_s0 + h);
      decay[(int64_t)t * H + h] =
          expf(-expf(a_log[h]) * softplus_f(av + dt_bias[h]));
      beta[(int64_t)t * H + h] = sigmoid_f(bv);
    }
  }
}

template <int PARTS>
KAITO_DEV float parts_sum(float x) {
#pragma unroll
  for (int off = 1; off < PARTS; off <<= 1) x += __shfl_xor(x, off, 64);
  return x;
}

template <typename T, int DP, int PARTS>
__global__ void delta_recurrence_kernel(
    float* __restrict__ o,                                 // [T, H, V]
    const float* __restrict__ qn, const float* __restrict__ kn,
    const T* __restrict__ v, const int64_t v_s0, const int64_t v_s1,
    const float* __restrict__ decay, const float* __restrict__ beta,
    float* __restrict__ state,                             // [slots, H, D, V]
    const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ starts, const int G, const int D, const int H,
    const int V) {
  extern __shared__ float lds[];
  const int b = blockIdx.x, h = blockIdx.y;
  const int slot = slots[b];
  const int r0 = cu[b], r1 = cu[b + 1];
  if (slot < 0 || r1 <= r0) return;
  const int g = h / (H / G);
  const int tid = threadIdx.x;
  const int j = tid / PARTS;          // state column (value dim)
  const int part = tid % PARTS;       // which DP rows of it
  const bool live = j < V;
  const int d0 = part * DP;
  // LDS tile: per token [k: D][q: D][v: V][decay, beta]
  const int row = 2 * D + V + 2;
  float S[DP];
  float* sp = state + (((int64_t)slot * H + h) * D) * V + j;
  const bool carried = starts[b] > 0;
#pragma unroll
  for (int i = 0; i < DP; i++) {
    const int d = d0 + i;
    S[i] = (carried && live && d < D) ? sp[(int64_t)d * V] : 0.0f;
  }
  for (int t0 = r0; t0 < r1; t0 += TOK_TILE) {
    const int nt = min(TOK_TILE, r1 - t0);
    __syncthreads();                  // previous tile fully consumed
    for (int e = tid; e < nt * row; e += blockDim.x) {
      const int tt = e / row, c = e % row;
      const int t = t0 + tt;
      float val;
      if (c < D) val = kn[((int64_t)t * G + g) * D + c];
      else if (c < 2 * D) val = qn[((int64_t)t * G + g) * D + (c - D)];
      else if (c < 2 * D + V)
        val = act_ld(v + (int64_t)t * v_s0 + (int64_t)h * v_s1 + (c - 2 * D));
      else if (c == 2 * D + V) val = decay[(int64_t)t * H + h];
      else val = beta[(int64_t)t * H + h];
      lds[e] = val;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; tt++) {
      const float* lk = lds + tt * row;
      const float* lq = lk + D;
      const float dec = lk[2 * D + V], bet = lk[2 * D + V + 1];
      const float vj = live ? lk[2 * D + j] : 0.0f;
      float pred = 0.0f;
#pragma unroll
      for (int i = 0; i < DP; i++) {
        const int d = d0 + i;
        const float kd = d < D ? lk[d] : 0.0f;
        S[i] *= dec;
        pred += S[i] * kd;
      }
      pred = parts_sum<PARTS>(pred);
      const float u = bet * (vj - pred);
      float oj = 0.0f;
#pragma unroll
      for (int i = 0; i < DP; i++) {
        const int d = d0 + i;
        const float kd = d < D ? lk[d] : 0.0f;
        const float qd = d < D ? lq[d] : 0.0f;
        S[i] += kd * u;
        oj += S[i] * qd;
      }
      oj = parts_sum<PARTS>(oj);
      if (live && part == 0)
        o[((int64_t)(t0 + tt) * H + h) * V + j] = oj;
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < DP; i++) {
      const int d = d0 + i;
      if (d < D) sp[(int64_t)d * V] = S[i];
    }
  }
}

// Wave-per-column-group recurrence (the fast path; dim % 4 == 0). The
// columns of S are independent, so a (chunk, head) pair is split over
// V / VB single-wave workgroups of VB = 64 / PARTS columns each: many
// more waves in flight than one workgroup per head, no workgroup barrier
// between waves, and the PARTS-wide sums are DPP butterflies. Token tiles
// are double-buffered: the next tile's global loads are issued before the
// current tile is consumed and parked in LDS afterwards. k and q rows are
// zero-padded to DP * PARTS in LDS so the inner loops read unconditional
// float4s; the dot products run on four independent accumulators.
template <typename T, int DP, int PARTS>
__global__ __launch_bounds__(64) void delta_recurrence_wave_kernel(
    float* __restrict__ o,                                 // [T, H, V]
    const float* __restrict__ qn, const float* __restrict__ kn,
    const float* __restrict__ kq,
    const T* __restrict__ v, const int64_t v_s0, const int64_t v_s1,
    const float* __restrict__ decay, const float* __restrict__ beta,
    float* __restrict__ state,                             // [slots, H, D, V]
    const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ starts, const int G, const int D, const int H,
    const int V) {
  constexpr int TT = TOK_TILE;
  constexpr int VB = 64 / PARTS;
  constexpr int DPAD = DP * PARTS;
  // In LDS each part's DP-slice of a k or q row is followed by 4 floats of
  // padding: lanes of different parts read their slices in the same
  // instruction, and slices a multiple of 32 floats apart would all land in
  // the same banks.
  constexpr int DPS = DP + 4;
  constexpr int KROW = PARTS * DPS;
  constexpr int ROW = 2 * KROW + VB + 4;      // k | q | v | decay beta k.q -
  constexpr int KQ4 = TT * DPAD / 4 / 64;     // float4 loads per lane
  constexpr int VN = (TT * VB + 63) / 64;
  __shared__ __attribute__((aligned(16))) float lds[2][TT * ROW];
  const int b = blockIdx.x, h = blockIdx.y;
  const int slot = slots[b];
  const int r0 = cu[b], r1 = cu[b + 1];
  if (slot < 0 || r1 <= r0) return;
  const int g = h / (H / G);
  const int tid = threadIdx.x;
  const int part = tid % PARTS;
  const int jl = tid / PARTS;                 // column inside the group
  const int j = blockIdx.z * VB + jl;
  const bool live = j < V;
  const int d0 = part * DP;
  float S[DP];
  float* sp = state + (((int64_t)slot * H + h) * D) * V + j;
  const bool carried = starts[b] > 0;
#pragma unroll
  for (int i = 0; i < DP; i++) {
    const int d = d0 + i;
    S[i] = (carried && live && d < D) ? sp[(int64_t)d * V] : 0.0f;
  }

  float4_t rk[KQ4], rq[KQ4];
  float rv[VN], rdb = 0.f;
  auto fetch = [&](int t0) {
    const int nt = min(TT, r1 - t0);
#pragma unroll
    for (int i = 0; i < KQ4; i++) {
      const int e = tid + i * 64;
      const int tt = e / (DPAD / 4), d = (e % (DPAD / 4)) * 4;
      const bool ok = tt < nt && d < D;
      const int64_t src = ((int64_t)(t0 + tt) * G + g) * D + d;
      rk[i] = ok ? *reinterpret_cast<const float4_t*>(kn + src)
                 : float4_t{0.f, 0.f, 0.f, 0.f};
      rq[i] = ok ? *reinterpret_cast<const float4_t*>(qn + src)
                 : float4_t{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int i = 0; i < VN; i++) {
      const int e = tid + i * 64;
      const int tt = e / VB, c = blockIdx.z * VB + e % VB;
      rv[i] = (e < TT * VB && tt < nt && c < V)
          ? act_ld(v + (int64_t)(t0 + tt) * v_s0 + (int64_t)h * v_s1 + c)
          : 0.f;
    }
    if (tid < 3 * TT) {
      const int tt = tid / 3, which = tid % 3;
      if (tt >= nt) rdb = 0.f;
      else if (which == 2) rdb = kq[(int64_t)(t0 + tt) * G + g];
      else rdb = (which ? beta : decay)[(int64_t)(t0 + tt) * H + h];
    }
  };
  auto park = [&](float* buf) {
#pragma unroll
    for (int i = 0; i < KQ4; i++) {
      const int e = tid + i * 64;
      const int tt = e / (DPAD / 4), d = (e % (DPAD / 4)) * 4;
      const int dd = (d / DP) * DPS + d % DP;
      *reinterpret_cast<float4_t*>(buf + tt * ROW + dd) = rk[i];
      *reinterpret_cast<float4_t*>(buf + tt * ROW + KROW + dd) = rq[i];
    }
#pragma unroll
    for (int i = 0; i < VN; i++) {
      const int e = tid + i * 64;
      if (e < TT * VB) buf[(e / VB) * ROW + 2 * KROW + e % VB] = rv[i];
    }
    if (tid < 3 * TT) buf[(tid / 3) * ROW + 2 * KROW + VB + tid % 3] = rdb;
  };

  fetch(r0);
  park(lds[0]);
  __syncthreads();
  int cur = 0;
  for (int t0 = r0; t0 < r1; t0 += TT) {
    const int nt = min(TT, r1 - t0);
    const bool more = t0 + TT < r1;
    if (more) fetch(t0 + TT);
    const float* buf = lds[cur];
    for (int tt = 0; tt < nt; tt++) {
      const float* lk = buf + tt * ROW + part * DPS;
      const float* lq = lk + KROW;
      const float dec = buf[tt * ROW + 2 * KROW + VB];
      const float bet = buf[tt * ROW + 2 * KROW + VB + 1];
      const float kqv = buf[tt * ROW + 2 * KROW + VB + 2];
      const float vj = buf[tt * ROW + 2 * KROW + jl];
      // Both read-outs are taken from the state BEFORE this token: with
      // S' = dec S + k u^T,  S'^T q = dec S^T q + u (k.q), so one pass and
      // one reduction stage give the prediction and the output, and the
      // update pass that follows has nothing waiting on it.
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
      float b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
#pragma unroll
      for (int i = 0; i < DP; i += 4) {
        const float4_t k4 = *reinterpret_cast<const float4_t*>(lk + i);
        const float4_t q4 = *reinterpret_cast<const float4_t*>(lq + i);
        a0 += S[i] * k4[0]; a1 += S[i + 1] * k4[1];
        a2 += S[i + 2] * k4[2]; a3 += S[i + 3] * k4[3];
        b0 += S[i] * q4[0]; b1 += S[i + 1] * q4[1];
        b2 += S[i + 2] * q4[2]; b3 += S[i + 3] * q4[3];
      }
      const float sk = group_reduce_sum<PARTS>((a0 + a1) + (a2 + a3));
      const float sq = group_reduce_sum<PARTS>((b0 + b1) + (b2 + b3));
      const float u = bet * (vj - dec * sk);
      const float oj = dec * sq + u * kqv;
#pragma unroll
      for (int i = 0; i < DP; i += 4) {
        const float4_t k4 = *reinterpret_cast<const float4_t*>(lk + i);
        S[i] = dec * S[i] + k4[0] * u;
        S[i + 1] = dec * S[i + 1] + k4[1] * u;
        S[i + 2] = dec * S[i + 2] + k4[2] * u;
        S[i + 3] = dec * S[i + 3] + k4[3] * u;
      }
      if (live && part == 0)
        o[((int64_t)(t0 + tt) * H + h) * V + j] = oj;
    }
    if (more) park(lds[cur ^ 1]);
    __syncthreads();
    cur ^= 1;
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < DP; i++) {
      const int d = d0 + i;
      if (d < D) sp[(int64_t)d * V] = S[i];
    }
  }
}

template <typename T>
__global__ void delta_epilogue_kernel(
    T* __restrict__ out,                                   // [T, H*V]
    const float* __restrict__ o,                           // [T, H, V]
    const T* __restrict__ gate, const int64_t g_s0, const int64_t g_s1,
    const float* __restrict__ norm_w, const int H, const int V,
    const float eps) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + ((int64_t)t * H + h) * V;
  float ss = 0.f;
  for (int j = lane; j < V; j += 64) ss += orow[j] * orow[j];
  ss = wave_reduce_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)V + eps);
  const T* gr = gate + (int64_t)t * g_s0 + (int64_t)h * g_s1;
  T* dst = out + ((int64_t)t * H + h) * V;
  for (int j = lane; j < V; j += 64)
    act_st(dst + j, orow[j] * inv * norm_w[j] * silu_f(act_ld(gr + j)));
}

template <typename T, int DP, int PARTS>
void launch_recurrence(int B, int H, int threads, size_t lds_bytes,
                       hipStream_t stream, float* o, const float* qn,
                       const float* kn, const at::Tensor& v,
                       const float* decay, const float* beta, float* state,
                       const int* cu, const int* slots, const int* starts,
                       int G, int D, int V) {
  hipLaunchKernelGGL((delta_recurrence_kernel<T, DP, PARTS>), dim3(B, H),
      dim3(threads), lds_bytes, stream, o, qn, kn, (const T*)v.data_ptr(),
      v.stride(0), v.stride(1), decay, beta, state, cu, slots, starts, G, D,
      H, V);
}

#define KAITO_DELTA_CASE(DP_, PARTS_)                                        \
  if (dp == DP_ && parts == PARTS_) {                                        \
    launch_recurrence<T, DP_, PARTS_>(B, H, threads, lds_bytes, stream,      \
        o.data_ptr<float>(), qn.data_ptr<float>(), kn.data_ptr<float>(), v,  \
        decay.data_ptr<float>(), beta.data_ptr<float>(),                     \
        state.data_ptr<float>(), cu_seqlens.data_ptr<int>(),                 \
        state_slots.data_ptr<int>(), seq_starts.data_ptr<int>(), G, D, V);   \
  }

template <typename T>
void run_delta(hipStream_t stream, at::Tensor& out, const at::Tensor& q,
               const at::Tensor& k, const at::Tensor& v,
               const at::Tensor& gate, const at::Tensor& a,
               const at::Tensor& b, const at::Tensor& a_log,
               const at::Tensor& dt_bias, const at::Tensor& norm_w,
               at::Tensor& state, const at::Tensor& cu_seqlens,
               const at::Tensor& state_slots, const at::Tensor& seq_starts,
               at::Tensor& qn, at::Tensor& kn, at::Tensor& kq,
               at::Tensor& decay, at::Tensor& beta, at::Tensor& o, int dp,
               int parts,
               int threads, size_t lds_bytes, float qk_eps, float norm_eps) {
  const int T_ = q.size(0), G = q.size(1), D = q.size(2);
  const int H = v.size(1), V = v.size(2);
  const int B = state_slots.size(0);
  hipLaunchKernelGGL((delta_prep_kernel<T>), dim3(T_, G), dim3(64), 0,
      stream, qn.data_ptr<float>(), kn.data_ptr<float>(),
      kq.data_ptr<float>(), decay.data_ptr<float>(), beta.data_ptr<float>(),
      (const T*)q.data_ptr(), q.stride(0), q.stride(1),
      (const T*)k.data_ptr(), k.stride(0), k.stride(1),
      (const T*)a.data_ptr(), a.stride(0), (const T*)b.data_ptr(),
      b.stride(0), a_log.data_ptr<float>(), dt_bias.data_ptr<float>(), G, D,
      H, qk_eps);
  int wparts = 1;
  while (wparts * 32 < D) wparts <<= 1;
  if (D % 4 == 0 && wparts <= 8) {
    // fast path: single-wave workgroups over groups of 64 / PARTS columns.
    // A wave64 VALU instruction occupies its SIMD for four cycles and the
    // token loop is serial, so the kernel is bound by how many SIMDs have a
    // wave: with few (chunk, head, column-group) triples, halve the rows per
    // lane (DP 16) to double the waves.
    int dpw = 32;
    const int64_t waves32 = (int64_t)B * H * ((V * wparts + 63) / 64);
    // KAITO_DELTA_ROWS_PER_LANE=16|32 pins the choice (A/B runs, tests)
    const char* pin = getenv("KAITO_DELTA_ROWS_PER_LANE");
    const int want = pin ? atoi(pin) : (waves32 < 4096 ? 16 : 32);
    if (want == 16 && wparts * 2 <= 16) { dpw = 16; wparts *= 2; }
#define KAITO_DELTA_WAVE(DP_, PARTS_)                                        \
    if (dpw == DP_ && wparts == PARTS_) {                                    \
      constexpr int VB = 64 / PARTS_;                                        \
      hipLaunchKernelGGL((delta_recurrence_wave_kernel<T, DP_, PARTS_>),     \
          dim3(B, H, (V + VB - 1) / VB), dim3(64), 0, stream,                \
          o.data_ptr<float>(), qn.data_ptr<float>(), kn.data_ptr<float>(),   \
          kq.data_ptr<float>(), (const T*)v.data_ptr(), v.stride(0),         \
          v.stride(1), decay.data_ptr<float>(), beta.data_ptr<float>(),      \
          state.data_ptr<float>(), cu_seqlens.data_ptr<int>(),               \
          state_slots.data_ptr<int>(), seq_starts.data_ptr<int>(), G, D, H,  \
          V);                                                                \
    }
    KAITO_DELTA_WAVE(32, 1) KAITO_DELTA_WAVE(32, 2) KAITO_DELTA_WAVE(32, 4)
    KAITO_DELTA_WAVE(32, 8) KAITO_DELTA_WAVE(16, 2) KAITO_DELTA_WAVE(16, 4)
    KAITO_DELTA_WAVE(16, 8) KAITO_DELTA_WAVE(16, 16)
#undef KAITO_DELTA_WAVE
  } else {
    KAITO_DELTA_CASE(32, 1) KAITO_DELTA_CASE(32, 2) KAITO_DELTA_CASE(32, 4)
    KAITO_DELTA_CASE(32, 8) KAITO_DELTA_CASE(64, 1) KAITO_DELTA_CASE(64, 2)
    KAITO_DELTA_CASE(64, 4) KAITO_DELTA_CASE(64, 8)
  }
  hipLaunchKernelGGL((delta_epilogue_kernel<T>), dim3(T_, H), dim3(64), 0,
      stream, (T*)out.data_ptr(), o.data_ptr<float>(),
      (const T*)gate.data_ptr(), gate.stride(0), gate.stride(1),
      norm_w.data_ptr<float>(), H, V, norm_eps);
}
#undef KAITO_DELTA_CASE

}  // namespace

void gated_delta_rule(at::Tensor out, at::Tensor q, at::Tensor k,
                      at::Tensor v, at::Tensor gate, at::Tensor a,
                      at::Tensor b, at::Tensor a_log, at::Tensor dt_bias,
                      at::Tensor norm_w, at::Tensor state,
                      at::Tensor cu_seqlens, at::Tensor state_slots,
                      at::Tensor seq_starts, double qk_eps, double norm_eps) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && k.dim() == 3 && v.dim() == 3 &&
              gate.dim() == 3 && a.dim() == 2 && b.dim() == 2);
  const int T = q.size(0), G = q.size(1), D = q.size(2);
  const int H = v.size(1), V = v.size(2);
  TORCH_CHECK(k.size(0) == T && k.size(1) == G && k.size(2) == D);
  TORCH_CHECK(v.size(0) == T && gate.size(0) == T && gate.size(1) == H &&
              gate.size(2) == V && a.size(0) == T && a.size(1) == H &&
              b.size(0) == T && b.size(1) == H);
  TORCH_CHECK(H % G == 0, "heads must be a multiple of qk heads");
  for (const at::Tensor* t : {&q, &k, &v, &gate, &a, &b})
    TORCH_CHECK(t->stride(-1) == 1 && t->dtype() == q.dtype(),
                "inputs must share a dtype and have unit inner stride");
  TORCH_CHECK(out.is_contiguous() && out.dtype() == q.dtype() &&
              out.numel() == (int64_t)T * H * V);
  KAITO_CHECK_F32(a_log); KAITO_CHECK_F32(dt_bias); KAITO_CHECK_F32(norm_w);
  KAITO_CHECK_F32(state);
  TORCH_CHECK(a_log.numel() == H && dt_bias.numel() == H &&
              norm_w.numel() == V);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D &&
              state.size(3) == V);
  KAITO_CHECK_I32(cu_seqlens); KAITO_CHECK_I32(state_slots);
  KAITO_CHECK_I32(seq_starts);
  const int B = state_slots.size(0);
  TORCH_CHECK(cu_seqlens.size(0) == B + 1 && seq_starts.size(0) == B);
  if (T == 0 || B == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  auto f32 = q.options().dtype(at::kFloat);
  at::Tensor qn = at::empty({T, G, D}, f32), kn = at::empty({T, G, D}, f32);
  at::Tensor decay = at::empty({T, H}, f32), beta = at::empty({T, H}, f32);
  at::Tensor kq = at::empty({T, G}, f32);
  // rows of padding chunks are never written by the recurrence: zero so
  // the epilogue reads defined values
  at::Tensor o = at::zeros({T, H, V}, f32);

  // rows per thread (DP) and threads per state column (PARTS)
  int dp = 32, parts = 1;
  while (parts * dp < D) parts <<= 1;
  if (parts > 8 || (int64_t)V * parts > 1024) {
    dp = 64; parts = 1;
    while (parts * dp < D) parts <<= 1;
  }
  TORCH_CHECK(parts <= 8 && (int64_t)V * parts <= 1024,
              "gated_delta_rule: head too large (dim ", D, ", vdim ", V, ")");
  const int threads = ((V * parts + 63) / 64) * 64;
  const size_t lds_bytes = (size_t)TOK_TILE * (2 * D + V + 2) * sizeof(float);
  TORCH_CHECK(lds_bytes <= 64 * 1024);

  KAITO_DISPATCH_ACT(q, {
    run_delta<act_t>(stream, out, q, k, v, gate, a, b, a_log, dt_bias, norm_w,
                     state, cu_seqlens, state_slots, seq_starts, qn, kn, kq,
                     decay, beta, o, dp, parts, threads, lds_bytes,
                     (float)qk_eps, (float)norm_eps);
  });
}

}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("gated_delta_rule(Tensor(a!) out, Tensor q, Tensor k, Tensor v, Tensor gate, Tensor a, Tensor b, Tensor a_log, Tensor dt_bias, Tensor norm_w, Tensor(b!) state, Tensor cu_seqlens, Tensor state_slots, Tensor seq_starts, float qk_eps, float norm_eps) -> ()");
}
TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("gated_delta_rule", &kaito::gated_delta_rule);
}
