// Linear recurrences with a matrix state and ONE scalar decay per head and
// token, for batches of chunks (prompt portions and single decode tokens
// alike):
//
//     S_t = keep_t * S_(t-1) + take_t * k_t v_t^T        S: [D, V] f32
//     o_t = S_t^T q_t
//
// Two mixers are built on it:
//
//   mlstm_scan  matrix memory with exponential gating. Log gates
//               i = cap tanh(ipre / cap), f = logsigmoid(cap tanh(fpre / cap)),
//               running maximum m (0 at the start of a sequence):
//                 m_t = max(f_t + m_(t-1), i_t)
//                 keep_t = exp(f_t + m_(t-1) - m_t),  take_t = exp(i_t - m_t)
//               The normaliser n_t = keep n + take k is carried as one more
//               state column whose value is 1, so n_t . q_t falls out of the
//               same pass. Read-out o / (max(|n.q|, exp(-m)) + floor), per-head
//               RMS norm, weight, sigmoid output gate.
//   ssd_scan    selective state space: step d = softplus(dt + bias),
//               keep = exp(-exp(a_log) d), take = d, k = B, q = C, v = x;
//               y = o + D x, times silu(z), RMS norm in equal parts, weight.
//
// Launches: gate/step activations (token-parallel) -> [mlstm: running-maximum
// scan, one wave per (chunk, head) over (max, +) pairs; exponentials
// token-parallel] -> recurrence -> epilogue (token-parallel).
//
// Recurrence kernel: one single-wave workgroup per (chunk, head, group of 8
// or 16 state columns); lane (column, part) keeps DP rows of its column in
// registers, so a token costs 3 DP VALU operations per lane and one 4- or
// 8-lane butterfly.
// Token tiles are double-buffered: the next tile's global loads are issued
// before the current tile is consumed and parked in LDS afterwards. k and q
// rows are zero-padded to DP * parts in LDS so the inner loop is unconditional
// float4 reads. A chunk that starts at position 0 starts from S = 0 whatever
// its slot held; slots < 0 are padding and skipped.
#include "mix_common.h"

namespace kaito {

namespace {

constexpr int RTT = 8;          // tokens per tile

// RPARTS lanes share one state column (DP rows each); a wave covers
// RVB = 64 / RPARTS columns
template <typename T, int DP, int RPARTS>
__global__ __launch_bounds__(64) void decay_recurrence_kernel(
    float* __restrict__ o,                    // [T, H, V]
    float* __restrict__ o_n,                  // [T, H] or null
    const T* __restrict__ q, const int64_t q_s0, const int64_t q_s1,
    const T* __restrict__ k, const int64_t k_s0, const int64_t k_s1,
    const T* __restrict__ v, const int64_t v_s0, const int64_t v_s1,
    const float* __restrict__ keep, const float* __restrict__ take,  // [T, H]
    float* __restrict__ state,                // [slots, H, D, V]
    float* __restrict__ state_n,              // [slots, H, D] or null
    const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ starts, const int G, const int D, const int H,
    const int V, const float q_scale) {
  constexpr int RVB = 64 / RPARTS;
  constexpr int DPAD = DP * RPARTS;
  // each part's DP-slice is followed by 4 floats of padding: lanes of
  // different parts read their slices in the same instruction, and slices a
  // multiple of 32 floats apart would land in the same banks
  constexpr int DPS = DP + 4;
  constexpr int KROW = RPARTS * DPS;
  constexpr int ROW = 2 * KROW + RVB + 4;        // k | q | v | keep take - -
  constexpr int KQN = RTT * DPAD / 64;           // k (and q) loads per lane
  constexpr int VN = RTT * RVB / 64;             // v loads per lane
  __shared__ __attribute__((aligned(16))) float lds[2][RTT * ROW];
  const int b = blockIdx.x, h = blockIdx.y;
  const int slot = slots[b];
  const int r0 = cu[b], r1 = cu[b + 1];
  if (slot < 0 || r1 <= r0) return;
  const int g = h / (H / G);
  const int tid = threadIdx.x;
  const int part = tid % RPARTS;
  const int jl = tid / RPARTS;                   // column inside the group
  const int j = blockIdx.z * RVB + jl;
  const bool ncol = state_n != nullptr && j == V;   // the normaliser column
  const bool live = j < V || ncol;
  const int d0 = part * DP;
  float S[DP];
  float* sp = ncol ? state_n + ((int64_t)slot * H + h) * D
                   : state + (((int64_t)slot * H + h) * D) * V + j;
  const int64_t sp_stride = ncol ? 1 : V;
  const bool carried = starts[b] > 0;
#pragma unroll
  for (int i = 0; i < DP; i++) {
    const int d = d0 + i;
    S[i] = (carried && live && d < D) ? sp[(int64_t)d * sp_stride] : 0.0f;
  }

  // fetch() issues every load of a tile unconditionally (rows and columns
  // clamped into range) so that none of them waits for another; what lies
  // outside the tile is zeroed when the registers are parked in LDS
  float rk[KQN], rq[KQN], rv[VN], rc = 0.f;
  int fetched_nt = 0;
  auto fetch = [&](int t0) {
    const int nt = min(RTT, r1 - t0);
    fetched_nt = nt;
#pragma unroll
    for (int i = 0; i < KQN; i++) {
      const int e = tid + i * 64;
      const int tt = min(e / DPAD, nt - 1), d = min(e % DPAD, D - 1);
      rk[i] = act_ld(k + (int64_t)(t0 + tt) * k_s0 + (int64_t)g * k_s1 + d);
      rq[i] = act_ld(q + (int64_t)(t0 + tt) * q_s0 + (int64_t)g * q_s1 + d);
    }
#pragma unroll
    for (int i = 0; i < VN; i++) {
      const int e = tid + i * 64;
      const int tt = min(e / RVB, nt - 1);
      const int c = min((int)blockIdx.z * RVB + e % RVB, V - 1);
      rv[i] = act_ld(v + (int64_t)(t0 + tt) * v_s0 + (int64_t)h * v_s1 + c);
    }
    if (tid < 2 * RTT) {
      const int tt = min(tid >> 1, nt - 1);
      rc = ((tid & 1) ? take : keep)[(int64_t)(t0 + tt) * H + h];
    }
  };
  auto park = [&](float* buf) {
    const int nt = fetched_nt;
#pragma unroll
    for (int i = 0; i < KQN; i++) {
      const int e = tid + i * 64;
      const int tt = e / DPAD, d = e % DPAD;
      const bool ok = tt < nt && d < D;
      const int dd = (d / DP) * DPS + d % DP;
      buf[tt * ROW + dd] = ok ? rk[i] : 0.f;
      buf[tt * ROW + KROW + dd] = ok ? rq[i] * q_scale : 0.f;
    }
#pragma unroll
    for (int i = 0; i < VN; i++) {
      const int e = tid + i * 64;
      const int tt = e / RVB, c = blockIdx.z * RVB + e % RVB;
      float val = 0.f;
      if (tt < nt) {
        if (c < V) val = rv[i];
        else if (state_n != nullptr && c == V) val = 1.0f;
      }
      buf[tt * ROW + 2 * KROW + e % RVB] = val;
    }
    if (tid < 2 * RTT)
      buf[(tid >> 1) * ROW + 2 * KROW + RVB + (tid & 1)] =
          (tid >> 1) < nt ? rc : 0.f;
  };

  fetch(r0);
  park(lds[0]);
  __syncthreads();
  int cur = 0;
  for (int t0 = r0; t0 < r1; t0 += RTT) {
    const int nt = min(RTT, r1 - t0);
    const bool more = t0 + RTT < r1;
    if (more) fetch(t0 + RTT);
    const float* buf = lds[cur];
    for (int tt = 0; tt < nt; tt++) {
      const float* lk = buf + tt * ROW + part * DPS;
      // all LDS reads of the token first, then three passes of mutually
      // independent instructions (a lone wave on a SIMD has nothing else
      // to cover the latency of back-to-back dependent ones)
      float4_t k4[DP / 4], q4[DP / 4];
#pragma unroll
      for (int i = 0; i < DP / 4; i++) {
        k4[i] = *reinterpret_cast<const float4_t*>(lk + 4 * i);
        q4[i] = *reinterpret_cast<const float4_t*>(lk + KROW + 4 * i);
      }
      const float kp = buf[tt * ROW + 2 * KROW + RVB];
      const float u = buf[tt * ROW + 2 * KROW + RVB + 1] *
                      buf[tt * ROW + 2 * KROW + jl];
      float w[DP];
#pragma unroll
      for (int i = 0; i < DP; i++) w[i] = k4[i / 4][i % 4] * u;
#pragma unroll
      for (int i = 0; i < DP; i++) S[i] = kp * S[i] + w[i];
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < DP; i++) acc[i % 4] += S[i] * q4[i / 4][i % 4];
      const float oj =
          group_reduce_sum<RPARTS>((acc[0] + acc[1]) + (acc[2] + acc[3]));
      if (part == 0) {
        if (j < V) o[((int64_t)(t0 + tt) * H + h) * V + j] = oj;
        else if (ncol) o_n[(int64_t)(t0 + tt) * H + h] = oj;
      }
    }
    if (more) park(lds[cur ^ 1]);
    __syncthreads();
    cur ^= 1;
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < DP; i++) {
      const int d = d0 + i;
      if (d < D) sp[(int64_t)d * sp_stride] = S[i];
    }
  }
}

struct RecurrenceArgs {
  float* o; float* o_n;
  const void *q, *k, *v;
  int64_t q_s0, q_s1, k_s0, k_s1, v_s0, v_s1;
  const float *keep, *take;
  float* state; float* state_n;
  const int *cu, *slots, *starts;
  int B, G, D, H, V;
  float q_scale;
};

template <typename T, int DP, int RPARTS>
void launch_recurrence_dp(const RecurrenceArgs& a, hipStream_t stream) {
  constexpr int RVB = 64 / RPARTS;
  const int cols = a.V + (a.state_n ? 1 : 0);
  hipLaunchKernelGGL((decay_recurrence_kernel<T, DP, RPARTS>),
      dim3(a.B, a.H, (cols + RVB - 1) / RVB), dim3(64), 0, stream, a.o, a.o_n,
      (const T*)a.q, a.q_s0, a.q_s1, (const T*)a.k, a.k_s0, a.k_s1,
      (const T*)a.v, a.v_s0, a.v_s1, a.keep, a.take, a.state, a.state_n, a.cu,
      a.slots, a.starts, a.G, a.D, a.H, a.V, a.q_scale);
}

template <typename T>
void launch_recurrence(const RecurrenceArgs& a, hipStream_t stream) {
  // few rows per lane keep the register count low enough for several
  // waves per SIMD; eight lanes per column also double the number of waves
  if (a.D <= 16) launch_recurrence_dp<T, 4, 4>(a, stream);
  else if (a.D <= 32) launch_recurrence_dp<T, 8, 4>(a, stream);
  else if (a.D <= 64) launch_recurrence_dp<T, 8, 8>(a, stream);
  else if (a.D <= 128) launch_recurrence_dp<T, 16, 8>(a, stream);
  else if (a.D <= 256) launch_recurrence_dp<T, 32, 8>(a, stream);
  else TORCH_CHECK(false, "state rows per head must be <= 256, got ", a.D);
}

KAITO_DEV float log_sigmoid_f(float x) {
  return fminf(x, 0.0f) - log1pf(expf(-fabsf(x)));
}

// ---- mLSTM ---------------------------------------------------------------
__global__ void mlstm_gate_kernel(
    float* __restrict__ gi, float* __restrict__ gf,          // [T, H]
    const float* __restrict__ ipre, const int64_t i_s0,
    const float* __restrict__ fpre, const int64_t f_s0, const int n,
    const int H, const float cap) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n) return;
  const int t = e / H, h = e % H;
  const float inv = 1.0f / cap;
  gi[e] = cap * tanhf(ipre[(int64_t)t * i_s0 + h] * inv);
  gf[e] = log_sigmoid_f(cap * tanhf(fpre[(int64_t)t * f_s0 + h] * inv));
}

// m after every token and m before it. The step m -> max(m + f, i) is a
// pair (A, B) acting as m -> max(m + A, B); pairs compose associatively:
// (A1, B1) then (A2, B2) = (A1 + A2, max(B1 + A2, B2)). One wave per
// (chunk, head): every lane folds a contiguous run of tokens into a pair,
// a shuffle scan over the 64 pairs gives each lane the m it starts from,
// and a second pass over the run writes the values.
__global__ __launch_bounds__(64) void mlstm_max_scan_kernel(
    float* __restrict__ m_after, float* __restrict__ m_before,   // [T, H]
    const float* __restrict__ gi, const float* __restrict__ gf,
    float* __restrict__ state_m,                                 // [slots, H]
    const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ starts, const int H) {
  const int b = blockIdx.x / H, h = blockIdx.x % H;
  const int lane = threadIdx.x;
  const int slot = slots[b];
  const int r0 = cu[b], r1 = cu[b + 1];
  if (slot < 0 || r1 <= r0) return;
  const float m0 = starts[b] > 0 ? state_m[(int64_t)slot * H + h] : 0.0f;
  const int run = (r1 - r0 + 63) / 64;
  const int s0 = min(r0 + lane * run, r1), s1 = min(s0 + run, r1);
  float A = 0.0f, B = -INFINITY;
  for (int t = s0; t < s1; t++) {
    const int64_t at = (int64_t)t * H + h;
    const float f = gf[at];
    A += f;
    B = fmaxf(B + f, gi[at]);
  }
  // inclusive scan of the pairs, earlier lanes on the left
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const float Al = __shfl_up(A, off, 64), Bl = __shfl_up(B, off, 64);
    if (lane >= off) {
      B = fmaxf(Bl + A, B);
      A = Al + A;
    }
  }
  const float Ap = __shfl_up(A, 1, 64), Bp = __shfl_up(B, 1, 64);
  float m = lane == 0 ? m0 : fmaxf(m0 + Ap, Bp);
  for (int t = s0; t < s1; t++) {
    const int64_t at = (int64_t)t * H + h;
    m_before[at] = m;
    m = fmaxf(gf[at] + m, gi[at]);
    m_after[at] = m;
  }
  if (lane == 63) state_m[(int64_t)slot * H + h] = fmaxf(m0 + A, B);
}

// in place: gf <- keep, gi <- take, m_before <- exp(-m)
__global__ void mlstm_coef_kernel(float* __restrict__ gi,
                                  float* __restrict__ gf,
                                  const float* __restrict__ m_after,
                                  float* __restrict__ m_before, const int n) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n) return;
  const float m = m_after[e];
  gf[e] = expf(gf[e] + m_before[e] - m);
  gi[e] = expf(gi[e] - m);
  m_before[e] = expf(-m);
}

// one wave per (token, head)
template <typename T>
__global__ void mlstm_epilogue_kernel(
    T* __restrict__ out,                                   // [T, H*V]
    const float* __restrict__ o, const float* __restrict__ o_n,
    const float* __restrict__ floor_m,                     // exp(-m) [T, H]
    const T* __restrict__ gate, const int64_t g_s0, const int64_t g_s1,
    const float* __restrict__ norm_w, const int H, const int V,
    const float norm_eps, const float denom_floor) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int64_t th = (int64_t)t * H + h;
  const float den = fmaxf(fabsf(o_n[th]), floor_m[th]) + denom_floor;
  const float inv_den = 1.0f / den;
  const float* orow = o + th * V;
  float ss = 0.f;
  for (int j = lane; j < V; j += 64) {
    const float x = orow[j] * inv_den;
    ss += x * x;
  }
  ss = wave_reduce_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)V + norm_eps);
  for (int j = lane; j < V; j += 64) {
    const float gz = act_ld(gate + (int64_t)t * g_s0 + (int64_t)h * g_s1 + j);
    act_st(out + th * V + j, orow[j] * inv_den * inv * norm_w[h * V + j] *
                                 sigmoid_f(gz));
  }
}

// ---- SSD -----------------------------------------------------------------
__global__ void ssd_step_kernel(float* __restrict__ keep,
                                float* __restrict__ take,
                                const float* __restrict__ dt,
                                const int64_t dt_s0,
                                const float* __restrict__ a_log,
                                const float* __restrict__ dt_bias,
                                const int n, const int H) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n) return;
  const int t = e / H, h = e % H;
  const float d = softplus_f(dt[(int64_t)t * dt_s0 + h] + dt_bias[h]);
  keep[e] = expf(-expf(a_log[h]) * d);
  take[e] = d;
}

// one workgroup per (token, norm part)
template <typename T>
__global__ void ssd_epilogue_kernel(
    T* __restrict__ out,                                   // [T, H*P]
    const float* __restrict__ o,                           // [T, H*P]
    const T* __restrict__ x, const int64_t x_s0, const int64_t x_s1,
    const T* __restrict__ z, const int64_t z_s0,
    const float* __restrict__ d_skip, const float* __restrict__ norm_w,
    const int inner, const int P, const int part_w, const float norm_eps) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  const int c0 = blockIdx.y * part_w;
  auto value = [&](int c) {
    const int h = c / P, p = c % P;
    const float xv = act_ld(x + (int64_t)t * x_s0 + (int64_t)h * x_s1 + p);
    const float y = o[(int64_t)t * inner + c] + d_skip[h] * xv;
    return y * silu_f(act_ld(z + (int64_t)t * z_s0 + c));
  };
  float ss = 0.f;
  for (int c = c0 + threadIdx.x; c < c0 + part_w; c += blockDim.x) {
    const float y = value(c);
    ss += y * y;
  }
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)part_w + norm_eps);
  for (int c = c0 + threadIdx.x; c < c0 + part_w; c += blockDim.x)
    act_st(out + (int64_t)t * inner + c, value(c) * inv * norm_w[c]);
}

void check_layout(const at::Tensor& cu, const at::Tensor& slots,
                  const at::Tensor& starts) {
  KAITO_CHECK_I32(cu); KAITO_CHECK_I32(slots); KAITO_CHECK_I32(starts);
  TORCH_CHECK(cu.size(0) == slots.size(0) + 1 &&
              starts.size(0) == slots.size(0));
}

}  // namespace

void mlstm_scan(at::Tensor out, at::Tensor q, at::Tensor k, at::Tensor v,
                at::Tensor ogate, at::Tensor ipre, at::Tensor fpre,
                at::Tensor norm_w, at::Tensor state_c, at::Tensor state_n,
                at::Tensor state_m, at::Tensor cu_seqlens,
                at::Tensor state_slots, at::Tensor seq_starts, double cap,
                double q_scale, double norm_eps, double denom_floor) {
  TORCH_CHECK(v.is_cuda() && q.dim() == 3 && k.dim() == 3 && v.dim() == 3 &&
              ogate.dim() == 3 && is_act_dtype(v));
  const int T = v.size(0), H = v.size(1), V = v.size(2), D = q.size(2);
  for (const at::Tensor* t : {&q, &k, &v, &ogate})
    TORCH_CHECK(t->stride(2) == 1 && t->dtype() == v.dtype() &&
                t->size(0) == T && t->size(1) == H);
  TORCH_CHECK(k.size(2) == D && ogate.size(2) == V);
  for (const at::Tensor* t : {&ipre, &fpre})
    TORCH_CHECK(t->is_cuda() && t->dtype() == at::kFloat && t->dim() == 2 &&
                t->size(0) == T && t->size(1) == H && t->stride(1) == 1);
  KAITO_CHECK_F32(norm_w); KAITO_CHECK_F32(state_c); KAITO_CHECK_F32(state_n);
  KAITO_CHECK_F32(state_m);
  TORCH_CHECK(norm_w.numel() == H * V);
  TORCH_CHECK(state_c.dim() == 4 && state_c.size(1) == H &&
              state_c.size(2) == D && state_c.size(3) == V);
  const int64_t nslots = state_c.size(0);
  TORCH_CHECK(state_n.dim() == 3 && state_n.size(0) == nslots &&
              state_n.size(1) == H && state_n.size(2) == D);
  TORCH_CHECK(state_m.dim() == 2 && state_m.size(0) == nslots &&
              state_m.size(1) == H);
  TORCH_CHECK(out.is_contiguous() && out.dtype() == v.dtype() &&
              out.dim() == 2 && out.size(0) == T && out.size(1) == H * V);
  TORCH_CHECK(cap > 0.0);
  check_layout(cu_seqlens, state_slots, seq_starts);
  const int B = state_slots.size(0);
  if (T == 0 || B == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  auto f32 = v.options().dtype(at::kFloat);
  // [gi | gf | m_after | m_before] then [o | o_n]
  at::Tensor coef = at::zeros({4, T, H}, f32);
  // padding chunks are skipped by the recurrence; their rows read zeros
  at::Tensor o = at::zeros({T, H, V}, f32);
  at::Tensor o_n = at::zeros({T, H}, f32);
  float* gi = coef.data_ptr<float>();
  float* gf = gi + (int64_t)T * H;
  float* m_after = gf + (int64_t)T * H;
  float* m_before = m_after + (int64_t)T * H;
  const int n = T * H;
  hipLaunchKernelGGL(mlstm_gate_kernel, dim3((n + 255) / 256), dim3(256), 0,
      stream, gi, gf, ipre.data_ptr<float>(), ipre.stride(0),
      fpre.data_ptr<float>(), fpre.stride(0), n, H, (float)cap);
  hipLaunchKernelGGL(mlstm_max_scan_kernel, dim3(B * H), dim3(64), 0, stream,
      m_after, m_before, gi, gf, state_m.data_ptr<float>(),
      cu_seqlens.data_ptr<int>(), state_slots.data_ptr<int>(),
      seq_starts.data_ptr<int>(), H);
  hipLaunchKernelGGL(mlstm_coef_kernel, dim3((n + 255) / 256), dim3(256), 0,
      stream, gi, gf, m_after, m_before, n);
  RecurrenceArgs a{o.data_ptr<float>(), o_n.data_ptr<float>(), q.data_ptr(),
      k.data_ptr(), v.data_ptr(), q.stride(0), q.stride(1), k.stride(0),
      k.stride(1), v.stride(0), v.stride(1), gf, gi,
      state_c.data_ptr<float>(), state_n.data_ptr<float>(),
      cu_seqlens.data_ptr<int>(), state_slots.data_ptr<int>(),
      seq_starts.data_ptr<int>(), B, H, D, H, V, (float)q_scale};
  KAITO_DISPATCH_ACT(v, {
    launch_recurrence<act_t>(a, stream);
    hipLaunchKernelGGL((mlstm_epilogue_kernel<act_t>), dim3(T, H), dim3(64),
        0, stream, (act_t*)out.data_ptr(), o.data_ptr<float>(),
        o_n.data_ptr<float>(), m_before, (const act_t*)ogate.data_ptr(),
        ogate.stride(0), ogate.stride(1), norm_w.data_ptr<float>(), H, V,
        (float)norm_eps, (float)denom_floor);
  });
}

void ssd_scan(at::Tensor out, at::Tensor x, at::Tensor Bm, at::Tensor Cm,
              at::Tensor dt, at::Tensor z, at::Tensor a_log,
              at::Tensor dt_bias, at::Tensor d_skip, at::Tensor norm_w,
              at::Tensor state, at::Tensor cu_seqlens, at::Tensor state_slots,
              at::Tensor seq_starts, int64_t norm_groups, double norm_eps) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 3 && Bm.dim() == 3 && Cm.dim() == 3 &&
              z.dim() == 2 && is_act_dtype(x));
  const int T = x.size(0), H = x.size(1), P = x.size(2);
  const int G = Bm.size(1), N = Bm.size(2);
  const int inner = H * P;
  for (const at::Tensor* t : {&x, &Bm, &Cm})
    TORCH_CHECK(t->stride(2) == 1 && t->dtype() == x.dtype() &&
                t->size(0) == T);
  TORCH_CHECK(Cm.size(1) == G && Cm.size(2) == N && G > 0 && H % G == 0);
  TORCH_CHECK(z.stride(1) == 1 && z.dtype() == x.dtype() && z.size(0) == T &&
              z.size(1) == inner);
  TORCH_CHECK(dt.is_cuda() && dt.dtype() == at::kFloat && dt.dim() == 2 &&
              dt.size(0) == T && dt.size(1) == H && dt.stride(1) == 1);
  KAITO_CHECK_F32(a_log); KAITO_CHECK_F32(dt_bias); KAITO_CHECK_F32(d_skip);
  KAITO_CHECK_F32(norm_w); KAITO_CHECK_F32(state);
  TORCH_CHECK(a_log.numel() == H && dt_bias.numel() == H &&
              d_skip.numel() == H && norm_w.numel() == inner);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == N &&
              state.size(3) == P);
  TORCH_CHECK(norm_groups > 0 && inner % norm_groups == 0);
  TORCH_CHECK(out.is_contiguous() && out.dtype() == x.dtype() &&
              out.dim() == 2 && out.size(0) == T && out.size(1) == inner);
  check_layout(cu_seqlens, state_slots, seq_starts);
  const int B = state_slots.size(0);
  if (T == 0 || B == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  auto f32 = x.options().dtype(at::kFloat);
  at::Tensor coef = at::empty({2, T, H}, f32);
  // padding chunks are skipped by the recurrence; their rows read zeros
  at::Tensor o = at::zeros({T, H, P}, f32);
  float* keep = coef.data_ptr<float>();
  float* take = keep + (int64_t)T * H;
  const int n = T * H;
  hipLaunchKernelGGL(ssd_step_kernel, dim3((n + 255) / 256), dim3(256), 0,
      stream, keep, take, dt.data_ptr<float>(), dt.stride(0),
      a_log.data_ptr<float>(), dt_bias.data_ptr<float>(), n, H);
  RecurrenceArgs a{o.data_ptr<float>(), nullptr, Cm.data_ptr(), Bm.data_ptr(),
      x.data_ptr(), Cm.stride(0), Cm.stride(1), Bm.stride(0), Bm.stride(1),
      x.stride(0), x.stride(1), keep, take, state.data_ptr<float>(), nullptr,
      cu_seqlens.data_ptr<int>(), state_slots.data_ptr<int>(),
      seq_starts.data_ptr<int>(), B, G, N, H, P, 1.0f};
  const int part_w = inner / (int)norm_groups;
  const int threads = part_w >= 1024 ? 256 : (part_w >= 256 ? 128 : 64);
  KAITO_DISPATCH_ACT(x, {
    launch_recurrence<act_t>(a, stream);
    hipLaunchKernelGGL((ssd_epilogue_kernel<act_t>),
        dim3(T, (int)norm_groups), dim3(threads), 0, stream,
        (act_t*)out.data_ptr(), o.data_ptr<float>(),
        (const act_t*)x.data_ptr(), x.stride(0), x.stride(1),
        (const act_t*)z.data_ptr(), z.stride(0), d_skip.data_ptr<float>(),
        norm_w.data_ptr<float>(), inner, P, part_w, (float)norm_eps);
  });
}

}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("mlstm_scan(Tensor(a!) out, Tensor q, Tensor k, Tensor v, Tensor ogate, Tensor ipre, Tensor fpre, Tensor norm_w, Tensor(b!) state_c, Tensor(c!) state_n, Tensor(d!) state_m, Tensor cu_seqlens, Tensor state_slots, Tensor seq_starts, float cap, float q_scale, float norm_eps, float denom_floor) -> ()");
  m.def("ssd_scan(Tensor(a!) out, Tensor x, Tensor B, Tensor C, Tensor dt, Tensor z, Tensor a_log, Tensor dt_bias, Tensor d_skip, Tensor norm_w, Tensor(b!) state, Tensor cu_seqlens, Tensor state_slots, Tensor seq_starts, int norm_groups, float norm_eps) -> ()");
}
TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("mlstm_scan", &kaito::mlstm_scan);
  m.impl("ssd_scan", &kaito::ssd_scan);
}
