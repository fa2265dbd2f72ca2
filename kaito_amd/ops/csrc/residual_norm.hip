// Norms for models that keep the residual stream in f32 and put the norm
// on the sub-layer OUTPUT:
//
//   post_norm_residual:  x32 += rms(m) * w           (in place, f32)
//       m = y                                          (one sub-layer), or
//       m = (rms(y) * w_y + rms(y2) * w_y2) / 2        (two side by side)
//     and x32's rounding to the activation dtype is emitted for the next
//     sub-layer in the same pass.
//   rms_norm_cast: rms(x) * w for f32 or bf16 rows → f32 or bf16.
//
// and for pre-norm models with an f32 stream:
//
//   residual_add_norm:   x32 += s1 * y (+ s2 * y2)   (in place, f32)
//                        h    = rms(x32) * w          (next sub-layer's input)
//
// One workgroup per row; m is staged in LDS (f32) between the passes.
// All weights are f32.
#include "mix_common.h"

namespace kaito {

namespace {

template <typename T, typename TO>
__global__ void post_norm_residual_kernel(
    float* __restrict__ x32, TO* __restrict__ xo, const bool write_xo,
    const T* __restrict__ y, const int64_t y_s0, const float* __restrict__ w,
    const T* __restrict__ y2, const int64_t y2_s0,
    const float* __restrict__ w_y, const float* __restrict__ w_y2,
    const int H, const float eps) {
  extern __shared__ float m[];          // [H]
  __shared__ float red[16];
  const int row = blockIdx.x;
  const T* yr = y + (int64_t)row * y_s0;
  if (y2 != nullptr) {
    const T* y2r = y2 + (int64_t)row * y2_s0;
    float s1 = 0.f, s2 = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const float a = act_ld(yr + i), b = act_ld(y2r + i);
      s1 += a * a;
      s2 += b * b;
    }
    s1 = block_reduce_sum(s1, red);
    __syncthreads();
    s2 = block_reduce_sum(s2, red);
    __syncthreads();
    const float i1 = 1.0f / sqrtf(s1 / (float)H + eps);
    const float i2 = 1.0f / sqrtf(s2 / (float)H + eps);
    for (int i = threadIdx.x; i < H; i += blockDim.x)
      m[i] = 0.5f * (act_ld(yr + i) * i1 * w_y[i] +
                     act_ld(y2r + i) * i2 * w_y2[i]);
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) m[i] = act_ld(yr + i);
  }
  // each thread re-reads only the m[] entries it wrote itself
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) ss += m[i] * m[i];
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  float* xr = x32 + (int64_t)row * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = xr[i] + m[i] * inv * w[i];
    xr[i] = v;
    if (write_xo) act_st(xo + (int64_t)row * H + i, v);
  }
}

template <typename TI, typename TO>
__global__ void rms_norm_cast_kernel(
    TO* __restrict__ out, const TI* __restrict__ x,
    const float* __restrict__ w, const int H, const float eps) {
  __shared__ float red[16];
  const int row = blockIdx.x;
  const TI* xr = x + (int64_t)row * H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = act_ld(xr + i);
    ss += v * v;
  }
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    act_st(out + (int64_t)row * H + i, act_ld(xr + i) * inv * w[i]);
}

// One workgroup per row. Each thread re-reads only the stream entries it
// wrote itself, so the row needs no LDS stage.
template <typename T, typename TO>
__global__ void residual_add_norm_kernel(
    float* __restrict__ x32, TO* __restrict__ h_out,
    const T* __restrict__ y, const int64_t y_s0,
    const T* __restrict__ y2, const int64_t y2_s0,
    const float* __restrict__ w, const float s1, const float s2, const int H,
    const float eps) {
  __shared__ float red[16];
  const int row = blockIdx.x;
  float* xr = x32 + (int64_t)row * H;
  const T* yr = y + (int64_t)row * y_s0;
  const T* y2r = y2 ? y2 + (int64_t)row * y2_s0 : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float add = s1 * act_ld(yr + i);
    if (y2r) add += s2 * act_ld(y2r + i);
    const float v = xr[i] + add;
    xr[i] = v;
    ss += v * v;
  }
  if (w == nullptr) return;
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    act_st(h_out + (int64_t)row * H + i, xr[i] * inv * w[i]);
}

int row_threads(int H) { return H >= 1024 ? 256 : (H >= 256 ? 128 : 64); }

}  // namespace

void post_norm_residual(at::Tensor x32, at::Tensor x_out, at::Tensor y,
                        at::Tensor w, double eps, at::Tensor y2,
                        at::Tensor w_y, at::Tensor w_y2) {
  KAITO_CHECK_F32(x32);
  TORCH_CHECK(x32.dim() == 2 && y.dim() == 2 && y.stride(1) == 1 &&
              y.sizes() == x32.sizes() && is_act_dtype(y));
  const int T = x32.size(0), H = x32.size(1);
  KAITO_CHECK_F32(w);
  TORCH_CHECK(w.numel() == H);
  const bool pair = y2.numel() > 0;
  if (pair) {
    TORCH_CHECK(y2.dim() == 2 && y2.stride(1) == 1 &&
                y2.sizes() == x32.sizes() && y2.dtype() == y.dtype());
    KAITO_CHECK_F32(w_y); KAITO_CHECK_F32(w_y2);
    TORCH_CHECK(w_y.numel() == H && w_y2.numel() == H);
  }
  const bool write_xo = x_out.data_ptr() != x32.data_ptr();
  TORCH_CHECK(x_out.is_contiguous() && x_out.sizes() == x32.sizes() &&
              is_act_dtype(x_out));
  TORCH_CHECK((size_t)H * 4 <= 64 * 1024, "row too wide for the LDS stage");
  if (T == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const int threads = row_threads(H);
  KAITO_DISPATCH_ACT(y, {
    using in_t = act_t;
    KAITO_DISPATCH_ACT(x_out, {
      hipLaunchKernelGGL((post_norm_residual_kernel<in_t, act_t>), dim3(T),
          dim3(threads), (size_t)H * 4, stream, x32.data_ptr<float>(),
          (act_t*)x_out.data_ptr(), write_xo, (const in_t*)y.data_ptr(),
          y.stride(0), w.data_ptr<float>(),
          pair ? (const in_t*)y2.data_ptr() : nullptr,
          pair ? y2.stride(0) : 0, pair ? w_y.data_ptr<float>() : nullptr,
          pair ? w_y2.data_ptr<float>() : nullptr, H, (float)eps);
    });
  });
}

void residual_add_norm(at::Tensor x32, at::Tensor h_out, at::Tensor y,
                       at::Tensor y2, at::Tensor w, double s1, double s2,
                       double eps) {
  KAITO_CHECK_F32(x32);
  TORCH_CHECK(x32.dim() == 2 && y.dim() == 2 && y.stride(1) == 1 &&
              y.sizes() == x32.sizes() && is_act_dtype(y));
  const int T = x32.size(0), H = x32.size(1);
  const bool pair = y2.numel() > 0;
  if (pair)
    TORCH_CHECK(y2.dim() == 2 && y2.stride(1) == 1 &&
                y2.sizes() == x32.sizes() && y2.dtype() == y.dtype());
  const bool norm = w.numel() > 0;
  if (norm) {
    KAITO_CHECK_F32(w);
    TORCH_CHECK(w.numel() == H && h_out.is_contiguous() &&
                h_out.sizes() == x32.sizes() && is_act_dtype(h_out) &&
                h_out.data_ptr() != x32.data_ptr());
  }
  if (T == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const int threads = row_threads(H);
  KAITO_DISPATCH_ACT(y, {
    using in_t = act_t;
    if (!norm || h_out.dtype() == at::kFloat) {
      hipLaunchKernelGGL((residual_add_norm_kernel<in_t, float>), dim3(T),
          dim3(threads), 0, stream, x32.data_ptr<float>(),
          norm ? h_out.data_ptr<float>() : nullptr,
          (const in_t*)y.data_ptr(), y.stride(0),
          pair ? (const in_t*)y2.data_ptr() : nullptr,
          pair ? y2.stride(0) : 0, norm ? w.data_ptr<float>() : nullptr,
          (float)s1, (float)s2, H, (float)eps);
    } else {
      hipLaunchKernelGGL((residual_add_norm_kernel<in_t, bf16_act>), dim3(T),
          dim3(threads), 0, stream, x32.data_ptr<float>(),
          (bf16_act*)h_out.data_ptr(), (const in_t*)y.data_ptr(),
          y.stride(0), pair ? (const in_t*)y2.data_ptr() : nullptr,
          pair ? y2.stride(0) : 0, w.data_ptr<float>(), (float)s1, (float)s2,
          H, (float)eps);
    }
  });
}

void rms_norm_cast(at::Tensor out, at::Tensor x, at::Tensor w, double eps) {
  TORCH_CHECK(x.is_cuda() && x.is_contiguous() && is_act_dtype(x) &&
              out.is_contiguous() && is_act_dtype(out) &&
              out.sizes() == x.sizes() && x.dim() >= 1);
  const int H = x.size(-1);
  const int T = H > 0 ? x.numel() / H : 0;
  KAITO_CHECK_F32(w);
  TORCH_CHECK(w.numel() == H);
  if (T == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const int threads = row_threads(H);
  KAITO_DISPATCH_ACT(x, {
    using in_t = act_t;
    KAITO_DISPATCH_ACT(out, {
      hipLaunchKernelGGL((rms_norm_cast_kernel<in_t, act_t>), dim3(T),
          dim3(threads), 0, stream, (act_t*)out.data_ptr(),
          (const in_t*)x.data_ptr(), w.data_ptr<float>(), H, (float)eps);
    });
  });
}

}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("post_norm_residual(Tensor(a!) x32, Tensor(b!) x_out, Tensor y, Tensor w, float eps, Tensor y2, Tensor w_y, Tensor w_y2) -> ()");
  m.def("rms_norm_cast(Tensor(a!) out, Tensor x, Tensor w, float eps) -> ()");
  m.def("residual_add_norm(Tensor(a!) x32, Tensor(b!) h_out, Tensor y, Tensor y2, Tensor w, float s1, float s2, float eps) -> ()");
}
TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("post_norm_residual", &kaito::post_norm_residual);
  m.impl("rms_norm_cast", &kaito::rms_norm_cast);
  m.impl("residual_add_norm", &kaito::residual_add_norm);
}
