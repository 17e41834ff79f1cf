// Residual stream kept in fp32: x += a (+ bias), then h = rmsnorm(x) with a
// weight stored as an offset from a constant (weight_offset + w). One block
// per row; the row's sum of squares is reduced in a fixed order, so a row's
// result does not depend on what else is in the batch.
#include "elem.h"

namespace kukeon {

template <typename T>
__global__ __launch_bounds__(256) void residual_add_rmsnorm_kernel(
    float* __restrict__ x, const T* __restrict__ a, long lda,
    const float* __restrict__ bias, const float* __restrict__ w,
    float w_offset, float eps, T* __restrict__ out, int W) {
  __shared__ float red[32];
  const long row = blockIdx.x;
  float* xr = x + row * (long)W;
  const bool upd = (a != nullptr) || (bias != nullptr);
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = xr[i];
    if (a) v += ldf(a + row * lda + i);
    if (bias) v += bias[i];
    if (upd) xr[i] = v;
    ss += v * v;
  }
  const float2 tot = block_sum2(ss, 0.f, red);
  const float rs = 1.0f / sqrtf(tot.x / (float)W + eps);
  T* orow = out + row * (long)W;
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    stf(orow + i, xr[i] * rs * (w_offset + w[i]));
}

// Vector form: W a multiple of 8 and at most 8 * 256 * NIT; the row is held
// in registers between the two passes and every load is 16 or 32 bytes.
template <typename T, int NIT>
__global__ __launch_bounds__(256) void residual_add_rmsnorm_vec_kernel(
    float* __restrict__ x, const T* __restrict__ a, long lda,
    const float* __restrict__ bias, const float* __restrict__ w,
    float w_offset, float eps, T* __restrict__ out, int W) {
  __shared__ float red[32];
  const long row = blockIdx.x;
  float* xr = x + row * (long)W;
  float v[NIT][8];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int i = (it * 256 + threadIdx.x) * 8;
    if (i < W) {
      ld8(xr + i, v[it]);
      if (a) {
        float t[8];
        ld8(a + row * lda + i, t);
#pragma unroll
        for (int k = 0; k < 8; ++k) v[it][k] += t[k];
      }
      if (bias) {
        float t[8];
        ld8(bias + i, t);
#pragma unroll
        for (int k = 0; k < 8; ++k) v[it][k] += t[k];
      }
      if (a || bias) st8(xr + i, v[it]);
#pragma unroll
      for (int k = 0; k < 8; ++k) ss += v[it][k] * v[it][k];
    }
  }
  const float2 tot = block_sum2(ss, 0.f, red);
  const float rs = 1.0f / sqrtf(tot.x / (float)W + eps);
  T* orow = out + row * (long)W;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int i = (it * 256 + threadIdx.x) * 8;
    if (i < W) {
      float t[8], o[8];
      ld8(w + i, t);
#pragma unroll
      for (int k = 0; k < 8; ++k) o[k] = v[it][k] * rs * (w_offset + t[k]);
      st8(orow + i, o);
    }
  }
}

// x [T,W] fp32 (in/out); a [T,>=W] rows of stride a.stride(0) or empty;
// bias [W] fp32 or empty; w [W] fp32; out [T,W] in the activation format.
void residual_add_rmsnorm(torch::Tensor x, torch::Tensor a, torch::Tensor bias,
                          torch::Tensor w, double w_offset, double eps,
                          torch::Tensor out) {
  check_f32(x, "x");
  check_f32(w, "w");
  check_act(out, "out");
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.is_contiguous());
  const long rows = x.size(0);
  const int W = (int)x.size(1);
  TORCH_CHECK(out.size(0) == rows && out.size(1) == W && w.numel() == W);
  const bool has_a = a.numel() > 0;
  const bool has_b = bias.numel() > 0;
  if (has_a) {
    TORCH_CHECK(a.scalar_type() == out.scalar_type() && a.dim() == 2 &&
                a.size(0) == rows && a.size(1) >= W && a.stride(1) == 1);
  }
  if (has_b) {
    check_f32(bias, "bias");
    TORCH_CHECK(bias.numel() == W);
  }
  if (rows == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool vec = W % 8 == 0 && W <= 8 * 256 * 4 && aligned16(x.data_ptr()) &&
                   aligned16(out.data_ptr()) && aligned16(w.data_ptr()) &&
                   (!has_a || (a.stride(0) % 8 == 0 &&
                               aligned16(a.data_ptr()))) &&
                   (!has_b || aligned16(bias.data_ptr()));
  if (vec) {
  KK_DISPATCH_ACT(out, {
      const T* ap = has_a ? reinterpret_cast<const T*>(a.data_ptr()) : nullptr;
      const long lda = has_a ? a.stride(0) : 0;
      const float* bp = has_b ? bias.data_ptr<float>() : nullptr;
      T* op = reinterpret_cast<T*>(out.data_ptr());
      if (W <= 2048)
        residual_add_rmsnorm_vec_kernel<T, 1><<<dim3((unsigned)rows), 256, 0,
                                                stream>>>(
            x.data_ptr<float>(), ap, lda, bp, w.data_ptr<float>(),
            (float)w_offset, (float)eps, op, W);
      else if (W <= 4096)
        residual_add_rmsnorm_vec_kernel<T, 2><<<dim3((unsigned)rows), 256, 0,
                                                stream>>>(
            x.data_ptr<float>(), ap, lda, bp, w.data_ptr<float>(),
            (float)w_offset, (float)eps, op, W);
      else
        residual_add_rmsnorm_vec_kernel<T, 4><<<dim3((unsigned)rows), 256, 0,
                                                stream>>>(
            x.data_ptr<float>(), ap, lda, bp, w.data_ptr<float>(),
            (float)w_offset, (float)eps, op, W);
    });
    HIP_CHECK_KERNEL();
    return;
  }
  KK_DISPATCH_ACT(out, {
    residual_add_rmsnorm_kernel<T><<<dim3((unsigned)rows), 256, 0, stream>>>(
        x.data_ptr<float>(),
        has_a ? reinterpret_cast<const T*>(a.data_ptr()) : nullptr,
        has_a ? a.stride(0) : 0,
        has_b ? bias.data_ptr<float>() : nullptr, w.data_ptr<float>(),
        (float)w_offset, (float)eps, reinterpret_cast<T*>(out.data_ptr()), W);
  });
  HIP_CHECK_KERNEL();
}

// Sandwich norms around a sublayer in one pass over the row:
//   x += y / rms(y) * post_w          (fp32 residual, in place)
//   out = x / rms(x) * w              (input of the next sublayer)
// One block per row, both sums reduced in a fixed order.
template <typename T>
__global__ __launch_bounds__(256) void postnorm_residual_rmsnorm_kernel(
    float* __restrict__ x, const T* __restrict__ y, long ldy,
    const float* __restrict__ post_w, const float* __restrict__ w, float eps,
    T* __restrict__ out, int W) {
  __shared__ float red[32];
  const long row = blockIdx.x;
  float* xr = x + row * (long)W;
  const T* yr = y + row * ldy;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float v = ldf(yr + i);
    ss += v * v;
  }
  const float2 t1 = block_sum2(ss, 0.f, red);
  const float ry = 1.0f / sqrtf(t1.x / (float)W + eps);
  float sx = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float v = xr[i] + ldf(yr + i) * ry * post_w[i];
    xr[i] = v;
    sx += v * v;
  }
  const float2 t2 = block_sum2(sx, 0.f, red);
  const float rx = 1.0f / sqrtf(t2.x / (float)W + eps);
  T* orow = out + row * (long)W;
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    stf(orow + i, xr[i] * rx * w[i]);
}

// Vector form: W a multiple of 8, at most 8 * 256 * NIT; y and x stay in
// registers between the passes.
template <typename T, int NIT>
__global__ __launch_bounds__(256) void postnorm_residual_rmsnorm_vec_kernel(
    float* __restrict__ x, const T* __restrict__ y, long ldy,
    const float* __restrict__ post_w, const float* __restrict__ w, float eps,
    T* __restrict__ out, int W) {
  __shared__ float red[32];
  const long row = blockIdx.x;
  float* xr = x + row * (long)W;
  const T* yr = y + row * ldy;
  float v[NIT][8];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int i = (it * 256 + threadIdx.x) * 8;
    if (i < W) {
      ld8(yr + i, v[it]);
#pragma unroll
      for (int k = 0; k < 8; ++k) ss += v[it][k] * v[it][k];
    }
  }
  const float2 t1 = block_sum2(ss, 0.f, red);
  const float ry = 1.0f / sqrtf(t1.x / (float)W + eps);
  float sx = 0.f;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int i = (it * 256 + threadIdx.x) * 8;
    if (i < W) {
      float xv[8], pw[8];
      ld8(xr + i, xv);
      ld8(post_w + i, pw);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        v[it][k] = xv[k] + v[it][k] * ry * pw[k];
        sx += v[it][k] * v[it][k];
      }
      st8(xr + i, v[it]);
    }
  }
  const float2 t2 = block_sum2(sx, 0.f, red);
  const float rx = 1.0f / sqrtf(t2.x / (float)W + eps);
  T* orow = out + row * (long)W;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int i = (it * 256 + threadIdx.x) * 8;
    if (i < W) {
      float t[8], o[8];
      ld8(w + i, t);
#pragma unroll
      for (int k = 0; k < 8; ++k) o[k] = v[it][k] * rx * t[k];
      st8(orow + i, o);
    }
  }
}

// x [T,W] fp32 (in/out); y [T,>=W] rows of stride y.stride(0) in the
// activation format; post_w, w [W] fp32; out [T,W] activation format.
void postnorm_residual_rmsnorm(torch::Tensor x, torch::Tensor y,
                               torch::Tensor post_w, torch::Tensor w,
                               double eps, torch::Tensor out) {
  check_f32(x, "x");
  check_f32(w, "w");
  check_f32(post_w, "post_w");
  check_act(out, "out");
  check_act(y, "y");
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.is_contiguous());
  const long rows = x.size(0);
  const int W = (int)x.size(1);
  TORCH_CHECK(out.size(0) == rows && out.size(1) == W && w.numel() == W &&
              post_w.numel() == W);
  TORCH_CHECK(y.scalar_type() == out.scalar_type() && y.dim() == 2 &&
              y.size(0) == rows && y.size(1) >= W && y.stride(1) == 1);
  if (rows == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool vec = W % 8 == 0 && W <= 8 * 256 * 4 && aligned16(x.data_ptr()) &&
                   aligned16(out.data_ptr()) && aligned16(w.data_ptr()) &&
                   aligned16(post_w.data_ptr()) && y.stride(0) % 8 == 0 &&
                   aligned16(y.data_ptr());
#define KK_ARGS x.data_ptr<float>(), yp, (long)y.stride(0),                \
        post_w.data_ptr<float>(), w.data_ptr<float>(), (float)eps, op, W
  KK_DISPATCH_ACT(out, {
    const T* yp = reinterpret_cast<const T*>(y.data_ptr());
    T* op = reinterpret_cast<T*>(out.data_ptr());
    dim3 grid((unsigned)rows);
    if (!vec)
      postnorm_residual_rmsnorm_kernel<T><<<grid, 256, 0, stream>>>(KK_ARGS);
    else if (W <= 2048)
      postnorm_residual_rmsnorm_vec_kernel<T, 1><<<grid, 256, 0, stream>>>(
          KK_ARGS);
    else if (W <= 4096)
      postnorm_residual_rmsnorm_vec_kernel<T, 2><<<grid, 256, 0, stream>>>(
          KK_ARGS);
    else
      postnorm_residual_rmsnorm_vec_kernel<T, 4><<<grid, 256, 0, stream>>>(
          KK_ARGS);
  });
#undef KK_ARGS
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
