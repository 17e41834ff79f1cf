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

}  // namespace kukeon
