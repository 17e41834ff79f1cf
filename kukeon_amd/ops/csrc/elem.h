// Element access for kernels that serve two activation formats: bf16
// (stored as raw ushort) for serving and float for the exact mode. All
// arithmetic is fp32 either way; only loads and stores differ.
#pragma once
#include "common.h"
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>

namespace kukeon {

typedef unsigned short bf16_t;

DEV_INLINE float ldf(const float* p) { return *p; }
DEV_INLINE float ldf(const bf16_t* p) { return us2f(*p); }
DEV_INLINE void stf(float* p, float v) { *p = v; }
DEV_INLINE void stf(bf16_t* p, float v) { *p = f2us(v); }

// 8 consecutive elements as fp32 (16 B of bf16, 32 B of float)
DEV_INLINE void ld8(const float* p, float* o) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
  o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}
DEV_INLINE void ld8(const bf16_t* p, float* o) {
  const bf16x8 v = load_bf16x8(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = v.f(i);
}
DEV_INLINE void st8(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = float4{v[0], v[1], v[2], v[3]};
  *reinterpret_cast<float4*>(p + 4) = float4{v[4], v[5], v[6], v[7]};
}
DEV_INLINE void st8(bf16_t* p, const float* v) {
  *reinterpret_cast<uint4*>(p) = pack_bf16x8(v);
}
// 8 raw elements of the storage format, kept unconverted while in flight
template <typename T> struct Raw8;
template <> struct Raw8<bf16_t> {
  uint4 v;
  DEV_INLINE void load(const bf16_t* p) {
    v = *reinterpret_cast<const uint4*>(p);
  }
  DEV_INLINE float get(int i) const {
    const unsigned int* w = reinterpret_cast<const unsigned int*>(&v);
    return us2f((unsigned short)((w[i >> 1] >> ((i & 1) * 16)) & 0xffffu));
  }
};
template <> struct Raw8<float> {
  float4 a, b;
  DEV_INLINE void load(const float* p) {
    a = *reinterpret_cast<const float4*>(p);
    b = *reinterpret_cast<const float4*>(p + 4);
  }
  DEV_INLINE float get(int i) const {
    const float* f = i < 4 ? reinterpret_cast<const float*>(&a)
                           : reinterpret_cast<const float*>(&b);
    return f[i & 3];
  }
};

__host__ __device__ inline bool aligned16(const void* p) {
  return reinterpret_cast<uintptr_t>(p) % 16 == 0;
}

// both-sum block reduction of a pair (one pass of barriers for two values)
DEV_INLINE float2 block_sum2(float a, float b, float* red /* >= 32 floats */) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int wid = threadIdx.x / WAVE;
  const int nwaves = (blockDim.x + WAVE - 1) / WAVE;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    a += __shfl_xor(a, off, WAVE);
    b += __shfl_xor(b, off, WAVE);
  }
  if (lane == 0) { red[2 * wid] = a; red[2 * wid + 1] = b; }
  __syncthreads();
  float ra = 0.f, rb = 0.f;
  for (int w = 0; w < nwaves; ++w) { ra += red[2 * w]; rb += red[2 * w + 1]; }
  __syncthreads();
  return float2{ra, rb};
}
DEV_INLINE float2 block_max2(float a, float b, float* red) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int wid = threadIdx.x / WAVE;
  const int nwaves = (blockDim.x + WAVE - 1) / WAVE;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    a = fmaxf(a, __shfl_xor(a, off, WAVE));
    b = fmaxf(b, __shfl_xor(b, off, WAVE));
  }
  if (lane == 0) { red[2 * wid] = a; red[2 * wid + 1] = b; }
  __syncthreads();
  float ra = -INFINITY, rb = -INFINITY;
  for (int w = 0; w < nwaves; ++w) {
    ra = fmaxf(ra, red[2 * w]);
    rb = fmaxf(rb, red[2 * w + 1]);
  }
  __syncthreads();
  return float2{ra, rb};
}

inline bool is_bf16(const torch::Tensor& t) {
  return t.scalar_type() == torch::kBFloat16;
}
inline void check_act(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be a device tensor");
  TORCH_CHECK(t.scalar_type() == torch::kBFloat16 ||
                  t.scalar_type() == torch::kFloat32,
              name, " must be bf16 or fp32");
}
inline void check_f32(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kFloat32 &&
                  t.is_contiguous(), name, " must be contiguous fp32");
}
inline void check_i32(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kInt32 &&
                  t.is_contiguous(), name, " must be contiguous int32");
}

// run BODY with `T` bound to the storage type of tensor `t`
#define KK_DISPATCH_ACT(t, ...)             \
  do {                                      \
    if (is_bf16(t)) {                       \
      typedef bf16_t T;                     \
      __VA_ARGS__                           \
    } else {                                \
      typedef float T;                      \
      __VA_ARGS__                           \
    }                                       \
  } while (0)

}  // namespace kukeon
