// Mixture of small experts chosen by a per-token-id table: token t with id
// v uses the experts table[v, 0..top) with weight 1/top each; an expert is
// down(relu(up h)^2). The routing needs no scores and no host round trip,
// so the pair of kernels below is graph-capturable as it stands:
//   table_moe_up    act[t, k, :] = relu(W_up[e_k] h_t)^2
//   table_moe_down  out[t, :]    = (1/top) sum_k W_down[e_k] act[t, k, :]
// Both are matrix-vector products per (token, expert) with fp32 sums: a
// wave owns output rows and its lanes stride over the reduction, so the
// sum order of a token is fixed whatever else is in the batch.
#include "elem.h"

namespace kukeon {

#define MOE_ROWS_PER_WAVE 8

template <typename T>
__global__ __launch_bounds__(256) void table_moe_up_kernel(
    T* __restrict__ act, const T* __restrict__ h, const int* __restrict__ ids,
    const int* __restrict__ table, const T* __restrict__ w_up, int W, int ff,
    int top, int vocab) {
  extern __shared__ float sh[];               // [W]
  const long tk = blockIdx.x;                 // token * top + k
  const long t = tk / top;
  const int k = (int)(tk - t * top);
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const int e = table[(long)id * top + k];
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    sh[i] = ldf(h + t * (long)W + i);
  __syncthreads();
  const int lane = threadIdx.x & (WAVE - 1);
  const int wave = threadIdx.x / WAVE;
  const int f0 = (blockIdx.y * 4 + wave) * MOE_ROWS_PER_WAVE;
  const T* we = w_up + (long)e * ff * W;
  for (int j = 0; j < MOE_ROWS_PER_WAVE; ++j) {
    const int f = f0 + j;
    if (f >= ff) break;
    const T* wr = we + (long)f * W;
    float acc = 0.f;
    for (int i = lane; i < W; i += WAVE) acc = fmaf(ldf(wr + i), sh[i], acc);
    acc = wave_sum(acc);
    if (lane == 0) {
      const float r = fmaxf(acc, 0.f);
      stf(act + tk * (long)ff + f, r * r);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void table_moe_down_kernel(
    T* __restrict__ out, const T* __restrict__ act,
    const int* __restrict__ ids, const int* __restrict__ table,
    const T* __restrict__ w_down, int W, int ff, int top, int vocab) {
  extern __shared__ float sa[];               // [top][ff]
  const long t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  for (int i = threadIdx.x; i < top * ff; i += blockDim.x)
    sa[i] = ldf(act + t * (long)top * ff + i);
  __syncthreads();
  const int lane = threadIdx.x & (WAVE - 1);
  const int wave = threadIdx.x / WAVE;
  const int c0 = (blockIdx.y * 4 + wave) * MOE_ROWS_PER_WAVE;
  const float share = 1.0f / (float)top;
  for (int j = 0; j < MOE_ROWS_PER_WAVE; ++j) {
    const int c = c0 + j;
    if (c >= W) break;
    float tot = 0.f;
    for (int k = 0; k < top; ++k) {
      const int e = table[(long)id * top + k];
      const T* wr = w_down + ((long)e * W + c) * ff;
      const float* a = sa + k * ff;
      float acc = 0.f;
      for (int i = lane; i < ff; i += WAVE) acc = fmaf(ldf(wr + i), a[i], acc);
      tot += wave_sum(acc);
    }
    if (lane == 0) stf(out + t * (long)W + c, tot * share);
  }
}

// ---- expert-major form for small batches ---------------------------------
// A decode step brings a few dozen tokens that share a handful of experts.
// Here a workgroup belongs to (expert, tile of output rows): it lists the
// (token, k) pairs routed to its expert, and each wave keeps one weight row
// in registers while it walks that list, so an expert's weights leave HBM
// once per step however many tokens use it. A pair's dot product is summed
// in an order fixed by the row length alone, never by the batch.
#define MOE_MAX_PAIRS 2048
#define MOE_SEG 16              // 8-element chunks of a row held per lane

DEV_INLINE int moe_list_pairs(int* list, int* count,
                              const int* __restrict__ ids,
                              const int* __restrict__ table, int pairs,
                              int top, int vocab, int e) {
  if (threadIdx.x == 0) *count = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
    int id = ids[i / top];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    if (table[(long)id * top + i % top] == e) list[atomicAdd(count, 1)] = i;
  }
  __syncthreads();
  return *count;
}

// one weight row (K elements, K % 8 == 0) against the rows src[pair * lds]
// of all listed pairs; FN(pair, value) consumes each result on lane 0
template <typename T, typename F>
DEV_INLINE void moe_row_times_pairs(const T* __restrict__ wrow, int K,
                                    const T* __restrict__ src, long lds,
                                    int div, const int* list, int n, F fn) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int chunks = K / 8;
  for (int seg0 = 0; seg0 < chunks; seg0 += MOE_SEG * WAVE) {
    Raw8<T> w[MOE_SEG];
#pragma unroll
    for (int c = 0; c < MOE_SEG; ++c) {
      const int ch = seg0 + c * WAVE + lane;
      if (ch < chunks) w[c].load(wrow + (long)ch * 8);
    }
    for (int j = 0; j < n; ++j) {
      const int pair = list[j];
      const T* x = src + (long)(pair / div) * lds;
      float acc = 0.f;
#pragma unroll
      for (int c = 0; c < MOE_SEG; ++c) {
        const int ch = seg0 + c * WAVE + lane;
        if (ch < chunks) {
          Raw8<T> xv;
          xv.load(x + (long)ch * 8);
#pragma unroll
          for (int k = 0; k < 8; ++k) acc = fmaf(w[c].get(k), xv.get(k), acc);
        }
      }
      acc = wave_sum(acc);
      fn(pair, acc, seg0 == 0);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void table_moe_up_expert_kernel(
    T* __restrict__ act, float* __restrict__ part, const T* __restrict__ h,
    const int* __restrict__ ids, const int* __restrict__ table,
    const T* __restrict__ w_up, int W, int ff, int top, int vocab,
    int pairs) {
  __shared__ int list[MOE_MAX_PAIRS];
  __shared__ int count;
  const int e = blockIdx.x;
  const int n = moe_list_pairs(list, &count, ids, table, pairs, top, vocab, e);
  if (n == 0) return;
  const int lane = threadIdx.x & (WAVE - 1);
  const int wave = threadIdx.x / WAVE;
  const int f0 = (blockIdx.y * 4 + wave) * MOE_ROWS_PER_WAVE;
  const bool one_seg = W / 8 <= MOE_SEG * WAVE;
  for (int j = 0; j < MOE_ROWS_PER_WAVE; ++j) {
    const int f = f0 + j;
    if (f >= ff) break;
    const T* wr = w_up + ((long)e * ff + f) * W;
    moe_row_times_pairs<T>(
        wr, W, h, (long)W, top, list, n,
        [&](int pair, float v, bool first) {
          if (lane != 0) return;
          if (one_seg) {
            const float r = fmaxf(v, 0.f);
            stf(act + (long)pair * ff + f, r * r);
          } else {       // long rows: sum the segments in fp32 first
            float* p = part + (long)pair * ff + f;
            *p = first ? v : *p + v;
          }
        });
    if (!one_seg && lane == 0) {
      for (int jj = 0; jj < n; ++jj) {
        const long at = (long)list[jj] * ff + f;
        const float r = fmaxf(part[at], 0.f);
        stf(act + at, r * r);
      }
    }
  }
}

// part[pair, c] = W_down[e][c, :] . act[pair, :]
template <typename T>
__global__ __launch_bounds__(256) void table_moe_down_expert_kernel(
    float* __restrict__ part, const T* __restrict__ act,
    const int* __restrict__ ids, const int* __restrict__ table,
    const T* __restrict__ w_down, int W, int ff, int top, int vocab,
    int pairs) {
  __shared__ int list[MOE_MAX_PAIRS];
  __shared__ int count;
  const int e = blockIdx.x;
  const int n = moe_list_pairs(list, &count, ids, table, pairs, top, vocab, e);
  if (n == 0) return;
  const int lane = threadIdx.x & (WAVE - 1);
  const int wave = threadIdx.x / WAVE;
  const int c0 = (blockIdx.y * 4 + wave) * MOE_ROWS_PER_WAVE;
  for (int j = 0; j < MOE_ROWS_PER_WAVE; ++j) {
    const int c = c0 + j;
    if (c >= W) break;
    const T* wr = w_down + ((long)e * W + c) * ff;
    moe_row_times_pairs<T>(wr, ff, act, (long)ff, 1, list, n,
                           [&](int pair, float v, bool first) {
                             if (lane != 0) return;
                             float* p = part + (long)pair * W + c;
                             *p = first ? v : *p + v;
                           });
  }
}

// out[t, :] = (1/top) sum_k part[t*top + k, :], k in order
template <typename T>
__global__ __launch_bounds__(256) void table_moe_mean_kernel(
    T* __restrict__ out, const float* __restrict__ part, long total, int W,
    int top) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long t = i / W;
  const int c = (int)(i - t * W);
  float acc = 0.f;
  for (int k = 0; k < top; ++k) acc += part[(t * top + k) * W + c];
  stf(out + i, acc * (1.0f / (float)top));
}

// ---- expert-major form on the matrix cores (bf16) -------------------------
// The same split of work, with v_mfma_f32_16x16x32_bf16: a wave owns 16
// weight rows (the A operand, lane = row, 8 consecutive k per lane) and up
// to 16 listed pairs at a time (the B operand, lane = pair). Each lane
// fetches 64 contiguous bytes of its weight row and of its pair's input per
// 128-wide k block; the same k permutation on both operands leaves the
// product unchanged. Output lane (pair = l & 15) holds rows 4 * (l >> 4) + r.
typedef __attribute__((__vector_size__(8 * sizeof(short)))) short moe_bf16x8_v;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float moe_f32x4_v;
DEV_INLINE moe_bf16x8_v moe_frag(const uint4& v) {
  return __builtin_bit_cast(moe_bf16x8_v, v);
}

// UP:   dst = act  [pairs, NR] bf16, relu(.)^2, source rows h[pair / top]
// !UP:  dst = part [pairs, NR] fp32, source rows act[pair]
template <bool UP>
__global__ __launch_bounds__(256) void table_moe_mfma_kernel(
    void* __restrict__ dst, const bf16_t* __restrict__ src,
    const int* __restrict__ ids, const int* __restrict__ table,
    const bf16_t* __restrict__ w, int NR, int K, int top, int vocab,
    int pairs) {
  __shared__ int list[MOE_MAX_PAIRS];
  __shared__ int count;
  const int e = blockIdx.x;
  const int n = moe_list_pairs(list, &count, ids, table, pairs, top, vocab, e);
  if (n == 0) return;
  const int lane = threadIdx.x & (WAVE - 1);
  const int wave = threadIdx.x / WAVE;
  const int rc = lane & 15;
  const int g4 = lane >> 4;
  const int r0 = (blockIdx.y * 4 + wave) * 16;
  if (r0 >= NR) return;
  const int arow = min(r0 + rc, NR - 1);
  const bf16_t* wrow = w + ((long)e * NR + arow) * K + g4 * 32;
  for (int g0 = 0; g0 < n; g0 += 16) {
    const int pair = g0 + rc < n ? list[g0 + rc] : -1;
    const bf16_t* xrow =
        src + (long)(pair < 0 ? 0 : (UP ? pair / top : pair)) * K + g4 * 32;
    moe_f32x4_v acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
    for (int k0 = 0; k0 < K; k0 += 128) {
      uint4 a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        a[i] = *reinterpret_cast<const uint4*>(wrow + k0 + i * 8);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        b[i] = pair < 0 ? uint4{0u, 0u, 0u, 0u}
                        : *reinterpret_cast<const uint4*>(xrow + k0 + i * 8);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(moe_frag(a[i]),
                                                      moe_frag(b[i]), acc, 0,
                                                      0, 0);
    }
    if (pair >= 0) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = r0 + 4 * g4 + r;
        if (row < NR) {
          if (UP) {
            const float v = fmaxf(acc[r], 0.f);
            reinterpret_cast<bf16_t*>(dst)[(long)pair * NR + row] =
                f2us(v * v);
          } else {
            reinterpret_cast<float*>(dst)[(long)pair * NR + row] = acc[r];
          }
        }
      }
    }
  }
}

// out, h [T, W]; ids [T] int32; table [vocab, top] int32; w_up [E, ff, W];
// w_down [E, W, ff].
void table_moe(torch::Tensor out, torch::Tensor h, torch::Tensor ids,
               torch::Tensor table, torch::Tensor w_up, torch::Tensor w_down) {
  check_act(out, "out"); check_act(h, "h");
  check_i32(ids, "ids"); check_i32(table, "table");
  TORCH_CHECK(h.dim() == 2 && h.is_contiguous() && out.is_contiguous());
  const long rows = h.size(0);
  const int W = (int)h.size(1);
  TORCH_CHECK(out.size(0) == rows && out.size(1) == W &&
              out.scalar_type() == h.scalar_type());
  TORCH_CHECK(w_up.dim() == 3 && w_down.dim() == 3 && w_up.is_contiguous() &&
              w_down.is_contiguous() && w_up.is_cuda() && w_down.is_cuda());
  const long E = w_up.size(0);
  const int ff = (int)w_up.size(1);
  TORCH_CHECK(w_up.size(2) == W && w_down.size(0) == E &&
              w_down.size(1) == W && w_down.size(2) == ff);
  TORCH_CHECK(w_up.scalar_type() == h.scalar_type() &&
              w_down.scalar_type() == h.scalar_type());
  TORCH_CHECK(table.dim() == 2 && ids.numel() == rows);
  const int vocab = (int)table.size(0);
  const int top = (int)table.size(1);
  TORCH_CHECK(top >= 1);
  if (rows == 0) return;
  auto act = torch::empty({rows * top, (long)ff}, h.options());
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const int per_block = 4 * MOE_ROWS_PER_WAVE;
  const long pairs = rows * top;
  // expert-major kernels: vector loads need whole 16-byte chunks
  const bool small = pairs <= MOE_MAX_PAIRS;
  const bool up_major = small && W % 8 == 0 && aligned16(h.data_ptr()) &&
                        aligned16(w_up.data_ptr());
  const bool down_major = small && ff % 8 == 0 && aligned16(act.data_ptr()) &&
                          aligned16(w_down.data_ptr());
  // the token-major kernels stage one row in LDS
  TORCH_CHECK(up_major || (size_t)W * 4 <= 64 * 1024,
              "table_moe: an input row does not fit LDS");
  TORCH_CHECK(down_major || (size_t)top * ff * 4 <= 64 * 1024,
              "table_moe: a token's expert rows do not fit LDS");
  torch::Tensor part;
  if (down_major || (up_major && W / 8 > MOE_SEG * WAVE))
    part = torch::empty({pairs, (long)std::max(W, ff)},
                        h.options().dtype(torch::kFloat32));
  float* pp = part.defined() ? part.data_ptr<float>() : nullptr;
  // bf16 rows of whole 128-element blocks go to the matrix cores
  const bool bf = is_bf16(h);
  const bool up_mfma = up_major && bf && W % 128 == 0;
  const bool down_mfma = down_major && bf && ff % 128 == 0;
  const bf16_t* hb = reinterpret_cast<const bf16_t*>(h.data_ptr());
  const bf16_t* ab = reinterpret_cast<const bf16_t*>(act.data_ptr());
  if (up_mfma)
    table_moe_mfma_kernel<true><<<
        dim3((unsigned)E, (unsigned)((ff + 63) / 64)), 256, 0, stream>>>(
        act.data_ptr(), hb, ids.data_ptr<int>(), table.data_ptr<int>(),
        reinterpret_cast<const bf16_t*>(w_up.data_ptr()), ff, W, top, vocab,
        (int)pairs);
  if (down_mfma) {
    table_moe_mfma_kernel<false><<<
        dim3((unsigned)E, (unsigned)((W + 63) / 64)), 256, 0, stream>>>(
        pp, ab, ids.data_ptr<int>(), table.data_ptr<int>(),
        reinterpret_cast<const bf16_t*>(w_down.data_ptr()), W, ff, top, vocab,
        (int)pairs);
    const long total = rows * W;
    table_moe_mean_kernel<bf16_t><<<dim3((unsigned)((total + 255) / 256)), 256,
                                    0, stream>>>(
        reinterpret_cast<bf16_t*>(out.data_ptr()), pp, total, W, top);
  }
  KK_DISPATCH_ACT(h, {
    if (up_mfma) {
    } else if (up_major)
      table_moe_up_expert_kernel<T><<<
          dim3((unsigned)E, (unsigned)((ff + per_block - 1) / per_block)), 256,
          0, stream>>>(
          reinterpret_cast<T*>(act.data_ptr()), pp,
          reinterpret_cast<const T*>(h.data_ptr()), ids.data_ptr<int>(),
          table.data_ptr<int>(), reinterpret_cast<const T*>(w_up.data_ptr()),
          W, ff, top, vocab, (int)pairs);
    else
      table_moe_up_kernel<T><<<
          dim3((unsigned)(rows * top),
               (unsigned)((ff + per_block - 1) / per_block)),
          256, (size_t)W * 4, stream>>>(
          reinterpret_cast<T*>(act.data_ptr()),
          reinterpret_cast<const T*>(h.data_ptr()), ids.data_ptr<int>(),
          table.data_ptr<int>(), reinterpret_cast<const T*>(w_up.data_ptr()),
          W, ff, top, vocab);
    if (down_mfma) {
    } else if (down_major) {
      table_moe_down_expert_kernel<T><<<
          dim3((unsigned)E, (unsigned)((W + per_block - 1) / per_block)), 256,
          0, stream>>>(
          pp, reinterpret_cast<const T*>(act.data_ptr()), ids.data_ptr<int>(),
          table.data_ptr<int>(),
          reinterpret_cast<const T*>(w_down.data_ptr()), W, ff, top, vocab,
          (int)pairs);
      const long total = rows * W;
      table_moe_mean_kernel<T><<<dim3((unsigned)((total + 255) / 256)), 256, 0,
                                 stream>>>(
          reinterpret_cast<T*>(out.data_ptr()), pp, total, W, top);
    } else {
      table_moe_down_kernel<T><<<
          dim3((unsigned)rows, (unsigned)((W + per_block - 1) / per_block)),
          256, (size_t)top * ff * 4, stream>>>(
          reinterpret_cast<T*>(out.data_ptr()),
          reinterpret_cast<const T*>(act.data_ptr()), ids.data_ptr<int>(),
          table.data_ptr<int>(),
          reinterpret_cast<const T*>(w_down.data_ptr()), W, ff, top, vocab);
    }
  });
  HIP_CHECK_KERNEL();
}

// ---- grouped form for long portions ---------------------------------------
// With the token ids known on the host, the (token, expert) pairs are sorted
// by expert there; the device gathers the rows in that order, every expert
// runs two vendor GEMMs over its contiguous rows with relu^2 in between, and
// combine_rows folds each token's `top` results with equal weights.

template <typename T>
__global__ __launch_bounds__(256) void gather_rows_kernel(
    T* __restrict__ out, const T* __restrict__ in, const int* __restrict__ map,
    int W) {
  const long r = blockIdx.x;
  const T* src = in + (long)map[r] * W;
  T* dst = out + r * (long)W;
  if (W % 8 == 0 && aligned16(in) && aligned16(out)) {
    for (int i = threadIdx.x * 8; i < W; i += blockDim.x * 8) {
      Raw8<T> v;
      v.load(src + i);
      *reinterpret_cast<Raw8<T>*>(dst + i) = v;
    }
    return;
  }
  for (int i = threadIdx.x; i < W; i += blockDim.x) dst[i] = src[i];
}

// out [n, W] = in[map[r], :]
void gather_rows(torch::Tensor out, torch::Tensor in, torch::Tensor map) {
  check_act(out, "out"); check_act(in, "in"); check_i32(map, "map");
  TORCH_CHECK(out.dim() == 2 && in.dim() == 2 && out.is_contiguous() &&
              in.is_contiguous() && out.size(1) == in.size(1) &&
              out.scalar_type() == in.scalar_type() &&
              map.numel() == out.size(0));
  const long n = out.size(0);
  if (n == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  KK_DISPATCH_ACT(out, {
    gather_rows_kernel<T><<<dim3((unsigned)n), 256, 0, stream>>>(
        reinterpret_cast<T*>(out.data_ptr()),
        reinterpret_cast<const T*>(in.data_ptr()), map.data_ptr<int>(),
        (int)out.size(1));
  });
  HIP_CHECK_KERNEL();
}

template <typename T>
__global__ __launch_bounds__(256) void relu_square_kernel(T* __restrict__ x,
                                                          long total) {
  const long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (i >= total) return;
  if (i + 8 <= total && aligned16(x)) {
    float v[8];
    ld8(x + i, v);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      v[k] = fmaxf(v[k], 0.f);
      v[k] *= v[k];
    }
    st8(x + i, v);
    return;
  }
  for (long j = i; j < total && j < i + 8; ++j) {
    const float v = fmaxf(ldf(x + j), 0.f);
    stf(x + j, v * v);
  }
}

void relu_square_(torch::Tensor x) {
  check_act(x, "x");
  TORCH_CHECK(x.is_contiguous());
  const long total = x.numel();
  if (total == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  KK_DISPATCH_ACT(x, {
    relu_square_kernel<T><<<dim3((unsigned)((total + 2047) / 2048)), 256, 0,
                            stream>>>(reinterpret_cast<T*>(x.data_ptr()),
                                      total);
  });
  HIP_CHECK_KERNEL();
}

template <typename T>
__global__ __launch_bounds__(256) void combine_rows_kernel(
    T* __restrict__ out, const T* __restrict__ in, const int* __restrict__ inv,
    int W, int top) {
  const long t = blockIdx.x;
  const float share = 1.0f / (float)top;
  if (W % 8 == 0 && aligned16(in) && aligned16(out)) {
    for (int i = threadIdx.x * 8; i < W; i += blockDim.x * 8) {
      float acc[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = 0.f;
      for (int k = 0; k < top; ++k) {
        float v[8];
        ld8(in + (long)inv[t * top + k] * W + i, v);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] += v[j];
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] *= share;
      st8(out + t * (long)W + i, acc);
    }
    return;
  }
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k)
      acc += ldf(in + (long)inv[t * top + k] * W + i);
    stf(out + t * (long)W + i, acc * share);
  }
}

// out [T, W] = mean_k in[inv[t, k], :]
void combine_rows(torch::Tensor out, torch::Tensor in, torch::Tensor inv) {
  check_act(out, "out"); check_act(in, "in"); check_i32(inv, "inv");
  TORCH_CHECK(out.dim() == 2 && in.dim() == 2 && out.is_contiguous() &&
              in.is_contiguous() && out.size(1) == in.size(1) &&
              out.scalar_type() == in.scalar_type());
  TORCH_CHECK(inv.dim() == 2 && inv.size(0) == out.size(0) &&
              inv.size(0) * inv.size(1) == in.size(0));
  const long n = out.size(0);
  if (n == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  KK_DISPATCH_ACT(out, {
    combine_rows_kernel<T><<<dim3((unsigned)n), 256, 0, stream>>>(
        reinterpret_cast<T*>(out.data_ptr()),
        reinterpret_cast<const T*>(in.data_ptr()), inv.data_ptr<int>(),
        (int)out.size(1), (int)inv.size(1));
  });
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
