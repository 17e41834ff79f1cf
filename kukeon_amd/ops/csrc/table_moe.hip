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
  TORCH_CHECK((size_t)W * 4 <= 64 * 1024 && (size_t)top * ff * 4 <= 64 * 1024,
              "table_moe: a row does not fit LDS");
  auto act = torch::empty({rows * top, (long)ff}, h.options());
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const int per_block = 4 * MOE_ROWS_PER_WAVE;
  KK_DISPATCH_ACT(h, {
    table_moe_up_kernel<T><<<dim3((unsigned)(rows * top),
                                  (unsigned)((ff + per_block - 1) / per_block)),
                             256, (size_t)W * 4, stream>>>(
        reinterpret_cast<T*>(act.data_ptr()),
        reinterpret_cast<const T*>(h.data_ptr()), ids.data_ptr<int>(),
        table.data_ptr<int>(), reinterpret_cast<const T*>(w_up.data_ptr()), W,
        ff, top, vocab);
    table_moe_down_kernel<T><<<dim3((unsigned)rows,
                                    (unsigned)((W + per_block - 1) / per_block)),
                               256, (size_t)top * ff * 4, stream>>>(
        reinterpret_cast<T*>(out.data_ptr()),
        reinterpret_cast<const T*>(act.data_ptr()), ids.data_ptr<int>(),
        table.data_ptr<int>(), reinterpret_cast<const T*>(w_down.data_ptr()),
        W, ff, top, vocab);
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
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const float v = fmaxf(ldf(x + i), 0.f);
  stf(x + i, v * v);
}

void relu_square_(torch::Tensor x) {
  check_act(x, "x");
  TORCH_CHECK(x.is_contiguous());
  const long total = x.numel();
  if (total == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  KK_DISPATCH_ACT(x, {
    relu_square_kernel<T><<<dim3((unsigned)((total + 255) / 256)), 256, 0,
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
