// Differential attention over a paged cache.
//
// Every query head carries two score maps (q row = [map1 | map2], k row the
// same) that attend over ONE shared value head:
//   a_m = softmax(q_m . k_m * scale) V           (m = 1, 2; causal)
//   o   = a_1 - lambda * a_2
//   out = o / sqrt(mean(o^2) + eps) * out_scale * sigmoid(gate)
// Scores, softmax weights and the accumulation are fp32.
//
// Row-wise kernel: one workgroup per (row, head), any map_dim / value width,
// used for prompts, portions of prompts and decoding alike. Each row walks
// its own keys in a fixed order, so its result does not depend on the rest
// of the batch.
#include "elem.h"

namespace kukeon {

struct AttnArgs {
  long ldq, ldo, ldg;      // row strides of q, out, gate
  int H, G, dim, vdim, BS, max_blocks;
  float scale, lambda, eps, out_scale;
};

template <typename T, int NT>
__global__ __launch_bounds__(NT) void diff_attn_rowwise_kernel(
    T* __restrict__ out, const T* __restrict__ q,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const T* __restrict__ gate, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ block_table,
    AttnArgs a) {
  extern __shared__ float smem[];
  const int tid = threadIdx.x;
  const int r = blockIdx.x, h = blockIdx.y;
  const int dim = a.dim, vdim = a.vdim;
  T* orow = out + (long)r * a.ldo + (long)h * vdim;
  const int p = positions[r];
  if (p < 0) {                               // inactive row: defined output
    for (int e = tid; e < vdim; e += NT) stf(orow + e, 0.f);
    return;
  }
  const int pw = vdim > NT ? vdim : NT;      // partial-sum row width
  float* qs = smem;                          // [2*dim]
  float* ps = qs + 2 * dim;                  // [2][NT]
  int* vrow = reinterpret_cast<int*>(ps + 2 * NT);   // [NT]
  float* red = reinterpret_cast<float*>(vrow + NT);  // [32]
  float* part = red + 32;                    // [2][pw]

  const int* bt = block_table + (long)row_seq[r] * a.max_blocks;
  const int g = h / (a.H / a.G);
  for (int i = tid; i < 2 * dim; i += NT)
    qs[i] = ldf(q + (long)r * a.ldq + (long)h * 2 * dim + i) * a.scale;
  __syncthreads();

  const int nsl = vdim >= NT ? 1 : NT / vdim;   // key slices in the PV step
  constexpr int R = 2;                          // vdim <= R*NT
  float acc1[R] = {0.f, 0.f}, acc2[R] = {0.f, 0.f};
  float m1 = -INFINITY, m2 = -INFINITY, l1 = 0.f, l2 = 0.f;
  const int nkeys = p + 1;
  for (int j0 = 0; j0 < nkeys; j0 += NT) {
    const int j = j0 + tid;
    float s1 = -INFINITY, s2 = -INFINITY;
    int vr = 0;
    if (j < nkeys) {
      const int blk = bt[j / a.BS];
      vr = (blk * a.G + g) * a.BS + j % a.BS;
      const T* kr = k_cache + (long)vr * 2 * dim;
      float d1 = 0.f, d2 = 0.f;
      for (int i = 0; i < dim; ++i) {
        d1 = fmaf(qs[i], ldf(kr + i), d1);
        d2 = fmaf(qs[dim + i], ldf(kr + dim + i), d2);
      }
      s1 = d1; s2 = d2;
    }
    const float2 tm = block_max2(s1, s2, red);
    const float n1 = fmaxf(m1, tm.x), n2 = fmaxf(m2, tm.y);
    const float p1 = j < nkeys ? expf(s1 - n1) : 0.f;
    const float p2 = j < nkeys ? expf(s2 - n2) : 0.f;
    ps[tid] = p1; ps[NT + tid] = p2; vrow[tid] = vr;
    const float2 ts = block_sum2(p1, p2, red);   // barriers publish ps/vrow
    const float c1 = expf(m1 - n1), c2 = expf(m2 - n2);
    l1 = l1 * c1 + ts.x; l2 = l2 * c2 + ts.y;
    m1 = n1; m2 = n2;
    const int nk = nkeys - j0 < NT ? nkeys - j0 : NT;
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
      const int idx = tid + rr * NT;
      if (idx < nsl * vdim) {
        const int e = idx % vdim, sl = idx / vdim;
        float x1 = acc1[rr] * c1, x2 = acc2[rr] * c2;
        for (int jj = sl; jj < nk; jj += nsl) {
          const float v = ldf(v_cache + (long)vrow[jj] * vdim + e);
          x1 = fmaf(ps[jj], v, x1);
          x2 = fmaf(ps[NT + jj], v, x2);
        }
        acc1[rr] = x1; acc2[rr] = x2;
      }
    }
    __syncthreads();                          // ps/vrow reused next tile
  }
  // fold the key slices, then the differential combine and the unit norm
  float ss = 0.f;
  float o[R];
#pragma unroll
  for (int rr = 0; rr < R; ++rr) {
    const int idx = tid + rr * NT;
    if (idx < nsl * vdim && (rr == 0 || vdim > NT)) {
      part[idx] = acc1[rr]; part[pw + idx] = acc2[rr];
    }
  }
  __syncthreads();
#pragma unroll
  for (int rr = 0; rr < R; ++rr) {
    const int e = tid + rr * NT;
    o[rr] = 0.f;
    if (e < vdim) {
      float x1 = 0.f, x2 = 0.f;
      for (int sl = 0; sl < nsl; ++sl) {
        x1 += part[sl * vdim + e];
        x2 += part[pw + sl * vdim + e];
      }
      o[rr] = x1 / l1 - a.lambda * (x2 / l2);
      ss += o[rr] * o[rr];
    }
  }
  const float2 tot = block_sum2(ss, 0.f, red);
  const float rs = 1.0f / sqrtf(tot.x / (float)vdim + a.eps);
  float gs = 1.f;
  if (gate) {
    const float gl = ldf(gate + (long)r * a.ldg + h);
    gs = 1.0f / (1.0f + expf(-gl));
  }
#pragma unroll
  for (int rr = 0; rr < R; ++rr) {
    const int e = tid + rr * NT;
    if (e < vdim) stf(orow + e, o[rr] * rs * a.out_scale * gs);
  }
}

// out [rows, >= H*vdim] view; q [rows, H*2*dim]; k_cache [NB, G, BS, 2*dim];
// v_cache [NB, G, BS, vdim]; gate [rows, H] view (logits) or empty;
// positions, row_seq [rows]; block_table [nseq, max_blocks].
void diff_attention(torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
                    torch::Tensor v_cache, torch::Tensor gate,
                    torch::Tensor positions, torch::Tensor row_seq,
                    torch::Tensor block_table, int64_t H, double scale,
                    double lambda, double eps, double out_scale) {
  check_act(q, "q");
  TORCH_CHECK(out.scalar_type() == q.scalar_type() &&
              k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type());
  check_i32(positions, "positions"); check_i32(row_seq, "row_seq");
  check_i32(block_table, "block_table");
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.is_contiguous() && v_cache.is_contiguous());
  AttnArgs a{};
  a.H = (int)H; a.G = (int)k_cache.size(1); a.BS = (int)k_cache.size(2);
  TORCH_CHECK(k_cache.size(3) % 2 == 0);
  a.dim = (int)(k_cache.size(3) / 2); a.vdim = (int)v_cache.size(3);
  TORCH_CHECK(v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == a.G &&
              v_cache.size(2) == a.BS);
  TORCH_CHECK(a.G >= 1 && a.H >= a.G && a.H % a.G == 0);
  const long rows = q.size(0);
  TORCH_CHECK(q.dim() == 2 && q.stride(1) == 1 && q.size(1) == H * 2 * a.dim);
  TORCH_CHECK(out.dim() == 2 && out.stride(1) == 1 && out.size(0) == rows &&
              out.size(1) >= H * a.vdim);
  TORCH_CHECK(positions.numel() == rows && row_seq.numel() == rows);
  TORCH_CHECK(block_table.dim() == 2);
  const bool has_gate = gate.numel() > 0;
  if (has_gate)
    TORCH_CHECK(gate.scalar_type() == q.scalar_type() && gate.dim() == 2 &&
                gate.size(0) == rows && gate.size(1) >= H &&
                gate.stride(1) == 1);
  constexpr int NT = 256;
  TORCH_CHECK(a.vdim <= 2 * NT, "value width above 512 is not supported");
  a.ldq = q.stride(0); a.ldo = out.stride(0);
  a.ldg = has_gate ? gate.stride(0) : 0;
  a.max_blocks = (int)block_table.size(1);
  a.scale = (float)scale; a.lambda = (float)lambda; a.eps = (float)eps;
  a.out_scale = (float)out_scale;
  if (rows == 0) return;
  const int pw = a.vdim > NT ? a.vdim : NT;
  const size_t shm = sizeof(float) * (2 * a.dim + 2 * NT + NT + 32 + 2 * pw);
  TORCH_CHECK(shm <= 64 * 1024, "map size too large for the row-wise kernel");
  auto stream = c10::hip::getCurrentHIPStream().stream();
  dim3 grid((unsigned)rows, (unsigned)H);
  KK_DISPATCH_ACT(q, {
    diff_attn_rowwise_kernel<T, NT><<<grid, NT, shm, stream>>>(
        reinterpret_cast<T*>(out.data_ptr()),
        reinterpret_cast<const T*>(q.data_ptr()),
        reinterpret_cast<const T*>(k_cache.data_ptr()),
        reinterpret_cast<const T*>(v_cache.data_ptr()),
        has_gate ? reinterpret_cast<const T*>(gate.data_ptr()) : nullptr,
        positions.data_ptr<int>(), row_seq.data_ptr<int>(),
        block_table.data_ptr<int>(), a);
  });
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
