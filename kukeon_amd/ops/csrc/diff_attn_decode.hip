// Differential attention for single decoded rows: split-KV over the paged
// cache, one workgroup per (row, kv head, key split).
//
// A workgroup reads its keys and values ONCE for all query heads of the
// group and both score maps (2 * H/G softmax rows), so the HBM traffic per
// step is the context's K and V, whatever the group size. Scores for a
// pass of 256 keys go to LDS, softmax statistics are kept per row with the
// usual running rescale, and every split leaves an unnormalised partial
// sum with its (max, sum). A second kernel merges the splits and applies
// the differential combine, the unit norm and the output gate.
// All arithmetic is fp32; T is the storage format (bf16 or float).
#include "elem.h"

namespace kukeon {

struct DecArgs {
  long ldq, ldo, ldg;
  int H, G, dim, vdim, BS, max_blocks, nsplit;
  float scale, lambda, eps, out_scale;
};

constexpr int DPASS = 256;   // keys per pass

template <typename T> struct Vec16;
template <> struct Vec16<float> {
  static constexpr int N = 4;
  DEV_INLINE static void load(const float* p, float* o) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
};
template <> struct Vec16<bf16_t> {
  static constexpr int N = 8;
  DEV_INLINE static void load(const bf16_t* p, float* o) {
    const bf16x8 v = load_bf16x8(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = v.f(i);
  }
};

template <typename T, int HP>   // HP: compile-time bound on H/G
__global__ __launch_bounds__(256) void diff_attn_decode_split_kernel(
    float* __restrict__ part_o,    // [rows, H, 2, nsplit, vdim]
    float* __restrict__ part_ml,   // [rows, H, 2, nsplit, 2]
    const T* __restrict__ q, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ block_table,
    DecArgs a) {
  extern __shared__ float smem[];
  constexpr int VN = Vec16<T>::N;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = blockIdx.x, g = blockIdx.y, split = blockIdx.z;
  const int dim = a.dim, vdim = a.vdim, kw = 2 * dim;
  const int hpg = a.H / a.G;
  const int nhm = 2 * hpg;
  float* qs = smem;                         // [hpg][kw]
  float* sc = qs + hpg * kw;                // [2*HP][DPASS]; later partials
  int* vrow = reinterpret_cast<int*>(sc + 2 * HP * DPASS);   // [DPASS]
  float* st_m = reinterpret_cast<float*>(vrow + DPASS);      // [2*HP]
  float* st_l = st_m + 2 * HP;
  float* st_c = st_l + 2 * HP;

  const int p = positions[r];
  const int nkeys = p + 1;
  int per = nkeys > 0 ? (nkeys + a.nsplit - 1) / a.nsplit : 0;
  per = (per + 63) / 64 * 64;
  const int kb = split * per;
  const int ke = kb + per < nkeys ? kb + per : nkeys;
  if (p < 0 || kb >= ke) {                  // nothing in this split
    for (int i = tid; i < nhm; i += 256) {
      const int h = g * hpg + i / 2, m = i & 1;
      float* ml = part_ml + ((((long)r * a.H + h) * 2 + m) * a.nsplit + split) * 2;
      ml[0] = -INFINITY; ml[1] = 0.f;
    }
    return;
  }
  const int* bt = block_table + (long)row_seq[r] * a.max_blocks;
  for (int i = tid; i < hpg * kw; i += 256)
    qs[i] = ldf(q + (long)r * a.ldq + (long)g * hpg * kw + i) * a.scale;
  if (tid < nhm) { st_m[tid] = -INFINITY; st_l[tid] = 0.f; }
  __syncthreads();

  const int nsl = 256 / vdim > 0 ? 256 / vdim : 1;     // vdim <= 256
  const int pv_e = tid % vdim, pv_sl = tid / vdim;
  const bool pv_on = tid < nsl * vdim;
  float acc[2 * HP];
#pragma unroll
  for (int i = 0; i < 2 * HP; ++i) acc[i] = 0.f;

  for (int j0 = kb; j0 < ke; j0 += DPASS) {
    const int nk = ke - j0 < DPASS ? ke - j0 : DPASS;
    // ---- scores: 4 lanes per key, 16-byte pieces of the key row ----
    const int sub = tid & 3;
    for (int ks = tid >> 2; ks < nk; ks += 64) {
      const int j = j0 + ks;
      const int vr = (bt[j / a.BS] * a.G + g) * a.BS + j % a.BS;
      const T* kr = k_cache + (long)vr * kw;
      float d[2 * HP];
#pragma unroll
      for (int i = 0; i < 2 * HP; ++i) d[i] = 0.f;
      for (int c = sub * VN; c < kw; c += 4 * VN) {
        float kv[VN];
        Vec16<T>::load(kr + c, kv);
        const int m = c >= dim ? 1 : 0;       // a piece never straddles maps
#pragma unroll
        for (int hq = 0; hq < HP; ++hq) {
          if (hq < hpg) {
            const float* qq = qs + hq * kw + c;
            float x = 0.f;
#pragma unroll
            for (int i = 0; i < VN; ++i) x = fmaf(qq[i], kv[i], x);
            if (m) d[2 * hq + 1] += x; else d[2 * hq] += x;
          }
        }
      }
#pragma unroll
      for (int i = 0; i < 2 * HP; ++i) {
        d[i] += __shfl_xor(d[i], 1, WAVE);
        d[i] += __shfl_xor(d[i], 2, WAVE);
      }
      if (sub == 0) {
        vrow[ks] = vr;
#pragma unroll
        for (int i = 0; i < 2 * HP; ++i)
          if (i < nhm) sc[i * DPASS + ks] = d[i];
      }
    }
    __syncthreads();
    // ---- softmax statistics: one wave per (head, map) row ----
    for (int hm = wave; hm < nhm; hm += 4) {
      float mx = -INFINITY;
      for (int jj = lane; jj < nk; jj += 64) mx = fmaxf(mx, sc[hm * DPASS + jj]);
      mx = wave_max(mx);
      const float mo = st_m[hm];
      const float mn = fmaxf(mo, mx);
      float sum = 0.f;
      for (int jj = lane; jj < nk; jj += 64) {
        const float e = expf(sc[hm * DPASS + jj] - mn);
        sc[hm * DPASS + jj] = e;
        sum += e;
      }
      sum = wave_sum(sum);
      if (lane == 0) {
        const float c = expf(mo - mn);
        st_c[hm] = c;
        st_l[hm] = st_l[hm] * c + sum;
        st_m[hm] = mn;
      }
    }
    __syncthreads();
    // ---- weighted values: thread (value column, key slice) ----
    if (pv_on) {
#pragma unroll
      for (int i = 0; i < 2 * HP; ++i)
        if (i < nhm) acc[i] *= st_c[i];
      for (int jj = pv_sl; jj < nk; jj += nsl) {
        const float v = ldf(v_cache + (long)vrow[jj] * vdim + pv_e);
#pragma unroll
        for (int i = 0; i < 2 * HP; ++i)
          if (i < nhm) acc[i] = fmaf(sc[i * DPASS + jj], v, acc[i]);
      }
    }
    __syncthreads();
  }
  // ---- fold key slices (sc is free now): part[hm][sl][e] ----
  if (pv_on) {
#pragma unroll
    for (int i = 0; i < 2 * HP; ++i)
      if (i < nhm) sc[(i * nsl + pv_sl) * vdim + pv_e] = acc[i];
  }
  __syncthreads();
  for (int idx = tid; idx < nhm * vdim; idx += 256) {
    const int hm = idx / vdim, e = idx % vdim;
    float x = 0.f;
    for (int sl = 0; sl < nsl; ++sl) x += sc[(hm * nsl + sl) * vdim + e];
    const int h = g * hpg + hm / 2, m = hm & 1;
    part_o[((((long)r * a.H + h) * 2 + m) * a.nsplit + split) * vdim + e] = x;
  }
  if (tid < nhm) {
    const int h = g * hpg + tid / 2, m = tid & 1;
    float* ml = part_ml + ((((long)r * a.H + h) * 2 + m) * a.nsplit + split) * 2;
    ml[0] = st_m[tid]; ml[1] = st_l[tid];
  }
}

template <typename T>
__global__ __launch_bounds__(128) void diff_attn_decode_merge_kernel(
    T* __restrict__ out, const float* __restrict__ part_o,
    const float* __restrict__ part_ml, const T* __restrict__ gate,
    const int* __restrict__ positions, DecArgs a) {
  __shared__ float red[32];
  __shared__ float wts[2][64];
  const int tid = threadIdx.x;
  const int r = blockIdx.x, h = blockIdx.y;
  const int vdim = a.vdim, ns = a.nsplit;
  T* orow = out + (long)r * a.ldo + (long)h * vdim;
  if (positions[r] < 0) {
    for (int e = tid; e < vdim; e += 128) stf(orow + e, 0.f);
    return;
  }
  const float* ml = part_ml + (((long)r * a.H + h) * 2) * ns * 2;
  if (tid < 2) {
    float M = -INFINITY;
    for (int s = 0; s < ns; ++s) M = fmaxf(M, ml[(tid * ns + s) * 2]);
    float L = 0.f;
    for (int s = 0; s < ns; ++s) {
      const float w = expf(ml[(tid * ns + s) * 2] - M);
      wts[tid][s] = w;
      L += w * ml[(tid * ns + s) * 2 + 1];
    }
    const float inv = 1.0f / L;
    for (int s = 0; s < ns; ++s) wts[tid][s] *= inv;
  }
  __syncthreads();
  const float* po = part_o + (((long)r * a.H + h) * 2) * ns * vdim;
  float o[4];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int e = tid + k * 128;
    o[k] = 0.f;
    if (e < vdim) {
      float x1 = 0.f, x2 = 0.f;
      for (int s = 0; s < ns; ++s) {
        if (wts[0][s] != 0.f) x1 = fmaf(wts[0][s], po[(long)s * vdim + e], x1);
        if (wts[1][s] != 0.f)
          x2 = fmaf(wts[1][s], po[((long)ns + s) * vdim + e], x2);
      }
      o[k] = x1 - a.lambda * x2;
      ss += o[k] * o[k];
    }
  }
  const float2 tot = block_sum2(ss, 0.f, red);
  const float rs = 1.0f / sqrtf(tot.x / (float)vdim + a.eps);
  float gs = 1.f;
  if (gate) gs = 1.0f / (1.0f + expf(-ldf(gate + (long)r * a.ldg + h)));
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int e = tid + k * 128;
    if (e < vdim) stf(orow + e, o[k] * rs * a.out_scale * gs);
  }
}

template <typename T>
static void launch_decode(torch::Tensor& out, torch::Tensor& q,
                          torch::Tensor& k_cache, torch::Tensor& v_cache,
                          torch::Tensor& gate, torch::Tensor& positions,
                          torch::Tensor& row_seq, torch::Tensor& block_table,
                          torch::Tensor& part_o, torch::Tensor& part_ml,
                          const DecArgs& a, int HP, size_t shm,
                          hipStream_t stream) {
  const long rows = q.size(0);
  const bool has_gate = gate.numel() > 0;
  dim3 grid((unsigned)rows, (unsigned)a.G, (unsigned)a.nsplit);
  const T* qp = reinterpret_cast<const T*>(q.data_ptr());
  const T* kp = reinterpret_cast<const T*>(k_cache.data_ptr());
  const T* vp = reinterpret_cast<const T*>(v_cache.data_ptr());
#define KK_DEC(N)                                                            \
  diff_attn_decode_split_kernel<T, N><<<grid, 256, shm, stream>>>(           \
      part_o.data_ptr<float>(), part_ml.data_ptr<float>(), qp, kp, vp,       \
      positions.data_ptr<int>(), row_seq.data_ptr<int>(),                    \
      block_table.data_ptr<int>(), a)
  if (HP == 1) KK_DEC(1);
  else if (HP == 2) KK_DEC(2);
  else if (HP == 4) KK_DEC(4);
  else KK_DEC(8);
#undef KK_DEC
  diff_attn_decode_merge_kernel<T><<<dim3((unsigned)rows, (unsigned)a.H), 128,
                                     0, stream>>>(
      reinterpret_cast<T*>(out.data_ptr()), part_o.data_ptr<float>(),
      part_ml.data_ptr<float>(),
      has_gate ? reinterpret_cast<const T*>(gate.data_ptr()) : nullptr,
      positions.data_ptr<int>(), a);
}

bool diff_attention_decode_supported(int64_t H, int64_t G, int64_t dim,
                                     int64_t vdim, bool bf16) {
  const int vn = bf16 ? 8 : 4;
  return H % G == 0 && H / G <= 8 && dim % vn == 0 && vdim <= 256 &&
         vdim >= 1;
}

// Same contract as diff_attention for rows that are single decoded tokens.
// part_o: fp32 [rows, H, 2, nsplit, vdim]; part_ml: fp32 [rows, H, 2,
// nsplit, 2]; nsplit <= 64.
void diff_attention_decode(torch::Tensor out, torch::Tensor q,
                           torch::Tensor k_cache, torch::Tensor v_cache,
                           torch::Tensor gate, torch::Tensor positions,
                           torch::Tensor row_seq, torch::Tensor block_table,
                           torch::Tensor part_o, torch::Tensor part_ml,
                           int64_t H, double scale, double lambda, double eps,
                           double out_scale) {
  check_act(q, "q");
  TORCH_CHECK(out.scalar_type() == q.scalar_type() &&
              k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type());
  check_i32(positions, "positions"); check_i32(row_seq, "row_seq");
  check_i32(block_table, "block_table");
  check_f32(part_o, "part_o"); check_f32(part_ml, "part_ml");
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.is_contiguous() && v_cache.is_contiguous());
  DecArgs a{};
  a.H = (int)H; a.G = (int)k_cache.size(1); a.BS = (int)k_cache.size(2);
  a.dim = (int)(k_cache.size(3) / 2); a.vdim = (int)v_cache.size(3);
  TORCH_CHECK(k_cache.size(3) == 2 * a.dim);
  TORCH_CHECK(v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == a.G &&
              v_cache.size(2) == a.BS);
  TORCH_CHECK(diff_attention_decode_supported(H, a.G, a.dim, a.vdim,
                                              is_bf16(q)),
              "sizes not served by the split decode kernel");
  const long rows = q.size(0);
  TORCH_CHECK(q.dim() == 2 && q.stride(1) == 1 &&
              q.size(1) == H * 2 * a.dim);
  TORCH_CHECK(out.dim() == 2 && out.stride(1) == 1 && out.size(0) == rows &&
              out.size(1) >= H * a.vdim);
  TORCH_CHECK(positions.numel() == rows && row_seq.numel() == rows &&
              block_table.dim() == 2);
  TORCH_CHECK(part_o.dim() == 5 && part_o.size(0) >= rows &&
              part_o.size(1) == H && part_o.size(2) == 2 &&
              part_o.size(4) == a.vdim);
  a.nsplit = (int)part_o.size(3);
  TORCH_CHECK(a.nsplit >= 1 && a.nsplit <= 64);
  TORCH_CHECK(part_ml.numel() >= rows * H * 2 * a.nsplit * 2);
  const bool has_gate = gate.numel() > 0;
  if (has_gate)
    TORCH_CHECK(gate.scalar_type() == q.scalar_type() && gate.dim() == 2 &&
                gate.size(0) == rows && gate.size(1) >= H &&
                gate.stride(1) == 1);
  a.ldq = q.stride(0); a.ldo = out.stride(0);
  a.ldg = has_gate ? gate.stride(0) : 0;
  a.max_blocks = (int)block_table.size(1);
  a.scale = (float)scale; a.lambda = (float)lambda; a.eps = (float)eps;
  a.out_scale = (float)out_scale;
  if (rows == 0) return;
  const int hpg = a.H / a.G;
  const int HP = hpg <= 1 ? 1 : hpg <= 2 ? 2 : hpg <= 4 ? 4 : 8;
  const int nsl = 256 / a.vdim > 0 ? 256 / a.vdim : 1;
  size_t scf = (size_t)2 * HP * DPASS;
  const size_t fold = (size_t)2 * hpg * nsl * a.vdim;
  if (fold > scf) scf = fold;
  // layout in the kernel: qs | sc(2*HP*DPASS) | vrow | stats — the fold
  // area must fit in sc
  TORCH_CHECK(fold <= (size_t)2 * HP * DPASS,
              "value width too large for the split decode kernel");
  const size_t shm = sizeof(float) * ((size_t)hpg * 2 * a.dim +
                                      (size_t)2 * HP * DPASS + DPASS +
                                      6 * HP);
  TORCH_CHECK(shm <= 64 * 1024);
  auto stream = c10::hip::getCurrentHIPStream().stream();
  if (is_bf16(q))
    launch_decode<bf16_t>(out, q, k_cache, v_cache, gate, positions, row_seq,
                          block_table, part_o, part_ml, a, HP, shm, stream);
  else
    launch_decode<float>(out, q, k_cache, v_cache, gate, positions, row_seq,
                         block_table, part_o, part_ml, a, HP, shm, stream);
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
