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
  int hsplit;          // units per kv head: each takes (H/G)/hsplit heads
  float scale, lambda, eps, out_scale;
};


// Sum NV values (a power of two, <= 16) over the 16 lanes that share
// `sub`'s upper bits. Lanes trade halves (xor 8, 4, 2, 1), so NV - 1
// exchanges replace 4 * NV; afterwards d[0] of the lanes with index >= 0
// holds the total of value `index`.
template <int NV>
DEV_INLINE int reduce_scatter16(float* d, int sub) {
  int idx = 0;
  int n = NV;
#pragma unroll
  for (int mask = 8; mask >= 1; mask >>= 1) {
    const bool up = (sub & mask) != 0;
    if (n > 1) {
      n >>= 1;
#pragma unroll
      for (int i = 0; i < NV / 2; ++i) {
        if (i < n) {
          const float send = up ? d[i] : d[i + n];
          const float keep = up ? d[i + n] : d[i];
          d[i] = keep + __shfl_xor(send, mask, WAVE);
        }
      }
      idx = idx * 2 + (up ? 1 : 0);
    } else {
      d[0] += __shfl_xor(d[0], mask, WAVE);
      if (up) idx = -1;                      // one writer per value
    }
  }
  return idx;
}

// One WAVE per (row, kv head, key split): the four waves of a workgroup
// are independent units with private LDS and never meet at a barrier, so a
// CU keeps as many splits in flight as its registers allow.
// HP: compile-time bound on H/G; CH: 8-element pieces of a key row per lane
// (16 lanes share a key, so a key row has at most 16 * CH pieces). A pass
// covers P = 16 keys: every lane issues all its K and V loads of the pass
// before using any, one HBM round trip per pass.
template <typename T, int HP, int CH>
__global__ __launch_bounds__(256) void diff_attn_decode_split_kernel(
    float* __restrict__ part_o,    // [rows, H, 2, nsplit, vdim]
    float* __restrict__ part_ml,   // [rows, H, 2, nsplit, 2]
    const T* __restrict__ q, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ block_table,
    DecArgs a, int units) {
  extern __shared__ float smem[];
  constexpr int KB = 4, P = 4 * KB;         // keys per lane group / per pass
  constexpr int VR = 256;                   // cache rows looked up at once
  constexpr int WSZ = 2 * HP * P + VR + 6 * HP;  // floats of LDS per wave
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int unit = blockIdx.x * 4 + wave;
  if (unit >= units) return;
  // units that differ only in their share of the group's heads are
  // neighbours, so the second reader of a K/V row finds it in cache
  const int gsub = unit % (a.G * a.hsplit);
  const int split = (unit / (a.G * a.hsplit)) % a.nsplit;
  const int r = unit / (a.nsplit * a.G * a.hsplit);
  const int g = gsub / a.hsplit;
  const int dim = a.dim, vdim = a.vdim, kw = 2 * dim;
  const int hpg = (a.H / a.G) / a.hsplit;   // heads of this unit
  const int h0 = g * (a.H / a.G) + (gsub % a.hsplit) * hpg;
  const int nhm = 2 * hpg;
  float* sc = smem + wave * WSZ;            // [2*HP][P]
  int* vrow_all = reinterpret_cast<int*>(sc + 2 * HP * P);   // [VR]
  float* st_m = reinterpret_cast<float*>(vrow_all + VR);     // [2*HP]
  float* st_l = st_m + 2 * HP;
  float* st_c = st_l + 2 * HP;

  const int p = positions[r];
  const int nkeys = p + 1;
  int per = nkeys > 0 ? (nkeys + a.nsplit - 1) / a.nsplit : 0;
  per = (per + P - 1) / P * P;
  const int kb = split * per;
  const int ke = kb + per < nkeys ? kb + per : nkeys;
  if (p < 0 || kb >= ke) {                  // nothing in this split
    if (lane < nhm) {
      const int h = h0 + lane / 2, m = lane & 1;
      float* ml = part_ml +
                  ((((long)r * a.H + h) * 2 + m) * a.nsplit + split) * 2;
      ml[0] = -INFINITY; ml[1] = 0.f;
    }
    return;
  }
  const int* bt = block_table + (long)row_seq[r] * a.max_blocks;
  const int sub = lane & 15, grp = lane >> 4;
  float qreg[HP][CH][8];
#pragma unroll
  for (int hq = 0; hq < HP; ++hq)
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
      const int c = (sub + 16 * ch) * 8;
#pragma unroll
      for (int i = 0; i < 8; ++i) qreg[hq][ch][i] = 0.f;
      if (hq < hpg && c < kw) {
        ld8(q + (long)r * a.ldq + (long)(h0 + hq) * kw + c,
            qreg[hq][ch]);
#pragma unroll
        for (int i = 0; i < 8; ++i) qreg[hq][ch][i] *= a.scale;
      }
    }
  if (lane < nhm) { st_m[lane] = -INFINITY; st_l[lane] = 0.f; }

  const int nvec = vdim / 8;                // power of two, <= 16
  const int nsl = 64 / nvec;                // key slices of the value step
  const int pv_v = lane % nvec, pv_sl = lane / nvec;
  float acc[2 * HP][8];
#pragma unroll
  for (int i = 0; i < 2 * HP; ++i)
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[i][k] = 0.f;

  for (int j0 = kb; j0 < ke; j0 += P) {
    const int nk = ke - j0 < P ? ke - j0 : P;
    // the page lookups of the next VR keys are made together, so a pass
    // waits on one memory round trip (its K and V rows), not two
    if ((j0 - kb) % VR == 0) {
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int t = 0; t < VR / 64; ++t) {
        const int j = j0 + lane + 64 * t;
        if (j < ke)
          vrow_all[lane + 64 * t] =
              (bt[j / a.BS] * a.G + g) * a.BS + j % a.BS;
      }
    }
    const int* vrow = vrow_all + (j0 - kb) % VR;
    __builtin_amdgcn_wave_barrier();
    // ---- all loads of the pass ----
    Raw8<T> kraw[KB][CH];
#pragma unroll
    for (int b = 0; b < KB; ++b) {
      const int ks = grp + 4 * b < nk ? grp + 4 * b : nk - 1;
      const T* kr = k_cache + (long)vrow[ks] * kw;
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) {
        const int c = (sub + 16 * ch) * 8;
        if (c < kw) kraw[b][ch].load(kr + c);
      }
    }
    Raw8<T> vraw[KB];                       // P / nsl <= KB keys per lane
#pragma unroll
    for (int b = 0; b < KB; ++b) {
      const int jj = pv_sl + b * nsl < nk ? pv_sl + b * nsl : nk - 1;
      vraw[b].load(v_cache + (long)vrow[jj] * vdim + pv_v * 8);
    }
    // ---- scores ----
#pragma unroll
    for (int b = 0; b < KB; ++b) {
      float d[2 * HP];
#pragma unroll
      for (int i = 0; i < 2 * HP; ++i) d[i] = 0.f;
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) {
        const int c = (sub + 16 * ch) * 8;
        if (c < kw) {
          const bool second = c >= dim;     // a piece lies in one map
          float kv[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) kv[i] = kraw[b][ch].get(i);
#pragma unroll
          for (int hq = 0; hq < HP; ++hq) {
            float x = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) x = fmaf(qreg[hq][ch][i], kv[i], x);
            if (second) d[2 * hq + 1] += x; else d[2 * hq] += x;
          }
        }
      }
      // reduce over the 16 lanes of the key, scattering the 2*HP sums:
      // each exchange halves the values a lane still carries
      const int idx = reduce_scatter16<2 * HP>(d, sub);
      const int ks = grp + 4 * b;
      if (idx >= 0 && idx < nhm && ks < nk) sc[idx * P + ks] = d[0];
    }
    __builtin_amdgcn_wave_barrier();
    // ---- softmax statistics: 8 lanes per (head, map) row ----
    for (int hm = lane >> 3; hm < ((nhm + 7) & ~7); hm += 8) {
      const int l8 = lane & 7;
      const bool on = hm < nhm;
      float s4[P / 8];
      float mx = -INFINITY;
#pragma unroll
      for (int t = 0; t < P / 8; ++t) {
        const int jj = l8 + 8 * t;
        s4[t] = (on && jj < nk) ? sc[hm * P + jj] : -INFINITY;
        mx = fmaxf(mx, s4[t]);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 1, WAVE));
      mx = fmaxf(mx, __shfl_xor(mx, 2, WAVE));
      mx = fmaxf(mx, __shfl_xor(mx, 4, WAVE));
      const float mo = on ? st_m[hm] : 0.f;
      const float mn = fmaxf(mo, mx);
      float sum = 0.f;
#pragma unroll
      for (int t = 0; t < P / 8; ++t) {
        const int jj = l8 + 8 * t;
        const float e = expf(s4[t] - mn);
        if (on && jj < nk) { sc[hm * P + jj] = e; sum += e; }
      }
      sum += __shfl_xor(sum, 1, WAVE);
      sum += __shfl_xor(sum, 2, WAVE);
      sum += __shfl_xor(sum, 4, WAVE);
      if (on && l8 == 0) {
        const float c = expf(mo - mn);
        st_c[hm] = c;
        st_l[hm] = st_l[hm] * c + sum;
        st_m[hm] = mn;
      }
    }
    __builtin_amdgcn_wave_barrier();
    // ---- weighted values ----
#pragma unroll
    for (int i = 0; i < 2 * HP; ++i)
      if (i < nhm) {
        const float c = st_c[i];
#pragma unroll
        for (int k = 0; k < 8; ++k) acc[i][k] *= c;
      }
#pragma unroll
    for (int b = 0; b < KB; ++b) {
      const int jj = pv_sl + b * nsl;
      if (jj < nk) {
        float v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = vraw[b].get(k);
#pragma unroll
        for (int i = 0; i < 2 * HP; ++i)
          if (i < nhm) {
            const float w = sc[i * P + jj];
#pragma unroll
            for (int k = 0; k < 8; ++k) acc[i][k] = fmaf(w, v[k], acc[i][k]);
          }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  // ---- fold the key slices by shuffles; lanes < nvec hold the sums ----
#pragma unroll
  for (int i = 0; i < 2 * HP; ++i)
#pragma unroll
    for (int k = 0; k < 8; ++k)
      for (int off = nvec; off < 64; off <<= 1)
        acc[i][k] += __shfl_xor(acc[i][k], off, WAVE);
  if (lane < nvec) {
#pragma unroll
    for (int i = 0; i < 2 * HP; ++i)
      if (i < nhm) {
        const int h = h0 + i / 2, m = i & 1;
        st8(part_o + ((((long)r * a.H + h) * 2 + m) * a.nsplit + split) *
                         vdim + lane * 8, acc[i]);
      }
  }
  if (lane < nhm) {
    const int h = h0 + lane / 2, m = lane & 1;
    float* ml = part_ml +
                ((((long)r * a.H + h) * 2 + m) * a.nsplit + split) * 2;
    ml[0] = st_m[lane]; ml[1] = st_l[lane];
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
                          const DecArgs& a, int HP, int CH, int region,
                          size_t shm, hipStream_t stream) {
  const long rows = q.size(0);
  const bool has_gate = gate.numel() > 0;
  const int units = (int)rows * a.G * a.hsplit * a.nsplit;
  dim3 grid((unsigned)((units + 3) / 4));
  const T* qp = reinterpret_cast<const T*>(q.data_ptr());
  const T* kp = reinterpret_cast<const T*>(k_cache.data_ptr());
  const T* vp = reinterpret_cast<const T*>(v_cache.data_ptr());
#define KK_DEC(N, C)                                                         \
  diff_attn_decode_split_kernel<T, N, C><<<grid, 256, shm, stream>>>(        \
      part_o.data_ptr<float>(), part_ml.data_ptr<float>(), qp, kp, vp,       \
      positions.data_ptr<int>(), row_seq.data_ptr<int>(),                    \
      block_table.data_ptr<int>(), a, units)
  if (CH == 1) {
    if (HP == 1) KK_DEC(1, 1);
    else if (HP == 2) KK_DEC(2, 1);
    else if (HP == 4) KK_DEC(4, 1);
    else KK_DEC(8, 1);
  } else {
    if (HP == 1) KK_DEC(1, 2);
    else if (HP == 2) KK_DEC(2, 2);
    else if (HP == 4) KK_DEC(4, 2);
    else KK_DEC(8, 2);
  }
#undef KK_DEC
  diff_attn_decode_merge_kernel<T><<<dim3((unsigned)rows, (unsigned)a.H), 128,
                                     0, stream>>>(
      reinterpret_cast<T*>(out.data_ptr()), part_o.data_ptr<float>(),
      part_ml.data_ptr<float>(),
      has_gate ? reinterpret_cast<const T*>(gate.data_ptr()) : nullptr,
      positions.data_ptr<int>(), a);
}

static int pad_hp(int hpg) {
  return hpg <= 1 ? 1 : hpg <= 2 ? 2 : hpg <= 4 ? 4 : 8;
}

bool diff_attention_decode_supported(int64_t H, int64_t G, int64_t dim,
                                     int64_t vdim, bool bf16) {
  (void)bf16;
  if (G < 1 || H % G != 0 || H / G > 8) return false;
  if (dim % 8 != 0 || 2 * dim > 256) return false;      // <= 32 pieces
  if (vdim % 8 != 0) return false;
  const int64_t nvec = vdim / 8;           // P / (64 / nvec) <= KB keys a lane
  return nvec <= 16 && (nvec & (nvec - 1)) == 0;
}

template <typename T>
static int64_t capacity_of(int HP, int CH, size_t shm) {
  int blocks = 0;
  hipError_t e = hipErrorUnknown;
#define KK_OCC(N, C)                                                        \
  e = hipOccupancyMaxActiveBlocksPerMultiprocessor(                         \
      &blocks, diff_attn_decode_split_kernel<T, N, C>, 256, shm)
  if (CH == 1) {
    if (HP == 1) KK_OCC(1, 1); else if (HP == 2) KK_OCC(2, 1);
    else if (HP == 4) KK_OCC(4, 1); else KK_OCC(8, 1);
  } else {
    if (HP == 1) KK_OCC(1, 2); else if (HP == 2) KK_OCC(2, 2);
    else if (HP == 4) KK_OCC(4, 2); else KK_OCC(8, 2);
  }
#undef KK_OCC
  if (e != hipSuccess || blocks < 1) blocks = 1;
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess)
    hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  return (int64_t)blocks * 4 * cus;
}

static void decode_shape(int hpg_all, int dim, int* hsplit, int* HP, int* CH,
                         size_t* shm) {
  *hsplit = (hpg_all > 2 && hpg_all % 2 == 0) ? hpg_all / 2 : 1;
  *HP = pad_hp(hpg_all / *hsplit);
  *CH = 2 * dim / 8 <= 16 ? 1 : 2;
  *shm = sizeof(float) * 4 * (size_t)(2 * *HP * 16 + 256 + 6 * *HP);
}

// How many (row, kv head share, split) units the device runs at once: the
// caller picks the split count so that one launch is one full wave of
// units (a second, partly filled round costs as much as the first).
int64_t diff_attention_decode_capacity(int64_t H, int64_t G, int64_t dim,
                                       bool bf16) {
  int hsplit, HP, CH;
  size_t shm;
  decode_shape((int)(H / G), (int)dim, &hsplit, &HP, &CH, &shm);
  return bf16 ? capacity_of<bf16_t>(HP, CH, shm)
              : capacity_of<float>(HP, CH, shm);
}

int64_t diff_attention_decode_units_per_row(int64_t H, int64_t G) {
  const int hpg_all = (int)(H / G);
  return G * ((hpg_all > 2 && hpg_all % 2 == 0) ? hpg_all / 2 : 1);
}

// Same arguments and result as diff_attention for rows that are single decoded tokens.
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
  int HP, CH;
  size_t shm;
  decode_shape(a.H / a.G, a.dim, &a.hsplit, &HP, &CH, &shm);
  const int region = 0;
  TORCH_CHECK(shm <= 64 * 1024);
  TORCH_CHECK(aligned16(q.data_ptr()) && q.stride(0) % 8 == 0 &&
              aligned16(k_cache.data_ptr()) && aligned16(v_cache.data_ptr()));
  auto stream = c10::hip::getCurrentHIPStream().stream();
  if (is_bf16(q))
    launch_decode<bf16_t>(out, q, k_cache, v_cache, gate, positions, row_seq,
                          block_table, part_o, part_ml, a, HP, CH, region, shm,
                          stream);
  else
    launch_decode<float>(out, q, k_cache, v_cache, gate, positions, row_seq,
                         block_table, part_o, part_ml, a, HP, CH, region, shm,
                          stream);
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
