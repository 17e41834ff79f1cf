// Latent attention: per token the paged cache holds ONE row
// [c (R entries) | k_rot (dr entries)] shared by all heads.
//
// latent_kv_append   norms the query latent and the key/value latent of
//                    every row, rotates the shared key part and writes the
//                    cache row.
// latent_attention   for every (row, head): scores over the last `window`
//                    positions, q_abs . c + rot(q_rot) . k_rot, softmax,
//                    and the weighted sum of the latents c. The products
//                    with the per-head key and value expansions live
//                    outside, on the query and output side.
//
// Everything is accumulated in fp32. A row walks its keys oldest first in
// chunks counted from the first visible key, so its result depends only on
// its own position and window.
#include "elem.h"

namespace kukeon {

// One block per row. cs [positions, dims] = [cos_0.. | sin_0..]; pairs
// (2i, 2i+1) of the first `dims` entries of the rotated part turn.
template <typename T>
__global__ __launch_bounds__(256) void latent_kv_append_kernel(
    T* __restrict__ cq_out, T* __restrict__ cache, const T* __restrict__ proj,
    long ldp, long q_col, long kv_col, const float* __restrict__ wq,
    const float* __restrict__ wkv, float eps, const float* __restrict__ cs,
    int cs_rows, int dims, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ block_table,
    int max_blocks, int Rq, int R, int dr, int BS) {
  __shared__ float red[32];
  const long r = blockIdx.x;
  const int p = positions[r];
  if (p < 0) return;
  const T* row = proj + r * ldp;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < Rq; i += blockDim.x) {
    const float v = ldf(row + q_col + i);
    sq += v * v;
  }
  for (int i = threadIdx.x; i < R; i += blockDim.x) {
    const float v = ldf(row + kv_col + i);
    sk += v * v;
  }
  const float2 tot = block_sum2(sq, sk, red);
  const float rq = 1.0f / sqrtf(tot.x / (float)Rq + eps);
  const float rk = 1.0f / sqrtf(tot.y / (float)R + eps);
  for (int i = threadIdx.x; i < Rq; i += blockDim.x)
    stf(cq_out + r * (long)Rq + i, ldf(row + q_col + i) * rq * wq[i]);
  const int s = row_seq[r];
  const long blk = block_table[(long)s * max_blocks + p / BS];
  T* crow = cache + (blk * BS + p % BS) * (long)(R + dr);
  for (int i = threadIdx.x; i < R; i += blockDim.x)
    stf(crow + i, ldf(row + kv_col + i) * rk * wkv[i]);
  const int pp = p < cs_rows ? p : cs_rows - 1;
  const float* ang = cs + (long)pp * dims;
  const int half = dims / 2;
  for (int i = threadIdx.x; i < dr; i += blockDim.x) {
    const float v = ldf(row + kv_col + R + i);
    float o = v;
    if (i < dims) {
      const int pr = i >> 1;
      const float other = ldf(row + kv_col + R + (i ^ 1));
      const float c = ang[pr], sn = ang[half + pr];
      o = (i & 1) ? fmaf(v, c, other * sn) : fmaf(v, c, -other * sn);
    }
    stf(crow + R + i, o);
  }
}

void latent_kv_append(torch::Tensor cq_out, torch::Tensor cache,
                      torch::Tensor proj, int64_t q_col, int64_t kv_col,
                      torch::Tensor wq, torch::Tensor wkv, double eps,
                      torch::Tensor cs, torch::Tensor positions,
                      torch::Tensor row_seq, torch::Tensor block_table) {
  check_act(proj, "proj");
  check_f32(wq, "wq"); check_f32(wkv, "wkv"); check_f32(cs, "cs");
  check_i32(positions, "positions"); check_i32(row_seq, "row_seq");
  check_i32(block_table, "block_table");
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1);
  const long rows = proj.size(0);
  const int Rq = (int)wq.numel(), R = (int)wkv.numel();
  TORCH_CHECK(cache.dim() == 4 && cache.is_contiguous() && cache.size(1) == 1 &&
              cache.scalar_type() == proj.scalar_type());
  const int BS = (int)cache.size(2);
  const int dr = (int)cache.size(3) - R;
  TORCH_CHECK(dr >= 0);
  TORCH_CHECK(cs.dim() == 2 && cs.size(0) >= 1);
  const int dims = (int)cs.size(1);
  TORCH_CHECK(dims % 2 == 0 && dims <= dr);
  TORCH_CHECK(q_col >= 0 && q_col + Rq <= proj.size(1) && kv_col >= 0 &&
              kv_col + R + dr <= proj.size(1));
  TORCH_CHECK(cq_out.dim() == 2 && cq_out.is_contiguous() &&
              cq_out.size(0) == rows && cq_out.size(1) == Rq &&
              cq_out.scalar_type() == proj.scalar_type());
  TORCH_CHECK(positions.numel() == rows && row_seq.numel() == rows);
  TORCH_CHECK(block_table.dim() == 2);
  if (rows == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  KK_DISPATCH_ACT(proj, {
    latent_kv_append_kernel<T><<<dim3((unsigned)rows), 256, 0, stream>>>(
        reinterpret_cast<T*>(cq_out.data_ptr()),
        reinterpret_cast<T*>(cache.data_ptr()),
        reinterpret_cast<const T*>(proj.data_ptr()), (long)proj.stride(0),
        (long)q_col, (long)kv_col, wq.data_ptr<float>(), wkv.data_ptr<float>(),
        (float)eps, cs.data_ptr<float>(), (int)cs.size(0), dims,
        positions.data_ptr<int>(), row_seq.data_ptr<int>(),
        block_table.data_ptr<int>(), (int)block_table.size(1), Rq, R, dr, BS);
  });
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
// Row-wise attention, any sizes, both formats. Block = (row, HB heads), 256
// threads. Keys are taken 256 at a time: thread j scores key j for the HB
// heads (the query vectors sit in LDS as fp32 and are read as broadcasts),
// the block agrees on the running maximum and sum, then thread d sums the
// weighted latents for output entries d, d+256, ...
#define LAT_HB 4
#define LAT_CH 256

template <typename T, int ND>
__global__ __launch_bounds__(256) void latent_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q_abs, const T* __restrict__ q,
    long ldq, const T* __restrict__ cache, const float* __restrict__ cs,
    int cs_rows, int dims, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ block_table,
    int max_blocks, long rows, int H, int dn, int dr, int R, int BS,
    int window, float scale) {
  extern __shared__ float sm[];
  const int KW = R + dr;
  float* sq = sm;                          // [HB][KW] query (latent | rot)
  float* sc = sq + LAT_HB * KW;            // [HB][CH] scores / weights
  __shared__ float red[32];
  __shared__ long srow[LAT_CH];            // first element of each key's row
  const long r = blockIdx.x;
  const int h0 = blockIdx.y * LAT_HB;
  const int tid = threadIdx.x;
  const int p = positions[r];
  if (p < 0) {
    for (int hb = 0; hb < LAT_HB && h0 + hb < H; ++hb)
      for (int d = tid; d < R; d += blockDim.x)
        stf(out + ((long)(h0 + hb) * rows + r) * R + d, 0.f);
    return;
  }
  const int s = row_seq[r];
  const int pp = p < cs_rows ? p : cs_rows - 1;
  const float* ang = cs + (long)pp * dims;
  const int half = dims / 2;
  for (int i = tid; i < LAT_HB * KW; i += blockDim.x) {
    const int hb = i / KW, d = i - hb * KW;
    const int h = h0 + hb;
    float v = 0.f;
    if (h < H) {
      if (d < R) {
        v = ldf(q_abs + ((long)h * rows + r) * R + d);
      } else {
        const int e = d - R;
        const T* qr = q + r * ldq + (long)h * (dn + dr) + dn;
        v = ldf(qr + e);
        if (e < dims) {
          const float other = ldf(qr + (e ^ 1));
          const float c = ang[e >> 1], sn = ang[half + (e >> 1)];
          v = (e & 1) ? fmaf(v, c, other * sn) : fmaf(v, c, -other * sn);
        }
      }
    }
    sq[i] = v;
  }
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int nkeys = p - lo + 1;
  float m[LAT_HB], l[LAT_HB], acc[LAT_HB][ND];
#pragma unroll
  for (int hb = 0; hb < LAT_HB; ++hb) {
    m[hb] = -INFINITY;
    l[hb] = 0.f;
#pragma unroll
    for (int k = 0; k < ND; ++k) acc[hb][k] = 0.f;
  }
  const int* bt = block_table + (long)s * max_blocks;
  for (int c0 = 0; c0 < nkeys; c0 += LAT_CH) {
    const int cn = min(LAT_CH, nkeys - c0);
    __syncthreads();                       // sq ready / previous chunk done
    float sv[LAT_HB];
#pragma unroll
    for (int hb = 0; hb < LAT_HB; ++hb) sv[hb] = -INFINITY;
    if (tid < cn) {
      const int j = lo + c0 + tid;
      const long base = ((long)bt[j / BS] * BS + j % BS) * KW;
      srow[tid] = base;
      const T* kr = cache + base;
      float a[LAT_HB];
#pragma unroll
      for (int hb = 0; hb < LAT_HB; ++hb) a[hb] = 0.f;
      for (int d = 0; d < KW; ++d) {
        const float kv = ldf(kr + d);
#pragma unroll
        for (int hb = 0; hb < LAT_HB; ++hb)
          a[hb] = fmaf(sq[hb * KW + d], kv, a[hb]);
      }
#pragma unroll
      for (int hb = 0; hb < LAT_HB; ++hb) sv[hb] = a[hb] * scale;
    }
    float alpha[LAT_HB];
#pragma unroll
    for (int hb = 0; hb < LAT_HB; hb += 2) {
      const float2 mx = block_max2(sv[hb], sv[hb + 1], red);
      const float m0 = fmaxf(m[hb], mx.x), m1 = fmaxf(m[hb + 1], mx.y);
      alpha[hb] = __expf(m[hb] - m0);       // first chunk: exp(-inf) = 0
      alpha[hb + 1] = __expf(m[hb + 1] - m1);
      m[hb] = m0;
      m[hb + 1] = m1;
      const float w0 = tid < cn ? __expf(sv[hb] - m0) : 0.f;
      const float w1 = tid < cn ? __expf(sv[hb + 1] - m1) : 0.f;
      sc[hb * LAT_CH + tid] = w0;
      sc[(hb + 1) * LAT_CH + tid] = w1;
      const float2 su = block_sum2(w0, w1, red);
      l[hb] = l[hb] * alpha[hb] + su.x;
      l[hb + 1] = l[hb + 1] * alpha[hb + 1] + su.y;
    }
    // block_sum2 ends with a barrier: sc and srow are visible
#pragma unroll
    for (int hb = 0; hb < LAT_HB; ++hb)
#pragma unroll
      for (int k = 0; k < ND; ++k) acc[hb][k] *= alpha[hb];
    for (int jj = 0; jj < cn; ++jj) {
      const T* kr = cache + srow[jj];
#pragma unroll
      for (int k = 0; k < ND; ++k) {
        const int d = tid + k * 256;
        if (d < R) {
          const float cv = ldf(kr + d);
#pragma unroll
          for (int hb = 0; hb < LAT_HB; ++hb)
            acc[hb][k] = fmaf(sc[hb * LAT_CH + jj], cv, acc[hb][k]);
        }
      }
    }
  }
#pragma unroll
  for (int hb = 0; hb < LAT_HB; ++hb) {
    const int h = h0 + hb;
    if (h >= H) break;
    const float inv = 1.0f / l[hb];
#pragma unroll
    for (int k = 0; k < ND; ++k) {
      const int d = tid + k * 256;
      if (d < R) stf(out + ((long)h * rows + r) * R + d, acc[hb][k] * inv);
    }
  }
}

// Vector form of the same walk: rows of whole 16-byte chunks, a latent of
// 8 * 2^k entries. Scores: thread j reads its key row in 16-byte pieces.
// Weighted sum: R/8 threads cover one latent row (8 entries each) and the
// 256 / (R/8) thread groups take every NG-th key of the chunk; the groups'
// partial sums meet in LDS at the end, added in group order.
template <typename T>
__global__ __launch_bounds__(256) void latent_attention_vec_kernel(
    T* __restrict__ out, const T* __restrict__ q_abs, const T* __restrict__ q,
    long ldq, const T* __restrict__ cache, const float* __restrict__ cs,
    int cs_rows, int dims, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ block_table,
    int max_blocks, long rows, int H, int dn, int dr, int R, int BS,
    int window, float scale, int NS, float* __restrict__ split_o,
    float* __restrict__ split_ml) {
  extern __shared__ float sm[];
  const int KW = R + dr;
  float* sq = sm;                          // [HB][KW]
  float* sc = sq + LAT_HB * KW;            // [HB][CH]
  float* part = sc + LAT_HB * LAT_CH;      // [NG][HB][R] = 256 * 32 floats
  __shared__ float red[32];
  __shared__ long srow[LAT_CH];
  const long r = blockIdx.x;
  const int h0 = blockIdx.y * LAT_HB;
  const int tid = threadIdx.x;
  const int p = positions[r];
  if (p < 0) {
    // an inactive row: zeros (from the first split; the merge is told by
    // a zero sum to write zeros too)
    for (int hb = 0; hb < LAT_HB && h0 + hb < H; ++hb) {
      if (NS == 1) {
        for (int d = tid; d < R; d += blockDim.x)
          stf(out + ((long)(h0 + hb) * rows + r) * R + d, 0.f);
      } else if (tid == 0) {
        float* ml = split_ml + ((r * H + h0 + hb) * NS + blockIdx.z) * 2;
        ml[0] = -INFINITY;
        ml[1] = 0.f;
      }
    }
    return;
  }
  const int s = row_seq[r];
  const int pp = p < cs_rows ? p : cs_rows - 1;
  const float* ang = cs + (long)pp * dims;
  const int half = dims / 2;
  for (int i = tid; i < LAT_HB * KW; i += blockDim.x) {
    const int hb = i / KW, d = i - hb * KW;
    const int h = h0 + hb;
    float v = 0.f;
    if (h < H) {
      if (d < R) {
        v = ldf(q_abs + ((long)h * rows + r) * R + d);
      } else {
        const int e = d - R;
        const T* qr = q + r * ldq + (long)h * (dn + dr) + dn;
        v = ldf(qr + e);
        if (e < dims) {
          const float other = ldf(qr + (e ^ 1));
          const float c = ang[e >> 1], sn = ang[half + (e >> 1)];
          v = (e & 1) ? fmaf(v, c, other * sn) : fmaf(v, c, -other * sn);
        }
      }
    }
    sq[i] = v;
  }
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int nkeys = p - lo + 1;
  // this block's share of the key chunks (all of them when NS == 1)
  const int nch = (nkeys + LAT_CH - 1) / LAT_CH;
  const int cps = (nch + NS - 1) / NS;
  const int key_begin = (int)blockIdx.z * cps * LAT_CH;
  const int key_end = min(nkeys, ((int)blockIdx.z + 1) * cps * LAT_CH);
  const int per_row = R / 8;               // threads that cover one latent
  const int NG = 256 / per_row;
  const int dg = tid % per_row;
  const int kg = tid / per_row;
  float m[LAT_HB], l[LAT_HB], acc[LAT_HB][8];
#pragma unroll
  for (int hb = 0; hb < LAT_HB; ++hb) {
    m[hb] = -INFINITY;
    l[hb] = 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[hb][k] = 0.f;
  }
  const int* bt = block_table + (long)s * max_blocks;
  const int nchunks8 = KW / 8;
  for (int c0 = key_begin; c0 < key_end; c0 += LAT_CH) {
    const int cn = min(LAT_CH, key_end - c0);
    __syncthreads();
    float sv[LAT_HB];
#pragma unroll
    for (int hb = 0; hb < LAT_HB; ++hb) sv[hb] = -INFINITY;
    if (tid < cn) {
      const int j = lo + c0 + tid;
      const long base = ((long)bt[j / BS] * BS + j % BS) * KW;
      srow[tid] = base;
      const T* kr = cache + base;
      float a[LAT_HB];
#pragma unroll
      for (int hb = 0; hb < LAT_HB; ++hb) a[hb] = 0.f;
#pragma unroll 4
      for (int d8 = 0; d8 < nchunks8; ++d8) {
        Raw8<T> kv;
        kv.load(kr + d8 * 8);
#pragma unroll
        for (int hb = 0; hb < LAT_HB; ++hb) {
          const float* qh = sq + hb * KW + d8 * 8;
#pragma unroll
          for (int k = 0; k < 8; ++k) a[hb] = fmaf(qh[k], kv.get(k), a[hb]);
        }
      }
#pragma unroll
      for (int hb = 0; hb < LAT_HB; ++hb) sv[hb] = a[hb] * scale;
    }
    float alpha[LAT_HB];
#pragma unroll
    for (int hb = 0; hb < LAT_HB; hb += 2) {
      const float2 mx = block_max2(sv[hb], sv[hb + 1], red);
      const float m0 = fmaxf(m[hb], mx.x), m1 = fmaxf(m[hb + 1], mx.y);
      alpha[hb] = __expf(m[hb] - m0);
      alpha[hb + 1] = __expf(m[hb + 1] - m1);
      m[hb] = m0;
      m[hb + 1] = m1;
      const float w0 = tid < cn ? __expf(sv[hb] - m0) : 0.f;
      const float w1 = tid < cn ? __expf(sv[hb + 1] - m1) : 0.f;
      sc[hb * LAT_CH + tid] = w0;
      sc[(hb + 1) * LAT_CH + tid] = w1;
      const float2 su = block_sum2(w0, w1, red);
      l[hb] = l[hb] * alpha[hb] + su.x;
      l[hb + 1] = l[hb + 1] * alpha[hb + 1] + su.y;
    }
#pragma unroll
    for (int hb = 0; hb < LAT_HB; ++hb)
#pragma unroll
      for (int k = 0; k < 8; ++k) acc[hb][k] *= alpha[hb];
#pragma unroll 4
    for (int jj = kg; jj < cn; jj += NG) {
      Raw8<T> cv;
      cv.load(cache + srow[jj] + dg * 8);
#pragma unroll
      for (int hb = 0; hb < LAT_HB; ++hb) {
        const float w = sc[hb * LAT_CH + jj];
#pragma unroll
        for (int k = 0; k < 8; ++k) acc[hb][k] = fmaf(w, cv.get(k), acc[hb][k]);
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int hb = 0; hb < LAT_HB; ++hb)
#pragma unroll
    for (int k = 0; k < 8; ++k)
      part[((long)kg * LAT_HB + hb) * R + dg * 8 + k] = acc[hb][k];
  __syncthreads();
  for (int i = tid; i < LAT_HB * R; i += blockDim.x) {
    const int hb = i / R, d = i - hb * R;
    const int h = h0 + hb;
    if (h >= H) continue;
    float sum = 0.f;
    for (int g = 0; g < NG; ++g) sum += part[((long)g * LAT_HB + hb) * R + d];
    // m and l are the same in every thread; pick them by a uniform chain
    float lh = l[0], mh = m[0];
#pragma unroll
    for (int x = 1; x < LAT_HB; ++x) {
      lh = hb == x ? l[x] : lh;
      mh = hb == x ? m[x] : mh;
    }
    if (NS == 1) {
      stf(out + ((long)h * rows + r) * R + d, sum / lh);
    } else {
      const long u = (r * H + h) * NS + blockIdx.z;
      split_o[u * R + d] = sum;
      if (d == 0) {
        split_ml[u * 2] = mh;
        split_ml[u * 2 + 1] = lh;
      }
    }
  }
}

// Folds the key splits of a row: out = sum_z e^(m_z - M) o_z / sum_z
// e^(m_z - M) l_z, splits in order. A row without keys gives zeros.
template <typename T>
__global__ __launch_bounds__(256) void latent_attention_merge_kernel(
    T* __restrict__ out, const float* __restrict__ split_o,
    const float* __restrict__ split_ml, long rows, int H, int R, int NS) {
  const long r = blockIdx.x;
  const int h = blockIdx.y;
  const long u0 = (r * H + h) * NS;
  float M = -INFINITY;
  for (int z = 0; z < NS; ++z) M = fmaxf(M, split_ml[(u0 + z) * 2]);
  float L = 0.f;
  for (int z = 0; z < NS; ++z) {
    const float mz = split_ml[(u0 + z) * 2];
    if (mz > -INFINITY) L += __expf(mz - M) * split_ml[(u0 + z) * 2 + 1];
  }
  for (int d = threadIdx.x; d < R; d += blockDim.x) {
    float acc = 0.f;
    for (int z = 0; z < NS; ++z) {
      const float mz = split_ml[(u0 + z) * 2];
      if (mz > -INFINITY) acc += __expf(mz - M) * split_o[(u0 + z) * R + d];
    }
    stf(out + ((long)h * rows + r) * R + d, L > 0.f ? acc / L : 0.f);
  }
}

// ---------------------------------------------------------------------------
// Matrix-core form for prompt portions (bf16). One wave owns (row, 16 heads)
// and walks the row's window 16 keys at a time; tiles start at multiples of
// 16 in absolute position, so a row's sums do not depend on where its portion
// began. No barriers: the two waves of a workgroup are independent and each
// has its own LDS area.
//   scores  S^T[key, head] = K[key, :] . Q[head, :]   v_mfma_f32_16x16x32_bf16
//           A = cache rows straight from memory (lane = key, 8 entries of the
//           row per k block), B = the query fragments held in registers.
//   softmax per head in fp32: a lane holds 4 keys of one head, two exchanges
//           across the 4 lane groups complete the maximum and the sum.
//   sum     O^T[d, head] += C^T[d, key] P[key, head]  v_mfma_f32_16x16x16bf16_1k
//           The score layout is already the B layout of P. The latent part
//           of the key tile is written to LDS as it arrives and read back
//           transposed as the A operand. P enters as hi + lo (two products)
//           so that the weights keep fp32 accuracy.
typedef __attribute__((__vector_size__(8 * sizeof(short)))) short lat_bf16x8_v;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short lat_bf16x4_v;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float lat_f32x4_v;

DEV_INLINE lat_bf16x8_v lat_frag8(const uint4& v) {
  return __builtin_bit_cast(lat_bf16x8_v, v);
}
DEV_INLINE lat_bf16x4_v lat_frag4(unsigned short a, unsigned short b,
                                  unsigned short c, unsigned short d) {
  lat_bf16x4_v v;
  v[0] = (short)a; v[1] = (short)b; v[2] = (short)c; v[3] = (short)d;
  return v;
}

template <int R, int DR>
__global__ __launch_bounds__(128) void latent_attention_mfma_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ q_abs,
    const bf16_t* __restrict__ q, long ldq, const bf16_t* __restrict__ cache,
    const float* __restrict__ cs, int cs_rows, int dims,
    const int* __restrict__ positions, const int* __restrict__ row_seq,
    const int* __restrict__ block_table, int max_blocks, long rows, int H,
    int dn, int BS, int window, float scale, int HT, int NS,
    float* __restrict__ split_o, float* __restrict__ split_ml) {
  constexpr int KW = R + DR, KST = KW / 32, VST = R / 32, NDT = R / 16;
  constexpr int LDV = R + 8;               // padded LDS row, 16-byte aligned
  extern __shared__ unsigned short lat_lds[];
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int rc = lane & 15;
  const int g4 = lane >> 4;
  const long unit = (long)blockIdx.x * 2 + wave;
  if (unit >= rows * HT) return;
  const long r = unit / HT;
  const int h = (int)(unit - r * HT) * 16 + rc;
  unsigned short* vl = lat_lds + wave * 16 * LDV;
  bf16_t* orow = out + ((long)(h < H ? h : 0) * rows + r) * R + 4 * g4;
  const int p = positions[r];
  // with NS > 1 the row's key tiles are shared out over gridDim.y waves
  // whose partial sums the merge kernel folds
  float* sml = split_ml + ((r * H + (h < H ? h : 0)) * NS + blockIdx.y) * 2;
  float* so = split_o + ((r * H + (h < H ? h : 0)) * NS + blockIdx.y) * (long)R +
              4 * g4;
  if (p < 0) {
    if (h < H) {
      if (NS == 1) {
        for (int dt = 0; dt < NDT; ++dt)
          *reinterpret_cast<uint2*>(orow + dt * 16) = uint2{0u, 0u};
      } else if (g4 == 0) {
        sml[0] = -INFINITY;
        sml[1] = 0.f;
      }
    }
    return;
  }
  const int s = row_seq[r];
  // ---- query fragments: latent part, then the rotated part ----
  uint4 qf[KST];
#pragma unroll
  for (int st = 0; st < VST; ++st)
    qf[st] = h < H ? *reinterpret_cast<const uint4*>(
                         q_abs + ((long)h * rows + r) * R + st * 32 + g4 * 8)
                   : uint4{0u, 0u, 0u, 0u};
  {
    const int pp = p < cs_rows ? p : cs_rows - 1;
    const float* ang = cs + (long)pp * dims;
    const int half = dims / 2;
#pragma unroll
    for (int st = 0; st < DR / 32; ++st) {
      uint4 v = uint4{0u, 0u, 0u, 0u};
      if (h < H) {
        float f[8];
        ld8(q + r * ldq + (long)h * (dn + DR) + dn + st * 32 + g4 * 8, f);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int e0 = st * 32 + g4 * 8 + 2 * i;
          if (e0 < dims) {
            const float c = ang[e0 >> 1], sn = ang[half + (e0 >> 1)];
            const float a = f[2 * i], b = f[2 * i + 1];
            f[2 * i] = fmaf(a, c, -b * sn);
            f[2 * i + 1] = fmaf(b, c, a * sn);
          }
        }
        v = pack_bf16x8(f);
      }
      qf[VST + st] = v;
    }
  }
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int* bt = block_table + (long)s * max_blocks;
  lat_f32x4_v o[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) o[dt] = lat_f32x4_v{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const int t_first = lo >> 4, t_count = (p >> 4) - t_first + 1;
  const int tps = (t_count + NS - 1) / NS;
  const int t_begin = t_first + (int)blockIdx.y * tps;
  const int t_end = min(t_first + t_count, t_begin + tps);
  for (int j0 = t_begin * 16; j0 < t_end * 16; j0 += 16) {
    // the lane's key, kept inside the visible range for the loads
    int jc = j0 + rc;
    jc = jc < lo ? lo : (jc > p ? p : jc);
    const bf16_t* kr =
        cache + ((long)bt[jc / BS] * BS + jc % BS) * KW + g4 * 8;
    lat_f32x4_v sacc = {0.f, 0.f, 0.f, 0.f};
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int st = 0; st < KST; ++st) {
      const uint4 a = *reinterpret_cast<const uint4*>(kr + st * 32);
      sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(lat_frag8(a),
                                                     lat_frag8(qf[st]), sacc,
                                                     0, 0, 0);
      if (st < VST)
        *reinterpret_cast<uint4*>(vl + rc * LDV + st * 32 + g4 * 8) = a;
    }
    __builtin_amdgcn_wave_barrier();
    // ---- online softmax: lane = (head rc, keys j0 + 4 g4 + i) ----
    float sv[4];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int j = j0 + 4 * g4 + i;
      sv[i] = (j >= lo && j <= p) ? sacc[i] * scale : -INFINITY;
      tmax = fmaxf(tmax, sv[i]);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, WAVE));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
    const float mn = fmaxf(m, tmax);       // every tile holds a visible key
    const float alpha = (m == -INFINITY) ? 0.f : __expf(m - mn);
    m = mn;
    float psum = 0.f;
    unsigned short ph[4], pl[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float w = (sv[i] == -INFINITY) ? 0.f : __expf(sv[i] - mn);
      psum += w;
      ph[i] = f2us(w);
      pl[i] = f2us(w - us2f(ph[i]));
    }
    psum += __shfl_xor(psum, 16, WAVE);
    psum += __shfl_xor(psum, 32, WAVE);
    l = l * alpha + psum;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) o[dt] *= alpha;
    }
    const lat_bf16x4_v phi = lat_frag4(ph[0], ph[1], ph[2], ph[3]);
    const lat_bf16x4_v plo = lat_frag4(pl[0], pl[1], pl[2], pl[3]);
    const unsigned short* vp = vl + (4 * g4) * LDV + rc;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      const lat_bf16x4_v a =
          lat_frag4(vp[dt * 16], vp[dt * 16 + LDV], vp[dt * 16 + 2 * LDV],
                    vp[dt * 16 + 3 * LDV]);
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, phi, o[dt], 0, 0, 0);
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, plo, o[dt], 0, 0, 0);
    }
  }
  if (h >= H) return;
  if (NS > 1) {
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
      *reinterpret_cast<float4*>(so + dt * 16) =
          float4{o[dt][0], o[dt][1], o[dt][2], o[dt][3]};
    if (g4 == 0) {
      sml[0] = m;
      sml[1] = l;
    }
    return;
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) {
    const unsigned int w0 = (unsigned int)f2us(o[dt][0] * inv) |
                            ((unsigned int)f2us(o[dt][1] * inv) << 16);
    const unsigned int w1 = (unsigned int)f2us(o[dt][2] * inv) |
                            ((unsigned int)f2us(o[dt][3] * inv) << 16);
    *reinterpret_cast<uint2*>(orow + dt * 16) = uint2{w0, w1};
  }
}

template <int R, int DR>
static void launch_latent_mfma(torch::Tensor& out, torch::Tensor& q_abs,
                               torch::Tensor& q, torch::Tensor& cache,
                               torch::Tensor& cs, torch::Tensor& positions,
                               torch::Tensor& row_seq,
                               torch::Tensor& block_table, long rows, int H,
                               int dn, int window, float scale,
                               hipStream_t stream) {
  const int HT = (H + 15) / 16;
  const long units = rows * HT;
  const size_t lds = (size_t)2 * 16 * (R + 8) * sizeof(unsigned short);
  // few rows (a decode step): share every row's key tiles out over up to
  // 16 waves so that the device fills, and fold the parts afterwards
  int NS = 1;
  while (NS < 16 && units * NS < 1024) NS <<= 1;
  const long span_tiles = ((window > 0 ? window : cs.size(0)) + 15) / 16 + 1;
  while (NS > 1 && (long)(NS - 1) * 4 >= span_tiles) NS >>= 1;
  torch::Tensor so, sml;
  if (NS > 1) {
    so = torch::empty({rows * H * NS, (long)R},
                      q.options().dtype(torch::kFloat32));
    sml = torch::empty({rows * H * NS, 2L}, q.options().dtype(torch::kFloat32));
  }
  latent_attention_mfma_kernel<R, DR>
      <<<dim3((unsigned)((units + 1) / 2), (unsigned)NS), 128, lds, stream>>>(
          reinterpret_cast<bf16_t*>(out.data_ptr()),
          reinterpret_cast<const bf16_t*>(q_abs.data_ptr()),
          reinterpret_cast<const bf16_t*>(q.data_ptr()), (long)q.stride(0),
          reinterpret_cast<const bf16_t*>(cache.data_ptr()),
          cs.data_ptr<float>(), (int)cs.size(0), (int)cs.size(1),
          positions.data_ptr<int>(), row_seq.data_ptr<int>(),
          block_table.data_ptr<int>(), (int)block_table.size(1), rows, H, dn,
          (int)cache.size(2), window, scale, HT, NS,
          NS > 1 ? so.data_ptr<float>() : nullptr,
          NS > 1 ? sml.data_ptr<float>() : nullptr);
  if (NS > 1)
    latent_attention_merge_kernel<bf16_t>
        <<<dim3((unsigned)rows, (unsigned)H), 256, 0, stream>>>(
            reinterpret_cast<bf16_t*>(out.data_ptr()), so.data_ptr<float>(),
            sml.data_ptr<float>(), rows, H, R, NS);
}

// sizes the matrix-core form serves
bool latent_attention_mfma_supported(int64_t R, int64_t dr) {
  return (R == 128 || R == 256 || R == 512) && (dr == 32 || dr == 64);
}

// out, q_abs [H, rows, R] contiguous; q [rows, >= H*(dn+dr)] (stride(1) ==
// 1); cache [blocks, 1, BS, R+dr]; cs [positions, dims] fp32.
void latent_attention(torch::Tensor out, torch::Tensor q_abs, torch::Tensor q,
                      torch::Tensor cache, torch::Tensor cs,
                      torch::Tensor positions, torch::Tensor row_seq,
                      torch::Tensor block_table, int64_t H, int64_t dn,
                      int64_t dr, int64_t window, double scale) {
  check_act(q, "q"); check_act(q_abs, "q_abs"); check_act(out, "out");
  check_f32(cs, "cs");
  check_i32(positions, "positions"); check_i32(row_seq, "row_seq");
  check_i32(block_table, "block_table");
  TORCH_CHECK(q_abs.dim() == 3 && q_abs.is_contiguous() && out.dim() == 3 &&
              out.is_contiguous());
  const long rows = q.size(0);
  const int R = (int)q_abs.size(2);
  TORCH_CHECK(q_abs.size(0) == H && q_abs.size(1) == rows &&
              out.size(0) == H && out.size(1) == rows && out.size(2) == R);
  TORCH_CHECK(q.dim() == 2 && q.stride(1) == 1 &&
              q.size(1) >= H * (dn + dr));
  TORCH_CHECK(cache.dim() == 4 && cache.is_contiguous() && cache.size(1) == 1 &&
              cache.size(3) == R + dr);
  TORCH_CHECK(q.scalar_type() == cache.scalar_type() &&
              q_abs.scalar_type() == cache.scalar_type() &&
              out.scalar_type() == cache.scalar_type());
  TORCH_CHECK(cs.dim() == 2 && cs.size(0) >= 1 && cs.size(1) % 2 == 0 &&
              cs.size(1) <= dr);
  TORCH_CHECK(positions.numel() == rows && row_seq.numel() == rows);
  TORCH_CHECK(block_table.dim() == 2);
  TORCH_CHECK(R <= 1024, "latent_attention: latent wider than 1024");
  if (rows == 0) return;
  const size_t lds = (size_t)(LAT_HB * (R + dr) + LAT_HB * LAT_CH) * 4;
  TORCH_CHECK(lds <= 60 * 1024, "latent_attention: queries do not fit LDS");
  auto stream = c10::hip::getCurrentHIPStream().stream();
  dim3 grid((unsigned)rows, (unsigned)((H + LAT_HB - 1) / LAT_HB));
  // bf16 at the served sizes: the matrix cores, for prompt portions and
  // (with the keys of a row split over several waves) for decoded rows
  if (is_bf16(q) && latent_attention_mfma_supported(R, dr) && dn % 8 == 0 &&
      q.stride(0) % 8 == 0 && aligned16(q.data_ptr()) &&
      aligned16(cache.data_ptr()) && aligned16(q_abs.data_ptr()) &&
      aligned16(out.data_ptr())) {
#define KK_MFMA(RR, DD)                                                      \
  launch_latent_mfma<RR, DD>(out, q_abs, q, cache, cs, positions, row_seq,   \
                             block_table, rows, (int)H, (int)dn, (int)window, \
                             (float)scale, stream)
    if (R == 128 && dr == 32) KK_MFMA(128, 32);
    else if (R == 128) KK_MFMA(128, 64);
    else if (R == 256 && dr == 32) KK_MFMA(256, 32);
    else if (R == 256) KK_MFMA(256, 64);
    else if (R == 512 && dr == 32) KK_MFMA(512, 32);
    else KK_MFMA(512, 64);
#undef KK_MFMA
    HIP_CHECK_KERNEL();
    return;
  }
  // vector form: whole 16-byte chunks and a latent of 8 * 2^k entries
  const int per_row = R / 8;
  const bool vec = R % 8 == 0 && dr % 8 == 0 && per_row >= 1 &&
                   per_row <= 256 && (per_row & (per_row - 1)) == 0 &&
                   aligned16(cache.data_ptr());
  const size_t lds_vec = lds + (size_t)256 * LAT_HB * 8 * 4;
#define KK_ARGS reinterpret_cast<T*>(out.data_ptr()),                        \
        reinterpret_cast<const T*>(q_abs.data_ptr()),                        \
        reinterpret_cast<const T*>(q.data_ptr()), (long)q.stride(0),         \
        reinterpret_cast<const T*>(cache.data_ptr()), cs.data_ptr<float>(),  \
        (int)cs.size(0), (int)cs.size(1), positions.data_ptr<int>(),         \
        row_seq.data_ptr<int>(), block_table.data_ptr<int>(),                \
        (int)block_table.size(1), rows, (int)H, (int)dn, (int)dr, R,         \
        (int)cache.size(2), (int)window, (float)scale
  KK_DISPATCH_ACT(q, {
    if (vec && lds_vec <= 60 * 1024) {
      // few rows: split every row's keys over several workgroups
      const long blocks = (long)grid.x * grid.y;
      int NS = 1;
      while (NS < 8 && blocks * NS < 1024) NS <<= 1;
      const long span = window > 0 ? window : cs.size(0);
      while (NS > 1 && (long)(NS - 1) * LAT_CH >= span) NS >>= 1;
      if (NS == 1) {
        latent_attention_vec_kernel<T><<<grid, 256, lds_vec, stream>>>(
            KK_ARGS, 1, nullptr, nullptr);
      } else {
        auto so = torch::empty({rows * H * NS, (long)R},
                               q.options().dtype(torch::kFloat32));
        auto sml = torch::empty({rows * H * NS, 2L},
                                q.options().dtype(torch::kFloat32));
        latent_attention_vec_kernel<T>
            <<<dim3(grid.x, grid.y, (unsigned)NS), 256, lds_vec, stream>>>(
                KK_ARGS, NS, so.data_ptr<float>(), sml.data_ptr<float>());
        latent_attention_merge_kernel<T>
            <<<dim3((unsigned)rows, (unsigned)H), 256, 0, stream>>>(
                reinterpret_cast<T*>(out.data_ptr()), so.data_ptr<float>(),
                sml.data_ptr<float>(), rows, (int)H, R, NS);
      }
    } else if (R <= 256)
      latent_attention_kernel<T, 1><<<grid, 256, lds, stream>>>(KK_ARGS);
    else if (R <= 512)
      latent_attention_kernel<T, 2><<<grid, 256, lds, stream>>>(KK_ARGS);
    else
      latent_attention_kernel<T, 4><<<grid, 256, lds, stream>>>(KK_ARGS);
  });
#undef KK_ARGS
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
