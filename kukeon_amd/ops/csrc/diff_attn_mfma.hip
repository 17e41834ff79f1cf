// Differential attention for packed prompt portions on the matrix cores
// (bf16 operands, fp32 accumulation; gfx950 v_mfma_f32_32x32x16_bf16).
//
// Workgroup = 8 waves over ONE kv head: a pair of waves (one per score
// map) serves query head (u % hpw) of the group and the 32-row query tile
// (u / hpw), u = 0..3, so the K and V tiles staged in LDS are shared by
// every wave and a wave carries one map's accumulators only. Per 32-key
// tile a wave computes, for its map,
//     S^T = K . Q^T           (keys x queries: a lane owns one query column,
//                              so the softmax statistics are lane-local
//                              plus one exchange between the half-waves)
//     O^T += V^T . P^T        (value rows x queries)
// V is staged transposed with its keys permuted so that the 8 keys a lane
// needs for the B operand are exactly the 8 softmax weights it already
// holds from S^T — no cross-lane movement between the two products.
// The softmax weights stay fp32-accurate through the bf16 matrix product:
// P = hi + lo with hi = bf16(P), lo = bf16(P - hi), two products per tile.
//
// Fragment maps (32x32x16): A lane l -> row l&31, k 8*(l>>5)+j; B lane l
// -> col l&31, k 8*(l>>5)+j; C lane l -> col l&31,
// row (r&3) + 8*(r>>2) + 4*(l>>5) for register r.
#include "elem.h"

namespace kukeon {

typedef __attribute__((__vector_size__(8 * sizeof(short)))) short frag8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float acc16_t;

struct TileArgs {
  long ldq, ldo, ldg;
  int H, G, BS, max_blocks, hpw;
  float qk_log2, lambda, eps, out_scale;
};

DEV_INLINE frag8_t frag_of(uint4 v) { return __builtin_bit_cast(frag8_t, v); }

// position of key kk (0..31) inside a transposed V row
DEV_INLINE int vt_pos(int kk) {
  const int w = kk & 15;
  return (kk & 16) + 8 * ((w >> 2) & 1) + ((w & 3) | ((w >> 3) << 2));
}

template <int DIM, int VDIM>
__global__ __launch_bounds__(512) void diff_attn_tile_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ q,
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const bf16_t* __restrict__ gate, const int* __restrict__ block_table,
    const int* __restrict__ cu_rows, const int* __restrict__ positions,
    const int* __restrict__ tile_seq, const int* __restrict__ tile_row0,
    TileArgs a) {
  constexpr int NT = 512;              // 8 waves: 4 (head, row tile) x 2 maps
  constexpr int KW = 2 * DIM;          // k row width
  constexpr int KLD = KW + 8;          // padded LDS row (bf16)
  constexpr int VLD = 40;              // 32 keys + pad
  constexpr int NC = DIM / 16;         // k-steps of the score product
  constexpr int NE = VDIM / 32;        // value row tiles
  constexpr int XR = NE > 1 ? 2 : 1;   // rounds of the map exchange
  constexpr int XE = NE / XR;          // value row tiles per round
  __shared__ __attribute__((aligned(16))) bf16_t Ks[32 * KLD];
  __shared__ __attribute__((aligned(16))) bf16_t Vt[VDIM * VLD];
  __shared__ float xch[4 * XE * 16 * 64];   // [unit][tile][register][lane]

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int unit = wave >> 1, mp = wave & 1;   // mp: which score map
  const int col = lane & 31, hh = lane >> 5;
  const int hpg = a.H / a.G;
  const int chunks = hpg / a.hpw;
  const int g = blockIdx.y / chunks;
  const int h = g * hpg + (blockIdx.y % chunks) * a.hpw + unit % a.hpw;
  const int qt = unit / a.hpw;
  const int QT = 4 / a.hpw;

  const int s = tile_seq[blockIdx.x];
  const int lr0 = tile_row0[blockIdx.x];
  const int row_base = cu_rows[s];
  const int n = cu_rows[s + 1] - row_base;
  const int p0 = positions[row_base];
  const int* bt = block_table + (long)s * a.max_blocks;

  const int wg_last = (lr0 + 32 * QT < n ? lr0 + 32 * QT : n) - 1;
  const int pmax = p0 + wg_last;                 // last key any wave sees
  const int my_lr = lr0 + 32 * qt + col;         // this lane's query row
  const bool wave_on = lr0 + 32 * qt < n;
  const int w_first = p0 + lr0 + 32 * qt;        // wave's first query pos
  const int w_lastrow = (lr0 + 32 * qt + 32 < n ? lr0 + 32 * qt + 32 : n) - 1;
  const int w_last = p0 + w_lastrow;
  const int qpos = p0 + my_lr;
  const bool row_on = wave_on && my_lr < n;

  // Q fragments of this wave's map (B operand): query `col`, 8 dims a step
  frag8_t qf[NC];
  {
    const bf16_t* qr = q + (long)(row_base + (row_on ? my_lr : 0)) * a.ldq +
                       (long)h * KW + mp * DIM;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      uint4 v = uint4{0u, 0u, 0u, 0u};
      if (row_on) v = *reinterpret_cast<const uint4*>(qr + 16 * c + 8 * hh);
      qf[c] = frag_of(v);
    }
  }
  acc16_t O[NE];
#pragma unroll
  for (int e = 0; e < NE; ++e)
#pragma unroll
    for (int r = 0; r < 16; ++r) O[e][r] = 0.f;
  float mrun = -INFINITY, lrun = 0.f;

  // The next tile's K and V rows travel global -> registers while the
  // current tile is being multiplied, registers -> LDS after it.
  constexpr int KCH = 32 * (KW / 8);            // 16-byte pieces of a K tile
  constexpr int NKC = (KCH + NT - 1) / NT;
  constexpr int VTASKS = 16 * (VDIM / 8);       // (key pair, 8 columns)
  static_assert(VTASKS <= NT, "one V task per thread");
  uint4 kreg[NKC], vreg0, vreg1;
  const uint4 zero4 = uint4{0u, 0u, 0u, 0u};
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < NKC; ++i) {
      const int c = tid + NT * i;
      kreg[i] = zero4;
      if (c < KCH) {
        const int kj = k0 + c / (KW / 8);
        if (kj <= pmax) {
          const long rowi = ((long)bt[kj / a.BS] * a.G + g) * a.BS +
                            kj % a.BS;
          kreg[i] = *reinterpret_cast<const uint4*>(
              k_cache + rowi * KW + (c % (KW / 8)) * 8);
        }
      }
    }
    vreg0 = zero4; vreg1 = zero4;
    if (tid < VTASKS) {
      const int kj = k0 + 2 * (tid % 16), eg = tid / 16;
      if (kj <= pmax) {
        const long rowi = ((long)bt[kj / a.BS] * a.G + g) * a.BS + kj % a.BS;
        vreg0 = *reinterpret_cast<const uint4*>(v_cache + rowi * VDIM +
                                                eg * 8);
      }
      if (kj + 1 <= pmax) {
        const int k1 = kj + 1;
        const long rowi = ((long)bt[k1 / a.BS] * a.G + g) * a.BS + k1 % a.BS;
        vreg1 = *reinterpret_cast<const uint4*>(v_cache + rowi * VDIM +
                                                eg * 8);
      }
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < NKC; ++i) {
      const int c = tid + NT * i;
      if (c < KCH)
        *reinterpret_cast<uint4*>(
            &Ks[(c / (KW / 8)) * KLD + (c % (KW / 8)) * 8]) = kreg[i];
    }
    if (tid < VTASKS) {
      const int kp = tid % 16, eg = tid / 16;
      const int pos = vt_pos(2 * kp);
      const unsigned int* w0 = reinterpret_cast<const unsigned int*>(&vreg0);
      const unsigned int* w1 = reinterpret_cast<const unsigned int*>(&vreg1);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const unsigned int lo = (w0[i >> 1] >> ((i & 1) * 16)) & 0xffffu;
        const unsigned int hi = (w1[i >> 1] >> ((i & 1) * 16)) & 0xffffu;
        *reinterpret_cast<unsigned int*>(&Vt[(eg * 8 + i) * VLD + pos]) =
            lo | (hi << 16);
      }
    }
  };

  const int ntiles = pmax / 32 + 1;
  fetch(0);
  for (int kt = 0; kt < ntiles; ++kt) {
    const int k0 = kt * 32;
    stash();
    __syncthreads();
    if (kt + 1 < ntiles) fetch(k0 + 32);

    if (wave_on && k0 <= w_last) {
      const bool diag = k0 + 31 > w_first;
      acc16_t sacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const frag8_t kf = frag_of(*reinterpret_cast<const uint4*>(
            &Ks[col * KLD + mp * DIM + 16 * c + 8 * hh]));
        sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[c], sacc, 0, 0,
                                                       0);
      }
      float t[16];
      float mx = -INFINITY;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        t[r] = sacc[r] * a.qk_log2;
        if (diag) {
          const int kj = k0 + (r & 3) + 8 * (r >> 2) + 4 * hh;
          if (kj > qpos) t[r] = -INFINITY;
        }
        mx = fmaxf(mx, t[r]);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
      float mn = fmaxf(mrun, mx);
      if (mn == -INFINITY) mn = 0.f;             // row with no key yet
      const float corr = exp2f(mrun - mn);
      float sum = 0.f;
      float p[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        p[r] = exp2f(t[r] - mn);
        sum += p[r];
      }
      sum += __shfl_xor(sum, 32, WAVE);
      lrun = lrun * corr + sum;
      mrun = mn;
      frag8_t ph[2], pl[2];                      // [key half]
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        unsigned int hw[4], lw[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float x0 = p[8 * t2 + 2 * i], x1 = p[8 * t2 + 2 * i + 1];
          const unsigned short h0 = f2us(x0), h1 = f2us(x1);
          hw[i] = (unsigned int)h0 | ((unsigned int)h1 << 16);
          lw[i] = (unsigned int)f2us(x0 - us2f(h0)) |
                  ((unsigned int)f2us(x1 - us2f(h1)) << 16);
        }
        ph[t2] = frag_of(uint4{hw[0], hw[1], hw[2], hw[3]});
        pl[t2] = frag_of(uint4{lw[0], lw[1], lw[2], lw[3]});
      }
      // the running maximum moves rarely after the first tiles
      if (__any(corr != 1.0f)) {
#pragma unroll
        for (int e = 0; e < NE; ++e)
#pragma unroll
          for (int r = 0; r < 16; ++r) O[e][r] *= corr;
      }
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
        for (int e = 0; e < NE; ++e) {
          const frag8_t vf = frag_of(*reinterpret_cast<const uint4*>(
              &Vt[(e * 32 + col) * VLD + 16 * t2 + 8 * hh]));
          O[e] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, ph[t2], O[e], 0,
                                                         0, 0);
          O[e] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pl[t2], O[e], 0,
                                                         0, 0);
        }
    }
    __syncthreads();
  }

  // ---- the second map's wave hands its normalised output to the first
  // through LDS (two rounds), which forms o = a1 - lambda a2 ----
  const float inv = lrun > 0.f ? 1.0f / lrun : 0.f;
  float* xu = xch + unit * (XE * 16 * 64);
#pragma unroll
  for (int rd = 0; rd < XR; ++rd) {
    if (mp == 1) {
#pragma unroll
      for (int e = 0; e < XE; ++e)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          xu[(e * 16 + r) * 64 + lane] = O[rd * XE + e][r] * inv;
    }
    __syncthreads();
    if (mp == 0) {
#pragma unroll
      for (int e = 0; e < XE; ++e)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          O[rd * XE + e][r] = O[rd * XE + e][r] * inv -
                              a.lambda * xu[(e * 16 + r) * 64 + lane];
    }
    __syncthreads();
  }
  if (mp == 1) return;
  // ---- unit norm, gate, store ----
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < NE; ++e)
#pragma unroll
    for (int r = 0; r < 16; ++r) ss += O[e][r] * O[e][r];
  ss += __shfl_xor(ss, 32, WAVE);
  if (!row_on) return;
  const float rs = 1.0f / sqrtf(ss / (float)VDIM + a.eps);
  float gs = 1.f;
  if (gate) {
    const float gl = us2f(gate[(long)(row_base + my_lr) * a.ldg + h]);
    gs = 1.0f / (1.0f + expf(-gl));
  }
  const float f = rs * a.out_scale * gs;
  bf16_t* orow = out + (long)(row_base + my_lr) * a.ldo + (long)h * VDIM;
#pragma unroll
  for (int e = 0; e < NE; ++e)
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      const int e0 = e * 32 + 8 * r4 + 4 * hh;
      uint2 w;
      w.x = cvtpk_bf16(O[e][4 * r4] * f, O[e][4 * r4 + 1] * f);
      w.y = cvtpk_bf16(O[e][4 * r4 + 2] * f, O[e][4 * r4 + 3] * f);
      *reinterpret_cast<uint2*>(orow + e0) = w;
    }
}

bool diff_attention_tiles_supported(int64_t dim, int64_t vdim) {
  return (dim == 16 && vdim == 32) || (dim == 32 && vdim == 32) ||
         (dim == 32 && vdim == 64) || (dim == 64 && vdim == 64) ||
         (dim == 64 && vdim == 128) || (dim == 128 && vdim == 128);
}

// Same arguments and result as diff_attention, for bf16 and the sizes listed above.
// tile_seq / tile_row0 [ntiles]: sequence and first local row of every
// workgroup's 32 * (4 / hpw) query rows; hpw = heads per workgroup (1, 2
// or 4, dividing H / G).
void diff_attention_tiles(torch::Tensor out, torch::Tensor q,
                          torch::Tensor k_cache, torch::Tensor v_cache,
                          torch::Tensor gate, torch::Tensor positions,
                          torch::Tensor cu_rows, torch::Tensor block_table,
                          torch::Tensor tile_seq, torch::Tensor tile_row0,
                          int64_t H, int64_t hpw, double scale, double lambda,
                          double eps, double out_scale) {
  TORCH_CHECK(is_bf16(q) && is_bf16(out) && is_bf16(k_cache) &&
              is_bf16(v_cache), "tile kernel is bf16 only");
  check_i32(positions, "positions"); check_i32(cu_rows, "cu_rows");
  check_i32(block_table, "block_table"); check_i32(tile_seq, "tile_seq");
  check_i32(tile_row0, "tile_row0");
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.is_contiguous() && v_cache.is_contiguous());
  TileArgs a{};
  a.H = (int)H; a.G = (int)k_cache.size(1); a.BS = (int)k_cache.size(2);
  const int dim = (int)(k_cache.size(3) / 2), vdim = (int)v_cache.size(3);
  TORCH_CHECK(diff_attention_tiles_supported(dim, vdim));
  TORCH_CHECK(v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == a.G &&
              v_cache.size(2) == a.BS);
  TORCH_CHECK(a.G >= 1 && a.H % a.G == 0);
  TORCH_CHECK((hpw == 1 || hpw == 2 || hpw == 4) && (a.H / a.G) % hpw == 0);
  const long rows = q.size(0);
  TORCH_CHECK(q.dim() == 2 && q.stride(1) == 1 && q.size(1) == H * 2 * dim);
  TORCH_CHECK(q.stride(0) % 8 == 0 &&
              reinterpret_cast<uintptr_t>(q.data_ptr()) % 16 == 0);
  TORCH_CHECK(out.dim() == 2 && out.stride(1) == 1 && out.size(0) == rows &&
              out.size(1) >= H * vdim && out.stride(0) % 4 == 0 &&
              reinterpret_cast<uintptr_t>(out.data_ptr()) % 8 == 0);
  TORCH_CHECK(positions.numel() == rows && block_table.dim() == 2);
  TORCH_CHECK(block_table.size(0) >= cu_rows.numel() - 1);
  TORCH_CHECK(tile_seq.numel() == tile_row0.numel());
  const bool has_gate = gate.numel() > 0;
  if (has_gate)
    TORCH_CHECK(is_bf16(gate) && gate.dim() == 2 && gate.size(0) == rows &&
                gate.size(1) >= H && gate.stride(1) == 1);
  a.ldq = q.stride(0); a.ldo = out.stride(0);
  a.ldg = has_gate ? gate.stride(0) : 0;
  a.max_blocks = (int)block_table.size(1);
  a.hpw = (int)hpw;
  a.qk_log2 = (float)(scale * 1.4426950408889634);
  a.lambda = (float)lambda; a.eps = (float)eps; a.out_scale = (float)out_scale;
  const long ntiles = tile_seq.numel();
  if (rows == 0 || ntiles == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  dim3 grid((unsigned)ntiles, (unsigned)(a.G * ((a.H / a.G) / a.hpw)));
#define KK_TILE(D, V)                                                        \
  if (dim == D && vdim == V) {                                               \
    diff_attn_tile_kernel<D, V><<<grid, 512, 0, stream>>>(                   \
        reinterpret_cast<bf16_t*>(out.data_ptr()),                           \
        reinterpret_cast<const bf16_t*>(q.data_ptr()),                       \
        reinterpret_cast<const bf16_t*>(k_cache.data_ptr()),                 \
        reinterpret_cast<const bf16_t*>(v_cache.data_ptr()),                 \
        has_gate ? reinterpret_cast<const bf16_t*>(gate.data_ptr())          \
                 : nullptr,                                                  \
        block_table.data_ptr<int>(), cu_rows.data_ptr<int>(),                \
        positions.data_ptr<int>(), tile_seq.data_ptr<int>(),                 \
        tile_row0.data_ptr<int>(), a);                                       \
  }
  KK_TILE(16, 32) KK_TILE(32, 32) KK_TILE(32, 64) KK_TILE(64, 64)
  KK_TILE(64, 128) KK_TILE(128, 128)
#undef KK_TILE
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
