// Short causal convolution over time on projected channels, with carried
// state, fused with the projection bias, interleaved partial rotary
// positions and the paged KV append.
//
// A packed batch holds rows of several sequences. Row r belongs to sequence
// row_seq[r] and sits at absolute position positions[r]; sequence s owns
// rows cu_rows[s] .. cu_rows[s+1]-1 and the state slot state_slots[s].
//   u_t[c]  = proj[t, col(c)] + bias[c]                  (fp32)
//   y_t[c]  = sum_j cw[j, c] * u_(t - taps + 1 + j)[c]   (zeros before t=0)
// Taps that reach back before the rows of this launch are read from the
// state slot, which keeps the last taps-1 values of u in fp32 — the same
// numbers the in-launch path computes, so cutting a sequence into portions
// changes nothing. conv_state_update runs after the convolution and shifts
// the portion's tail into the slot.
//
// Channels are laid out [q | k | v]. q and k are split in maps of map_dim
// channels; the first rot_dims channels of every map are rotated as pairs
// (2i, 2i+1) by the angle table cs[pos] = [cos_0.. | sin_0..]. q goes to a
// dense buffer, k and v to the paged cache (k/v: [blocks, G, BS, kw|vw]).
#include "elem.h"

namespace kukeon {

struct ConvArgs {
  long ldp;            // row stride of proj
  long q_col, k_col, v_col;   // first column of each segment in proj
  int Cq, Ck, Cv;      // segment widths (Ck = Cv = 0: no keys/values)
  int taps;
  int map_dim, rot_dims;
  int G, BS, kw, vw;   // cache geometry (kw = k row width per head)
  int max_blocks;
  int cs_rows;         // rows of the angle table
};

template <typename T>
DEV_INLINE float conv_channel(const T* __restrict__ proj,
                              const float* __restrict__ bias,
                              const float* __restrict__ cw,
                              const float* __restrict__ state_slot,
                              const ConvArgs& a, int C, int c, long col,
                              long row0, int i, int p) {
  float acc = 0.f;
  const int back = a.taps - 1;
  for (int j = 0; j < a.taps; ++j) {
    const int src = i - back + j;
    if (p - back + j < 0) continue;          // before the sequence start
    float u;
    if (src >= 0)
      u = ldf(proj + (row0 + src) * a.ldp + col) + bias[c];
    else
      u = state_slot[(long)(back + src) * C + c];
    acc = fmaf(cw[(long)j * C + c], u, acc);
  }
  return acc;
}

template <typename T>
__global__ __launch_bounds__(256) void conv_rope_append_kernel(
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const T* __restrict__ proj, const float* __restrict__ bias,
    const float* __restrict__ cw, const float* __restrict__ state,
    const float* __restrict__ cs, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ cu_rows,
    const int* __restrict__ state_slots, const int* __restrict__ block_table,
    ConvArgs a) {
  const int r = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int C = a.Cq + a.Ck + a.Cv;
  if (c >= C) return;
  const int p = positions[r];
  if (p < 0) return;                          // inactive row
  const int s = row_seq[r];
  const long row0 = cu_rows[s];
  const int i = r - (int)row0;
  const float* st = state + (long)state_slots[s] * (a.taps - 1) * C;

  int seg, w;                                 // segment, index inside it
  long col;
  if (c < a.Cq) { seg = 0; w = c; col = a.q_col + w; }
  else if (c < a.Cq + a.Ck) { seg = 1; w = c - a.Cq; col = a.k_col + w; }
  else { seg = 2; w = c - a.Cq - a.Ck; col = a.v_col + w; }

  float y = conv_channel<T>(proj, bias, cw, st, a, C, c, col, row0, i, p);
  if (seg < 2) {
    const int m = w % a.map_dim;
    if (m < a.rot_dims) {
      const int d = (m & 1) ? -1 : 1;         // partner channel
      const float yp = conv_channel<T>(proj, bias, cw, st, a, C, c + d,
                                       col + d, row0, i, p);
      const int pp = p < a.cs_rows ? p : a.cs_rows - 1;
      const float* ang = cs + (long)pp * a.rot_dims;
      const float co = ang[m >> 1];
      const float si = ang[(a.rot_dims >> 1) + (m >> 1)];
      y = (m & 1) ? fmaf(yp, si, y * co) : fmaf(-yp, si, y * co);
    }
  }
  if (seg == 0) {
    stf(q_out + (long)r * a.Cq + w, y);
    return;
  }
  const int blk = block_table[(long)s * a.max_blocks + p / a.BS];
  const int off = p % a.BS;
  if (seg == 1) {
    const int g = w / a.kw, e = w % a.kw;
    stf(k_cache + (((long)blk * a.G + g) * a.BS + off) * a.kw + e, y);
  } else {
    const int g = w / a.vw, e = w % a.vw;
    stf(v_cache + (((long)blk * a.G + g) * a.BS + off) * a.vw + e, y);
  }
}

// Vector form: a thread owns 8 consecutive channels of one row (16-byte
// loads and stores); a workgroup covers 32 channel groups x 8 consecutive
// rows, so the taps that reach back into neighbouring rows hit in cache.
// Needs every segment width, column offset, map_dim and cache row width to
// be a multiple of 8.
template <typename T>
__global__ __launch_bounds__(256) void conv_rope_append_vec_kernel(
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const T* __restrict__ proj, const float* __restrict__ bias,
    const float* __restrict__ cw, const float* __restrict__ state,
    const float* __restrict__ cs, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ cu_rows,
    const int* __restrict__ state_slots, const int* __restrict__ block_table,
    ConvArgs a, int rows, int shift_state) {
  const int C = a.Cq + a.Ck + a.Cv;
  const int cv = blockIdx.y * 32 + (threadIdx.x & 31);
  const int r = blockIdx.x * 8 + (threadIdx.x >> 5);
  const int c = cv * 8;
  if (c >= C || r >= rows) return;
  const int p = positions[r];
  if (p < 0) return;
  const int s = row_seq[r];
  const long row0 = cu_rows[s];
  const int i = r - (int)row0;
  const int back = a.taps - 1;
  const float* st = state + (long)state_slots[s] * back * C;
  int seg, w;
  long col;
  if (c < a.Cq) { seg = 0; w = c; col = a.q_col + w; }
  else if (c < a.Cq + a.Ck) { seg = 1; w = c - a.Cq; col = a.k_col + w; }
  else { seg = 2; w = c - a.Cq - a.Ck; col = a.v_col + w; }
  float b8[8], y[8];
  ld8(bias + c, b8);
#pragma unroll
  for (int k = 0; k < 8; ++k) y[k] = 0.f;
  for (int j = 0; j < a.taps; ++j) {
    const int src = i - back + j;
    if (p - back + j < 0) continue;
    float u[8], wj[8];
    if (src >= 0) {
      ld8(proj + (row0 + src) * a.ldp + col, u);
#pragma unroll
      for (int k = 0; k < 8; ++k) u[k] += b8[k];
      if (shift_state && j == back) {
        // every sequence brings one row: this thread alone owns the
        // slot's 8 channels, so it shifts them here (all reads of the
        // slot were made in earlier iterations of this loop)
        float* sw = const_cast<float*>(st);
        for (int t = 0; t + 1 < back; ++t) {
          float m[8];
          ld8(sw + (long)(t + 1) * C + c, m);
          st8(sw + (long)t * C + c, m);
        }
        if (back > 0) st8(sw + (long)(back - 1) * C + c, u);
      }
    } else {
      ld8(st + (long)(back + src) * C + c, u);
    }
    ld8(cw + (long)j * C + c, wj);
#pragma unroll
    for (int k = 0; k < 8; ++k) y[k] = fmaf(wj[k], u[k], y[k]);
  }
  if (seg < 2) {
    const int m0 = w % a.map_dim;               // multiple of 8
    if (m0 < a.rot_dims) {
      const int pp = p < a.cs_rows ? p : a.cs_rows - 1;
      const float* ang = cs + (long)pp * a.rot_dims;
#pragma unroll
      for (int k = 0; k < 8; k += 2) {
        if (m0 + k < a.rot_dims) {
          const float co = ang[(m0 + k) >> 1];
          const float si = ang[(a.rot_dims >> 1) + ((m0 + k) >> 1)];
          const float ya = y[k], yb = y[k + 1];
          y[k] = fmaf(-yb, si, ya * co);
          y[k + 1] = fmaf(ya, si, yb * co);
        }
      }
    }
  }
  if (seg == 0) {
    st8(q_out + (long)r * a.Cq + w, y);
    return;
  }
  const int blk = block_table[(long)s * a.max_blocks + p / a.BS];
  const int off = p % a.BS;
  if (seg == 1) {
    const int g = w / a.kw, e = w % a.kw;
    st8(k_cache + (((long)blk * a.G + g) * a.BS + off) * a.kw + e, y);
  } else {
    const int g = w / a.vw, e = w % a.vw;
    st8(v_cache + (((long)blk * a.G + g) * a.BS + off) * a.vw + e, y);
  }
}

// Sliding form for long portions: a thread walks RB consecutive rows of its
// 8 channels and keeps the last TAPS-1 inputs in registers, so every input
// row is loaded once instead of TAPS times. The window is rebuilt from the
// rows before (or the state slot) whenever a row starts another sequence.
template <typename T, int TAPS, int RB>
__global__ __launch_bounds__(256) void conv_rope_append_slide_kernel(
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const T* __restrict__ proj, const float* __restrict__ bias,
    const float* __restrict__ cw, const float* __restrict__ state,
    const float* __restrict__ cs, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ cu_rows,
    const int* __restrict__ state_slots, const int* __restrict__ block_table,
    ConvArgs a, int rows) {
  constexpr int BACK = TAPS - 1;
  const int C = a.Cq + a.Ck + a.Cv;
  const int cv = blockIdx.y * 64 + (threadIdx.x & 63);
  const int rb = (blockIdx.x * 4 + (threadIdx.x >> 6)) * RB;
  const int c = cv * 8;
  if (c >= C || rb >= rows) return;
  int seg, w;
  long col;
  if (c < a.Cq) { seg = 0; w = c; col = a.q_col + w; }
  else if (c < a.Cq + a.Ck) { seg = 1; w = c - a.Cq; col = a.k_col + w; }
  else { seg = 2; w = c - a.Cq - a.Ck; col = a.v_col + w; }
  float b8[8], wt[TAPS][8], win[BACK > 0 ? BACK : 1][8];
  ld8(bias + c, b8);
#pragma unroll
  for (int j = 0; j < TAPS; ++j) ld8(cw + (long)j * C + c, wt[j]);
  const int m0 = seg < 2 ? w % a.map_dim : a.rot_dims;   // multiple of 8
  // indices and inputs of all RB rows are requested before any is used
  int pr[RB], sq[RB], bk[RB];
  Raw8<T> raw[RB];
#pragma unroll
  for (int rr = 0; rr < RB; ++rr) {
    const int r = rb + rr < rows ? rb + rr : rows - 1;
    pr[rr] = rb + rr < rows ? positions[r] : -1;
    sq[rr] = row_seq[r];
    raw[rr].load(proj + (long)r * a.ldp + col);
  }
#pragma unroll
  for (int rr = 0; rr < RB; ++rr) {
    bk[rr] = 0;
    if (seg > 0 && pr[rr] >= 0)
      bk[rr] = block_table[(long)sq[rr] * a.max_blocks + pr[rr] / a.BS];
  }
  int prev_s = -1;
#pragma unroll
  for (int rr = 0; rr < RB; ++rr) {
    const int r = rb + rr;
    const int p = pr[rr];
    if (p < 0) { prev_s = -1; continue; }
    const int s = sq[rr];
    const long row0 = cu_rows[s];
    const int i = r - (int)row0;
    if (s != prev_s) {                       // (re)build the window
      const float* st = state + (long)state_slots[s] * BACK * C;
#pragma unroll
      for (int j = 0; j < BACK; ++j) {
        const int src = i - BACK + j;
        if (p - BACK + j < 0) {
#pragma unroll
          for (int k = 0; k < 8; ++k) win[j][k] = 0.f;
        } else if (src >= 0) {
          ld8(proj + (row0 + src) * a.ldp + col, win[j]);
#pragma unroll
          for (int k = 0; k < 8; ++k) win[j][k] += b8[k];
        } else {
          ld8(st + (long)(BACK + src) * C + c, win[j]);
        }
      }
      prev_s = s;
    }
    float u[8], y[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) { u[k] = raw[rr].get(k) + b8[k]; y[k] = 0.f; }
    // same order of accumulation as the other forms: oldest tap first
#pragma unroll
    for (int j = 0; j < BACK; ++j)
#pragma unroll
      for (int k = 0; k < 8; ++k) y[k] = fmaf(wt[j][k], win[j][k], y[k]);
#pragma unroll
    for (int k = 0; k < 8; ++k) y[k] = fmaf(wt[BACK][k], u[k], y[k]);
#pragma unroll
    for (int j = 0; j + 1 < BACK; ++j)
#pragma unroll
      for (int k = 0; k < 8; ++k) win[j][k] = win[j + 1][k];
    if (BACK > 0) {
#pragma unroll
      for (int k = 0; k < 8; ++k) win[BACK - 1][k] = u[k];
    }
    if (m0 < a.rot_dims) {
      const int pp = p < a.cs_rows ? p : a.cs_rows - 1;
      const float* ang = cs + (long)pp * a.rot_dims;
#pragma unroll
      for (int k = 0; k < 8; k += 2) {
        if (m0 + k < a.rot_dims) {
          const float co = ang[(m0 + k) >> 1];
          const float si = ang[(a.rot_dims >> 1) + ((m0 + k) >> 1)];
          const float ya = y[k], yb = y[k + 1];
          y[k] = fmaf(-yb, si, ya * co);
          y[k + 1] = fmaf(ya, si, yb * co);
        }
      }
    }
    if (seg == 0) {
      st8(q_out + (long)r * a.Cq + w, y);
    } else {
      const int blk = bk[rr];
      const int off = p % a.BS;
      if (seg == 1) {
        const int g = w / a.kw, e = w % a.kw;
        st8(k_cache + (((long)blk * a.G + g) * a.BS + off) * a.kw + e, y);
      } else {
        const int g = w / a.vw, e = w % a.vw;
        st8(v_cache + (((long)blk * a.G + g) * a.BS + off) * a.vw + e, y);
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void conv_state_update_kernel(
    float* __restrict__ state, const T* __restrict__ proj,
    const float* __restrict__ bias, const int* __restrict__ positions,
    const int* __restrict__ cu_rows, const int* __restrict__ state_slots,
    ConvArgs a) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int C = a.Cq + a.Ck + a.Cv;
  if (c >= C) return;
  const long row0 = cu_rows[s];
  const int n = cu_rows[s + 1] - (int)row0;
  if (n <= 0 || positions[row0] < 0) return;
  long col;
  if (c < a.Cq) col = a.q_col + c;
  else if (c < a.Cq + a.Ck) col = a.k_col + (c - a.Cq);
  else col = a.v_col + (c - a.Cq - a.Ck);
  const int back = a.taps - 1;
  float* st = state + (long)state_slots[s] * back * C;
  // ascending k reads slot entries k+n > k, not yet overwritten
  for (int k = 0; k < back; ++k) {
    const int src = n - back + k;
    float v;
    if (src >= 0) v = ldf(proj + (row0 + src) * a.ldp + col) + bias[c];
    else v = st[(long)(k + n) * C + c];
    st[(long)k * C + c] = v;
  }
}

static ConvArgs make_args(const torch::Tensor& proj, int64_t q_col,
                          int64_t k_col, int64_t v_col, int64_t Cq, int64_t Ck,
                          int64_t Cv, int64_t taps, int64_t map_dim,
                          int64_t rot_dims) {
  ConvArgs a{};
  a.ldp = proj.stride(0);
  a.q_col = q_col; a.k_col = k_col; a.v_col = v_col;
  a.Cq = (int)Cq; a.Ck = (int)Ck; a.Cv = (int)Cv;
  a.taps = (int)taps; a.map_dim = (int)map_dim; a.rot_dims = (int)rot_dims;
  a.G = 1; a.BS = 1; a.kw = 1; a.vw = 1; a.max_blocks = 0; a.cs_rows = 1;
  return a;
}

// Returns true when the kernel also shifted the state slots (one row per
// sequence, vector form) so that no conv_state_update launch is needed.
// proj [rows, ld] (stride(1)==1); bias [C], cw [taps, C], state
// [slots, taps-1, C] fp32 with C = Cq+Ck+Cv; cs [P, rot_dims] fp32;
// q_out [rows, Cq]; k_cache [NB, G, BS, kw], v_cache [NB, G, BS, vw] (empty
// tensors when Ck == 0).
bool conv_rope_append(torch::Tensor q_out, torch::Tensor k_cache,
                      torch::Tensor v_cache, torch::Tensor proj,
                      torch::Tensor bias, torch::Tensor cw,
                      torch::Tensor state, torch::Tensor cs,
                      torch::Tensor positions, torch::Tensor row_seq,
                      torch::Tensor cu_rows, torch::Tensor state_slots,
                      torch::Tensor block_table, int64_t q_col, int64_t k_col,
                      int64_t v_col, int64_t Cq, int64_t Ck, int64_t Cv,
                      int64_t map_dim, int64_t rot_dims,
                      bool one_row_per_seq) {
  check_act(proj, "proj");
  check_f32(bias, "bias"); check_f32(cw, "cw"); check_f32(state, "state");
  check_f32(cs, "cs");
  check_i32(positions, "positions"); check_i32(row_seq, "row_seq");
  check_i32(cu_rows, "cu_rows"); check_i32(state_slots, "state_slots");
  check_i32(block_table, "block_table");
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1);
  const long rows = proj.size(0);
  const long C = Cq + Ck + Cv;
  TORCH_CHECK(cw.dim() == 2 && cw.size(1) == C && bias.numel() == C);
  const long taps = cw.size(0);
  TORCH_CHECK(taps >= 1 && state.dim() == 3 && state.size(1) == taps - 1 &&
              state.size(2) == C);
  TORCH_CHECK(q_col >= 0 && q_col + Cq <= proj.size(1));
  TORCH_CHECK(positions.numel() == rows && row_seq.numel() == rows);
  const long nseq = cu_rows.numel() - 1;
  TORCH_CHECK(nseq >= 1 && state_slots.numel() >= nseq);
  TORCH_CHECK(q_out.scalar_type() == proj.scalar_type() &&
              q_out.is_contiguous() && q_out.size(0) == rows &&
              q_out.size(1) == Cq);
  TORCH_CHECK(rot_dims % 2 == 0 && rot_dims <= map_dim && map_dim >= 1);
  TORCH_CHECK(Cq % map_dim == 0 && Ck % map_dim == 0);
  TORCH_CHECK(cs.dim() == 2 && cs.size(1) == rot_dims && cs.size(0) >= 1);
  ConvArgs a = make_args(proj, q_col, k_col, v_col, Cq, Ck, Cv, taps, map_dim,
                         rot_dims);
  a.cs_rows = (int)cs.size(0);
  if (Ck > 0 || Cv > 0) {
    TORCH_CHECK(k_cache.scalar_type() == proj.scalar_type() &&
                v_cache.scalar_type() == proj.scalar_type());
    TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 &&
                k_cache.is_contiguous() && v_cache.is_contiguous());
    a.G = (int)k_cache.size(1); a.BS = (int)k_cache.size(2);
    a.kw = (int)k_cache.size(3); a.vw = (int)v_cache.size(3);
    TORCH_CHECK(v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == a.G &&
                v_cache.size(2) == a.BS);
    TORCH_CHECK((long)a.G * a.kw == Ck && (long)a.G * a.vw == Cv);
    TORCH_CHECK(k_col >= 0 && k_col + Ck <= proj.size(1) && v_col >= 0 &&
                v_col + Cv <= proj.size(1));
    TORCH_CHECK(block_table.dim() == 2 && block_table.size(0) >= nseq);
    a.max_blocks = (int)block_table.size(1);
  }
  if (rows == 0) return false;
  TORCH_CHECK(!one_row_per_seq || rows == nseq);
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool kv = Ck > 0 || Cv > 0;
  const bool vec =
      Cq % 8 == 0 && Ck % 8 == 0 && Cv % 8 == 0 && q_col % 8 == 0 &&
      (!kv || (k_col % 8 == 0 && v_col % 8 == 0 && a.kw % 8 == 0 &&
               a.vw % 8 == 0 && aligned16(k_cache.data_ptr()) &&
               aligned16(v_cache.data_ptr()))) &&
      map_dim % 8 == 0 && proj.stride(0) % 8 == 0 &&
      aligned16(proj.data_ptr()) && aligned16(q_out.data_ptr()) &&
      aligned16(bias.data_ptr()) && aligned16(cw.data_ptr()) &&
      aligned16(state.data_ptr());
  if (vec && rows >= 2048 && taps >= 2 && taps <= 4) {
    constexpr int RB = 8;
    dim3 sgrid((unsigned)((rows + 4 * RB - 1) / (4 * RB)),
               (unsigned)((C / 8 + 63) / 64));
#define KK_SLIDE(TP)                                                         \
  KK_DISPATCH_ACT(proj, {                                                    \
    conv_rope_append_slide_kernel<T, TP, RB><<<sgrid, 256, 0, stream>>>(     \
        reinterpret_cast<T*>(q_out.data_ptr()),                              \
        Ck ? reinterpret_cast<T*>(k_cache.data_ptr()) : nullptr,             \
        Cv ? reinterpret_cast<T*>(v_cache.data_ptr()) : nullptr,             \
        reinterpret_cast<const T*>(proj.data_ptr()), bias.data_ptr<float>(), \
        cw.data_ptr<float>(), state.data_ptr<float>(), cs.data_ptr<float>(), \
        positions.data_ptr<int>(), row_seq.data_ptr<int>(),                  \
        cu_rows.data_ptr<int>(), state_slots.data_ptr<int>(),                \
        block_table.data_ptr<int>(), a, (int)rows);                          \
  })
    if (taps == 2) KK_SLIDE(2);
    else if (taps == 3) KK_SLIDE(3);
    else KK_SLIDE(4);
#undef KK_SLIDE
    HIP_CHECK_KERNEL();
    return false;
  }
  if (vec) {
    dim3 vgrid((unsigned)((rows + 7) / 8), (unsigned)((C / 8 + 31) / 32));
    KK_DISPATCH_ACT(proj, {
      conv_rope_append_vec_kernel<T><<<vgrid, 256, 0, stream>>>(
          reinterpret_cast<T*>(q_out.data_ptr()),
          Ck ? reinterpret_cast<T*>(k_cache.data_ptr()) : nullptr,
          Cv ? reinterpret_cast<T*>(v_cache.data_ptr()) : nullptr,
          reinterpret_cast<const T*>(proj.data_ptr()), bias.data_ptr<float>(),
          cw.data_ptr<float>(), state.data_ptr<float>(), cs.data_ptr<float>(),
          positions.data_ptr<int>(), row_seq.data_ptr<int>(),
          cu_rows.data_ptr<int>(), state_slots.data_ptr<int>(),
          block_table.data_ptr<int>(), a, (int)rows,
          one_row_per_seq ? 1 : 0);
    });
    HIP_CHECK_KERNEL();
    return one_row_per_seq;
  }
  dim3 grid((unsigned)rows, (unsigned)((C + 255) / 256));
  KK_DISPATCH_ACT(proj, {
    conv_rope_append_kernel<T><<<grid, 256, 0, stream>>>(
        reinterpret_cast<T*>(q_out.data_ptr()),
        Ck ? reinterpret_cast<T*>(k_cache.data_ptr()) : nullptr,
        Cv ? reinterpret_cast<T*>(v_cache.data_ptr()) : nullptr,
        reinterpret_cast<const T*>(proj.data_ptr()), bias.data_ptr<float>(),
        cw.data_ptr<float>(), state.data_ptr<float>(), cs.data_ptr<float>(),
        positions.data_ptr<int>(), row_seq.data_ptr<int>(),
        cu_rows.data_ptr<int>(), state_slots.data_ptr<int>(),
        block_table.data_ptr<int>(), a);
  });
  HIP_CHECK_KERNEL();
  return false;
}

void conv_state_update(torch::Tensor state, torch::Tensor proj,
                       torch::Tensor bias, torch::Tensor positions,
                       torch::Tensor cu_rows, torch::Tensor state_slots,
                       int64_t q_col, int64_t k_col, int64_t v_col, int64_t Cq,
                       int64_t Ck, int64_t Cv) {
  check_act(proj, "proj");
  check_f32(bias, "bias"); check_f32(state, "state");
  check_i32(positions, "positions"); check_i32(cu_rows, "cu_rows");
  check_i32(state_slots, "state_slots");
  const long C = Cq + Ck + Cv;
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1);
  TORCH_CHECK(state.dim() == 3 && state.size(2) == C && bias.numel() == C);
  const long nseq = cu_rows.numel() - 1;
  TORCH_CHECK(nseq >= 1 && state_slots.numel() >= nseq);
  TORCH_CHECK(positions.numel() == proj.size(0));
  const long taps = state.size(1) + 1;
  if (taps <= 1 || proj.size(0) == 0) return;
  ConvArgs a = make_args(proj, q_col, k_col, v_col, Cq, Ck, Cv, taps, 1, 0);
  auto stream = c10::hip::getCurrentHIPStream().stream();
  dim3 grid((unsigned)nseq, (unsigned)((C + 255) / 256));
  KK_DISPATCH_ACT(proj, {
    conv_state_update_kernel<T><<<grid, 256, 0, stream>>>(
        state.data_ptr<float>(), reinterpret_cast<const T*>(proj.data_ptr()),
        bias.data_ptr<float>(), positions.data_ptr<int>(),
        cu_rows.data_ptr<int>(), state_slots.data_ptr<int>(), a);
  });
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
