// Short causal convolution per channel with carried taps, a bias after the
// sum and an activation:
//   out[r, c] = act(sum_j cw[j, c] * u[i - back + j, c] + bias[c])
// where u is column col0 + c of the projection for rows of this portion and
// the sequence's state slot for the back = taps-1 inputs before it; inputs
// before position 0 count as zero, so a slot's earlier content is never
// read by a new sequence. Taps are summed oldest first whatever the
// portion's length, so a position's value does not depend on how the
// prompt was cut. The slot itself is shifted afterwards by
// conv_state_update, or by this kernel when every sequence brings exactly
// one row (a decode step): then a thread owns its channels of the slot.
#include "elem.h"

namespace kukeon {

template <typename T>
__global__ __launch_bounds__(256) void conv_act_kernel(
    T* __restrict__ out, const T* __restrict__ proj, long ldp, long col0,
    const float* __restrict__ cw, const float* __restrict__ bias,
    float* __restrict__ state, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ cu_rows,
    const int* __restrict__ state_slots, int C, int taps, int act,
    int shift) {
  const long r = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int p = positions[r];
  if (p < 0) return;                          // inactive row
  const int s = row_seq[r];
  const long row0 = cu_rows[s];
  const int i = (int)(r - row0);
  const int back = taps - 1;
  float* st = state + (long)state_slots[s] * back * C;
  float acc = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int src = i - back + j;
    if (p - back + j < 0) continue;           // before the sequence start
    const float u = src >= 0 ? ldf(proj + (row0 + src) * ldp + col0 + c)
                             : st[(long)(back + src) * C + c];
    acc = fmaf(cw[(long)j * C + c], u, acc);
  }
  acc += bias[c];
  if (act == 1) acc = acc / (1.0f + __expf(-acc));
  stf(out + r * (long)C + c, acc);
  if (shift && back > 0) {
    // the sequence's only row: this thread owns its channel of the slot
    for (int k = 0; k + 1 < back; ++k)
      st[(long)k * C + c] = st[(long)(k + 1) * C + c];
    st[(long)(back - 1) * C + c] = ldf(proj + r * ldp + col0 + c);
  }
}

// Vector form: 8 consecutive channels per thread, every tap one 16-byte (bf16)
// or 32-byte (fp32) load; the same sums in the same order.
template <typename T>
__global__ __launch_bounds__(256) void conv_act_vec_kernel(
    T* __restrict__ out, const T* __restrict__ proj, long ldp, long col0,
    const float* __restrict__ cw, const float* __restrict__ bias,
    float* __restrict__ state, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ cu_rows,
    const int* __restrict__ state_slots, int C, int taps, int act,
    int shift) {
  const long r = blockIdx.x;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (c >= C) return;
  const int p = positions[r];
  if (p < 0) return;
  const int s = row_seq[r];
  const long row0 = cu_rows[s];
  const int i = (int)(r - row0);
  const int back = taps - 1;
  float* st = state + (long)state_slots[s] * back * C;
  float acc[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) acc[k] = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int src = i - back + j;
    if (p - back + j < 0) continue;
    float u[8], w[8];
    if (src >= 0) ld8(proj + (row0 + src) * ldp + col0 + c, u);
    else ld8(st + (long)(back + src) * C + c, u);
    ld8(cw + (long)j * C + c, w);
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[k] = fmaf(w[k], u[k], acc[k]);
  }
  float b[8];
  ld8(bias + c, b);
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    acc[k] += b[k];
    if (act == 1) acc[k] = acc[k] / (1.0f + __expf(-acc[k]));
  }
  st8(out + r * (long)C + c, acc);
  if (shift && back > 0) {
    float u[8];
    for (int k = 0; k + 1 < back; ++k) {
      ld8(st + (long)(k + 1) * C + c, u);
      st8(st + (long)k * C + c, u);
    }
    ld8(proj + r * ldp + col0 + c, u);
    st8(st + (long)(back - 1) * C + c, u);
  }
}

// out [rows, C] contiguous; proj [rows, ld] (stride(1) == 1) read at
// columns col0 .. col0+C-1; cw [taps, C], bias [C] fp32; state
// [slots, taps-1, C] fp32.
void conv_act(torch::Tensor out, torch::Tensor proj, int64_t col0,
              torch::Tensor cw, torch::Tensor bias, torch::Tensor state,
              torch::Tensor positions, torch::Tensor row_seq,
              torch::Tensor cu_rows, torch::Tensor state_slots, int64_t act,
              bool shift_state) {
  check_act(proj, "proj");
  check_f32(cw, "cw"); check_f32(bias, "bias"); check_f32(state, "state");
  check_i32(positions, "positions"); check_i32(row_seq, "row_seq");
  check_i32(cu_rows, "cu_rows"); check_i32(state_slots, "state_slots");
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1);
  const long rows = proj.size(0);
  TORCH_CHECK(cw.dim() == 2);
  const long taps = cw.size(0), C = cw.size(1);
  TORCH_CHECK(taps >= 1 && bias.numel() == C);
  TORCH_CHECK(state.dim() == 3 && state.size(1) == taps - 1 &&
              state.size(2) == C);
  TORCH_CHECK(col0 >= 0 && col0 + C <= proj.size(1));
  TORCH_CHECK(out.scalar_type() == proj.scalar_type() && out.is_contiguous() &&
              out.dim() == 2 && out.size(0) == rows && out.size(1) == C);
  TORCH_CHECK(positions.numel() == rows && row_seq.numel() == rows);
  const long nseq = cu_rows.numel() - 1;
  TORCH_CHECK(nseq >= 1 && state_slots.numel() >= nseq);
  if (rows == 0) return;
  TORCH_CHECK(!shift_state || rows == nseq,
              "the state is shifted in place only when every sequence brings "
              "one row");
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool vec = C % 8 == 0 && col0 % 8 == 0 && proj.stride(0) % 8 == 0 &&
                   aligned16(proj.data_ptr()) && aligned16(out.data_ptr()) &&
                   aligned16(cw.data_ptr()) && aligned16(bias.data_ptr()) &&
                   aligned16(state.data_ptr());
  if (vec) {
    const int threads = C / 8 >= 256 ? 256 : 64;
    dim3 vgrid((unsigned)rows, (unsigned)((C / 8 + threads - 1) / threads));
    KK_DISPATCH_ACT(proj, {
      conv_act_vec_kernel<T><<<vgrid, threads, 0, stream>>>(
          reinterpret_cast<T*>(out.data_ptr()),
          reinterpret_cast<const T*>(proj.data_ptr()), (long)proj.stride(0),
          (long)col0, cw.data_ptr<float>(), bias.data_ptr<float>(),
          state.data_ptr<float>(), positions.data_ptr<int>(),
          row_seq.data_ptr<int>(), cu_rows.data_ptr<int>(),
          state_slots.data_ptr<int>(), (int)C, (int)taps, (int)act,
          (int)shift_state);
    });
    HIP_CHECK_KERNEL();
    return;
  }
  dim3 grid((unsigned)rows, (unsigned)((C + 255) / 256));
  KK_DISPATCH_ACT(proj, {
    conv_act_kernel<T><<<grid, 256, 0, stream>>>(
        reinterpret_cast<T*>(out.data_ptr()),
        reinterpret_cast<const T*>(proj.data_ptr()), (long)proj.stride(0),
        (long)col0, cw.data_ptr<float>(), bias.data_ptr<float>(),
        state.data_ptr<float>(), positions.data_ptr<int>(),
        row_seq.data_ptr<int>(), cu_rows.data_ptr<int>(),
        state_slots.data_ptr<int>(), (int)C, (int)taps, (int)act,
        (int)shift_state);
  });
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
