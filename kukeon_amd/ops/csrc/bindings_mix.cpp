// Python bindings for the sequence-mixer kernel group (fp32 residual norm,
// clamped gated activation, short convolution + rotary + KV append,
// differential attention). Built as its own module so a model that needs
// only these does not wait for the rest of the kernel library.
#include <torch/extension.h>

namespace kukeon {
void residual_add_rmsnorm(torch::Tensor x, torch::Tensor a, torch::Tensor bias,
                          torch::Tensor w, double w_offset, double eps,
                          torch::Tensor out);
void clamp_glu(torch::Tensor out, torch::Tensor gate, torch::Tensor up,
               torch::Tensor bg, torch::Tensor bu, double limit, double alpha,
               double up_shift);
bool conv_rope_append(torch::Tensor q_out, torch::Tensor k_cache,
                      torch::Tensor v_cache, torch::Tensor proj,
                      torch::Tensor bias, torch::Tensor cw,
                      torch::Tensor state, torch::Tensor cs,
                      torch::Tensor positions, torch::Tensor row_seq,
                      torch::Tensor cu_rows, torch::Tensor state_slots,
                      torch::Tensor block_table, int64_t q_col, int64_t k_col,
                      int64_t v_col, int64_t Cq, int64_t Ck, int64_t Cv,
                      int64_t map_dim, int64_t rot_dims,
                      bool one_row_per_seq);
void conv_state_update(torch::Tensor state, torch::Tensor proj,
                       torch::Tensor bias, torch::Tensor positions,
                       torch::Tensor cu_rows, torch::Tensor state_slots,
                       int64_t q_col, int64_t k_col, int64_t v_col, int64_t Cq,
                       int64_t Ck, int64_t Cv);
void diff_attention(torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
                    torch::Tensor v_cache, torch::Tensor gate,
                    torch::Tensor positions, torch::Tensor row_seq,
                    torch::Tensor block_table, int64_t H, double scale,
                    double lambda, double eps, double out_scale);
bool diff_attention_tiles_supported(int64_t dim, int64_t vdim);
void diff_attention_tiles(torch::Tensor out, torch::Tensor q,
                          torch::Tensor k_cache, torch::Tensor v_cache,
                          torch::Tensor gate, torch::Tensor positions,
                          torch::Tensor cu_rows, torch::Tensor block_table,
                          torch::Tensor tile_seq, torch::Tensor tile_row0,
                          int64_t H, int64_t hpw, double scale, double lambda,
                          double eps, double out_scale);
bool diff_attention_decode_supported(int64_t H, int64_t G, int64_t dim,
                                     int64_t vdim, bool bf16);
int64_t diff_attention_decode_capacity(int64_t H, int64_t G, int64_t dim,
                                       bool bf16);
int64_t diff_attention_decode_units_per_row(int64_t H, int64_t G);
void diff_attention_decode(torch::Tensor out, torch::Tensor q,
                           torch::Tensor k_cache, torch::Tensor v_cache,
                           torch::Tensor gate, torch::Tensor positions,
                           torch::Tensor row_seq, torch::Tensor block_table,
                           torch::Tensor part_o, torch::Tensor part_ml,
                           int64_t H, double scale, double lambda, double eps,
                           double out_scale);
}  // namespace kukeon

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("residual_add_rmsnorm", &kukeon::residual_add_rmsnorm,
        "fp32 residual += a (+bias); out = rmsnorm(x) * (offset + w)");
  m.def("clamp_glu", &kukeon::clamp_glu,
        "clamped gate * sigmoid(alpha gate) * (up + shift)");
  m.def("conv_rope_append", &kukeon::conv_rope_append,
        "bias + short causal conv (carried state) + rotary + paged KV append");
  m.def("conv_state_update", &kukeon::conv_state_update,
        "shift a portion's tail into the convolution state slots");
  m.def("diff_attention", &kukeon::diff_attention,
        "paged differential attention with unit norm and output gate");
  m.def("diff_attention_tiles_supported",
        &kukeon::diff_attention_tiles_supported);
  m.def("diff_attention_tiles", &kukeon::diff_attention_tiles,
        "differential attention for prompt portions on the matrix cores");
  m.def("diff_attention_decode_supported",
        &kukeon::diff_attention_decode_supported);
  m.def("diff_attention_decode_capacity",
        &kukeon::diff_attention_decode_capacity);
  m.def("diff_attention_decode_units_per_row",
        &kukeon::diff_attention_decode_units_per_row);
  m.def("diff_attention_decode", &kukeon::diff_attention_decode,
        "split-KV differential attention for decoded rows");
}
