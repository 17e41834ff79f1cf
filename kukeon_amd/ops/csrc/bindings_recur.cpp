// Python bindings for the recurrent / latent kernel group: sandwich norms
// on an fp32 residual stream, short convolution with an activation and
// carried taps, selective state-space scan, gated part-wise norm, latent
// attention over a shared low-rank cache row, table-routed experts, xIELU
// and the tanh soft cap. Built as its own module so that a model needing
// only these compiles nothing else.
#include <torch/extension.h>

namespace kukeon {
void residual_add_rmsnorm(torch::Tensor x, torch::Tensor a, torch::Tensor bias,
                          torch::Tensor w, double w_offset, double eps,
                          torch::Tensor out);
void postnorm_residual_rmsnorm(torch::Tensor x, torch::Tensor y,
                               torch::Tensor post_w, torch::Tensor w,
                               double eps, torch::Tensor out);
void conv_act(torch::Tensor out, torch::Tensor proj, int64_t col0,
              torch::Tensor cw, torch::Tensor bias, torch::Tensor state,
              torch::Tensor positions, torch::Tensor row_seq,
              torch::Tensor cu_rows, torch::Tensor state_slots, int64_t act,
              bool shift_state);
void conv_state_update(torch::Tensor state, torch::Tensor proj,
                       torch::Tensor bias, torch::Tensor positions,
                       torch::Tensor cu_rows, torch::Tensor state_slots,
                       int64_t q_col, int64_t k_col, int64_t v_col, int64_t Cq,
                       int64_t Ck, int64_t Cv);
void ssm_scan(torch::Tensor y, torch::Tensor xbc, torch::Tensor dt,
              torch::Tensor dt_bias, torch::Tensor rate, torch::Tensor skip,
              torch::Tensor state, torch::Tensor positions,
              torch::Tensor cu_rows, torch::Tensor state_slots, int64_t H,
              int64_t P, int64_t N, int64_t G);
void gated_group_rmsnorm(torch::Tensor out, torch::Tensor y, torch::Tensor z,
                         torch::Tensor w, int64_t parts, double eps);
void head_gate(torch::Tensor out, torch::Tensor o, torch::Tensor gate);
void xielu(torch::Tensor out, torch::Tensor z, double ap, double aq);
void softcap_(torch::Tensor logits, double cap);
void latent_kv_append(torch::Tensor cq_out, torch::Tensor cache,
                      torch::Tensor proj, int64_t q_col, int64_t kv_col,
                      torch::Tensor wq, torch::Tensor wkv, double eps,
                      torch::Tensor cs, torch::Tensor positions,
                      torch::Tensor row_seq, torch::Tensor block_table);
void latent_attention(torch::Tensor out, torch::Tensor q_abs, torch::Tensor q,
                      torch::Tensor cache, torch::Tensor cs,
                      torch::Tensor positions, torch::Tensor row_seq,
                      torch::Tensor block_table, int64_t H, int64_t dn,
                      int64_t dr, int64_t window, double scale);
void table_moe(torch::Tensor out, torch::Tensor h, torch::Tensor ids,
               torch::Tensor table, torch::Tensor w_up, torch::Tensor w_down);
void gather_rows(torch::Tensor out, torch::Tensor in, torch::Tensor map);
void relu_square_(torch::Tensor x);
void combine_rows(torch::Tensor out, torch::Tensor in, torch::Tensor inv);
}  // namespace kukeon

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("residual_add_rmsnorm", &kukeon::residual_add_rmsnorm,
        "fp32 residual += a (+bias); out = rmsnorm(x) * (offset + w)");
  m.def("postnorm_residual_rmsnorm", &kukeon::postnorm_residual_rmsnorm,
        "x += rmsnorm(y) * post_w; out = rmsnorm(x) * w");
  m.def("conv_act", &kukeon::conv_act,
        "short causal conv with carried taps, bias and activation");
  m.def("conv_state_update", &kukeon::conv_state_update,
        "shift a portion's tail into the convolution state slots");
  m.def("ssm_scan", &kukeon::ssm_scan,
        "selective state-space scan with carried fp32 state");
  m.def("gated_group_rmsnorm", &kukeon::gated_group_rmsnorm,
        "rmsnorm by parts of y * silu(z), times w");
  m.def("head_gate", &kukeon::head_gate,
        "per-head sigmoid gate, [H,T,dv] -> [T,H*dv]");
  m.def("xielu", &kukeon::xielu, "xIELU activation");
  m.def("softcap_", &kukeon::softcap_, "cap * tanh(x / cap), in place");
  m.def("latent_kv_append", &kukeon::latent_kv_append,
        "norm the latents, rotate the shared key part, write the cache row");
  m.def("latent_attention", &kukeon::latent_attention,
        "windowed attention over the shared latent cache row");
  m.def("gather_rows", &kukeon::gather_rows, "out[r] = in[map[r]]");
  m.def("relu_square_", &kukeon::relu_square_, "x <- relu(x)^2, in place");
  m.def("combine_rows", &kukeon::combine_rows,
        "out[t] = mean over k of in[inv[t, k]]");
  m.def("table_moe", &kukeon::table_moe,
        "experts chosen by a token-id table, relu^2, equal weights");
}
