// Python bindings for the recurrent-mixer kernel library (gfx950): matrix
// memories, state-space layers, decayed outer-product memories, short
// convolutions and capped softmax attention.  Built as its own extension
// so a process that serves such a model compiles and loads only these
// kernels; the fused add + RMS norm and the squared-ReLU activation are
// the row kernels of csrc_hybrid, compiled in here as well.
#include <torch/extension.h>

namespace igw {
void embed_pair_norm(torch::Tensor out, torch::Tensor tokens,
                     torch::Tensor positions, torch::Tensor prev_tok,
                     torch::Tensor seq_cu, torch::Tensor seq_start,
                     torch::Tensor seq_slots, torch::Tensor row_seq,
                     torch::Tensor embed, torch::Tensor pair, torch::Tensor pos,
                     torch::Tensor w, double scale, int64_t buckets,
                     int64_t mul_prev, int64_t mul_cur, double eps);
void causal_conv(torch::Tensor out, torch::Tensor x, torch::Tensor w,
                 c10::optional<torch::Tensor> bias, torch::Tensor state,
                 torch::Tensor seq_cu, torch::Tensor seq_start,
                 torch::Tensor seq_slots, torch::Tensor row_seq, bool silu);
void token_shift_mix(torch::Tensor out, torch::Tensor h, torch::Tensor mu,
                     torch::Tensor state, torch::Tensor seq_cu,
                     torch::Tensor seq_start, torch::Tensor seq_slots,
                     torch::Tensor row_seq);
void mlstm_gates(torch::Tensor out, torch::Tensor pre, double cap,
                 torch::Tensor m_state, torch::Tensor seq_cu,
                 torch::Tensor seq_start, torch::Tensor seq_slots);
void ssm_gates(torch::Tensor out, torch::Tensor dt_pre, torch::Tensor a_log);
void head_norm_gate(torch::Tensor out, torch::Tensor o, torch::Tensor gate,
                    torch::Tensor w, double eps, int64_t group,
                    int64_t gate_act, bool gate_first,
                    c10::optional<torch::Tensor> den,
                    c10::optional<torch::Tensor> floor_);
void append_paged_kv(torch::Tensor k, torch::Tensor v, torch::Tensor kcache,
                     torch::Tensor vcache, torch::Tensor slot_mapping);
void rmsnorm_pair_mean(torch::Tensor out, torch::Tensor a, torch::Tensor b,
                       torch::Tensor wa, torch::Tensor wb, double eps);
void outer_scan(torch::Tensor out, c10::optional<torch::Tensor> norm_out,
                torch::Tensor q, torch::Tensor k,
                torch::Tensor v, torch::Tensor decay,
                c10::optional<torch::Tensor> kscale,
                c10::optional<torch::Tensor> bonus,
                c10::optional<torch::Tensor> skip, torch::Tensor state,
                torch::Tensor seq_cu, torch::Tensor seq_start,
                torch::Tensor seq_slots, int64_t decay_mode, bool ones_col,
                double qscale);
void softcap_attention(torch::Tensor out, torch::Tensor q, torch::Tensor kcache,
                       torch::Tensor vcache, torch::Tensor block_table,
                       torch::Tensor row_seq, torch::Tensor positions,
                       double scale, double softcap, double temp_coef,
                       int64_t temp_every, int64_t window,
                       c10::optional<torch::Tensor> slopes, int64_t chunk,
                       c10::optional<torch::Tensor> sinks,
                       c10::optional<torch::Tensor> gate);
bool softcap_attention_mfma(torch::Tensor out, torch::Tensor q,
                            torch::Tensor kcache, torch::Tensor vcache,
                            torch::Tensor block_table, torch::Tensor seq_cu,
                            torch::Tensor seq_start, torch::Tensor tile_seq,
                            torch::Tensor tile_off, torch::Tensor dec_seq,
                            double scale, double softcap, double temp_coef,
                            int64_t temp_every, int64_t window,
                            c10::optional<torch::Tensor> slopes,
                            int64_t chunk, c10::optional<torch::Tensor> sinks,
                            c10::optional<torch::Tensor> gate);
int64_t softcap_attention_tile_rows();
void delta_scan(torch::Tensor out, torch::Tensor q, torch::Tensor k,
                torch::Tensor v, torch::Tensor decay, torch::Tensor beta,
                torch::Tensor state, torch::Tensor seq_cu,
                torch::Tensor seq_start, torch::Tensor seq_slots,
                double unit_eps, double qscale);
void decay_beta_gates(torch::Tensor out, torch::Tensor pre,
                      torch::Tensor a_log, torch::Tensor dt_bias);
void qk_norm_rope_append(torch::Tensor qout, torch::Tensor proj,
                         torch::Tensor positions, torch::Tensor slot_mapping,
                         torch::Tensor kcache, torch::Tensor vcache,
                         c10::optional<torch::Tensor> qnorm_w,
                         c10::optional<torch::Tensor> knorm_w,
                         c10::optional<torch::Tensor> inv_freq, double mag,
                         double eps, int64_t heads, int64_t kv_heads,
                         int64_t dim, int64_t vdim);
void moe_group_route(torch::Tensor weights, torch::Tensor idx,
                     torch::Tensor logits, torch::Tensor correction,
                     c10::optional<torch::Tensor> dst,
                     c10::optional<torch::Tensor> counts, int64_t capacity,
                     int64_t groups, int64_t keep);
void add_normed_rmsnorm(torch::Tensor out, torch::Tensor residual,
                        c10::optional<torch::Tensor> delta,
                        c10::optional<torch::Tensor> w_post,
                        c10::optional<torch::Tensor> w_pre, double eps);
void gelu_mul_rows(torch::Tensor out, torch::Tensor z, torch::Tensor table,
                   torch::Tensor tokens, int64_t col0);
// csrc_hybrid/parallel_ops.hip, csrc_hybrid/hybrid_ops.hip
void add_rmsnorm_pair(torch::Tensor out1, c10::optional<torch::Tensor> out2,
                      torch::Tensor residual,
                      c10::optional<torch::Tensor> delta_a,
                      c10::optional<torch::Tensor> delta_b, torch::Tensor w1,
                      c10::optional<torch::Tensor> w2, double eps);
void relu2(torch::Tensor out, torch::Tensor in);
void gated_act(torch::Tensor out, torch::Tensor in, int64_t mode, double limit,
               double alpha);
}  // namespace igw

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("embed_pair_norm", &igw::embed_pair_norm,
        "token + hashed pair + position rows, RMS norm -> fp32 residual");
  m.def("causal_conv", &igw::causal_conv,
        "short per-channel causal filter over ragged sequences");
  m.def("token_shift_mix", &igw::token_shift_mix,
        "blends of each row with the previous row of its sequence");
  m.def("mlstm_gates", &igw::mlstm_gates,
        "capped exponential gates with a running maximum");
  m.def("ssm_gates", &igw::ssm_gates, "softplus step sizes and decays");
  m.def("head_norm_gate", &igw::head_norm_gate,
        "memory read-out epilogue: normaliser, grouped RMS norm, gate");
  m.def("append_paged_kv", &igw::append_paged_kv,
        "keys and values of unequal width into paged caches");
  m.def("rmsnorm_pair_mean", &igw::rmsnorm_pair_mean,
        "average of two RMS-normed branches");
  m.def("outer_scan", &igw::outer_scan,
        "outer-product memory recurrence, state columns in registers");
  m.def("softcap_attention", &igw::softcap_attention,
        "causal paged softmax attention with a tanh score cap");
  m.def("softcap_attention_mfma", &igw::softcap_attention_mfma,
        "capped softmax attention on MFMA tiles (bf16); false = sizes do "
        "not fit, use softcap_attention");
  m.def("softcap_attention_tile_rows", &igw::softcap_attention_tile_rows,
        "query rows per MFMA tile");
  m.def("add_rmsnorm_pair", &igw::add_rmsnorm_pair,
        "fp32 residual += two deltas; one RMS statistic, two weighted outputs");
  m.def("relu2", &igw::relu2, "squared ReLU activation");
  m.def("gated_act", &igw::gated_act,
        "gated activations: silu(g)*u or the clamped (u+1) form");
  m.def("delta_scan", &igw::delta_scan,
        "gated delta-rule memory recurrence, state columns in registers");
  m.def("decay_beta_gates", &igw::decay_beta_gates,
        "softplus decay and sigmoid write strength of a delta-rule memory");
  m.def("qk_norm_rope_append", &igw::qk_norm_rope_append,
        "per-head q/k RMS norm, partial pair rotation, paged K/V append");
  m.def("moe_group_route", &igw::moe_group_route,
        "sigmoid router with a choice correction and expert groups");
  m.def("add_normed_rmsnorm", &igw::add_normed_rmsnorm,
        "fp32 residual += RMS-normed delta; RMS norm of the sum");
  m.def("gelu_mul_rows", &igw::gelu_mul_rows,
        "gelu_tanh(z) times a slice of a table row gathered by token");
}
