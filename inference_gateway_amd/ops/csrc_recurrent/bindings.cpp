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
                       int64_t temp_every, int64_t window);
bool softcap_attention_mfma(torch::Tensor out, torch::Tensor q,
                            torch::Tensor kcache, torch::Tensor vcache,
                            torch::Tensor block_table, torch::Tensor seq_cu,
                            torch::Tensor seq_start, torch::Tensor tile_seq,
                            torch::Tensor tile_off, torch::Tensor dec_seq,
                            double scale, double softcap, double temp_coef,
                            int64_t temp_every, int64_t window);
int64_t softcap_attention_tile_rows();
// csrc_hybrid/parallel_ops.hip, csrc_hybrid/hybrid_ops.hip
void add_rmsnorm_pair(torch::Tensor out1, c10::optional<torch::Tensor> out2,
                      torch::Tensor residual,
                      c10::optional<torch::Tensor> delta_a,
                      c10::optional<torch::Tensor> delta_b, torch::Tensor w1,
                      c10::optional<torch::Tensor> w2, double eps);
void relu2(torch::Tensor out, torch::Tensor in);
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
}
