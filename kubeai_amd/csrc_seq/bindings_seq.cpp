// Python bindings of the sequence-state kernels (kubeai_amd._C_seq).
#include <torch/extension.h>

void add_layernorm(torch::Tensor out, c10::optional<torch::Tensor> branch,
                   torch::Tensor residual, torch::Tensor weight,
                   torch::Tensor bias, double eps);
void gated_rmsnorm(torch::Tensor out, torch::Tensor o, torch::Tensor weight,
                   torch::Tensor gate, int64_t groups, int64_t act, double eps,
                   double out_scale);
void relu_squared(torch::Tensor out, torch::Tensor x);
void causal_conv(torch::Tensor y, torch::Tensor x, torch::Tensor w,
                 torch::Tensor tails, torch::Tensor start_loc,
                 torch::Tensor slots, torch::Tensor token_seq,
                 torch::Tensor positions, bool residual, int64_t act);
void token_shift_mix(torch::Tensor out, torch::Tensor h, torch::Tensor mu,
                     torch::Tensor prev, torch::Tensor start_loc,
                     torch::Tensor slots, torch::Tensor token_seq,
                     torch::Tensor positions);
void mingru_scan(torch::Tensor y, torch::Tensor zxg, torch::Tensor bz,
                 torch::Tensor bx, torch::Tensor state, torch::Tensor start_loc,
                 torch::Tensor slots, torch::Tensor positions, int64_t max_len);
void linear_attn_scan(torch::Tensor o, torch::Tensor q, torch::Tensor k,
                      torch::Tensor v, torch::Tensor decay,
                      c10::optional<torch::Tensor> bonus,
                      c10::optional<torch::Tensor> w_bias, torch::Tensor state,
                      torch::Tensor start_loc, torch::Tensor slots,
                      torch::Tensor positions, bool silu_inputs, int64_t max_len);
void rope_pairs_and_cache(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                          torch::Tensor positions, torch::Tensor inv_freq,
                          torch::Tensor k_cache, torch::Tensor v_cache,
                          torch::Tensor slot_mapping);
void masked_paged_attention(torch::Tensor out, torch::Tensor q,
                            torch::Tensor k_cache, torch::Tensor v_cache,
                            torch::Tensor block_tables, torch::Tensor start_loc,
                            torch::Tensor token_seq, torch::Tensor positions,
                            int64_t max_len, double scale, double softcap,
                            int64_t chunk, int64_t window, double out_scale,
                            c10::optional<torch::Tensor> sink_scores);
void qknorm_rope_half_and_cache(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                                c10::optional<torch::Tensor> q_weight,
                                c10::optional<torch::Tensor> k_weight, double eps,
                                torch::Tensor positions, torch::Tensor inv_freq,
                                torch::Tensor k_cache, torch::Tensor v_cache,
                                torch::Tensor slot_mapping);
void sandwich_rmsnorm(torch::Tensor out, c10::optional<torch::Tensor> branch,
                      c10::optional<torch::Tensor> post_weight,
                      torch::Tensor residual, torch::Tensor pre_weight, double eps);
void rmsnorm_to_cache(torch::Tensor cache, torch::Tensor x, torch::Tensor weight,
                      torch::Tensor slot_mapping, double eps);
void sigmoid_gate(torch::Tensor out, torch::Tensor x, torch::Tensor gate);
void head_linear(torch::Tensor y, torch::Tensor x, torch::Tensor w,
                 c10::optional<torch::Tensor> gate);
void router_topk(torch::Tensor logits, torch::Tensor dense, torch::Tensor weights,
                 torch::Tensor index);
void relu_squared_weighted(torch::Tensor out, torch::Tensor u, torch::Tensor w,
                           int64_t group);
void scaled_add_rmsnorm(torch::Tensor out, torch::Tensor residual,
                        c10::optional<torch::Tensor> a,
                        c10::optional<torch::Tensor> a_scale,
                        c10::optional<torch::Tensor> b,
                        c10::optional<torch::Tensor> b_scale, double mult,
                        c10::optional<torch::Tensor> extra,
                        c10::optional<torch::Tensor> extra_row, torch::Tensor weight,
                        double eps);
void rmsnorm_rows(torch::Tensor out, torch::Tensor x, torch::Tensor weight, double eps);
void gelu(torch::Tensor out, torch::Tensor x);
void tanh_cap(torch::Tensor x, double cap);
void latent_rope_to_cache(torch::Tensor cache, torch::Tensor x, torch::Tensor weight,
                          double eps, c10::optional<torch::Tensor> q_rot,
                          c10::optional<torch::Tensor> q_out, torch::Tensor positions,
                          torch::Tensor inv_freq, double rot_mult,
                          torch::Tensor slot_mapping);
void router_scores_topk(torch::Tensor logits, c10::optional<torch::Tensor> bias,
                        torch::Tensor dense, torch::Tensor weights,
                        torch::Tensor index, double scale);
void glu_weighted(torch::Tensor out, torch::Tensor gu, c10::optional<torch::Tensor> w,
                  int64_t group, double alpha, double limit, double up_shift,
                  bool w_sigmoid);
void embed_sinusoid(torch::Tensor out, torch::Tensor ids, torch::Tensor table,
                    double scale, torch::Tensor positions, torch::Tensor freqs);
void hyper_mix_rmsnorm(torch::Tensor out, torch::Tensor streams,
                       c10::optional<torch::Tensor> y, c10::optional<torch::Tensor> gate,
                       c10::optional<torch::Tensor> mix,
                       c10::optional<torch::Tensor> write_w, torch::Tensor read_w,
                       torch::Tensor weight, double eps);
void scale_q_and_cache(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                       torch::Tensor positions, double coef, int64_t every,
                       torch::Tensor k_cache, torch::Tensor v_cache,
                       torch::Tensor slot_mapping);
void diff_combine(torch::Tensor out, torch::Tensor att, double lam, double gain,
                  double eps);
void diag_rank1_scan(torch::Tensor o, torch::Tensor r, torch::Tensor k, torch::Tensor v,
                     torch::Tensor w_pre, torch::Tensor a_pre, torch::Tensor w_bias,
                     torch::Tensor a_bias, torch::Tensor state, torch::Tensor start_loc,
                     torch::Tensor slots, torch::Tensor positions, double decay_scale,
                     double key_eps, int64_t max_len);
void gated_delta_scan(torch::Tensor o, torch::Tensor q, torch::Tensor k,
                      torch::Tensor v, torch::Tensor beta_pre, torch::Tensor decay_pre,
                      torch::Tensor a_log, torch::Tensor dt_bias, torch::Tensor state,
                      torch::Tensor start_loc, torch::Tensor slots,
                      torch::Tensor positions, double norm_eps, int64_t max_len);

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("add_layernorm", &add_layernorm, "fp32 residual add + LayerNorm");
  m.def("gated_rmsnorm", &gated_rmsnorm, "grouped RMS norm * weight * gate");
  m.def("relu_squared", &relu_squared, "relu(x)^2");
  m.def("causal_conv", &causal_conv, "depthwise causal conv with carried tails");
  m.def("token_shift_mix", &token_shift_mix, "previous-token interpolation mixes");
  m.def("mingru_scan", &mingru_scan, "elementwise gated recurrence");
  m.def("linear_attn_scan", &linear_attn_scan, "matrix-state linear attention");
  m.def("rope_pairs_and_cache", &rope_pairs_and_cache,
        "interleaved-pair rotary + paged cache write");
  m.def("masked_paged_attention", &masked_paged_attention,
        "chunk/window-masked paged softmax attention, optional sink");
  m.def("qknorm_rope_half_and_cache", &qknorm_rope_half_and_cache,
        "whole-row q/k RMS norm + split-half rotary + paged cache write");
  m.def("sandwich_rmsnorm", &sandwich_rmsnorm,
        "post-norm of a branch + fp32 residual add + next pre-norm");
  m.def("rmsnorm_to_cache", &rmsnorm_to_cache, "RMS norm written into a paged cache");
  m.def("sigmoid_gate", &sigmoid_gate, "x * sigmoid(gate)");
  m.def("head_linear", &head_linear,
        "per-head linear maps with an optional sigmoid output gate");
  m.def("router_topk", &router_topk, "top-k routing with softmax over the chosen");
  m.def("relu_squared_weighted", &relu_squared_weighted,
        "relu(u)^2 times a per-row, per-group weight");
  m.def("scaled_add_rmsnorm", &scaled_add_rmsnorm,
        "fp32 residual += scaled sum of two branches (+ extras), then RMS norm");
  m.def("rmsnorm_rows", &rmsnorm_rows, "row RMS norm of a strided view");
  m.def("gelu", &gelu, "exact (erf) GELU");
  m.def("tanh_cap", &tanh_cap, "cap * tanh(x / cap), in place, fp32");
  m.def("latent_rope_to_cache", &latent_rope_to_cache,
        "latent RMS norm + rotated shared key part into a paged cache, query rotation");
  m.def("router_scores_topk", &router_scores_topk,
        "softmax scores, biased top-k choice, unnormalised score weights");
  m.def("glu_weighted", &glu_weighted,
        "clamped gate * sigmoid(alpha gate) * (up + shift) times a per-row, per-expert weight");
  m.def("embed_sinusoid", &embed_sinusoid,
        "embedding lookup + sinusoidal position vector into every residual stream");
  m.def("hyper_mix_rmsnorm", &hyper_mix_rmsnorm,
        "residual streams: gated write, stream mix, read, RMS norm");
  m.def("scale_q_and_cache", &scale_q_and_cache,
        "query temperature by position + paged cache write");
  m.def("diff_combine", &diff_combine,
        "difference of two attention maps + per-head RMS norm");
  m.def("diag_rank1_scan", &diag_rank1_scan,
        "generalized delta rule recurrence (diagonal decay + rank-one removal)");
  m.def("gated_delta_scan", &gated_delta_scan, "gated delta rule recurrence");
}
