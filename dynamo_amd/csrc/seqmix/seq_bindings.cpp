// Python bindings for the sequence-mixer kernels (dynamo_amd._hip_seq):
// recurrent mixers (matrix-state and gated linear), paged attention over
// rows (biased, windowed, multi-map, latent, sigmoid-weighted), routed
// experts and their row-wise companions. Built apart from dynamo_amd._hip so that a model which only
// needs these compiles in seconds.
#include <torch/extension.h>
#include <pybind11/pybind11.h>

using torch::Tensor;
using OptTensor = c10::optional<torch::Tensor>;

void embed_scale_pos(Tensor out, Tensor ids, Tensor positions, Tensor embed,
                     OptTensor pos, double scale);
void add_scalar_rmsnorm(Tensor out, Tensor res, OptTensor delta, Tensor g,
                        double eps);
void causal_conv_silu(Tensor out, Tensor x, Tensor w, Tensor conv_state,
                      Tensor tok_seq, Tensor seq_start, Tensor seq_len,
                      Tensor seq_slot, Tensor seq_pos0);
void causal_conv(Tensor out, Tensor x, Tensor w, OptTensor bias, bool silu,
                 Tensor conv_state, Tensor tok_seq, Tensor seq_start,
                 Tensor seq_len, Tensor seq_slot, Tensor seq_pos0);
void token_shift_mix(Tensor out, Tensor h, Tensor mu, Tensor prev_state,
                     Tensor tok_seq, Tensor seq_start, Tensor seq_len,
                     Tensor seq_slot, Tensor seq_pos0);
void head_norm_gate(Tensor out, Tensor o, Tensor w, int64_t w_stride,
                    OptTensor gate, int64_t gate_act, double eps);
void clamped_glu(Tensor out, Tensor gate_up, double limit, double alpha);
void dual_rmsnorm_mean(Tensor out, Tensor a, Tensor b, Tensor wa, Tensor wb,
                       double eps);
void softcap_(Tensor x, double cap);
void gated_delta_rule(Tensor out, Tensor qkv, Tensor proj, int64_t off_b,
                      int64_t off_a, Tensor A_log, Tensor dt_bias, Tensor state,
                      Tensor seq_start, Tensor seq_len, Tensor seq_slot,
                      Tensor seq_pos0, int64_t G, double qscale,
                      double unit_eps);
void rwkv_time_mix(Tensor out, Tensor r, Tensor k, Tensor v, Tensor wraw,
                   Tensor w0, Tensor u, Tensor state, Tensor seq_start,
                   Tensor seq_len, Tensor seq_slot, Tensor seq_pos0);
void mlstm_memory(Tensor out, Tensor proj, int64_t off_q, int64_t off_k,
                  int64_t off_v, int64_t off_i, int64_t off_f, Tensor i_bias,
                  Tensor f_bias, Tensor state_S, Tensor state_n, Tensor state_m,
                  Tensor seq_start, Tensor seq_len, Tensor seq_slot,
                  Tensor seq_pos0, double qscale, double cap, double den_eps);
void kv_append_norm(Tensor kcache, Tensor vcache, Tensor proj, int64_t off_k,
                    int64_t off_v, Tensor slot_mapping, bool vnorm, double eps);
void biased_attention(Tensor out, Tensor proj, int64_t off_q, Tensor kcache,
                      Tensor vcache, Tensor page_table, Tensor tok_seq,
                      Tensor positions, Tensor seq_len, OptTensor r1,
                      OptTensor r2, double scale, double temp_coef,
                      int64_t temp_every);
void paged_attention_rows(Tensor out, Tensor proj, int64_t off_q, Tensor kcache,
                          OptTensor vcache, Tensor page_table, Tensor tok_seq,
                          Tensor positions, Tensor seq_len, OptTensor r1,
                          OptTensor r2, double scale, double temp_coef,
                          int64_t temp_every, int64_t kmaps, int64_t window,
                          int64_t keep_first, OptTensor head_bias,
                          bool sigmoid, double softcap, OptTensor dist_bias,
                          OptTensor sink);
void residual_layernorm(OptTensor out, Tensor res, OptTensor delta,
                        OptTensor post_w, double mult, OptTensor w, double eps);
void xielu(Tensor out, Tensor x, Tensor pq);
void rope_rows(Tensor dst, int64_t dst_col, int64_t dst_vec, Tensor src,
               int64_t src_col, int64_t src_vec, Tensor positions, Tensor freqs,
               int64_t nvec, int64_t len, bool interleaved);
void latent_append(Tensor cache, Tensor z, int64_t z_col, Tensor norm_w,
                   Tensor slot_mapping, Tensor positions, Tensor freqs,
                   bool interleaved, double eps);
void diff_norm_gate(Tensor out, Tensor a, Tensor lambda, double post,
                    OptTensor gate, double eps);
void head_sigmoid_scale(Tensor out, Tensor x, Tensor gate);
void rglru_scan(Tensor out, Tensor u, Tensor gates, Tensor br, Tensor bi,
                Tensor lam, Tensor y, Tensor state, Tensor seq_start,
                Tensor seq_len, Tensor seq_slot, Tensor seq_pos0, double decay,
                int64_t max_len);
bool biased_attention_mfma_supported(int64_t dk, int64_t dv);
bool paged_attention_mfma_supported(int64_t dk, int64_t dv, bool f32out,
                                    bool extras);
void paged_attention_mfma(Tensor out, Tensor proj, int64_t off_q, Tensor kcache,
                          OptTensor vcache, Tensor page_table, Tensor tile_row0,
                          Tensor tile_rows, int64_t max_tile_rows,
                          Tensor tok_seq, Tensor positions, OptTensor r1,
                          OptTensor r2, double scale, double temp_coef,
                          int64_t temp_every, int64_t kmaps, int64_t window,
                          int64_t keep_first, OptTensor head_bias,
                          bool sigmoid, double softcap, OptTensor dist_bias,
                          OptTensor sink);
void biased_attention_mfma(Tensor out, Tensor proj, int64_t off_q,
                           Tensor kcache, Tensor vcache, Tensor page_table,
                           Tensor tile_row0, Tensor tile_rows,
                           int64_t max_tile_rows, Tensor tok_seq,
                           Tensor positions, OptTensor r1, OptTensor r2,
                           double scale, double temp_coef, int64_t temp_every);

void paged_attention_mfma_decode(Tensor out, Tensor partial, Tensor proj,
                                 int64_t off_q, Tensor kcache, OptTensor vcache,
                                 Tensor page_table, Tensor tok_seq,
                                 Tensor positions, Tensor seq_len, double scale,
                                 double temp_coef, int64_t temp_every,
                                 int64_t kmaps, int64_t window,
                                 int64_t keep_first, OptTensor head_bias,
                                 bool sigmoid, double softcap,
                                 OptTensor dist_bias, OptTensor sink);
void residual_conv(Tensor out, Tensor x, Tensor w, Tensor conv_state,
                   Tensor tok_seq, Tensor seq_start, Tensor seq_len,
                   Tensor seq_slot, Tensor seq_pos0);
bool join_conv_single(Tensor out, Tensor res, OptTensor delta, OptTensor post_w,
                      double eps, Tensor w, Tensor conv_state, Tensor tok_seq,
                      Tensor seq_len, Tensor seq_slot, Tensor seq_pos0);
void headnorm_rope_append(Tensor proj, int64_t H, int64_t G, int64_t dk,
                          int64_t dv, int64_t off_k, int64_t off_v, Tensor qw,
                          Tensor kw, OptTensor freqs, bool interleaved,
                          double eps, Tensor positions, Tensor kcache,
                          Tensor vcache, Tensor slot_mapping);
void mingru_scan(Tensor out, Tensor proj, Tensor state, Tensor seq_start,
                 Tensor seq_len, Tensor seq_slot, Tensor seq_pos0,
                 int64_t max_len);
void relu_squared(Tensor out, Tensor x);
void moe_route(Tensor idx, Tensor wgt, Tensor logits, OptTensor router,
               Tensor correction, int64_t groups, int64_t keep, double scale);
void moe_dispatch(Tensor rank, Tensor counts, Tensor idx);
void moe_gather(Tensor xg, Tensor h, Tensor idx, Tensor rank, Tensor base,
                int64_t E);
void moe_combine(Tensor out, Tensor y, Tensor h, Tensor idx, Tensor wgt,
                 Tensor rank, Tensor base, int64_t E, OptTensor shared,
                 OptTensor shared_gate);
void embed_pair_hash(Tensor out, Tensor ids, Tensor embed, Tensor table,
                     int64_t mul_prev, int64_t mul_cur, Tensor prev_state,
                     Tensor tok_seq, Tensor seq_start, Tensor seq_len,
                     Tensor seq_slot, Tensor seq_pos0);
void stream_step(OptTensor out, Tensor xs, OptTensor delta, OptTensor mix,
                 OptTensor out_w, double mult, OptTensor in_w, OptTensor norm_w,
                 double eps);
void rms_norm_cols(Tensor out, Tensor x, int64_t col, Tensor w, double eps);
void rownorm_append(Tensor proj, int64_t nq, int64_t off_k, int64_t nk,
                    int64_t off_v, int64_t nv, Tensor qw, OptTensor kw,
                    double eps, OptTensor kcache, OptTensor vcache,
                    Tensor slot_mapping);
void heads_major(Tensor out, Tensor x);
void heads_gate(Tensor out, Tensor o, Tensor gate);
void ssd_scan(Tensor out, Tensor xbc, Tensor dt_raw, Tensor dt_bias,
              Tensor A_log, Tensor D, Tensor state, Tensor seq_start,
              Tensor seq_len, Tensor seq_slot, Tensor seq_pos0, int64_t G);
void gated_group_norm(Tensor out, Tensor y, Tensor z, Tensor w, int64_t groups,
                      double eps);
void gelu_erf(Tensor out, Tensor x);
void silu_glu(Tensor out, Tensor gate_up);
void moe_route_topk(Tensor idx, Tensor wgt, Tensor logits, int64_t n,
                    OptTensor bias);

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "dynamo_amd sequence-mixer kernels (gfx950)";
  m.def("embed_scale_pos", &embed_scale_pos);
  m.def("add_scalar_rmsnorm", &add_scalar_rmsnorm);
  m.def("causal_conv_silu", &causal_conv_silu);
  m.def("causal_conv", &causal_conv);
  m.def("token_shift_mix", &token_shift_mix);
  m.def("head_norm_gate", &head_norm_gate);
  m.def("clamped_glu", &clamped_glu);
  m.def("dual_rmsnorm_mean", &dual_rmsnorm_mean);
  m.def("softcap_", &softcap_);
  m.def("gated_delta_rule", &gated_delta_rule);
  m.def("rwkv_time_mix", &rwkv_time_mix);
  m.def("mlstm_memory", &mlstm_memory);
  m.def("kv_append_norm", &kv_append_norm);
  m.def("biased_attention", &biased_attention);
  m.def("paged_attention_rows", &paged_attention_rows);
  m.def("residual_layernorm", &residual_layernorm);
  m.def("xielu", &xielu);
  m.def("rope_rows", &rope_rows);
  m.def("latent_append", &latent_append);
  m.def("diff_norm_gate", &diff_norm_gate);
  m.def("head_sigmoid_scale", &head_sigmoid_scale);
  m.def("rglru_scan", &rglru_scan);
  m.def("biased_attention_mfma_supported", &biased_attention_mfma_supported);
  m.def("biased_attention_mfma", &biased_attention_mfma);
  m.def("paged_attention_mfma_supported", &paged_attention_mfma_supported);
  m.def("paged_attention_mfma", &paged_attention_mfma);
  m.def("paged_attention_mfma_decode", &paged_attention_mfma_decode);
  m.def("residual_conv", &residual_conv);
  m.def("join_conv_single", &join_conv_single);
  m.def("headnorm_rope_append", &headnorm_rope_append);
  m.def("mingru_scan", &mingru_scan);
  m.def("relu_squared", &relu_squared);
  m.def("moe_route", &moe_route);
  m.def("moe_dispatch", &moe_dispatch);
  m.def("moe_gather", &moe_gather);
  m.def("moe_combine", &moe_combine);
  m.def("embed_pair_hash", &embed_pair_hash);
  m.def("stream_step", &stream_step);
  m.def("rms_norm_cols", &rms_norm_cols);
  m.def("rownorm_append", &rownorm_append);
  m.def("heads_major", &heads_major);
  m.def("heads_gate", &heads_gate);
  m.def("ssd_scan", &ssd_scan);
  m.def("gated_group_norm", &gated_group_norm);
  m.def("gelu_erf", &gelu_erf);
  m.def("silu_glu", &silu_glu);
  m.def("moe_route_topk", &moe_route_topk);
}
