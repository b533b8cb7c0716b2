// pybind bindings for the sequence-mixer kernels of the hybrid decoders
// (module polyrl_amd._hip_seq: builds on its own, so an engine that serves
// only such a model compiles nothing else).
#include <torch/extension.h>

void seq_add_rmsnorm(torch::Tensor out, torch::Tensor res, torch::Tensor y,
                     torch::Tensor weight, double eps, int64_t mode,
                     double offset, torch::Tensor weight2, double y_scale,
                     torch::Tensor extra, torch::Tensor extra_vec);
void seq_embed_compose(torch::Tensor out, torch::Tensor table,
                       torch::Tensor tokens, double scale,
                       torch::Tensor pair_table, torch::Tensor prev_tokens,
                       int64_t mul_prev, int64_t mul_cur, int64_t buckets,
                       torch::Tensor positions, torch::Tensor inv_freq);
void seq_gla_scan(torch::Tensor out, torch::Tensor q, torch::Tensor k,
                  torch::Tensor v, torch::Tensor z_lin, torch::Tensor z_bias,
                  torch::Tensor state, torch::Tensor cu_q,
                  torch::Tensor state_slot, double q_scale, double inv_tau);
void seq_causal_conv(torch::Tensor out, torch::Tensor x, torch::Tensor w,
                     torch::Tensor bias, torch::Tensor state,
                     torch::Tensor cu_q, torch::Tensor state_slot,
                     torch::Tensor seq_of_tok, bool add_input, bool act_silu);
void seq_group_rmsnorm(torch::Tensor out, torch::Tensor y,
                       torch::Tensor weight, int64_t groups, double eps,
                       torch::Tensor gate, int64_t gate_act);
void seq_rope_partial(torch::Tensor q, int64_t offset, torch::Tensor inv_freq,
                      torch::Tensor positions, double amp, bool interleaved);
void seq_gated_add_layernorm(torch::Tensor out1, torch::Tensor out2,
                             torch::Tensor res, torch::Tensor y1,
                             torch::Tensor g1, torch::Tensor y2,
                             torch::Tensor g2, torch::Tensor w1,
                             torch::Tensor w2, double eps);
void seq_sigmoid_mul_heads(torch::Tensor out, torch::Tensor x,
                           torch::Tensor gate);
void seq_rglru_scan(torch::Tensor out, torch::Tensor u, torch::Tensor gates,
                    torch::Tensor gate_bias, torch::Tensor lam,
                    torch::Tensor y_lin, torch::Tensor state,
                    torch::Tensor cu_q, torch::Tensor state_slot,
                    double decay_mult, int64_t max_rows);
void seq_latent_kv_store(torch::Tensor dkv, int64_t rank, torch::Tensor norm_w,
                         double eps, torch::Tensor positions,
                         torch::Tensor inv_freq, torch::Tensor cache,
                         torch::Tensor slot_mapping, double amp,
                         bool interleaved);
void seq_act_mul(torch::Tensor out, torch::Tensor a, torch::Tensor b,
                 int64_t mode, double p0, double p1, double p2);
void seq_gelu_mul_rows(torch::Tensor out, torch::Tensor gate,
                       torch::Tensor table, torch::Tensor tokens,
                       int64_t col0);
void seq_moe_combine(torch::Tensor res, torch::Tensor y, torch::Tensor inv,
                     double scale);
void seq_delta_rule(torch::Tensor out, torch::Tensor r, torch::Tensor k,
                    torch::Tensor v, torch::Tensor w_lin, torch::Tensor a_lin,
                    torch::Tensor w0, torch::Tensor a_bias,
                    torch::Tensor state, torch::Tensor cu_q,
                    torch::Tensor state_slot, double decay_scale,
                    double key_eps);
void seq_ssm_scan(torch::Tensor out, torch::Tensor xbc, torch::Tensor dt,
                  torch::Tensor z, torch::Tensor dt_bias, torch::Tensor a_log,
                  torch::Tensor d_skip, torch::Tensor state,
                  torch::Tensor cu_q, torch::Tensor state_slot,
                  int64_t groups);
void seq_latent_attention(torch::Tensor out, torch::Tensor q_lat,
                          torch::Tensor q_rot, torch::Tensor cache,
                          torch::Tensor page_table, torch::Tensor seq_of_tok,
                          torch::Tensor positions, int64_t window,
                          torch::Tensor sink, double scale);
void seq_moe_table_ffn(torch::Tensor y, torch::Tensor act, torch::Tensor h,
                       torch::Tensor tokens, torch::Tensor table,
                       torch::Tensor w_gu, torch::Tensor w_down);
void seq_latent_attention_mfma(torch::Tensor out, torch::Tensor q,
                               torch::Tensor cache, torch::Tensor page_table,
                               torch::Tensor seq_of_tok,
                               torch::Tensor positions, torch::Tensor tile_n0,
                               torch::Tensor tile_cnt, int64_t rank,
                               int64_t window, torch::Tensor sink,
                               double scale, int64_t mode);

void seq_gqa_prepare_store(torch::Tensor q_out, torch::Tensor q,
                           torch::Tensor k, torch::Tensor v,
                           torch::Tensor q_norm, torch::Tensor k_norm,
                           double eps, torch::Tensor inv_freq, double amp,
                           torch::Tensor positions, torch::Tensor cache,
                           torch::Tensor slot_mapping, int64_t H, int64_t G,
                           int64_t D, int64_t Dv, bool head_unit,
                           torch::Tensor v_inv_freq);
void seq_gqa_window_attention(torch::Tensor out, torch::Tensor q,
                              torch::Tensor cache, torch::Tensor page_table,
                              torch::Tensor seq_of_tok,
                              torch::Tensor positions, int64_t H, int64_t G,
                              int64_t D, int64_t Dv, int64_t window,
                              int64_t keep_first, torch::Tensor rel,
                              torch::Tensor dist_bucket, torch::Tensor gate,
                              double scale, torch::Tensor sink,
                              double q_temp_coef, int64_t q_temp_every,
                              double softcap, torch::Tensor head_bias,
                              bool sigmoid_weights, torch::Tensor v_inv_freq);
void seq_gqa_window_attention_mfma(
    torch::Tensor out, torch::Tensor q, torch::Tensor tile_n0,
    torch::Tensor tile_cnt, torch::Tensor cache, torch::Tensor page_table,
    torch::Tensor seq_of_tok, torch::Tensor positions, int64_t H, int64_t G,
    int64_t D, int64_t Dv, int64_t window, int64_t keep_first,
    torch::Tensor rel, torch::Tensor dist_bucket, torch::Tensor gate,
    double scale, torch::Tensor sink, double q_temp_coef,
    int64_t q_temp_every, double softcap, torch::Tensor head_bias,
    bool sigmoid_weights, torch::Tensor v_inv_freq);
void seq_moe_route(torch::Tensor idx, torch::Tensor w, torch::Tensor logits,
                   torch::Tensor correction, int64_t groups, int64_t keep,
                   int64_t act, int64_t group_top);
void seq_moe_routed_ffn(torch::Tensor y, torch::Tensor act, torch::Tensor h,
                        torch::Tensor idx, torch::Tensor w_up,
                        torch::Tensor w_down, bool gated);
void seq_moe_weighted_combine(torch::Tensor out, torch::Tensor ys,
                              torch::Tensor idx, torch::Tensor w,
                              torch::Tensor h, torch::Tensor shared,
                              int64_t E, double weight_eps, double scale);

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("seq_gqa_prepare_store", &seq_gqa_prepare_store,
        "whole-row q/k norm + partial rotation + K/V cache rows");
  m.def("seq_gqa_window_attention", &seq_gqa_window_attention,
        "grouped-query window attention over paged K/V rows (any dtype)");
  m.def("seq_gqa_window_attention_mfma", &seq_gqa_window_attention_mfma,
        "grouped-query window attention on the matrix cores (bf16)");
  m.def("seq_moe_route", &seq_moe_route,
        "softmax / sigmoid router with correction and group-limited top-k");
  m.def("seq_moe_routed_ffn", &seq_moe_routed_ffn,
        "router-chosen plain or gated experts for decode-sized bf16 batches");
  m.def("seq_gated_add_layernorm", &seq_gated_add_layernorm,
        "fp32 residual += gated branches, layer norm once per weight vector");
  m.def("seq_sigmoid_mul_heads", &seq_sigmoid_mul_heads,
        "rows times one sigmoid gate per head");
  m.def("seq_rglru_scan", &seq_rglru_scan,
        "real-gated linear recurrence (fp32 state, in place)");
  m.def("seq_moe_weighted_combine", &seq_moe_weighted_combine,
        "weighted sum of chosen experts, identity experts and shared");
  m.def("seq_embed_compose", &seq_embed_compose,
        "scaled embedding row + hashed pair row + sinusoid, fp32");
  m.def("seq_gla_scan", &seq_gla_scan,
        "gated linear attention scan (fp32 state, in place)");
  m.def("seq_add_rmsnorm", &seq_add_rmsnorm,
        "fp32 residual add + RMS norm / cast / unit-RMS add");
  m.def("seq_causal_conv", &seq_causal_conv,
        "stateful depthwise causal convolution over packed rows");
  m.def("seq_group_rmsnorm", &seq_group_rmsnorm,
        "grouped RMS norm with optional sigmoid / SiLU gate");
  m.def("seq_rope_partial", &seq_rope_partial,
        "RoPE (halves or interleaved pairs) on a slice of each head, in place");
  m.def("seq_latent_kv_store", &seq_latent_kv_store,
        "norm + rotate + write latent cache rows");
  m.def("seq_act_mul", &seq_act_mul, "silu*b / sigmoid*b / tanh / gelu / clamped gated unit");
  m.def("seq_gelu_mul_rows", &seq_gelu_mul_rows,
        "gelu_tanh(gate) * table rows gathered by token");
  m.def("seq_moe_combine", &seq_moe_combine,
        "residual += scale * sum of a token's expert rows");
  m.def("seq_moe_table_ffn", &seq_moe_table_ffn,
        "table-routed expert feed-forward for decode-sized bf16 batches");
  m.def("seq_latent_attention_mfma", &seq_latent_attention_mfma,
        "windowed latent attention with sink on the matrix cores (bf16)");
  m.def("seq_delta_rule", &seq_delta_rule,
        "generalised delta rule scan (fp32 state, in place)");
  m.def("seq_ssm_scan", &seq_ssm_scan,
        "selective state-space scan (fp32 state, in place)");
  m.def("seq_latent_attention", &seq_latent_attention,
        "windowed latent attention with softmax sink over paged cache");
}
