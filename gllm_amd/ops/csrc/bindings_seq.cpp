// Python bindings for the dtype-generic sequence-mixer kernels
// (gllm_amd._kernels_seq): fp32-residual layer norm, hyper-connection
// streams, windowed sink attention, talking-heads attention, varlen
// gated delta rule, minGRU, plus the grouped MoE GEMM and the
// activations they are served with.
#include <torch/extension.h>

void layernorm_f32(torch::Tensor out, torch::Tensor x, torch::Tensor w,
                   c10::optional<torch::Tensor> b, double eps);
void residual_layernorm(torch::Tensor x, torch::Tensor y,
                        torch::Tensor w_post,
                        c10::optional<torch::Tensor> b_post,
                        c10::optional<torch::Tensor> h,
                        c10::optional<torch::Tensor> w_pre,
                        c10::optional<torch::Tensor> b_pre, double eps,
                        c10::optional<torch::Tensor> gate);
void qk_norm_rope_store(torch::Tensor q, c10::optional<torch::Tensor> k,
                        c10::optional<torch::Tensor> v,
                        c10::optional<torch::Tensor> q_w,
                        c10::optional<torch::Tensor> k_w,
                        torch::Tensor positions, torch::Tensor slot_mapping,
                        torch::Tensor freqs, double mag, long rot_dims,
                        c10::optional<torch::Tensor> k_cache,
                        c10::optional<torch::Tensor> v_cache, long H, long G,
                        long D, long Dv, double eps, bool half_layout,
                        bool norm_last, bool do_norm,
                        c10::optional<torch::Tensor> v_freqs, bool norm_span,
                        bool v_unit, c10::optional<torch::Tensor> q_out);
void rotate_scale_rows(torch::Tensor out, torch::Tensor x,
                       torch::Tensor positions, torch::Tensor freqs,
                       long heads, long D, double sign, double scale,
                       bool half_layout);
void rms_weight_store(torch::Tensor out, torch::Tensor x, torch::Tensor w,
                      double eps, c10::optional<torch::Tensor> cache,
                      c10::optional<torch::Tensor> slot_mapping);
void hyper_streams(torch::Tensor xs, c10::optional<torch::Tensor> y,
                   c10::optional<torch::Tensor> y2,
                   c10::optional<torch::Tensor> gate,
                   c10::optional<torch::Tensor> mix,
                   c10::optional<torch::Tensor> out_w,
                   c10::optional<torch::Tensor> h,
                   c10::optional<torch::Tensor> in_w,
                   c10::optional<torch::Tensor> g, double eps);
void mingru_varlen(torch::Tensor out, torch::Tensor zx, torch::Tensor gp,
                   torch::Tensor state, torch::Tensor slots,
                   torch::Tensor has_init, torch::Tensor query_start_loc,
                   double scale, long max_query_len);
void clamp_swiglu(torch::Tensor out, torch::Tensor x, double limit,
                  double alpha);
void talking_attention(torch::Tensor out, torch::Tensor q,
                       torch::Tensor k_cache, torch::Tensor v_cache,
                       torch::Tensor block_table, torch::Tensor seq_lens,
                       torch::Tensor query_start_loc, double scale,
                       torch::Tensor talk, c10::optional<torch::Tensor> sink,
                       long max_query_len);
void xielu(torch::Tensor out, torch::Tensor x, double a_pos, double a_neg);
void relu2(torch::Tensor out, torch::Tensor x);
void window_attention(torch::Tensor out, torch::Tensor q,
                      c10::optional<torch::Tensor> gate,
                      torch::Tensor k_cache, torch::Tensor v_cache,
                      torch::Tensor block_table, torch::Tensor seq_lens,
                      torch::Tensor query_start_loc, double scale,
                      long window, long keep_first, bool sink,
                      c10::optional<torch::Tensor> sinks, double softcap);
void window_attention_mfma(torch::Tensor out, torch::Tensor q,
                           c10::optional<torch::Tensor> gate,
                           torch::Tensor k_cache, torch::Tensor v_cache,
                           torch::Tensor block_table, torch::Tensor seq_lens,
                           torch::Tensor query_start_loc, long max_query_len,
                           double scale, long window, long keep_first,
                           bool sink, c10::optional<torch::Tensor> sinks,
                           double softcap);
bool window_attention_decode(torch::Tensor out, torch::Tensor q,
                             c10::optional<torch::Tensor> gate,
                             torch::Tensor k_cache, torch::Tensor v_cache,
                             torch::Tensor block_table,
                             torch::Tensor seq_lens, double scale,
                             long window, long keep_first, bool sink,
                             c10::optional<torch::Tensor> sinks,
                             double softcap);
void causal_conv_silu(torch::Tensor out, torch::Tensor x, torch::Tensor w,
                      torch::Tensor conv_state, torch::Tensor slots,
                      torch::Tensor has_init, torch::Tensor query_start_loc,
                      bool activation, long max_query_len);
void delta_rule_varlen(torch::Tensor o, torch::Tensor q, torch::Tensor k,
                       torch::Tensor v, torch::Tensor a, torch::Tensor b,
                       torch::Tensor A_log, torch::Tensor dt_bias,
                       torch::Tensor state, torch::Tensor slots,
                       torch::Tensor has_init, torch::Tensor query_start_loc,
                       double q_scale, long max_query_len);
void rms_gate(torch::Tensor out, torch::Tensor o, torch::Tensor z,
              torch::Tensor w, long H, double eps, bool sigmoid_gate,
              double scale);
void token_shift(torch::Tensor out, torch::Tensor h, torch::Tensor mu,
                 torch::Tensor state, torch::Tensor slots,
                 torch::Tensor has_init, torch::Tensor query_start_loc,
                 long max_query_len);
void general_delta_rule(torch::Tensor o, torch::Tensor r, torch::Tensor k,
                        torch::Tensor v, torch::Tensor w_logit,
                        torch::Tensor a_logit, torch::Tensor w0,
                        double decay_scale, torch::Tensor state,
                        torch::Tensor slots, torch::Tensor has_init,
                        torch::Tensor query_start_loc, long max_query_len);
void stream_rmsnorm(torch::Tensor x, c10::optional<torch::Tensor> y,
                    c10::optional<torch::Tensor> y2,
                    c10::optional<torch::Tensor> w_post,
                    c10::optional<torch::Tensor> add,
                    c10::optional<torch::Tensor> h,
                    c10::optional<torch::Tensor> w_pre, double eps,
                    double mult, double y_scale);
void gated_act_mul(torch::Tensor out, torch::Tensor x, long act);
void tanh_rows(torch::Tensor out, torch::Tensor x);
void sigmoid_group_topk(torch::Tensor weights, torch::Tensor ids,
                        torch::Tensor logits,
                        c10::optional<torch::Tensor> correction,
                        long n_group, long keep, double scale);
// shared with the full extension (skinny_gemm.hip, moe.hip,
// elementwise.hip): what ops.linear / FusedMoE dispatch to in bf16
void skinny_gemm(torch::Tensor out, torch::Tensor x, torch::Tensor w,
                 c10::optional<torch::Tensor> bias,
                 torch::Tensor workspace, long splitk);
void silu_and_mul(torch::Tensor out, torch::Tensor x);
void moe_align(torch::Tensor topk_ids, long E_local, long expert_start,
               long block_m, torch::Tensor sorted_ids,
               torch::Tensor expert_blocks, torch::Tensor n_post_pad);
void moe_gemm(torch::Tensor C, torch::Tensor A, torch::Tensor W,
              torch::Tensor sorted_ids, torch::Tensor expert_blocks,
              torch::Tensor n_post_pad,
              c10::optional<torch::Tensor> topk_weights, long n_pairs,
              long topk, long block_m, bool scatter);
void moe_sum(torch::Tensor out, torch::Tensor pair_out, long topk);
void topk_softmax_rows(torch::Tensor weights, torch::Tensor ids,
                       torch::Tensor logits);

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("layernorm_f32", &layernorm_f32, "h = LN(x fp32) in the model dtype");
  m.def("residual_layernorm", &residual_layernorm,
        "x += LN_post(y [* sigmoid(gate)]); optionally h = LN_pre(x)");
  m.def("qk_norm_rope_store", &qk_norm_rope_store,
        "per-head q/k RMS norm + rotary (pair or half layout, either "
        "order) + paged K/V store");
  m.def("talking_attention", &talking_attention,
        "ragged paged causal attention with cross-head score mixing "
        "and a per-head sink");
  m.def("rotate_scale_rows", &rotate_scale_rows,
        "turn head-row pairs by sign * position * frequency and scale");
  m.def("rms_weight_store", &rms_weight_store,
        "weighted RMS norm of rows, optionally scattered into a paged "
        "single-head cache");
  m.def("hyper_streams", &hyper_streams,
        "multi-stream residual: write a sublayer result back / read the "
        "next sublayer's scalar-gain RMS-normed input");
  m.def("mingru_varlen", &mingru_varlen,
        "ragged minGRU recurrence with a per-slot fp32 state");
  m.def("clamp_swiglu", &clamp_swiglu,
        "min(g, limit) * sigmoid(alpha g) * (clamp(u) + 1)");
  m.def("xielu", &xielu, "xIELU activation over row-strided input");
  m.def("relu2", &relu2, "max(x, 0)^2 over row-strided input");
  m.def("window_attention", &window_attention,
        "ragged paged attention: window + kept first tokens + sink + gate");
  m.def("window_attention_mfma", &window_attention_mfma,
        "MFMA tile form (bf16, D == Dv in {64,128}) of window_attention");
  m.def("window_attention_decode", &window_attention_decode,
        "split-KV decode kernels with window + kept first + sink + gate; "
        "false = geometry not instantiated");
  m.def("causal_conv_silu", &causal_conv_silu,
        "ragged short causal conv + silu with per-slot state");
  m.def("delta_rule_varlen", &delta_rule_varlen,
        "ragged gated delta rule, fp32 state in registers");
  m.def("rms_gate", &rms_gate, "scale * o / rms(o) * w * act(z) per head");
  m.def("token_shift", &token_shift,
        "ragged token shift over the per-slot last-row state");
  m.def("general_delta_rule", &general_delta_rule,
        "ragged delta rule with per-channel decay and removal rate");
  m.def("stream_rmsnorm", &stream_rmsnorm,
        "x += mult * RMS(y) w_post (+ add); h = RMS(x) w_pre");
  m.def("gated_act_mul", &gated_act_mul, "act(x[:d]) * x[d:], silu or gelu");
  m.def("tanh_rows", &tanh_rows, "tanh over strided rows");
  m.def("sigmoid_group_topk", &sigmoid_group_topk,
        "sigmoid router with correction and group limits");
  m.def("skinny_gemm", &skinny_gemm,
        "decode-regime weight-streaming GEMM (M<=256)");
  m.def("silu_and_mul", &silu_and_mul, "silu(x[:d]) * x[d:]");
  m.def("moe_align", &moe_align, "device-side moe_align_block_size");
  m.def("moe_gemm", &moe_gemm, "grouped MFMA GEMM over sorted pairs");
  m.def("moe_sum", &moe_sum, "sum pair outputs over topk");
  m.def("topk_softmax_rows", &topk_softmax_rows,
        "top-k of router logits, softmax over the chosen");
}
