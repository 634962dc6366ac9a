// pybind bindings for colossalai_amd._C_serving (ragged serving kernels every ragged model uses:
// paged attention, norms, element-wise steps, router and experts; gfx950). The kernels of
// fixed-size sequence state live in colossalai_amd._C_serving_state.
#include <torch/extension.h>

namespace cai {
namespace serving {

at::Tensor token_shift(at::Tensor x, at::Tensor mu, at::Tensor prev, at::Tensor cu, at::Tensor start,
                       at::Tensor slots, at::Tensor tok_seq, at::ScalarType out_dtype);
at::Tensor relu_squared(at::Tensor x);
at::Tensor softcap(at::Tensor x, double cap);
void paged_kv_write(at::Tensor k, at::Tensor v, at::Tensor kpool, at::Tensor vpool, at::Tensor rows);
at::Tensor grouped_rms_norm(at::Tensor x, at::Tensor weight, int64_t groups, double eps,
                            c10::optional<at::Tensor> residual, at::ScalarType out_dtype);
at::Tensor head_rms_norm_gate(at::Tensor x, at::Tensor weight, double eps, c10::optional<at::Tensor> gate,
                              at::ScalarType out_dtype);
at::Tensor merge_rms_norm(at::Tensor a, at::Tensor wa, at::Tensor b, at::Tensor wb, double eps, at::Tensor out_w,
                          int64_t groups, at::Tensor residual);
at::Tensor paged_attention(at::Tensor q, at::Tensor kpool, at::Tensor vpool, at::Tensor block_tables, at::Tensor cu,
                           at::Tensor start, at::Tensor tok_seq, at::Tensor positions, double scale, int64_t window,
                           int64_t keep_first, c10::optional<at::Tensor> slopes, c10::optional<at::Tensor> gate,
                           int64_t num_tiles, double softcap, bool sink, int64_t num_tiles128);
at::Tensor paged_attention_ext(at::Tensor q, at::Tensor kpool, at::Tensor vpool, at::Tensor block_tables, at::Tensor cu,
                               at::Tensor start, at::Tensor tok_seq, at::Tensor positions, double scale, int64_t window,
                               int64_t keep_first, c10::optional<at::Tensor> slopes, c10::optional<at::Tensor> gate,
                               double softcap, bool sink, c10::optional<at::Tensor> sink_logits,
                               c10::optional<at::Tensor> dist_bias, c10::optional<at::Tensor> ksum,
                               c10::optional<at::Tensor> vsum, int64_t sum_block, bool cross, int64_t num_tiles,
                               int64_t num_tiles128);
void paged_pool_write(at::Tensor kpool, at::Tensor vpool, at::Tensor ksum, at::Tensor vsum, at::Tensor block_tables,
                      at::Tensor cu, at::Tensor start, int64_t block, int64_t most_blocks);
at::Tensor rotate_halves_unit_norm(at::Tensor x, at::Tensor positions, c10::optional<at::Tensor> freqs, double eps,
                                   at::ScalarType out_dtype);
at::Tensor lerp_rows(at::Tensor a, at::Tensor b, double lam);
at::Tensor talk_mix(at::Tensor o, at::Tensor talk, at::ScalarType out_dtype);
c10::optional<at::Tensor> add_scaled_unit_norm(at::Tensor residual, at::Tensor a, c10::optional<at::Tensor> b,
                                               double scale_a, double scale_b, double gain, double eps,
                                               c10::optional<at::ScalarType> out_dtype);
at::Tensor silu_mul(at::Tensor packed);
c10::optional<at::Tensor> add_rms_norm(at::Tensor residual, at::Tensor a, c10::optional<at::Tensor> b,
                                       c10::optional<at::Tensor> weight, double eps, at::ScalarType out_dtype);
std::vector<at::Tensor> grouped_topk_route(at::Tensor logits, c10::optional<at::Tensor> correction, int64_t top,
                                           int64_t group_count, int64_t group_keep, int64_t group_top,
                                           double renorm_eps, int64_t score_fn, bool renorm);
at::Tensor expert_ffn_gemv(at::Tensor h, at::Tensor w_up, at::Tensor w_down, at::Tensor ids, at::Tensor weights,
                           c10::optional<at::Tensor> base, c10::optional<at::Tensor> base_gate, bool gated, bool identity);
at::Tensor expert_combine(at::Tensor y, at::Tensor inv, at::Tensor weights, c10::optional<at::Tensor> base,
                          c10::optional<at::Tensor> base_gate, c10::optional<at::Tensor> ids, int64_t num_experts,
                          c10::optional<at::Tensor> identity_rows);
at::Tensor gelu_tanh_mul(at::Tensor packed);
at::Tensor gated_grouped_rms_norm(at::Tensor x, at::Tensor gate, at::Tensor weight, int64_t groups, double eps,
                                  at::ScalarType out_dtype);
c10::optional<at::Tensor> add_layer_norm(c10::optional<at::Tensor> residual, at::Tensor y,
                                         c10::optional<at::Tensor> w_out, double mult,
                                         c10::optional<at::Tensor> w_next, double eps, at::ScalarType out_dtype);
void rotate_pairs(at::Tensor x, at::Tensor positions, at::Tensor freqs, at::Tensor out);
void latent_kv_write(at::Tensor dkv, at::Tensor norm_w, double eps, at::Tensor freqs, at::Tensor positions,
                     at::Tensor pool, at::Tensor rows);
std::vector<at::Tensor> expert_sort(at::Tensor ids, int64_t num_experts);
at::Tensor expert_grouped_gemm(at::Tensor a, c10::optional<at::Tensor> a_rows, at::Tensor w, at::Tensor offsets,
                               int64_t rows, bool relu_squared);

}  // namespace serving
}  // namespace cai

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  namespace s = cai::serving;
  m.def("token_shift", &s::token_shift, "token shift over a ragged batch with a carried previous row");
  m.def("relu_squared", &s::relu_squared, "max(x, 0)^2");
  m.def("softcap", &s::softcap, "cap * tanh(x / cap), float32");
  m.def("paged_kv_write", &s::paged_kv_write, "scatter a ragged batch's keys/values into pool rows");
  m.def("grouped_rms_norm", &s::grouped_rms_norm, "grouped RMS norm, optional in-place residual add");
  m.def("head_rms_norm_gate", &s::head_rms_norm_gate, "per-head RMS norm with shared weight and sigmoid gate");
  m.def("merge_rms_norm", &s::merge_rms_norm, "average of two RMS-normed branches, group norm, residual add");
  m.def("paged_attention", &s::paged_attention, "ragged paged attention: window, kept prefix, distance bias, gate, soft cap, sink");
  m.def("paged_attention_ext", &s::paged_attention_ext,
        "split-key ragged paged attention with a learned sink, a distance table, block summaries, cross-head values");
  m.def("paged_pool_write", &s::paged_pool_write, "means of the key/value blocks a step completes, into the summary pools");
  m.def("rotate_halves_unit_norm", &s::rotate_halves_unit_norm, "rotate-half rotary on the first channels, then unit RMS per head");
  m.def("lerp_rows", &s::lerp_rows, "(1 - lam) a + lam b, float32 inside");
  m.def("talk_mix", &s::talk_mix, "talking heads: mix cross-head attention outputs with a square matrix");
  m.def("add_scaled_unit_norm", &s::add_scaled_unit_norm,
        "residual += gain * unit_rms(sa * a + sb * b) in place, optional cast of the updated rows");
  m.def("silu_mul", &s::silu_mul, "silu(gate) * up of a packed [N, 2F] tensor");
  m.def("add_rms_norm", &s::add_rms_norm, "residual += a (+ b) in place, then the RMS norm of the sum");
  m.def("grouped_topk_route", &s::grouped_topk_route,
        "sigmoid or softmax router: correction, group-limited top-k, renormalised or not");
  m.def("gelu_tanh_mul", &s::gelu_tanh_mul, "gelu_tanh(gate) * up of a packed [N, 2F] tensor");
  m.def("gated_grouped_rms_norm", &s::gated_grouped_rms_norm, "x * silu(gate), then grouped RMS norm");
  m.def("add_layer_norm", &s::add_layer_norm,
        "residual += mult * layer_norm(y) * w_out in place, then the layer norm of the sum (weight, no bias)");
  m.def("rotate_pairs", &s::rotate_pairs, "rotary positions on neighbouring pairs, strided in and out");
  m.def("latent_kv_write", &s::latent_kv_write, "latent row: RMS norm + pair rotation + scatter into pool rows");
  m.def("expert_ffn_gemv", &s::expert_ffn_gemv, "chosen experts' feed-forward of a small step, matrix-vector kernels");
  m.def("expert_sort", &s::expert_sort, "stable sort of (token, expert) pairs by expert: offsets, source tokens, inverse");
  m.def("expert_grouped_gemm", &s::expert_grouped_gemm,
        "rows sorted by expert times their expert's matrix (bfloat16, MFMA), optional row gather and relu^2");
  m.def("expert_combine", &s::expert_combine, "base + weighted sum of each token's expert outputs, float32");
}
