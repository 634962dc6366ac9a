// pybind bindings for colossalai_amd._C_serving_state (kernels of fixed-size per-sequence state:
// matrix-state recurrences, the selective scan and the short convolution with a carried tail; gfx950). A model
// without such layers never loads, or compiles, this extension.
#include <torch/extension.h>

namespace cai {
namespace serving {

at::Tensor short_conv(at::Tensor x, at::Tensor taps, c10::optional<at::Tensor> tail, at::Tensor cu, at::Tensor start,
                      at::Tensor slots, at::Tensor tok_seq, bool silu, at::ScalarType out_dtype,
                      c10::optional<at::Tensor> bias);
at::Tensor ssd_recurrence(at::Tensor x, at::Tensor Bm, at::Tensor Cm, at::Tensor dt_raw, at::Tensor A_log,
                          at::Tensor dt_bias, at::Tensor D_skip, at::Tensor state, at::Tensor cu, at::Tensor start,
                          at::Tensor slots);
at::Tensor gated_delta_rule(at::Tensor q, at::Tensor k, at::Tensor v, at::Tensor beta_logit, at::Tensor dt,
                            at::Tensor A_log, at::Tensor dt_bias, at::Tensor state, at::Tensor cu, at::Tensor start,
                            at::Tensor slots, double unit_eps, double q_scale);
at::Tensor tied_gate_recurrence(at::Tensor q, at::Tensor f_logit, at::Tensor v, at::Tensor f_bias, at::Tensor lower,
                                at::Tensor state, at::Tensor cu, at::Tensor start, at::Tensor slots);
at::Tensor selective_scan(at::Tensor x, at::Tensor dt_raw, at::Tensor A_log, at::Tensor Bm, at::Tensor Cm,
                          at::Tensor D_skip, at::Tensor dt_bias, at::Tensor z, at::Tensor state, at::Tensor cu,
                          at::Tensor start, at::Tensor slots, at::ScalarType out_dtype,
                          c10::optional<at::Tensor> chunks, c10::optional<at::Tensor> seq_chunks);

}  // namespace serving
}  // namespace cai

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  namespace s = cai::serving;
  m.def("short_conv", &s::short_conv, "short causal depthwise convolution with carried tail and optional bias");
  m.def("ssd_recurrence", &s::ssd_recurrence, "state-space recurrence with one decay per head, carried state");
  m.def("gated_delta_rule", &s::gated_delta_rule, "gated delta rule with per-channel decay, carried state");
  m.def("selective_scan", &s::selective_scan, "diagonal recurrence with a decay per channel, place and token, carried state");
  m.def("tied_gate_recurrence", &s::tied_gate_recurrence, "HGRN2-style recurrence, carried state");
}
