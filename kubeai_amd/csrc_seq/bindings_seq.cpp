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
                 torch::Tensor positions, bool residual);
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
                            int64_t chunk, int64_t window, double out_scale);

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
        "chunk/window-masked paged softmax attention");
}
