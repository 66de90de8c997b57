// Python bindings of the sequence-mixing kernel library (gfx950).
#include <torch/extension.h>
#include <vector>

std::vector<torch::Tensor> offset_rmsnorm(torch::Tensor x, torch::Tensor w,
                                          double eps, bool out_bf16, double offset,
                                          int64_t groups);
void gated_residual_add(torch::Tensor x, torch::Tensor mix,
                        c10::optional<torch::Tensor> ff, torch::Tensor gates,
                        torch::Tensor gate_b, double mult);
std::vector<torch::Tensor> gated_residual_norm(
    torch::Tensor x, torch::Tensor mix, c10::optional<torch::Tensor> ff,
    torch::Tensor gates, torch::Tensor gate_b, double mult, torch::Tensor next_w,
    double eps, bool out_bf16);
torch::Tensor causal_tap_conv(torch::Tensor h, torch::Tensor w, torch::Tensor tails,
                              torch::Tensor cu, torch::Tensor tok_seq,
                              torch::Tensor slots, bool out_bf16);
torch::Tensor latent_prepare(torch::Tensor q, c10::optional<torch::Tensor> dkv, int64_t heads,
                             int64_t dim, int64_t rot_dim, int64_t kv_rank,
                             c10::optional<torch::Tensor> norm_w, double eps,
                             torch::Tensor positions, double rope_base,
                             int64_t rope_dims, torch::Tensor page_slot,
                             torch::Tensor cache, c10::optional<torch::Tensor> freqs,
                             double mag, bool pairs);
torch::Tensor latent_window_attention(torch::Tensor q_lat, torch::Tensor q_rot,
                                      torch::Tensor cache, int64_t kv_rank,
                                      torch::Tensor block_tables, int64_t block_size,
                                      torch::Tensor tok_seq, torch::Tensor positions,
                                      int64_t window, double scale,
                                      c10::optional<torch::Tensor> tiles,
                                      int64_t max_tile_queries,
                                      c10::optional<torch::Tensor> sink,
                                      c10::optional<torch::Tensor> gate);
torch::Tensor mingru_scan(torch::Tensor zxg, torch::Tensor bias, torch::Tensor state,
                          torch::Tensor cu, torch::Tensor slots,
                          c10::optional<torch::Tensor> chunks,
                          c10::optional<torch::Tensor> chunk_cu);
std::vector<torch::Tensor> moe_route(torch::Tensor h, torch::Tensor router_w,
                                     torch::Tensor router_b, int64_t top);
torch::Tensor moe_experts(torch::Tensor h, torch::Tensor idx, torch::Tensor wts,
                          torch::Tensor exp_gu, torch::Tensor exp_down);

std::vector<torch::Tensor> moe_route_all(torch::Tensor h, torch::Tensor router_w,
                                         c10::optional<torch::Tensor> correction,
                                         int64_t top, double scale);
torch::Tensor moe_experts_glu(torch::Tensor h, torch::Tensor idx, torch::Tensor wts,
                              torch::Tensor exp_gu, torch::Tensor exp_down, double limit);
torch::Tensor tap_conv_silu(torch::Tensor x, torch::Tensor w, torch::Tensor tails,
                            torch::Tensor cu, torch::Tensor tok_seq, torch::Tensor slots,
                            bool out_bf16);
c10::optional<torch::Tensor> sandwich_residual_norm(
    torch::Tensor x, torch::Tensor y, c10::optional<torch::Tensor> y2,
    c10::optional<torch::Tensor> post_w, c10::optional<torch::Tensor> next_w, double eps,
    bool out_bf16, double offset, double y_scale, double y2_scale, bool cast_next,
    int64_t groups);
torch::Tensor gelu_tanh(torch::Tensor x);
std::vector<torch::Tensor> moe_route_sigmoid(torch::Tensor h, torch::Tensor router_w, int64_t top);
torch::Tensor moe_experts_scaled_input(torch::Tensor h, torch::Tensor idx, torch::Tensor wts,
                                       torch::Tensor exp_gu, torch::Tensor exp_down);
torch::Tensor qk_prepare_kv_write(torch::Tensor proj, int64_t heads, int64_t kv_heads, int64_t dim,
                                  int64_t vdim, c10::optional<torch::Tensor> q_norm_w,
                                  c10::optional<torch::Tensor> k_norm_w, double eps,
                                  torch::Tensor positions, c10::optional<torch::Tensor> freqs,
                                  double mag, c10::optional<torch::Tensor> mix,
                                  torch::Tensor page_slot, torch::Tensor cache);
torch::Tensor window_attention(torch::Tensor q, torch::Tensor cache, int64_t heads,
                               int64_t kv_heads, int64_t dim, int64_t vdim, bool whole_key,
                               torch::Tensor block_tables, int64_t block_size,
                               torch::Tensor tok_seq, torch::Tensor positions, double scale,
                               int64_t window, int64_t keep_first,
                               c10::optional<torch::Tensor> r1, c10::optional<torch::Tensor> r2,
                               c10::optional<torch::Tensor> gate,
                               c10::optional<torch::Tensor> tiles, int64_t max_tile_queries);
torch::Tensor capped_glu(torch::Tensor gu, double limit);
torch::Tensor silu_glu(torch::Tensor gu);
torch::Tensor qk_norm_kv_write(torch::Tensor proj, int64_t heads, int64_t kv_heads, int64_t dim,
                               int64_t vdim, torch::Tensor q_norm_w, torch::Tensor k_norm_w,
                               double eps, torch::Tensor page_slot, torch::Tensor cache);
torch::Tensor sigmoid_attention(torch::Tensor q, torch::Tensor cache, int64_t heads,
                                int64_t kv_heads, int64_t dim, int64_t vdim,
                                torch::Tensor block_tables, int64_t block_size,
                                torch::Tensor tok_seq, torch::Tensor positions, double scale,
                                int64_t window, int64_t keep_first, torch::Tensor slopes,
                                torch::Tensor pos_bias, c10::optional<torch::Tensor> tiles,
                                int64_t max_tile_queries);
torch::Tensor rope_kv_write(torch::Tensor proj, int64_t heads, int64_t kv_heads, int64_t dim,
                            int64_t vdim, torch::Tensor positions, double rope_base,
                            int64_t rope_dims, torch::Tensor page_slot, torch::Tensor cache,
                            c10::optional<torch::Tensor> vmix,
                            c10::optional<torch::Tensor> v_first);
torch::Tensor sink_attention(torch::Tensor q, torch::Tensor cache, int64_t heads,
                             int64_t kv_heads, int64_t dim, int64_t vdim,
                             torch::Tensor block_tables, int64_t block_size,
                             torch::Tensor tok_seq, torch::Tensor positions, double scale,
                             double softcap, c10::optional<torch::Tensor> sink,
                             c10::optional<torch::Tensor> talk,
                             c10::optional<torch::Tensor> tiles, int64_t max_tile_queries);
torch::Tensor gated_delta_rule(torch::Tensor qkv, torch::Tensor gate,
                               c10::optional<torch::Tensor> ab,
                               c10::optional<torch::Tensor> h,
                               c10::optional<torch::Tensor> ab_w, torch::Tensor a_log, torch::Tensor dt_bias, torch::Tensor onorm_w,
                               double eps, torch::Tensor state, torch::Tensor cu,
                               torch::Tensor slots, int64_t heads, int64_t kv_heads,
                               int64_t dim, int64_t vdim,
                               c10::optional<torch::Tensor> decay_up, bool gate_sigmoid);

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("offset_rmsnorm", &offset_rmsnorm, "offset-weight RMS norm -> (fp32, dtype)");
  m.def("gated_residual_add", &gated_residual_add, "gated parallel-residual update");
  m.def("gated_residual_norm", &gated_residual_norm,
        "gated residual update fused with the next offset RMS norm");
  m.def("causal_tap_conv", &causal_tap_conv, "short causal depthwise conv with slot tails");
  m.def("latent_prepare", &latent_prepare, "latent cache write + query rotation");
  m.def("latent_window_attention", &latent_window_attention,
        "windowed paged attention in latent space");
  m.def("mingru_scan", &mingru_scan, "minGRU scan with per-slot fp32 state");
  m.def("moe_route", &moe_route, "fp32 top-k router");
  m.def("moe_experts", &moe_experts, "grouped-GEMM mixture of SiLU-gated experts");
  m.def("moe_route_all", &moe_route_all, "fp32 router: softmax over all, corrected choice");
  m.def("moe_experts_glu", &moe_experts_glu,
        "grouped-GEMM mixture of clamped-GLU experts with identity experts");
  m.def("tap_conv_silu", &tap_conv_silu, "short causal conv + SiLU with slot tails");
  m.def("sandwich_residual_norm", &sandwich_residual_norm,
        "closing norm + residual sum + next opening norm");
  m.def("capped_glu", &capped_glu, "clamped GLU activation");
  m.def("silu_glu", &silu_glu, "SiLU-gated GLU activation");
  m.def("qk_norm_kv_write", &qk_norm_kv_write, "per-head RMS norm of q/k, K/V cache write");
  m.def("sigmoid_attention", &sigmoid_attention,
        "paged GQA with sigmoid weights, distance penalty, window with kept first tokens");
  m.def("rope_kv_write", &rope_kv_write, "pair rotary on q/k, value blend, K/V cache write");
  m.def("sink_attention", &sink_attention,
        "paged GQA with capped scores, sinks and head mixing");
  m.def("gated_delta_rule", &gated_delta_rule, "gated delta rule with per-slot fp32 state");
  m.def("gelu_tanh", &gelu_tanh, "tanh-form GELU activation");
  m.def("moe_route_sigmoid", &moe_route_sigmoid, "fp32 router: sigmoid scores, top-k, no renormalisation");
  m.def("moe_experts_scaled_input", &moe_experts_scaled_input,
        "grouped-GEMM mixture of SiLU-gated experts whose input carries the routing weight");
  m.def("qk_prepare_kv_write", &qk_prepare_kv_write,
        "q/k norm, half rotary, score-mixing fold of the queries, K/V cache write");
  m.def("window_attention", &window_attention,
        "paged GQA softmax attention: window with kept first tokens, log distance bias, output gate");
}
