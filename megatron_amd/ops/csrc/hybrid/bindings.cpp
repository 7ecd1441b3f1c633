// Python bindings of the hybrid serving kernels: plain fp32 residual with
// grouped RMS norm, attention over a sliding window plus pooled blocks,
// generalized delta rule, routed clamped-GLU experts.
#include <torch/extension.h>
#include <vector>

torch::Tensor embed_plain(torch::Tensor tokens, torch::Tensor embed);
std::vector<torch::Tensor> residual_group_norm(torch::Tensor x, torch::Tensor y, torch::Tensor wa, torch::Tensor wb,
                                               int64_t groups, double eps, bool out_bf16);
std::vector<torch::Tensor> moe_route(torch::Tensor logits, int64_t E, int64_t top, int64_t groups, int64_t keep,
                                     double scale);
std::vector<torch::Tensor> moe_router(torch::Tensor h, torch::Tensor wr, torch::Tensor bias, int64_t E, int64_t top,
                                      int64_t groups, int64_t keep, double scale, int64_t score);
torch::Tensor clamped_glu(torch::Tensor gu, double limit, double alpha, int64_t kind);
torch::Tensor moe_combine(torch::Tensor down, torch::Tensor inv, torch::Tensor wts, torch::Tensor shared,
                          torch::Tensor gate, torch::Tensor add);
torch::Tensor expert_pairs(torch::Tensor h, torch::Tensor ids, torch::Tensor wgu, torch::Tensor wd, double limit,
                           double alpha, int64_t kind);
torch::Tensor qk_norm_store(torch::Tensor proj, int64_t q_off, int64_t qw, int64_t k_off, int64_t kw, int64_t v_off,
                            int64_t vw, torch::Tensor wq, torch::Tensor wk, double eps, torch::Tensor pool,
                            torch::Tensor tok_row);
void pool_blocks(torch::Tensor pool, torch::Tensor pooled, int64_t P, int64_t rpp, torch::Tensor cu,
                 torch::Tensor start_pos, torch::Tensor tables, int64_t bs, int64_t max_new);
void pooled_window_attention(torch::Tensor q, torch::Tensor pool, torch::Tensor pooled, int64_t H, int64_t G,
                             int64_t D, int64_t V, double scale, int64_t window, int64_t P, int64_t rpp,
                             torch::Tensor tok_req, torch::Tensor tok_pos, torch::Tensor tables, int64_t bs,
                             torch::Tensor out, int64_t out_col, double out_scale);
void pooled_window_attention_mfma(torch::Tensor q, torch::Tensor pool, torch::Tensor pooled, int64_t H, int64_t G,
                                  int64_t D, int64_t V, double scale, int64_t window, int64_t P, int64_t rpp,
                                  torch::Tensor tiles, torch::Tensor cu, torch::Tensor start_pos,
                                  torch::Tensor tables, int64_t bs, int64_t nsplit, torch::Tensor out,
                                  int64_t out_col, double out_scale);
void delta_rule_scan(torch::Tensor proj, int64_t r_off, int64_t k_off, int64_t v_off, int64_t g_off, int64_t a_off,
                     int64_t w_off, int64_t rank, torch::Tensor w2, torch::Tensor w0, torch::Tensor a_b,
                     torch::Tensor norm_w, int64_t H, int64_t D, double eps, torch::Tensor state, torch::Tensor cu,
                     torch::Tensor slots, torch::Tensor out, int64_t out_col, double out_scale);

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("embed_plain", &embed_plain);
  m.def("residual_group_norm", &residual_group_norm);
  m.def("moe_route", &moe_route);
  m.def("moe_router", &moe_router);
  m.def("clamped_glu", &clamped_glu);
  m.def("moe_combine", &moe_combine);
  m.def("expert_pairs", &expert_pairs);
  m.def("qk_norm_store", &qk_norm_store);
  m.def("pool_blocks", &pool_blocks);
  m.def("pooled_window_attention", &pooled_window_attention);
  m.def("pooled_window_attention_mfma", &pooled_window_attention_mfma);
  m.def("delta_rule_scan", &delta_rule_scan);
}
