// Python bindings of the serving kernels of layers with norms on both sides of a sublayer:
// sandwich norm + residual add, restart of a repeated block, rotation (pairs / halves) with unit
// norm and cache store, attention with one or two softmax maps a head (capped scores), gated and
// differential finish, squared ReLU; and of the kernels this extension shares with the others
// through their sources (embedding into a plain residual, grouped norm, router, GLU, experts).
#include <torch/extension.h>
#include <vector>

torch::Tensor sandwich_norm_add(torch::Tensor x, torch::Tensor y, torch::Tensor w_post, torch::Tensor w_pre,
                                double eps, bool out_bf16, torch::Tensor copy_to);
std::vector<torch::Tensor> restart_norm(torch::Tensor y, torch::Tensor bias, torch::Tensor w_pre, double eps,
                                        bool out_bf16);
torch::Tensor gate_finish(torch::Tensor A, torch::Tensor gate, bool out_bf16);
torch::Tensor differential_finish(torch::Tensor A, torch::Tensor gate, torch::Tensor lam, double diff, double eps,
                                  int64_t H, int64_t V, bool out_bf16);
torch::Tensor relu2(torch::Tensor z);
torch::Tensor rope_norm_store(torch::Tensor proj, int64_t QH, int64_t KH, int64_t D, int64_t VW, torch::Tensor freqs,
                              int64_t layout, bool unit, double eps, torch::Tensor pool, torch::Tensor tok_pos,
                              torch::Tensor tok_row);
torch::Tensor map_attention(torch::Tensor q, torch::Tensor pool, int64_t H, int64_t G, int64_t M, int64_t D, int64_t V,
                            double scale, double cap, torch::Tensor tok_req, torch::Tensor tok_pos,
                            torch::Tensor tables, int64_t bs);
torch::Tensor map_attention_mfma(torch::Tensor q, torch::Tensor gate, torch::Tensor pool, int64_t H, int64_t G,
                                 int64_t M, int64_t D, int64_t V, double scale, double cap, torch::Tensor tiles,
                                 torch::Tensor cu, torch::Tensor start_pos, torch::Tensor tables, int64_t bs,
                                 int64_t nsplit, int64_t tile_rows);
// hybrid/rows.hip, hybrid/experts.hip
torch::Tensor embed_plain(torch::Tensor tokens, torch::Tensor embed);
std::vector<torch::Tensor> residual_group_norm(torch::Tensor x, torch::Tensor y, torch::Tensor wa, torch::Tensor wb,
                                               int64_t groups, double eps, bool out_bf16);
std::vector<torch::Tensor> moe_router(torch::Tensor h, torch::Tensor wr, torch::Tensor bias, int64_t E, int64_t top,
                                      int64_t groups, int64_t keep, double scale, int64_t score);
torch::Tensor clamped_glu(torch::Tensor gu, double limit, double alpha, int64_t kind);
torch::Tensor moe_combine(torch::Tensor down, torch::Tensor inv, torch::Tensor wts, torch::Tensor shared,
                          torch::Tensor gate, torch::Tensor add);
torch::Tensor expert_pairs(torch::Tensor h, torch::Tensor ids, torch::Tensor wgu, torch::Tensor wd, double limit,
                           double alpha, int64_t kind);
torch::Tensor expert_pairs_plain(torch::Tensor h, torch::Tensor ids, torch::Tensor wu, torch::Tensor wd);

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("sandwich_norm_add", &sandwich_norm_add);
  m.def("restart_norm", &restart_norm);
  m.def("gate_finish", &gate_finish);
  m.def("differential_finish", &differential_finish);
  m.def("relu2", &relu2);
  m.def("rope_norm_store", &rope_norm_store);
  m.def("map_attention", &map_attention);
  m.def("map_attention_mfma", &map_attention_mfma);
  m.def("embed_plain", &embed_plain);
  m.def("residual_group_norm", &residual_group_norm);
  m.def("moe_router", &moe_router);
  m.def("clamped_glu", &clamped_glu);
  m.def("moe_combine", &moe_combine);
  m.def("expert_pairs", &expert_pairs);
  m.def("expert_pairs_plain", &expert_pairs_plain);
}
