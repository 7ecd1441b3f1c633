// Python bindings of the talking-heads serving kernels: post-sublayer norm with
// a depth-weighted residual history, per-head q/k norm with pairwise rotation,
// value mixing and cache store, chunked talking-heads attention, tanh-GELU;
// and of the kernels this extension shares with the others through their
// sources (embedding into a plain residual, grouped norm, mLSTM, routed experts).
#include <torch/extension.h>
#include <vector>

torch::Tensor post_norm_add(torch::Tensor x, torch::Tensor y, torch::Tensor w, double eps, bool out_bf16,
                            torch::Tensor hist, int64_t depth, torch::Tensor dwa);
torch::Tensor gelu_tanh(torch::Tensor z);
torch::Tensor head_norm_rope_store(torch::Tensor proj, int64_t H, int64_t G, int64_t D, int64_t V, torch::Tensor wq,
                                   torch::Tensor wk, double eps, torch::Tensor freqs, torch::Tensor v_first,
                                   torch::Tensor lam, torch::Tensor pool, torch::Tensor tok_pos,
                                   torch::Tensor tok_row);
torch::Tensor talking_attention(torch::Tensor q, torch::Tensor pool, int64_t H, int64_t G, int64_t D, int64_t V,
                                double scale, torch::Tensor temp, torch::Tensor talk, int64_t chunk,
                                torch::Tensor tok_req, torch::Tensor tok_pos, torch::Tensor tables, int64_t bs);
torch::Tensor talking_attention_mfma(torch::Tensor q, torch::Tensor pool, int64_t H, int64_t G, int64_t D, int64_t V,
                                     double scale, torch::Tensor temp, torch::Tensor talk, int64_t chunk,
                                     torch::Tensor tiles, torch::Tensor cu, torch::Tensor start_pos,
                                     torch::Tensor tables, int64_t bs, int64_t nsplit);
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
// ragged/recurrent.hip
torch::Tensor mlstm_scan(torch::Tensor qkvg, torch::Tensor gates, torch::Tensor bi, torch::Tensor bfg,
                         torch::Tensor norm_w, int64_t H, int64_t D, int64_t V, double cap, double eps,
                         torch::Tensor stS, torch::Tensor stn, torch::Tensor stm, torch::Tensor cu,
                         torch::Tensor slots);

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("post_norm_add", &post_norm_add);
  m.def("gelu_tanh", &gelu_tanh);
  m.def("head_norm_rope_store", &head_norm_rope_store);
  m.def("talking_attention", &talking_attention);
  m.def("talking_attention_mfma", &talking_attention_mfma);
  m.def("embed_plain", &embed_plain);
  m.def("residual_group_norm", &residual_group_norm);
  m.def("moe_router", &moe_router);
  m.def("clamped_glu", &clamped_glu);
  m.def("moe_combine", &moe_combine);
  m.def("expert_pairs", &expert_pairs);
  m.def("mlstm_scan", &mlstm_scan);
}
