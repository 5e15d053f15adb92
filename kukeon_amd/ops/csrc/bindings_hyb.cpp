// Python bindings for the hybrid kernel group: layer norm on the output side
// of a sublayer over an fp32 residual stream, chunk-local grouped-query
// attention with whole-projection norms and a score cap, linear attention
// with a fixed decay per head, gelu- and clamp-gated activations, routed
// experts, and the latent attention over a shared low-rank cache row. Built
// as its own module so that a model needing only these compiles nothing else.
#include <torch/extension.h>

namespace kukeon {
void layernorm_residual(torch::Tensor x, torch::Tensor y, torch::Tensor w,
                        double eps, torch::Tensor out);
void layernorm(torch::Tensor out, torch::Tensor x, torch::Tensor w,
               double eps);
void gelu_glu(torch::Tensor out, torch::Tensor gate, torch::Tensor up);
void clamp_glu(torch::Tensor out, torch::Tensor gate, torch::Tensor up,
               torch::Tensor bg, torch::Tensor bu, double limit, double alpha,
               double up_shift);
void qk_norm_append(torch::Tensor q_out, torch::Tensor k_cache,
                    torch::Tensor v_cache, torch::Tensor proj, int64_t q_col,
                    int64_t k_col, int64_t v_col, torch::Tensor wq,
                    torch::Tensor wk, double eps, torch::Tensor positions,
                    torch::Tensor row_seq, torch::Tensor block_table);
void chunk_attention(torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
                     torch::Tensor v_cache, torch::Tensor positions,
                     torch::Tensor row_seq, torch::Tensor block_table,
                     int64_t H, double scale, double softcap, int64_t chunk);
bool chunk_attention_tiles_supported(int64_t d, int64_t dv, int64_t BS);
void chunk_attention_tiles(torch::Tensor out, torch::Tensor q,
                           torch::Tensor k_cache, torch::Tensor v_cache,
                           torch::Tensor block_table, torch::Tensor seq_lens,
                           torch::Tensor q_starts, torch::Tensor qb_seq,
                           torch::Tensor qb_start, double scale,
                           double softcap, int64_t chunk);
void lightning_scan(torch::Tensor y, torch::Tensor proj, int64_t q_col,
                    int64_t k_col, int64_t v_col, torch::Tensor decay,
                    torch::Tensor state, torch::Tensor positions,
                    torch::Tensor cu_rows, torch::Tensor state_slots,
                    int64_t H, int64_t d, int64_t dv);
void gated_rmsnorm(torch::Tensor out, torch::Tensor y, torch::Tensor gate,
                   torch::Tensor w, double eps);
void router_topk(torch::Tensor idx, torch::Tensor wts, torch::Tensor logits,
                 int64_t top, int64_t dense_rows);
void combine_rows_weighted(torch::Tensor out, torch::Tensor in,
                           torch::Tensor inv, torch::Tensor wts);
void head_gate(torch::Tensor out, torch::Tensor o, torch::Tensor gate);
void latent_kv_append(torch::Tensor cq_out, torch::Tensor cache,
                      torch::Tensor proj, int64_t q_col, int64_t kv_col,
                      torch::Tensor wq, torch::Tensor wkv, double eps,
                      torch::Tensor cs, torch::Tensor positions,
                      torch::Tensor row_seq, torch::Tensor block_table);
void latent_attention(torch::Tensor out, torch::Tensor q_abs, torch::Tensor q,
                      torch::Tensor cache, torch::Tensor cs,
                      torch::Tensor positions, torch::Tensor row_seq,
                      torch::Tensor block_table, int64_t H, int64_t dn,
                      int64_t dr, int64_t window, double scale);
void gather_rows(torch::Tensor out, torch::Tensor in, torch::Tensor map);
}  // namespace kukeon

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("layernorm_residual", &kukeon::layernorm_residual,
        "x += layernorm(y) * w; out = x in the activation format");
  m.def("layernorm", &kukeon::layernorm, "out = layernorm(x) * w");
  m.def("gelu_glu", &kukeon::gelu_glu, "gelu_tanh(gate) * up");
  m.def("clamp_glu", &kukeon::clamp_glu,
        "clamped gate * sigmoid(alpha gate) * (up + shift)");
  m.def("qk_norm_append", &kukeon::qk_norm_append,
        "whole-projection q/k norms, paged K/V append");
  m.def("chunk_attention", &kukeon::chunk_attention,
        "grouped-query attention over the query's own chunk, capped scores");
  m.def("chunk_attention_tiles_supported",
        &kukeon::chunk_attention_tiles_supported);
  m.def("chunk_attention_tiles", &kukeon::chunk_attention_tiles,
        "chunk-local attention for prompt portions on the matrix cores");
  m.def("lightning_scan", &kukeon::lightning_scan,
        "linear attention with a fixed decay per head, carried fp32 state");
  m.def("gated_rmsnorm", &kukeon::gated_rmsnorm,
        "rmsnorm(y) * w * sigmoid(gate)");
  m.def("router_topk", &kukeon::router_topk,
        "top experts per row and the softmax over their logits");
  m.def("combine_rows_weighted", &kukeon::combine_rows_weighted,
        "out[t] = sum over k of w[t, k] * in[inv[t, k]]");
  m.def("head_gate", &kukeon::head_gate,
        "sigmoid output gate per head or per entry, [H,T,dv] -> [T,H*dv]");
  m.def("latent_kv_append", &kukeon::latent_kv_append,
        "norm the latents, rotate the shared key part, write the cache row");
  m.def("latent_attention", &kukeon::latent_attention,
        "attention over the shared latent cache row");
  m.def("gather_rows", &kukeon::gather_rows, "out[r] = in[map[r]]");
}
