// Python bindings for the stream kernel group: several residual streams with
// learned read and write weights, token shift, linear attention with a
// token-dependent decay per key channel, sliding-window attention with a
// distance bias whose values are its keys (with a short convolution on q and
// k), group-limited routing and the expert-side helpers. Built as its own
// module so that a model needing only these compiles nothing else.
#include <torch/extension.h>

namespace kukeon {
void embed_streams(torch::Tensor xs, torch::Tensor ids, torch::Tensor positions,
                   torch::Tensor table, torch::Tensor pos_table, double scale);
void stream_read_norm(torch::Tensor out, torch::Tensor xs, torch::Tensor coef,
                      torch::Tensor w, double eps);
void stream_write_read_norm(torch::Tensor xs, torch::Tensor y,
                            torch::Tensor mix, torch::Tensor outc,
                            torch::Tensor coef, torch::Tensor w, double eps,
                            torch::Tensor out);
void token_shift(torch::Tensor out, torch::Tensor h, torch::Tensor mu,
                 torch::Tensor state, torch::Tensor positions,
                 torch::Tensor row_seq, torch::Tensor cu_rows,
                 torch::Tensor state_slots, bool shift_state);
void token_shift_tail(torch::Tensor state, torch::Tensor h,
                      torch::Tensor positions, torch::Tensor cu_rows,
                      torch::Tensor state_slots);
void head_rmsnorm_gate(torch::Tensor out, torch::Tensor y, torch::Tensor gate,
                       torch::Tensor w, int64_t H, double eps, int64_t act,
                       double scale);
void scaled_gate(torch::Tensor out, torch::Tensor a, torch::Tensor gate,
                 int64_t act, double scale);
void decay_scan(torch::Tensor y, torch::Tensor q, torch::Tensor k,
                torch::Tensor v, torch::Tensor lo, torch::Tensor w2,
                torch::Tensor zb, torch::Tensor bonus, torch::Tensor state,
                torch::Tensor positions, torch::Tensor cu_rows,
                torch::Tensor state_slots, int64_t H, int64_t d, int64_t dv,
                int64_t mode, double tau, double q_scale);
void conv_scale_append(torch::Tensor q_out, torch::Tensor k_cache,
                       torch::Tensor proj, int64_t q_col, int64_t k_col,
                       torch::Tensor cw, torch::Tensor state, double coef,
                       int64_t every, torch::Tensor positions,
                       torch::Tensor row_seq, torch::Tensor cu_rows,
                       torch::Tensor state_slots, torch::Tensor block_table,
                       bool shift_state);
void conv_state_update(torch::Tensor state, torch::Tensor proj,
                       torch::Tensor bias, torch::Tensor positions,
                       torch::Tensor cu_rows, torch::Tensor state_slots,
                       int64_t q_col, int64_t k_col, int64_t v_col, int64_t Cq,
                       int64_t Ck, int64_t Cv);
void window_attention(torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
                      torch::Tensor v_cache, torch::Tensor slopes,
                      torch::Tensor positions, torch::Tensor row_seq,
                      torch::Tensor block_table, int64_t H, double scale,
                      int64_t window);
bool window_attention_tiles_supported(int64_t d, int64_t BS);
void window_attention_tiles(torch::Tensor out, torch::Tensor q,
                            torch::Tensor k_cache, torch::Tensor slopes,
                            torch::Tensor block_table, torch::Tensor seq_lens,
                            torch::Tensor q_starts, torch::Tensor qb_seq,
                            torch::Tensor qb_start, double scale,
                            int64_t window);
void router_select(torch::Tensor idx, torch::Tensor wts, torch::Tensor logits,
                   int64_t top, int64_t groups, int64_t keep, double scale,
                   int64_t dense_rows);
void router_topk(torch::Tensor idx, torch::Tensor wts, torch::Tensor logits,
                 int64_t top, int64_t dense_rows);
void combine_rows_weighted(torch::Tensor out, torch::Tensor in,
                           torch::Tensor inv, torch::Tensor wts);
void clamp_glu(torch::Tensor out, torch::Tensor gate, torch::Tensor up,
               torch::Tensor bg, torch::Tensor bu, double limit, double alpha,
               double up_shift);
void gather_rows(torch::Tensor out, torch::Tensor in, torch::Tensor map);
}  // namespace kukeon

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("embed_streams", &kukeon::embed_streams,
        "every stream = table[id] * scale + pos_table[position]");
  m.def("stream_read_norm", &kukeon::stream_read_norm,
        "out = rmsnorm(sum_s coef[s] x_s) * w");
  m.def("stream_write_read_norm", &kukeon::stream_write_read_norm,
        "streams' update from a sublayer output, then the next read and norm");
  m.def("token_shift", &kukeon::token_shift,
        "out[n] = h + (row before - h) * mu[n], carried last row");
  m.def("token_shift_tail", &kukeon::token_shift_tail,
        "slot <- last row of a portion");
  m.def("head_rmsnorm_gate", &kukeon::head_rmsnorm_gate,
        "per head y / rms(y) * w * act(gate) * scale");
  m.def("scaled_gate", &kukeon::scaled_gate, "a * act(gate) * scale");
  m.def("decay_scan", &kukeon::decay_scan,
        "linear attention with a token-dependent decay per key channel");
  m.def("conv_scale_append", &kukeon::conv_scale_append,
        "short convolution on q and k, query temperature, paged key append");
  m.def("conv_state_update", &kukeon::conv_state_update,
        "shift a portion's tail into the convolution state slots");
  m.def("window_attention", &kukeon::window_attention,
        "sliding-window attention with a distance bias");
  m.def("window_attention_tiles_supported",
        &kukeon::window_attention_tiles_supported);
  m.def("window_attention_tiles", &kukeon::window_attention_tiles,
        "sliding-window attention for prompt portions on the matrix cores");
  m.def("router_select", &kukeon::router_select,
        "group-limited choice by softmax scores, normalised weights");
  m.def("router_topk", &kukeon::router_topk,
        "top experts per row and the softmax over their logits");
  m.def("combine_rows_weighted", &kukeon::combine_rows_weighted,
        "out[t] = sum over k of w[t, k] * in[inv[t, k]]");
  m.def("clamp_glu", &kukeon::clamp_glu,
        "clamped gate * sigmoid(alpha gate) * (up + shift)");
  m.def("gather_rows", &kukeon::gather_rows, "out[r] = in[map[r]]");
}
