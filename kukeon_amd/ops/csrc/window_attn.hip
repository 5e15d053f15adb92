// Query/key preparation of an attention whose projections pass a short causal
// convolution and whose values are its keys:
//   y[r, c] = sum_j cw[j, c] * u[i - back + j, c]          (no bias)
// over the query columns and the key columns of one fused projection, u
// being the projection for rows of this portion and the sequence's state
// slot for the back = taps-1 inputs before it (zeros before position 0, so
// a slot's earlier content is never read by a new sequence; taps are summed
// oldest first whatever the portion's length). The queries are multiplied by
// the temperature 1 + coef ln(floor((p + 1) / every) + 1) of their position
// and go to a dense buffer; the keys go to the row's page. When every
// sequence brings exactly one row the same launch shifts the slots;
// otherwise conv_state_update does afterwards.
#include "elem.h"

namespace kukeon {

// VEC: 8 consecutive channels per thread; Cq, d, the columns and the row
// strides are multiples of 8 then, so a piece never straddles q and k or two
// heads.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void conv_scale_append_kernel(
    T* __restrict__ q_out, T* __restrict__ k_cache, const T* __restrict__ proj,
    long ldp, long q_col, long k_col, const float* __restrict__ cw,
    float* __restrict__ state, float coef, int every,
    const int* __restrict__ positions, const int* __restrict__ row_seq,
    const int* __restrict__ cu_rows, const int* __restrict__ state_slots,
    const int* __restrict__ block_table, int max_blocks, int Cq, int Ck, int G,
    int d, int BS, int taps, int shift) {
  constexpr int V = VEC ? 8 : 1;
  const long r = blockIdx.x;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * V;
  const int C = Cq + Ck;
  if (c >= C) return;
  const int p = positions[r];
  if (p < 0) return;
  const int s = row_seq[r];
  const long row0 = cu_rows[s];
  const int i = (int)(r - row0);
  const int back = taps - 1;
  const long col = c < Cq ? q_col + c : k_col + (c - Cq);
  float* st = state + (long)state_slots[s] * back * C;
  float acc[V];
#pragma unroll
  for (int k = 0; k < V; ++k) acc[k] = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int src = i - back + j;
    if (p - back + j < 0) continue;           // before the sequence start
    float u[V], w[V];
    if (VEC) {
      if (src >= 0) ld8(proj + (row0 + src) * ldp + col, u);
      else ld8(st + (long)(back + src) * C + c, u);
      ld8(cw + (long)j * C + c, w);
    } else {
      u[0] = src >= 0 ? ldf(proj + (row0 + src) * ldp + col)
                      : st[(long)(back + src) * C + c];
      w[0] = cw[(long)j * C + c];
    }
#pragma unroll
    for (int k = 0; k < V; ++k) acc[k] = fmaf(w[k], u[k], acc[k]);
  }
  if (c < Cq) {
    if (every > 0) {
      const float temp =
          1.0f + coef * logf((float)((p + 1) / every) + 1.0f);
#pragma unroll
      for (int k = 0; k < V; ++k) acc[k] *= temp;
    }
    if (VEC) st8(q_out + r * (long)Cq + c, acc);
    else stf(q_out + r * (long)Cq + c, acc[0]);
  } else {
    const int ck = c - Cq;
    const int g = ck / d, dd = ck - g * d;
    const long blk = block_table[(long)s * max_blocks + p / BS];
    T* dst = k_cache + ((blk * G + g) * BS + p % BS) * (long)d + dd;
    if (VEC) st8(dst, acc);
    else stf(dst, acc[0]);
  }
  if (shift && back > 0) {
    // the sequence's only row: this thread owns its channels of the slot
    float u[V];
    for (int k = 0; k + 1 < back; ++k) {
      if (VEC) {
        ld8(st + (long)(k + 1) * C + c, u);
        st8(st + (long)k * C + c, u);
      } else {
        st[(long)k * C + c] = st[(long)(k + 1) * C + c];
      }
    }
    if (VEC) {
      ld8(proj + r * ldp + col, u);
      st8(st + (long)(back - 1) * C + c, u);
    } else {
      st[(long)(back - 1) * C + c] = ldf(proj + r * ldp + col);
    }
  }
}

// q_out [T, Cq] contiguous; k_cache [blocks, G, BS, d]; proj [T, ld]
// (stride(1) == 1); cw [taps, Cq + G*d] fp32; state [slots, taps-1, Cq + G*d]
// fp32.
void conv_scale_append(torch::Tensor q_out, torch::Tensor k_cache,
                       torch::Tensor proj, int64_t q_col, int64_t k_col,
                       torch::Tensor cw, torch::Tensor state, double coef,
                       int64_t every, torch::Tensor positions,
                       torch::Tensor row_seq, torch::Tensor cu_rows,
                       torch::Tensor state_slots, torch::Tensor block_table,
                       bool shift_state) {
  check_act(proj, "proj"); check_f32(cw, "cw"); check_f32(state, "state");
  check_i32(positions, "positions"); check_i32(row_seq, "row_seq");
  check_i32(cu_rows, "cu_rows"); check_i32(state_slots, "state_slots");
  check_i32(block_table, "block_table");
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1);
  const long rows = proj.size(0);
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.is_contiguous() &&
              k_cache.scalar_type() == proj.scalar_type());
  const int G = (int)k_cache.size(1), BS = (int)k_cache.size(2);
  const int d = (int)k_cache.size(3);
  TORCH_CHECK(q_out.dim() == 2 && q_out.is_contiguous() &&
              q_out.size(0) == rows &&
              q_out.scalar_type() == proj.scalar_type());
  const int Cq = (int)q_out.size(1), Ck = G * d;
  const long C = Cq + Ck;
  TORCH_CHECK(cw.dim() == 2 && cw.size(1) == C && cw.size(0) >= 1);
  const long taps = cw.size(0);
  TORCH_CHECK(state.dim() == 3 && state.size(1) == taps - 1 &&
              state.size(2) == C);
  TORCH_CHECK(q_col >= 0 && q_col + Cq <= proj.size(1) && k_col >= 0 &&
              k_col + Ck <= proj.size(1));
  TORCH_CHECK(positions.numel() == rows && row_seq.numel() == rows);
  TORCH_CHECK(block_table.dim() == 2 && every >= 0);
  const long nseq = cu_rows.numel() - 1;
  TORCH_CHECK(nseq >= 0 && state_slots.numel() >= nseq);
  if (rows == 0) return;
  TORCH_CHECK(!shift_state || rows == nseq,
              "the state is shifted in place only when every sequence brings "
              "one row");
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool vec = Cq % 8 == 0 && d % 8 == 0 && q_col % 8 == 0 &&
                   k_col % 8 == 0 && proj.stride(0) % 8 == 0 &&
                   aligned16(proj.data_ptr()) && aligned16(q_out.data_ptr()) &&
                   aligned16(k_cache.data_ptr()) && aligned16(cw.data_ptr()) &&
                   aligned16(state.data_ptr());
#define KK_ARGS reinterpret_cast<T*>(q_out.data_ptr()),                         \
        reinterpret_cast<T*>(k_cache.data_ptr()),                               \
        reinterpret_cast<const T*>(proj.data_ptr()), (long)proj.stride(0),      \
        (long)q_col, (long)k_col, cw.data_ptr<float>(),                         \
        state.data_ptr<float>(), (float)coef, (int)every,                       \
        positions.data_ptr<int>(), row_seq.data_ptr<int>(),                     \
        cu_rows.data_ptr<int>(), state_slots.data_ptr<int>(),                   \
        block_table.data_ptr<int>(), (int)block_table.size(1), Cq, Ck, G, d,    \
        BS, (int)taps, (int)shift_state
  KK_DISPATCH_ACT(proj, {
    if (vec) {
      const int threads = C / 8 >= 256 ? 256 : 64;
      dim3 grid((unsigned)rows, (unsigned)((C / 8 + threads - 1) / threads));
      conv_scale_append_kernel<T, true><<<grid, threads, 0, stream>>>(KK_ARGS);
    } else {
      dim3 grid((unsigned)rows, (unsigned)((C + 255) / 256));
      conv_scale_append_kernel<T, false><<<grid, 256, 0, stream>>>(KK_ARGS);
    }
  });
#undef KK_ARGS
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
