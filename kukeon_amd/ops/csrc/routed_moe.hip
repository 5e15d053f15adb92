// Router side of a mixture of experts chosen by learned logits:
//   router_topk            per row, the `top` largest logits (ties: the lower
//                          index) and the softmax over just those, fp32
//   router_select          scores = softmax over ALL logits; the experts form
//                          equal runs of neighbours of which only the best
//                          few (by their largest score) can be chosen; the
//                          chosen scores are divided by their sum and scaled
//   combine_rows_weighted  out[t] = sum_k w[t, k] * in[inv[t, k]], the k-th
//                          term added k-th, fp32 sums
// The expert GEMMs themselves are vendor GEMMs over gathered rows.
#include "elem.h"

namespace kukeon {

// One thread per row. The k-th pick is the largest (value, -index) pair
// below the previous pick, so no list of taken experts is kept; a NaN logit
// counts as -inf, which keeps every index in range.
__global__ __launch_bounds__(256) void router_topk_kernel(
    int* __restrict__ idx, float* __restrict__ wts,
    const float* __restrict__ logits, long rows, int E, int top,
    long dense_rows) {
  const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= rows) return;
  const float* z = logits + t * (long)E;
  float pv = INFINITY;
  int pe = -1;
  float vmax = 0.f, sum = 0.f;
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int be = -1;
    for (int e = 0; e < E; ++e) {
      float v = z[e];
      v = v == v ? v : -INFINITY;
      const bool below = v < pv || (v == pv && e > pe);
      const bool better = be < 0 || v > bv;
      if (below && better) { bv = v; be = e; }
    }
    pv = bv;
    pe = be;
    if (k == 0) vmax = bv;
    const float w = expf(bv - vmax);
    wts[t * top + k] = w;
    sum += w;
    idx[t * top + k] = dense_rows > 0 ? (int)(be * dense_rows + t) : be;
  }
  const float inv = 1.0f / sum;
  for (int k = 0; k < top; ++k) wts[t * top + k] *= inv;
}

// idx [T, top] int32, wts [T, top] fp32, logits [T, E] fp32. With
// dense_rows = T the index written is expert * T + row.
void router_topk(torch::Tensor idx, torch::Tensor wts, torch::Tensor logits,
                 int64_t top, int64_t dense_rows) {
  check_i32(idx, "idx"); check_f32(wts, "wts"); check_f32(logits, "logits");
  TORCH_CHECK(logits.dim() == 2);
  const long rows = logits.size(0);
  const int E = (int)logits.size(1);
  TORCH_CHECK(top >= 1 && top <= E);
  TORCH_CHECK(idx.numel() == rows * top && wts.numel() == rows * top);
  TORCH_CHECK(dense_rows == 0 || dense_rows == rows);
  TORCH_CHECK((long)E * rows < (1L << 31));
  if (rows == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  router_topk_kernel<<<dim3((unsigned)((rows + 255) / 256)), 256, 0, stream>>>(
      idx.data_ptr<int>(), wts.data_ptr<float>(), logits.data_ptr<float>(),
      rows, E, (int)top, (long)dense_rows);
  HIP_CHECK_KERNEL();
}

// One thread per row. A softmax keeps the order of the logits, so runs and
// experts are ranked by logit; every pick is the largest (value, -index) pair
// below the previous pick. A NaN logit counts as -inf.
__global__ __launch_bounds__(256) void router_select_kernel(
    int* __restrict__ idx, float* __restrict__ wts, long ldi, long ldw,
    const float* __restrict__ logits, long ldz, long rows, int E, int top,
    int groups, int keep, float scale, long dense_rows) {
  const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= rows) return;
  const float* z = logits + t * ldz;
  float vmax = -INFINITY;
  for (int e = 0; e < E; ++e) {
    const float v = z[e];
    if (v == v) vmax = fmaxf(vmax, v);
  }
  if (vmax == -INFINITY) vmax = 0.f;         // a row of NaN: finite weights
  float sum = 0.f;
  for (int e = 0; e < E; ++e) {
    const float v = z[e];
    if (v == v) sum += expf(v - vmax);
  }
  unsigned long long allowed = ~0ull;        // one bit per run
  const int per = groups > 0 ? E / groups : E;
  if (groups > 0) {
    allowed = 0ull;
    float pv = INFINITY;
    int pg = -1;
    for (int k = 0; k < keep; ++k) {
      float bv = -INFINITY;
      int bg = -1;
      for (int g = 0; g < groups; ++g) {
        float gv = -INFINITY;
        for (int e = g * per; e < (g + 1) * per; ++e) {
          const float v = z[e];
          if (v == v) gv = fmaxf(gv, v);
        }
        const bool below = gv < pv || (gv == pv && g > pg);
        const bool better = bg < 0 || gv > bv;
        if (below && better) { bv = gv; bg = g; }
      }
      pv = bv;
      pg = bg;
      allowed |= 1ull << bg;
    }
  }
  float pv = INFINITY;
  int pe = -1;
  float wsum = 0.f;
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int be = -1;
    for (int e = 0; e < E; ++e) {
      if (groups > 0 && !((allowed >> (e / per)) & 1ull)) continue;
      float v = z[e];
      v = v == v ? v : -INFINITY;
      const bool below = v < pv || (v == pv && e > pe);
      const bool better = be < 0 || v > bv;
      if (below && better) { bv = v; be = e; }
    }
    pv = bv;
    pe = be;
    const float w = expf(bv - vmax) / sum;
    wts[t * ldw + k] = w;
    wsum += w;
    idx[t * ldi + k] = dense_rows > 0 ? (int)(be * dense_rows + t) : be;
  }
  const float f = scale / (wsum + 1e-20f);
  for (int k = 0; k < top; ++k) wts[t * ldw + k] *= f;
}

// idx [T, >= top] int32, wts [T, >= top] fp32 (rows may be wider than top:
// the other columns are left alone), logits [T, E] fp32 (any row stride: the
// first E columns of a wider product).
void router_select(torch::Tensor idx, torch::Tensor wts, torch::Tensor logits,
                   int64_t top, int64_t groups, int64_t keep, double scale,
                   int64_t dense_rows) {
  TORCH_CHECK(logits.is_cuda() && logits.scalar_type() == torch::kFloat32 &&
              logits.dim() == 2 && logits.stride(1) == 1,
              "logits must be fp32 rows");
  TORCH_CHECK(idx.is_cuda() && idx.scalar_type() == torch::kInt32 &&
              wts.is_cuda() && wts.scalar_type() == torch::kFloat32);
  TORCH_CHECK(idx.dim() == 2 && wts.dim() == 2);
  const long rows = logits.size(0);
  const int E = (int)logits.size(1);
  TORCH_CHECK(top >= 1 && top <= E);
  TORCH_CHECK(idx.size(0) == rows && wts.size(0) == rows &&
              idx.size(1) >= top && wts.size(1) >= top &&
              idx.stride(1) == 1 && wts.stride(1) == 1);
  TORCH_CHECK(groups >= 0 && groups <= 64);
  if (groups > 0)
    TORCH_CHECK(E % groups == 0 && keep >= 1 && keep <= groups &&
                top <= keep * (E / groups));
  TORCH_CHECK(dense_rows == 0 || dense_rows == rows);
  TORCH_CHECK((long)E * rows < (1L << 31));
  if (rows == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  router_select_kernel<<<dim3((unsigned)((rows + 255) / 256)), 256, 0,
                         stream>>>(
      idx.data_ptr<int>(), wts.data_ptr<float>(), (long)idx.stride(0),
      (long)wts.stride(0), logits.data_ptr<float>(), (long)logits.stride(0),
      rows, E, (int)top, (int)groups, (int)keep, (float)scale,
      (long)dense_rows);
  HIP_CHECK_KERNEL();
}

template <typename T>
__global__ __launch_bounds__(256) void combine_rows_weighted_kernel(
    T* __restrict__ out, const T* __restrict__ in, const int* __restrict__ inv,
    const float* __restrict__ wts, int W, int top) {
  const long t = blockIdx.x;
  if (W % 8 == 0 && aligned16(in) && aligned16(out)) {
    for (int i = threadIdx.x * 8; i < W; i += blockDim.x * 8) {
      float acc[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = 0.f;
      for (int k = 0; k < top; ++k) {
        float v[8];
        ld8(in + (long)inv[t * top + k] * W + i, v);
        const float w = wts[t * top + k];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = fmaf(w, v[j], acc[j]);
      }
      st8(out + t * (long)W + i, acc);
    }
    return;
  }
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k)
      acc = fmaf(wts[t * top + k], ldf(in + (long)inv[t * top + k] * W + i),
                 acc);
    stf(out + t * (long)W + i, acc);
  }
}

// out [T, W]; in [n, W]; inv [T, top] rows of `in`; wts [T, top] fp32.
void combine_rows_weighted(torch::Tensor out, torch::Tensor in,
                           torch::Tensor inv, torch::Tensor wts) {
  check_act(out, "out"); check_act(in, "in"); check_i32(inv, "inv");
  check_f32(wts, "wts");
  TORCH_CHECK(out.dim() == 2 && in.dim() == 2 && out.is_contiguous() &&
              in.is_contiguous() && out.size(1) == in.size(1) &&
              out.scalar_type() == in.scalar_type());
  TORCH_CHECK(inv.dim() == 2 && inv.size(0) == out.size(0) &&
              wts.dim() == 2 && wts.size(0) == inv.size(0) &&
              wts.size(1) == inv.size(1));
  const long n = out.size(0);
  if (n == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  KK_DISPATCH_ACT(out, {
    combine_rows_weighted_kernel<T><<<dim3((unsigned)n), 256, 0, stream>>>(
        reinterpret_cast<T*>(out.data_ptr()),
        reinterpret_cast<const T*>(in.data_ptr()), inv.data_ptr<int>(),
        wts.data_ptr<float>(), (int)out.size(1), (int)inv.size(1));
  });
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
