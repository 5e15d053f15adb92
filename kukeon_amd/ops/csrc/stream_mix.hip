// Several residual streams per token, kept in fp32 as xs [T, S, W]:
//   embed_streams            every stream = table[id] * scale + pos_table[p]
//   stream_read_norm         out = rmsnorm(sum_s coef[s] x_s) * w
//   stream_write_read_norm   x_j <- sum_s mix[s, j] x_s + outc[j] y  for all j
//                            from the old streams, in place, then the next
//                            sublayer's read and norm in the same pass over
//                            the row (the blend waits in LDS for the sum of
//                            squares)
// and the element-wise companions of the recurrent mixers:
//   token_shift              out[n] = h + (row before - h) * mu[n]; the row
//                            before a portion's first row is the sequence's
//                            state slot (zeros at position 0)
//   token_shift_tail         slot <- last row of a portion
//   head_rmsnorm_gate        per head y / rms(y) * w * act(gate) * scale
//   scaled_gate              a * act(gate) * scale
// One workgroup per row for the stream kernels; all arithmetic in fp32.
#include "elem.h"

namespace kukeon {

#define SM_MAX_S 8

DEV_INLINE float gate_act(float g, int act) {
  const float s = 1.0f / (1.0f + expf(-g));
  return act == 0 ? g * s : s;
}

template <typename T>
__global__ __launch_bounds__(256) void embed_streams_kernel(
    float* __restrict__ xs, const int* __restrict__ ids,
    const int* __restrict__ positions, const T* __restrict__ table,
    const T* __restrict__ pos_table, float scale, int S, int W, long vocab,
    long npos) {
  const long r = blockIdx.x;
  const int p = positions[r];
  float* xr = xs + r * (long)S * W;
  if (p < 0) {
    for (int i = threadIdx.x; i < S * W; i += blockDim.x) xr[i] = 0.f;
    return;
  }
  long id = ids[r];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* er = table + id * (long)W;
  const T* pr = pos_table ? pos_table + (long)(p < npos ? p : npos - 1) * W
                          : nullptr;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = ldf(er + i) * scale;
    if (pr) v += ldf(pr + i);
    for (int s = 0; s < S; ++s) xr[(long)s * W + i] = v;
  }
}

void embed_streams(torch::Tensor xs, torch::Tensor ids, torch::Tensor positions,
                   torch::Tensor table, torch::Tensor pos_table, double scale) {
  check_f32(xs, "xs"); check_i32(ids, "ids"); check_i32(positions, "positions");
  check_act(table, "table");
  TORCH_CHECK(xs.dim() == 3 && table.dim() == 2 && table.is_contiguous());
  const long rows = xs.size(0);
  const int S = (int)xs.size(1), W = (int)xs.size(2);
  TORCH_CHECK(table.size(1) == W && ids.numel() == rows &&
              positions.numel() == rows);
  const bool hp = pos_table.numel() > 0;
  if (hp)
    TORCH_CHECK(pos_table.dim() == 2 && pos_table.size(1) == W &&
                pos_table.is_contiguous() && pos_table.is_cuda() &&
                pos_table.scalar_type() == table.scalar_type());
  if (rows == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  KK_DISPATCH_ACT(table, {
    embed_streams_kernel<T><<<dim3((unsigned)rows), 256, 0, stream>>>(
        xs.data_ptr<float>(), ids.data_ptr<int>(), positions.data_ptr<int>(),
        reinterpret_cast<const T*>(table.data_ptr()),
        hp ? reinterpret_cast<const T*>(pos_table.data_ptr()) : nullptr,
        (float)scale, S, W, (long)table.size(0),
        hp ? (long)pos_table.size(0) : 0L);
  });
  HIP_CHECK_KERNEL();
}

// 4 consecutive elements in the storage format
DEV_INLINE void ld4(const float* p, float* o) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
}
DEV_INLINE void ld4(const bf16_t* p, float* o) {
  const uint2 a = *reinterpret_cast<const uint2*>(p);
  o[0] = us2f((unsigned short)(a.x & 0xffffu)); o[1] = us2f((unsigned short)(a.x >> 16));
  o[2] = us2f((unsigned short)(a.y & 0xffffu)); o[3] = us2f((unsigned short)(a.y >> 16));
}
DEV_INLINE void st4(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = float4{v[0], v[1], v[2], v[3]};
}
DEV_INLINE void st4(bf16_t* p, const float* v) {
  *reinterpret_cast<uint2*>(p) =
      uint2{(unsigned)f2us(v[0]) | ((unsigned)f2us(v[1]) << 16),
            (unsigned)f2us(v[2]) | ((unsigned)f2us(v[3]) << 16)};
}

// WRITE: first the streams' update from y, then the read. The blend u waits
// in LDS (W floats) while the row's sum of squares is reduced. V = 4: W is a
// multiple of 4 and all rows 16-byte aligned, every access a 16-byte piece
// (8 bytes for bf16); the workgroup is as wide as the row allows, so that a
// step of few rows still has all of a row's loads in flight at once.
template <typename T, bool WRITE, int V>
__global__ __launch_bounds__(1024) void stream_norm_kernel(
    float* __restrict__ xs, const T* __restrict__ y, long ldy,
    const float* __restrict__ mix, const float* __restrict__ outc,
    const float* __restrict__ coef, const float* __restrict__ w, float eps,
    T* __restrict__ out, int S, int W) {
  extern __shared__ float su[];            // [W] blend, then 32 for the sum
  float* red = su + W;
  __shared__ float smix[SM_MAX_S * SM_MAX_S], sout[SM_MAX_S], scoef[SM_MAX_S];
  if (threadIdx.x < S) {
    scoef[threadIdx.x] = coef[threadIdx.x];
    if (WRITE) sout[threadIdx.x] = outc[threadIdx.x];
  }
  if (WRITE && threadIdx.x < S * S) smix[threadIdx.x] = mix[threadIdx.x];
  __syncthreads();
  const long r = blockIdx.x;
  float* xr = xs + r * (long)S * W;
  const T* yr = WRITE ? y + r * ldy : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x * V; i < W; i += blockDim.x * V) {
    float xo[SM_MAX_S][V];
#pragma unroll
    for (int s = 0; s < SM_MAX_S; ++s) {
      if (s < S) {
        if (V == 4) ld4(xr + (long)s * W + i, xo[s]);
        else xo[s][0] = xr[(long)s * W + i];
      }
    }
    float u[V];
#pragma unroll
    for (int k = 0; k < V; ++k) u[k] = 0.f;
    if (WRITE) {
      float yv[V];
      if (V == 4) ld4(yr + i, yv);
      else yv[0] = ldf(yr + i);
#pragma unroll
      for (int j = 0; j < SM_MAX_S; ++j) {
        if (j < S) {
          float v[V];
#pragma unroll
          for (int k = 0; k < V; ++k) {
            float a = 0.f;
#pragma unroll
            for (int s = 0; s < SM_MAX_S; ++s)
              if (s < S) a = fmaf(smix[s * S + j], xo[s][k], a);
            v[k] = fmaf(sout[j], yv[k], a);
            u[k] = fmaf(scoef[j], v[k], u[k]);
          }
          if (V == 4) st4(xr + (long)j * W + i, v);
          else xr[(long)j * W + i] = v[0];
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < SM_MAX_S; ++s)
        if (s < S)
#pragma unroll
          for (int k = 0; k < V; ++k) u[k] = fmaf(scoef[s], xo[s][k], u[k]);
    }
#pragma unroll
    for (int k = 0; k < V; ++k) {
      su[i + k] = u[k];
      ss = fmaf(u[k], u[k], ss);
    }
  }
  const float rs = 1.0f / sqrtf(block_sum2(ss, 0.f, red).x / (float)W + eps);
  T* orow = out + r * (long)W;
  for (int i = threadIdx.x * V; i < W; i += blockDim.x * V) {
    float o[V];
#pragma unroll
    for (int k = 0; k < V; ++k) o[k] = su[i + k] * rs * w[i + k];
    if (V == 4) st4(orow + i, o);
    else stf(orow + i, o[0]);
  }
}

// threads of a workgroup for rows of W entries taken V at a time
static int stream_threads(int W, int V) {
  const int want = (W / V + 63) / 64 * 64;
  return want < 64 ? 64 : (want > 1024 ? 1024 : want);
}

static void stream_check(const torch::Tensor& xs, const torch::Tensor& coef,
                         const torch::Tensor& w, const torch::Tensor& out) {
  check_f32(xs, "xs"); check_f32(coef, "coef"); check_f32(w, "w");
  check_act(out, "out");
  TORCH_CHECK(xs.dim() == 3 && out.dim() == 2 && out.is_contiguous());
  const long S = xs.size(1);
  TORCH_CHECK(S >= 1 && S <= SM_MAX_S, "1 to 8 streams are served");
  TORCH_CHECK(coef.numel() == S && w.numel() == xs.size(2) &&
              out.size(0) == xs.size(0) && out.size(1) == xs.size(2));
  TORCH_CHECK((xs.size(2) + 32) * sizeof(float) <= 64 * 1024,
              "row too wide for the blend buffer");
}

void stream_read_norm(torch::Tensor out, torch::Tensor xs, torch::Tensor coef,
                      torch::Tensor w, double eps) {
  stream_check(xs, coef, w, out);
  const long rows = xs.size(0);
  const int S = (int)xs.size(1), W = (int)xs.size(2);
  if (rows == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const size_t shmem = (size_t)(W + 32) * sizeof(float);
  const bool vec = W % 4 == 0 && aligned16(xs.data_ptr()) &&
                   aligned16(w.data_ptr()) && aligned16(out.data_ptr());
#define KK_GO(V_)                                                             \
  {                                                                           \
    auto kern = stream_norm_kernel<T, false, V_>;                             \
    static size_t allowed = 48 * 1024;                                        \
    if (shmem > allowed) {                                                    \
      hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                \
                          hipFuncAttributeMaxDynamicSharedMemorySize,         \
                          (int)shmem);                                        \
      allowed = shmem;                                                        \
    }                                                                         \
    kern<<<dim3((unsigned)rows), stream_threads(W, V_), shmem, stream>>>(     \
        xs.data_ptr<float>(), nullptr, 0L, nullptr, nullptr,                  \
        coef.data_ptr<float>(), w.data_ptr<float>(), (float)eps,              \
        reinterpret_cast<T*>(out.data_ptr()), S, W);                          \
  }
  KK_DISPATCH_ACT(out, {
    if (vec) KK_GO(4) else KK_GO(1)
  });
#undef KK_GO
  HIP_CHECK_KERNEL();
}

void stream_write_read_norm(torch::Tensor xs, torch::Tensor y,
                            torch::Tensor mix, torch::Tensor outc,
                            torch::Tensor coef, torch::Tensor w, double eps,
                            torch::Tensor out) {
  stream_check(xs, coef, w, out);
  check_act(y, "y"); check_f32(mix, "mix"); check_f32(outc, "outc");
  const long rows = xs.size(0);
  const int S = (int)xs.size(1), W = (int)xs.size(2);
  TORCH_CHECK(y.dim() == 2 && y.size(0) == rows && y.size(1) == W &&
              y.stride(1) == 1 && y.scalar_type() == out.scalar_type());
  TORCH_CHECK(mix.numel() == (long)S * S && outc.numel() == S);
  if (rows == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const size_t shmem = (size_t)(W + 32) * sizeof(float);
  const bool vec = W % 4 == 0 && y.stride(0) % 4 == 0 &&
                   aligned16(xs.data_ptr()) && aligned16(w.data_ptr()) &&
                   aligned16(out.data_ptr()) && aligned16(y.data_ptr());
#define KK_GO(V_)                                                             \
  {                                                                           \
    auto kern = stream_norm_kernel<T, true, V_>;                              \
    static size_t allowed = 48 * 1024;                                        \
    if (shmem > allowed) {                                                    \
      hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                \
                          hipFuncAttributeMaxDynamicSharedMemorySize,         \
                          (int)shmem);                                        \
      allowed = shmem;                                                        \
    }                                                                         \
    kern<<<dim3((unsigned)rows), stream_threads(W, V_), shmem, stream>>>(     \
        xs.data_ptr<float>(), reinterpret_cast<const T*>(y.data_ptr()),       \
        (long)y.stride(0), mix.data_ptr<float>(), outc.data_ptr<float>(),     \
        coef.data_ptr<float>(), w.data_ptr<float>(), (float)eps,              \
        reinterpret_cast<T*>(out.data_ptr()), S, W);                          \
  }
  KK_DISPATCH_ACT(out, {
    if (vec) KK_GO(4) else KK_GO(1)
  });
#undef KK_GO
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
// out [N, T, W]; h [T, W]; mu [N, W] fp32; state [slots, W] fp32.
template <typename T>
__global__ __launch_bounds__(256) void token_shift_kernel(
    T* __restrict__ out, const T* __restrict__ h, const float* __restrict__ mu,
    float* __restrict__ state, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ cu_rows,
    const int* __restrict__ state_slots, long rows, int N, int W, int shift) {
  const long r = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int p = positions[r];
  if (p < 0) return;
  const int s = row_seq[r];
  const long row0 = cu_rows[s];
  float* st = state + (long)state_slots[s] * W;
  const float cur = ldf(h + r * (long)W + c);
  const float prev = r > row0 ? ldf(h + (r - 1) * (long)W + c)
                              : (p > 0 ? st[c] : 0.f);
  const float dlt = prev - cur;
  for (int n = 0; n < N; ++n)
    stf(out + ((long)n * rows + r) * W + c, fmaf(dlt, mu[(long)n * W + c], cur));
  if (shift) st[c] = cur;      // the sequence's only row: this thread's entry
}

// 8 consecutive entries per thread (W a multiple of 8, 16-byte aligned rows)
template <typename T>
__global__ __launch_bounds__(256) void token_shift_vec_kernel(
    T* __restrict__ out, const T* __restrict__ h, const float* __restrict__ mu,
    float* __restrict__ state, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ cu_rows,
    const int* __restrict__ state_slots, long rows, int N, int W, int shift) {
  const long r = blockIdx.x;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (c >= W) return;
  const int p = positions[r];
  if (p < 0) return;
  const int s = row_seq[r];
  const long row0 = cu_rows[s];
  float* st = state + (long)state_slots[s] * W;
  float cur[8], prev[8];
  ld8(h + r * (long)W + c, cur);
  if (r > row0) {
    ld8(h + (r - 1) * (long)W + c, prev);
  } else if (p > 0) {
    ld8(st + c, prev);
  } else {
#pragma unroll
    for (int k = 0; k < 8; ++k) prev[k] = 0.f;
  }
  for (int n = 0; n < N; ++n) {
    float m[8], o[8];
    ld8(mu + (long)n * W + c, m);
#pragma unroll
    for (int k = 0; k < 8; ++k) o[k] = fmaf(prev[k] - cur[k], m[k], cur[k]);
    st8(out + ((long)n * rows + r) * W + c, o);
  }
  if (shift) st8(st + c, cur);
}

void token_shift(torch::Tensor out, torch::Tensor h, torch::Tensor mu,
                 torch::Tensor state, torch::Tensor positions,
                 torch::Tensor row_seq, torch::Tensor cu_rows,
                 torch::Tensor state_slots, bool shift_state) {
  check_act(h, "h"); check_f32(mu, "mu"); check_f32(state, "state");
  check_i32(positions, "positions"); check_i32(row_seq, "row_seq");
  check_i32(cu_rows, "cu_rows"); check_i32(state_slots, "state_slots");
  TORCH_CHECK(h.dim() == 2 && h.is_contiguous() && out.dim() == 3 &&
              out.is_contiguous() && out.scalar_type() == h.scalar_type());
  const long rows = h.size(0);
  const int W = (int)h.size(1), N = (int)out.size(0);
  TORCH_CHECK(out.size(1) == rows && out.size(2) == W && mu.dim() == 2 &&
              mu.size(0) == N && mu.size(1) == W);
  TORCH_CHECK(state.dim() == 2 && state.size(1) == W);
  TORCH_CHECK(positions.numel() == rows && row_seq.numel() == rows);
  const long nseq = cu_rows.numel() - 1;
  TORCH_CHECK(nseq >= 0 && state_slots.numel() >= nseq);
  if (rows == 0) return;
  TORCH_CHECK(!shift_state || rows == nseq,
              "the slot is shifted in place only when every sequence brings "
              "one row");
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool vec = W % 8 == 0 && aligned16(out.data_ptr()) &&
                   aligned16(h.data_ptr()) && aligned16(mu.data_ptr()) &&
                   aligned16(state.data_ptr());
#define KK_ARGS reinterpret_cast<T*>(out.data_ptr()),                          \
        reinterpret_cast<const T*>(h.data_ptr()), mu.data_ptr<float>(),       \
        state.data_ptr<float>(), positions.data_ptr<int>(),                   \
        row_seq.data_ptr<int>(), cu_rows.data_ptr<int>(),                     \
        state_slots.data_ptr<int>(), rows, N, W, (int)shift_state
  KK_DISPATCH_ACT(h, {
    if (vec) {
      const int threads = W / 8 >= 256 ? 256 : 64;
      dim3 grid((unsigned)rows, (unsigned)((W / 8 + threads - 1) / threads));
      token_shift_vec_kernel<T><<<grid, threads, 0, stream>>>(KK_ARGS);
    } else {
      dim3 grid((unsigned)rows, (unsigned)((W + 255) / 256));
      token_shift_kernel<T><<<grid, 256, 0, stream>>>(KK_ARGS);
    }
  });
#undef KK_ARGS
  HIP_CHECK_KERNEL();
}

template <typename T>
__global__ __launch_bounds__(256) void token_shift_tail_kernel(
    float* __restrict__ state, const T* __restrict__ h,
    const int* __restrict__ positions, const int* __restrict__ cu_rows,
    const int* __restrict__ state_slots, int W) {
  const int s = blockIdx.x;
  const long r0 = cu_rows[s], r1 = cu_rows[s + 1];
  if (r1 <= r0 || positions[r0] < 0) return;
  float* st = state + (long)state_slots[s] * W;
  const T* row = h + (r1 - 1) * (long)W;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < W;
       c += gridDim.y * blockDim.x)
    st[c] = ldf(row + c);
}

void token_shift_tail(torch::Tensor state, torch::Tensor h,
                      torch::Tensor positions, torch::Tensor cu_rows,
                      torch::Tensor state_slots) {
  check_act(h, "h"); check_f32(state, "state");
  check_i32(positions, "positions"); check_i32(cu_rows, "cu_rows");
  check_i32(state_slots, "state_slots");
  TORCH_CHECK(h.dim() == 2 && h.is_contiguous() && state.dim() == 2 &&
              state.size(1) == h.size(1) && positions.numel() == h.size(0));
  const long nseq = cu_rows.numel() - 1;
  TORCH_CHECK(nseq >= 0 && state_slots.numel() >= nseq);
  if (nseq == 0 || h.size(0) == 0) return;
  const int W = (int)h.size(1);
  auto stream = c10::hip::getCurrentHIPStream().stream();
  dim3 grid((unsigned)nseq, (unsigned)std::min(16, (W + 255) / 256));
  KK_DISPATCH_ACT(h, {
    token_shift_tail_kernel<T><<<grid, 256, 0, stream>>>(
        state.data_ptr<float>(), reinterpret_cast<const T*>(h.data_ptr()),
        positions.data_ptr<int>(), cu_rows.data_ptr<int>(),
        state_slots.data_ptr<int>(), W);
  });
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
// One wave per (row, head): lanes stride over the head's dv entries.
template <typename T>
__global__ __launch_bounds__(256) void head_rmsnorm_gate_kernel(
    T* __restrict__ out, long ldo, const float* __restrict__ y,
    const T* __restrict__ gate, long ldg, const float* __restrict__ w, long rows,
    int H, int dv, float eps, int act, float scale) {
  const long unit = (long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  if (unit >= rows * H) return;
  const int lane = threadIdx.x & (WAVE - 1);
  const long r = unit / H;
  const int hd = (int)(unit - r * H);
  const float* yr = y + (r * H + hd) * (long)dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += WAVE) ss = fmaf(yr[i], yr[i], ss);
  const float rs = scale / sqrtf(wave_sum(ss) / (float)dv + eps);
  const long c0 = (long)hd * dv;
  for (int i = lane; i < dv; i += WAVE)
    stf(out + r * ldo + c0 + i,
        yr[i] * rs * w[c0 + i] * gate_act(ldf(gate + r * ldg + c0 + i), act));
}

// LPH = dv / 8 lanes per (row, head), 8 consecutive entries per lane; the sum
// of squares meets over the LPH neighbouring lanes.
template <typename T>
__global__ __launch_bounds__(256) void head_rmsnorm_gate_vec_kernel(
    T* __restrict__ out, long ldo, const float* __restrict__ y,
    const T* __restrict__ gate, long ldg, const float* __restrict__ w, long rows,
    int H, int dv, int LPH, float eps, int act, float scale) {
  const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long unit = t / LPH;
  const int sub = (int)(t - unit * LPH);
  const bool live = unit < rows * H;
  const long r = live ? unit / H : 0;
  const int hd = live ? (int)(unit - r * H) : 0;
  const long c0 = (long)hd * dv + sub * 8;
  float v[8];
  ld8(y + r * (long)H * dv + c0, v);
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < 8; ++k) ss = fmaf(v[k], v[k], ss);
  for (int off = LPH >> 1; off > 0; off >>= 1) ss += __shfl_xor(ss, off, WAVE);
  if (!live) return;
  const float rs = scale / sqrtf(ss / (float)dv + eps);
  float g[8], ww[8], o[8];
  ld8(gate + r * ldg + c0, g);
  ld8(w + c0, ww);
#pragma unroll
  for (int k = 0; k < 8; ++k) o[k] = v[k] * rs * ww[k] * gate_act(g[k], act);
  st8(out + r * ldo + c0, o);
}

void head_rmsnorm_gate(torch::Tensor out, torch::Tensor y, torch::Tensor gate,
                       torch::Tensor w, int64_t H, double eps, int64_t act,
                       double scale) {
  check_act(out, "out"); check_act(gate, "gate"); check_f32(y, "y");
  check_f32(w, "w");
  TORCH_CHECK(y.dim() == 2 && out.dim() == 2 && gate.dim() == 2);
  const long rows = y.size(0);
  const long C = y.size(1);
  TORCH_CHECK(H >= 1 && C % H == 0 && w.numel() == C);
  TORCH_CHECK(out.size(0) == rows && out.size(1) == C && out.stride(1) == 1 &&
              gate.size(0) == rows && gate.size(1) == C &&
              gate.stride(1) == 1 && gate.scalar_type() == out.scalar_type());
  if (rows == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const long units = rows * H;
  const int dvh = (int)(C / H);
  const int LPH = dvh / 8;
  const bool vec = dvh % 8 == 0 && LPH <= WAVE && (LPH & (LPH - 1)) == 0 &&
                   out.stride(0) % 8 == 0 && gate.stride(0) % 8 == 0 &&
                   aligned16(out.data_ptr()) && aligned16(y.data_ptr()) &&
                   aligned16(gate.data_ptr()) && aligned16(w.data_ptr());
  if (vec) {
    const long threads = units * LPH;
    KK_DISPATCH_ACT(out, {
      head_rmsnorm_gate_vec_kernel<T><<<dim3((unsigned)((threads + 255) / 256)),
                                        256, 0, stream>>>(
          reinterpret_cast<T*>(out.data_ptr()), (long)out.stride(0),
          y.data_ptr<float>(), reinterpret_cast<const T*>(gate.data_ptr()),
          (long)gate.stride(0), w.data_ptr<float>(), rows, (int)H, dvh, LPH,
          (float)eps, (int)act, (float)scale);
    });
    HIP_CHECK_KERNEL();
    return;
  }
  KK_DISPATCH_ACT(out, {
    head_rmsnorm_gate_kernel<T><<<dim3((unsigned)((units + 3) / 4)), 256, 0,
                                  stream>>>(
        reinterpret_cast<T*>(out.data_ptr()), (long)out.stride(0),
        y.data_ptr<float>(), reinterpret_cast<const T*>(gate.data_ptr()),
        (long)gate.stride(0), w.data_ptr<float>(), rows, (int)H, (int)(C / H),
        (float)eps, (int)act, (float)scale);
  });
  HIP_CHECK_KERNEL();
}

template <typename T>
__global__ __launch_bounds__(256) void scaled_gate_kernel(
    T* __restrict__ out, long ldo, const T* __restrict__ a, long lda,
    const T* __restrict__ gate, long ldg, int C, long total, int act,
    float scale) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long r = i / C;
  const int c = (int)(i - r * C);
  stf(out + r * ldo + c,
      ldf(a + r * lda + c) * gate_act(ldf(gate + r * ldg + c), act) * scale);
}

template <typename T>
__global__ __launch_bounds__(256) void scaled_gate_vec_kernel(
    T* __restrict__ out, long ldo, const T* __restrict__ a, long lda,
    const T* __restrict__ gate, long ldg, int C8, long total8, int act,
    float scale) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total8) return;
  const long r = i / C8;
  const int c = (int)(i - r * C8) * 8;
  float av[8], g[8];
  ld8(a + r * lda + c, av);
  ld8(gate + r * ldg + c, g);
#pragma unroll
  for (int k = 0; k < 8; ++k) av[k] = av[k] * gate_act(g[k], act) * scale;
  st8(out + r * ldo + c, av);
}

void scaled_gate(torch::Tensor out, torch::Tensor a, torch::Tensor gate,
                 int64_t act, double scale) {
  check_act(out, "out"); check_act(a, "a"); check_act(gate, "gate");
  TORCH_CHECK(out.dim() == 2 && a.dim() == 2 && gate.dim() == 2);
  const long rows = out.size(0);
  const int C = (int)out.size(1);
  TORCH_CHECK(a.size(0) == rows && a.size(1) == C && gate.size(0) == rows &&
              gate.size(1) == C && out.stride(1) == 1 && a.stride(1) == 1 &&
              gate.stride(1) == 1);
  TORCH_CHECK(a.scalar_type() == out.scalar_type() &&
              gate.scalar_type() == out.scalar_type());
  const long total = rows * C;
  if (total == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool vec = C % 8 == 0 && out.stride(0) % 8 == 0 &&
                   a.stride(0) % 8 == 0 && gate.stride(0) % 8 == 0 &&
                   aligned16(out.data_ptr()) && aligned16(a.data_ptr()) &&
                   aligned16(gate.data_ptr());
  KK_DISPATCH_ACT(out, {
    if (vec)
      scaled_gate_vec_kernel<T><<<dim3((unsigned)((total / 8 + 255) / 256)),
                                  256, 0, stream>>>(
          reinterpret_cast<T*>(out.data_ptr()), (long)out.stride(0),
          reinterpret_cast<const T*>(a.data_ptr()), (long)a.stride(0),
          reinterpret_cast<const T*>(gate.data_ptr()), (long)gate.stride(0),
          C / 8, total / 8, (int)act, (float)scale);
    else
      scaled_gate_kernel<T><<<dim3((unsigned)((total + 255) / 256)), 256, 0,
                              stream>>>(
          reinterpret_cast<T*>(out.data_ptr()), (long)out.stride(0),
          reinterpret_cast<const T*>(a.data_ptr()), (long)a.stride(0),
          reinterpret_cast<const T*>(gate.data_ptr()), (long)gate.stride(0),
          C, total, (int)act, (float)scale);
  });
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
