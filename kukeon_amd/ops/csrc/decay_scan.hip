// Linear attention with a decay per key channel that depends on the token,
// the recurrent form, in two flavours that share one kernel:
//   MODE 0  a_t = exp(-exp(z_t + zb));   the read comes first and gives the
//           current token a bonus:   y_t = (S + diag(u) k_t v_t^T)^T q_t,
//           then S = diag(a_t) S + k_t v_t^T
//   MODE 1  a_t = sigmoid(z_t + zb)^(1/tau);  S = diag(a_t) S + k_t v_t^T,
//           then y_t = S^T (q_scale q_t)
// The decay's pre-activation comes from a low-rank pair: z_t = W2 f(lo_t),
// lo_t [R] being the fp32 output of the first projection (f = tanh in MODE 0,
// the identity in MODE 1) and W2 [H d, R]; the second product is a handful
// of multiply-adds per channel, so it is done here, in fp32, while a tile of
// tokens is staged (the head's rows of W2 wait in LDS), and z never exists in
// memory. The bonus term of MODE 0 does not depend on the value column:
// (diag(u) k v^T)^T q = v (sum_i u_i k_i q_i), so that sum is formed once per
// token while the tile is staged and the inner loop keeps no copy of u. The
// exponentials, the decay and the whole recurrence are fp32. One
// workgroup per (sequence, head). The
// state stays in registers for the whole portion: thread (e, l) owns the NR
// consecutive key rows l NR .. l NR + NR - 1 of value column e, so a step is
// a few fused multiply-adds per row plus a reduction over the LN neighbouring
// lanes. q, k, the decay and v of TT tokens are staged in LDS at a time, the
// key-side rows padded with zeros to LN NR entries, which keeps state rows
// past d at zero. The slot holds S^T ([H, dv, d]); it is read once at the
// start of the portion (zeros at position 0, whatever the slot held) and
// written once at its end. Tokens are visited in order, so a position's
// result does not depend on how the sequence was cut.
#include "elem.h"

namespace kukeon {

#define DS_TT 16

DEV_INLINE float log_sigmoid(float x) {
  return fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
}

template <typename T, int NR, int MODE>
__global__ __launch_bounds__(1024) void decay_scan_kernel(
    float* __restrict__ y, const T* __restrict__ q, long ldq,
    const T* __restrict__ k, long ldk, const T* __restrict__ v, long ldv,
    const float* __restrict__ lo, long ldl, int R,
    const float* __restrict__ w2, const float* __restrict__ zb,
    const float* __restrict__ bonus, float* __restrict__ state,
    const int* __restrict__ positions, const int* __restrict__ cu_rows,
    const int* __restrict__ state_slots, int H, int d, int dv, int LN,
    float inv_tau, float q_scale) {
  extern __shared__ float sm[];
  const int DP = LN * NR;               // padded key-side row
  float* sQ = sm;                       // [TT][DP]
  float* sK = sQ + DS_TT * DP;          // [TT][DP]
  float* sA = sK + DS_TT * DP;          // [TT][DP]
  float* sV = sA + DS_TT * DP;          // [TT][dv]
  float* sLo = sV + DS_TT * dv;         // [TT][R]
  float* sW2 = sLo + DS_TT * R;         // [d][R + 1]
  float* sU = sW2 + d * (R + 1);        // [d] bonus (MODE 0)
  float* sC = sU + d;                   // [TT] sum_i u_i k_i q_i (MODE 0)
  const int s = blockIdx.x;
  const int h = blockIdx.y;
  const long row0 = cu_rows[s];
  const int n = cu_rows[s + 1] - (int)row0;
  if (n <= 0) return;
  const int p0 = positions[row0];
  const int tid = threadIdx.x;
  const int nthreads = blockDim.x;
  const int inner = H * dv;
  if (p0 < 0) {                         // inactive sequence: zeros out
    for (int i = tid; i < n * dv; i += nthreads)
      y[(row0 + i / dv) * (long)inner + h * dv + i % dv] = 0.f;
    return;
  }
  // A short portion (a decode step above all) is one dependent chain: the
  // loads' completion is counted in issue order, so whatever is loaded after
  // the state waits for the state. Its few inputs are therefore fetched into
  // registers BEFORE the state loads are issued, and only committed to LDS
  // afterwards; W2's rows likewise (up to four entries per thread).
  const bool pre = n <= DS_TT && n * DP <= nthreads && n * dv <= nthreads &&
                   n * R <= nthreads;
  const bool prew = d * R <= 4 * nthreads;
  float pw[4] = {0.f, 0.f, 0.f, 0.f};
  float pq = 0.f, pk = 0.f, pv = 0.f, plo = 0.f, pu = 0.f;
  if (prew) {
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int i = tid + m * nthreads;
      if (i < d * R) pw[m] = w2[(long)h * d * R + i];
    }
  }
  if (MODE == 0 && tid < d) pu = bonus[(long)h * d + tid];
  if (pre) {
    if (tid < n * DP) {
      const int t = tid / DP, dd = tid - t * DP;
      if (dd < d) {
        pq = ldf(q + (row0 + t) * ldq + (long)h * d + dd);
        pk = ldf(k + (row0 + t) * ldk + (long)h * d + dd);
      }
    }
    if (tid < n * dv)
      pv = ldf(v + (row0 + tid / dv) * ldv + (long)h * dv + tid % dv);
    if (tid < n * R) plo = lo[(row0 + tid / R) * ldl + tid % R];
  }
  const int e = tid / LN;
  const int l = tid - e * LN;
  const bool live = e < dv;
  float* st = state + (((long)state_slots[s] * H + h) * dv + (live ? e : 0)) *
                          (long)d + l * NR;
  const bool vec4 = (d & 3) == 0;
  float S[NR];
#pragma unroll
  for (int i4 = 0; i4 < NR / 4; ++i4) {
    const int dd = l * NR + 4 * i4;
    float4 sv = float4{0.f, 0.f, 0.f, 0.f};
    if (live && p0 > 0) {
      if (vec4) {
        if (dd < d) sv = *reinterpret_cast<const float4*>(st + 4 * i4);
      } else {
        if (dd + 0 < d) sv.x = st[4 * i4 + 0];
        if (dd + 1 < d) sv.y = st[4 * i4 + 1];
        if (dd + 2 < d) sv.z = st[4 * i4 + 2];
        if (dd + 3 < d) sv.w = st[4 * i4 + 3];
      }
    }
    S[4 * i4 + 0] = sv.x; S[4 * i4 + 1] = sv.y;
    S[4 * i4 + 2] = sv.z; S[4 * i4 + 3] = sv.w;
  }
  if (prew) {
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int i = tid + m * nthreads;
      if (i < d * R) sW2[(i / R) * (R + 1) + i % R] = pw[m];
    }
  } else {
    for (int i = tid; i < d * R; i += nthreads)
      sW2[(i / R) * (R + 1) + i % R] = w2[(long)h * d * R + i];
  }
  if (MODE == 0) {
    if (tid < d) sU[tid] = pu;
    for (int i = tid + nthreads; i < d; i += nthreads)
      sU[i] = bonus[(long)h * d + i];
  }
  for (int t0 = 0; t0 < n; t0 += DS_TT) {
    const int nt = min(DS_TT, n - t0);
    __syncthreads();
    for (int i = tid; i < nt * R; i += nthreads) {
      const int t = i / R, j = i - t * R;
      const float x = pre ? plo : lo[(row0 + t0 + t) * ldl + j];
      sLo[i] = MODE == 0 ? tanhf(x) : x;
    }
    __syncthreads();
    for (int i = tid; i < nt * DP; i += nthreads) {
      const int t = i / DP, dd = i - t * DP;
      const long r = row0 + t0 + t;
      const long c = (long)h * d + dd;
      float qv = 0.f, kv = 0.f, av = 0.f;
      if (dd < d) {
        qv = (pre ? pq : ldf(q + r * ldq + c)) * q_scale;
        kv = pre ? pk : ldf(k + r * ldk + c);
        float zz = zb[c];
        for (int j = 0; j < R; ++j)
          zz = fmaf(sLo[t * R + j], sW2[dd * (R + 1) + j], zz);
        av = MODE == 0 ? expf(-expf(zz)) : expf(log_sigmoid(zz) * inv_tau);
      }
      sQ[i] = qv; sK[i] = kv; sA[i] = av;
    }
    for (int i = tid; i < nt * dv; i += nthreads) {
      const int t = i / dv, ee = i - t * dv;
      sV[i] = pre ? pv : ldf(v + (row0 + t0 + t) * ldv + (long)h * dv + ee);
    }
    __syncthreads();
    if (MODE == 0) {
      // 16 lanes per token share out the key channels
      for (int i = tid; i < nt * 16; i += nthreads) {
        const int t = i >> 4, part = i & 15;
        float c = 0.f;
        for (int dd = part; dd < d; dd += 16)
          c = fmaf(sU[dd] * sK[t * DP + dd], sQ[t * DP + dd], c);
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) c += __shfl_xor(c, off, WAVE);
        if (part == 0) sC[t] = c;
      }
      __syncthreads();
    }
    if (live) {
      for (int t = 0; t < nt; ++t) {
        const float vv = sV[t * dv + e];
        const float4* kq =
            reinterpret_cast<const float4*>(sK + t * DP + l * NR);
        const float4* qq =
            reinterpret_cast<const float4*>(sQ + t * DP + l * NR);
        const float4* aq =
            reinterpret_cast<const float4*>(sA + t * DP + l * NR);
        float o = 0.f;
#pragma unroll
        for (int i4 = 0; i4 < NR / 4; ++i4) {
          const float4 k4 = kq[i4];
          const float4 q4 = qq[i4];
          const float4 a4 = aq[i4];
          const float kk[4] = {k4.x, k4.y, k4.z, k4.w};
          const float q_[4] = {q4.x, q4.y, q4.z, q4.w};
          const float aa[4] = {a4.x, a4.y, a4.z, a4.w};
          float* Si = S + 4 * i4;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float kvp = kk[j] * vv;
            if (MODE == 0) {
              o = fmaf(Si[j], q_[j], o);
              Si[j] = fmaf(aa[j], Si[j], kvp);
            } else {
              Si[j] = fmaf(aa[j], Si[j], kvp);
              o = fmaf(Si[j], q_[j], o);
            }
          }
        }
        for (int off = LN >> 1; off > 0; off >>= 1)
          o += __shfl_xor(o, off, WAVE);
        if (MODE == 0) o = fmaf(vv, sC[t], o);
        if (l == 0) y[(row0 + t0 + t) * (long)inner + h * dv + e] = o;
      }
    }
  }
  if (live) {
#pragma unroll
    for (int i4 = 0; i4 < NR / 4; ++i4) {
      const int dd = l * NR + 4 * i4;
      if (vec4) {
        if (dd < d)
          *reinterpret_cast<float4*>(st + 4 * i4) =
              float4{S[4 * i4], S[4 * i4 + 1], S[4 * i4 + 2], S[4 * i4 + 3]};
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (dd + j < d) st[4 * i4 + j] = S[4 * i4 + j];
      }
    }
  }
}

// y [T, H*dv] fp32; q, k [T, H*d], v [T, H*dv] views (stride(1) == 1) in the
// activation format; lo [T, R] fp32 (stride(1) == 1); w2 [H*d, R], zb, bonus
// [H*d] fp32 (bonus empty in mode 1); state [slots, H, dv, d] fp32.
void decay_scan(torch::Tensor y, torch::Tensor q, torch::Tensor k,
                torch::Tensor v, torch::Tensor lo, torch::Tensor w2,
                torch::Tensor zb, torch::Tensor bonus, torch::Tensor state,
                torch::Tensor positions, torch::Tensor cu_rows,
                torch::Tensor state_slots, int64_t H, int64_t d, int64_t dv,
                int64_t mode, double tau, double q_scale) {
  check_act(q, "q"); check_act(k, "k"); check_act(v, "v");
  check_f32(y, "y"); check_f32(zb, "zb"); check_f32(state, "state");
  check_i32(positions, "positions"); check_i32(cu_rows, "cu_rows");
  check_i32(state_slots, "state_slots");
  TORCH_CHECK(lo.is_cuda() && lo.scalar_type() == torch::kFloat32 &&
              lo.dim() == 2 && lo.stride(1) == 1, "lo must be fp32 rows");
  check_f32(w2, "w2");
  const int R = (int)lo.size(1);
  TORCH_CHECK(R >= 1 && w2.dim() == 2 && w2.size(0) == H * d &&
              w2.size(1) == R);
  TORCH_CHECK(mode == 0 || mode == 1);
  const long rows = q.size(0);
  TORCH_CHECK(q.dim() == 2 && k.dim() == 2 && v.dim() == 2 &&
              q.stride(1) == 1 && k.stride(1) == 1 && v.stride(1) == 1);
  TORCH_CHECK(q.size(1) == H * d && k.size(1) == H * d && v.size(1) == H * dv &&
              k.size(0) == rows && v.size(0) == rows && lo.size(0) == rows);
  TORCH_CHECK(k.scalar_type() == q.scalar_type() &&
              v.scalar_type() == q.scalar_type());
  TORCH_CHECK(y.dim() == 2 && y.size(0) == rows && y.size(1) == H * dv);
  TORCH_CHECK(zb.numel() == H * d);
  if (mode == 0) {
    check_f32(bonus, "bonus");
    TORCH_CHECK(bonus.numel() == H * d);
  } else {
    TORCH_CHECK(tau > 0.0);
  }
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == dv &&
              state.size(3) == d);
  TORCH_CHECK(positions.numel() == rows);
  const long nseq = cu_rows.numel() - 1;
  TORCH_CHECK(nseq >= 0 && state_slots.numel() >= nseq);
  TORCH_CHECK(dv >= 1 && dv <= 1024 && d >= 1);
  if (rows == 0 || nseq == 0) return;
  // lanes per column: enough that a thread holds at most 32 state rows,
  // more while the workgroup stays within 256 threads
  int LN = 1;
  while ((d + LN - 1) / LN > 32) LN *= 2;
  while (LN < 64 && dv * LN * 2 <= 256 && (d + LN - 1) / LN > 4) LN *= 2;
  TORCH_CHECK(LN <= 64 && dv * LN <= 1024,
              "head sizes exceed one workgroup");
  const int need = (int)((d + LN - 1) / LN);
  const int NR = need <= 4 ? 4 : need <= 8 ? 8 : need <= 16 ? 16 : 32;
  const int threads = (int)((dv * LN + 63) / 64 * 64);
  const size_t shmem = ((size_t)DS_TT * (3 * LN * NR + dv + R + 1) +
                        (size_t)d * (R + 2)) * sizeof(float);
  TORCH_CHECK(shmem <= 64 * 1024, "head sizes exceed the staging buffers");
  auto stream = c10::hip::getCurrentHIPStream().stream();
  dim3 grid((unsigned)nseq, (unsigned)H);
#define KK_ARGS y.data_ptr<float>(), reinterpret_cast<const T*>(q.data_ptr()),    \
        (long)q.stride(0), reinterpret_cast<const T*>(k.data_ptr()),              \
        (long)k.stride(0), reinterpret_cast<const T*>(v.data_ptr()),              \
        (long)v.stride(0), lo.data_ptr<float>(), (long)lo.stride(0), R,           \
        w2.data_ptr<float>(), zb.data_ptr<float>(),                               \
        mode == 0 ? bonus.data_ptr<float>() : nullptr,                            \
        state.data_ptr<float>(), positions.data_ptr<int>(),                       \
        cu_rows.data_ptr<int>(), state_slots.data_ptr<int>(), (int)H, (int)d,     \
        (int)dv, LN, (float)(1.0 / (mode == 0 ? 1.0 : tau)), (float)q_scale
#define KK_LAUNCH(NR_, MODE_)                                                     \
  {                                                                               \
    auto kern = decay_scan_kernel<T, NR_, MODE_>;                                 \
    static size_t allowed = 48 * 1024;                                            \
    if (shmem > allowed) {                                                        \
      hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                    \
                          hipFuncAttributeMaxDynamicSharedMemorySize,             \
                          (int)shmem);                                            \
      allowed = shmem;                                                            \
    }                                                                             \
    kern<<<grid, threads, shmem, stream>>>(KK_ARGS);                              \
  }
#define KK_BY_NR(MODE_)                                                           \
  switch (NR) {                                                                   \
    case 4: KK_LAUNCH(4, MODE_) break;                                            \
    case 8: KK_LAUNCH(8, MODE_) break;                                            \
    case 16: KK_LAUNCH(16, MODE_) break;                                          \
    default: KK_LAUNCH(32, MODE_)                                                 \
  }
  KK_DISPATCH_ACT(q, {
    if (mode == 0) { KK_BY_NR(0) } else { KK_BY_NR(1) }
  });
#undef KK_BY_NR
#undef KK_LAUNCH
#undef KK_ARGS
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
