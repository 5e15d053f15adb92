// Linear attention with a fixed decay per head, the recurrent form:
//   q_t, k_t, v_t = silu of the projection columns (fp32 from here on)
//   S_t = decay_h S_(t-1) + k_t v_t^T                      (S: d x dv)
//   y_t = S_t^T q_t
// One workgroup per (sequence, head). The state stays in registers for the
// whole portion: thread (e, l) owns the NR consecutive rows
// l NR .. l NR + NR - 1 of column e, so a step is 2 NR fused multiply-adds
// per thread plus a reduction over the LN neighbouring lanes. q, k and v of
// TT tokens are staged in LDS at a time, q and k padded with zeros to LN NR
// entries, which keeps state rows past d at zero. The slot holds S^T
// ([H, dv, d]) so that a thread's rows are one contiguous run; it is read
// once at the start of the portion (zeros at position 0, whatever the slot
// held) and written once at its end. Tokens are visited in order, so a
// position's result does not depend on how the sequence was cut.
//
// gated_rmsnorm: out = y / rms(y) * w * sigmoid(gate), the norm over the
// whole row (all heads together).
#include "elem.h"

namespace kukeon {

#define LT_TT 16

DEV_INLINE float silu_x(float v) { return v / (1.0f + expf(-v)); }

template <typename T, int NR>
__global__ __launch_bounds__(1024) void lightning_scan_kernel(
    float* __restrict__ y, const T* __restrict__ proj, long ldp, long q_col,
    long k_col, long v_col, const float* __restrict__ decay,
    float* __restrict__ state, const int* __restrict__ positions,
    const int* __restrict__ cu_rows, const int* __restrict__ state_slots,
    int H, int d, int dv, int LN) {
  extern __shared__ float sm[];
  const int DP = LN * NR;               // padded q / k row
  float* sQ = sm;                       // [TT][DP]
  float* sK = sQ + LT_TT * DP;          // [TT][DP]
  float* sV = sK + LT_TT * DP;          // [TT][dv]
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
  const int e = tid / LN;
  const int l = tid - e * LN;
  const bool live = e < dv;
  float* st = state + (((long)state_slots[s] * H + h) * dv + (live ? e : 0)) *
                          (long)d + l * NR;
  // whole 16-byte pieces of the slot when the rows allow it
  const bool vec4 = (d & 3) == 0;
  float S[NR];
#pragma unroll
  for (int i4 = 0; i4 < NR / 4; ++i4) {
    const int dd = l * NR + 4 * i4;
    float4 v = float4{0.f, 0.f, 0.f, 0.f};
    if (live && p0 > 0) {
      if (vec4) {
        if (dd < d) v = *reinterpret_cast<const float4*>(st + 4 * i4);
      } else {
        if (dd + 0 < d) v.x = st[4 * i4 + 0];
        if (dd + 1 < d) v.y = st[4 * i4 + 1];
        if (dd + 2 < d) v.z = st[4 * i4 + 2];
        if (dd + 3 < d) v.w = st[4 * i4 + 3];
      }
    }
    S[4 * i4 + 0] = v.x; S[4 * i4 + 1] = v.y;
    S[4 * i4 + 2] = v.z; S[4 * i4 + 3] = v.w;
  }
  const float a = decay[h];
  for (int t0 = 0; t0 < n; t0 += LT_TT) {
    const int nt = min(LT_TT, n - t0);
    __syncthreads();
    for (int i = tid; i < nt * DP; i += nthreads) {
      const int t = i / DP, dd = i - t * DP;
      const T* row = proj + (row0 + t0 + t) * ldp;
      sQ[i] = dd < d ? silu_x(ldf(row + q_col + (long)h * d + dd)) : 0.f;
      sK[i] = dd < d ? silu_x(ldf(row + k_col + (long)h * d + dd)) : 0.f;
    }
    for (int i = tid; i < nt * dv; i += nthreads) {
      const int t = i / dv, ee = i - t * dv;
      const T* row = proj + (row0 + t0 + t) * ldp;
      sV[i] = silu_x(ldf(row + v_col + (long)h * dv + ee));
    }
    __syncthreads();
    if (live) {
      for (int t = 0; t < nt; ++t) {
        const float v = sV[t * dv + e];
        const float4* kq =
            reinterpret_cast<const float4*>(sK + t * DP + l * NR);
        const float4* qq =
            reinterpret_cast<const float4*>(sQ + t * DP + l * NR);
        float o = 0.f;
#pragma unroll
        for (int i4 = 0; i4 < NR / 4; ++i4) {
          const float4 k4 = kq[i4];
          const float4 q4 = qq[i4];
          float* Si = S + 4 * i4;
          Si[0] = fmaf(a, Si[0], k4.x * v); o = fmaf(Si[0], q4.x, o);
          Si[1] = fmaf(a, Si[1], k4.y * v); o = fmaf(Si[1], q4.y, o);
          Si[2] = fmaf(a, Si[2], k4.z * v); o = fmaf(Si[2], q4.z, o);
          Si[3] = fmaf(a, Si[3], k4.w * v); o = fmaf(Si[3], q4.w, o);
        }
        for (int off = LN >> 1; off > 0; off >>= 1)
          o += __shfl_xor(o, off, WAVE);
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

// y [T, H*dv] fp32; proj [T, cols] activation format; state
// [slots, H, dv, d] fp32; decay [H] fp32.
void lightning_scan(torch::Tensor y, torch::Tensor proj, int64_t q_col,
                    int64_t k_col, int64_t v_col, torch::Tensor decay,
                    torch::Tensor state, torch::Tensor positions,
                    torch::Tensor cu_rows, torch::Tensor state_slots,
                    int64_t H, int64_t d, int64_t dv) {
  check_act(proj, "proj");
  check_f32(y, "y"); check_f32(decay, "decay"); check_f32(state, "state");
  check_i32(positions, "positions"); check_i32(cu_rows, "cu_rows");
  check_i32(state_slots, "state_slots");
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1);
  const long rows = proj.size(0);
  TORCH_CHECK(y.dim() == 2 && y.size(0) == rows && y.size(1) == H * dv);
  TORCH_CHECK(decay.numel() == H);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == dv &&
              state.size(3) == d);
  TORCH_CHECK(q_col >= 0 && q_col + H * d <= proj.size(1) && k_col >= 0 &&
              k_col + H * d <= proj.size(1) && v_col >= 0 &&
              v_col + H * dv <= proj.size(1));
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
  const size_t shmem = (size_t)LT_TT * (2 * LN * NR + dv) * sizeof(float);
  auto stream = c10::hip::getCurrentHIPStream().stream();
  dim3 grid((unsigned)nseq, (unsigned)H);
#define KK_ARGS y.data_ptr<float>(), reinterpret_cast<const T*>(proj.data_ptr()), \
        (long)proj.stride(0), (long)q_col, (long)k_col, (long)v_col,            \
        decay.data_ptr<float>(), state.data_ptr<float>(),                        \
        positions.data_ptr<int>(), cu_rows.data_ptr<int>(),                      \
        state_slots.data_ptr<int>(), (int)H, (int)d, (int)dv, LN
  KK_DISPATCH_ACT(proj, {
    switch (NR) {
      case 4:
        lightning_scan_kernel<T, 4><<<grid, threads, shmem, stream>>>(KK_ARGS);
        break;
      case 8:
        lightning_scan_kernel<T, 8><<<grid, threads, shmem, stream>>>(KK_ARGS);
        break;
      case 16:
        lightning_scan_kernel<T, 16><<<grid, threads, shmem, stream>>>(KK_ARGS);
        break;
      default:
        lightning_scan_kernel<T, 32><<<grid, threads, shmem, stream>>>(KK_ARGS);
    }
  });
#undef KK_ARGS
  HIP_CHECK_KERNEL();
}

// One block per row.
template <typename T>
__global__ __launch_bounds__(256) void gated_rmsnorm_kernel(
    T* __restrict__ out, const float* __restrict__ y, const T* __restrict__ g,
    long ldg, const float* __restrict__ w, float eps, int C) {
  __shared__ float red[32];
  const long row = blockIdx.x;
  const float* yr = y + row * (long)C;
  const T* gr = g + row * ldg;
  float ss = 0.f;
  for (int i = threadIdx.x; i < C; i += blockDim.x) ss += yr[i] * yr[i];
  const float rs = 1.0f / sqrtf(block_sum2(ss, 0.f, red).x / (float)C + eps);
  T* orow = out + row * (long)C;
  for (int i = threadIdx.x; i < C; i += blockDim.x)
    stf(orow + i, yr[i] * rs * w[i] / (1.0f + expf(-ldf(gr + i))));
}

template <typename T, int NIT>
__global__ __launch_bounds__(256) void gated_rmsnorm_vec_kernel(
    T* __restrict__ out, const float* __restrict__ y, const T* __restrict__ g,
    long ldg, const float* __restrict__ w, float eps, int C) {
  __shared__ float red[32];
  const long row = blockIdx.x;
  const float* yr = y + row * (long)C;
  const T* gr = g + row * ldg;
  float v[NIT][8];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int i = (it * 256 + threadIdx.x) * 8;
    if (i < C) {
      ld8(yr + i, v[it]);
#pragma unroll
      for (int k = 0; k < 8; ++k) ss += v[it][k] * v[it][k];
    }
  }
  const float rs = 1.0f / sqrtf(block_sum2(ss, 0.f, red).x / (float)C + eps);
  T* orow = out + row * (long)C;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int i = (it * 256 + threadIdx.x) * 8;
    if (i < C) {
      float t[8], gg[8], o[8];
      ld8(w + i, t);
      ld8(gr + i, gg);
#pragma unroll
      for (int k = 0; k < 8; ++k)
        o[k] = v[it][k] * rs * t[k] / (1.0f + expf(-gg[k]));
      st8(orow + i, o);
    }
  }
}

// out [T,C] activation format; y [T,C] fp32; gate [T,C] view (stride(1)==1)
// in the activation format; w [C] fp32.
void gated_rmsnorm(torch::Tensor out, torch::Tensor y, torch::Tensor gate,
                   torch::Tensor w, double eps) {
  check_act(out, "out"); check_act(gate, "gate");
  check_f32(y, "y"); check_f32(w, "w");
  TORCH_CHECK(out.dim() == 2 && out.is_contiguous() && y.dim() == 2);
  const long rows = y.size(0);
  const int C = (int)y.size(1);
  TORCH_CHECK(out.size(0) == rows && out.size(1) == C && w.numel() == C);
  TORCH_CHECK(gate.dim() == 2 && gate.size(0) == rows && gate.size(1) == C &&
              gate.stride(1) == 1 && gate.scalar_type() == out.scalar_type());
  if (rows == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  dim3 grid((unsigned)rows);
  const bool vec = C % 8 == 0 && C <= 8 * 256 * 4 && gate.stride(0) % 8 == 0 &&
                   aligned16(out.data_ptr()) && aligned16(y.data_ptr()) &&
                   aligned16(gate.data_ptr()) && aligned16(w.data_ptr());
#define KK_ARGS reinterpret_cast<T*>(out.data_ptr()), y.data_ptr<float>(),      \
        reinterpret_cast<const T*>(gate.data_ptr()), (long)gate.stride(0),      \
        w.data_ptr<float>(), (float)eps, C
  KK_DISPATCH_ACT(out, {
    if (!vec)
      gated_rmsnorm_kernel<T><<<grid, 256, 0, stream>>>(KK_ARGS);
    else if (C <= 2048)
      gated_rmsnorm_vec_kernel<T, 1><<<grid, 256, 0, stream>>>(KK_ARGS);
    else if (C <= 4096)
      gated_rmsnorm_vec_kernel<T, 2><<<grid, 256, 0, stream>>>(KK_ARGS);
    else
      gated_rmsnorm_vec_kernel<T, 4><<<grid, 256, 0, stream>>>(KK_ARGS);
  });
#undef KK_ARGS
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
