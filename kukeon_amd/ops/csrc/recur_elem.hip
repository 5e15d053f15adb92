// Small per-row and per-element kernels of the recurrent / latent group:
//   gated_group_rmsnorm  out = rmsnorm_by_part(y * silu(z)) * w
//   head_gate            out[t, h, :] = o[h, t, :] * sigmoid(gate[t, h]), or
//                        entry by entry with a gate of H*dv columns
//   xielu                piecewise quadratic / exponential activation
//   softcap_             logits <- cap * tanh(logits / cap)
#include "elem.h"

namespace kukeon {

DEV_INLINE float silu_f(float v) { return v / (1.0f + __expf(-v)); }

// One block per (row, part): the gate comes BEFORE the norm, each part is
// divided by its own root mean square.
template <typename T>
__global__ __launch_bounds__(256) void gated_group_rmsnorm_kernel(
    T* __restrict__ out, const float* __restrict__ y, const T* __restrict__ z,
    long ldz, const float* __restrict__ w, float eps, int C, int parts) {
  __shared__ float red[32];
  const long row = blockIdx.x;
  const int part = blockIdx.y;
  const int Cp = C / parts;
  const int c0 = part * Cp;
  const float* yr = y + row * (long)C + c0;
  const T* zr = z + row * ldz + c0;
  float ss = 0.f;
  for (int i = threadIdx.x; i < Cp; i += blockDim.x) {
    const float v = yr[i] * silu_f(ldf(zr + i));
    ss += v * v;
  }
  const float2 tot = block_sum2(ss, 0.f, red);
  const float rs = 1.0f / sqrtf(tot.x / (float)Cp + eps);
  T* orow = out + row * (long)C + c0;
  for (int i = threadIdx.x; i < Cp; i += blockDim.x) {
    const float v = yr[i] * silu_f(ldf(zr + i));
    stf(orow + i, v * rs * w[c0 + i]);
  }
}

// Vector form: a part of at most 8 * 256 * NIT entries, a multiple of 8; the
// gated values stay in registers between the two passes.
template <typename T, int NIT>
__global__ __launch_bounds__(256) void gated_group_rmsnorm_vec_kernel(
    T* __restrict__ out, const float* __restrict__ y, const T* __restrict__ z,
    long ldz, const float* __restrict__ w, float eps, int C, int parts) {
  __shared__ float red[32];
  const long row = blockIdx.x;
  const int part = blockIdx.y;
  const int Cp = C / parts;
  const int c0 = part * Cp;
  const float* yr = y + row * (long)C + c0;
  const T* zr = z + row * ldz + c0;
  float v[NIT][8];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int i = (it * 256 + threadIdx.x) * 8;
    if (i < Cp) {
      float g[8];
      ld8(yr + i, v[it]);
      ld8(zr + i, g);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        v[it][k] *= silu_f(g[k]);
        ss += v[it][k] * v[it][k];
      }
    }
  }
  const float2 tot = block_sum2(ss, 0.f, red);
  const float rs = 1.0f / sqrtf(tot.x / (float)Cp + eps);
  T* orow = out + row * (long)C + c0;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int i = (it * 256 + threadIdx.x) * 8;
    if (i < Cp) {
      float t[8], o[8];
      ld8(w + c0 + i, t);
#pragma unroll
      for (int k = 0; k < 8; ++k) o[k] = v[it][k] * rs * t[k];
      st8(orow + i, o);
    }
  }
}

void gated_group_rmsnorm(torch::Tensor out, torch::Tensor y, torch::Tensor z,
                         torch::Tensor w, int64_t parts, double eps) {
  check_act(out, "out"); check_act(z, "z");
  check_f32(y, "y"); check_f32(w, "w");
  TORCH_CHECK(out.dim() == 2 && out.is_contiguous() && y.dim() == 2);
  const long rows = y.size(0);
  const int C = (int)y.size(1);
  TORCH_CHECK(out.size(0) == rows && out.size(1) == C && w.numel() == C);
  TORCH_CHECK(z.dim() == 2 && z.size(0) == rows && z.size(1) == C &&
              z.stride(1) == 1 && z.scalar_type() == out.scalar_type());
  TORCH_CHECK(parts >= 1 && C % parts == 0);
  if (rows == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  dim3 grid((unsigned)rows, (unsigned)parts);
  const int Cp = C / (int)parts;
  if (Cp % 8 == 0 && Cp <= 8 * 256 * 2 && z.stride(0) % 8 == 0 &&
      aligned16(out.data_ptr()) && aligned16(y.data_ptr()) &&
      aligned16(z.data_ptr()) && aligned16(w.data_ptr())) {
    KK_DISPATCH_ACT(out, {
      T* op = reinterpret_cast<T*>(out.data_ptr());
      const T* zp = reinterpret_cast<const T*>(z.data_ptr());
      if (Cp <= 2048)
        gated_group_rmsnorm_vec_kernel<T, 1><<<grid, 256, 0, stream>>>(
            op, y.data_ptr<float>(), zp, (long)z.stride(0),
            w.data_ptr<float>(), (float)eps, C, (int)parts);
      else
        gated_group_rmsnorm_vec_kernel<T, 2><<<grid, 256, 0, stream>>>(
            op, y.data_ptr<float>(), zp, (long)z.stride(0),
            w.data_ptr<float>(), (float)eps, C, (int)parts);
    });
    HIP_CHECK_KERNEL();
    return;
  }
  KK_DISPATCH_ACT(out, {
    gated_group_rmsnorm_kernel<T><<<grid, 256, 0, stream>>>(
        reinterpret_cast<T*>(out.data_ptr()), y.data_ptr<float>(),
        reinterpret_cast<const T*>(z.data_ptr()), (long)z.stride(0),
        w.data_ptr<float>(), (float)eps, C, (int)parts);
  });
  HIP_CHECK_KERNEL();
}

// gw: gate columns per head (1: one gate per head, dv: one per entry)
template <typename T>
__global__ __launch_bounds__(256) void head_gate_kernel(
    T* __restrict__ out, const T* __restrict__ o, const T* __restrict__ gate,
    long ldg, long rows, int H, int dv, int gw) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long total = rows * H * dv;
  if (i >= total) return;
  const int d = (int)(i % dv);
  const int h = (int)((i / dv) % H);
  const long t = i / ((long)dv * H);
  const long gc = gw == 1 ? h : (long)h * dv + d;
  const float g = 1.0f / (1.0f + __expf(-ldf(gate + t * ldg + gc)));
  stf(out + i, ldf(o + ((long)h * rows + t) * dv + d) * g);
}

// 8 values of one head at a time (dv a multiple of 8)
template <typename T>
__global__ __launch_bounds__(256) void head_gate_vec_kernel(
    T* __restrict__ out, const T* __restrict__ o, const T* __restrict__ gate,
    long ldg, long rows, int H, int dv, int gw) {
  const long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 8;
  const long total = rows * H * dv;
  if (i >= total) return;
  const int d = (int)(i % dv);
  const int h = (int)((i / dv) % H);
  const long t = i / ((long)dv * H);
  float v[8];
  ld8(o + ((long)h * rows + t) * dv + d, v);
  if (gw == 1) {
    const float g = 1.0f / (1.0f + __expf(-ldf(gate + t * ldg + h)));
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] *= g;
  } else {
    float g[8];
    ld8(gate + t * ldg + (long)h * dv + d, g);
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] *= 1.0f / (1.0f + expf(-g[k]));
  }
  st8(out + i, v);
}

// out [T, H*dv]; o [H, T, dv] contiguous; gate [T, H] or [T, H*dv] (any row
// stride).
void head_gate(torch::Tensor out, torch::Tensor o, torch::Tensor gate) {
  check_act(out, "out"); check_act(o, "o"); check_act(gate, "gate");
  TORCH_CHECK(o.dim() == 3 && o.is_contiguous() && out.is_contiguous());
  const long H = o.size(0), rows = o.size(1), dv = o.size(2);
  TORCH_CHECK(out.dim() == 2 && out.size(0) == rows && out.size(1) == H * dv);
  TORCH_CHECK(gate.dim() == 2 && gate.size(0) == rows &&
              (gate.size(1) == H || gate.size(1) == H * dv) &&
              gate.stride(1) == 1);
  const int gw = gate.size(1) == H ? 1 : (int)dv;
  TORCH_CHECK(o.scalar_type() == out.scalar_type() &&
              gate.scalar_type() == out.scalar_type());
  const long total = rows * H * dv;
  if (total == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  if (dv % 8 == 0 && aligned16(out.data_ptr()) && aligned16(o.data_ptr()) &&
      (gw == 1 || (gate.stride(0) % 8 == 0 && aligned16(gate.data_ptr())))) {
    KK_DISPATCH_ACT(out, {
      head_gate_vec_kernel<T><<<dim3((unsigned)((total / 8 + 255) / 256)), 256,
                                0, stream>>>(
          reinterpret_cast<T*>(out.data_ptr()),
          reinterpret_cast<const T*>(o.data_ptr()),
          reinterpret_cast<const T*>(gate.data_ptr()), (long)gate.stride(0),
          rows, (int)H, (int)dv, gw);
    });
    HIP_CHECK_KERNEL();
    return;
  }
  KK_DISPATCH_ACT(out, {
    head_gate_kernel<T><<<dim3((unsigned)((total + 255) / 256)), 256, 0,
                          stream>>>(
        reinterpret_cast<T*>(out.data_ptr()),
        reinterpret_cast<const T*>(o.data_ptr()),
        reinterpret_cast<const T*>(gate.data_ptr()), (long)gate.stride(0),
        rows, (int)H, (int)dv, gw);
  });
  HIP_CHECK_KERNEL();
}

// z > 0: ap z^2 + z/2;  z <= 0: aq (exp(z) - 1 - z) + z/2
template <typename T>
__global__ __launch_bounds__(256) void xielu_kernel(
    T* __restrict__ out, const T* __restrict__ z, long total, float ap,
    float aq) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const float v = ldf(z + i);
  const float r = v > 0.f ? fmaf(ap * v, v, 0.5f * v)
                          : fmaf(aq, expm1f(v) - v, 0.5f * v);
  stf(out + i, r);
}

template <typename T>
__global__ __launch_bounds__(256) void xielu_vec_kernel(
    T* __restrict__ out, const T* __restrict__ z, long total8, float ap,
    float aq) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total8) return;
  float v[8], r[8];
  ld8(z + i * 8, v);
#pragma unroll
  for (int k = 0; k < 8; ++k)
    r[k] = v[k] > 0.f ? fmaf(ap * v[k], v[k], 0.5f * v[k])
                      : fmaf(aq, expm1f(v[k]) - v[k], 0.5f * v[k]);
  st8(out + i * 8, r);
}

void xielu(torch::Tensor out, torch::Tensor z, double ap, double aq) {
  check_act(out, "out"); check_act(z, "z");
  TORCH_CHECK(out.is_contiguous() && z.is_contiguous() &&
              out.numel() == z.numel() &&
              out.scalar_type() == z.scalar_type());
  const long total = z.numel();
  if (total == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  if (total % 8 == 0 && aligned16(out.data_ptr()) && aligned16(z.data_ptr())) {
    const long total8 = total / 8;
    KK_DISPATCH_ACT(out, {
      xielu_vec_kernel<T><<<dim3((unsigned)((total8 + 255) / 256)), 256, 0,
                            stream>>>(
          reinterpret_cast<T*>(out.data_ptr()),
          reinterpret_cast<const T*>(z.data_ptr()), total8, (float)ap,
          (float)aq);
    });
    HIP_CHECK_KERNEL();
    return;
  }
  KK_DISPATCH_ACT(out, {
    xielu_kernel<T><<<dim3((unsigned)((total + 255) / 256)), 256, 0, stream>>>(
        reinterpret_cast<T*>(out.data_ptr()),
        reinterpret_cast<const T*>(z.data_ptr()), total, (float)ap, (float)aq);
  });
  HIP_CHECK_KERNEL();
}

__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ x,
                                                      long total, float cap) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  x[i] = cap * tanhf(x[i] / cap);
}

void softcap_(torch::Tensor logits, double cap) {
  check_f32(logits, "logits");
  const long total = logits.numel();
  if (total == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  softcap_kernel<<<dim3((unsigned)((total + 255) / 256)), 256, 0, stream>>>(
      logits.data_ptr<float>(), total, (float)cap);
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
