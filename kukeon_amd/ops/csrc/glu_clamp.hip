// Clamped gated activation for a fused [.. gate .. up ..] projection row:
//   g = min(gate + bg, limit), u = clamp(up + bu, -limit, limit)
//   y = g * sigmoid(alpha * g) * (u + up_shift)
// The projection biases are added here (in fp32) instead of in the GEMM.
// Also the gelu-gated product of a dense gated layer (tanh form of gelu).
#include "elem.h"

namespace kukeon {

template <typename T>
__global__ __launch_bounds__(256) void clamp_glu_kernel(
    T* __restrict__ out, long ldo, const T* __restrict__ gate,
    const T* __restrict__ up, long ldg, const float* __restrict__ bg,
    const float* __restrict__ bu, float limit, float alpha, float up_shift,
    int F, long total) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const long r = idx / F;
  const int f = (int)(idx - r * F);
  float g = ldf(gate + r * ldg + f) + (bg ? bg[f] : 0.f);
  float u = ldf(up + r * ldg + f) + (bu ? bu[f] : 0.f);
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  const float sg = 1.0f / (1.0f + expf(-alpha * g));
  stf(out + r * ldo + f, g * sg * (u + up_shift));
}

template <typename T>
__global__ __launch_bounds__(256) void clamp_glu_vec_kernel(
    T* __restrict__ out, long ldo, const T* __restrict__ gate,
    const T* __restrict__ up, long ldg, const float* __restrict__ bg,
    const float* __restrict__ bu, float limit, float alpha, float up_shift,
    int F8, long total8) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total8) return;
  const long r = idx / F8;
  const int f = (int)(idx - r * F8) * 8;
  float g[8], u[8], y[8];
  ld8(gate + r * ldg + f, g);
  ld8(up + r * ldg + f, u);
  if (bg) {
    float t[8], s[8];
    ld8(bg + f, t);
    ld8(bu + f, s);
#pragma unroll
    for (int k = 0; k < 8; ++k) { g[k] += t[k]; u[k] += s[k]; }
  }
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const float gg = fminf(g[k], limit);
    const float uu = fminf(fmaxf(u[k], -limit), limit);
    y[k] = gg * (1.0f / (1.0f + expf(-alpha * gg))) * (uu + up_shift);
  }
  st8(out + r * ldo + f, y);
}

// out [T,F] view (stride(1)==1); gate, up [T,F] views into one projection
// buffer sharing a row stride; bg, bu [F] fp32 or empty.
void clamp_glu(torch::Tensor out, torch::Tensor gate, torch::Tensor up,
               torch::Tensor bg, torch::Tensor bu, double limit, double alpha,
               double up_shift) {
  check_act(out, "out");
  TORCH_CHECK(gate.scalar_type() == out.scalar_type() &&
              up.scalar_type() == out.scalar_type());
  TORCH_CHECK(out.dim() == 2 && gate.dim() == 2 && up.dim() == 2);
  const long rows = out.size(0);
  const int F = (int)out.size(1);
  TORCH_CHECK(gate.size(0) == rows && up.size(0) == rows &&
              gate.size(1) == F && up.size(1) == F);
  TORCH_CHECK(out.stride(1) == 1 && gate.stride(1) == 1 &&
              up.stride(1) == 1 && gate.stride(0) == up.stride(0));
  const bool hb = bg.numel() > 0;
  if (hb) {
    check_f32(bg, "bg");
    check_f32(bu, "bu");
    TORCH_CHECK(bg.numel() == F && bu.numel() == F);
  }
  const long total = rows * F;
  if (total == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  if (F % 8 == 0 && out.stride(0) % 8 == 0 && gate.stride(0) % 8 == 0 &&
      aligned16(out.data_ptr()) && aligned16(gate.data_ptr()) &&
      aligned16(up.data_ptr()) &&
      (!hb || (aligned16(bg.data_ptr()) && aligned16(bu.data_ptr())))) {
    const long total8 = total / 8;
    KK_DISPATCH_ACT(out, {
      clamp_glu_vec_kernel<T><<<dim3((unsigned)((total8 + 255) / 256)), 256,
                                0, stream>>>(
          reinterpret_cast<T*>(out.data_ptr()), out.stride(0),
          reinterpret_cast<const T*>(gate.data_ptr()),
          reinterpret_cast<const T*>(up.data_ptr()), gate.stride(0),
          hb ? bg.data_ptr<float>() : nullptr,
          hb ? bu.data_ptr<float>() : nullptr, (float)limit, (float)alpha,
          (float)up_shift, F / 8, total8);
    });
    HIP_CHECK_KERNEL();
    return;
  }
  KK_DISPATCH_ACT(out, {
    clamp_glu_kernel<T><<<dim3((unsigned)((total + 255) / 256)), 256, 0,
                          stream>>>(
        reinterpret_cast<T*>(out.data_ptr()), out.stride(0),
        reinterpret_cast<const T*>(gate.data_ptr()),
        reinterpret_cast<const T*>(up.data_ptr()), gate.stride(0),
        hb ? bg.data_ptr<float>() : nullptr,
        hb ? bu.data_ptr<float>() : nullptr, (float)limit, (float)alpha,
        (float)up_shift, F, total);
  });
  HIP_CHECK_KERNEL();
}

// ---- gelu-gated product: out = gelu_tanh(gate) * up ------------------------
DEV_INLINE float gelu_tanh_f(float g) {
  return 0.5f * g *
         (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
}

template <typename T>
__global__ __launch_bounds__(256) void gelu_glu_kernel(
    T* __restrict__ out, long ldo, const T* __restrict__ gate,
    const T* __restrict__ up, long ldg, int F, long total) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const long r = idx / F;
  const int f = (int)(idx - r * F);
  stf(out + r * ldo + f,
      gelu_tanh_f(ldf(gate + r * ldg + f)) * ldf(up + r * ldg + f));
}

template <typename T>
__global__ __launch_bounds__(256) void gelu_glu_vec_kernel(
    T* __restrict__ out, long ldo, const T* __restrict__ gate,
    const T* __restrict__ up, long ldg, int F8, long total8) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total8) return;
  const long r = idx / F8;
  const int f = (int)(idx - r * F8) * 8;
  float g[8], u[8], y[8];
  ld8(gate + r * ldg + f, g);
  ld8(up + r * ldg + f, u);
#pragma unroll
  for (int k = 0; k < 8; ++k) y[k] = gelu_tanh_f(g[k]) * u[k];
  st8(out + r * ldo + f, y);
}

// out [T,F] (stride(1)==1); gate, up [T,F] views into one projection buffer
// sharing a row stride.
void gelu_glu(torch::Tensor out, torch::Tensor gate, torch::Tensor up) {
  check_act(out, "out");
  TORCH_CHECK(gate.scalar_type() == out.scalar_type() &&
              up.scalar_type() == out.scalar_type());
  TORCH_CHECK(out.dim() == 2 && gate.dim() == 2 && up.dim() == 2);
  const long rows = out.size(0);
  const int F = (int)out.size(1);
  TORCH_CHECK(gate.size(0) == rows && up.size(0) == rows &&
              gate.size(1) == F && up.size(1) == F);
  TORCH_CHECK(out.stride(1) == 1 && gate.stride(1) == 1 &&
              up.stride(1) == 1 && gate.stride(0) == up.stride(0));
  const long total = rows * F;
  if (total == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  if (F % 8 == 0 && out.stride(0) % 8 == 0 && gate.stride(0) % 8 == 0 &&
      aligned16(out.data_ptr()) && aligned16(gate.data_ptr()) &&
      aligned16(up.data_ptr())) {
    const long total8 = total / 8;
    KK_DISPATCH_ACT(out, {
      gelu_glu_vec_kernel<T><<<dim3((unsigned)((total8 + 255) / 256)), 256, 0,
                               stream>>>(
          reinterpret_cast<T*>(out.data_ptr()), out.stride(0),
          reinterpret_cast<const T*>(gate.data_ptr()),
          reinterpret_cast<const T*>(up.data_ptr()), gate.stride(0), F / 8,
          total8);
    });
    HIP_CHECK_KERNEL();
    return;
  }
  KK_DISPATCH_ACT(out, {
    gelu_glu_kernel<T><<<dim3((unsigned)((total + 255) / 256)), 256, 0,
                         stream>>>(
        reinterpret_cast<T*>(out.data_ptr()), out.stride(0),
        reinterpret_cast<const T*>(gate.data_ptr()),
        reinterpret_cast<const T*>(up.data_ptr()), gate.stride(0), F, total);
  });
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
