// Layer norm (mean taken off, a weight, no bias) on the OUTPUT side of a
// sublayer, over an fp32 residual stream:
//   layernorm_residual  x += (y - mean(y)) / sqrt(var(y) + eps) * w ;
//                       out = x in the activation format (the next sublayer
//                       reads the stream itself)
//   layernorm           out = (x - mean(x)) / sqrt(var(x) + eps) * w
// The variance is the mean of the squared deviations, taken in a second pass
// over values that stay in registers. One block per row; all sums fp32, in a
// fixed order.
#include "elem.h"

namespace kukeon {

template <typename TI, typename TO, bool RESID>
__global__ __launch_bounds__(256) void layernorm_kernel(
    float* __restrict__ x, const TI* __restrict__ src, long lds,
    const float* __restrict__ w, float eps, TO* __restrict__ out, int W) {
  __shared__ float red[32];
  const long row = blockIdx.x;
  const TI* sr = src + row * lds;
  float s = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) s += ldf(sr + i);
  const float mean = block_sum2(s, 0.f, red).x / (float)W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float d = ldf(sr + i) - mean;
    ss += d * d;
  }
  const float rs = 1.0f / sqrtf(block_sum2(ss, 0.f, red).x / (float)W + eps);
  TO* orow = out + row * (long)W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = (ldf(sr + i) - mean) * rs * w[i];
    if (RESID) {
      v += x[row * (long)W + i];
      x[row * (long)W + i] = v;
    }
    stf(orow + i, v);
  }
}

// Vector form: W a multiple of 8, at most 8 * 256 * NIT entries.
template <typename TI, typename TO, bool RESID, int NIT>
__global__ __launch_bounds__(256) void layernorm_vec_kernel(
    float* __restrict__ x, const TI* __restrict__ src, long lds,
    const float* __restrict__ w, float eps, TO* __restrict__ out, int W) {
  __shared__ float red[32];
  const long row = blockIdx.x;
  const TI* sr = src + row * lds;
  float v[NIT][8];
  float s = 0.f;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int i = (it * 256 + threadIdx.x) * 8;
    if (i < W) {
      ld8(sr + i, v[it]);
#pragma unroll
      for (int k = 0; k < 8; ++k) s += v[it][k];
    }
  }
  const float mean = block_sum2(s, 0.f, red).x / (float)W;
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int i = (it * 256 + threadIdx.x) * 8;
    if (i < W) {
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        v[it][k] -= mean;
        ss += v[it][k] * v[it][k];
      }
    }
  }
  const float rs = 1.0f / sqrtf(block_sum2(ss, 0.f, red).x / (float)W + eps);
  TO* orow = out + row * (long)W;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int i = (it * 256 + threadIdx.x) * 8;
    if (i < W) {
      float t[8];
      ld8(w + i, t);
#pragma unroll
      for (int k = 0; k < 8; ++k) v[it][k] = v[it][k] * rs * t[k];
      if (RESID) {
        float xv[8];
        ld8(x + row * (long)W + i, xv);
#pragma unroll
        for (int k = 0; k < 8; ++k) v[it][k] += xv[k];
        st8(x + row * (long)W + i, v[it]);
      }
      st8(orow + i, v[it]);
    }
  }
}

template <typename TI, typename TO, bool RESID>
static void launch_layernorm(float* x, const TI* src, long lds, const float* w,
                             float eps, TO* out, int W, long rows, bool vec,
                             hipStream_t stream) {
  dim3 grid((unsigned)rows);
  if (!vec)
    layernorm_kernel<TI, TO, RESID><<<grid, 256, 0, stream>>>(x, src, lds, w,
                                                              eps, out, W);
  else if (W <= 2048)
    layernorm_vec_kernel<TI, TO, RESID, 1><<<grid, 256, 0, stream>>>(
        x, src, lds, w, eps, out, W);
  else if (W <= 4096)
    layernorm_vec_kernel<TI, TO, RESID, 2><<<grid, 256, 0, stream>>>(
        x, src, lds, w, eps, out, W);
  else
    layernorm_vec_kernel<TI, TO, RESID, 4><<<grid, 256, 0, stream>>>(
        x, src, lds, w, eps, out, W);
}

// x [T,W] fp32 (in/out); y [T,>=W] rows of stride y.stride(0) in the
// activation format; w [W] fp32; out [T,W] activation format.
void layernorm_residual(torch::Tensor x, torch::Tensor y, torch::Tensor w,
                        double eps, torch::Tensor out) {
  check_f32(x, "x");
  check_f32(w, "w");
  check_act(out, "out");
  check_act(y, "y");
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.is_contiguous());
  const long rows = x.size(0);
  const int W = (int)x.size(1);
  TORCH_CHECK(out.size(0) == rows && out.size(1) == W && w.numel() == W);
  TORCH_CHECK(y.scalar_type() == out.scalar_type() && y.dim() == 2 &&
              y.size(0) == rows && y.size(1) >= W && y.stride(1) == 1);
  if (rows == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool vec = W % 8 == 0 && W <= 8 * 256 * 4 && aligned16(x.data_ptr()) &&
                   aligned16(out.data_ptr()) && aligned16(w.data_ptr()) &&
                   y.stride(0) % 8 == 0 && aligned16(y.data_ptr());
  KK_DISPATCH_ACT(out, {
    launch_layernorm<T, T, true>(
        x.data_ptr<float>(), reinterpret_cast<const T*>(y.data_ptr()),
        (long)y.stride(0), w.data_ptr<float>(), (float)eps,
        reinterpret_cast<T*>(out.data_ptr()), W, rows, vec, stream);
  });
  HIP_CHECK_KERNEL();
}

// x [T,W] fp32; w [W] fp32; out [T,W] activation format.
void layernorm(torch::Tensor out, torch::Tensor x, torch::Tensor w,
               double eps) {
  check_f32(x, "x");
  check_f32(w, "w");
  check_act(out, "out");
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.is_contiguous());
  const long rows = x.size(0);
  const int W = (int)x.size(1);
  TORCH_CHECK(out.size(0) == rows && out.size(1) == W && w.numel() == W);
  if (rows == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool vec = W % 8 == 0 && W <= 8 * 256 * 4 && aligned16(x.data_ptr()) &&
                   aligned16(out.data_ptr()) && aligned16(w.data_ptr());
  KK_DISPATCH_ACT(out, {
    launch_layernorm<float, T, false>(
        nullptr, x.data_ptr<float>(), (long)W, w.data_ptr<float>(), (float)eps,
        reinterpret_cast<T*>(out.data_ptr()), W, rows, vec, stream);
  });
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
