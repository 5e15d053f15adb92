// Grouped-query attention whose scores carry no positions: queries and keys
// are RMS-normed over their WHOLE projection row, scores are scaled and may
// be capped (cap tanh(score / cap)), and a query at position p sees the keys
// lo .. p, lo being the first position of p's chunk (0 without chunks). The
// same kernel serves a sliding window (lo = p - window + 1), a distance bias
// slope_h (p - j) taken off head h's scores, and caches without value rows,
// where the values are the keys (window_attention).
//
// qk_norm_append   norms q (and k) of every row, writes q to a dense buffer
//                  and k, v to the row's page.
// chunk_attention  one workgroup per (row, kv head, four of its query heads).
//                  Keys are taken 64 at a time counted from lo, tile t by
//                  wave t mod NW: lane j scores key j for all the heads from
//                  one read of the key row (the queries sit in LDS as fp32),
//                  the wave agrees on each head's running maximum and sum,
//                  then dv/8 lanes cover one value row with 16-byte loads
//                  while the 64/(dv/8) lane groups take every NG-th key; the
//                  groups' partial sums meet in LDS, added in group order,
//                  and the waves' results are folded in wave order.
//                  Everything is fp32; a row's result depends only on its
//                  own position and chunk.
#include "elem.h"

namespace kukeon {

// One block per row. k_cache [blocks, G, BS, d], v_cache [blocks, G, BS, dv]
// (null for a layer that reads another layer's pages).
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_append_kernel(
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const T* __restrict__ proj, long ldp, long q_col, long k_col, long v_col,
    const float* __restrict__ wq, const float* __restrict__ wk, float eps,
    const int* __restrict__ positions, const int* __restrict__ row_seq,
    const int* __restrict__ block_table, int max_blocks, int Cq, int G, int d,
    int dv, int BS) {
  __shared__ float red[32];
  const long r = blockIdx.x;
  const int p = positions[r];
  if (p < 0) return;
  const T* row = proj + r * ldp;
  const int Ck = k_cache ? G * d : 0;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < Cq; i += blockDim.x) {
    const float v = ldf(row + q_col + i);
    sq += v * v;
  }
  for (int i = threadIdx.x; i < Ck; i += blockDim.x) {
    const float v = ldf(row + k_col + i);
    sk += v * v;
  }
  const float2 tot = block_sum2(sq, sk, red);
  const float rq = 1.0f / sqrtf(tot.x / (float)Cq + eps);
  for (int i = threadIdx.x; i < Cq; i += blockDim.x)
    stf(q_out + r * (long)Cq + i, ldf(row + q_col + i) * rq * wq[i]);
  if (!k_cache) return;
  const float rk = 1.0f / sqrtf(tot.y / (float)Ck + eps);
  const int s = row_seq[r];
  const long blk = block_table[(long)s * max_blocks + p / BS];
  const int at = p % BS;
  for (int i = threadIdx.x; i < Ck; i += blockDim.x) {
    const int g = i / d, dd = i - g * d;
    stf(k_cache + ((blk * G + g) * BS + at) * (long)d + dd,
        ldf(row + k_col + i) * rk * wk[i]);
  }
  const int Cv = G * dv;
  for (int i = threadIdx.x; i < Cv; i += blockDim.x) {
    const int g = i / dv, dd = i - g * dv;
    v_cache[((blk * G + g) * BS + at) * (long)dv + dd] = row[v_col + i];
  }
}

// Vector form: 8 entries per thread and step; d, dv, the columns and the row
// stride are multiples of 8 and all rows 16-byte aligned, so that a piece of
// 8 never straddles two heads.
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_append_vec_kernel(
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const T* __restrict__ proj, long ldp, long q_col, long k_col, long v_col,
    const float* __restrict__ wq, const float* __restrict__ wk, float eps,
    const int* __restrict__ positions, const int* __restrict__ row_seq,
    const int* __restrict__ block_table, int max_blocks, int Cq, int G, int d,
    int dv, int BS) {
  __shared__ float red[32];
  const long r = blockIdx.x;
  const int p = positions[r];
  if (p < 0) return;
  const T* row = proj + r * ldp;
  const int Ck = k_cache ? G * d : 0;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x * 8; i < Cq; i += blockDim.x * 8) {
    float v[8];
    ld8(row + q_col + i, v);
#pragma unroll
    for (int k = 0; k < 8; ++k) sq += v[k] * v[k];
  }
  for (int i = threadIdx.x * 8; i < Ck; i += blockDim.x * 8) {
    float v[8];
    ld8(row + k_col + i, v);
#pragma unroll
    for (int k = 0; k < 8; ++k) sk += v[k] * v[k];
  }
  const float2 tot = block_sum2(sq, sk, red);
  const float rq = 1.0f / sqrtf(tot.x / (float)Cq + eps);
  for (int i = threadIdx.x * 8; i < Cq; i += blockDim.x * 8) {
    float v[8], w[8];
    ld8(row + q_col + i, v);
    ld8(wq + i, w);
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = v[k] * rq * w[k];
    st8(q_out + r * (long)Cq + i, v);
  }
  if (!k_cache) return;
  const float rk = 1.0f / sqrtf(tot.y / (float)Ck + eps);
  const int s = row_seq[r];
  const long blk = block_table[(long)s * max_blocks + p / BS];
  const int at = p % BS;
  for (int i = threadIdx.x * 8; i < Ck; i += blockDim.x * 8) {
    const int g = i / d, dd = i - g * d;
    float v[8], w[8];
    ld8(row + k_col + i, v);
    ld8(wk + i, w);
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = v[k] * rk * w[k];
    st8(k_cache + ((blk * G + g) * BS + at) * (long)d + dd, v);
  }
  const int Cv = G * dv;
  for (int i = threadIdx.x * 8; i < Cv; i += blockDim.x * 8) {
    const int g = i / dv, dd = i - g * dv;
    Raw8<T> v;
    v.load(row + v_col + i);
    *reinterpret_cast<Raw8<T>*>(v_cache +
                                ((blk * G + g) * BS + at) * (long)dv + dd) = v;
  }
}

void qk_norm_append(torch::Tensor q_out, torch::Tensor k_cache,
                    torch::Tensor v_cache, torch::Tensor proj, int64_t q_col,
                    int64_t k_col, int64_t v_col, torch::Tensor wq,
                    torch::Tensor wk, double eps, torch::Tensor positions,
                    torch::Tensor row_seq, torch::Tensor block_table) {
  check_act(proj, "proj");
  check_f32(wq, "wq");
  check_i32(positions, "positions"); check_i32(row_seq, "row_seq");
  check_i32(block_table, "block_table");
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1);
  const long rows = proj.size(0);
  const int Cq = (int)wq.numel();
  TORCH_CHECK(q_out.dim() == 2 && q_out.is_contiguous() &&
              q_out.size(0) == rows && q_out.size(1) == Cq &&
              q_out.scalar_type() == proj.scalar_type());
  TORCH_CHECK(q_col >= 0 && q_col + Cq <= proj.size(1));
  const bool own = k_cache.numel() > 0;
  int G = 0, d = 0, dv = 0, BS = 1;
  if (own) {
    check_f32(wk, "wk");
    TORCH_CHECK(k_cache.dim() == 4 && k_cache.is_contiguous() &&
                v_cache.dim() == 4 && v_cache.is_contiguous() &&
                k_cache.scalar_type() == proj.scalar_type() &&
                v_cache.scalar_type() == proj.scalar_type());
    G = (int)k_cache.size(1); BS = (int)k_cache.size(2);
    d = (int)k_cache.size(3); dv = (int)v_cache.size(3);
    TORCH_CHECK(v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == G &&
                v_cache.size(2) == BS);
    TORCH_CHECK(wk.numel() == (long)G * d);
    TORCH_CHECK(k_col >= 0 && k_col + (long)G * d <= proj.size(1) &&
                v_col >= 0 && v_col + (long)G * dv <= proj.size(1));
  }
  TORCH_CHECK(positions.numel() == rows && row_seq.numel() == rows);
  TORCH_CHECK(block_table.dim() == 2);
  if (rows == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool vec =
      Cq % 8 == 0 && q_col % 8 == 0 && proj.stride(0) % 8 == 0 &&
      aligned16(proj.data_ptr()) && aligned16(q_out.data_ptr()) &&
      aligned16(wq.data_ptr()) &&
      (!own || (d % 8 == 0 && dv % 8 == 0 && k_col % 8 == 0 &&
                v_col % 8 == 0 && aligned16(k_cache.data_ptr()) &&
                aligned16(v_cache.data_ptr()) && aligned16(wk.data_ptr())));
#define KK_ARGS reinterpret_cast<T*>(q_out.data_ptr()),                        \
        own ? reinterpret_cast<T*>(k_cache.data_ptr()) : nullptr,              \
        own ? reinterpret_cast<T*>(v_cache.data_ptr()) : nullptr,              \
        reinterpret_cast<const T*>(proj.data_ptr()), (long)proj.stride(0),     \
        (long)q_col, (long)k_col, (long)v_col, wq.data_ptr<float>(),           \
        own ? wk.data_ptr<float>() : nullptr, (float)eps,                      \
        positions.data_ptr<int>(), row_seq.data_ptr<int>(),                    \
        block_table.data_ptr<int>(), (int)block_table.size(1), Cq, G, d, dv,   \
        BS
  KK_DISPATCH_ACT(proj, {
    if (vec)
      qk_norm_append_vec_kernel<T><<<dim3((unsigned)rows), 256, 0, stream>>>(
          KK_ARGS);
    else
      qk_norm_append_kernel<T><<<dim3((unsigned)rows), 256, 0, stream>>>(
          KK_ARGS);
  });
#undef KK_ARGS
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
#define CA_HB 4

// One workgroup per (row, kv head, up to CA_HB of its query heads). Its NW
// waves (4 for many rows, 16 for few, where the keys are the only source of
// parallel work) share out the row's key tiles (tile t of 64 keys, counted
// from lo, goes to wave t mod NW); every wave serves all the heads from one
// read of a key or value row. VEC: d and dv multiples of 8 and 16-byte aligned rows;
// otherwise scalar loads, and lane e owns value entries e, e + 64, ...
template <typename T, bool VEC>
__global__ __launch_bounds__(1024) void chunk_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ kc,
    const T* __restrict__ vc, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ block_table,
    int max_blocks, int H, int G, int d, int dq, int dv, int BS, float scale,
    float cap, int chunk, int window, const float* __restrict__ slopes) {
  extern __shared__ float sm[];
  const int tid = threadIdx.x;
  const int wave = tid / WAVE;
  const int lane = tid & (WAVE - 1);
  const int NW = blockDim.x / WAVE;
  const int NL = VEC ? dv / 8 : 1;          // lanes per value row
  const int NG = VEC ? WAVE / NL : 1;       // key groups
  // workgroup: queries [HB][dq = d rounded up to even] | (max, sum) of every
  // wave and head | partial outputs [waves][HB][dv]
  // wave: weights [HB][64] | row offsets [64] (8 bytes each) | partial sums
  // of the key groups [NG][dv], one head at a time
  float* sq = sm;
  float* sml = sq + CA_HB * dq;
  float* smo = sml + NW * CA_HB * 2;
  const int perw = CA_HB * WAVE + 2 * WAVE + (VEC ? NG * dv : 0);
  float* sp = smo + NW * CA_HB * dv + (long)wave * perw;
  long* soff = reinterpret_cast<long*>(sp + CA_HB * WAVE);
  float* spart = sp + CA_HB * WAVE + 2 * WAVE;

  const long r = blockIdx.x;
  const int g = blockIdx.y;
  const int HPG = H / G;
  const int hz = blockIdx.z * CA_HB;
  const int nh = min(CA_HB, HPG - hz);
  const int h0 = g * HPG + hz;
  const int p = positions[r];
  T* orow = out + (r * H + h0) * (long)dv;
  if (p < 0) {
    for (int i = tid; i < nh * dv; i += blockDim.x) stf(orow + i, 0.f);
    return;
  }
  const T* qr = q + (r * H + h0) * (long)d;
  for (int i = tid; i < CA_HB * dq; i += blockDim.x) {
    const int hb = i / dq, dd = i - hb * dq;
    sq[i] = (hb < nh && dd < d) ? ldf(qr + (long)hb * d + dd) : 0.f;
  }
  __syncthreads();

  const int s = row_seq[r];
  int lo = chunk > 0 ? (p / chunk) * chunk : 0;
  if (window > 0) lo = max(lo, p - window + 1);
  float slope[CA_HB];
#pragma unroll
  for (int hb = 0; hb < CA_HB; ++hb)
    slope[hb] = (slopes && hb < nh) ? slopes[h0 + hb] : 0.f;
  float m[CA_HB], l[CA_HB], acc[CA_HB][8];
#pragma unroll
  for (int hb = 0; hb < CA_HB; ++hb) {
    m[hb] = -INFINITY;
    l[hb] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[hb][i] = 0.f;
  }
  const int grp = VEC ? lane / NL : 0;
  const int sub = VEC ? lane - grp * NL : lane;
  const bool vlive = VEC ? grp < NG : true;

  for (int j0 = lo + wave * WAVE; j0 <= p; j0 += NW * WAVE) {
    const int j = j0 + lane;
    float sc[CA_HB];
#pragma unroll
    for (int hb = 0; hb < CA_HB; ++hb) sc[hb] = -INFINITY;
    long voff = 0;
    if (j <= p) {
      const long blk = block_table[(long)s * max_blocks + j / BS];
      const long slot = (blk * G + g) * BS + j % BS;
      const T* kr = kc + slot * d;
      voff = slot * dv;
      float dot[CA_HB];
#pragma unroll
      for (int hb = 0; hb < CA_HB; ++hb) dot[hb] = 0.f;
      if (VEC) {
        for (int i = 0; i < d; i += 8) {
          float kv[8];
          ld8(kr + i, kv);
#pragma unroll
          for (int hb = 0; hb < CA_HB; ++hb)
#pragma unroll
            for (int k = 0; k < 8; ++k)
              dot[hb] = fmaf(kv[k], sq[hb * dq + i + k], dot[hb]);
        }
      } else {
        for (int i = 0; i < d; ++i) {
          const float kv = ldf(kr + i);
#pragma unroll
          for (int hb = 0; hb < CA_HB; ++hb)
            dot[hb] = fmaf(kv, sq[hb * dq + i], dot[hb]);
        }
      }
#pragma unroll
      for (int hb = 0; hb < CA_HB; ++hb) {
        sc[hb] = dot[hb] * scale;
        if (cap > 0.f) sc[hb] = cap * tanhf(sc[hb] / cap);
        sc[hb] -= slope[hb] * (float)(p - j);
      }
    }
#pragma unroll
    for (int hb = 0; hb < CA_HB; ++hb) {
      const float mn = fmaxf(m[hb], wave_max(sc[hb]));
      const float w = j <= p ? expf(sc[hb] - mn) : 0.f;
      const float alpha = expf(m[hb] - mn);   // m = -inf at first: alpha = 0
      l[hb] = l[hb] * alpha + wave_sum(w);
      m[hb] = mn;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[hb][i] *= alpha;
      sp[hb * WAVE + lane] = w;
    }
    soff[lane] = voff;
    // wave-private LDS: a wave's LDS operations complete in order
    __builtin_amdgcn_wave_barrier();
    const int nk = min(WAVE, p - j0 + 1);
    if (VEC) {
      if (vlive) {
        for (int k = grp; k < nk; k += NG) {
          float vv[8];
          ld8(vc + soff[k] + sub * 8, vv);
#pragma unroll
          for (int hb = 0; hb < CA_HB; ++hb) {
            const float wk = sp[hb * WAVE + k];
#pragma unroll
            for (int i = 0; i < 8; ++i)
              acc[hb][i] = fmaf(wk, vv[i], acc[hb][i]);
          }
        }
      }
    } else {
      for (int k = 0; k < nk; ++k) {
        const T* vr = vc + soff[k];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int e = lane + i * WAVE;
          if (e < dv) {
            const float x = ldf(vr + e);
#pragma unroll
            for (int hb = 0; hb < CA_HB; ++hb)
              acc[hb][i] = fmaf(sp[hb * WAVE + k], x, acc[hb][i]);
          }
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }

  // the wave's partial result, key groups added in group order
  if (VEC) {
#pragma unroll
    for (int hb = 0; hb < CA_HB; ++hb) {
      if (hb < nh) {
        if (vlive) {
#pragma unroll
          for (int i = 0; i < 8; ++i)
            spart[grp * dv + sub * 8 + i] = acc[hb][i];
        }
        __builtin_amdgcn_wave_barrier();
        for (int e = lane; e < dv; e += WAVE) {
          float t = 0.f;
          for (int k = 0; k < NG; ++k) t += spart[k * dv + e];
          smo[(wave * CA_HB + hb) * dv + e] = t;
        }
        __builtin_amdgcn_wave_barrier();
      }
    }
  } else {
#pragma unroll
    for (int hb = 0; hb < CA_HB; ++hb)
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int e = lane + i * WAVE;
        if (e < dv && hb < nh) smo[(wave * CA_HB + hb) * dv + e] = acc[hb][i];
      }
  }
  if (lane == 0) {
#pragma unroll
    for (int hb = 0; hb < CA_HB; ++hb) {
      sml[(wave * CA_HB + hb) * 2] = m[hb];
      sml[(wave * CA_HB + hb) * 2 + 1] = l[hb];
    }
  }
  __syncthreads();
  // fold the waves in wave order; a wave without keys has max -inf, weight 0
  for (int i = tid; i < nh * dv; i += blockDim.x) {
    const int hb = i / dv, e = i - hb * dv;
    float M = -INFINITY;
    for (int w = 0; w < NW; ++w)
      M = fmaxf(M, sml[(w * CA_HB + hb) * 2]);
    float num = 0.f, den = 0.f;
    for (int w = 0; w < NW; ++w) {
      const float f = expf(sml[(w * CA_HB + hb) * 2] - M);
      num = fmaf(f, smo[(w * CA_HB + hb) * dv + e], num);
      den = fmaf(f, sml[(w * CA_HB + hb) * 2 + 1], den);
    }
    stf(orow + i, num / den);
  }
}

// out [T, H*dv], q [T, H*d] contiguous; caches as in qk_norm_append. An
// empty v_cache means that the values are the keys; slopes [H] fp32 or empty.
static void masked_attention(torch::Tensor out, torch::Tensor q,
                             torch::Tensor k_cache, torch::Tensor v_cache,
                             torch::Tensor slopes, torch::Tensor positions,
                             torch::Tensor row_seq, torch::Tensor block_table,
                             int64_t H, double scale, double softcap,
                             int64_t chunk, int64_t window) {
  check_act(q, "q");
  if (v_cache.numel() == 0) v_cache = k_cache;
  const bool biased = slopes.numel() > 0;
  if (biased) {
    check_f32(slopes, "slopes");
    TORCH_CHECK(slopes.numel() == H);
  }
  TORCH_CHECK(window >= 0);
  check_i32(positions, "positions"); check_i32(row_seq, "row_seq");
  check_i32(block_table, "block_table");
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.is_contiguous() &&
              v_cache.dim() == 4 && v_cache.is_contiguous());
  const int G = (int)k_cache.size(1), BS = (int)k_cache.size(2);
  const int d = (int)k_cache.size(3), dv = (int)v_cache.size(3);
  const long rows = q.size(0);
  TORCH_CHECK(H >= 1 && G >= 1 && H % G == 0);
  TORCH_CHECK(q.dim() == 2 && q.is_contiguous() && q.size(1) == H * d);
  TORCH_CHECK(out.dim() == 2 && out.is_contiguous() && out.size(0) == rows &&
              out.size(1) == H * dv);
  TORCH_CHECK(out.scalar_type() == q.scalar_type() &&
              k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type());
  TORCH_CHECK(positions.numel() == rows && row_seq.numel() == rows);
  TORCH_CHECK(block_table.dim() == 2 && chunk >= 0);
  TORCH_CHECK(dv <= 8 * WAVE, "value rows of more than 512 entries");
  if (rows == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  // the row-offset slots are 8-byte entries behind dq + 64 floats
  const int dq = (d + 1) & ~1;
  const bool vec = d % 8 == 0 && dv % 8 == 0 && dv / 8 <= WAVE &&
                   aligned16(q.data_ptr()) && aligned16(k_cache.data_ptr()) &&
                   aligned16(v_cache.data_ptr());
  const int NG = vec ? WAVE / (dv / 8) : 0;
  // few rows (decode steps): the keys are the only parallel work there is
  int NW = rows <= 64 ? 16 : 4;
  const size_t perw = CA_HB * WAVE + 2 * WAVE + (size_t)NG * dv;
  auto lds = [&](int nw) {
    return ((size_t)CA_HB * dq + (size_t)nw * CA_HB * 2 +
            (size_t)nw * CA_HB * dv + nw * perw) * sizeof(float);
  };
  while (NW > 1 && lds(NW) > 120 * 1024) NW /= 2;
  const size_t shmem = lds(NW);
  TORCH_CHECK(shmem <= 160 * 1024, "head sizes exceed the LDS");
  const int HPG = (int)(H / G);
  dim3 grid((unsigned)rows, (unsigned)G,
            (unsigned)((HPG + CA_HB - 1) / CA_HB));
#define KK_ARGS reinterpret_cast<T*>(out.data_ptr()),                      \
        reinterpret_cast<const T*>(q.data_ptr()),                          \
        reinterpret_cast<const T*>(k_cache.data_ptr()),                    \
        reinterpret_cast<const T*>(v_cache.data_ptr()),                    \
        positions.data_ptr<int>(), row_seq.data_ptr<int>(),                \
        block_table.data_ptr<int>(), (int)block_table.size(1), (int)H, G,  \
        d, dq, dv, BS, (float)scale, (float)softcap, (int)chunk,           \
        (int)window, biased ? slopes.data_ptr<float>() : nullptr
  KK_DISPATCH_ACT(q, {
    if (vec) {
      auto kern = chunk_attention_kernel<T, true>;
      // raised once per size, outside any graph capture (the eager warm-up
      // step comes first)
      static size_t allowed = 48 * 1024;
      if (shmem > allowed) {
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)shmem);
        allowed = shmem;
      }
      kern<<<grid, NW * WAVE, shmem, stream>>>(KK_ARGS);
    } else {
      auto kern = chunk_attention_kernel<T, false>;
      static size_t allowed = 48 * 1024;
      if (shmem > allowed) {
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)shmem);
        allowed = shmem;
      }
      kern<<<grid, NW * WAVE, shmem, stream>>>(KK_ARGS);
    }
  });
#undef KK_ARGS
  HIP_CHECK_KERNEL();
}

void chunk_attention(torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
                     torch::Tensor v_cache, torch::Tensor positions,
                     torch::Tensor row_seq, torch::Tensor block_table,
                     int64_t H, double scale, double softcap, int64_t chunk) {
  masked_attention(out, q, k_cache, v_cache,
                   torch::empty({0}, positions.options().dtype(torch::kFloat32)),
                   positions, row_seq, block_table, H, scale, softcap, chunk,
                   0);
}

// Sliding-window attention with a distance bias; an empty v_cache makes the
// keys the values.
void window_attention(torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
                      torch::Tensor v_cache, torch::Tensor slopes,
                      torch::Tensor positions, torch::Tensor row_seq,
                      torch::Tensor block_table, int64_t H, double scale,
                      int64_t window) {
  masked_attention(out, q, k_cache, v_cache, slopes, positions, row_seq,
                   block_table, H, scale, 0.0, 0, window);
}

}  // namespace kukeon
