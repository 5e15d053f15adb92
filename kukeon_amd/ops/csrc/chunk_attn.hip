// Grouped-query attention whose scores carry no positions: queries and keys
// are RMS-normed over their WHOLE projection row, scores are scaled and may
// be capped (cap tanh(score / cap)), and a query at position p sees the keys
// lo .. p, lo being the first position of p's chunk (0 without chunks).
//
// qk_norm_append   norms q (and k) of every row, writes q to a dense buffer
//                  and k, v to the row's page.
// chunk_attention  one WAVE per (row, head), no barriers. Keys are taken 64 at
//                  a time counted from lo: lane j scores key j (the query sits
//                  in wave-private LDS as fp32), the wave agrees on the
//                  running maximum and sum, then dv/8 lanes cover one value
//                  row with 16-byte loads while the 64/(dv/8) lane groups
//                  take every NG-th key; the groups' partial sums meet in LDS
//                  at the end, added in group order. Everything is fp32; a
//                  row's result depends only on its own position and chunk.
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
  KK_DISPATCH_ACT(proj, {
    qk_norm_append_kernel<T><<<dim3((unsigned)rows), 256, 0, stream>>>(
        reinterpret_cast<T*>(q_out.data_ptr()),
        own ? reinterpret_cast<T*>(k_cache.data_ptr()) : nullptr,
        own ? reinterpret_cast<T*>(v_cache.data_ptr()) : nullptr,
        reinterpret_cast<const T*>(proj.data_ptr()), (long)proj.stride(0),
        (long)q_col, (long)k_col, (long)v_col, wq.data_ptr<float>(),
        own ? wk.data_ptr<float>() : nullptr, (float)eps,
        positions.data_ptr<int>(), row_seq.data_ptr<int>(),
        block_table.data_ptr<int>(), (int)block_table.size(1), Cq, G, d, dv,
        BS);
  });
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
#define CA_WAVES 4

// VEC: d and dv multiples of 8 and 16-byte aligned rows. Otherwise scalar
// loads, and lane e owns value entries e, e + 64, ...
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void chunk_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ kc,
    const T* __restrict__ vc, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const int* __restrict__ block_table,
    int max_blocks, int H, int G, int d, int dq, int dv, int BS, float scale,
    float cap, int chunk) {
  extern __shared__ float sm[];
  const int wave = threadIdx.x / WAVE;
  const int lane = threadIdx.x & (WAVE - 1);
  const int NL = VEC ? dv / 8 : 1;          // lanes per value row
  const int NG = VEC ? WAVE / NL : 1;       // key groups
  // per wave: query [dq = d rounded up to even] | weights [64] | row
  // offsets [64] (8 bytes each) | partial sums [NG][dv]
  const int per = dq + WAVE + 2 * WAVE + (VEC ? NG * dv : 0);
  float* sq = sm + (long)wave * per;
  float* sp = sq + dq;
  long* soff = reinterpret_cast<long*>(sp + WAVE);
  float* spart = sp + 3 * WAVE;
  const long r = blockIdx.x;
  const int h = blockIdx.y * CA_WAVES + wave;
  if (h >= H) return;
  const int p = positions[r];
  T* orow = out + (r * H + h) * (long)dv;
  if (p < 0) {
    for (int e = lane; e < dv; e += WAVE) stf(orow + e, 0.f);
    return;
  }
  const int s = row_seq[r];
  const int g = h / (H / G);
  const int lo = chunk > 0 ? (p / chunk) * chunk : 0;
  const T* qr = q + (r * H + h) * (long)d;
  for (int i = lane; i < d; i += WAVE) sq[i] = ldf(qr + i);
  // wave-private LDS: a wave's LDS operations complete in order
  __builtin_amdgcn_wave_barrier();

  float m = -INFINITY, l = 0.f;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  const int grp = VEC ? lane / NL : 0;
  const int sub = VEC ? lane - grp * NL : lane;
  const bool vlive = VEC ? grp < NG : true;

  for (int j0 = lo; j0 <= p; j0 += WAVE) {
    const int j = j0 + lane;
    float sc = -INFINITY;
    long voff = 0;
    if (j <= p) {
      const long blk = block_table[(long)s * max_blocks + j / BS];
      const long slot = (blk * G + g) * BS + j % BS;
      const T* kr = kc + slot * d;
      voff = slot * dv;
      float dot = 0.f;
      if (VEC) {
        for (int i = 0; i < d; i += 8) {
          float kv[8];
          ld8(kr + i, kv);
#pragma unroll
          for (int k = 0; k < 8; ++k) dot = fmaf(kv[k], sq[i + k], dot);
        }
      } else {
        for (int i = 0; i < d; ++i) dot = fmaf(ldf(kr + i), sq[i], dot);
      }
      sc = dot * scale;
      if (cap > 0.f) sc = cap * tanhf(sc / cap);
    }
    const float mn = fmaxf(m, wave_max(sc));
    const float w = j <= p ? expf(sc - mn) : 0.f;
    const float alpha = expf(m - mn);     // m = -inf at first: alpha = 0
    l = l * alpha + wave_sum(w);
    m = mn;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] *= alpha;
    sp[lane] = w;
    soff[lane] = voff;
      __builtin_amdgcn_wave_barrier();
    const int nk = min(WAVE, p - j0 + 1);
    if (VEC) {
      if (vlive) {
        for (int k = grp; k < nk; k += NG) {
          float vv[8];
          ld8(vc + soff[k] + sub * 8, vv);
          const float wk = sp[k];
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[i] = fmaf(wk, vv[i], acc[i]);
        }
      }
    } else {
      for (int k = 0; k < nk; ++k) {
        const float wk = sp[k];
        const T* vr = vc + soff[k];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int e = lane + i * WAVE;
          if (e < dv) acc[i] = fmaf(wk, ldf(vr + e), acc[i]);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  const float inv = 1.0f / l;
  if (VEC) {
    if (vlive) {
#pragma unroll
      for (int i = 0; i < 8; ++i) spart[grp * dv + sub * 8 + i] = acc[i];
    }
      __builtin_amdgcn_wave_barrier();
    for (int e = lane; e < dv; e += WAVE) {
      float t = 0.f;
      for (int k = 0; k < NG; ++k) t += spart[k * dv + e];
      stf(orow + e, t * inv);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int e = lane + i * WAVE;
      if (e < dv) stf(orow + e, acc[i] * inv);
    }
  }
}

// out [T, H*dv], q [T, H*d] contiguous; caches as in qk_norm_append.
void chunk_attention(torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
                     torch::Tensor v_cache, torch::Tensor positions,
                     torch::Tensor row_seq, torch::Tensor block_table,
                     int64_t H, double scale, double softcap, int64_t chunk) {
  check_act(q, "q");
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
  const size_t per = dq + 3 * WAVE + (size_t)NG * dv;
  const size_t shmem = CA_WAVES * per * sizeof(float);
  TORCH_CHECK(shmem <= 160 * 1024, "head sizes exceed the LDS");
  dim3 grid((unsigned)rows, (unsigned)((H + CA_WAVES - 1) / CA_WAVES));
#define KK_ARGS reinterpret_cast<T*>(out.data_ptr()),                      \
        reinterpret_cast<const T*>(q.data_ptr()),                          \
        reinterpret_cast<const T*>(k_cache.data_ptr()),                    \
        reinterpret_cast<const T*>(v_cache.data_ptr()),                    \
        positions.data_ptr<int>(), row_seq.data_ptr<int>(),                \
        block_table.data_ptr<int>(), (int)block_table.size(1), (int)H, G,  \
        d, dq, dv, BS, (float)scale, (float)softcap, (int)chunk
  KK_DISPATCH_ACT(q, {
    if (vec) {
      auto kern = chunk_attention_kernel<T, true>;
      if (shmem > 48 * 1024)
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)shmem);
      kern<<<grid, 256, shmem, stream>>>(KK_ARGS);
    } else {
      auto kern = chunk_attention_kernel<T, false>;
      if (shmem > 48 * 1024)
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)shmem);
      kern<<<grid, 256, shmem, stream>>>(KK_ARGS);
    }
  });
#undef KK_ARGS
  HIP_CHECK_KERNEL();
}

}  // namespace kukeon
