// Exact single-query attention over the active set: softmax(q K^T / sqrt(d)) V, split
// along the slot axis so that one head fills many CUs, then a per-head combine of the
// partial (max, sum, accumulator) triples.  (A device-scope fence per workgroup, which a
// single-launch "last arrival combines" scheme needs, costs more than the second launch:
// the L2 is per XCD.)
#include <math.h>

#include "common.hpp"
#include "ctx.hpp"

namespace lrqk {

constexpr int kAttnThreads = 256;
constexpr int kAttnWaves = kAttnThreads / kWave;

// Partial layout per (head, split): [m, l, acc[d]] fp32.
// Each K/V row of d elements is read as d*sizeof(T)/16 chunks by `lpr` adjacent lanes, so a
// wave covers 64/lpr rows per load instruction with fully coalesced 16-byte accesses.
template <typename T>
__global__ __launch_bounds__(kAttnThreads) void attn_partial_kernel(const T* __restrict__ q, const T* __restrict__ K,
                                                                    const T* __restrict__ V, int n_slots, int n_valid,
                                                                    int d, int lpr_log2, float scale_log2e,
                                                                    float* __restrict__ part, int S) {
  constexpr int VEC = Vec16<T>::N;
  __shared__ float red[kAttnWaves][2 + 256];
  const int h = blockIdx.y, s = blockIdx.x;
  const int lane = lane_id(), wave = wave_id();
  const int lpr = 1 << lpr_log2;
  const int sub = lane & (lpr - 1);
  const int grp = lane >> lpr_log2;
  const int gpw = kWave >> lpr_log2;  // row groups per wave
  const int rows_per_iter = gpw * kAttnWaves;
  const int rows_per_split = (n_valid + S - 1) / S;
  const int r0 = s * rows_per_split;
  const int r1 = min(n_valid, r0 + rows_per_split);

  float qf[VEC];
  {
    Vec16<T> qv;
    qv.load(q + (int64_t)h * d + sub * VEC);
    qv.unpack(qf);
#pragma unroll
    for (int e = 0; e < VEC; ++e) qf[e] *= scale_log2e;
  }
  const T* Kh = K + (int64_t)h * n_slots * d;
  const T* Vh = V + (int64_t)h * n_slots * d;

  float m_run = -INFINITY, l_run = 0.0f;
  float acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = 0.0f;

  // four row groups per pass: their K and V loads are issued together (one memory latency)
  for (int base = r0; base < r1; base += 4 * rows_per_iter) {
    Vec16<T> kv[4], vv[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int rr = min(base + u * rows_per_iter + wave * gpw + grp, r1 - 1);
      kv[u].load(Kh + (int64_t)rr * d + sub * VEC);
      vv[u].load(Vh + (int64_t)rr * d + sub * VEC);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const bool valid = base + u * rows_per_iter + wave * gpw + grp < r1;
      float kf[VEC], vf[VEC];
      kv[u].unpack(kf);
      vv[u].unpack(vf);
      float sc = 0.0f;
#pragma unroll
      for (int e = 0; e < VEC; ++e) sc = fmaf(kf[e], qf[e], sc);
      for (int off = 1; off < lpr; off <<= 1) sc += __shfl_xor(sc, off, kWave);
      if (!valid) sc = -INFINITY;
      const float m_new = fmaxf(m_run, sc);
      // exp2 of (-inf) - (-inf) must not produce NaN: while nothing valid was seen keep zeros
      const float alpha = (m_new == -INFINITY) ? 0.0f : exp2f(m_run - m_new);
      const float p = (m_new == -INFINITY) ? 0.0f : exp2f(sc - m_new);
      l_run = l_run * alpha + p;
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[e] = acc[e] * alpha + p * vf[e];
      m_run = m_new;
    }
  }
  // merge the row groups of this wave
  for (int off = lpr; off < kWave; off <<= 1) {
    const float m_o = __shfl_xor(m_run, off, kWave);
    const float l_o = __shfl_xor(l_run, off, kWave);
    const float m_new = fmaxf(m_run, m_o);
    const float a = (m_new == -INFINITY) ? 0.0f : exp2f(m_run - m_new);
    const float b = (m_new == -INFINITY) ? 0.0f : exp2f(m_o - m_new);
    l_run = l_run * a + l_o * b;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float o = __shfl_xor(acc[e], off, kWave);
      acc[e] = acc[e] * a + o * b;
    }
    m_run = m_new;
  }
  if (grp == 0) {
    if (sub == 0) {
      red[wave][0] = m_run;
      red[wave][1] = l_run;
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) red[wave][2 + sub * VEC + e] = acc[e];
  }
  __syncthreads();
  float* pout = part + ((int64_t)h * S + s) * (d + 2);
  float M = -INFINITY;
#pragma unroll
  for (int w = 0; w < kAttnWaves; ++w) M = fmaxf(M, red[w][0]);
  for (int c = threadIdx.x; c < d + 2; c += kAttnThreads) {
    float v = 0.0f;
    if (c == 0) {
      v = M;
    } else {
#pragma unroll
      for (int w = 0; w < kAttnWaves; ++w) {
        const float f = (M == -INFINITY) ? 0.0f : exp2f(red[w][0] - M);
        v += red[w][c] * f;
      }
    }
    pout[c] = v;
  }
}

// One workgroup per head merges the S partial triples.  d is a power of two <= 256: thread ->
// (column c, split group tg); every batch of loads is independent, so it costs one latency.
template <typename T>
__global__ __launch_bounds__(kAttnThreads) void attn_combine_kernel(const float* __restrict__ part, int S, int d,
                                                                    T* __restrict__ out) {
  __shared__ float red[kAttnThreads];
  const int h = blockIdx.x;
  const float* p = part + (int64_t)h * S * (d + 2);
  __shared__ float ms_s[64], ls_s[64];  // S <= 64
  if (threadIdx.x < 64) {
    const int t = min((int)threadIdx.x, S - 1);
    const float mv = p[(int64_t)t * (d + 2)], lv = p[(int64_t)t * (d + 2) + 1];
    ms_s[threadIdx.x] = mv;
    ls_s[threadIdx.x] = lv;
  }
  __syncthreads();
  float Mh = -INFINITY;
  for (int t = 0; t < S; ++t) Mh = fmaxf(Mh, ms_s[t]);
  float L = 0.0f;
  for (int t = 0; t < S; ++t) L += (ms_s[t] == -INFINITY) ? 0.0f : ls_s[t] * exp2f(ms_s[t] - Mh);
  // d is a power of two <= 256: thread -> (column c, split group tg)
  const int c = threadIdx.x & (d - 1);
  const int ntg = kAttnThreads / d;
  const int tg = threadIdx.x / d;
  float v = 0.0f;
  for (int t0 = tg; t0 < S; t0 += 8 * ntg) {
    float x[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int t = t0 + u * ntg;
      x[u] = p[(int64_t)min(t, S - 1) * (d + 2) + 2 + c];  // unconditional (clamped), masked below
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int t = t0 + u * ntg;
      if (t < S && ms_s[t] != -INFINITY) v = fmaf(x[u], exp2f(ms_s[t] - Mh), v);
    }
  }
  float* comb = red;
  comb[threadIdx.x] = v;
  __syncthreads();
  if (tg == 0) {
    float tot = 0.0f;
    for (int g = 0; g < ntg; ++g) tot += comb[g * d + c];
    st_f32<T>(out, (int64_t)h * d + c, L > 0.0f ? tot / L : 0.0f);
  }
}

template <typename T>
static int attention_impl(lrqk_ctx* ctx, const void* q, const void* k_act, const void* v_act, int n_slots, int n_valid,
                          void* out, int bh, int d, hipStream_t st) {
  constexpr int VEC = Vec16<T>::N;
  const int lpr = d / VEC;
  int lpr_log2 = 0;
  while ((1 << lpr_log2) < lpr) ++lpr_log2;
  LRQK_REQUIRE(d % VEC == 0 && (1 << lpr_log2) == lpr && lpr <= kWave && d <= 256, LRQK_ELIMIT,
               "head_dim %d unsupported (need a power-of-two number of 16-byte chunks, <= 256 elements)", d);
  int S = (n_valid + 63) / 64;
  if (S < 1) S = 1;
  if (S > 64) S = 64;
  int rc = ctx->attn_part.ensure((size_t)bh * S * (d + 2) * sizeof(float));
  if (rc) return rc;
  const float scale_log2e = (1.0f / sqrtf((float)d)) * 1.4426950408889634f;
  hipLaunchKernelGGL((attn_partial_kernel<T>), dim3((unsigned)S, (unsigned)bh), dim3(kAttnThreads), 0, st,
                     (const T*)q, (const T*)k_act, (const T*)v_act, n_slots, n_valid, d, lpr_log2, scale_log2e,
                     (float*)ctx->attn_part.p, S);
  LRQK_HIP_CHECK(hipGetLastError());
  hipLaunchKernelGGL((attn_combine_kernel<T>), dim3((unsigned)bh), dim3(kAttnThreads), 0, st,
                     (const float*)ctx->attn_part.p, S, d, (T*)out);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

}  // namespace lrqk

using namespace lrqk;

extern "C" int lrqk_attention(lrqk_ctx* ctx, const void* q, const void* k_act, const void* v_act, int n_slots,
                              int n_valid, void* out, int bh, int d, int dtype, void* stream) {
  LRQK_REQUIRE(ctx && q && k_act && v_act && out, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(dtype == LRQK_F32 || dtype == LRQK_BF16, LRQK_EINVAL, "dtype=%d", dtype);
  LRQK_REQUIRE(bh > 0 && bh <= 65535 && d > 0, LRQK_EINVAL, "bad sizes bh=%d d=%d", bh, d);
  LRQK_REQUIRE(n_valid > 0 && n_valid <= n_slots, LRQK_EINVAL, "n_valid=%d outside 1..%d", n_valid, n_slots);
  LRQK_REQUIRE(((uintptr_t)q % 16 == 0) && ((uintptr_t)k_act % 16 == 0) && ((uintptr_t)v_act % 16 == 0), LRQK_EINVAL,
               "pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == LRQK_F32) return attention_impl<float>(ctx, q, k_act, v_act, n_slots, n_valid, out, bh, d, st);
  return attention_impl<bf16_t>(ctx, q, k_act, v_act, n_slots, n_valid, out, bh, d, st);
}
