// Per-step factor update (the decode half of the alternating least squares).
//
//   gram   : per head, split over the active rows: A^T [A | w] with w = K_prev q
//            (A = gathered active A_K rows) -> partial sums
//   solve  : per head: reduce partials, form the r x r Gram systems, run every
//            alternating iteration and record each iterate + its squared change
//   finish : per head: pick the iterate at which the batch-wide stopping test fired,
//            take the exact line-search step on B_Q, B_K, round and store
#include "common.hpp"
#include "ctx.hpp"

namespace lrqk {

constexpr int kAlsThreads = 256;
constexpr int kTileRows = 32;

template <typename T>
__global__ __launch_bounds__(kAlsThreads) void als_gram_kernel(const T* __restrict__ a_k, int64_t head_stride,
                                                               int64_t a_rows, const int32_t* __restrict__ active_idx,
                                                               int64_t idx_stride, const T* __restrict__ k_prev,
                                                               int kprev_slots, int n, const T* __restrict__ q, int r,
                                                               int d, int lpr_log2, float* __restrict__ part, int S) {
  constexpr int VEC = Vec16<T>::N;
  __shared__ float a_s[kTileRows][LRQK_MAX_R + 2];  // [row][0..r) = A row, [r] = w
  const int h = blockIdx.y, s = blockIdx.x;
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int lpr = 1 << lpr_log2;
  const int sub = lane & (lpr - 1), grp = lane >> lpr_log2, gpw = kWave >> lpr_log2;
  const int rows_per_split = (n + S - 1) / S;
  const int r0 = s * rows_per_split;
  const int r1 = min(n, r0 + rows_per_split);
  const T* A = a_k + (int64_t)h * head_stride;
  const T* Kp = k_prev + (int64_t)h * kprev_slots * d;

  float qf[VEC];
  {
    Vec16<T> qv;
    qv.load(q + (int64_t)h * d + sub * VEC);
    qv.unpack(qf);
  }
  const int ne = r * (r + 1);
  constexpr int kMaxPer = (LRQK_MAX_R * (LRQK_MAX_R + 1) + kAlsThreads - 1) / kAlsThreads;
  float acc[kMaxPer];
#pragma unroll
  for (int i = 0; i < kMaxPer; ++i) acc[i] = 0.0f;

  for (int t0 = r0; t0 < r1; t0 += kTileRows) {
    const int rows = min(kTileRows, r1 - t0);
    // A rows (gathered) -> LDS
    for (int e = tid; e < rows * r; e += kAlsThreads) {
      const int row = e / r, j = e % r;
      const int64_t src = active_idx ? (int64_t)active_idx[(int64_t)h * idx_stride + t0 + row] : (int64_t)(t0 + row);
      a_s[row][j] = (src >= 0 && src < a_rows) ? ld_f32<T>(A, src * r + j) : 0.0f;
    }
    // w = K_prev[row] . q
    for (int base = 0; base < rows; base += gpw * (kAlsThreads / kWave)) {
      const int row = base + wave * gpw + grp;
      const bool valid = row < rows;
      const int rr = valid ? row : rows - 1;
      Vec16<T> kv;
      kv.load(Kp + (int64_t)(t0 + rr) * d + sub * VEC);
      float kf[VEC];
      kv.unpack(kf);
      float w = 0.0f;
#pragma unroll
      for (int e = 0; e < VEC; ++e) w = fmaf(kf[e], qf[e], w);
      for (int off = 1; off < lpr; off <<= 1) w += __shfl_xor(w, off, kWave);
      if (valid && sub == 0) a_s[row][r] = w;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kMaxPer; ++i) {
      const int e = tid + i * kAlsThreads;
      if (e < ne) {
        const int j = e / (r + 1), j2 = e % (r + 1);
        float v = acc[i];
        for (int row = 0; row < rows; ++row) v = fmaf(a_s[row][j], a_s[row][j2], v);
        acc[i] = v;
      }
    }
    __syncthreads();
  }
  float* out = part + ((int64_t)h * S + s) * ne;
#pragma unroll
  for (int i = 0; i < kMaxPer; ++i) {
    const int e = tid + i * kAlsThreads;
    if (e < ne) out[e] = acc[i];
  }
}

// Gauss-Jordan elimination without pivoting on the augmented r x (r+1) system in LDS
// (the systems here are Gram matrices plus positive semidefinite terms).  Row stride ldm.
// On return x[i] = Mx[i][r] / Mx[i][i].  One barrier per eliminated column.
__device__ __forceinline__ void solve_lds(float* Mx, int ldm, int r, float* x) {
  const int tid = threadIdx.x;
  for (int p = 0; p < r; ++p) {
    const float inv = 1.0f / Mx[p * ldm + p];
    const int w = r - p;  // columns p+1 .. r
    for (int e = tid; e < r * w; e += kAlsThreads) {
      const int i = e / w, j = p + 1 + e % w;
      if (i != p) Mx[i * ldm + j] = fmaf(-(Mx[i * ldm + p] * inv), Mx[p * ldm + j], Mx[i * ldm + j]);
    }
    __syncthreads();
  }
  for (int i = tid; i < r; i += kAlsThreads) x[i] = Mx[i * ldm + r] / Mx[i * ldm + i];
  __syncthreads();
}

// iter_out layout per head: [max_iter][2r] (q_hat then k_hat of each iteration),
// deltas: [bh][max_iter] sum over r of (k_hat - k_hat')^2.
template <typename T>
__global__ __launch_bounds__(kAlsThreads) void als_solve_kernel(const T* __restrict__ b_q, const T* __restrict__ b_k,
                                                                const float* __restrict__ part, int S,
                                                                const T* __restrict__ q, const T* __restrict__ k_new,
                                                                int hq, int hkv, int r, int d, int max_iter,
                                                                float* __restrict__ iter_out,
                                                                float* __restrict__ deltas) {
  extern __shared__ __align__(16) float sm[];
  float* BQ = sm;                    // [r][d+1]
  float* BK = BQ + r * (d + 1);      // [r][d+1]
  float* qv = BK + r * (d + 1);      // [d]
  float* kv = qv + d;                // [d]
  float* GQ = kv + d;                // [r][r+1]
  float* GK = GQ + r * (r + 1);      // [r][r+1]
  float* Mx = GK + r * (r + 1);      // [r][r+2]
  float* rhs_q = Mx + r * (r + 2);   // 5 vectors of r
  float* kB = rhs_q + r;
  float* hat_k = kB + r;
  float* hat_q = hat_k + r;
  float* new_k = hat_q + r;
  __shared__ float s_qk;
  const int lg = r + 1, lm = r + 2;
  const int tid = threadIdx.x;
  const int h = blockIdx.x;
  const int b = h / hq, head = h % hq;
  const int kvh = head / (hq / hkv);
  const int ld = d + 1;
  const int ne = r * (r + 1);

  for (int e = tid; e < r * d; e += kAlsThreads) {
    BQ[(e / d) * ld + e % d] = ld_f32<T>(b_q, (int64_t)h * r * d + e);
    BK[(e / d) * ld + e % d] = ld_f32<T>(b_k, (int64_t)h * r * d + e);
  }
  for (int c = tid; c < d; c += kAlsThreads) {
    qv[c] = ld_f32<T>(q, (int64_t)h * d + c);
    kv[c] = ld_f32<T>(k_new, ((int64_t)b * hkv + kvh) * d + c);
  }
  __syncthreads();
  // G_Q = B_Q B_Q^T + A^T A ; G_K = B_K B_K^T ; rhs_q = q B_Q^T + (q K^T) A ; kB = k B_K^T ; s = q.k
  for (int e = tid; e < r * r; e += kAlsThreads) {
    const int i = e / r, j = e % r;
    float gq = 0.0f, gk = 0.0f;
    for (int c = 0; c < d; ++c) {
      gq = fmaf(BQ[i * ld + c], BQ[j * ld + c], gq);
      gk = fmaf(BK[i * ld + c], BK[j * ld + c], gk);
    }
    float ata = 0.0f;
    for (int s = 0; s < S; ++s) ata += part[((int64_t)h * S + s) * ne + i * (r + 1) + j];
    GQ[i * lg + j] = gq + ata;
    GK[i * lg + j] = gk;
  }
  for (int i = tid; i < r; i += kAlsThreads) {
    float a = 0.0f, c2 = 0.0f;
    for (int c = 0; c < d; ++c) {
      a = fmaf(qv[c], BQ[i * ld + c], a);
      c2 = fmaf(kv[c], BK[i * ld + c], c2);
    }
    float wa = 0.0f;
    for (int s = 0; s < S; ++s) wa += part[((int64_t)h * S + s) * ne + i * (r + 1) + r];
    rhs_q[i] = a + wa;
    kB[i] = c2;
  }
  if (tid == 0) {
    float s = 0.0f;
    for (int c = 0; c < d; ++c) s = fmaf(qv[c], kv[c], s);
    s_qk = s;
  }
  __syncthreads();
  // k_hat_0 = kB G_K^{-1}
  for (int e = tid; e < r * (r + 1); e += kAlsThreads) {
    const int i = e / (r + 1), j = e % (r + 1);
    Mx[i * lm + j] = j < r ? GK[i * lg + j] : kB[i];
  }
  __syncthreads();
  solve_lds(Mx, lm, r, hat_k);
  for (int it = 0; it < max_iter; ++it) {
    // q_hat (G_Q + k_hat^T k_hat) = rhs_q + s k_hat      (all matrices symmetric)
    for (int e = tid; e < r * (r + 1); e += kAlsThreads) {
      const int i = e / (r + 1), j = e % (r + 1);
      Mx[i * lm + j] = j < r ? fmaf(hat_k[i], hat_k[j], GQ[i * lg + j]) : fmaf(s_qk, hat_k[i], rhs_q[i]);
    }
    __syncthreads();
    solve_lds(Mx, lm, r, hat_q);
    // k_hat' (G_K + q_hat^T q_hat) = kB + s q_hat
    for (int e = tid; e < r * (r + 1); e += kAlsThreads) {
      const int i = e / (r + 1), j = e % (r + 1);
      Mx[i * lm + j] = j < r ? fmaf(hat_q[i], hat_q[j], GK[i * lg + j]) : fmaf(s_qk, hat_q[i], kB[i]);
    }
    __syncthreads();
    solve_lds(Mx, lm, r, new_k);
    if (tid < kWave) {
      float dsq = 0.0f;
      for (int i = tid; i < r; i += kWave) {
        const float df = hat_k[i] - new_k[i];
        dsq = fmaf(df, df, dsq);
      }
      dsq = wave_sum(dsq);
      if (tid == 0) deltas[(int64_t)h * max_iter + it] = dsq;
    }
    float* o = iter_out + ((int64_t)h * max_iter + it) * 2 * r;
    for (int i = tid; i < r; i += kAlsThreads) {
      o[i] = hat_q[i];
      o[r + i] = new_k[i];
    }
    __syncthreads();
    for (int i = tid; i < r; i += kAlsThreads) hat_k[i] = new_k[i];
    __syncthreads();
  }
}

template <typename T>
__global__ __launch_bounds__(kAlsThreads) void als_finish_kernel(T* __restrict__ b_q, T* __restrict__ b_k,
                                                                 const T* __restrict__ q, const T* __restrict__ k_new,
                                                                 const float* __restrict__ iter_out,
                                                                 const float* __restrict__ deltas, int bh, int hq,
                                                                 int hkv, int r, int d, int max_iter, float tol,
                                                                 T* __restrict__ q_hat_out, T* __restrict__ k_hat_out,
                                                                 T* __restrict__ a_k, int64_t head_stride,
                                                                 int64_t append_row) {
  __shared__ float hat[2][LRQK_MAX_R];
  __shared__ float err[2][256];
  __shared__ float red[2][kAlsThreads / kWave];
  __shared__ int s_it;
  const int tid = threadIdx.x;
  const int h = blockIdx.x;
  const int b = h / hq, head = h % hq;
  const int kvh = head / (hq / hkv);
  // batch-wide stopping test, summed in a fixed order
  if (tid == 0) {
    int chosen = max_iter - 1;
    for (int it = 0; it < max_iter; ++it) {
      float s = 0.0f;
      for (int hh = 0; hh < bh; ++hh) s += deltas[(int64_t)hh * max_iter + it];
      if (s / (float)((int64_t)bh * r) < tol) {
        chosen = it;
        break;
      }
    }
    s_it = chosen;
  }
  __syncthreads();
  const float* o = iter_out + ((int64_t)h * max_iter + s_it) * 2 * r;
  for (int i = tid; i < 2 * r; i += kAlsThreads) hat[i / r][i % r] = o[i];
  __syncthreads();
  // e_q = q_hat B_Q - q ; e_k = k_hat B_K - k
  float hn[2] = {0.0f, 0.0f};
  for (int i = 0; i < r; ++i) {
    hn[0] = fmaf(hat[0][i], hat[0][i], hn[0]);
    hn[1] = fmaf(hat[1][i], hat[1][i], hn[1]);
  }
  float en[2] = {0.0f, 0.0f};
  for (int c = tid; c < d; c += kAlsThreads) {
    float eq = 0.0f, ek = 0.0f;
    for (int i = 0; i < r; ++i) {
      eq = fmaf(hat[0][i], ld_f32<T>(b_q, ((int64_t)h * r + i) * d + c), eq);
      ek = fmaf(hat[1][i], ld_f32<T>(b_k, ((int64_t)h * r + i) * d + c), ek);
    }
    eq -= ld_f32<T>(q, (int64_t)h * d + c);
    ek -= ld_f32<T>(k_new, ((int64_t)b * hkv + kvh) * d + c);
    err[0][c] = eq;
    err[1][c] = ek;
    en[0] = fmaf(eq, eq, en[0]);
    en[1] = fmaf(ek, ek, en[1]);
  }
  en[0] = wave_sum(en[0]);
  en[1] = wave_sum(en[1]);
  if (lane_id() == 0) {
    red[0][wave_id()] = en[0];
    red[1][wave_id()] = en[1];
  }
  __syncthreads();
  float e2[2] = {0.0f, 0.0f};
  for (int w = 0; w < kAlsThreads / kWave; ++w) {
    e2[0] += red[0][w];
    e2[1] += red[1][w];
  }
  // dB = hat^T e : |dB|^2 = |hat|^2 |e|^2 ; hat dB = |hat|^2 e : |hat dB|^2 = |hat|^4 |e|^2
  float lr[2];
  for (int s = 0; s < 2; ++s) lr[s] = (hn[s] * e2[s]) / (hn[s] * hn[s] * e2[s] + 1e-6f);
  for (int e = tid; e < r * d; e += kAlsThreads) {
    const int i = e / d, c = e % d;
    const int64_t off = (int64_t)h * r * d + e;
    const float nq = ld_f32<T>(b_q, off) - lr[0] * (hat[0][i] * err[0][c]);
    const float nk = ld_f32<T>(b_k, off) - lr[1] * (hat[1][i] * err[1][c]);
    st_f32<T>(b_q, off, nq);
    st_f32<T>(b_k, off, nk);
  }
  for (int i = tid; i < r; i += kAlsThreads) {
    st_f32<T>(q_hat_out, (int64_t)h * r + i, hat[0][i]);
    st_f32<T>(k_hat_out, (int64_t)h * r + i, hat[1][i]);
    if (append_row >= 0) st_f32<T>(a_k, (int64_t)h * head_stride + append_row * r + i, hat[1][i]);
  }
}

template <typename T>
static int als_decode_impl(lrqk_ctx* ctx, void* b_q, void* b_k, void* a_k, int64_t head_stride,
                           const int32_t* active_idx, int64_t idx_stride, const void* k_prev, int kprev_slots, int n,
                           const void* q, const void* k_new, int b, int hq, int hkv, int r, int d, int max_iter,
                           float tol, void* q_hat, void* k_hat, int64_t append_row, hipStream_t st) {
  constexpr int VEC = Vec16<T>::N;
  const int bh = b * hq;
  const int lpr = d / VEC;
  int lpr_log2 = 0;
  while ((1 << lpr_log2) < lpr) ++lpr_log2;
  LRQK_REQUIRE(d % VEC == 0 && (1 << lpr_log2) == lpr && lpr <= kWave && d <= 256, LRQK_ELIMIT,
               "head_dim %d unsupported (need a power-of-two number of 16-byte chunks, <= 256 elements)", d);
  int S = (n + 63) / 64;
  if (S < 1) S = 1;
  if (S > 64) S = 64;
  const int ne = r * (r + 1);
  int rc = ctx->als_part.ensure((size_t)bh * S * ne * sizeof(float));
  if (rc) return rc;
  rc = ctx->als_iter.ensure((size_t)bh * max_iter * (2 * r + 1) * sizeof(float));
  if (rc) return rc;
  float* part = (float*)ctx->als_part.p;
  float* iter_out = (float*)ctx->als_iter.p;
  float* deltas = iter_out + (size_t)bh * max_iter * 2 * r;
  const int64_t a_rows = head_stride / r;
  hipLaunchKernelGGL((als_gram_kernel<T>), dim3((unsigned)S, (unsigned)bh), dim3(kAlsThreads), 0, st, (const T*)a_k,
                     head_stride, a_rows, active_idx, idx_stride, (const T*)k_prev, kprev_slots, n, (const T*)q, r, d,
                     lpr_log2, part, S);
  LRQK_HIP_CHECK(hipGetLastError());
  const size_t smem = ((size_t)2 * r * (d + 1) + 2 * d + 2 * r * (r + 1) + r * (r + 2) + 5 * r) * sizeof(float);
  if (smem > 48 * 1024) {
    LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)als_solve_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem));
  }
  hipLaunchKernelGGL((als_solve_kernel<T>), dim3((unsigned)bh), dim3(kAlsThreads), smem, st, (const T*)b_q,
                     (const T*)b_k, part, S, (const T*)q, (const T*)k_new, hq, hkv, r, d, max_iter, iter_out, deltas);
  LRQK_HIP_CHECK(hipGetLastError());
  hipLaunchKernelGGL((als_finish_kernel<T>), dim3((unsigned)bh), dim3(kAlsThreads), 0, st, (T*)b_q, (T*)b_k,
                     (const T*)q, (const T*)k_new, iter_out, deltas, bh, hq, hkv, r, d, max_iter, tol, (T*)q_hat,
                     (T*)k_hat, (T*)a_k, head_stride, append_row);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

}  // namespace lrqk

using namespace lrqk;

extern "C" int lrqk_als_decode(lrqk_ctx* ctx, void* b_q, void* b_k, void* a_k, int64_t head_stride,
                               const int32_t* active_idx, int64_t idx_stride, const void* k_prev, int kprev_slots,
                               int n, const void* q, const void* k_new, int b, int hq, int hkv, int r, int d,
                               int max_iter, float tol, void* q_hat, void* k_hat, int64_t append_row, int dtype,
                               void* stream) {
  LRQK_REQUIRE(ctx && b_q && b_k && a_k && k_prev && q && k_new && q_hat && k_hat, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(dtype == LRQK_F32 || dtype == LRQK_BF16, LRQK_EINVAL, "dtype=%d", dtype);
  LRQK_REQUIRE(b > 0 && hq > 0 && hkv > 0 && hq % hkv == 0 && (int64_t)b * hq <= 65535, LRQK_EINVAL,
               "bad heads b=%d hq=%d hkv=%d", b, hq, hkv);
  LRQK_REQUIRE(r > 0 && r <= LRQK_MAX_R, LRQK_ELIMIT, "r=%d not in 1..%d", r, LRQK_MAX_R);
  LRQK_REQUIRE(n > 0 && n <= kprev_slots, LRQK_EINVAL, "n=%d outside 1..%d", n, kprev_slots);
  LRQK_REQUIRE(!active_idx || idx_stride >= n, LRQK_EINVAL, "idx_stride < n");
  LRQK_REQUIRE(head_stride >= r && head_stride % r == 0, LRQK_EINVAL, "head_stride must be a multiple of r");
  LRQK_REQUIRE(active_idx || (int64_t)n * r <= head_stride, LRQK_EINVAL, "n rows exceed the A_K head");
  LRQK_REQUIRE(append_row < head_stride / r, LRQK_EINVAL, "append_row beyond the A_K capacity");
  if (max_iter < 1) max_iter = 1;
  LRQK_REQUIRE(max_iter <= LRQK_MAX_DECODE_ITERS, LRQK_ELIMIT, "max_iter=%d > %d", max_iter, LRQK_MAX_DECODE_ITERS);
  LRQK_REQUIRE(((uintptr_t)q % 16 == 0) && ((uintptr_t)k_prev % 16 == 0), LRQK_EINVAL, "pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == LRQK_F32)
    return als_decode_impl<float>(ctx, b_q, b_k, a_k, head_stride, active_idx, idx_stride, k_prev, kprev_slots, n, q,
                                  k_new, b, hq, hkv, r, d, max_iter, tol, q_hat, k_hat, append_row, st);
  return als_decode_impl<bf16_t>(ctx, b_q, b_k, a_k, head_stride, active_idx, idx_stride, k_prev, kprev_slots, n, q,
                                 k_new, b, hq, hkv, r, d, max_iter, tol, q_hat, k_hat, append_row, st);
}
