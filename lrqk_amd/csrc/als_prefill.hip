// Prefill factorisation: joint rank-r alternating least squares for Q ~ A_Q B_Q, K ~ A_K B_K
// with the coupling term Q K^T ~ A_Q A_K^T (all weights 1).
//
// Per iteration the long axis is streamed twice (once over Q, once over K):
//   apply(X, Mt, A): A <- X Mt^T row by row, and in the same pass accumulate the new
//                    A^T A, A^T X and the squared change of A.
// The r x r / r x d systems between the passes are solved per head by `small` kernels.
// The stopping test (a batch-wide mean squared change) is evaluated on the device; once
// it fires the remaining launches of the loop return immediately, so the host never
// waits inside the loop.
#include <algorithm>

#include "common.hpp"
#include "ctx.hpp"

namespace lrqk {

constexpr int kPfThreads = 256;
constexpr int kPfTile = 32;
constexpr int kPfMaxPer = 32;  // accumulators per thread: r*(r+d) <= 256*32

// acc[e] += sum_rows a_s[row][j] * (c < r ? a_s[row][c] : x_s[row][c-r]),  e = j*(r+d)+c
__device__ __forceinline__ void accumulate_gram(const float* a_s, int lda, const float* x_s, int ldx, int rows, int r,
                                                int d, float* acc) {
  const int ne = r * (r + d);
#pragma unroll
  for (int i = 0; i < kPfMaxPer; ++i) {
    const int e = threadIdx.x + i * kPfThreads;
    if (e < ne) {
      const int j = e / (r + d), c = e % (r + d);
      float v = acc[i];
      if (c < r) {
        for (int row = 0; row < rows; ++row) v = fmaf(a_s[row * lda + j], a_s[row * lda + c], v);
      } else {
        for (int row = 0; row < rows; ++row) v = fmaf(a_s[row * lda + j], x_s[row * ldx + c - r], v);
      }
      acc[i] = v;
    }
  }
}

// X: [b][xh][l][d] storage dtype; head h of the factors reads X head (h % hq) / (hq / xh).
template <typename T>
__global__ __launch_bounds__(kPfThreads) void pf_pass_kernel(const T* __restrict__ X, int xh, int hq, int64_t l, int r,
                                                             int d, const float* __restrict__ Mt, float* __restrict__ A,
                                                             float* __restrict__ part, float* __restrict__ delta_part,
                                                             const int* __restrict__ done_flag, int S) {
  if (done_flag && *done_flag) return;
  extern __shared__ __align__(16) float sm[];
  const int ldx = d + 1, lda = r + 1;
  float* x_s = sm;                       // [tile][d+1]
  float* a_s = x_s + kPfTile * ldx;      // [tile][r+1]
  float* m_s = a_s + kPfTile * lda;      // [r][d+1]   (apply only)
  __shared__ float red[kPfThreads / kWave];
  const int tid = threadIdx.x;
  const int h = blockIdx.y, s = blockIdx.x;
  const int b = h / hq, head = h % hq;
  const int64_t xhead = (int64_t)b * xh + head / (hq / xh);
  const T* Xh = X + xhead * l * d;
  float* Ah = A + (int64_t)h * l * r;
  const bool apply = Mt != nullptr;
  if (apply) {
    for (int e = tid; e < r * d; e += kPfThreads) m_s[(e / d) * ldx + e % d] = Mt[(int64_t)h * r * d + e];
  }
  const int64_t rows_per_split = (l + S - 1) / S;
  const int64_t r0 = (int64_t)s * rows_per_split;
  const int64_t r1 = min(l, r0 + rows_per_split);
  float acc[kPfMaxPer];
#pragma unroll
  for (int i = 0; i < kPfMaxPer; ++i) acc[i] = 0.0f;
  float dsum = 0.0f;
  __syncthreads();
  for (int64_t t0 = r0; t0 < r1; t0 += kPfTile) {
    const int rows = (int)min((int64_t)kPfTile, r1 - t0);
    for (int e = tid; e < rows * d; e += kPfThreads) x_s[(e / d) * ldx + e % d] = ld_f32<T>(Xh, t0 * d + e);
    if (!apply) {
      for (int e = tid; e < rows * r; e += kPfThreads) a_s[(e / r) * lda + e % r] = Ah[t0 * r + e];
    }
    __syncthreads();
    if (apply) {
      for (int e = tid; e < rows * r; e += kPfThreads) {
        const int row = e / r, j = e % r;
        float v = 0.0f;
        for (int c = 0; c < d; ++c) v = fmaf(x_s[row * ldx + c], m_s[j * ldx + c], v);
        const float old = Ah[t0 * r + e];
        const float df = old - v;
        dsum = fmaf(df, df, dsum);
        Ah[t0 * r + e] = v;
        a_s[row * lda + j] = v;
      }
      __syncthreads();
    }
    accumulate_gram(a_s, lda, x_s, ldx, rows, r, d, acc);
    __syncthreads();
  }
  const int ne = r * (r + d);
  float* out = part + ((int64_t)h * S + s) * ne;
#pragma unroll
  for (int i = 0; i < kPfMaxPer; ++i) {
    const int e = tid + i * kPfThreads;
    if (e < ne) out[e] = acc[i];
  }
  if (apply) {
    dsum = wave_sum(dsum);
    if (lane_id() == 0) red[wave_id()] = dsum;
    __syncthreads();
    if (tid == 0) {
      float t = 0.0f;
      for (int w = 0; w < kPfThreads / kWave; ++w) t += red[w];
      delta_part[(int64_t)h * S + s] = t;
    }
  }
}

// Gauss-Jordan, no pivoting, r x r system with nrhs right-hand sides stored as columns
// r .. r+nrhs-1 of Mx (row stride ldm).  Afterwards X[i][c] = Mx[i][r+c] / Mx[i][i].
__device__ __forceinline__ void solve_multi(float* Mx, int ldm, int r, int nrhs) {
  const int tid = threadIdx.x;
  for (int p = 0; p < r; ++p) {
    const float inv = 1.0f / Mx[p * ldm + p];
    const int w = r + nrhs - p - 1;  // columns p+1 .. r+nrhs-1
    for (int e = tid; e < r * w; e += kPfThreads) {
      const int i = e / w, j = p + 1 + e % w;
      if (i != p) Mx[i * ldm + j] = fmaf(-(Mx[i * ldm + p] * inv), Mx[p * ldm + j], Mx[i * ldm + j]);
    }
    __syncthreads();
  }
}

__device__ __forceinline__ void reduce_part(const float* part, int S, int ne, float* dst) {
  for (int e = threadIdx.x; e < ne; e += kPfThreads) {
    float v = 0.0f;
    for (int s = 0; s < S; ++s) v += part[(int64_t)s * ne + e];
    dst[e] = v;
  }
}

// stage 0: (stopping test) B_Q, B_K from the current Grams, then Mt for the A_Q update
// stage 1: Mt for the A_K update from the new A_Q Grams
// stage 2: final B_Q, B_K
__global__ __launch_bounds__(kPfThreads) void pf_small_kernel(int stage, int it, const float* __restrict__ partQ,
                                                              const float* __restrict__ partK, int S, int bh, int r,
                                                              int d, int64_t l, float tol,
                                                              const float* __restrict__ delta_all, int* __restrict__ flags,
                                                              float* __restrict__ Mt, float* __restrict__ b_q,
                                                              float* __restrict__ b_k) {
  extern __shared__ __align__(16) float sm[];
  const int ldm = r + d + 1;
  const int ne = r * (r + d);
  float* G1 = sm;               // [r][r+d] packed (ne)   Gram of the first operand
  float* G2 = G1 + ne;          // [r][r+d] packed (ne)
  float* Mx = G2 + ne;          // [r][ldm]
  float* Bs = Mx + r * ldm;     // [r][d+1]
  __shared__ int s_done;
  const int tid = threadIdx.x;
  const int h = blockIdx.x;

  if (stage == 0) {
    if (tid == 0) {
      int done = 0;
      if (it > 0) {
        done = flags[it - 1];
        if (!done) {
          const float* dq = delta_all + ((int64_t)(it - 1) * 2 + 0) * bh * S;
          const float* dk = delta_all + ((int64_t)(it - 1) * 2 + 1) * bh * S;
          float sq = 0.0f, sk = 0.0f;
          for (int i = 0; i < bh * S; ++i) {
            sq += dq[i];
            sk += dk[i];
          }
          const float n = (float)bh * (float)l * (float)r;
          done = fmaxf(sq / n, sk / n) < tol;
        }
      }
      s_done = done;
    }
    __syncthreads();
    // every head computes the same decision; all must have read flags[it-1] and the deltas
    // before anything of this iteration is overwritten, which the launch order guarantees
    if (h == 0 && tid == 0) flags[it] = s_done;
    if (s_done) return;
  } else if (stage == 1) {
    if (flags[it]) return;
  }

  const float* pq = partQ + (int64_t)h * S * ne;
  const float* pk = partK + (int64_t)h * S * ne;
  if (stage == 0 || stage == 2) {
    reduce_part(pq, S, ne, G1);
    reduce_part(pk, S, ne, G2);
    __syncthreads();
    // B_Q = (A_Q^T A_Q)^-1 A_Q^T Q
    for (int e = tid; e < ne; e += kPfThreads) Mx[(e / (r + d)) * ldm + e % (r + d)] = G1[e];
    __syncthreads();
    solve_multi(Mx, ldm, r, d);
    for (int e = tid; e < r * d; e += kPfThreads) {
      const int i = e / d, c = e % d;
      const float v = Mx[i * ldm + r + c] / Mx[i * ldm + i];
      Bs[i * (d + 1) + c] = v;
      b_q[(int64_t)h * r * d + e] = v;
    }
    __syncthreads();
    // B_K
    for (int e = tid; e < ne; e += kPfThreads) Mx[(e / (r + d)) * ldm + e % (r + d)] = G2[e];
    __syncthreads();
    solve_multi(Mx, ldm, r, d);
    for (int e = tid; e < r * d; e += kPfThreads) {
      const int i = e / d, c = e % d;
      b_k[(int64_t)h * r * d + e] = Mx[i * ldm + r + c] / Mx[i * ldm + i];
    }
    __syncthreads();
    if (stage == 2) return;
    // Mt_Q = (A_K^T A_K + B_Q B_Q^T)^-1 (A_K^T K + B_Q)
    for (int e = tid; e < ne; e += kPfThreads) {
      const int i = e / (r + d), c = e % (r + d);
      float v = G2[e];
      if (c < r) {
        float g = 0.0f;
        for (int x = 0; x < d; ++x) g = fmaf(Bs[i * (d + 1) + x], Bs[c * (d + 1) + x], g);
        v += g;
      } else {
        v += Bs[i * (d + 1) + c - r];
      }
      Mx[i * ldm + c] = v;
    }
  } else {
    // stage 1: Mt_K = (A_Q^T A_Q + B_K B_K^T)^-1 (A_Q^T Q + B_K)
    reduce_part(pq, S, ne, G1);
    for (int e = tid; e < r * d; e += kPfThreads) Bs[(e / d) * (d + 1) + e % d] = b_k[(int64_t)h * r * d + e];
    __syncthreads();
    for (int e = tid; e < ne; e += kPfThreads) {
      const int i = e / (r + d), c = e % (r + d);
      float v = G1[e];
      if (c < r) {
        float g = 0.0f;
        for (int x = 0; x < d; ++x) g = fmaf(Bs[i * (d + 1) + x], Bs[c * (d + 1) + x], g);
        v += g;
      } else {
        v += Bs[i * (d + 1) + c - r];
      }
      Mx[i * ldm + c] = v;
    }
  }
  __syncthreads();
  solve_multi(Mx, ldm, r, d);
  for (int e = tid; e < r * d; e += kPfThreads) {
    const int i = e / d, c = e % d;
    Mt[(int64_t)h * r * d + e] = Mx[i * ldm + r + c] / Mx[i * ldm + i];
  }
}

template <typename T>
static int prefill_impl(lrqk_ctx* ctx, const void* q, const void* k, float* a_q, float* a_k, float* b_q, float* b_k,
                        int b, int hq, int hkv, int64_t l, int r, int d, int max_iter, float tol, hipStream_t st) {
  const int bh = b * hq;
  const int ne = r * (r + d);
  LRQK_REQUIRE(ne <= kPfThreads * kPfMaxPer, LRQK_ELIMIT, "r*(r+d)=%d exceeds %d", ne, kPfThreads * kPfMaxPer);
  int S = (int)std::min<int64_t>(64, (l + 255) / 256);
  if (S < 1) S = 1;
  const int iters = max_iter > 0 ? max_iter : 0;
  // workspace: partQ, partK, Mt, deltas[iters][2][bh][S], flags[iters+1]
  const size_t n_part = (size_t)bh * S * ne;
  const size_t n_mt = (size_t)bh * r * d;
  const size_t n_delta = (size_t)(iters > 0 ? iters : 1) * 2 * bh * S;
  const size_t total = (2 * n_part + n_mt + n_delta) * sizeof(float) + (size_t)(iters + 1) * sizeof(int);
  int rc = ctx->prefill_ws.ensure(total);
  if (rc) return rc;
  float* partQ = (float*)ctx->prefill_ws.p;
  float* partK = partQ + n_part;
  float* Mt = partK + n_part;
  float* deltas = Mt + n_mt;
  int* flags = (int*)(deltas + n_delta);
  LRQK_HIP_CHECK(hipMemsetAsync(flags, 0, (size_t)(iters + 1) * sizeof(int), st));

  const size_t smem_pass = ((size_t)kPfTile * (d + 1) + (size_t)kPfTile * (r + 1) + (size_t)r * (d + 1)) * sizeof(float);
  const size_t smem_small = ((size_t)2 * ne + (size_t)r * (r + d + 1) + (size_t)r * (d + 1)) * sizeof(float);
  if (smem_pass > 48 * 1024)
    LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)pf_pass_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem_pass));
  if (smem_small > 48 * 1024)
    LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)pf_small_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem_small));
  LRQK_REQUIRE(smem_small <= 160 * 1024 && smem_pass <= 160 * 1024, LRQK_ELIMIT, "r=%d d=%d need too much LDS", r, d);
  const dim3 grid((unsigned)S, (unsigned)bh), blk(kPfThreads);
  const T* Q = (const T*)q;
  const T* K = (const T*)k;
  hipLaunchKernelGGL((pf_pass_kernel<T>), grid, blk, smem_pass, st, Q, hq, hq, l, r, d, (const float*)nullptr, a_q, partQ,
                     (float*)nullptr, (const int*)nullptr, S);
  hipLaunchKernelGGL((pf_pass_kernel<T>), grid, blk, smem_pass, st, K, hkv, hq, l, r, d, (const float*)nullptr, a_k, partK,
                     (float*)nullptr, (const int*)nullptr, S);
  LRQK_HIP_CHECK(hipGetLastError());
  for (int it = 0; it < iters; ++it) {
    float* dq = deltas + ((size_t)it * 2 + 0) * bh * S;
    float* dk = deltas + ((size_t)it * 2 + 1) * bh * S;
    hipLaunchKernelGGL(pf_small_kernel, dim3((unsigned)bh), blk, smem_small, st, 0, it, partQ, partK, S, bh, r, d, l, tol,
                       deltas, flags, Mt, b_q, b_k);
    hipLaunchKernelGGL((pf_pass_kernel<T>), grid, blk, smem_pass, st, Q, hq, hq, l, r, d, (const float*)Mt, a_q, partQ, dq,
                       (const int*)(flags + it), S);
    hipLaunchKernelGGL(pf_small_kernel, dim3((unsigned)bh), blk, smem_small, st, 1, it, partQ, partK, S, bh, r, d, l, tol,
                       deltas, flags, Mt, b_q, b_k);
    hipLaunchKernelGGL((pf_pass_kernel<T>), grid, blk, smem_pass, st, K, hkv, hq, l, r, d, (const float*)Mt, a_k, partK, dk,
                       (const int*)(flags + it), S);
    LRQK_HIP_CHECK(hipGetLastError());
  }
  hipLaunchKernelGGL(pf_small_kernel, dim3((unsigned)bh), blk, smem_small, st, 2, iters, partQ, partK, S, bh, r, d, l, tol,
                     deltas, flags, Mt, b_q, b_k);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

}  // namespace lrqk

using namespace lrqk;

extern "C" int lrqk_als_prefill(lrqk_ctx* ctx, const void* q, const void* k, float* a_q, float* a_k, float* b_q,
                                float* b_k, int b, int hq, int hkv, int64_t l, int r, int d, int max_iter, float tol,
                                int dtype, void* stream) {
  LRQK_REQUIRE(ctx && q && k && a_q && a_k && b_q && b_k, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(dtype == LRQK_F32 || dtype == LRQK_BF16, LRQK_EINVAL, "dtype=%d", dtype);
  LRQK_REQUIRE(b > 0 && hq > 0 && hkv > 0 && hq % hkv == 0 && (int64_t)b * hq <= 65535, LRQK_EINVAL,
               "bad heads b=%d hq=%d hkv=%d", b, hq, hkv);
  LRQK_REQUIRE(r > 0 && r <= LRQK_MAX_R && d > 0 && l > 0 && l < ((int64_t)1 << 31), LRQK_EINVAL, "bad sizes r=%d d=%d l=%lld",
               r, d, (long long)l);
  LRQK_REQUIRE(max_iter <= 64, LRQK_ELIMIT, "max_iter=%d > 64", max_iter);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == LRQK_F32) return prefill_impl<float>(ctx, q, k, a_q, a_k, b_q, b_k, b, hq, hkv, l, r, d, max_iter, tol, st);
  return prefill_impl<bf16_t>(ctx, q, k, a_q, a_k, b_q, b_k, b, hq, hkv, l, r, d, max_iter, tol, st);
}
