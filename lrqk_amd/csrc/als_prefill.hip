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
//
// Two implementations of each kernel: fp32 MFMA (32x32x2) tiles for r <= 32 and head
// dimensions that are a multiple of the 16-byte vector, and a generic VALU version for
// every other shape.  Both write the same partial-sum layout.
#include <algorithm>
#include <stdlib.h>

#include "common.hpp"
#include "ctx.hpp"
#include "small_inverse.hpp"

namespace lrqk {

constexpr int kPfThreads = 256;
constexpr int kPfTile = 32;
constexpr int kPfMaxPer = 48;  // accumulators per thread: r*(r+d) <= 256*48 (r = 64 with rows of 128 elements)

// Sums of a tile: out[j][c] += sum_rows a_s[row][j] * (c < r ? a_s[row][c] : x_s[row][c-r]),  0 <= j < r,
// 0 <= c < r + d.  The 256 threads form a 16 x 16 grid; thread (tj, tc) owns rows j = tj + 16 i (i < I) and columns
// c = tc + 16 k (k < 48 / I) and keeps them in acc[i * K + k]: I values of A and K of [A | X] per tile row feed
// I * K products (a sixth of the LDS reads of one output at a time).  I = ceil(r / 16), which the limit
// r (r + d) <= 12288 makes enough: 16 K >= r + d.
template <int I>
__device__ __forceinline__ void accumulate_gram_tile(const float* a_s, int lda, const float* x_s, int ldx, int rows, int r,
                                                     int d, float* acc) {
  constexpr int K = kPfMaxPer / I;
  const int tj = threadIdx.x >> 4, tc = threadIdx.x & 15;
  const float* cp[K];  // column c of a row: in the A tile or in the X tile
  int cs[K];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const int c = min(tc + 16 * k, r + d - 1);
    cp[k] = c < r ? a_s + c : x_s + (c - r);
    cs[k] = c < r ? lda : ldx;
  }
  for (int row = 0; row < rows; ++row) {
    float av[I], cv[K];
#pragma unroll
    for (int i = 0; i < I; ++i) av[i] = a_s[row * lda + min(tj + 16 * i, r - 1)];
#pragma unroll
    for (int k = 0; k < K; ++k) cv[k] = cp[k][row * cs[k]];
#pragma unroll
    for (int i = 0; i < I; ++i)
#pragma unroll
      for (int k = 0; k < K; ++k) acc[i * K + k] = fmaf(av[i], cv[k], acc[i * K + k]);
  }
}
__device__ __forceinline__ void accumulate_gram(const float* a_s, int lda, const float* x_s, int ldx, int rows, int r,
                                                int d, float* acc) {
  if (r <= 16)
    accumulate_gram_tile<1>(a_s, lda, x_s, ldx, rows, r, d, acc);
  else if (r <= 32)
    accumulate_gram_tile<2>(a_s, lda, x_s, ldx, rows, r, d, acc);
  else if (r <= 48)
    accumulate_gram_tile<3>(a_s, lda, x_s, ldx, rows, r, d, acc);
  else
    accumulate_gram_tile<4>(a_s, lda, x_s, ldx, rows, r, d, acc);
}
// The sums of accumulate_gram to `out` (packed [r][r + d]).
__device__ __forceinline__ void store_gram(const float* acc, int r, int d, float* __restrict__ out) {
  const int I = r <= 16 ? 1 : r <= 32 ? 2 : r <= 48 ? 3 : 4;
  const int K = kPfMaxPer / I;
  const int tj = threadIdx.x >> 4, tc = threadIdx.x & 15;
#pragma unroll
  for (int e = 0; e < kPfMaxPer; ++e) {
    const int i = e / K, k = e % K;
    const int j = tj + 16 * i, c = tc + 16 * k;
    if (i < I && j < r && c < r + d) out[j * (r + d) + c] = acc[e];
  }
}

// X: [b][xh][l][d] storage dtype; head h of the factors reads X head (h % hq) / (hq / xh).
template <typename T>
__global__ __launch_bounds__(kPfThreads) void pf_pass_generic_kernel(const T* __restrict__ X, int xh, int hq, int64_t l, int r,
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
      // thread -> (row of the tile, eight columns j = jg + 8 u of the new A): one element of X feeds eight products
      static_assert(kPfTile == 32 && kPfThreads == 256, "32 rows x 8 column groups");
      const int row = tid & (kPfTile - 1), jg = tid >> 5;
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = 0.0f;
      const float* mrow[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) mrow[u] = m_s + min(jg + 8 * u, r - 1) * ldx;
      for (int c = 0; c < d; ++c) {
        const float x = x_s[row * ldx + c];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = fmaf(x, mrow[u][c], v[u]);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int j = jg + 8 * u;
        if (row < rows && j < r) {
          const float old = Ah[(t0 + row) * r + j];
          const float df = old - v[u];
          dsum = fmaf(df, df, dsum);
          Ah[(t0 + row) * r + j] = v[u];
          a_s[row * lda + j] = v[u];
        }
      }
      __syncthreads();
    }
    accumulate_gram(a_s, lda, x_s, ldx, rows, r, d, acc);
    __syncthreads();
  }
  const int ne = r * (r + d);
  store_gram(acc, r, d, part + ((int64_t)h * S + s) * ne);
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
    // (more than 16 partial sums -- long prompts -- are added in fp64)
    float v = 0.0f;
    double w = 0.0;
    for (int s = 0; s < S; ++s) {
      const float x = part[(int64_t)s * ne + e];
      v += x;
      w += (double)x;
    }
    dst[e] = S > 16 ? (float)w : v;
  }
}

// stage 0: (stopping test) B_Q, B_K from the current Grams, then Mt for the A_Q update
// stage 1: Mt for the A_K update from the new A_Q Grams
// stage 2: final B_Q, B_K
__global__ __launch_bounds__(kPfThreads) void pf_small_generic_kernel(int stage, int it, const float* __restrict__ partQ,
                                                              const float* __restrict__ partK, int S, int bh, int r,
                                                              int d, int64_t l, float tol,
                                                              const float* __restrict__ delta_all, int* __restrict__ flags,
                                                              float* __restrict__ Mt, float* __restrict__ b_q,
                                                              float* __restrict__ b_k) {
  extern __shared__ __align__(16) float sm[];
  const int ldm = r + d + 1;
  const int ne = r * (r + d);
  float* G2 = sm;               // [r][r+d] packed (ne)   the K side's sums (the Q side's go straight into Mx)
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
  // sum over the splits of element e of a head's packed [G | C] block, in split order
  auto summed = [&](const float* part, int e) {
    float v = 0.0f;
    double w = 0.0;
    for (int s = 0; s < S; ++s) {
      const float x = part[(int64_t)s * ne + e];
      v += x;
      w += (double)x;
    }
    return S > 16 ? (float)w : v;
  };
  if (stage == 0 || stage == 2) {
    reduce_part(pk, S, ne, G2);
    // B_Q = (A_Q^T A_Q)^-1 A_Q^T Q
    for (int e = tid; e < ne; e += kPfThreads) Mx[(e / (r + d)) * ldm + e % (r + d)] = summed(pq, e);
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
    for (int e = tid; e < r * d; e += kPfThreads) Bs[(e / d) * (d + 1) + e % d] = b_k[(int64_t)h * r * d + e];
    __syncthreads();
    for (int e = tid; e < ne; e += kPfThreads) {
      const int i = e / (r + d), c = e % (r + d);
      float v = summed(pq, e);
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


// ============================================================================ MFMA path
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kPfSmallThreads = 320;  // one thread per column of [32 x 32 | 32 x d], d <= 288

// C tile of mfma_f32_32x32x2f32: lane l, element v -> row (the column is l & 31)
__device__ __forceinline__ int pf_mfma_row(int lane, int v) { return ((v >> 2) << 3) + ((lane >> 5) << 2) + (v & 3); }

// One wave owns 32 rows of X at a time (staged as fp32 in its private LDS tile, row stride
// 32*NB+4, zero beyond d and beyond the last row).
//   apply:  C[32 x 32] = X[32 x d] Mt^T          (A operand from LDS, B operand = Mt)
//   gram:   G_AA += C^T C, G_AX += C^T X          (the C registers are the A operand as they are:
//           element v of lane l is row pf_mfma_row(l, v), and a sum over rows may visit them in any order)
// The k index of the apply and the column index of G_AX are permuted so that every lane reads
// consecutive floats of its LDS row with 16-byte loads: MFMA step kk multiplies columns kk and
// kk + 16*NB; tile nb of G_AX holds the columns n*NB + nb.
// NB = number of 32-column blocks of X.  NW waves per workgroup; the tiles are wave-private, so
// the waves only meet at the start and in the final reduction and otherwise drift apart (one
// wave's staging overlaps another's MFMAs on the same SIMD).  MT_LDS: Mt is kept in LDS (shared
// by the waves) instead of registers, which leaves room for two waves per SIMD.

// orders this wave's LDS writes before its later LDS reads (the tile is exchanged between lanes)
__device__ __forceinline__ void pf_wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <typename T, int NB, int NW, bool MT_LDS>
__global__ __launch_bounds__(NW * kWave) void pf_pass_mfma_kernel(const T* __restrict__ X, int xh, int hq, int64_t l,
                                                                  int r, int d, const float* __restrict__ Mt,
                                                                  float* __restrict__ A, float* __restrict__ part,
                                                                  float* __restrict__ delta_part,
                                                                  const int* __restrict__ done_flag, int S) {
  if (done_flag && *done_flag) return;
  constexpr int LDX = 32 * NB + 4;
  constexpr int KH = 16 * NB;
  constexpr int VEC = Vec16<T>::N;
  constexpr int NL = 32 * 32 * NB / (kWave * VEC);
  constexpr int NT = NW * kWave;
  extern __shared__ __align__(16) float sm[];
  __shared__ float red[NW];
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int col = lane & 31, half = lane >> 5;
  float* x_s = sm + wave * 32 * LDX;
  float* mt_s = sm + NW * 32 * LDX;  // [32][LDX], MT_LDS only
  const int h = blockIdx.y, s = blockIdx.x;
  const int b = h / hq, head = h % hq;
  const int64_t xhead = (int64_t)b * xh + head / (hq / xh);
  const T* Xh = X + xhead * l * d;
  float* Ah = A + (int64_t)h * l * r;
  const bool apply = Mt != nullptr;
  const bool full_rows = d == 32 * NB;  // row / column of a flat element index by shifts

  float mt[MT_LDS ? 1 : KH];
  if (apply) {
    const float* Mh = Mt + (int64_t)h * r * d;
    if constexpr (MT_LDS) {
      for (int e = tid; e < 32 * 32 * NB; e += NT) {
        const int n = e / (32 * NB), k = e % (32 * NB);
        const float v = Mh[min(n, r - 1) * d + min(k, d - 1)];
        mt_s[n * LDX + k] = (n < r && k < d) ? v : 0.0f;
      }
    } else {
#pragma unroll
      for (int kk = 0; kk < KH; ++kk) {
        const int k = kk + half * KH;
        const float v = Mh[min(col, r - 1) * d + min(k, d - 1)];
        mt[kk] = (col < r && k < d) ? v : 0.0f;
      }
    }
  }
  for (int e = lane; e < 32 * LDX; e += kWave) x_s[e] = 0.0f;

  const int64_t rows_per_split = (((l + S - 1) / S) + 31) / 32 * 32;
  const int64_t r0 = (int64_t)s * rows_per_split;
  const int64_t r1 = min(l, r0 + rows_per_split);

  floatx16 gAA;
  floatx16 gAX[NB];
#pragma unroll
  for (int v = 0; v < 16; ++v) gAA[v] = 0.0f;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int v = 0; v < 16; ++v) gAX[nb][v] = 0.0f;
  float dsum = 0.0f;

  Vec16<T> pre[NL];
  auto issue = [&](int64_t t0) {
    const int nvalid = t0 < r1 ? (int)min((int64_t)32, r1 - t0) * d : 0;
    const int64_t base = (t0 < r1 ? t0 : r0) * d;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int e = (i * kWave + lane) * VEC;
      pre[i].load(Xh + base + (e < nvalid ? e : 0));
    }
  };
  if (r0 + (int64_t)wave * 32 < r1) issue(r0 + (int64_t)wave * 32);
  __syncthreads();  // Mt staged, tiles cleared

  for (int64_t t0 = r0 + (int64_t)wave * 32; t0 < r1; t0 += 32 * NW) {
    const int rows = (int)min((int64_t)32, r1 - t0);
    // stage this wave's rows
    {
      const int nvalid = rows * d;
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const int e = (i * kWave + lane) * VEC;
        if (e < 32 * d) {
          float f[VEC];
          pre[i].unpack(f);
          const int row = full_rows ? e / (32 * NB) : e / d;
          const int c0 = full_rows ? e % (32 * NB) : e - row * d;
          const bool ok = e < nvalid;
#pragma unroll
          for (int u = 0; u < VEC; u += 4)
            *reinterpret_cast<float4*>(&x_s[row * LDX + c0 + u]) =
                make_float4(ok ? f[u] : 0.0f, ok ? f[u + 1] : 0.0f, ok ? f[u + 2] : 0.0f, ok ? f[u + 3] : 0.0f);
        }
      }
    }
    pf_wave_sync();
    if (t0 + 32 * NW < r1) issue(t0 + 32 * NW);

    floatx16 c;
    float old[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      // unconditional (clamped) load, masked below
      const int64_t rr = min(t0 + pf_mfma_row(lane, v), l - 1);
      old[v] = Ah[rr * r + min(col, r - 1)];
    }
    if (apply) {
#pragma unroll
      for (int v = 0; v < 16; ++v) c[v] = 0.0f;
      // operands of group g4 + 1 are fetched from LDS while the MFMAs of group g4 run
      auto lds4 = [&](const float* base, int g4) {
        return *reinterpret_cast<const float4*>(&base[col * LDX + half * KH + 4 * g4]);
      };
      float4 xa = lds4(x_s, 0);
      float4 mb;
      if constexpr (MT_LDS) mb = lds4(mt_s, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, MT_LDS ? 2 : 1, 0);  // the first reads have their own slot
#pragma unroll
      for (int g4 = 0; g4 < KH / 4; ++g4) {
        float4 xn = xa, mn = mb;
        if (g4 + 1 < KH / 4) {
          xn = lds4(x_s, g4 + 1);
          if constexpr (MT_LDS) mn = lds4(mt_s, g4 + 1);
        }
        if constexpr (!MT_LDS)
          mb = make_float4(mt[(4 * g4) % (MT_LDS ? 1 : KH)], mt[(4 * g4 + 1) % (MT_LDS ? 1 : KH)],
                           mt[(4 * g4 + 2) % (MT_LDS ? 1 : KH)], mt[(4 * g4 + 3) % (MT_LDS ? 1 : KH)]);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(xa.x, mb.x, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(xa.y, mb.y, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(xa.z, mb.z, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(xa.w, mb.w, c, 0, 0, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, MT_LDS ? 2 : 1, 0);  // DS reads of the next group
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);               // then this group's MFMAs
        xa = xn;
        if constexpr (MT_LDS) mb = mn;
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = pf_mfma_row(lane, v);
        if (row < rows && col < r) {
          const float df = old[v] - c[v];
          dsum = fmaf(df, df, dsum);
          Ah[(t0 + row) * r + col] = c[v];
        }
      }
    } else {
#pragma unroll
      for (int v = 0; v < 16; ++v) c[v] = (pf_mfma_row(lane, v) < rows && col < r) ? old[v] : 0.0f;
    }
    auto ldsb = [&](int v, float (&xb)[NB]) {
      const int row = pf_mfma_row(lane, v);
      if constexpr (NB == 1) {
        xb[0] = x_s[row * LDX + col];
      } else if constexpr (NB == 2) {
        const float2 t = *reinterpret_cast<const float2*>(&x_s[row * LDX + col * 2]);
        xb[0] = t.x; xb[1] = t.y;
      } else {
#pragma unroll
        for (int q = 0; q < NB / 4; ++q) {
          const float4 t = *reinterpret_cast<const float4*>(&x_s[row * LDX + col * NB + 4 * q]);
          xb[4 * q] = t.x; xb[4 * q + 1] = t.y; xb[4 * q + 2] = t.z; xb[4 * q + 3] = t.w;
        }
      }
    };
    float xb[NB];
    ldsb(0, xb);
    __builtin_amdgcn_sched_group_barrier(0x100, NB == 8 ? 2 : 1, 0);  // the first read has its own slot
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      float xn[NB];
      if (v + 1 < 16) ldsb(v + 1, xn);
      gAA = __builtin_amdgcn_mfma_f32_32x32x2f32(c[v], c[v], gAA, 0, 0, 0);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) gAX[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(c[v], xb[nb], gAX[nb], 0, 0, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, NB == 8 ? 2 : 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, NB + 1, 0);
      if (v + 1 < 16) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) xb[nb] = xn[nb];
      }
    }
    pf_wave_sync();  // this wave's reads of the tile precede its next staging writes
  }
  __syncthreads();  // every wave is done with its tile (and with Mt): the LDS is reused below

  // reduce the waves' tiles through LDS, one 32 x 32 block at a time
  const int ne = r * (r + d);
  float* out = part + ((int64_t)h * S + s) * ne;
  for (int blk = 0; blk <= NB; ++blk) {
    float* mine = sm + wave * 1024;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      float val = gAA[v];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        if (blk == nb + 1) val = gAX[nb][v];
      mine[pf_mfma_row(lane, v) * 32 + col] = val;
    }
    __syncthreads();
    for (int e = tid; e < 1024; e += NT) {
      float v = 0.0f;
#pragma unroll
      for (int w = 0; w < NW; ++w) v += sm[w * 1024 + e];
      const int m = e >> 5, n = e & 31;
      if (blk == 0) {
        if (m < r && n < r) out[m * (r + d) + n] = v;
      } else {
        const int cx = n * NB + (blk - 1);
        if (m < r && cx < d) out[m * (r + d) + r + cx] = v;
      }
    }
    __syncthreads();
  }
  if (apply) {
    dsum = wave_sum(dsum);
    if (lane == 0) red[wave] = dsum;
    __syncthreads();
    if (tid == 0) {
      float t = 0.0f;
      for (int w = 0; w < NW; ++w) t += red[w];
      delta_part[(int64_t)h * S + s] = t;
    }
  }
}

// ---- the same pass for bf16 input on the bf16 matrix cores (16 x the fp32 MFMA rate), without giving up
// fp32 accuracy: an fp32 number is the exact sum of three bf16 numbers (8 + 8 + 8 mantissa bits, by
// truncation), a product of two bf16 numbers is exact in fp32, and the MFMA accumulates in fp32.  So
//   apply:  C = X Mt^T            = X (Mt_hi + Mt_mid + Mt_lo)^T            (X is bf16 as it is: 3 products)
//   gram:   G_AX += C^T X         = (C_hi + C_mid + C_lo)^T X                (3 products)
//           G_AA += C^T C         = all piece pairs except lo*lo (8 products, error 2^-32; the pieces of a number
//                                   share its sign, so dropping mid*lo as well would bias the diagonal by ~2^-24,
//                                   which the r x r systems amplify by their condition number)
// with 32x32x16 tiles.  The Gram products sum over the rows of the tile, and C comes out of the apply in
// the accumulator layout (lane l, element v: row pf_mfma_row(l, v), column l % 32), where a lane holds
// rows 4 h .. 4 h + 3 (+ 8, 16, 24) of its column, h = l / 32: taken eight at a time these are the k
// elements of an MFMA operand, in an order that does not matter as long as the other operand uses the
// same one.  X gets into that layout by a product with the identity (2 MFMAs per 32 columns, exact).
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// the three bf16 pieces of x (as the upper halves of fp32 bit patterns)
__device__ __forceinline__ void pf_split3(float x, uint32_t& hi, uint32_t& mid, uint32_t& lo) {
  hi = __float_as_uint(x) & 0xffff0000u;
  const float r1 = x - __uint_as_float(hi);  // exact
  mid = __float_as_uint(r1) & 0xffff0000u;
  const float r2 = r1 - __uint_as_float(mid);  // exact, at most 8 significant bits
  lo = __float_as_uint(r2) & 0xffff0000u;
}
// two bf16 values (upper halves of a, b) in one word, a first
__device__ __forceinline__ uint32_t pf_pack2(uint32_t a, uint32_t b) { return (a >> 16) | (b & 0xffff0000u); }
__device__ __forceinline__ bf16x8 pf_bf16x8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  return __builtin_bit_cast(bf16x8, make_uint4(a, b, c, d));
}

// GRAMS = false: only A <- X Mt^T (the last pass of the iteration on Gram matrices, which needs neither the sums
// over the new rows nor their change): the old rows are not read and nothing is reduced.
// GIVEN = true: only the sums over the given rows of A (Mt must be null); the rows of A are requested one tile
// ahead, like the rows of X.
template <int NB, int NW, bool GRAMS = true, bool GIVEN = false>
__global__ __launch_bounds__(NW * kWave) void pf_pass_bf16_kernel(const bf16_t* __restrict__ X, int xh, int hq,
                                                                  int64_t l, int r, int d,
                                                                  const float* __restrict__ Mt, float* __restrict__ A,
                                                                  float* __restrict__ part,
                                                                  float* __restrict__ delta_part,
                                                                  const int* __restrict__ done_flag, int S) {
  if (done_flag && *done_flag) return;
  // row stride of a bf16 tile (elements): 16-byte operand reads want rows 4 banks apart, the transposing reads of
  // the GIVEN form 8 banks
  constexpr int LDB = 32 * NB + (GIVEN ? 16 : 8);
  constexpr int KB = 2 * NB;        // 16-column blocks of X
  constexpr int VEC = 8;
  constexpr int NL = 32 * 32 * NB / (kWave * VEC);
  constexpr int NT = NW * kWave;
  extern __shared__ __align__(16) float sm[];
  __shared__ float red[NW];
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int col = lane & 31, half = lane >> 5;
  uint16_t* x_s = reinterpret_cast<uint16_t*>(sm) + wave * 32 * LDB;           // this wave's rows of X
  uint16_t* mt_s = reinterpret_cast<uint16_t*>(sm) + NW * 32 * LDB;            // [3][32][LDB] pieces of Mt
  const int h = blockIdx.y, s = blockIdx.x;
  const int b = h / hq, head = h % hq;
  const int64_t xhead = (int64_t)b * xh + head / (hq / xh);
  const bf16_t* Xh = X + xhead * l * d;
  float* Ah = A + (int64_t)h * l * r;
  const bool apply = !GIVEN && Mt != nullptr;
  const bool full_rows = d == 32 * NB;

  if (apply) {
    const float* Mh = Mt + (int64_t)h * r * d;
    for (int e = tid; e < 32 * 32 * NB; e += NT) {
      const int n = e / (32 * NB), k = e % (32 * NB);
      const float v = Mh[min(n, r - 1) * d + min(k, d - 1)];
      uint32_t p0, p1, p2;
      pf_split3((n < r && k < d) ? v : 0.0f, p0, p1, p2);
      mt_s[(0 * 32 + n) * LDB + k] = (uint16_t)(p0 >> 16);
      mt_s[(1 * 32 + n) * LDB + k] = (uint16_t)(p1 >> 16);
      mt_s[(2 * 32 + n) * LDB + k] = (uint16_t)(p2 >> 16);
    }
  }
  for (int e = lane; e < 32 * LDB / 2; e += kWave) reinterpret_cast<uint32_t*>(x_s)[e] = 0u;

  const int64_t rows_per_split = (((l + S - 1) / S) + 31) / 32 * 32;
  const int64_t r0 = (int64_t)s * rows_per_split;
  const int64_t r1 = min(l, r0 + rows_per_split);

  floatx16 gAA;
  floatx16 gAX[NB];
#pragma unroll
  for (int v = 0; v < 16; ++v) gAA[v] = 0.0f;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int v = 0; v < 16; ++v) gAX[nb][v] = 0.0f;
  float dsum = 0.0f;
  // B operand of the identity product for the two 16-column halves of a 32-column block: element j of
  // lane (col, half) is row 16 kb2 + 8 half + j of the identity, column col
  bf16x8 ident[2];
#pragma unroll
  for (int kb2 = 0; kb2 < 2; ++kb2) {
    uint32_t w[4];
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int k0 = 16 * kb2 + 8 * half + 2 * jj;
      w[jj] = (col == k0 ? 0x3f80u : 0u) | (col == k0 + 1 ? 0x3f800000u : 0u);  // bf16 1.0 = 0x3f80
    }
    ident[kb2] = pf_bf16x8(w[0], w[1], w[2], w[3]);
  }

  uint4 pre[NL];
  auto issue = [&](int64_t t0) {
    const int nvalid = t0 < r1 ? (int)min((int64_t)32, r1 - t0) * d : 0;
    const int64_t base = (t0 < r1 ? t0 : r0) * d;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int e = (((i + wave) % NL) * kWave + lane) * VEC;  // (the waves start at different KB of their tiles)
      pre[i] = *reinterpret_cast<const uint4*>(Xh + base + (e < nvalid ? e : 0));
    }
  };
  float old_next[GIVEN ? 16 : 1];
  auto issue_old = [&](int64_t t0) {
    if constexpr (GIVEN) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int64_t rr = min(t0 + pf_mfma_row(lane, v), l - 1);
        old_next[v] = Ah[rr * r + min(col, r - 1)];
      }
    }
  };
  if (r0 + (int64_t)wave * 32 < r1) {
    issue(r0 + (int64_t)wave * 32);
    issue_old(r0 + (int64_t)wave * 32);
  }
  __syncthreads();  // Mt staged, tiles cleared

  for (int64_t t0 = r0 + (int64_t)wave * 32; t0 < r1; t0 += 32 * NW) {
    const int rows = (int)min((int64_t)32, r1 - t0);
    {
      const int nvalid = rows * d;
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const int e = (((i + wave) % NL) * kWave + lane) * VEC;
        if (e < 32 * d) {
          const int row = full_rows ? e / (32 * NB) : e / d;
          const int c0 = full_rows ? e % (32 * NB) : e - row * d;
          *reinterpret_cast<uint4*>(&x_s[row * LDB + c0]) = e < nvalid ? pre[i] : make_uint4(0, 0, 0, 0);
        }
      }
    }
    pf_wave_sync();
    floatx16 c;
    float old[16];
    if constexpr (GIVEN) {
#pragma unroll
      for (int v = 0; v < 16; ++v) old[v] = old_next[v];
    }
    if (t0 + 32 * NW < r1) {
      issue(t0 + 32 * NW);
      issue_old(t0 + 32 * NW);
    }
    if constexpr (GRAMS && !GIVEN) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int64_t rr = min(t0 + pf_mfma_row(lane, v), l - 1);
        old[v] = Ah[rr * r + min(col, r - 1)];
      }
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) c[v] = 0.0f;
    auto x_op = [&](int kb) {  // rows of X as an A operand: row col, columns 16 kb + 8 half .. + 7
      return *reinterpret_cast<const bf16x8*>(&x_s[col * LDB + kb * 16 + 8 * half]);
    };
    if (apply) {
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const bf16x8 a = x_op(kb);
#pragma unroll
        for (int p = 0; p < 3; ++p) {
          const bf16x8 m = *reinterpret_cast<const bf16x8*>(&mt_s[(p * 32 + col) * LDB + kb * 16 + 8 * half]);
          c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, m, c, 0, 0, 0);
        }
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = pf_mfma_row(lane, v);
        if (row < rows && col < r) {
          if constexpr (GRAMS) {
            const float df = old[v] - c[v];
            dsum = fmaf(df, df, dsum);
          }
          Ah[(t0 + row) * r + col] = c[v];
        }
      }
    } else {
#pragma unroll
      for (int v = 0; v < 16; ++v) c[v] = (pf_mfma_row(lane, v) < rows && col < r) ? old[v] : 0.0f;
    }
    if constexpr (!GRAMS) {
      pf_wave_sync();  // this wave's reads of the tile precede its next staging writes
      continue;
    }
    // the three pieces of C, eight rows (one k block) at a time
    bf16x8 cp[3][2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      uint32_t pc[3][8];
#pragma unroll
      for (int j = 0; j < 8; ++j) pf_split3(c[8 * kb + j], pc[0][j], pc[1][j], pc[2][j]);
#pragma unroll
      for (int p = 0; p < 3; ++p)
        cp[p][kb] = pf_bf16x8(pf_pack2(pc[p][0], pc[p][1]), pf_pack2(pc[p][2], pc[p][3]), pf_pack2(pc[p][4], pc[p][5]),
                              pf_pack2(pc[p][6], pc[p][7]));
    }
    // The matrix cores do not round to nearest when they add to their accumulator: over thousands of
    // additions to a growing sum that is a bias (measured: -2e-5 relative on a sum of 16K squares, ten times
    // the fp32 pipe's).  So a tile's products are summed in a fresh accumulator, smallest pieces first, and
    // the tile's sum joins the running total by an ordinary fp32 addition.
    {
      floatx16 t;
#pragma unroll
      for (int v = 0; v < 16; ++v) t[v] = 0.0f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cp[1][kb], cp[2][kb], t, 0, 0, 0);
        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cp[2][kb], cp[1][kb], t, 0, 0, 0);
        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cp[0][kb], cp[2][kb], t, 0, 0, 0);
        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cp[2][kb], cp[0][kb], t, 0, 0, 0);
      }
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cp[1][kb], cp[1][kb], t, 0, 0, 0);
        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cp[0][kb], cp[1][kb], t, 0, 0, 0);
        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cp[1][kb], cp[0][kb], t, 0, 0, 0);
      }
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cp[0][kb], cp[0][kb], t, 0, 0, 0);
#pragma unroll
      for (int v = 0; v < 16; ++v) gAA[v] += t[v];
    }
    // per 32 columns of X: the block in the accumulator layout (identity product), packed to bf16 --
    // xb[kb] = this lane's eight rows of k block kb, column 32 nb + col -- then its Gram products
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      bf16x8 xb[2];
      if constexpr (GIVEN) {
        // the transposing LDS read hands a lane four successive rows of its column (within 16 lanes, lane s points
        // at row s / 4, columns 4 (s % 4) .. + 3, and lane t receives column t of the four rows): rows
        // 16 kb + 4 half .. + 3 and the same + 8, the order of the accumulator layout
        typedef short v4s __attribute__((ext_vector_type(4)));
        typedef v4s __attribute__((address_space(3))) * lds_v4s;
        const int s16 = lane & 15;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          const uint16_t* p = &x_s[(16 * kb + 4 * half + (s16 >> 2)) * LDB + 32 * nb + (col & 16) + 4 * (s16 & 3)];
          const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)p);
          const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)(p + 8 * LDB));
          xb[kb] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
      } else {
        floatx16 xa;
#pragma unroll
        for (int v = 0; v < 16; ++v) xa[v] = 0.0f;
        xa = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x_op(2 * nb), ident[0], xa, 0, 0, 0);
        xa = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x_op(2 * nb + 1), ident[1], xa, 0, 0, 0);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
          xb[kb] = pf_bf16x8(pf_pack2(__float_as_uint(xa[8 * kb + 0]), __float_as_uint(xa[8 * kb + 1])),
                             pf_pack2(__float_as_uint(xa[8 * kb + 2]), __float_as_uint(xa[8 * kb + 3])),
                             pf_pack2(__float_as_uint(xa[8 * kb + 4]), __float_as_uint(xa[8 * kb + 5])),
                             pf_pack2(__float_as_uint(xa[8 * kb + 6]), __float_as_uint(xa[8 * kb + 7])));
      }
      floatx16 t;
#pragma unroll
      for (int v = 0; v < 16; ++v) t[v] = 0.0f;
#pragma unroll
      for (int p = 2; p >= 0; --p)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cp[p][kb], xb[kb], t, 0, 0, 0);
#pragma unroll
      for (int v = 0; v < 16; ++v) gAX[nb][v] += t[v];
    }
    pf_wave_sync();  // this wave's reads of the tile precede its next staging writes
  }
  if constexpr (!GRAMS) return;
  __syncthreads();  // every wave is done with its tile (and with Mt): the LDS is reused below

  // reduce the waves' tiles through LDS, one 32 x 32 block at a time (tile nb of G_AX: columns 32 nb + n)
  const int ne = r * (r + d);
  float* out = part + ((int64_t)h * S + s) * ne;
  for (int blk = 0; blk <= NB; ++blk) {
    float* mine = sm + wave * 1024;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      float val = gAA[v];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        if (blk == nb + 1) val = gAX[nb][v];
      mine[pf_mfma_row(lane, v) * 32 + col] = val;
    }
    __syncthreads();
    for (int e = tid; e < 1024; e += NT) {
      float v = 0.0f;
#pragma unroll
      for (int w = 0; w < NW; ++w) v += sm[w * 1024 + e];
      const int m = e >> 5, n = e & 31;
      if (blk == 0) {
        if (m < r && n < r) out[m * (r + d) + n] = v;
      } else {
        const int cx = 32 * (blk - 1) + n;
        if (m < r && cx < d) out[m * (r + d) + r + cx] = v;
      }
    }
    __syncthreads();
  }
  if (apply) {
    dsum = wave_sum(dsum);
    if (lane == 0) red[wave] = dsum;
    __syncthreads();
    if (tid == 0) {
      float t = 0.0f;
      for (int w = 0; w < NW; ++w) t += red[w];
      delta_part[(int64_t)h * S + s] = t;
    }
  }
}

// ---- small per-head systems, r <= 32: X = G^-1 RHS for a packed block [G (r x r) | RHS (r x d)] in LDS.
// Gauss-Jordan elimination of [G | RHS] as symmetric sweeps on the matrix cores, 64 columns of the
// right-hand side per wave (every wave repeats the sweeps of G itself).  No pivoting: G is a Gram matrix
// (plus B B^T), positive definite.
struct PfSmallShared {
  __align__(16) float scale[kPfSmallThreads / kWave][32];  // row scales of the solve each wave has in flight
};

// X = G^-1 RHS for the packed block G0 = [G (r x r) | RHS (r x d)] in LDS: the waves of the workgroup share
// the 32-column blocks of the right-hand side, two per solve; emit(i, j, x) for i < r, j < d.
template <typename Emit>
__device__ __forceinline__ void pf_solve_blocks(const float* G0, int r, int d, int cb0, float* scale, Emit&& emit) {
  const int ld = r + d;
  solve_sweep_mfma<2>([&](int i, int j) { return G0[min(i, r - 1) * ld + min(j, r - 1)]; },
                      [&](int b, int i, int col) {
                        const int j = (cb0 + b) * 32 + col;
                        const float x = G0[min(i, r - 1) * ld + r + min(j, d - 1)];
                        return j < d ? x : 0.0f;
                      },
                      r, scale,
                      [&](int b, int i, int col, float x) {
                        const int j = (cb0 + b) * 32 + col;
                        if (j < d) emit(i, j, x);
                      });
}

// sum of the S partial [r][r+d] blocks; 16 elements x 8 partials of loads in flight per thread
__device__ __forceinline__ void pf_reduce_part(const float* __restrict__ part, int S, int ne, float* dst) {
  constexpr int EB = 16;
  for (int e0 = threadIdx.x; e0 < ne; e0 += EB * kPfSmallThreads) {
    float v[EB];
    double w[EB];  // (more than 16 partial sums -- long prompts -- are added in fp64)
#pragma unroll
    for (int q = 0; q < EB; ++q) {
      v[q] = 0.0f;
      w[q] = 0.0;
    }
    for (int s0 = 0; s0 < S; s0 += 8) {
      float x[EB][8];
#pragma unroll
      for (int q = 0; q < EB; ++q)
#pragma unroll
        for (int u = 0; u < 8; ++u)
          x[q][u] = part[(int64_t)min(s0 + u, S - 1) * ne + min(e0 + q * kPfSmallThreads, ne - 1)];
#pragma unroll
      for (int q = 0; q < EB; ++q)
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < S) {
            v[q] += x[q][u];
            w[q] += (double)x[q][u];
          }
    }
#pragma unroll
    for (int q = 0; q < EB; ++q)
      if (e0 + q * kPfSmallThreads < ne) dst[e0 + q * kPfSmallThreads] = S > 16 ? (float)w[q] : v[q];
  }
}

// G0[i][c] (packed [r][r+d]) <- G[i][c] + (c < r ? (B B^T)[i][c] : B[i][c-r]),  B in LDS [r][d+4], d % 4 == 0
__device__ __forceinline__ void pf_add_bbt(const float* G, const float* Bs, int r, int d, float* G0) {
  const int ldb = d + 4;
  // right-hand side block
  for (int e = threadIdx.x; e < r * d; e += kPfSmallThreads) {
    const int i = e / d, c = e - i * d;
    G0[i * (r + d) + r + c] = G[i * (r + d) + r + c] + Bs[i * ldb + c];
  }
  // Gram block: lanes run over c (16-byte reads, conflict-free at this row stride), i is wave-uniform
  for (int o = threadIdx.x; o < 32 * r; o += kPfSmallThreads) {
    const int i = o >> 5, c = o & 31;
    if (c < r) {
      const float4* bi = reinterpret_cast<const float4*>(Bs + i * ldb);
      const float4* bc = reinterpret_cast<const float4*>(Bs + c * ldb);
      float g0 = 0.0f, g1 = 0.0f;
      for (int x = 0; x < d / 4; ++x) {
        const float4 a = bi[x], b = bc[x];
        g0 = fmaf(a.x, b.x, g0); g1 = fmaf(a.y, b.y, g1);
        g0 = fmaf(a.z, b.z, g0); g1 = fmaf(a.w, b.w, g1);
      }
      G0[i * (r + d) + c] = G[i * (r + d) + c] + (g0 + g1);
    }
  }
}

// stage 0: (stopping test) B_Q, B_K from the current Grams, then Mt for the A_Q update
// stage 1: Mt for the A_K update from the new A_Q Grams
// stage 2: final B_Q, B_K
__global__ __launch_bounds__(kPfSmallThreads) void pf_small32_kernel(int stage, int it, const float* __restrict__ partQ,
                                                                     const float* __restrict__ partK, int S, int bh,
                                                                     int r, int d, int64_t l, float tol,
                                                                     const float* __restrict__ delta_all,
                                                                     int* __restrict__ flags, float* __restrict__ Mt,
                                                                     float* __restrict__ b_q, float* __restrict__ b_k) {
  extern __shared__ __align__(16) float sm[];
  const int ne = r * (r + d);
  float* G1 = sm;            // [r][r+d] packed
  float* G2 = G1 + ne;       // [r][r+d] packed
  float* G0 = G2 + ne;       // [r][r+d] packed, system being solved
  float* Bs = sm + ((3 * ne + 3) & ~3);  // [r][d+4], 16-byte aligned
  __shared__ PfSmallShared sh;
  __shared__ int s_done;
  __shared__ float s_red[kPfSmallThreads / kWave][2];
  const int tid = threadIdx.x;
  const int h = blockIdx.x;
  const int wave = wave_id();
  constexpr int kWaves = kPfSmallThreads / kWave;
  const int njob = (d + 63) / 64;  // pairs of 32-column blocks of a right-hand side

  if (stage == 0) {
    int done = 0;
    if (it > 0) {
      done = flags[it - 1];
      if (!done) {
        const float* dq = delta_all + ((int64_t)(it - 1) * 2 + 0) * bh * S;
        const float* dk = delta_all + ((int64_t)(it - 1) * 2 + 1) * bh * S;
        float sq = 0.0f, sk = 0.0f;
        for (int i = tid; i < bh * S; i += kPfSmallThreads) {
          sq += dq[i];
          sk += dk[i];
        }
        sq = wave_sum(sq);
        sk = wave_sum(sk);
        if (lane_id() == 0) {
          s_red[wave_id()][0] = sq;
          s_red[wave_id()][1] = sk;
        }
        __syncthreads();
        if (tid == 0) {
          float tq = 0.0f, tk = 0.0f;
          for (int w = 0; w < kPfSmallThreads / kWave; ++w) {
            tq += s_red[w][0];
            tk += s_red[w][1];
          }
          const float n = (float)bh * (float)l * (float)r;
          s_done = fmaxf(tq / n, tk / n) < tol;
        }
        __syncthreads();
        done = s_done;
      }
    }
    // every head computes the same decision from data that no launch of this iteration overwrites
    if (h == 0 && tid == 0) flags[it] = done;
    if (done) return;
  } else if (stage == 1) {
    if (flags[it]) return;
  }

  const float* pq = partQ + (int64_t)h * S * ne;
  const float* pk = partK + (int64_t)h * S * ne;
  if (stage == 0 || stage == 2) {
    pf_reduce_part(pq, S, ne, G1);
    pf_reduce_part(pk, S, ne, G2);
    __syncthreads();
    // B_Q = (A_Q^T A_Q)^-1 A_Q^T Q and B_K likewise: both systems side by side, two column blocks per wave
    for (int job = wave; job < 2 * njob; job += kWaves) {
      if (job < njob) {
        pf_solve_blocks(G1, r, d, 2 * job, sh.scale[wave], [&](int i, int j, float x) {
          Bs[i * (d + 4) + j] = x;
          b_q[(int64_t)h * r * d + i * d + j] = x;
        });
      } else {
        pf_solve_blocks(G2, r, d, 2 * (job - njob), sh.scale[wave],
                        [&](int i, int j, float x) { b_k[(int64_t)h * r * d + i * d + j] = x; });
      }
    }
    if (stage == 2) return;
    __syncthreads();
    // Mt_Q = (A_K^T A_K + B_Q B_Q^T)^-1 (A_K^T K + B_Q)
    pf_add_bbt(G2, Bs, r, d, G0);
  } else {
    // stage 1: Mt_K = (A_Q^T A_Q + B_K B_K^T)^-1 (A_Q^T Q + B_K)
    pf_reduce_part(pq, S, ne, G1);
    for (int e = tid; e < r * d; e += kPfSmallThreads) Bs[(e / d) * (d + 4) + e % d] = b_k[(int64_t)h * r * d + e];
    __syncthreads();
    pf_add_bbt(G1, Bs, r, d, G0);
  }
  __syncthreads();
  for (int job = wave; job < njob; job += kWaves)
    pf_solve_blocks(G0, r, d, 2 * job, sh.scale[wave],
                    [&](int i, int j, float x) { Mt[(int64_t)h * r * d + i * d + j] = x; });
}

template <typename T>
using PfPassFn = void (*)(const T*, int, int, int64_t, int, int, const float*, float*, float*, float*, const int*, int);

template <typename T>
static int prefill_impl(lrqk_ctx* ctx, const void* q, const void* k, float* a_q, float* a_k, float* b_q, float* b_k,
                        int b, int hq, int hkv, int64_t l, int r, int d, int max_iter, float tol, hipStream_t st) {
  constexpr int VEC = Vec16<T>::N;
  const int bh = b * hq;
  const int ne = r * (r + d);
  const bool mfma = r <= 32 && d % VEC == 0 && d <= 256 && ((uintptr_t)q % 16 == 0) && ((uintptr_t)k % 16 == 0);
  const bool small32 = r <= 32 && d <= kPfSmallThreads - 32 && d % 4 == 0;
  LRQK_REQUIRE(mfma || ne <= kPfThreads * kPfMaxPer, LRQK_ELIMIT, "r*(r+d)=%d exceeds %d", ne, kPfThreads * kPfMaxPer);
  // (the general pass: a 16 x 16 thread grid with ceil(r / 16) rows and 48 / that many columns of the sums per thread)
  LRQK_REQUIRE(mfma || (r <= 64 && 16 * (kPfMaxPer / ((r + 15) / 16)) >= r + d), LRQK_ELIMIT,
               "r=%d with rows of %d elements exceeds the general kernel's tile", r, d);
  // splits of the long axis: about one workgroup per CU (a pass keeps one wave per SIMD busy), but
  // at least 128 rows per split
  int S = std::max(1, std::min(64, 256 / bh));
  // The row-by-row formulation solves its r x r systems from these sums in fp32, and a split adds its rows up in
  // fp32: at most 2048 rows per split there (the partial sums are added in fp64), however few splits fill the GPU.
  // (The iteration on Gram matrices takes only its first sums from here, where the systems are well conditioned.)
  // (At most 64 splits per head: beyond 128K rows a split of the row-by-row formulation adds up l / 64 rows.)
  // bf16 rows of 128 elements, 16-byte aligned: every iteration runs on the d x d Gram matrices (fp64)
  const bool gram_domain = sizeof(T) == 2 && mfma && d == 128 && r <= 32 && !getenv("LRQK_PREFILL_ROWWISE");
  if (!gram_domain) S = (int)std::min<int64_t>(64, std::max<int64_t>(S, (l + 2047) / 2048));
  S = (int)std::max<int64_t>(1, std::min<int64_t>(S, (l + 127) / 128));
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

  PfPassFn<T> pass = pf_pass_generic_kernel<T>;
  size_t smem_pass = ((size_t)kPfTile * (d + 1) + (size_t)kPfTile * (r + 1) + (size_t)r * (d + 1)) * sizeof(float);
  int pass_threads = kPfThreads;
  if (mfma) {
    const int nb = d <= 32 ? 1 : d <= 64 ? 2 : d <= 128 ? 4 : 8;
    pass = nb == 1 ? pf_pass_mfma_kernel<T, 1, 8, true> : nb == 2 ? pf_pass_mfma_kernel<T, 2, 8, true>
         : nb == 4 ? pf_pass_mfma_kernel<T, 4, 8, true> : pf_pass_mfma_kernel<T, 8, 4, false>;
    const int nw = nb == 8 ? 4 : 8;
    pass_threads = nw * kWave;
    smem_pass = std::max((size_t)(nw + (nb == 8 ? 0 : 1)) * 32 * (32 * nb + 4), (size_t)nw * 1024) * sizeof(float);
    if constexpr (sizeof(T) == 2) {
      if (nb <= 4) {  // bf16 input: the pass on the bf16 matrix cores (three-piece split, fp32 accuracy)
        pass = nb == 1 ? pf_pass_bf16_kernel<1, 8> : nb == 2 ? pf_pass_bf16_kernel<2, 8> : pf_pass_bf16_kernel<4, 8>;
        smem_pass = std::max((size_t)(8 + 3) * 32 * (32 * nb + 16) * sizeof(uint16_t), (size_t)8 * 1024 * sizeof(float));
      }
    }
  }
  auto small = small32 ? pf_small32_kernel : pf_small_generic_kernel;
  const size_t smem_small = small32 ? ((size_t)3 * ne + 4 + (size_t)r * (d + 4)) * sizeof(float)
                                    : ((size_t)ne + (size_t)r * (r + d + 1) + (size_t)r * (d + 1)) * sizeof(float);
  LRQK_REQUIRE(smem_small <= 160 * 1024 && smem_pass <= 160 * 1024, LRQK_ELIMIT, "r=%d d=%d need too much LDS", r, d);
  if (smem_pass > 48 * 1024)
    LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)pass, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_pass));
  if (smem_small > 48 * 1024)
    LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)small, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_small));
  const dim3 grid((unsigned)S, (unsigned)bh), blk((unsigned)pass_threads), sblk(small32 ? kPfSmallThreads : kPfThreads);
  const T* Q = (const T*)q;
  const T* K = (const T*)k;
  // bf16 rows of 128 elements: every iteration on the d x d Gram matrices (fp64), then one pass per side that
  // applies the last Mq, Mk; the Q side's sums over the given factors are formed together with Q^T Q (one
  // reading of Q), the K side's by the pass below (A_K has a head per query head, K per kv head)
  const bool fused_sums = gram_domain && !getenv("LRQK_PREFILL_SEPARATE_SUMS");  // (the Q side's, with Q^T Q)
  // (the iteration on Gram matrices writes every stopping flag before it reads it)
  if (!gram_domain) LRQK_HIP_CHECK(hipMemsetAsync(flags, 0, (size_t)(iters + 1) * sizeof(int), st));
  {
    PfPassFn<T> first = pass;  // the sums over the given initial factors
    if constexpr (sizeof(T) == 2) {
      if (mfma && d == 128) {
        first = (PfPassFn<T>)pf_pass_bf16_kernel<4, 8, true, true>;
        if (smem_pass > 48 * 1024)
          LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)first, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_pass));
      }
    }
    if (!fused_sums)
      hipLaunchKernelGGL(first, grid, blk, smem_pass, st, Q, hq, hq, l, r, d, (const float*)nullptr, a_q, partQ,
                         (float*)nullptr, (const int*)nullptr, S);
    hipLaunchKernelGGL(first, grid, blk, smem_pass, st, K, hkv, hq, l, r, d, (const float*)nullptr, a_k, partK,
                       (float*)nullptr, (const int*)nullptr, S);
    LRQK_HIP_CHECK(hipGetLastError());
  }
  if constexpr (sizeof(T) == 2) {
    if (gram_domain) {
      float *mt_q = nullptr, *mt_k = nullptr;
      if ((rc = prefill_gram_domain(ctx, q, k, fused_sums ? nullptr : partQ, partK, S, fused_sums ? a_q : nullptr, b_q,
                                    b_k, b, hq, hkv, l, r, iters, tol, flags, &mt_q, &mt_k, st)))
        return rc;
      if (iters > 0) {
        PfPassFn<T> lean = (PfPassFn<T>)pf_pass_bf16_kernel<4, 8, false>;
        if (smem_pass > 48 * 1024)
          LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)lean, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_pass));
        hipLaunchKernelGGL(lean, grid, blk, smem_pass, st, Q, hq, hq, l, r, d, (const float*)mt_q, a_q, partQ, deltas,
                           (const int*)nullptr, S);
        int rck = LRQK_OK;
        if (getenv("LRQK_PREFILL_SEPARATE_SUMS") || !prefill_apply_shared(k, mt_k, a_k, b, hq, hkv, l, r, st, &rck))
          hipLaunchKernelGGL(lean, grid, blk, smem_pass, st, K, hkv, hq, l, r, d, (const float*)mt_k, a_k, partK,
                             deltas + (size_t)bh * S, (const int*)nullptr, S);
        if (rck) return rck;
        LRQK_HIP_CHECK(hipGetLastError());
      }
      return LRQK_OK;
    }
  }
  for (int it = 0; it < iters; ++it) {
    float* dq = deltas + ((size_t)it * 2 + 0) * bh * S;
    float* dk = deltas + ((size_t)it * 2 + 1) * bh * S;
    hipLaunchKernelGGL(small, dim3((unsigned)bh), sblk, smem_small, st, 0, it, partQ, partK, S, bh, r, d, l, tol,
                       deltas, flags, Mt, b_q, b_k);
    hipLaunchKernelGGL(pass, grid, blk, smem_pass, st, Q, hq, hq, l, r, d, (const float*)Mt, a_q, partQ, dq,
                       (const int*)(flags + it), S);
    hipLaunchKernelGGL(small, dim3((unsigned)bh), sblk, smem_small, st, 1, it, partQ, partK, S, bh, r, d, l, tol,
                       deltas, flags, Mt, b_q, b_k);
    hipLaunchKernelGGL(pass, grid, blk, smem_pass, st, K, hkv, hq, l, r, d, (const float*)Mt, a_k, partK, dk,
                       (const int*)(flags + it), S);
    LRQK_HIP_CHECK(hipGetLastError());
  }
  hipLaunchKernelGGL(small, dim3((unsigned)bh), sblk, smem_small, st, 2, iters, partQ, partK, S, bh, r, d, l, tol,
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
