// Prefill factorisation, iterations carried out on Gram matrices (bf16 input, d = 128, r <= 32).
//
// After the first half-step of lrqk_attention.py:359-421 every factor is a linear image of its input,
// A_Q = Q Mq and A_K = K Mk with Mq, Mk of size d x r.  Everything an iteration needs from the long axis
// is then a product with Sq = Q^T Q or Sk = K^T K (d x d):
//     A_Q^T A_Q = Mq^T Sq Mq,   A_Q^T Q = Mq^T Sq,   Q^T A_Q = Sq Mq   (likewise for K),
// and the change mse(A, A') that the stopping test looks at is
//     |A - A'|^2 = tr(A^T A) - 2 tr((A^T X) M') + tr(A'^T A').
// With (G, C) = (A^T A, A^T X) as the state of each side, one iteration is, in the reference's order
// (Gauss-Seidel: the A_K update sees the new A_Q),
//     B_Q = Gq^-1 Cq,  B_K = Gk^-1 Ck
//     Mq'^T = (Gk + B_Q B_Q^T)^-1 (Ck + B_Q)          T = Mq'^T Sq      Gq' = Mq'^T T^T     Cq' = T
//     Mk'^T = (Gq' + B_K B_K^T)^-1 (T + B_K)          U = Mk'^T Sk      Gk' = Mk'^T U^T     Ck' = U
// and this holds from the first iteration on (there G, C come from the given initial factors).  The long
// axis is read for Sq, Sk and the initial (G, C) before the loop and once more at the end, to form
// A_Q = Q Mq and A_K = K Mk: six passes whatever the iteration count, where the row-by-row formulation
// makes two per iteration plus two.
//
// Sq and Sk square the condition number of the inputs, so the d x d algebra is done in fp64 (vector
// ALU: these are 32 independent problems of a few MFLOP each); the sums Sq, Sk themselves are exact
// bf16 x bf16 products added in fp32 tile by tile and across tiles, then across splits in fp64.  Measured
// against the fp64 restatement the results are closer than the same iteration in fp32 LAPACK.
#include <algorithm>

#include "common.hpp"
#include "ctx.hpp"

namespace lrqk {

typedef float gd_floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 gd_bf16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ int gd_mfma_row(int lane, int v) { return ((v >> 2) << 3) + ((lane >> 5) << 2) + (v & 3); }

// ----------------------------------------------------------------------------- X^T X
// grid (S, x heads); 8 waves share the rows (128 per step, staged in LDS as they lie in memory); wave w owns
// the output blocks (w / 2, 2 (w % 2)) and (w / 2, 2 (w % 2) + 1) of 32 x 32.  A lane's operand for column
// block nb is eight rows of one column, read from the tile as eight 16-bit values; every 32-row tile is summed
// in a fresh accumulator and added to the running total in fp32 (the matrix cores do not round to nearest
// when they add to a large accumulator).
constexpr int kXtxWaves = 8, kXtxThreads = kXtxWaves * kWave, kXtxRows = 128, kXtxD = 128;
constexpr int kXtxLd = kXtxD + 16;  // bf16 elements per staged row: 288 bytes, so four successive rows start 8 banks apart

__global__ __launch_bounds__(kXtxThreads) void pf_xtx_kernel(const bf16_t* __restrict__ X, int64_t l,
                                                             float* __restrict__ part, int S) {
  __shared__ __align__(16) uint16_t x_s[kXtxRows * kXtxLd];
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int col = lane & 31, half = lane >> 5;
  const int xh = blockIdx.y, s = blockIdx.x;
  const bf16_t* Xh = X + (int64_t)xh * l * kXtxD;
  const int nb1 = wave >> 1, nb2 = 2 * (wave & 1);
  constexpr int NL = kXtxRows * kXtxD / (kXtxThreads * 8);  // 16-byte loads per thread and step
  // One step ahead is all that pays: with two steps of rows in flight per workgroup the kernel is slower
  // (65 against 54 us at 32 heads x 32K rows).
  uint4 pre_a[NL];
  auto issue = [&](int64_t t0, uint4 (&dst)[NL]) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int e = (i * kXtxThreads + tid) * 8;  // element of the 128 x 128 step
      const int64_t row = t0 + e / kXtxD;
      dst[i] = *reinterpret_cast<const uint4*>(Xh + min(row, l - 1) * kXtxD + e % kXtxD);
    }
  };
  gd_floatx16 acc0, acc1;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc0[v] = acc1[v] = 0.0f;
  // An operand of the 32x32x16 product, lane (col, half): rows row0 + 8 half .. + 7 of column 32 nb + col.  The
  // transposing LDS read hands a lane four successive rows of its column: within 16 lanes, lane s points at
  // row s / 4, columns 4 (s % 4) .. + 3, and lane t receives column t of the four rows.
  auto operand = [&](int row0, int nb) {
    const int s16 = lane & 15;
    const uint16_t* p = &x_s[(row0 + 8 * half + (s16 >> 2)) * kXtxLd + 32 * nb + (col & 16) + 4 * (s16 & 3)];
    typedef short gd_v4s __attribute__((ext_vector_type(4)));
    typedef gd_v4s __attribute__((address_space(3))) * gd_lds_v4s;
    const gd_v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((gd_lds_v4s)p);
    const gd_v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((gd_lds_v4s)(p + 4 * kXtxLd));
    return __builtin_bit_cast(gd_bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  // split s takes the steps s, s + S, ...: the workgroups of a head walk the head's rows side by side
  const int64_t stride = (int64_t)S * kXtxRows;
  // one step: stage `cur` (the rows from t0 on), ask for the next step into `cur`, multiply
  auto step = [&](int64_t t0, uint4 (&cur)[NL]) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int e = (i * kXtxThreads + tid) * 8;
      const int row = e / kXtxD;
      *reinterpret_cast<uint4*>(&x_s[row * kXtxLd + e % kXtxD]) = t0 + row < l ? cur[i] : make_uint4(0, 0, 0, 0);
    }
    __syncthreads();
    if (t0 + stride < l) issue(t0 + stride, cur);
    const int tiles = (int)min((int64_t)4, (l - t0 + 31) / 32);
    for (int tile = 0; tile < tiles; ++tile) {
      gd_floatx16 t0a, t1a;
#pragma unroll
      for (int v = 0; v < 16; ++v) t0a[v] = t1a[v] = 0.0f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const int row0 = 32 * tile + 16 * kb;
        const gd_bf16x8 a = operand(row0, nb1);
        const gd_bf16x8 b0 = operand(row0, nb2), b1 = operand(row0, nb2 + 1);
        t0a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b0, t0a, 0, 0, 0);
        t1a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b1, t1a, 0, 0, 0);
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        acc0[v] += t0a[v];
        acc1[v] += t1a[v];
      }
    }
    __syncthreads();
  };
  const int64_t first = (int64_t)s * kXtxRows;
  if (first < l) issue(first, pre_a);
  for (int64_t t0 = first; t0 < l; t0 += stride) step(t0, pre_a);
  float* out = part + ((int64_t)xh * S + s) * kXtxD * kXtxD;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int i = 32 * nb1 + gd_mfma_row(lane, v);
    out[i * kXtxD + 32 * nb2 + col] = acc0[v];
    out[i * kXtxD + 32 * (nb2 + 1) + col] = acc1[v];
  }
}

// S64[x][e] = sum over splits of part[x][s][e], in fp64
__global__ __launch_bounds__(256) void pf_xtx_reduce_kernel(const float* __restrict__ part, int S, int n,
                                                            double* __restrict__ out) {
  const int x = blockIdx.y;
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= n) return;
  double v = 0.0;
  for (int s = 0; s < S; ++s) v += (double)part[((int64_t)x * S + s) * n + e];
  out[(int64_t)x * n + e] = v;
}

// ----------------------------------------------------------------------------- d x d algebra, fp64
constexpr int kGdThreads = 320;   // two groups of 32 + 128 threads: one column of [W | RHS] each
constexpr int kGdGroup = 160;
constexpr int kGdD = 128;
constexpr int kGdLd = 34;         // doubles per row of a transposed r x d matrix in LDS ([d][34], 16-byte rows)
constexpr int kGdLg = 33;         // doubles per row of an r x r matrix in LDS

// Gauss-Jordan elimination of [W | RHS] (W 32 x 32 symmetric positive definite, rows/columns beyond r
// the identity), one column per thread of a group, the column in registers, two pivots per step: the owners of
// columns p, p + 1 publish them, every thread inverts the 2 x 2 pivot block itself (positive definite, no
// pivoting needed) and applies the rank-two update to its column.  One barrier per step: the two LDS buffers
// are used in turn, and a buffer is rewritten two steps later, when the barrier in between has every thread
// past its reads.  The pivot rows of a step sit at fixed register positions (0..3 for the two steps of the loop
// body, then the column is rotated by four), so every register index is static and the loop stays rolled.
// piv: 128 doubles of LDS per group.  Every thread of the workgroup calls this; `col` is the thread's column in
// its group (< 0: the thread only keeps the barriers).
__device__ __forceinline__ void gd_solve(double (&x)[32], int col, double* __restrict__ piv) {
  for (int pb = 0; pb < 32; pb += 4) {
#pragma unroll
    for (int q = 0; q < 4; q += 2) {
      double* pv = piv + (q >> 1) * 64;  // [2][32]: columns p and p + 1
      const int p = pb + q;
      if (col == p || col == p + 1) {
        double* mine = pv + (col - p) * 32;
#pragma unroll
        for (int i = 0; i < 32; ++i) mine[i] = x[i];
      }
      __syncthreads();
      if (col >= 0) {  // (wave-uniform but for the last wave of a group: idle threads stay off the LDS)
        // the two columns as 16-byte reads
        double c0[32], c1[32];
#pragma unroll
        for (int i = 0; i < 32; i += 2) {
          const double2 u0 = *reinterpret_cast<const double2*>(pv + i);
          const double2 u1 = *reinterpret_cast<const double2*>(pv + 32 + i);
          c0[i] = u0.x;
          c0[i + 1] = u0.y;
          c1[i] = u1.x;
          c1[i + 1] = u1.y;
        }
        // inverse of the pivot block [[a, b], [b', c]] (rows q, q + 1 of the two columns)
        const double a = c0[q], bb = c1[q], b2 = c0[q + 1], c = c1[q + 1];
        const double det = fma(a, c, -bb * b2);
        double inv = __builtin_amdgcn_rcp(det);
        inv = fma(fma(-det, inv, 1.0), inv, inv);
        inv = fma(fma(-det, inv, 1.0), inv, inv);
        const double xa = (c * x[q] - bb * x[q + 1]) * inv;
        const double xb = (a * x[q + 1] - b2 * x[q]) * inv;
#pragma unroll
        for (int i = 0; i < 32; ++i) {
          if (i != q && i != q + 1) x[i] = fma(-c0[i], xa, fma(-c1[i], xb, x[i]));
        }
        x[q] = xa;
        x[q + 1] = xb;
      }
    }
    // rotate by four: the next pivot rows move to positions 0..3
    const double t0 = x[0], t1 = x[1], t2 = x[2], t3 = x[3];
#pragma unroll
    for (int i = 0; i < 28; ++i) x[i] = x[i + 4];
    x[28] = t0;
    x[29] = t1;
    x[30] = t2;
    x[31] = t3;
  }
  __syncthreads();
}

// out[i][j] (+)= sum over c < 128 of PT[c][i] * RT[c][j]   (two r x d matrices, stored transposed), by threads
// 0..255: thread (i = tid / 8, j = 4 (tid % 8) .. + 3).  Rows/columns beyond r come out as what the zero
// padding of PT, RT gives.
__device__ __forceinline__ void gd_outer(const double* __restrict__ PT, const double* __restrict__ RT, double (&o)[4]) {
  const int tid = threadIdx.x;
  const int i = tid >> 3, j0 = (tid & 7) * 4;
  o[0] = o[1] = o[2] = o[3] = 0.0;
  if (tid < 256) {
#pragma unroll 4
    for (int c = 0; c < kGdD; ++c) {
      const double p = PT[c * kGdLd + i];
      const double2 ra = *reinterpret_cast<const double2*>(&RT[c * kGdLd + j0]);
      const double2 rb = *reinterpret_cast<const double2*>(&RT[c * kGdLd + j0 + 2]);
      o[0] = fma(p, ra.x, o[0]);
      o[1] = fma(p, ra.y, o[1]);
      o[2] = fma(p, rb.x, o[2]);
      o[3] = fma(p, rb.y, o[3]);
    }
  }
}

// TT[c][i] = sum over k of MT[k][i] * S[k][c]   (the transposed form of Mt S, S symmetric d x d in global
// memory) on the fp64 matrix cores: 16 x 16 x 4 tiles, A operand lane l = Mt[i0 + l % 16][k0 + l / 16] (from the
// LDS copy), B operand lane l = S[k0 + l / 16][c0 + l % 16] (16 independent loads per lane in flight), result
// element v of lane l = row l / 16 + 4 v, column l % 16 of the tile.  Waves 0..3 take 32 columns each.
// One barrier.
typedef double gd_v4d __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void gd_times_s(const double* __restrict__ MT, const double* __restrict__ S,
                                           double* __restrict__ TT) {
  const int lane = lane_id(), wave = wave_id();
  if (wave < 4) {
    const int li = lane & 15, lk = lane >> 4;
    const int c0 = 32 * wave;
    gd_v4d acc[2][2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int ct = 0; ct < 2; ++ct) acc[rt][ct] = gd_v4d{0.0, 0.0, 0.0, 0.0};
    for (int kb = 0; kb < kGdD; kb += 32) {
      double bv[8][2];
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) bv[u][ct] = S[(int64_t)(kb + 4 * u + lk) * kGdD + c0 + 16 * ct + li];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int k = kb + 4 * u + lk;
        const double a0 = MT[k * kGdLd + li], a1 = MT[k * kGdLd + 16 + li];
        acc[0][0] = __builtin_amdgcn_mfma_f64_16x16x4f64(a0, bv[u][0], acc[0][0], 0, 0, 0);
        acc[0][1] = __builtin_amdgcn_mfma_f64_16x16x4f64(a0, bv[u][1], acc[0][1], 0, 0, 0);
        acc[1][0] = __builtin_amdgcn_mfma_f64_16x16x4f64(a1, bv[u][0], acc[1][0], 0, 0, 0);
        acc[1][1] = __builtin_amdgcn_mfma_f64_16x16x4f64(a1, bv[u][1], acc[1][1], 0, 0, 0);
      }
    }
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int ct = 0; ct < 2; ++ct)
#pragma unroll
        for (int v = 0; v < 4; ++v) TT[(c0 + 16 * ct + li) * kGdLd + 16 * rt + lk + 4 * v] = acc[rt][ct][v];
  }
  __syncthreads();
}

// sum of v over the workgroup, result in every thread.  red: kGdThreads / 64 doubles.  Two barriers.
__device__ __forceinline__ double gd_block_sum(double v, double* red) {
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  if (lane_id() == 0) red[wave_id()] = v;
  __syncthreads();
  double t = 0.0;
  for (int w = 0; w < kGdThreads / kWave; ++w) t += red[w];
  __syncthreads();
  return t;
}

struct GdArgs {
  // initial (G, C) of the two sides as the first Gram passes left them: S partial sums of [r][r + d] floats per head
  const float* partQ;
  const float* partK;
  int S;
  const double* Sq;     // [bh][d][d]
  const double* Sk;     // [b * hkv][d][d]
  double* G;            // [2][bh][32][32]  (side 0: Q, 1: K), padded with the identity
  double* C;            // [2][bh][32][d]   zero rows beyond r
  double* delta;        // [iters][2][bh]   squared changes |A - A'|^2 per head
  int* flags;           // [iters + 1]
  float* Mt_q;          // [bh][r][d]  Mq^T, Mk^T for the final row-by-row pass
  float* Mt_k;
  float* b_q;           // [bh][r][d] outputs
  float* b_k;
  int bh, hq, hkv, r;
  int64_t l;
  float tol;
};

// The state (G, C) of both sides from the first Gram passes: S partial sums of [G | C] packed as [r][r + d]
// floats per head, added in fp64; G padded with the identity, C with zero rows.  grid (ceil(32 * 160 / 256), bh, 2).
__global__ __launch_bounds__(256) void pf_gramdom_init_kernel(GdArgs a) {
  const int h = blockIdx.y, side = blockIdx.z;
  const int r = a.r, d = kGdD;
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= 32 * (32 + d)) return;
  const int ne = r * (r + d);
  const float* part = (side ? a.partK : a.partQ) + (int64_t)h * a.S * ne;
  const int i = e / (32 + d), j = e % (32 + d);
  double v = 0.0;
  if (i < r && (j >= 32 || j < r)) {
    const int src = i * (r + d) + (j < 32 ? j : r + (j - 32));
    for (int s = 0; s < a.S; ++s) v += (double)part[(int64_t)s * ne + src];
  } else if (j < 32) {
    v = i == j ? 1.0 : 0.0;
  }
  if (j < 32)
    a.G[((int64_t)side * a.bh + h) * 1024 + i * 32 + j] = v;
  else
    a.C[((int64_t)side * a.bh + h) * 32 * d + i * d + (j - 32)] = v;
}

// stage 0: one iteration `it`; stage 2: the final B_Q, B_K from the state.
__global__ __launch_bounds__(kGdThreads) void pf_gramdom_kernel(int stage, int it, GdArgs a) {
  extern __shared__ __align__(16) double gsm[];
  double* MT = gsm;                         // [128][34]  Mq'^T, later Mk'^T (transposed storage)
  double* TT = MT + kGdD * kGdLd;           // [128][34]  T, later U
  double* BT = TT + kGdD * kGdLd;           // [128][34]  B_Q, later B_K
  double* Gs = BT + kGdD * kGdLd;           // [3][32][33]
  double* piv = Gs + 3 * 32 * kGdLg;        // [2 groups][2][2][32]
  double* red = piv + 256;                  // [8]
  const int tid = threadIdx.x;
  const int h = blockIdx.x;
  const int r = a.r, d = kGdD, bh = a.bh;
  const int grp = tid >= kGdGroup ? 1 : 0;     // 0: the Q side's system, 1: the K side's
  const int t = tid - grp * kGdGroup;          // column of [W | RHS] within the group
  const int c = t - 32;                        // RHS column (valid when t >= 32)
  const int b = h / a.hq, kvh = (h % a.hq) / (a.hq / a.hkv);
  const double* Sq = a.Sq + (int64_t)h * d * d;
  const double* Sk = a.Sk + ((int64_t)b * a.hkv + kvh) * d * d;
  double* Gq = a.G + (int64_t)h * 1024;
  double* Gk = a.G + ((int64_t)bh + h) * 1024;
  double* Cq = a.C + (int64_t)h * 32 * d;
  double* Ck = a.C + ((int64_t)bh + h) * 32 * d;

  if (stage == 0) {
    // ---- the stopping test of the previous iteration (batch-wide, as the reference takes it)
    int done = 0;
    if (it > 0) {
      done = a.flags[it - 1];
      if (!done) {
        const double* dq = a.delta + ((int64_t)(it - 1) * 2 + 0) * bh;
        const double* dk = a.delta + ((int64_t)(it - 1) * 2 + 1) * bh;
        double sq = 0.0, sk = 0.0;
        for (int i = tid; i < bh; i += kGdThreads) {
          sq += dq[i];
          sk += dk[i];
        }
        sq = gd_block_sum(sq, red);
        sk = gd_block_sum(sk, red);
        const double n = (double)bh * (double)a.l * (double)r;
        done = fmax(sq / n, sk / n) < (double)a.tol;
      }
    }
    if (h == 0 && tid == 0) a.flags[it] = done;
    if (done) return;
  }

  // ---- B_Q = Gq^-1 Cq and B_K = Gk^-1 Ck, side by side
  double x[32];
  {
    const double* G = grp ? Gk : Gq;
    const double* C = grp ? Ck : Cq;
#pragma unroll
    for (int i = 0; i < 32; ++i) x[i] = t < 32 ? G[i * 32 + t] : C[i * d + c];
  }
  gd_solve(x, t, piv + 128 * grp);
  if (stage == 2) {
    if (t >= 32) {
      float* out = (grp ? a.b_k : a.b_q) + (int64_t)h * r * d;
#pragma unroll
      for (int i = 0; i < 32; ++i)
        if (i < r) out[i * d + c] = (float)x[i];
    }
    return;
  }
  double bcol[32];  // this thread's column of B_Q (group 0) or B_K (group 1)
#pragma unroll
  for (int i = 0; i < 32; ++i) bcol[i] = x[i];
  if (grp == 0 && t >= 32) {
#pragma unroll
    for (int i = 0; i < 32; ++i) BT[c * kGdLd + i] = bcol[i];
  }
  __syncthreads();
  // ---- W1 = Gk + B_Q B_Q^T
  {
    double o[4];
    gd_outer(BT, BT, o);
    if (tid < 256) {
      const int i = tid >> 3, j0 = (tid & 7) * 4;
#pragma unroll
      for (int u = 0; u < 4; ++u) Gs[i * kGdLg + j0 + u] = Gk[i * 32 + j0 + u] + o[u];
    }
  }
  __syncthreads();
  // ---- B_K B_K^T (the B tile now holds B_K)
  if (grp == 1 && t >= 32) {
#pragma unroll
    for (int i = 0; i < 32; ++i) BT[c * kGdLd + i] = bcol[i];
  }
  __syncthreads();
  {
    double o[4];
    gd_outer(BT, BT, o);
    if (tid < 256) {
      const int i = tid >> 3, j0 = (tid & 7) * 4;
#pragma unroll
      for (int u = 0; u < 4; ++u) Gs[32 * kGdLg + i * kGdLg + j0 + u] = o[u];
    }
  }
  // ---- Mq'^T = W1^-1 (Ck + B_Q)   (group 0; group 1 keeps the barriers)
  if (grp == 0) {
#pragma unroll
    for (int i = 0; i < 32; ++i) x[i] = t < 32 ? Gs[i * kGdLg + t] : Ck[i * d + c] + bcol[i];
  }
  __syncthreads();  // (W1 is read above from what the previous block wrote; B_K B_K^T is complete)
  gd_solve(x, grp == 0 ? t : -1, piv);
  double part_q = 0.0;  // sum of Cq (the old one) . Mq'^T over this thread's column
  if (grp == 0 && t >= 32) {
    float* mt = a.Mt_q + (int64_t)h * r * d;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      MT[c * kGdLd + i] = x[i];
      part_q = fma(Cq[i * d + c], x[i], part_q);
    }
#pragma unroll
    for (int i = 0; i < 32; ++i)
      if (i < r) mt[i * d + c] = (float)x[i];
  }
  double tr_old = 0.0;
  if (tid < 32) tr_old = tid < r ? Gq[tid * 32 + tid] : 0.0;
  __syncthreads();
  // ---- T = Mq'^T Sq, Gq' = Mq'^T T^T
  gd_times_s(MT, Sq, TT);
  {
    double o[4];
    gd_outer(MT, TT, o);
    double tr_new = 0.0;
    if (tid < 256) {
      const int i = tid >> 3, j0 = (tid & 7) * 4;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = j0 + u;
        const double v = (i < r && j < r) ? o[u] : (i == j ? 1.0 : 0.0);
        Gs[2 * 32 * kGdLg + i * kGdLg + j] = v;
        Gq[i * 32 + j] = v;
        if (i == j && i < r) tr_new += v;
      }
    }
    const double dq = gd_block_sum(tr_old - 2.0 * part_q + tr_new, red);
    if (tid == 0) a.delta[((int64_t)it * 2 + 0) * bh + h] = dq;
  }
  // Cq' = T (rows beyond r stay zero: Mq'^T has zero rows there)
  if (tid < d) {
#pragma unroll
    for (int i = 0; i < 32; ++i) Cq[i * d + tid] = TT[tid * kGdLd + i];
  }
  // ---- Mk'^T = (Gq' + B_K B_K^T)^-1 (T + B_K)   (group 1)
  if (grp == 1) {
#pragma unroll
    for (int i = 0; i < 32; ++i)
      x[i] = t < 32 ? Gs[2 * 32 * kGdLg + i * kGdLg + t] + Gs[32 * kGdLg + i * kGdLg + t] : TT[c * kGdLd + i] + bcol[i];
  }
  __syncthreads();
  gd_solve(x, grp == 1 ? t : -1, piv + 128);
  double part_k = 0.0;
  if (grp == 1 && t >= 32) {
    float* mt = a.Mt_k + (int64_t)h * r * d;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      MT[c * kGdLd + i] = x[i];
      part_k = fma(Ck[i * d + c], x[i], part_k);
    }
#pragma unroll
    for (int i = 0; i < 32; ++i)
      if (i < r) mt[i * d + c] = (float)x[i];
  }
  double trk_old = 0.0;
  if (tid < 32) trk_old = tid < r ? Gk[tid * 32 + tid] : 0.0;
  __syncthreads();
  // ---- U = Mk'^T Sk, Gk' = Mk'^T U^T, Ck' = U
  gd_times_s(MT, Sk, TT);
  {
    double o[4];
    gd_outer(MT, TT, o);
    double tr_new = 0.0;
    if (tid < 256) {
      const int i = tid >> 3, j0 = (tid & 7) * 4;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = j0 + u;
        const double v = (i < r && j < r) ? o[u] : (i == j ? 1.0 : 0.0);
        Gk[i * 32 + j] = v;
        if (i == j && i < r) tr_new += v;
      }
    }
    const double dk = gd_block_sum(trk_old - 2.0 * part_k + tr_new, red);
    if (tid == 0) a.delta[((int64_t)it * 2 + 1) * bh + h] = dk;
  }
  if (tid < d) {
#pragma unroll
    for (int i = 0; i < 32; ++i) Ck[i * d + tid] = TT[tid * kGdLd + i];
  }
}

// Workspace (bytes) of the Gram-domain iteration for bh heads over bkv distinct K heads.
static size_t gramdom_bytes(int bh, int bkv, int Sx, int Sxk, int iters) {
  const size_t dd = (size_t)kGdD * kGdD;
  return ((size_t)bh * Sx + (size_t)bkv * Sxk) * dd * sizeof(float)      // X^T X partial sums
         + ((size_t)bh + bkv) * dd * sizeof(double)                       // Sq, Sk
         + (size_t)2 * bh * (1024 + 32 * kGdD) * sizeof(double)           // G, C
         + (size_t)std::max(iters, 1) * 2 * bh * sizeof(double)           // squared changes
         + (size_t)2 * bh * 32 * kGdD * sizeof(float) + 256;              // Mq^T, Mk^T
}

// Runs all iterations on the Gram matrices.  On return Mt_q / Mt_k (device pointers written to *mt_q, *mt_k)
// hold Mq^T, Mk^T of the last iteration that ran, and b_q, b_k the final B factors; the caller applies
// A_Q = Q Mq, A_K = K Mk.  partQ / partK: the initial [G | C] partial sums (S splits).
int prefill_gram_domain(lrqk_ctx* ctx, const void* q, const void* k, const float* partQ, const float* partK, int S,
                        float* b_q, float* b_k, int b, int hq, int hkv, int64_t l, int r, int iters, float tol, int* flags,
                        float** mt_q, float** mt_k, hipStream_t st) {
  const int bh = b * hq, bkv = b * hkv;
  const int d = kGdD;
  // splits of the long axis for the X^T X sums: about two workgroups per CU (measured: 89 us against 103 with one)
  int Sx = (int)std::max<int64_t>(1, std::min<int64_t>(std::max(1, 512 / bh), (l + 511) / 512));
  int Sxk = (int)std::max<int64_t>(1, std::min<int64_t>(std::max(1, 512 / bkv), (l + 511) / 512));
  int rc = ctx->prefill_gd.ensure(gramdom_bytes(bh, bkv, Sx, Sxk, iters));
  if (rc) return rc;
  const size_t dd = (size_t)d * d;
  char* p = (char*)ctx->prefill_gd.p;
  double* Sq = (double*)p;                  p += (size_t)bh * dd * sizeof(double);
  double* Sk = (double*)p;                  p += (size_t)bkv * dd * sizeof(double);
  double* G = (double*)p;                   p += (size_t)2 * bh * 1024 * sizeof(double);
  double* C = (double*)p;                   p += (size_t)2 * bh * 32 * d * sizeof(double);
  double* delta = (double*)p;               p += (size_t)std::max(iters, 1) * 2 * bh * sizeof(double);
  float* Mtq = (float*)p;                   p += (size_t)bh * 32 * d * sizeof(float);
  float* Mtk = (float*)p;                   p += (size_t)bh * 32 * d * sizeof(float);
  float* xq_part = (float*)p;               p += (size_t)bh * Sx * dd * sizeof(float);
  float* xk_part = (float*)p;
  hipLaunchKernelGGL(pf_xtx_kernel, dim3((unsigned)Sx, (unsigned)bh), dim3(kXtxThreads), 0, st, (const bf16_t*)q, l,
                     xq_part, Sx);
  hipLaunchKernelGGL(pf_xtx_kernel, dim3((unsigned)Sxk, (unsigned)bkv), dim3(kXtxThreads), 0, st, (const bf16_t*)k, l,
                     xk_part, Sxk);
  hipLaunchKernelGGL(pf_xtx_reduce_kernel, dim3((unsigned)((dd + 255) / 256), (unsigned)bh), dim3(256), 0, st,
                     (const float*)xq_part, Sx, (int)dd, Sq);
  hipLaunchKernelGGL(pf_xtx_reduce_kernel, dim3((unsigned)((dd + 255) / 256), (unsigned)bkv), dim3(256), 0, st,
                     (const float*)xk_part, Sxk, (int)dd, Sk);
  LRQK_HIP_CHECK(hipGetLastError());
  const size_t smem = ((size_t)3 * kGdD * kGdLd + 3 * 32 * kGdLg + 256 + 8) * sizeof(double);
  static std::atomic<bool> attr_dev[kMaxDeviceSlots];
  std::atomic<bool>& attr = attr_dev[per_device_slot()];
  if (!attr) {
    LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)pf_gramdom_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem));
    attr = true;
  }
  GdArgs a{partQ, partK, S, Sq, Sk, G, C, delta, flags, Mtq, Mtk, b_q, b_k, bh, hq, hkv, r, l, tol};
  hipLaunchKernelGGL(pf_gramdom_init_kernel, dim3((unsigned)((32 * (32 + kGdD) + 255) / 256), (unsigned)bh, 2u), dim3(256), 0,
                     st, a);
  for (int it = 0; it < iters; ++it)
    hipLaunchKernelGGL(pf_gramdom_kernel, dim3((unsigned)bh), dim3(kGdThreads), smem, st, 0, it, a);
  hipLaunchKernelGGL(pf_gramdom_kernel, dim3((unsigned)bh), dim3(kGdThreads), smem, st, 2, iters, a);
  LRQK_HIP_CHECK(hipGetLastError());
  *mt_q = Mtq;
  *mt_k = Mtk;
  return LRQK_OK;
}

}  // namespace lrqk
