// Inverse of a small symmetric positive definite matrix on the matrix cores, shared by the decode
// and the prefill half of the factorisation.
#pragma once
#include "common.hpp"

namespace lrqk {

typedef float v16f __attribute__((ext_vector_type(16)));

// C tile of mfma_f32_32x32x2f32: lane l, element v -> row (the column is l & 31)
__device__ __forceinline__ int mfma_row(int lane, int v) { return ((v >> 2) << 3) + ((lane >> 5) << 2) + (v & 3); }

constexpr int kLdi = 33;  // row stride of an inverse in LDS

// Inverse of one SPD 32 x 32 matrix by one wave, as 32 symmetric sweeps on the matrix cores.  The
// matrix sits in the accumulator layout of the 32x32x2 fp32 MFMA (acc[v] of lane l: row mfma_row(l, v),
// column l % 32).  A sweep on pivot p (d = a_pp) maps
//   a_ij -> a_ij - a_ip a_pj / d,   a_ip -> a_ip / d,   a_pj -> a_pj / d,   a_pp -> -1 / d,
// keeps the matrix symmetric and, after all p, leaves -G^-1.  All four cases are one rank-2 update
// acc -= A B with operands made from row p alone (held by the lanes of one half: by symmetry it is also
// column p): A_i = a_pi / d, B_j = a_pj, except A_p = 1 - 1/d and B_p = d - 1 (which turn row and column p
// into a_p. / d), and the second rank, supplied by the other half, subtracts 2 at (p, p).  B_p = d - 1
// cancels badly for large d, so the matrix is first scaled to unit diagonal (then every pivot is <= 1);
// the scaling is undone on the way out.  Rows and columns >= r are an identity block and are skipped.
// g(i, j) returns element (i, j); sbuf: 32 floats of LDS owned by this wave; inv: [32][kLdi].
template <typename GetG>
__device__ __forceinline__ void invert_sweep_mfma(GetG&& g, int r, float* sbuf, float* inv) {
  const int lane = lane_id();
  const int col = lane & 31, half = lane >> 5;
  v16f acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int i = mfma_row(lane, v);
    const float x = g(i, col);
    acc[v] = (i < r && col < r) ? x : (i == col ? 1.0f : 0.0f);
  }
  const float s_col = col < r ? __builtin_amdgcn_rsqf(g(col, col)) : 1.0f;
  if (lane < 32) sbuf[lane] = s_col;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  float sc[16];  // s_row * s_col of every element this lane holds
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const float4 s4 = reinterpret_cast<const float4*>(sbuf)[2 * a + half];  // rows 8a + 4 half + 0..3
    sc[4 * a + 0] = s4.x * s_col;
    sc[4 * a + 1] = s4.y * s_col;
    sc[4 * a + 2] = s4.z * s_col;
    sc[4 * a + 3] = s4.w * s_col;
  }
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] *= sc[v];
  // The lane-dependent cases are taken by weights of 0 and 1, not by selects: selects between expressions
  // compile to divergent branches, which cost more than the sweep's arithmetic.  (The matrix is finite, so a
  // product with a weight of 0 is 0.)
  const float in0 = half == 0 ? 1.0f : 0.0f, in1 = 1.0f - in0;
#pragma unroll
  for (int p = 0; p < 32; ++p) {
    if (p < r) {  // (wave-uniform)
      const int v = ((p >> 3) << 2) + (p & 3), hp = (p >> 2) & 1;
      const float rv = acc[v];
      const float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(rv), p + 32 * hp));
      float rc = __builtin_amdgcn_rcpf(d);
      rc = fmaf(fmaf(-d, rc, 1.0f), rc, rc);
      const float win = hp ? in1 : in0, wout = hp ? in0 : in1;  // this lane's half holds row p / the other half
      const float wp = col == p ? 1.0f : 0.0f;
      // A = in: (p: 1 - rc, else rv rc); out: (p: 2, else 0).   B = in: (p: d - 1, else rv); out: (p: 1, else 0)
      const float a_in = fmaf(wp, (1.0f - rc) - rv * rc, rv * rc);
      const float b_in = fmaf(wp, (d - 1.0f) - rv, rv);
      const float A = fmaf(win, a_in, wout * (2.0f * wp));
      const float B = fmaf(win, b_in, wout * wp);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(-A, B, acc, 0, 0, 0);
    }
  }
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int i = mfma_row(lane, v);
    inv[i * kLdi + col] = (i < r && col < r) ? -acc[v] * sc[v] : (i == col ? 1.0f : 0.0f);
  }
}

// X = G^-1 RHS for NB blocks of 32 right-hand-side columns, by one wave: the same 32 sweeps, applied to
// the augmented matrix [G | RHS] (Gauss-Jordan elimination of the right-hand side, no explicit inverse).
// For a positive definite G this is backward stable: the residual RHS - G X stays at 2^-24 relative however
// badly G is conditioned, as with a factorisation-based solve, whereas a product with a computed inverse
// leaves cond(G) * 2^-24.  At pivot p the right-hand side takes the same rank-1 update as G, with row p of
// the block as the B operand: r_ij -= (a_ip / d) r_pj, r_pj -= (1 - 1/d) r_pj.  G is scaled to unit diagonal
// as in invert_sweep_mfma: the rows of RHS are scaled on the way in and the rows of X on the way out.
// g(i, j): element of G (any i, j < 32; values outside r x r are ignored); rhs(b, i, col): element (i, col)
// of block b (0 outside the matrix); emit(b, i, col, x) receives X for i < r.  sbuf: 32 floats of LDS
// owned by this wave.
template <int NB, typename GetG, typename GetR, typename Emit>
__device__ __forceinline__ void solve_sweep_mfma(GetG&& g, GetR&& rhs, int r, float* sbuf, Emit&& emit) {
  const int lane = lane_id();
  const int col = lane & 31, half = lane >> 5;
  v16f acc, xr[NB];
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int i = mfma_row(lane, v);
    const float x = g(i, col);
    acc[v] = (i < r && col < r) ? x : (i == col ? 1.0f : 0.0f);
  }
  const float s_col = col < r ? __builtin_amdgcn_rsqf(g(col, col)) : 1.0f;
  __builtin_amdgcn_wave_barrier();  // (an earlier use of sbuf by this wave is complete)
  if (lane < 32) sbuf[lane] = s_col;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  float sr[16];  // s_row of every element this lane holds
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const float4 s4 = reinterpret_cast<const float4*>(sbuf)[2 * a + half];  // rows 8a + 4 half + 0..3
    sr[4 * a + 0] = s4.x;
    sr[4 * a + 1] = s4.y;
    sr[4 * a + 2] = s4.z;
    sr[4 * a + 3] = s4.w;
  }
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] *= sr[v] * s_col;
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int i = mfma_row(lane, v);
      xr[b][v] = i < r ? rhs(b, i, col) * sr[v] : 0.0f;
    }
#pragma unroll
  for (int p = 0; p < 32; ++p) {
    if (p < r) {  // (wave-uniform)
      const int v = ((p >> 3) << 2) + (p & 3), hp = (p >> 2) & 1;
      const float rv = acc[v];
      const float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(rv), p + 32 * hp));
      float rc = __builtin_amdgcn_rcpf(d);
      rc = fmaf(fmaf(-d, rc, 1.0f), rc, rc);
      const bool inhalf = half == hp, isp = col == p;
      const float A = inhalf ? (isp ? 1.0f - rc : rv * rc) : (isp ? 2.0f : 0.0f);
      const float B = inhalf ? (isp ? d - 1.0f : rv) : (isp ? 1.0f : 0.0f);
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        const float BR = inhalf ? xr[b][v] : 0.0f;
        xr[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(-A, BR, xr[b], 0, 0, 0);
      }
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(-A, B, acc, 0, 0, 0);
    }
  }
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int i = mfma_row(lane, v);
      if (i < r) emit(b, i, col, xr[b][v] * sr[v]);
    }
}

}  // namespace lrqk
