// Inverse of a small symmetric positive definite matrix on the matrix cores, shared by the decode
// and the prefill half of the factorisation.
#pragma once
#include "common.hpp"

namespace lrqk {

typedef float v16f __attribute__((ext_vector_type(16)));

// C tile of mfma_f32_32x32x2f32: lane l, element v -> row (the column is l & 31)
__device__ __forceinline__ int mfma_row(int lane, int v) { return ((v >> 2) << 3) + ((lane >> 5) << 2) + (v & 3); }

constexpr int kLdi = 33;  // row stride of an inverse in LDS

// Lanes 0..31 get lo_src and lanes 32..63 get hi_src, both taken from the half `hp` (a compile-time 0 or 1) of
// the sources' lanes.
__device__ __forceinline__ float half_pair(float lo_src, float hi_src, int hp) {
  const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(lo_src), __float_as_uint(hi_src), false, false);
  return __uint_as_float(hp ? sw[1] : sw[0]);
}

// Inverse of one SPD 32 x 32 matrix by one wave, as symmetric sweeps on the matrix cores, two pivots at a time.  The
// matrix sits in the accumulator layout of the 32x32x2 fp32 MFMA (acc[v] of lane l: row mfma_row(l, v),
// column l % 32).  A sweep on pivot p (d = a_pp) maps
//   a_ij -> a_ij - a_ip a_pj / d,   a_ip -> a_ip / d,   a_pj -> a_pj / d,   a_pp -> -1 / d,
// keeps the matrix symmetric and, after all p, leaves -G^-1.  It is one rank-1 update acc -= A B with operands made
// from row p alone (held by the lanes of one half: by symmetry it is also column p): B_j = a_pj except
// B_p = d - 1, and A = B / d (so A_p = 1 - 1/d); that leaves 2 - 1/d at (p, p), and since an entry (p, p) feeds
// nothing after its own sweep, the 2 is taken off every diagonal entry once, at the end.  The sweeps on p and
// p + 1 go into ONE MFMA, as its two k elements: the second sweep's operands need row p + 1 as the first sweep
// leaves it, a'_(p+1)j = a_(p+1)j - (a_(p+1)p / d) B_j, which the vector ALUs form from the two rows (the lower half
// of the wave carries the first sweep, the upper half the second: v_permlane32_swap moves the rows there).  (The
// algebraically equal update with the inverse of the 2 x 2 pivot block loses digits when that block is nearly
// singular; this form is the two sweeps themselves.)  An odd r ends with a sweep on one pivot.  B_p = d - 1
// cancels badly for large d, so the matrix is first scaled to unit diagonal (then every pivot is <= 1); the
// scaling is undone on the way out.  Rows and columns >= r are an identity block and are skipped.
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
  for (int p = 0; p < 32; p += 2) {
    const int v = ((p >> 3) << 2) + (p & 3), hp = (p >> 2) & 1;  // rows p, p + 1: elements v, v + 1 of half hp
    if (p + 1 < r) {  // (wave-uniform)
      const float r0 = acc[v], r1 = acc[v + 1];
      const float da = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(r0), p + 32 * hp));
      const float db = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(r0), p + 1 + 32 * hp));
      const float dc = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(r1), p + 1 + 32 * hp));
      float rc0 = __builtin_amdgcn_rcpf(da);
      rc0 = fmaf(fmaf(-da, rc0, 1.0f), rc0, rc0);
      const float brc = db * rc0;
      const float c1 = fmaf(-db, brc, dc);  // the second pivot as the first sweep leaves it
      float rc1 = __builtin_amdgcn_rcpf(c1);
      rc1 = fmaf(fmaf(-c1, rc1, 1.0f), rc1, rc1);
      const float wp0 = col == p ? 1.0f : 0.0f, wp1 = col == p + 1 ? 1.0f : 0.0f;
      const float U = half_pair(r0, r1, hp), V = half_pair(r1, r0, hp);  // [row p | row p + 1], [row p + 1 | row p]
      const float B1 = (half ? V : U) - wp0;        // the first sweep's B, in every lane
      const float B2 = fmaf(-brc, B1, U) - wp1;     // (upper half) the second sweep's B
      const float B = half ? B2 : B1;
      const float A = B * (half ? rc1 : rc0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(-A, B, acc, 0, 0, 0);
    } else if (p < r) {  // the last pivot of an odd r
      const float rv = acc[v];
      const float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(rv), p + 32 * hp));
      float rc = __builtin_amdgcn_rcpf(d);
      rc = fmaf(fmaf(-d, rc, 1.0f), rc, rc);
      const float win = hp ? in1 : in0;  // 1 in the half that holds row p
      const float wp = col == p ? 1.0f : 0.0f;
      const float A = win * fmaf(wp, (1.0f - rc) - rv * rc, rv * rc);
      const float B = win * fmaf(wp, (d - 1.0f) - rv, rv);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(-A, B, acc, 0, 0, 0);
    }
  }
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int i = mfma_row(lane, v);
    const float fix = i == col ? 2.0f : 0.0f;  // (the 2 left on the diagonal of every pivot block)
    inv[i * kLdi + col] = (i < r && col < r) ? -(acc[v] - fix) * sc[v] : (i == col ? 1.0f : 0.0f);
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
