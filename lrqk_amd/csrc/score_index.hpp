// Score index: an 8-bit copy of the A_K rows, in whitened coordinates, that lets the proxy-score
// scan read 34 instead of 64 bytes per cached token.  The scan bounds every row's score from the
// copy and rescores exactly (from A_K itself) only the rows whose bound reaches the filter
// threshold, so the candidate list -- and everything after it -- is unchanged.
//
// Per head there is one upper-triangular matrix W (r x r, about the inverse Cholesky factor of the
// rows' second-moment matrix, so that the transformed rows a' = a W have unit, uncorrelated
// columns whatever direction the proxy query has) and, per row, one scale:
//   a'_j = (u_j - 128) * scale + d_j,  |d_j| <= 0.50002 * scale.
// The scan solves W q' = q by back substitution and uses  a . q = a' . q'.  Any nonsingular W keeps
// the bound valid (a stale or poor W only loosens it), because every rounding error is charged to
// the row: with g_j = sum_i |a_i| |W_ij| and c = 5 (r + 2) 2^-24, the errors of forming a' in fp32
// (3 r 2^-24 would do for round-to-nearest chains; the margin covers a matrix pipe that truncates),
// of the back substitution (backward error in W) and of the exact fp32 score chain are together at
// most c * sum_j g_j |q'_j|, and the scale of a row is raised until c * max_j g_j <= kSidxBeta * scale:
//   |score - scale * sum_j (u_j - 128) q'_j| <= scale * |q'|_1 * (0.50002 + kSidxBeta + fp32 slack of the sum)
// The index is derived state: it must be dropped whenever rows of A_K change in place.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lrqk {

constexpr float kSidxBeta = 0.008f;
// 0.50002 + kSidxBeta + at most 1.6e-3 (fp32 evaluation of the sum at r <= 64), with the 4e-6 relative
// error of |q'|_1 itself
constexpr float kSidxDFactor = 0.511f;

struct ScoreIndexView {
  const uint8_t* qa;  // [bh][head_rows][r]
  const uint16_t* qs; // [bh][head_rows] the rows' scales as fp16 bit patterns (score_index_scale returns such values)
  const float* wm;    // [bh][r*r + r]: W row-major (zeros below the diagonal), then 1 / W_jj
  int64_t head_rows;  // rows per head of qa and qs (= rows per head of A_K)
};

// Scale of a row from max_j |a'_j| and max_j g_j.  The floor keeps the bound above anything a
// flush of subnormal products could lose (r * 1.2e-38 per element); a row with a NaN or an
// infinity gets a NaN scale, which makes the scan rescore it exactly every time.
// The scale is stored in 16 bits: any scale at least as large as the one required keeps the bound valid (the codes
// are formed with the stored value), so it is rounded up to the next fp16 number (at most 0.1 % more; +infinity
// beyond the fp16 range, which like the NaN makes the scan rescore the row every time).
__device__ __forceinline__ float sidx_round_up_f16(float x) {
  _Float16 h = (_Float16)x;
  if ((float)h < x) h = __builtin_bit_cast(_Float16, (uint16_t)(__builtin_bit_cast(uint16_t, h) + 1));  // (x > 0)
  return (float)h;
}
__device__ __forceinline__ uint16_t sidx_scale_bits(float scale) { return __builtin_bit_cast(uint16_t, (_Float16)scale); }
__device__ __forceinline__ float sidx_scale_from_bits(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
__device__ __forceinline__ float score_index_scale(float row_max, float g_max, int r) {
  const float coef = 5.0f * (float)(r + 2) * 5.9604645e-8f * (1.000001f / kSidxBeta);
  float scale = fmaxf(fmaxf(row_max * (1.0f / 127.0f), g_max * coef), 1e-30f);
  scale = sidx_round_up_f16(scale);
  if (!(g_max < INFINITY)) scale = NAN;
  return scale;
}
__device__ __forceinline__ uint8_t score_index_code(float a, float inv_scale) {
  float qv = rintf(a * inv_scale);
  qv = fminf(fmaxf(qv, -127.0f), 127.0f);  // (also turns a NaN into a number: the NaN scale keeps the row)
  return (uint8_t)((int)qv + 128);
}

__device__ __forceinline__ float sidx_readlane(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// Column `lane` of a head's W into registers (lanes >= R get zeros).
template <int R>
__device__ __forceinline__ void score_index_load_wcol(const float* __restrict__ wm_head, int lane, float (&wcol)[R]) {
#pragma unroll
  for (int i = 0; i < R; ++i) wcol[i] = lane < R ? wm_head[i * R + lane] : 0.0f;
}

// Encodes one row.  Executed by a whole wave: lane i (< R) passes element a_i of the row as stored,
// lanes >= R pass 0; wcol is this lane's column of W.  Lane j < R gets byte u_j; all lanes get the scale.
template <int R>
__device__ __forceinline__ uint8_t score_index_encode_row(float a_lane, const float (&wcol)[R], float* scale_out) {
  float acc = 0.0f, g = 0.0f;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const float ai = sidx_readlane(a_lane, i);
    acc = __builtin_fmaf(ai, wcol[i], acc);
    g = __builtin_fmaf(fabsf(ai), fabsf(wcol[i]), g);
  }
  const float row_max = wave_max(fabsf(acc));
  const float g_max = wave_max(g);
  const float scale = score_index_scale(row_max, g_max, R);
  const float inv = 1.0f / scale;
  *scale_out = scale;
  return score_index_code(acc, inv);
}

}  // namespace lrqk
