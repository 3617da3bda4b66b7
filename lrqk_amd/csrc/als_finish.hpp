// Last stage of the per-step factor update, shared by the stand-alone finish kernel and by the
// decode step (where it runs as extra workgroups of the fetch / attention launch).
#pragma once
#include "common.hpp"
#include "score_index.hpp"

namespace lrqk {

constexpr int kAlsMaxR = 32;  // one 32x32 MFMA tile (the tuned factor-update kernels)
constexpr int kFinMaxR = 64;  // the finish stage itself takes the ranks of the general kernels too
constexpr int kFinThreads = 256;

// The stopping test of the decode iterations is batch-wide: iteration `it` stops the loop if the
// mean over all heads of |k_hat - k_hat'|^2 is below tol.  deltas: [bh][max_iter] per-head sums.
// Executed by one whole wave; every lane returns the index of the iterate to keep.  The sums are
// formed in one fixed order, so every caller reaches the same decision.
// MAXIT >= max_iter bounds the register arrays.  Every load is unconditional (index clamped, value masked): a
// conditional load compiles to a branch with a full wait, which would put one memory latency per iteration on the
// chain of whoever calls this; as it is they all go out together.
template <int MAXIT>
__device__ __forceinline__ void als_delta_sums(const float* __restrict__ deltas, int bh, int max_iter,
                                               float (&sacc)[MAXIT]) {
  // the first 64 heads in straight-line code (the caller's other requests can go out before these are waited for)
  {
    const int hh = min(lane_id(), bh - 1);
    float v[MAXIT];
#pragma unroll
    for (int it = 0; it < MAXIT; ++it) v[it] = deltas[(int64_t)hh * max_iter + min(it, max_iter - 1)];
#pragma unroll
    for (int it = 0; it < MAXIT; ++it) sacc[it] = (lane_id() < bh && it < max_iter) ? v[it] : 0.0f;
  }
  for (int hh = lane_id() + kWave; hh < bh; hh += kWave) {
    float v[MAXIT];
#pragma unroll
    for (int it = 0; it < MAXIT; ++it) v[it] = deltas[(int64_t)hh * max_iter + min(it, max_iter - 1)];
#pragma unroll
    for (int it = 0; it < MAXIT; ++it) sacc[it] += it < max_iter ? v[it] : 0.0f;
  }
}
template <int MAXIT>
__device__ __forceinline__ int als_decide(float (&sacc)[MAXIT], int bh, int max_iter, int r, float tol) {
  int chosen = max_iter - 1;
  bool found = false;
#pragma unroll
  for (int it = 0; it < MAXIT; ++it) {
    if (it < max_iter) {  // (uniform: iterations that do not exist cost nothing)
      const float tot = wave_sum(sacc[it]);
      if (!found && tot / (float)((int64_t)bh * r) < tol) {
        chosen = it;
        found = true;
      }
    }
  }
  return chosen;
}
__device__ __forceinline__ int als_choose_iterate(const float* __restrict__ deltas, int bh, int max_iter, int r,
                                                  float tol) {
  float sacc[LRQK_MAX_DECODE_ITERS];
  als_delta_sums<LRQK_MAX_DECODE_ITERS>(deltas, bh, max_iter, sacc);
  return als_decide<LRQK_MAX_DECODE_ITERS>(sacc, bh, max_iter, r, tol);
}

// Type-erased arguments of the finish stage (kept in the ctx while it is pending).
struct FinishArgs {
  void* b_q;
  void* b_k;
  const void* q;
  const void* k_new;
  const float* iter_out;
  const float* deltas;
  int bh, hq, hkv, r, d, vshift, max_iter;
  float tol;
  void* q_hat_out;
  void* k_hat_out;
  void* a_k;
  int64_t head_stride, append_row;
  uint8_t* qa;       // score index (8-bit copy of A_K) to extend with the appended row, or nullptr
  uint16_t* qs;      // its rows' scales (fp16 bit patterns)
  const float* qw;   // its per-head transforms [bh][r*r + r]
  int64_t q_head_rows;
};

// The row that the finish stage appends to A_K (k_hat of the chosen iterate, as stored), encoded
// into the score index.  Executed by one whole wave per head; it repeats the stopping decision, so
// it does not depend on the finish stage and can run beside it.
template <typename T, int R>
__device__ __forceinline__ void als_index_append_rows(const FinishArgs& fa, int h) {
  const int lane = lane_id();
  float wcol[R];
  score_index_load_wcol<R>(fa.qw + (int64_t)h * (R * R + R), lane, wcol);
  const int chosen = als_choose_iterate(fa.deltas, fa.bh, fa.max_iter, R, fa.tol);
  float v = fa.iter_out[((int64_t)h * fa.max_iter + chosen) * 2 * R + R + min(lane, R - 1)];
  if (sizeof(T) == 2) v = round_to_bf16_f32(v);
  if (lane >= R) v = 0.0f;
  float scale;
  const uint8_t u = score_index_encode_row<R>(v, wcol, &scale);
  if (lane < R) fa.qa[((int64_t)h * fa.q_head_rows + fa.append_row) * R + lane] = u;
  if (lane == 0) fa.qs[(int64_t)h * fa.q_head_rows + fa.append_row] = sidx_scale_bits(scale);
}
template <typename T>
__device__ __forceinline__ void als_index_append_body(const FinishArgs& fa, int h) {
  if (fa.qa == nullptr || fa.append_row < 0 || wave_id() != 0) return;
  if (fa.r == 32)
    als_index_append_rows<T, 32>(fa, h);
  else if (fa.r == 16)
    als_index_append_rows<T, 16>(fa, h);
  else if (fa.r == 64)
    als_index_append_rows<T, 64>(fa, h);
}

// One workgroup (kFinThreads threads) per head h: batch-wide stopping decision, line-search update
// of B_Q and B_K (held in registers as 16-byte vectors: vector vi = tid + 256 u covers row
// vi >> vshift, columns (vi & (vpr-1)) * VEC ..), rounded q_hat / k_hat outputs, k_hat -> A_K row.
template <typename T>
__device__ __forceinline__ void als_finish_body(const FinishArgs& fa, int h) {
  T* __restrict__ b_q = (T*)fa.b_q;
  T* __restrict__ b_k = (T*)fa.b_k;
  const T* __restrict__ q = (const T*)fa.q;
  const T* __restrict__ k_new = (const T*)fa.k_new;
  const float* __restrict__ iter_out = fa.iter_out;
  const float* __restrict__ deltas = fa.deltas;
  const int bh = fa.bh, hq = fa.hq, hkv = fa.hkv, r = fa.r, d = fa.d, vshift = fa.vshift, max_iter = fa.max_iter;
  const float tol = fa.tol;
  T* __restrict__ q_hat_out = (T*)fa.q_hat_out;
  T* __restrict__ k_hat_out = (T*)fa.k_hat_out;
  T* __restrict__ a_k = (T*)fa.a_k;
  const int64_t head_stride = fa.head_stride, append_row = fa.append_row;
  constexpr int VEC = Vec16<T>::N;
  constexpr int kMaxVec = 8;  // vectors per thread per matrix: r * d / VEC <= 2048
  __shared__ float hat[2][kFinMaxR];
  __shared__ float err[2][256];
  __shared__ float red[kFinThreads / kWave][2][256];
  __shared__ int s_it;
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int b = h / hq, head = h % hq;
  const int kvh = head / (hq / hkv);
  const int vpr = 1 << vshift;  // vectors per row, a power of two <= 64
  const int nvec = r << vshift;
  // B tiles -> registers (independent loads, issued first)
  Vec16<T> vq[kMaxVec], vk[kMaxVec];
#pragma unroll
  for (int u = 0; u < kMaxVec; ++u) {
    const int vi = min(tid + u * kFinThreads, nvec - 1);
    vq[u].load(b_q + (int64_t)h * r * d + (int64_t)vi * VEC);
    vk[u].load(b_k + (int64_t)h * r * d + (int64_t)vi * VEC);
  }
  const float qreg = ld_f32<T>(q, (int64_t)h * d + min(tid, d - 1));
  const float kreg = ld_f32<T>(k_new, ((int64_t)b * hkv + kvh) * d + min(tid, d - 1));
  if (wave == 0) {
    const int chosen = als_choose_iterate(deltas, bh, max_iter, r, tol);
    if (lane == 0) s_it = chosen;
  }
  __syncthreads();
  const float* o = iter_out + ((int64_t)h * max_iter + s_it) * 2 * r;
  if (tid < 2 * r) hat[tid >= r ? 1 : 0][tid >= r ? tid - r : tid] = o[tid];
  __syncthreads();
  // column sums  sum_i hat[i] B[i][c]  for this thread's column group, both matrices
  const int cg = tid & (vpr - 1);  // vpr divides 256, so the column group is fixed per thread
  float pq[VEC], pk[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) pq[e] = pk[e] = 0.0f;
#pragma unroll
  for (int u = 0; u < kMaxVec; ++u) {
    const int vi = tid + u * kFinThreads;
    if (vi < nvec) {
      const int row = vi >> vshift;
      float fq[VEC], fk[VEC];
      vq[u].unpack(fq);
      vk[u].unpack(fk);
      const float hq_ = hat[0][row], hk_ = hat[1][row];
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        pq[e] = fmaf(hq_, fq[e], pq[e]);
        pk[e] = fmaf(hk_, fk[e], pk[e]);
      }
    }
  }
  // lanes of a wave that share a column group differ in the lane-id bits >= vshift
  for (int off = vpr; off < kWave; off <<= 1) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      pq[e] += __shfl_xor(pq[e], off, kWave);
      pk[e] += __shfl_xor(pk[e], off, kWave);
    }
  }
  if (lane < vpr) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      red[wave][0][cg * VEC + e] = pq[e];
      red[wave][1][cg * VEC + e] = pk[e];
    }
  }
  __syncthreads();
  float en0 = 0.0f, en1 = 0.0f;
  if (tid < d) {
    float eq = -qreg, ek = -kreg;
#pragma unroll
    for (int w = 0; w < kFinThreads / kWave; ++w) {
      eq += red[w][0][tid];
      ek += red[w][1][tid];
    }
    err[0][tid] = eq;
    err[1][tid] = ek;
    en0 = eq * eq;
    en1 = ek * ek;
  }
  en0 = wave_sum(en0);
  en1 = wave_sum(en1);
  __syncthreads();  // everyone is done reading red
  if (lane == 0) {
    red[wave][0][0] = en0;
    red[wave][1][0] = en1;
  }
  __syncthreads();
  float e2q = 0.0f, e2k = 0.0f, hnq = 0.0f, hnk = 0.0f;
  for (int w = 0; w < kFinThreads / kWave; ++w) {
    e2q += red[w][0][0];
    e2k += red[w][1][0];
  }
  for (int i = 0; i < r; ++i) {
    hnq = fmaf(hat[0][i], hat[0][i], hnq);
    hnk = fmaf(hat[1][i], hat[1][i], hnk);
  }
  // dB = hat^T e : |dB|^2 = |hat|^2 |e|^2 ; hat dB = |hat|^2 e : |hat dB|^2 = |hat|^4 |e|^2
  const float lrq = (hnq * e2q) / (hnq * hnq * e2q + 1e-6f);
  const float lrk = (hnk * e2k) / (hnk * hnk * e2k + 1e-6f);
#pragma unroll
  for (int u = 0; u < kMaxVec; ++u) {
    const int vi = tid + u * kFinThreads;
    if (vi < nvec) {
      const int row = vi >> vshift;
      float fq[VEC], fk[VEC];
      vq[u].unpack(fq);
      vk[u].unpack(fk);
      const float sq = lrq * hat[0][row], sk = lrk * hat[1][row];
      const int64_t off = (int64_t)h * r * d + (int64_t)vi * VEC;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        fq[e] -= sq * err[0][cg * VEC + e];
        fk[e] -= sk * err[1][cg * VEC + e];
      }
      Vec16<T> oq, ok;  // one 16-byte store per vector (b_q, b_k are 16-byte aligned: they are read that way)
      oq.pack(fq);
      ok.pack(fk);
      oq.store(b_q + off);
      ok.store(b_k + off);
    }
  }
  if (tid < r) {
    st_f32<T>(q_hat_out, (int64_t)h * r + tid, hat[0][tid]);
    st_f32<T>(k_hat_out, (int64_t)h * r + tid, hat[1][tid]);
    if (append_row >= 0) st_f32<T>(a_k, (int64_t)h * head_stride + append_row * r + tid, hat[1][tid]);
  }
}

}  // namespace lrqk
