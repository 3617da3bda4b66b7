// Proxy-score scan q_hat . A_K^T, the per-head top-k selector, and (fused behind it) the
// hit/miss diff against the resident set.
//
// Score contract: fp32 fmaf chain over j = 0..r-1 starting at +0, optional rounding to
// bf16, -0 -> +0.  Selection order: (score descending, token index ascending); the
// result is written ascending by index.
//
// Decode-time structure (two launches, scores never reach HBM):
//   score_filter : streams A_K once; a row becomes a CANDIDATE if its key is >= the head's
//                  running lower bound t_low (the key that had rank ~1.5k at the previous
//                  call).  Candidates (key, index) are packed per workgroup in LDS and
//                  appended to a small per-head list.
//   select       : one workgroup per head.  If the list holds at least k (and not too many)
//                  candidates it provably contains the exact top-k including every tie at
//                  the threshold, and the exact radix select runs on the list alone, held
//                  in registers.  Otherwise (first call, distribution shift) the workgroup
//                  recomputes the head's scores itself and selects over all of them.  Either
//                  way it leaves the next t_low.  Results never depend on t_low, only speed.
//                  The radix digits are taken from (key - lowest key) shifted so that the
//                  occupied range fills the 4096 bins: one or two passes instead of three.
//                  The selected ids are emitted in order through two bitmaps (key > T,
//                  key == T) and, when asked, diffed in place against the resident set.
#include <vector>

#include "common.hpp"
#include "ctx.hpp"
#include "als_finish.hpp"
#include "score_index.hpp"

namespace lrqk {

// --------------------------------------------------------------------------- score of one row
template <typename T, int R>
struct RowScorer {
  static constexpr int VEC = Vec16<T>::N;
  float qf[R > 0 ? R : 1];
  const T* qh;
  int r;
  int round_bf16;
  __device__ __forceinline__ void init(const T* q_head, int r_, int round_) {
    qh = q_head;
    r = r_;
    round_bf16 = round_;
    if (R > 0) {
#pragma unroll
      for (int j = 0; j < R; ++j) qf[j] = ld_f32<T>(q_head, j);
    }
  }
  // the proxy query from a lane-distributed fp32 vector (lane j holds element j of an iterate of
  // the factor update), rounded to the storage type and broadcast to every lane
  __device__ __forceinline__ void init_from_lanes(float qv, int r_, int round_) {
    qh = nullptr;
    r = r_;
    round_bf16 = round_;
    if (sizeof(T) == 2) qv = round_to_bf16_f32(qv);
    if (R > 0) {
#pragma unroll
      for (int j = 0; j < R; ++j)
        qf[j] = j < r_ ? __int_as_float(__builtin_amdgcn_readlane(__float_as_int(qv), j)) : 0.0f;
    }
  }
  // a row as 16-byte vectors (R > 0 only): requested now, scored later
  struct Row {
    Vec16<T> v[R / VEC > 0 ? R / VEC : 1];
  };
  __device__ __forceinline__ void load_row(const T* A, int64_t i, Row& row) const {
    const T* p = A + i * R;
#pragma unroll
    for (int c = 0; c < R / VEC; ++c) row.v[c].load(p + c * VEC);
  }
  __device__ __forceinline__ float score_row(const Row& row) const {
    float acc = 0.0f;
#pragma unroll
    for (int c = 0; c < R / VEC; ++c) {
      float f[VEC];
      row.v[c].unpack(f);
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc = __builtin_fmaf(f[e], qf[c * VEC + e], acc);
    }
    if (round_bf16) acc = round_to_bf16_f32(acc);
    if (acc == 0.0f) acc = 0.0f;
    return acc;
  }
  __device__ __forceinline__ float q_norm() const {
    float s = 0.0f;
    if (R > 0) {
#pragma unroll
      for (int j = 0; j < R; ++j) s = __builtin_fmaf(qf[j], qf[j], s);
    } else {
      for (int j = 0; j < r; ++j) {
        const float x = ld_f32<T>(qh, j);
        s = __builtin_fmaf(x, x, s);
      }
    }
    return sqrtf(s);
  }
  __device__ __forceinline__ float score(const T* A, int64_t i) const {
    float acc = 0.0f;
    if (R > 0) {
      const T* row = A + i * R;
      Vec16<T> v[R / VEC > 0 ? R / VEC : 1];
#pragma unroll
      for (int c = 0; c < R / VEC; ++c) v[c].load(row + c * VEC);
#pragma unroll
      for (int c = 0; c < R / VEC; ++c) {
        float f[VEC];
        v[c].unpack(f);
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc = __builtin_fmaf(f[e], qf[c * VEC + e], acc);
      }
    } else {
      const T* row = A + i * r;
      for (int j = 0; j < r; ++j) acc = __builtin_fmaf(ld_f32<T>(row, j), ld_f32<T>(qh, j), acc);
    }
    if (round_bf16) acc = round_to_bf16_f32(acc);
    if (acc == 0.0f) acc = 0.0f;
    return acc;
  }
};

// --------------------------------------------------------------------------- plain scores
// One thread per cached token row.  R > 0: row of R elements fetched with 16-byte loads.
// R == 0: any r, scalar loads.
template <typename T, int R>
__global__ __launch_bounds__(256) void score_kernel(const T* __restrict__ a_k, int64_t head_stride,
                                                    const T* __restrict__ q_hat, int64_t m, int r,
                                                    int round_bf16, uint32_t* __restrict__ keys,
                                                    int64_t key_stride, float* __restrict__ scores) {
  const int h = blockIdx.y;
  const T* A = a_k + (int64_t)h * head_stride;
  RowScorer<T, R> rs;
  rs.init(q_hat + (int64_t)h * r, r, round_bf16);
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < m; i += (int64_t)gridDim.x * blockDim.x) {
    const float acc = rs.score(A, i);
    if (keys) keys[(int64_t)h * key_stride + i] = score_key(acc);
    if (scores) scores[(int64_t)h * m + i] = acc;
  }
}

__global__ __launch_bounds__(256) void keys_from_scores_kernel(const float* __restrict__ scores, int64_t m,
                                                               uint32_t* __restrict__ keys,
                                                               int64_t key_stride) {
  const int h = blockIdx.y;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < m; i += (int64_t)gridDim.x * blockDim.x)
    keys[(int64_t)h * key_stride + i] = score_key(scores[(int64_t)h * m + i]);
}

__global__ __launch_bounds__(256) void arange_kernel(int32_t* out, int64_t out_stride, int count) {
  const int h = blockIdx.y;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < count; i += gridDim.x * blockDim.x)
    out[(int64_t)h * out_stride + i] = i;
}

// Per-head selector state: t_low (key that had rank ~1.5k at the previous call), q_norm (|q_hat|
// of that call), t_used / q_cur (bound and norm the filter of the current call used).
// The per-head counters of the candidate lists take atomic additions from every workgroup of a scan: each sits in a
// 128-byte line of its own (additions to one line are served one after the other, about 11 ns each, whichever
// word of the line they name).
constexpr int kCountStride = 32;

struct SelState {
  uint32_t* t_low;
  float* q_norm;
  uint32_t* t_used;
  float* q_cur;
  int* cand_count;   // [bh * kCountStride], element h * kCountStride
  int* level;        // slack of the carried bound per head (see bound_rank): level | calm calls << 8
  int* stats;
  int* rescored;     // per workgroup of the last index scan: rows whose bound passed (rescored exactly)
  int rescored_cap;
};

__global__ void init_select_state_kernel(SelState st, int bh) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < bh) {
    st.t_low[i] = 0xffffffffu;
    st.q_norm[i] = 0.0f;
    st.t_used[i] = 0xffffffffu;
    st.q_cur[i] = 0.0f;
    st.cand_count[i * kCountStride] = 0;
    st.level[i] = 0;
  }
  if (i < 3) st.stats[i] = 0;
}

// The proxy scores scale with |q_hat|, so the bound carried over from the previous call is
// rescaled by the ratio of the norms (positive bounds only) and relaxed by 2 %.
// With scores rounded to bf16 every key ends in 0x0000 (score >= 0) or 0xffff (score < 0); the bound is
// lowered to the next key of that form, so that (key - bound) keeps its 16 trailing zero bits and
// the radix select of the candidates needs one pass instead of two or three.
__device__ __forceinline__ uint32_t rescaled_bound(uint32_t t_low, float q_norm_prev, float q_norm_now,
                                                   int round_bf16) {
  if (t_low == 0xffffffffu || !(q_norm_prev > 0.0f) || !(q_norm_now > 0.0f)) return t_low;
  const float s = key_score(t_low);
  if (!(s > 0.0f)) return t_low;
  uint32_t key = score_key(s * (q_norm_now / q_norm_prev) * 0.98f);
  if (round_bf16) key &= 0xffff0000u;  // (s > 0: the key is in the upper half, where rounding down clears the low bits)
  return key;
}

// --------------------------------------------------------------------------- score + filter
constexpr int kFiltThreads = 256;
#ifndef LRQK_FILT_RPT
#define LRQK_FILT_RPT 8
#endif
constexpr int kFiltRPT = LRQK_FILT_RPT;  // rows per thread and tile
#ifndef LRQK_FILT_TILES
#define LRQK_FILT_TILES 2
#endif
constexpr int kFiltTiles = LRQK_FILT_TILES;  // tiles per workgroup: one global list reservation for all of them
constexpr int kFiltRows = kFiltThreads * kFiltRPT;
constexpr int kFiltMaxIt = 8;  // most iterations of the factor update whose pending iterate the filter can pick itself

// Proxy query taken straight from the iterates of the factor update whose finish stage has not
// run yet (iter_out == nullptr: q_hat is read instead).  Workgroup 0 of every head writes the
// chosen, rounded iterate to q_hat_out.
struct FilterQ {
  const float* iter_out;  // [bh][max_iter][2r]
  const float* deltas;    // [bh][max_iter]
  int bh, max_iter;
  float tol;
  void* q_hat_out;        // [bh][r] storage dtype
};

template <typename T, int R>
__global__ __launch_bounds__(kFiltThreads) void score_filter_kernel(const T* __restrict__ a_k, int64_t head_stride,
                                                                    const T* __restrict__ q_hat, int64_t m, int r,
                                                                    int round_bf16, SelState st,
                                                                    uint2* __restrict__ cand, int cand_cap,
                                                                    FilterQ fq) {
  extern __shared__ __align__(16) uint32_t filt_dyn[];
  uint2* lc = reinterpret_cast<uint2*>(filt_dyn);  // [kFiltRows * kFiltTiles]
  __shared__ int l_count, g_base;
  const int h = blockIdx.y;
  const int tid = threadIdx.x, lane = lane_id();
  const T* A = a_k + (int64_t)h * head_stride;
  RowScorer<T, R> rs;
  if (tid == 0) l_count = 0;
  __syncthreads();
  const uint32_t t_prev = st.t_low[h];
  const float qn_prev = st.q_norm[h];
  uint32_t tl = 0;
  // The small loads go first (memory returns in order: issued after the rows they would arrive
  // last).  With a pending finish stage every wave fetches the stopping-test terms and element
  // `lane` of every iterate, decides, and broadcasts the chosen iterate from its lanes (no barrier,
  // no LDS); otherwise q_hat is read.
  const bool pending = fq.iter_out != nullptr;
  float sacc[kFiltMaxIt], oit[kFiltMaxIt];
  if (pending) {
    als_delta_sums<kFiltMaxIt>(fq.deltas, fq.bh, fq.max_iter, sacc);
#pragma unroll
    for (int it = 0; it < kFiltMaxIt; ++it)
      oit[it] = fq.iter_out[((int64_t)h * fq.max_iter + min(it, fq.max_iter - 1)) * 2 * r + min(lane, r - 1)];
  } else {
    rs.init(q_hat + (int64_t)h * r, r, round_bf16);
  }
#pragma unroll 1
  for (int tile = 0; tile < kFiltTiles; ++tile) {
    const int64_t base = ((int64_t)blockIdx.x * kFiltTiles + tile) * kFiltRows;
    if (base >= m) break;
    // pure streaming part: loads unconditional (clamped), hits kept as a mask
    uint32_t keys[kFiltRPT];
    if constexpr (R > 0) {
      // the first rows are requested before the pending iterate is resolved, so that its latency
      // and theirs overlap
      constexpr int kPre = 2;  // more would cost occupancy (16 registers per row)
      typename RowScorer<T, R>::Row rows[kPre];
#pragma unroll
      for (int it = 0; it < kPre; ++it) {
        const int64_t i = base + it * kFiltThreads + tid;
        rs.load_row(A, min(i, m - 1), rows[it]);
      }
      if (tile == 0 && pending) {
        const int chosen = als_decide<kFiltMaxIt>(sacc, fq.bh, fq.max_iter, r, fq.tol);
        float qv = oit[0];
#pragma unroll
        for (int it = 1; it < kFiltMaxIt; ++it) qv = chosen == it ? oit[it] : qv;
        if (blockIdx.x == 0 && tid < r) st_f32<T>((T*)fq.q_hat_out, (int64_t)h * r + tid, qv);
        rs.init_from_lanes(qv, r, round_bf16);
      }
#pragma unroll
      for (int it = 0; it < kPre; ++it) keys[it] = score_key(rs.score_row(rows[it]));
#pragma unroll
      for (int it = kPre; it < kFiltRPT; ++it) {
        const int64_t i = base + it * kFiltThreads + tid;
        keys[it] = score_key(rs.score(A, min(i, m - 1)));
      }
    } else {
#pragma unroll
      for (int it = 0; it < kFiltRPT; ++it) {
        const int64_t i = base + it * kFiltThreads + tid;
        keys[it] = score_key(rs.score(A, min(i, m - 1)));
      }
    }
    if (tile == 0) {
      const float qn = rs.q_norm();
      tl = rescaled_bound(t_prev, qn_prev, qn, round_bf16);
      if (tid == 0 && blockIdx.x == 0) {
        st.t_used[h] = tl;
        st.q_cur[h] = qn;
      }
    }
    uint32_t mask = 0;
#pragma unroll
    for (int it = 0; it < kFiltRPT; ++it) {
      const int64_t i = base + it * kFiltThreads + tid;
      if (i < m && keys[it] >= tl) mask |= 1u << it;
    }
    // one LDS allocation per wave for all of its hits
    const int cnt = __popc(mask);
    const int incl = wave_inclusive_sum(cnt);
    const int wtot = __shfl(incl, kWave - 1, kWave);
    if (wtot) {
      int wbase = 0;
      if (lane == kWave - 1) wbase = atomicAdd(&l_count, wtot);
      wbase = __shfl(wbase, kWave - 1, kWave);
      int pos = wbase + incl - cnt;
#pragma unroll
      for (int it = 0; it < kFiltRPT; ++it) {
        if ((mask >> it) & 1u) lc[pos++] = make_uint2(keys[it], (uint32_t)(base + it * kFiltThreads + tid));
      }
    }
  }
  __syncthreads();
  const int n = l_count;
  if (n == 0) return;
  if (tid == 0) g_base = atomicAdd(&st.cand_count[h * kCountStride], n);
  __syncthreads();
  const int gb = g_base;
  for (int j = tid; j < n; j += kFiltThreads) {
    const int p = gb + j;
    if (p < cand_cap) cand[(int64_t)h * cand_cap + p] = lc[j];
  }
}

// --------------------------------------------------------------------------- score + filter through the score index
// Same output as score_filter_kernel (the candidate list of all rows with key >= bound, as a set), read from
// the 8-bit copy of A_K in whitened coordinates: 34 bytes per row instead of 64.  Every wave solves
// W q' = q (back substitution, lane i holds row i of W; q' ends up in scalar registers); for every
// row an upper bound of its (rounded) score follows from the copy:
//   |score - s~| <= D = scale * |q'|_1 * kSidxDFactor,   s~ = scale * sum_j (u_j - 128) q'_j
//   round_bf16(score) <= s~ + D + (|s~| + D) / 256       (half a bf16 ulp)
// Rows whose bound reaches the threshold (or is not a number) are rescored exactly from A_K; only
// those that really pass enter the list.  Laid out for the memory system:
//  * consecutive lanes read consecutive 16-byte vectors of the copy (a row of R bytes is shared by R / 16 lanes, which
//    each keep the 16 elements of q' they need and add their partial sums across lanes), with non-temporal loads;
//  * a wave works on steps of kScanU vectors per lane and requests the next step's vectors before it evaluates the
//    current ones, so its loads never drain;
//  * nothing is done per workgroup: every wave keeps its own list of rows to rescore and its own list of exact hits
//    in LDS, rescoring 64 rows at a time while its next vectors are in flight, so that there is no barrier and
//    no common phase in which every workgroup of the launch has stopped reading.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
constexpr int kScanU = 4;
constexpr int kScanWaves = kFiltThreads / kWave;

template <typename T, int R>
__global__ __launch_bounds__(kFiltThreads) void score_prefilter_kernel(
    const T* __restrict__ a_k, int64_t head_stride, const T* __restrict__ q_hat, int64_t m, int r, int round_bf16,
    SelState st, uint2* __restrict__ cand, int cand_cap, FilterQ fq, ScoreIndexView six) {
  static_assert(R == 16 || R == 32 || R == 64, "the score index covers ranks 16, 32, 64");
  constexpr int QV = R / 16;                  // lanes per row
  constexpr int kRowsPerLoad = kWave / QV;    // rows that one load of a wave covers
  constexpr int kStepRows = kRowsPerLoad * kScanU;
  constexpr int kMaybeCap = kWave + kStepRows;
  constexpr int kHitCap = 2 * kWave;
  __shared__ uint32_t maybe_s[kScanWaves][kMaybeCap];
  __shared__ uint2 hits_s[kScanWaves][kHitCap];
  __shared__ __align__(16) float qx_s[kScanWaves][R];  // the proxy query as the exact score uses it (a copy per wave)
  __shared__ int resc_s;
  const int h = blockIdx.y;
  const int tid = threadIdx.x, lane = lane_id(), w = wave_id();
  const T* A = a_k + (int64_t)h * head_stride;
  const uint8_t* QA = six.qa + (int64_t)h * six.head_rows * R;
  const uint16_t* QS = six.qs + (int64_t)h * six.head_rows;
  uint32_t* maybe = maybe_s[w];
  uint2* hits = hits_s[w];
  if (tid == 0) resc_s = 0;
  const int sub = lane % QV;        // which 16 bytes of its row this lane reads
  const int lrow = lane / QV;       // row of this lane within a load
  const int64_t n_steps = (m + kStepRows - 1) / kStepRows;
  const int64_t s_stride = (int64_t)gridDim.x * kScanWaves;
  int64_t s_cur = (int64_t)blockIdx.x * kScanWaves + w;
  const bool has_work = s_cur < n_steps;  // (wave-uniform)

  u32x4_t buf[2][kScanU];
  uint16_t scb[2][kScanU];
  auto request = [&](int b, int64_t s) {
#pragma unroll
    for (int u = 0; u < kScanU; ++u) {
      const int64_t row = min(s * kStepRows + u * kRowsPerLoad + lrow, m - 1);
      buf[b][u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(QA + row * R) + sub);
      scb[b][u] = __builtin_nontemporal_load(QS + row);
    }
  };
  if (has_work) {  // two steps are on their way while the proxy query is resolved
    request(0, s_cur);
    if (s_cur + s_stride < n_steps) request(1, s_cur + s_stride);
  }

  const uint32_t t_prev = st.t_low[h];
  const float qn_prev = st.q_norm[h];
  const bool pending = fq.iter_out != nullptr;
  float sacc[kFiltMaxIt], oit[kFiltMaxIt];
  if (pending) {
    als_delta_sums<kFiltMaxIt>(fq.deltas, fq.bh, fq.max_iter, sacc);
#pragma unroll
    for (int it = 0; it < kFiltMaxIt; ++it)
      oit[it] = fq.iter_out[((int64_t)h * fq.max_iter + min(it, fq.max_iter - 1)) * 2 * r + min(lane, r - 1)];
  }
  // row `lane` of W and 1 / W_ll (lanes >= R repeat the last row; their results are never read)
  const float* Wm = six.wm + (int64_t)h * (R * R + R);
  float qh[16];  // the 16 elements of q' that meet this lane's bytes
  float qsum = 0.0f, ql1 = 0.0f, ql2 = 0.0f;
  {
    float wrow[R];
    const float4* wp = reinterpret_cast<const float4*>(Wm + min(lane, R - 1) * R);
#pragma unroll
    for (int c = 0; c < R / 4; ++c) {
      const float4 w4 = wp[c];
      wrow[4 * c + 0] = w4.x;
      wrow[4 * c + 1] = w4.y;
      wrow[4 * c + 2] = w4.z;
      wrow[4 * c + 3] = w4.w;
    }
    const float dinv = Wm[R * R + min(lane, R - 1)];
    float q_lane = 0.0f;  // element `lane` of the proxy query as the exact score uses it
    if (!pending) q_lane = ld_f32<T>(q_hat, (int64_t)h * r + min(lane, R - 1));
    if (pending) {
      const int chosen = als_decide<kFiltMaxIt>(sacc, fq.bh, fq.max_iter, r, fq.tol);
      float qv = oit[0];
#pragma unroll
      for (int it = 1; it < kFiltMaxIt; ++it) qv = chosen == it ? oit[it] : qv;
      if (blockIdx.x == 0 && tid < r) st_f32<T>((T*)fq.q_hat_out, (int64_t)h * r + tid, qv);
      q_lane = sizeof(T) == 2 ? round_to_bf16_f32(qv) : qv;
    }
    if (lane < R) qx_s[w][lane] = lane < r ? q_lane : 0.0f;
    // q' from W q' = q, last unknown first; lane i keeps the residual of equation i
    float qc[R];
    float resid = q_lane;
#pragma unroll
    for (int j = R - 1; j >= 0; --j) {
      const float x = sidx_readlane(resid * dinv, j);
      qc[j] = x;
      resid = __builtin_fmaf(-x, wrow[j], resid);
    }
#pragma unroll
    for (int j = 0; j < R; ++j) {
      qsum += qc[j];
      ql1 += fabsf(qc[j]);
      ql2 = fmaf(qc[j], qc[j], ql2);
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      float x = qc[e];
#pragma unroll
      for (int c = 1; c < QV; ++c) x = sub == c ? qc[c * 16 + e] : x;
      qh[e] = x;
    }
  }
  const float qn = sqrtf(ql2);
  const uint32_t tl = rescaled_bound(t_prev, qn_prev, qn, round_bf16);
  if (tid == 0 && blockIdx.x == 0) {
    st.t_used[h] = tl;
    st.q_cur[h] = qn;
  }
  const float dfac = ql1 * kSidxDFactor;
  const bool any = tl != 0xffffffffu;
  const float thr = key_score(tl);
  const float thr_lo = thr - fabsf(thr) * 1e-6f;
  __syncthreads();  // (resc_s is zero)

  int n_maybe = 0, n_hits = 0, n_resc = 0;  // (wave-uniform)
  auto lds_wave_sync = [&]() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  // this wave's exact hits go to the head's list
  auto flush_hits = [&]() {
    if (n_hits == 0) return;
    int gb = 0;
    if (lane == 0) gb = atomicAdd(&st.cand_count[h * kCountStride], n_hits);
    gb = __builtin_amdgcn_readfirstlane(gb);
    lds_wave_sync();
    for (int j = lane; j < n_hits; j += kWave) {
      const int p = gb + j;
      if (p < cand_cap) cand[(int64_t)h * cand_cap + p] = hits[j];  // (beyond the capacity the count alone tells the select kernel)
    }
    lds_wave_sync();
    n_hits = 0;
  };
  // exact scores of the last (up to) 64 rows of this wave's list
  auto rescore = [&]() {
    const int take = min(n_maybe, kWave);
    const int first = n_maybe - take;
    lds_wave_sync();
    const uint32_t i = maybe[first + min(lane, take - 1)];
    // the exact score of row i: the chain of RowScorer::score, with the query read from LDS (unconditional load,
    // masked below)
    constexpr int VEC = Vec16<T>::N;
    Vec16<T> xv[R / VEC];
#pragma unroll
    for (int c = 0; c < R / VEC; ++c) xv[c].load(A + (int64_t)i * R + c * VEC);
    float acc = 0.0f;
#pragma unroll
    for (int c = 0; c < R / VEC; ++c) {
      float f[VEC];
      xv[c].unpack(f);
#pragma unroll
      for (int e4 = 0; e4 < VEC / 4; ++e4) {
        const float4 q4 = reinterpret_cast<const float4*>(qx_s[w])[(c * VEC) / 4 + e4];
        acc = __builtin_fmaf(f[4 * e4 + 0], q4.x, acc);
        acc = __builtin_fmaf(f[4 * e4 + 1], q4.y, acc);
        acc = __builtin_fmaf(f[4 * e4 + 2], q4.z, acc);
        acc = __builtin_fmaf(f[4 * e4 + 3], q4.w, acc);
      }
    }
    if (round_bf16) acc = round_to_bf16_f32(acc);
    if (acc == 0.0f) acc = 0.0f;
    const uint32_t key = score_key(acc);
    const bool hit = lane < take && key >= tl;
    int wt;
    const int rk = wave_rank(hit, wt);
    if (hit) hits[n_hits + rk] = make_uint2(key, i);
    n_hits += wt;
    n_maybe = first;
    n_resc += take;
    if (n_hits > kHitCap - kWave) flush_hits();
  };
  auto evaluate = [&](int b, int64_t s) {
    uint32_t mask = 0;
#pragma unroll
    for (int u = 0; u < kScanU; ++u) {
      const uint32_t wv[4] = {buf[b][u].x, buf[b][u].y, buf[b][u].z, buf[b][u].w};
      float t = 0.0f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        t = fmaf((float)((wv[e] >> 0) & 0xffu), qh[e * 4 + 0], t);
        t = fmaf((float)((wv[e] >> 8) & 0xffu), qh[e * 4 + 1], t);
        t = fmaf((float)((wv[e] >> 16) & 0xffu), qh[e * 4 + 2], t);
        t = fmaf((float)((wv[e] >> 24) & 0xffu), qh[e * 4 + 3], t);
      }
      t = group_sum(t, QV);
      const float scale = sidx_scale_from_bits(scb[b][u]);
      const float sa = scale * (t - 128.0f * qsum);
      const float dd = scale * dfac;
      const float ub = sa + dd + (fabsf(sa) + dd) * (1.0f / 256.0f);
      const int64_t row = s * kStepRows + u * kRowsPerLoad + lrow;
      if (any && sub == 0 && row < m && !(ub < thr_lo)) mask |= 1u << u;
    }
    const int cnt = __popc(mask);
    const int incl = wave_inclusive_sum(cnt);
    const int wtot = __builtin_amdgcn_readlane(incl, kWave - 1);
    if (wtot) {
      int pos = n_maybe + incl - cnt;
#pragma unroll
      for (int u = 0; u < kScanU; ++u)
        if ((mask >> u) & 1u) maybe[pos++] = (uint32_t)(s * kStepRows + u * kRowsPerLoad + lrow);
      n_maybe += wtot;
    }
  };
  if (has_work) {
    // evaluate a step, ask for the step after the next into the registers it leaves, then rescore what has gathered
    while (true) {
      evaluate(0, s_cur);
      if (s_cur + 2 * s_stride < n_steps) request(0, s_cur + 2 * s_stride);
      while (n_maybe >= kWave) rescore();
      s_cur += s_stride;
      if (s_cur >= n_steps) break;
      evaluate(1, s_cur);
      if (s_cur + 2 * s_stride < n_steps) request(1, s_cur + 2 * s_stride);
      while (n_maybe >= kWave) rescore();
      s_cur += s_stride;
      if (s_cur >= n_steps) break;
    }
    if (n_maybe > 0) rescore();
    flush_hits();
    if (lane == 0 && n_resc) atomicAdd(&resc_s, n_resc);
  }
  __syncthreads();
  if (tid == 0) {
    const int slot = h * (int)gridDim.x + (int)blockIdx.x;
    if (slot < st.rescored_cap) st.rescored[slot] = resc_s;
  }
}

// --------------------------------------------------------------------------- select (+ diff)
#ifndef LRQK_SEL_THREADS
#define LRQK_SEL_THREADS 1024
#endif
constexpr int kSelThreads = LRQK_SEL_THREADS;
// The bound carried to the next call is the key of rank 1.5 k: the list then holds ~1.5 k candidates per
// head and stays usable as long as the number of rows above the (rescaled) bound does not drop by a third
// from one call to the next.  (2 k: 1.3 us slower per 128K step; 1.25 k: 3 rescans in 16384 head-steps.)
constexpr int kBoundRankNum = 3, kBoundRankDen = 2;
constexpr int kSelWaves = kSelThreads / kWave;
constexpr int kChunkBits = 262144;            // token ids covered by one bitmap pass
constexpr int kChunkWords = kChunkBits / 32;  // 8192 words = 32 KB per bitmap
constexpr int kBins = 4096;
constexpr int kBinsPT = kBins / kSelThreads;          // histogram bins per thread
constexpr int kWordsPT = kChunkWords / kSelThreads;   // bitmap words per thread
constexpr int kFusedDiffMaxK = 4096;          // LDS budget of the in-kernel diff

// Inclusive block scan of two counters at once.  scratch: 2 * kSelWaves ints.  Two barriers.
__device__ __forceinline__ void block_inclusive_sum2(int& a, int& b, int* scratch, int& tot_a, int& tot_b) {
  const int ia = wave_inclusive_sum(a), ib = wave_inclusive_sum(b);
  if (lane_id() == kWave - 1) {
    scratch[wave_id()] = ia;
    scratch[kSelWaves + wave_id()] = ib;
  }
  __syncthreads();
  int base_a = 0, base_b = 0, ta = 0, tb = 0;
#pragma unroll
  for (int w = 0; w < kSelWaves; ++w) {
    const int ca = scratch[w], cb = scratch[kSelWaves + w];
    if (w < wave_id()) {
      base_a += ca;
      base_b += cb;
    }
    ta += ca;
    tb += cb;
  }
  __syncthreads();
  a = base_a + ia;
  b = base_b + ib;
  tot_a = ta;
  tot_b = tb;
}

// Workgroup-wide exclusive ranks of two predicates in thread order (ballots, no scan).
// scratch: 2 * kSelWaves ints.  Two barriers.
__device__ __forceinline__ void block_rank2(bool pa, bool pb, int* scratch, int& rank_a, int& rank_b, int& tot_a,
                                            int& tot_b) {
  int wa, wb;
  const int ra = wave_rank(pa, wa), rb = wave_rank(pb, wb);
  if (lane_id() == 0) {
    scratch[wave_id()] = wa;
    scratch[kSelWaves + wave_id()] = wb;
  }
  __syncthreads();
  int base_a = 0, base_b = 0, ta = 0, tb = 0;
#pragma unroll
  for (int w = 0; w < kSelWaves; ++w) {
    const int ca = scratch[w], cb = scratch[kSelWaves + w];
    if (w < wave_id()) {
      base_a += ca;
      base_b += cb;
    }
    ta += ca;
    tb += cb;
  }
  __syncthreads();
  rank_a = base_a + ra;
  rank_b = base_b + rb;
  tot_a = ta;
  tot_b = tb;
}

// From two histograms of kBins bins (kBinsPT bins per thread): the digit of the need_a-th largest
// element of hist_a and of the need_b-th largest of hist_b, with the ranks inside those
// digits.  s_res: 4 shared ints.  Three barriers.
__device__ __forceinline__ void find_digits(const uint32_t* hist_a, const uint32_t* hist_b, int need_a, int need_b,
                                            int* scratch, int* s_res, int& dig_a, int& rem_a, int& dig_b, int& rem_b) {
  const int tid = threadIdx.x;
  int ca[kBinsPT], cb[kBinsPT], la = 0, lb = 0;
#pragma unroll
  for (int x = 0; x < kBinsPT; ++x) {
    ca[x] = (int)hist_a[tid * kBinsPT + x];
    cb[x] = (int)hist_b[tid * kBinsPT + x];
    la += ca[x];
    lb += cb[x];
  }
  int ia = la, ib = lb, ta, tb;
  block_inclusive_sum2(ia, ib, scratch, ta, tb);
  const int above_a = ta - ia, above_b = tb - ib;  // elements in bins above this thread's bins
  if (above_a < need_a && need_a <= above_a + la) {
    int c = above_a;
#pragma unroll
    for (int x = kBinsPT - 1; x >= 0; --x) {
      if (c < need_a && c + ca[x] >= need_a) {
        s_res[0] = tid * kBinsPT + x;
        s_res[1] = need_a - c;
      }
      c += ca[x];
    }
  }
  if (above_b < need_b && need_b <= above_b + lb) {
    int c = above_b;
#pragma unroll
    for (int x = kBinsPT - 1; x >= 0; --x) {
      if (c < need_b && c + cb[x] >= need_b) {
        s_res[2] = tid * kBinsPT + x;
        s_res[3] = need_b - c;
      }
      c += cb[x];
    }
  }
  __syncthreads();
  dig_a = s_res[0];
  rem_a = s_res[1];
  dig_b = s_res[2];
  rem_b = s_res[3];
}

struct DiffArgs {
  int32_t* hit;        // [bh][hit_stride] resident token ids, nullptr = no diff
  int64_t hit_stride;
  uint8_t* evict;      // [bh][k] or nullptr
  int32_t* miss_slots; // [bh][k] or nullptr
  int32_t* miss_count; // [bh] or nullptr
  int replace_all;     // ablation: hit <- new, everything refetched
  int32_t* miss_old;   // [bh][k] or nullptr: token that the j-th refetched slot held before
  int32_t* miss_new;   // [bh][k] or nullptr: token that the j-th refetched slot holds now
  int32_t* vic_ptr;    // victim FIFO bookkeeping (nullptr = no victim cache): next insert position per head,
  int32_t* vic_base;   //   and where this step's victims start
  int vic_nv;
};

// mode: 0 = use the candidate list if valid, else compute the head's keys from A_K;
//       1 = keys[] already holds the head's keys (caller-provided scores).
// Dynamic LDS: gt | eq bitmaps (2 * kChunkWords words), then, with a diff, 10*k bytes.
// LDS blocks of the selector (declared by the kernels, so that the two bodies below share them)
struct SelLds {
  uint32_t* dyn;     // dynamic LDS
  uint32_t* hist;    // [kBins]
  uint32_t* hist_b;  // [kBins], directly behind hist
  int* scratch;      // [2 * kSelWaves]
  uint32_t* wred;    // [2 * kSelWaves]
  int* s_res;        // [8]
  int* s_n;          // [1]
};
#define LRQK_SEL_LDS(L)                                           \
  extern __shared__ __align__(16) uint32_t dyn_lds[];             \
  __shared__ __align__(16) uint32_t hist2_lds[2 * kBins];         \
  __shared__ int scratch_lds[2 * kSelWaves];                      \
  __shared__ uint32_t wred_lds[2 * kSelWaves];                    \
  __shared__ int s_res_lds[8];                                    \
  __shared__ int s_n_lds;                                         \
  SelLds L{dyn_lds, hist2_lds, hist2_lds + kBins, scratch_lds, wred_lds, s_res_lds, &s_n_lds};

// n_list: the length of the head's candidate list if the caller has read it already (and every thread of the
// workgroup with it), else -1.
template <typename T, int R>
__device__ __forceinline__ void select_generic(const SelLds& L, int mode, const uint2* __restrict__ cand_all, int cand_cap,
                                               SelState st, uint32_t* __restrict__ keys_all, int64_t key_stride,
                                               const T* __restrict__ a_k, int64_t head_stride,
                                               const T* __restrict__ q_hat, int64_t m, int r, int round_bf16, int k,
                                               int32_t* __restrict__ out_all, int64_t out_stride, DiffArgs df,
                                               int n_list, int bound_rank_k = 0) {
  uint32_t* const dyn = L.dyn;
  uint32_t* const hist = L.hist;
  uint32_t* const hist_b = L.hist_b;
  int* const scratch = L.scratch;
  uint32_t* const wred = L.wred;
  int* const s_res = L.s_res;
  int& s_n = *L.s_n;
  uint32_t* gt = dyn;
  uint32_t* eq = dyn + kChunkWords;
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int h = blockIdx.x;
  uint32_t* keys = keys_all + (int64_t)h * key_stride;
  const uint2* cand = cand_all + (int64_t)h * cand_cap;
  int32_t* out = out_all + (int64_t)h * out_stride;

  // the resident token ids of the fused diff do not depend on the selection: requested now,
  // used at the end (items tid*kDiffIpt .. +kDiffIpt-1, contiguous per thread to keep slot order)
  constexpr int kDiffIpt = kFusedDiffMaxK / kSelThreads;
  const int ipt = (k + kSelThreads - 1) / kSelThreads;  // items per thread actually in use (<= kDiffIpt)
  int32_t hv[kDiffIpt];
  if (df.hit != nullptr && !df.replace_all) {
#pragma unroll
    for (int u = 0; u < kDiffIpt; ++u)
      hv[u] = df.hit[(int64_t)h * df.hit_stride + min(tid * ipt + u, k - 1)];
  }
  bool fast = false;
  int64_t N = m;
  uint32_t lo = 0;
  if (mode == 0) {
    if (tid == 0 && n_list < 0) s_n = st.cand_count[h * kCountStride];
    __syncthreads();
    if (tid == 0) st.cand_count[h * kCountStride] = 0;  // re-arm for the next call (every thread has read the count by now)
    const int n = n_list < 0 ? s_n : n_list;
    fast = n >= k && n <= cand_cap;
    if (fast) {
      N = n;
      lo = st.t_used[h];  // every candidate key is >= the bound the filter used
    } else {
      const T* A = a_k + (int64_t)h * head_stride;
      RowScorer<T, R> rs;
      rs.init(q_hat + (int64_t)h * r, r, round_bf16);
      for (int64_t i = tid; i < m; i += kSelThreads) keys[i] = score_key(rs.score(A, i));
      __threadfence_block();
      __syncthreads();
    }
    if (tid == 0) atomicAdd(&st.stats[fast ? 0 : (n < k ? 1 : 2)], 1);
  }
  // The candidate list is read once into registers (one batch of independent loads); the
  // rescan path walks the key array in batches of 8 independent loads per thread.
  constexpr int kRegCand = 8192 / kSelThreads;
  const bool in_regs = fast && N <= (int64_t)kRegCand * kSelThreads;
  uint2 creg[kRegCand];
  if (in_regs) {
#pragma unroll
    for (int u = 0; u < kRegCand; ++u) {
      const int64_t j = tid + (int64_t)u * kSelThreads;
      creg[u] = cand[min(j, N - 1)];  // unconditional (clamped); entries with j >= N are never used
    }
  }
  auto for_each = [&](auto&& f) {
    if (in_regs) {
#pragma unroll
      for (int u = 0; u < kRegCand; ++u) {
        const int64_t j = tid + (int64_t)u * kSelThreads;
        if (j < N) f(creg[u].x, (int64_t)creg[u].y);
      }
    } else if (fast) {
      for (int64_t j = tid; j < N; j += kSelThreads) {
        const uint2 c = cand[j];
        f(c.x, (int64_t)c.y);
      }
    } else {
      for (int64_t j0 = tid; j0 < N; j0 += (int64_t)8 * kSelThreads) {
        uint32_t kk[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) kk[u] = keys[min(j0 + (int64_t)u * kSelThreads, N - 1)];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int64_t j = j0 + (int64_t)u * kSelThreads;
          if (j < N) f(kk[u], j);
        }
      }
    }
  };

  // ---- range of the keys: lowest key (known for candidates), highest key, and the common
  // trailing zero bits of (key - lo) (bf16-rounded scores leave 16 of them)
  uint32_t vmin = 0xffffffffu, vmax = 0u, vor = 0u;
  for_each([&](uint32_t key, int64_t) {
    vmin = min(vmin, key);
    vmax = max(vmax, key);
  });
  if (!fast) {
    vmin = wave_reduce_u32(vmin, [](uint32_t a, uint32_t b) { return a < b ? a : b; });
    if (lane == 0) wred[wave] = vmin;
    __syncthreads();
    vmin = 0xffffffffu;
#pragma unroll
    for (int w = 0; w < kSelWaves; ++w) vmin = min(vmin, wred[w]);
    lo = vmin;
    __syncthreads();
  }
  for_each([&](uint32_t key, int64_t) { vor |= key - lo; });
  vmax = wave_reduce_u32(vmax, [](uint32_t a, uint32_t b) { return a > b ? a : b; });
  vor = wave_reduce_u32(vor, [](uint32_t a, uint32_t b) { return a | b; });
  if (lane == 0) {
    wred[wave] = vmax;
    wred[kSelWaves + wave] = vor;
  }
  for (int i = tid; i < kBins; i += kSelThreads) {  // first-pass histograms, zeroed under the same barrier
    hist[i] = 0;
    hist_b[i] = 0;
  }
  if (tid == 0) s_res[0] = s_res[1] = s_res[2] = s_res[3] = 0;
  __syncthreads();
  vmax = 0u;
  vor = 0u;
#pragma unroll
  for (int w = 0; w < kSelWaves; ++w) {
    vmax = max(vmax, wred[w]);
    vor |= wred[kSelWaves + w];
  }
  const uint32_t range = vmax - lo;
  const int tz = vor ? (__ffs((int)vor) - 1) : 0;              // bits that are zero in every offset
  const int nbits = range ? (32 - __clz((int)(range >> tz))) : 0;  // significant bits of (key - lo) >> tz
  const int s1 = max(nbits - 12, 0), s2 = max(s1 - 12, 0);

  // rank that defines the next t_low
  const int k2 = (int)min(bound_rank_k > 0 ? (int64_t)bound_rank_k : ((int64_t)kBoundRankNum * k) / kBoundRankDen, N);
  // ---- pass 1 (both ranks share it)
  for_each([&](uint32_t key, int64_t) { atomicAdd(&hist[((key - lo) >> tz) >> s1], 1u); });
  __syncthreads();
  int D1, need1, E1, needE;
  find_digits(hist, hist, k, k2, scratch, s_res, D1, need1, E1, needE);
  uint32_t offT = (uint32_t)D1 << s1, offE = (uint32_t)E1 << s1;
  int need_eq = need1;
  if (s1 > 0) {
    // ---- pass 2: next (up to) 12 bits under each prefix
    for (int i = tid; i < kBins; i += kSelThreads) {
      hist[i] = 0;
      hist_b[i] = 0;
    }
    __syncthreads();
    const uint32_t m2 = (1u << (s1 - s2)) - 1u;
    for_each([&](uint32_t key, int64_t) {
      const uint32_t o = (key - lo) >> tz;
      const uint32_t top = o >> s1;
      if (top == (uint32_t)D1) atomicAdd(&hist[(o >> s2) & m2], 1u);
      if (top == (uint32_t)E1) atomicAdd(&hist_b[(o >> s2) & m2], 1u);
    });
    __syncthreads();
    int D2, need2, E2, needE2;
    find_digits(hist, hist_b, need1, needE, scratch, s_res, D2, need2, E2, needE2);
    offT |= (uint32_t)D2 << s2;
    offE |= (uint32_t)E2 << s2;
    need_eq = need2;
    if (s2 > 0) {
      // ---- pass 3: the last s2 <= 8 bits
      for (int i = tid; i < kBins; i += kSelThreads) hist[i] = 0;
      __syncthreads();
      const uint32_t m3 = (1u << s2) - 1u;
      const uint32_t pre = offT >> s2;
      for_each([&](uint32_t key, int64_t) {
        const uint32_t o = (key - lo) >> tz;
        if ((o >> s2) == pre) atomicAdd(&hist[o & m3], 1u);
      });
      __syncthreads();
      int D3, need3, dummy_d, dummy_r;
      find_digits(hist, hist, need2, need2, scratch, s_res, D3, need3, dummy_d, dummy_r);
      offT |= (uint32_t)D3;
      need_eq = need3;
    }
  }
  const uint32_t Tk = lo + (offT << tz);
  if (tid == 0) {
    st.t_low[h] = lo + (offE << tz);  // rank >= 1.5k (rounded down to the resolved bits)
    st.q_norm[h] = mode == 0 ? st.q_cur[h] : 0.0f;
  }

  // ---- ordered output through two bitmaps over the token ids: gt (key > T), eq (key == T).
  // Every index with key > T is emitted, plus the first need_eq indices with key == T.
  const bool do_diff = df.hit != nullptr;
  int32_t* new_s = reinterpret_cast<int32_t*>(dyn + 2 * kChunkWords);  // [k] when do_diff
  int out_pos = 0, eq_seen = 0;
  for (int64_t c0 = 0; c0 < m; c0 += kChunkBits) {
    const int span = (int)min((int64_t)kChunkBits, m - c0);
    const int words = (span + 31) >> 5;
    // each thread owns W consecutive words (4 or 8: whole 16-byte vectors, read once into registers)
    const int W = (((words + kSelThreads - 1) / kSelThreads) + 3) & ~3;
    {
      uint4* g4 = reinterpret_cast<uint4*>(gt);
      uint4* e4 = reinterpret_cast<uint4*>(eq);
      for (int i = tid; i < W * kSelThreads / 4; i += kSelThreads) {
        g4[i] = make_uint4(0, 0, 0, 0);
        e4[i] = make_uint4(0, 0, 0, 0);
      }
    }
    __syncthreads();
    for_each([&](uint32_t key, int64_t idx) {
      const int64_t rel = idx - c0;
      if (key >= Tk && rel >= 0 && rel < span) atomicOr(key > Tk ? &gt[rel >> 5] : &eq[rel >> 5], 1u << (rel & 31));
    });
    __syncthreads();
    const int w0 = tid * W;
    uint32_t gwr[kWordsPT], ewr[kWordsPT];
#pragma unroll
    for (int q = 0; q < kWordsPT / 4; ++q) {
      uint4 a = make_uint4(0, 0, 0, 0), b = a;
      if (q * 4 < W) {
        a = reinterpret_cast<const uint4*>(gt)[(w0 >> 2) + q];
        b = reinterpret_cast<const uint4*>(eq)[(w0 >> 2) + q];
      }
      gwr[4 * q] = a.x; gwr[4 * q + 1] = a.y; gwr[4 * q + 2] = a.z; gwr[4 * q + 3] = a.w;
      ewr[4 * q] = b.x; ewr[4 * q + 1] = b.y; ewr[4 * q + 2] = b.z; ewr[4 * q + 3] = b.w;
    }
    int cg = 0, ce = 0;
#pragma unroll
    for (int x = 0; x < kWordsPT; ++x) {
      cg += __popc(gwr[x]);
      ce += __popc(ewr[x]);
    }
    int g_incl = cg, e_incl = ce, g_tot, e_tot;
    block_inclusive_sum2(g_incl, e_incl, scratch, g_tot, e_tot);
    int e_run = eq_seen + e_incl - ce;  // equal keys before this thread's words (all chunks)
    int pos = out_pos + (g_incl - cg) + (min(e_run, need_eq) - min(eq_seen, need_eq));
#pragma unroll
    for (int x = 0; x < kWordsPT; ++x) {
      const uint32_t gw = gwr[x], ew = ewr[x];
      uint32_t both = gw | ew;
      uint32_t sel = gw;
      while (both) {
        const int bit = __ffs((int)both) - 1;
        both &= both - 1;
        const int32_t idx = (int32_t)(c0 + (int64_t)(w0 + x) * 32 + bit);
        bool take = true;
        if (!((gw >> bit) & 1u)) {
          take = e_run < need_eq;
          ++e_run;
          if (take) sel |= 1u << bit;
        }
        if (take) {
          out[pos] = idx;
          if (do_diff) new_s[pos] = idx;
          ++pos;
        }
      }
      if (do_diff && sel != gw) gt[w0 + x] = sel;  // gt then marks exactly the selected tokens (used by the diff)
    }
    out_pos += g_tot + (min(eq_seen + e_tot, need_eq) - min(eq_seen, need_eq));
    eq_seen += e_tot;
    __syncthreads();
  }
  if (!do_diff) return;

  // ---- hit/miss diff of this head (the selection is still in LDS).  new_s is ascending, so
  // membership of a resident token is a binary search; a resident token that is found marks
  // its position as matched, which yields the missing tokens without sorting the resident set.
  int32_t* hit = df.hit + (int64_t)h * df.hit_stride;
  if (df.replace_all) {
    for (int s = tid; s < k; s += kSelThreads) {
      hit[s] = new_s[s];
      if (df.evict) df.evict[(int64_t)h * k + s] = 1;
      if (df.miss_slots) df.miss_slots[(int64_t)h * k + s] = s;
    }
    if (tid == 0 && df.miss_count) df.miss_count[h] = k;
    return;
  }
  int32_t* miss_s = new_s + k;                                   // [k] missing tokens, ascending
  uint8_t* matched = reinterpret_cast<uint8_t*>(miss_s + k);     // [k]
  uint8_t* evict_s = matched + k;                                // [k]
  if (m <= kChunkBits) {
    // One chunk: gt[] still marks the selected tokens.  eq[] becomes the bitmap of the resident
    // tokens; membership either way is one bit test.
    const int words = (int)((m + 31) >> 5);
    for (int i = tid; i < words; i += kSelThreads) eq[i] = 0;
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kDiffIpt; ++u) {
      const int s = tid * ipt + u;
      if (u < ipt && s < k) {
        const int32_t v = hv[u];
        const bool in_range = v >= 0 && v < m;
        if (in_range) atomicOr(&eq[v >> 5], 1u << (v & 31));
        const bool found = in_range && ((gt[in_range ? (v >> 5) : 0] >> (v & 31)) & 1u);
        evict_s[s] = found ? 0 : 1;
      }
    }
    __syncthreads();
    for (int i = tid; i < k; i += kSelThreads) {
      const int32_t t = new_s[i];
      matched[i] = (uint8_t)((eq[t >> 5] >> (t & 31)) & 1u);
    }
  } else {
    for (int i = tid; i < k; i += kSelThreads) matched[i] = 0;
    __syncthreads();
    // lower bound of every resident id in new_s; the searches of a thread's items advance in step
    int lo_i[kDiffIpt], len[kDiffIpt];
#pragma unroll
    for (int u = 0; u < kDiffIpt; ++u) {
      lo_i[u] = 0;
      len[u] = k;
    }
    for (int step = 32 - __clz(k); step > 0; --step) {
      int32_t probe[kDiffIpt];
#pragma unroll
      for (int u = 0; u < kDiffIpt; ++u)
        if (u < ipt) probe[u] = new_s[min(lo_i[u] + (len[u] >> 1), k - 1)];
#pragma unroll
      for (int u = 0; u < kDiffIpt; ++u) {
        const int half = len[u] >> 1;
        if (u < ipt && len[u] > 0) {
          if (probe[u] < hv[u]) {
            lo_i[u] += half + 1;
            len[u] -= half + 1;
          } else {
            len[u] = half;
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < kDiffIpt; ++u) {
      const int s = tid * ipt + u;
      if (u < ipt && s < k) {
        const bool found = lo_i[u] < k && new_s[min(lo_i[u], k - 1)] == hv[u];
        if (found) matched[lo_i[u]] = 1;
        evict_s[s] = found ? 0 : 1;
      }
    }
  }
  __syncthreads();
  // both ordered compactions in one sweep: rank of missing tokens and of evicted slots
  int n_missing, n_evict;
  {
    bool miss[kDiffIpt], ev[kDiffIpt];
    int a = 0, b2 = 0;
#pragma unroll
    for (int u = 0; u < kDiffIpt; ++u) {
      const int i = tid * ipt + u;
      miss[u] = u < ipt && i < k && matched[min(i, k - 1)] == 0;
      ev[u] = u < ipt && i < k && evict_s[min(i, k - 1)] != 0;
      a += miss[u] ? 1 : 0;
      b2 += ev[u] ? 1 : 0;
    }
    int ia = a, ib = b2;
    block_inclusive_sum2(ia, ib, scratch, n_missing, n_evict);
    int pa = ia - a, pb = ib - b2;
#pragma unroll
    for (int u = 0; u < kDiffIpt; ++u) {
      const int i = tid * ipt + u;
      if (miss[u]) miss_s[pa++] = new_s[i];
      if (ev[u]) reinterpret_cast<int32_t*>(gt)[pb++] = i;  // evicted slots, ascending (bitmaps are free now)
    }
  }
  __syncthreads();
  const int n_pair = min(n_missing, n_evict);
  const int32_t* ev_list = reinterpret_cast<const int32_t*>(gt);
  for (int j = tid; j < n_pair; j += kSelThreads) {
    const int s = ev_list[j];
    if (df.miss_old) df.miss_old[(int64_t)h * k + j] = hit[s];
    if (df.miss_new) df.miss_new[(int64_t)h * k + j] = miss_s[j];
    hit[s] = miss_s[j];
    if (df.miss_slots) df.miss_slots[(int64_t)h * k + j] = s;
  }
  if (tid == 0 && df.vic_ptr) {
    const int base = df.vic_ptr[h];
    df.vic_base[h] = base;
    df.vic_ptr[h] = (base + min(n_pair, df.vic_nv)) % df.vic_nv;
  }
  if (df.evict) {
    for (int s = tid; s < k; s += kSelThreads) df.evict[(int64_t)h * k + s] = evict_s[s];
  }
  if (tid == 0 && df.miss_count) df.miss_count[h] = n_pair;
}

template <typename T, int R>
__global__ __launch_bounds__(kSelThreads) void select_kernel(int mode, const uint2* __restrict__ cand_all, int cand_cap,
                                                             SelState st, uint32_t* __restrict__ keys_all,
                                                             int64_t key_stride, const T* __restrict__ a_k,
                                                             int64_t head_stride, const T* __restrict__ q_hat, int64_t m,
                                                             int r, int round_bf16, int k, int32_t* __restrict__ out_all,
                                                             int64_t out_stride, DiffArgs df) {
  LRQK_SEL_LDS(L);
  select_generic<T, R>(L, mode, cand_all, cand_cap, st, keys_all, key_stride, a_k, head_stride, q_hat, m, r, round_bf16, k,
                       out_all, out_stride, df, -1);
}

// --------------------------------------------------------------------------- select + diff of the decode step
// The decode step does not need the ascending list of the selected tokens, only what changes: which slots lose
// their token and which tokens come in (row-major pairing: the j-th freed slot takes the j-th smallest new
// token).  With a usable candidate list (k <= n <= 16384 entries, all token ids below 262144) that is done
// without ever ordering the selection: the candidates stay in registers; three bitmaps over the token ids
// (selected, tied at the threshold, resident) turn every membership question into one bit test; the only
// ordered quantities are the ranks of the tied candidates (to take the lowest ids among them) and of the
// incoming tokens, both a prefix count over bitmap words; workgroup scans take one barrier (wave scans by lane
// moves, the wave totals rescanned by every wave).  Anything else (no list, overflow, longer contexts) goes
// through select_generic in the same launch.

// Exclusive scan of two counters in thread order; one barrier.  slot: 2 * kSelWaves ints; consecutive calls must
// be separated by a barrier.
__device__ __forceinline__ void step_scan2(int a, int b, int* slot, int& ex_a, int& ex_b, int& tot_a, int& tot_b) {
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(wave_id());
  const int ia = wave_inclusive_sum(a), ib = wave_inclusive_sum(b);
  if (lane == kWave - 1) {
    slot[wave] = ia;
    slot[kSelWaves + wave] = ib;
  }
  __syncthreads();
  const int ta = lane < kSelWaves ? slot[lane] : 0;
  const int tb = lane < kSelWaves ? slot[kSelWaves + lane] : 0;
  const int sa = wave_inclusive_sum(ta), sb = wave_inclusive_sum(tb);
  const int base_a = wave ? __builtin_amdgcn_readlane(sa, wave - 1) : 0;
  const int base_b = wave ? __builtin_amdgcn_readlane(sb, wave - 1) : 0;
  tot_a = __builtin_amdgcn_readlane(sa, kSelWaves - 1);
  tot_b = __builtin_amdgcn_readlane(sb, kSelWaves - 1);
  ex_a = base_a + ia - a;
  ex_b = base_b + ib - b;
}

// Like find_digits, with the one-barrier scan; cnt_a: number of elements in the digit found for need_a.
// s_res: 5 ints.  Two barriers.
__device__ __forceinline__ void step_find_digits(const uint32_t* hist_a, const uint32_t* hist_b, int need_a, int need_b,
                                                 int* slot, int* s_res, int& dig_a, int& rem_a, int& dig_b, int& rem_b,
                                                 int& cnt_a) {
  const int tid = threadIdx.x;
  int ca[kBinsPT], cb[kBinsPT], la = 0, lb = 0;
#pragma unroll
  for (int x = 0; x < kBinsPT; ++x) {
    ca[x] = (int)hist_a[tid * kBinsPT + x];
    cb[x] = (int)hist_b[tid * kBinsPT + x];
    la += ca[x];
    lb += cb[x];
  }
  int ea, eb, ta, tb;
  step_scan2(la, lb, slot, ea, eb, ta, tb);
  const int above_a = ta - ea - la, above_b = tb - eb - lb;  // elements in bins above this thread's bins
  if (above_a < need_a && need_a <= above_a + la) {
    int c = above_a;
#pragma unroll
    for (int x = kBinsPT - 1; x >= 0; --x) {
      if (c < need_a && c + ca[x] >= need_a) {
        s_res[0] = tid * kBinsPT + x;
        s_res[1] = need_a - c;
        s_res[4] = ca[x];
      }
      c += ca[x];
    }
  }
  if (above_b < need_b && need_b <= above_b + lb) {
    int c = above_b;
#pragma unroll
    for (int x = kBinsPT - 1; x >= 0; --x) {
      if (c < need_b && c + cb[x] >= need_b) {
        s_res[2] = tid * kBinsPT + x;
        s_res[3] = need_b - c;
      }
      c += cb[x];
    }
  }
  __syncthreads();
  dig_a = s_res[0];
  rem_a = s_res[1];
  dig_b = s_res[2];
  rem_b = s_res[3];
  cnt_a = s_res[4];
}

// Dynamic LDS of the step's select: three bitmaps of `words4` words, word prefixes (u16), incoming tokens,
// outgoing tokens (i32 [k] each), freed slots (u16 [k]).
static inline size_t step_select_words4(int64_t m) { return (size_t)(((m + 31) >> 5) + 3) & ~(size_t)3; }
static inline size_t step_select_smem(int64_t m, int k) {
  return step_select_words4(m) * (3 * 4 + 2) + (size_t)k * (4 + 4 + 4 + 2) + 16;
}

template <int CPT>
__device__ __forceinline__ void select_step_fast(const SelLds& L, const uint2* __restrict__ cand, int N, uint32_t lo,
                                                 SelState st, int h, int64_t m, int k, int k2, const DiffArgs& df) {
  const int tid = threadIdx.x;
  const int words = (int)((m + 31) >> 5);
  const int words4 = (words + 3) & ~3;
  uint32_t* bmS = L.dyn;              // selected tokens
  uint32_t* bmE = bmS + words4;       // candidates tied at the threshold
  uint32_t* bmH = bmE + words4;       // resident tokens
  uint16_t* wpre = reinterpret_cast<uint16_t*>(bmH + words4);  // [words4] marked tokens in the words before
  int32_t* miss_s = reinterpret_cast<int32_t*>(wpre + words4);  // [k] incoming tokens, ascending
  int32_t* ev_old = miss_s + k;                                 // [k] tokens of the freed slots
  int32_t* hit_s = ev_old + k;                                  // [k] resident token of every slot (as the step found it)
  uint16_t* ev_slot = reinterpret_cast<uint16_t*>(hit_s + k);   // [k] freed slots, ascending
  uint32_t* hist = L.hist;
  uint32_t* hist_b = L.hist_b;
  uint32_t* bmM = L.hist;             // incoming tokens (takes the place of the two histograms, 2 * kBins words)
  int* s_res = L.s_res;
  int32_t* hit = df.hit + (int64_t)h * df.hit_stride;

  // ---- requests first: the candidates and the resident ids (contiguous per thread, to keep slot order)
  uint2 c[CPT];
#pragma unroll
  for (int u = 0; u < CPT; ++u) c[u] = cand[min(tid + u * kSelThreads, N - 1)];
  constexpr int kIpt = kFusedDiffMaxK / kSelThreads;
  const int ipt = (k + kSelThreads - 1) / kSelThreads;
  int32_t hv[kIpt];
#pragma unroll
  for (int u = 0; u < kIpt; ++u) hv[u] = hit[min(tid * ipt + u, k - 1)];
  // ---- meanwhile: clear the bitmaps and the first histogram
  {
    uint4* z = reinterpret_cast<uint4*>(bmS);
    for (int i = tid; i < 3 * words4 / 4; i += kSelThreads) z[i] = make_uint4(0, 0, 0, 0);
    for (int i = tid; i < kBins; i += kSelThreads) hist[i] = 0;
    if (tid < 8) s_res[tid] = 0;
    if (tid < 2) L.wred[tid] = 0;
  }
  __syncthreads();
  // ---- resident bitmap (the ids also go to LDS: they are needed again after the selection, and registers held
  // that long were spilled); range of the keys
#pragma unroll
  for (int u = 0; u < kIpt; ++u) {
    const int32_t v = hv[u];
    if (u < ipt && tid * ipt + u < k) {
      hit_s[tid * ipt + u] = v;
      if (v >= 0 && v < m) atomicOr(&bmH[v >> 5], 1u << (v & 31));
    }
  }
  uint32_t vmax = 0u, vor = 0u;
#pragma unroll
  for (int u = 0; u < CPT; ++u) {
    if (tid + u * kSelThreads < N) {
      vmax = max(vmax, c[u].x);
      vor |= c[u].x - lo;
    }
  }
  vmax = wave_reduce_u32(vmax, [](uint32_t a, uint32_t b) { return a > b ? a : b; });
  vor = wave_reduce_u32(vor, [](uint32_t a, uint32_t b) { return a | b; });
  if (lane_id() == 0) {
    atomicMax(&L.wred[0], vmax);
    atomicOr(&L.wred[1], vor);
  }
  __syncthreads();
  vmax = L.wred[0];
  vor = L.wred[1];
  const uint32_t range = vmax - lo;
  const int tz = vor ? (__ffs((int)vor) - 1) : 0;
  const int nbits = range ? (32 - __clz((int)(range >> tz))) : 0;
  const int s1 = max(nbits - 12, 0), s2 = max(s1 - 12, 0);
  // ---- radix select of the k-th and k2-th largest keys (one pass for bf16-rounded scores)
#pragma unroll
  for (int u = 0; u < CPT; ++u)
    if (tid + u * kSelThreads < N) atomicAdd(&hist[((c[u].x - lo) >> tz) >> s1], 1u);
  __syncthreads();
  int D1, need1, E1, needE, cntT;
  step_find_digits(hist, hist, k, k2, L.scratch, s_res, D1, need1, E1, needE, cntT);
  uint32_t offT = (uint32_t)D1 << s1, offE = (uint32_t)E1 << s1;
  int need_eq = need1;
  if (s1 > 0) {
    for (int i = tid; i < 2 * kBins; i += kSelThreads) hist[i] = 0;
    __syncthreads();
    const uint32_t m2 = (1u << (s1 - s2)) - 1u;
#pragma unroll
    for (int u = 0; u < CPT; ++u) {
      if (tid + u * kSelThreads < N) {
        const uint32_t o = (c[u].x - lo) >> tz;
        const uint32_t top = o >> s1;
        if (top == (uint32_t)D1) atomicAdd(&hist[(o >> s2) & m2], 1u);
        if (top == (uint32_t)E1) atomicAdd(&hist_b[(o >> s2) & m2], 1u);
      }
    }
    __syncthreads();
    int D2, need2, E2, needE2;
    step_find_digits(hist, hist_b, need1, needE, L.scratch, s_res, D2, need2, E2, needE2, cntT);
    offT |= (uint32_t)D2 << s2;
    offE |= (uint32_t)E2 << s2;
    need_eq = need2;
    if (s2 > 0) {
      for (int i = tid; i < kBins; i += kSelThreads) hist[i] = 0;
      __syncthreads();
      const uint32_t m3 = (1u << s2) - 1u;
      const uint32_t pre = offT >> s2;
#pragma unroll
      for (int u = 0; u < CPT; ++u) {
        if (tid + u * kSelThreads < N) {
          const uint32_t o = (c[u].x - lo) >> tz;
          if ((o >> s2) == pre) atomicAdd(&hist[o & m3], 1u);
        }
      }
      __syncthreads();
      int D3, need3, dd, dr;
      step_find_digits(hist, hist, need2, need2, L.scratch, s_res, D3, need3, dd, dr, cntT);
      offT |= (uint32_t)D3;
      need_eq = need3;
    }
  }
  const uint32_t Tk = lo + (offT << tz);
  if (tid == 0) {
    st.t_low[h] = lo + (offE << tz);
    st.q_norm[h] = st.q_cur[h];
  }
  const bool all_eq = need_eq >= cntT;  // every candidate tied at the threshold is selected: no order needed
  // ---- classify (the histograms are dead: their block becomes the bitmap of the incoming tokens)
  for (int i = tid; i < words4; i += kSelThreads) bmM[i] = 0;
  uint32_t selmask = 0u, eqmask = 0u;
#pragma unroll
  for (int u = 0; u < CPT; ++u) {
    if (tid + u * kSelThreads < N) {
      const uint32_t key = c[u].x, idx = c[u].y;
      if (key > Tk || (all_eq && key == Tk)) {
        selmask |= 1u << u;
        atomicOr(&bmS[idx >> 5], 1u << (idx & 31));
      } else if (key == Tk) {
        eqmask |= 1u << u;
        atomicOr(&bmE[idx >> 5], 1u << (idx & 31));
      }
    }
  }
  __syncthreads();
  const int wpt = (words4 + kSelThreads - 1) / kSelThreads;  // bitmap words per thread (<= kWordsPT)
  const int w0 = tid * wpt;
  if (!all_eq) {
    // the need_eq lowest token ids among the tied candidates: rank = marked tokens before it
    int cnt = 0;
    for (int x = 0; x < wpt; ++x) cnt += (w0 + x < words4) ? __popc(bmE[w0 + x]) : 0;
    int ex, exb, tot, totb;
    step_scan2(cnt, 0, L.scratch, ex, exb, tot, totb);
    for (int x = 0; x < wpt; ++x) {
      if (w0 + x < words4) {
        wpre[w0 + x] = (uint16_t)ex;
        ex += __popc(bmE[w0 + x]);
      }
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < CPT; ++u) {
      if ((eqmask >> u) & 1u) {
        const uint32_t idx = c[u].y;
        const int rank = (int)wpre[idx >> 5] + __popc(bmE[idx >> 5] & ((1u << (idx & 31)) - 1u));
        if (rank < need_eq) {
          selmask |= 1u << u;
          atomicOr(&bmS[idx >> 5], 1u << (idx & 31));
        }
      }
    }
    __syncthreads();
  }
  // ---- diff: slots whose token left the selection; selected tokens that are not resident
  bool ev[kIpt];
  int n_ev = 0;
#pragma unroll
  for (int u = 0; u < kIpt; ++u) {
    const bool live = u < ipt && tid * ipt + u < k;
    const int32_t v = hit_s[live ? tid * ipt + u : 0];
    const bool in_range = v >= 0 && v < m;
    const bool found = in_range && ((bmS[in_range ? (v >> 5) : 0] >> (v & 31)) & 1u);
    ev[u] = live && !found;
    n_ev += ev[u] ? 1 : 0;
  }
  uint32_t missmask = 0u;
#pragma unroll
  for (int u = 0; u < CPT; ++u) {
    if ((selmask >> u) & 1u) {
      const uint32_t idx = c[u].y;
      if (!((bmH[idx >> 5] >> (idx & 31)) & 1u)) {
        missmask |= 1u << u;
        atomicOr(&bmM[idx >> 5], 1u << (idx & 31));
      }
    }
  }
  __syncthreads();
  int cnt_m = 0;
  for (int x = 0; x < wpt; ++x) cnt_m += (w0 + x < words4) ? __popc(bmM[w0 + x]) : 0;
  int ex_ev, ex_m, n_evict, n_missing;
  step_scan2(n_ev, cnt_m, L.scratch, ex_ev, ex_m, n_evict, n_missing);
#pragma unroll
  for (int u = 0; u < kIpt; ++u) {
    if (ev[u]) {
      ev_slot[ex_ev] = (uint16_t)(tid * ipt + u);
      ev_old[ex_ev] = hit_s[tid * ipt + u];
      ++ex_ev;
    }
  }
  for (int x = 0; x < wpt; ++x) {
    if (w0 + x < words4) {
      wpre[w0 + x] = (uint16_t)ex_m;
      ex_m += __popc(bmM[w0 + x]);
    }
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < CPT; ++u) {
    if ((missmask >> u) & 1u) {
      const uint32_t idx = c[u].y;
      miss_s[(int)wpre[idx >> 5] + __popc(bmM[idx >> 5] & ((1u << (idx & 31)) - 1u))] = (int32_t)idx;
    }
  }
  __syncthreads();
  const int n_pair = min(n_missing, n_evict);
  for (int j = tid; j < n_pair; j += kSelThreads) {
    const int s = ev_slot[j];
    const int32_t t_new = miss_s[j];
    if (df.miss_old) df.miss_old[(int64_t)h * k + j] = ev_old[j];
    if (df.miss_new) df.miss_new[(int64_t)h * k + j] = t_new;
    hit[s] = t_new;
    if (df.miss_slots) df.miss_slots[(int64_t)h * k + j] = s;
  }
  if (df.evict) {
#pragma unroll
    for (int u = 0; u < kIpt; ++u)
      if (u < ipt && tid * ipt + u < k) df.evict[(int64_t)h * k + tid * ipt + u] = ev[u] ? 1 : 0;
  }
  if (tid == 0) {
    if (df.vic_ptr) {
      const int base = df.vic_ptr[h];
      df.vic_base[h] = base;
      df.vic_ptr[h] = (base + min(n_pair, df.vic_nv)) % df.vic_nv;
    }
    if (df.miss_count) df.miss_count[h] = n_pair;
    st.cand_count[h * kCountStride] = 0;  // re-arm for the next call
  }
}

// Rank of the key that the next scan's bound is taken from: 1.5 k, doubled (twice at most) for a head
// whose list was unusable lately -- a head whose proxy query jumps from step to step needs more slack, and
// only that head pays for it with more rows to rescore.  state: level in the low byte, calm calls above it.
__device__ __forceinline__ int bound_rank(int k, int level, int64_t n) {
  return (int)min((((int64_t)kBoundRankNum * k) / kBoundRankDen) << level, n);
}
constexpr int kCalmCalls = 32;  // usable lists in a row before a head's slack is halved again

template <typename T, int R>
__global__ __launch_bounds__(kSelThreads) void select_step_kernel(const uint2* __restrict__ cand_all, int cand_cap,
                                                                  SelState st, uint32_t* __restrict__ keys_all,
                                                                  int64_t key_stride, const T* __restrict__ a_k,
                                                                  int64_t head_stride, const T* __restrict__ q_hat,
                                                                  int64_t m, int r, int round_bf16, int k,
                                                                  int32_t* __restrict__ out_all, int64_t out_stride,
                                                                  DiffArgs df) {
  LRQK_SEL_LDS(L);
  const int h = blockIdx.x;
  const int n = __builtin_amdgcn_readfirstlane(st.cand_count[h * kCountStride]);
  const int lvl = __builtin_amdgcn_readfirstlane(st.level[h]);
  const bool fast = n >= k && n <= cand_cap && n <= 16 * kSelThreads;
  int level = lvl & 0xff, calm = lvl >> 8;
  if (!fast) {
    level = 2;
    calm = 0;
  } else if (level > 0 && ++calm >= kCalmCalls) {
    --level;
    calm = 0;
  }
  if (fast) {
    if (threadIdx.x == 0) atomicAdd(&st.stats[0], 1);
    const uint2* cand = cand_all + (int64_t)h * cand_cap;
    const uint32_t lo = st.t_used[h];
    const int k2 = bound_rank(k, level, n);
    if (n <= 4 * kSelThreads)
      select_step_fast<4>(L, cand, n, lo, st, h, m, k, k2, df);
    else if (n <= 8 * kSelThreads)
      select_step_fast<8>(L, cand, n, lo, st, h, m, k, k2, df);
    else
      select_step_fast<16>(L, cand, n, lo, st, h, m, k, k2, df);
  } else {
    select_generic<T, R>(L, 0, cand_all, cand_cap, st, keys_all, key_stride, a_k, head_stride, q_hat, m, r, round_bf16, k,
                         out_all, out_stride, df, n, bound_rank(k, level, m));
  }
  // (both bodies hold barriers, so every thread has read the old value by now)
  if (threadIdx.x == 0) st.level[h] = level | (calm << 8);
}

// --------------------------------------------------------------------------- host side
template <typename T>
static int launch_scores(const void* a_k, int64_t head_stride, const void* q_hat, int bh, int64_t m, int r,
                         int round_bf16, uint32_t* keys, int64_t key_stride, float* scores, hipStream_t st) {
  const T* A = (const T*)a_k;
  const T* q = (const T*)q_hat;
  const int threads = 256;
  int64_t blocks = (m + threads - 1) / threads;
  if (blocks > 65535) blocks = 65535;
  dim3 grid((unsigned)blocks, (unsigned)bh);
  const bool vec_ok = ((uintptr_t)a_k % 16 == 0) && ((head_stride * sizeof(T)) % 16 == 0);
#define LRQK_SCORE_CASE(RR)                                                                              \
  hipLaunchKernelGGL((score_kernel<T, RR>), grid, dim3(threads), 0, st, A, head_stride, q, m, r, round_bf16, \
                     keys, key_stride, scores)
  if (vec_ok && r == 64) LRQK_SCORE_CASE(64);
  else if (vec_ok && r == 32) LRQK_SCORE_CASE(32);
  else if (vec_ok && r == 16) LRQK_SCORE_CASE(16);
  else if (vec_ok && r == 8) LRQK_SCORE_CASE(8);
  else LRQK_SCORE_CASE(0);
#undef LRQK_SCORE_CASE
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

static size_t select_smem(int k, bool with_diff) {
  return (size_t)2 * kChunkWords * sizeof(uint32_t) + (with_diff ? (size_t)k * 10 : 0);
}

struct SelectBufs {
  uint2* cand;
  int cand_cap;
  SelState st;
  uint32_t* keys;
  int64_t key_stride;
};

// Sizes the workspace of one selection.  The per-head state (t_low, counters) is
// re-initialised whenever the buffer is (re)allocated or the head count changes.
static int prepare_select(lrqk_ctx* ctx, int bh, int64_t m, int topk, hipStream_t st, SelectBufs* sb) {
  int rc;
  sb->key_stride = (m + 63) & ~(int64_t)63;
  if ((rc = ctx->keys.ensure((size_t)bh * sb->key_stride * 4))) return rc;
  sb->keys = (uint32_t*)ctx->keys.p;
  sb->cand_cap = 8 * topk < 4096 ? 4096 : 8 * topk;  // (the register-resident paths take up to 8192 and 16384 entries)
  if ((rc = ctx->cand.ensure((size_t)bh * sb->cand_cap * sizeof(uint2)))) return rc;
  sb->cand = (uint2*)ctx->cand.p;
  // layout: t_low u32 [bh] | q_norm f32 [bh] | t_used u32 [bh] | q_cur f32 [bh] | (unused) [bh] | level i32 [bh] |
  // stats i32 [3]: served from the list, rescans because the list was too short, because it overflowed |
  // rescored i32 [bh + kRescSlots] | cand_count i32 [bh * kCountStride] on a 128-byte boundary
  void* before = ctx->cand_cnt.p;
  constexpr int kRescSlots = 8192;  // workgroups of one index scan (never more than the GPU holds at a time)
  const size_t count_at = ((size_t)(6 * bh + 3 + bh + kRescSlots) + 31) & ~(size_t)31;  // (in words)
  if ((rc = ctx->cand_cnt.ensure((count_at + (size_t)bh * kCountStride) * 4))) return rc;
  uint32_t* base = (uint32_t*)ctx->cand_cnt.p;
  sb->st.t_low = base;
  sb->st.q_norm = (float*)(base + bh);
  sb->st.t_used = base + 2 * bh;
  sb->st.q_cur = (float*)(base + 3 * bh);
  sb->st.cand_count = (int*)(base + count_at);
  sb->st.level = (int*)(base + 5 * bh);
  sb->st.stats = (int*)(base + 6 * bh);
  sb->st.rescored = (int*)(base + 6 * bh + 3);
  sb->st.rescored_cap = bh + kRescSlots;
  if (before != ctx->cand_cnt.p || ctx->sel_bh != bh) {
    hipLaunchKernelGGL(init_select_state_kernel, dim3((unsigned)((bh + 255) / 256)), dim3(256), 0, st, sb->st, bh);
    LRQK_HIP_CHECK(hipGetLastError());
    ctx->sel_bh = bh;
  }
  return LRQK_OK;
}

template <typename T, int R>
static int launch_filter_select(lrqk_ctx* ctx, const SelectBufs& sb, const void* a_k, int64_t head_stride,
                                const void* q_hat, int bh, int64_t m, int r, int round_bf16, int topk, int32_t* out_idx,
                                int64_t out_stride, const DiffArgs& df, hipStream_t st, bool want_out = true) {
  size_t smem = select_smem(topk, df.hit != nullptr);
  // the decode step's select + diff (no ascending output): as long as its bitmaps fit the LDS beside the
  // generic path's blocks
  constexpr size_t kLdsStatic = (size_t)2 * kBins * 4 + 1024;
  const bool step_path = !want_out && df.hit != nullptr && !df.replace_all && m <= kChunkBits && topk <= kFusedDiffMaxK &&
                         std::max(smem, step_select_smem(m, topk)) + kLdsStatic <= (size_t)160 * 1024;
  if (step_path) {
    smem = std::max(smem, step_select_smem(m, topk));
    static std::atomic<size_t> step_allowed_dev[kMaxDeviceSlots];
    std::atomic<size_t>& step_allowed = step_allowed_dev[per_device_slot()];
    if (smem > step_allowed) {
      LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)select_step_kernel<T, R>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
      step_allowed = smem;
    }
  }
  static std::atomic<size_t> smem_allowed_dev[kMaxDeviceSlots];
  std::atomic<size_t>& smem_allowed = smem_allowed_dev[per_device_slot()];
  if (!step_path && smem > smem_allowed) {
    LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)select_kernel<T, R>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem));
    smem_allowed = smem;
  }
  const bool timed = ctx->tev && ctx->tev_used < ctx->tev_pairs && (ctx->tev_seen++ % ctx->tev_every) == 0;
  if (timed) LRQK_HIP_CHECK(hipEventRecord(ctx->tev[2 * ctx->tev_used], st));
  constexpr size_t filt_smem = (size_t)kFiltRows * kFiltTiles * sizeof(uint2);
  static std::atomic<bool> filt_attr_dev[kMaxDeviceSlots];
  std::atomic<bool>& filt_attr = filt_attr_dev[per_device_slot()];
  if (!filt_attr && filt_smem > 48 * 1024) {
    LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)score_filter_kernel<T, R>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)filt_smem));
    filt_attr = true;
  }
  // a finish stage of the factor update that is still pending: the filter reads the iterate itself
  FilterQ fq{nullptr, nullptr, 0, 0, 0.0f, nullptr};
  if (ctx->qhat_pending) {
    if (R > 0 && R <= 64 && ctx->fin.q_hat_out == q_hat && ctx->fin.r == r && ctx->fin.bh == bh &&
        ctx->fin.max_iter <= kFiltMaxIt) {
      fq = FilterQ{ctx->fin.iter_out, ctx->fin.deltas, bh, ctx->fin.max_iter, ctx->fin.tol, ctx->fin.q_hat_out};
      ctx->qhat_pending = false;
    } else {
      int rcf = flush_pending_finish(ctx, st);
      if (rcf) return rcf;
    }
  }
  dim3 grid((unsigned)((m + (int64_t)kFiltRows * kFiltTiles - 1) / ((int64_t)kFiltRows * kFiltTiles)), (unsigned)bh);
  bool via_index = false;
  if constexpr (R == 16 || R == 32 || R == 64) {
    ScoreIndexView six{};
    const int ri = score_index_prepare(ctx, a_k, head_stride, bh, m, r, sizeof(T) == 4 ? LRQK_F32 : LRQK_BF16, st, &six);
    if (ri < 0) return ri;
    if (ri == 1) {
      // As many workgroups as the GPU holds at a time, shared out over the heads: every wave then runs once, from
      // the first row to the last (a second round of workgroups would pay the solve for q' and the final
      // rescoring again, with the memory idle meanwhile).
      static std::atomic<int> slots_dev[kMaxDeviceSlots];
      std::atomic<int>& slots_a = slots_dev[per_device_slot()];
      int slots = slots_a;
      if (slots == 0) {
        int per_cu = 0, dev = 0, n_cu = 0;
        LRQK_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, score_prefilter_kernel<T, R>,
                                                                    kFiltThreads, 0));
        LRQK_HIP_CHECK(hipGetDevice(&dev));
        LRQK_HIP_CHECK(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev));
        slots = std::max(1, per_cu * n_cu);
        slots_a = slots;
      }
      constexpr int kStepRowsWg = (kWave / (R / 16)) * kScanU * kScanWaves;  // rows one step of a workgroup's waves covers
      const int64_t need = (m + kStepRowsWg - 1) / kStepRowsWg;
      const int64_t wgs = std::max<int64_t>(1, std::min<int64_t>(need, slots / bh));
      dim3 grid_st((unsigned)wgs, (unsigned)bh);
      hipLaunchKernelGGL((score_prefilter_kernel<T, R>), grid_st, dim3(kFiltThreads), 0, st, (const T*)a_k,
                         head_stride, (const T*)q_hat, m, r, round_bf16, sb.st, sb.cand, sb.cand_cap, fq, six);
      via_index = true;
      ctx->scan_wgs = (int)std::min<int64_t>((int64_t)grid_st.x * bh, sb.st.rescored_cap);
      ctx->scan_rows = (int64_t)bh * m;
    }
  }
  if (!via_index) ctx->scan_wgs = 0;
  if (!via_index)
    hipLaunchKernelGGL((score_filter_kernel<T, R>), grid, dim3(kFiltThreads), filt_smem, st, (const T*)a_k, head_stride,
                       (const T*)q_hat, m, r, round_bf16, sb.st, sb.cand, sb.cand_cap, fq);
  LRQK_HIP_CHECK(hipGetLastError());
  if (timed) {
    LRQK_HIP_CHECK(hipEventRecord(ctx->tev[2 * ctx->tev_used + 1], st));
    ++ctx->tev_used;
  }
  if (step_path)
    hipLaunchKernelGGL((select_step_kernel<T, R>), dim3((unsigned)bh), dim3(kSelThreads), smem, st, sb.cand, sb.cand_cap,
                       sb.st, sb.keys, sb.key_stride, (const T*)a_k, head_stride, (const T*)q_hat, m, r, round_bf16, topk,
                       out_idx, out_stride, df);
  else
    hipLaunchKernelGGL((select_kernel<T, R>), dim3((unsigned)bh), dim3(kSelThreads), smem, st, 0, sb.cand, sb.cand_cap,
                       sb.st, sb.keys, sb.key_stride, (const T*)a_k, head_stride, (const T*)q_hat, m, r, round_bf16, topk,
                       out_idx, out_stride, df);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

template <typename T>
static int dispatch_filter_select(lrqk_ctx* ctx, const SelectBufs& sb, const void* a_k, int64_t head_stride,
                                  const void* q_hat, int bh, int64_t m, int r, int round_bf16, int topk,
                                  int32_t* out_idx, int64_t out_stride, const DiffArgs& df, hipStream_t st,
                                  bool want_out = true) {
  const bool vec_ok = ((uintptr_t)a_k % 16 == 0) && ((head_stride * sizeof(T)) % 16 == 0);
#define LRQK_FS_CASE(RR)                                                                                            \
  return launch_filter_select<T, RR>(ctx, sb, a_k, head_stride, q_hat, bh, m, r, round_bf16, topk, out_idx, out_stride, \
                                     df, st, want_out)
  if (vec_ok && r == 64) LRQK_FS_CASE(64);
  if (vec_ok && r == 32) LRQK_FS_CASE(32);
  if (vec_ok && r == 16) LRQK_FS_CASE(16);
  if (vec_ok && r == 8) LRQK_FS_CASE(8);
  LRQK_FS_CASE(0);
#undef LRQK_FS_CASE
}

static int check_select_args(lrqk_ctx* ctx, int bh, int64_t m, int topk, const void* out_idx, int64_t out_stride) {
  LRQK_REQUIRE(ctx != nullptr, LRQK_EINVAL, "ctx is null");
  LRQK_REQUIRE(bh > 0 && bh <= 65535, LRQK_EINVAL, "bh=%d out of range", bh);
  LRQK_REQUIRE(m >= 0 && m < (int64_t)1 << 31, LRQK_EINVAL, "m=%lld out of range", (long long)m);
  LRQK_REQUIRE(topk > 0 && topk <= LRQK_MAX_TOPK, LRQK_ELIMIT, "topk=%d not in 1..%d", topk, LRQK_MAX_TOPK);
  LRQK_REQUIRE(out_idx != nullptr, LRQK_EINVAL, "out_idx is null");
  LRQK_REQUIRE(out_stride >= (m < topk ? m : topk), LRQK_EINVAL, "out_stride=%lld too small", (long long)out_stride);
  return LRQK_OK;
}

static int arange_result(int bh, int64_t m, int32_t* out_idx, int64_t out_stride, hipStream_t st) {
  if (m > 0) {
    hipLaunchKernelGGL(arange_kernel, dim3((unsigned)((m + 255) / 256), (unsigned)bh), dim3(256), 0, st, out_idx,
                       out_stride, (int)m);
    LRQK_HIP_CHECK(hipGetLastError());
  }
  return (int)m;
}

// Scan + select with the hit/miss diff fused into the select kernel (k <= kFusedDiffMaxK and
// m > k); used by the fused decode step.  Returns 1 if the diff was fused, 0 if the caller
// still has to run it, negative on error.
int score_select_diff(lrqk_ctx* ctx, const void* a_k, int64_t head_stride, const void* q_hat, int bh, int64_t m, int r,
                      int topk, int dtype, int round_bf16, int32_t* new_idx, int32_t* hit, int64_t hit_stride,
                      uint8_t* evict, int32_t* miss_slots, int32_t* miss_count, int replace_all, hipStream_t st,
                      int32_t* miss_old, const VictimView* vic, int32_t* miss_new, bool want_new_idx) {
  int rc = check_select_args(ctx, bh, m, topk, new_idx, topk);
  if (rc) return rc;
  if (m <= topk || topk > kFusedDiffMaxK) {
    rc = lrqk_score_select(ctx, a_k, head_stride, q_hat, bh, m, r, topk, dtype, round_bf16, new_idx, topk, st);
    return rc < 0 ? rc : 0;
  }
  SelectBufs sb;
  if ((rc = prepare_select(ctx, bh, m, topk, st, &sb))) return rc;
  DiffArgs df{hit, hit_stride, evict, miss_slots, miss_count, replace_all, miss_old, miss_new,
              vic && vic->nv > 0 ? vic->ptr : nullptr, vic && vic->nv > 0 ? vic->base : nullptr, vic ? vic->nv : 0};
  if (dtype == LRQK_F32)
    rc = dispatch_filter_select<float>(ctx, sb, a_k, head_stride, q_hat, bh, m, r, 0, topk, new_idx, topk, df, st,
                                       want_new_idx);
  else
    rc = dispatch_filter_select<bf16_t>(ctx, sb, a_k, head_stride, q_hat, bh, m, r, round_bf16, topk, new_idx, topk, df,
                                        st, want_new_idx);
  return rc ? rc : 1;
}

}  // namespace lrqk

using namespace lrqk;

extern "C" int lrqk_proxy_scores(const void* a_k, int64_t head_stride, const void* q_hat, int bh, int64_t m, int r,
                                 int dtype, int round_bf16, float* out_scores, void* stream) {
  LRQK_REQUIRE(a_k && q_hat && out_scores, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(dtype == LRQK_F32 || dtype == LRQK_BF16, LRQK_EINVAL, "dtype=%d", dtype);
  LRQK_REQUIRE(bh > 0 && bh <= 65535 && m >= 0 && r > 0 && r <= LRQK_MAX_R, LRQK_EINVAL, "bad sizes bh=%d m=%lld r=%d", bh,
               (long long)m, r);
  LRQK_REQUIRE(head_stride >= m * r, LRQK_EINVAL, "head_stride=%lld < m*r", (long long)head_stride);
  if (m == 0) return LRQK_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == LRQK_F32)
    return launch_scores<float>(a_k, head_stride, q_hat, bh, m, r, 0, nullptr, 0, out_scores, st);
  return launch_scores<bf16_t>(a_k, head_stride, q_hat, bh, m, r, round_bf16, nullptr, 0, out_scores, st);
}

extern "C" int lrqk_score_select(lrqk_ctx* ctx, const void* a_k, int64_t head_stride, const void* q_hat, int bh,
                                 int64_t m, int r, int topk, int dtype, int round_bf16, int32_t* out_idx,
                                 int64_t out_stride, void* stream) {
  int rc = check_select_args(ctx, bh, m, topk, out_idx, out_stride);
  if (rc) return rc;
  LRQK_REQUIRE(a_k && q_hat, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(dtype == LRQK_F32 || dtype == LRQK_BF16, LRQK_EINVAL, "dtype=%d", dtype);
  LRQK_REQUIRE(r > 0 && r <= LRQK_MAX_R, LRQK_EINVAL, "r=%d", r);
  LRQK_REQUIRE(head_stride >= m * r, LRQK_EINVAL, "head_stride=%lld < m*r", (long long)head_stride);
  hipStream_t st = (hipStream_t)stream;
  if (m <= topk) return arange_result(bh, m, out_idx, out_stride, st);
  SelectBufs sb;
  if ((rc = prepare_select(ctx, bh, m, topk, st, &sb))) return rc;
  DiffArgs df{nullptr, 0, nullptr, nullptr, nullptr, 0, nullptr, nullptr, nullptr, nullptr, 0};
  if (dtype == LRQK_F32)
    rc = dispatch_filter_select<float>(ctx, sb, a_k, head_stride, q_hat, bh, m, r, 0, topk, out_idx, out_stride, df, st);
  else
    rc = dispatch_filter_select<bf16_t>(ctx, sb, a_k, head_stride, q_hat, bh, m, r, round_bf16, topk, out_idx,
                                        out_stride, df, st);
  return rc ? rc : topk;
}

extern "C" int lrqk_score_select_diff(lrqk_ctx* ctx, const void* a_k, int64_t head_stride, const void* q_hat, int bh,
                                      int64_t m, int r, int topk, int dtype, int round_bf16, int32_t* new_idx,
                                      int32_t* hit, int64_t hit_stride, uint8_t* evict, int32_t* miss_slots,
                                      int32_t* miss_count, void* stream) {
  LRQK_REQUIRE(ctx && a_k && q_hat && hit && miss_slots && miss_count, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(dtype == LRQK_F32 || dtype == LRQK_BF16, LRQK_EINVAL, "dtype=%d", dtype);
  LRQK_REQUIRE(r > 0 && r <= LRQK_MAX_R, LRQK_EINVAL, "r=%d", r);
  LRQK_REQUIRE(bh > 0 && bh <= 65535, LRQK_EINVAL, "bh=%d out of range", bh);
  LRQK_REQUIRE(topk > 0 && topk <= LRQK_MAX_TOPK, LRQK_ELIMIT, "topk=%d not in 1..%d", topk, LRQK_MAX_TOPK);
  const bool want_new = new_idx != nullptr;
  if (!want_new) {  // the caller only wants what changes: the selection is never put in order
    int rce = ctx->new_idx.ensure((size_t)bh * topk * sizeof(int32_t));
    if (rce) return rce;
    new_idx = (int32_t*)ctx->new_idx.p;
  }
  // (m == topk is the first step after the growing-prefix branch, py:1560-1562: every row is selected)
  LRQK_REQUIRE(m >= topk, LRQK_EINVAL, "m=%lld is below topk=%d (no diff happens in the prefix branch)",
               (long long)m, topk);
  LRQK_REQUIRE(head_stride >= m * r && hit_stride >= topk, LRQK_EINVAL, "stride too small");
  int rc = score_select_diff(ctx, a_k, head_stride, q_hat, bh, m, r, topk, dtype, round_bf16, new_idx, hit, hit_stride,
                             evict, miss_slots, miss_count, 0, (hipStream_t)stream, nullptr, nullptr, nullptr, want_new);
  if (rc < 0) return rc;
  if (rc == 0) return lrqk_diff(new_idx, topk, hit, hit_stride, bh, topk, evict, miss_slots, miss_count, stream);
  return LRQK_OK;
}

extern "C" int lrqk_select_from_scores(lrqk_ctx* ctx, const float* scores, int bh, int64_t m, int topk,
                                       int32_t* out_idx, int64_t out_stride, void* stream) {
  int rc = check_select_args(ctx, bh, m, topk, out_idx, out_stride);
  if (rc) return rc;
  LRQK_REQUIRE(scores != nullptr, LRQK_EINVAL, "scores is null");
  hipStream_t st = (hipStream_t)stream;
  if (m <= topk) return arange_result(bh, m, out_idx, out_stride, st);
  SelectBufs sb;
  if ((rc = prepare_select(ctx, bh, m, topk, st, &sb))) return rc;
  int64_t blocks = (m + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  hipLaunchKernelGGL(keys_from_scores_kernel, dim3((unsigned)blocks, (unsigned)bh), dim3(256), 0, st, scores, m, sb.keys,
                     sb.key_stride);
  LRQK_HIP_CHECK(hipGetLastError());
  const size_t smem = select_smem(topk, false);
  static std::atomic<bool> attr_done_dev[kMaxDeviceSlots];
  std::atomic<bool>& attr_done = attr_done_dev[per_device_slot()];
  if (!attr_done) {
    LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)select_kernel<float, 0>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem));
    attr_done = true;
  }
  DiffArgs df{nullptr, 0, nullptr, nullptr, nullptr, 0, nullptr, nullptr, nullptr, nullptr, 0};
  hipLaunchKernelGGL((select_kernel<float, 0>), dim3((unsigned)bh), dim3(kSelThreads), smem, st, 1, sb.cand, sb.cand_cap,
                     sb.st, sb.keys, sb.key_stride, (const float*)nullptr, (int64_t)0, (const float*)nullptr, m, 1, 0,
                     topk, out_idx, out_stride, df);
  LRQK_HIP_CHECK(hipGetLastError());
  return topk;
}

extern "C" int lrqk_scan_stats(lrqk_ctx* ctx, int64_t* rows_scanned, int64_t* rows_rescored) {
  LRQK_REQUIRE(ctx && rows_scanned && rows_rescored, LRQK_EINVAL, "null pointer");
  *rows_scanned = *rows_rescored = 0;
  if (!ctx->cand_cnt.p || ctx->sel_bh <= 0 || ctx->scan_wgs <= 0) return LRQK_OK;
  std::vector<int> v((size_t)ctx->scan_wgs);
  // the counters belong to the last scan, which may still be running on a stream that does not wait for the
  // null stream's copy
  LRQK_HIP_CHECK(hipDeviceSynchronize());
  LRQK_HIP_CHECK(hipMemcpy(v.data(), (int*)ctx->cand_cnt.p + 6 * ctx->sel_bh + 3, v.size() * sizeof(int),
                           hipMemcpyDeviceToHost));
  int64_t t = 0;
  for (int x : v) t += x;
  *rows_scanned = ctx->scan_rows;
  *rows_rescored = t;
  return LRQK_OK;
}

extern "C" int lrqk_select_stats(lrqk_ctx* ctx, int* fast_heads, int* full_heads, int reset) {
  LRQK_REQUIRE(ctx && fast_heads && full_heads, LRQK_EINVAL, "null pointer");
  *fast_heads = *full_heads = 0;
  if (!ctx->cand_cnt.p || ctx->sel_bh <= 0) return LRQK_OK;
  int* stats = (int*)ctx->cand_cnt.p + 6 * ctx->sel_bh;
  int v[3];
  LRQK_HIP_CHECK(hipDeviceSynchronize());
  LRQK_HIP_CHECK(hipMemcpy(v, stats, sizeof(v), hipMemcpyDeviceToHost));
  *fast_heads = v[0];
  *full_heads = v[1] + v[2];
  ctx->last_short = v[1];
  ctx->last_overflow = v[2];
  if (reset) LRQK_HIP_CHECK(hipMemset(stats, 0, sizeof(v)));
  return LRQK_OK;
}

