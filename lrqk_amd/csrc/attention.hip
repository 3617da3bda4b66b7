// Exact single-query attention over the active set: softmax(q K^T / sqrt(d)) V, split
// along the slot axis so that one head fills many CUs, then a per-head combine of the
// partial (max, sum, accumulator) triples.  (A device-scope fence per workgroup, which a
// single-launch "last arrival combines" scheme needs, costs more than the second launch:
// the L2 is per XCD.)
//
// Inside the decode step the partial pass shares its launch with the miss fetch: the
// workgroups that copy the missed rows from the host store are bound by the host link,
// the others meanwhile run the attention over the slots that stay resident; the combine
// kernel then adds the freshly fetched slots of its head before merging.
#include <math.h>

#include <mutex>

#include "common.hpp"
#include "ctx.hpp"
#include "rows.hpp"
#include "als_finish.hpp"
#include "victim.hpp"

namespace lrqk {

constexpr int kAttnThreads = 256;          // partial pass
constexpr int kAttnWaves = kAttnThreads / kWave;
constexpr int kCombThreads = 1024;         // combine: wide enough to take a head's refetched rows in one pass

// Online-softmax state of one lane group: running max, sum and the accumulator slice.
template <int VEC>
struct AttnAcc {
  float m, l;
  float acc[VEC];
  __device__ __forceinline__ void init() {
    m = -INFINITY;
    l = 0.0f;
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = 0.0f;
  }
};

// Items begin..end-1 of a sequence; row_of(i, valid) gives the slot row of item i (always a
// readable row; `valid` says whether it counts).  Each K/V row of d elements is read as
// d*sizeof(T)/16 chunks by `lpr` adjacent lanes, so a wave covers 64/lpr rows per load
// instruction with fully coalesced 16-byte accesses; U row groups per pass have their loads
// issued together (one memory latency), unconditionally, and are masked afterwards.
template <typename T, int NW, int U, typename RowOf>
__device__ __forceinline__ void attn_scan(const float* qf, const T* __restrict__ Kh, const T* __restrict__ Vh, int d,
                                          int lpr_log2, int begin, int end, RowOf row_of,
                                          AttnAcc<Vec16<T>::N>& st) {
  constexpr int VEC = Vec16<T>::N;
  const int lane = lane_id(), wave = wave_id();
  const int lpr = 1 << lpr_log2;
  const int sub = lane & (lpr - 1);
  const int grp = lane >> lpr_log2;
  const int gpw = kWave >> lpr_log2;  // row groups per wave
  const int rows_per_iter = gpw * NW;
  for (int base = begin; base < end; base += U * rows_per_iter) {
    Vec16<T> kv[U], vv[U];
    bool ok[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = base + u * rows_per_iter + wave * gpw + grp;
      bool valid;
      const int rr = row_of(min(i, end - 1), valid);
      ok[u] = valid && i < end;
      kv[u].load(Kh + (int64_t)rr * d + sub * VEC);
      vv[u].load(Vh + (int64_t)rr * d + sub * VEC);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float kf[VEC], vf[VEC];
      kv[u].unpack(kf);
      vv[u].unpack(vf);
      float sc = 0.0f;
#pragma unroll
      for (int e = 0; e < VEC; ++e) sc = fmaf(kf[e], qf[e], sc);
      sc = group_sum(sc, lpr);
      if (!ok[u]) sc = -INFINITY;
      const float m_new = fmaxf(st.m, sc);
      // exp2 of (-inf) - (-inf) must not produce NaN: while nothing valid was seen keep zeros
      const float alpha = (m_new == -INFINITY) ? 0.0f : exp2f(st.m - m_new);
      const float p = (m_new == -INFINITY) ? 0.0f : exp2f(sc - m_new);
      st.l = st.l * alpha + p;
#pragma unroll
      for (int e = 0; e < VEC; ++e) st.acc[e] = st.acc[e] * alpha + p * vf[e];
      st.m = m_new;
    }
  }
}

// The same pass when the products K q of the rows are already known (`w`, one float per slot, unscaled):
// only the V rows are read.
template <typename T, int NW, int U, typename RowOf>
__device__ __forceinline__ void attn_scan_w(const float* __restrict__ w, float scale_log2e, const T* __restrict__ Vh,
                                            int d, int lpr_log2, int begin, int end, RowOf row_of,
                                            AttnAcc<Vec16<T>::N>& st) {
  constexpr int VEC = Vec16<T>::N;
  const int lane = lane_id(), wave = wave_id();
  const int lpr = 1 << lpr_log2;
  const int sub = lane & (lpr - 1);
  const int grp = lane >> lpr_log2;
  const int gpw = kWave >> lpr_log2;
  const int rows_per_iter = gpw * NW;
  for (int base = begin; base < end; base += U * rows_per_iter) {
    Vec16<T> vv[U];
    float wl[U];
    bool ok[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = base + u * rows_per_iter + wave * gpw + grp;
      bool valid;
      const int rr = row_of(min(i, end - 1), valid);
      ok[u] = valid && i < end;
      wl[u] = w[rr];
      vv[u].load(Vh + (int64_t)rr * d + sub * VEC);
    }
    // (the products are only used for rows that count; without this the compiler moves each of their loads into
    // that condition, where it becomes a branch with a full wait per row group)
#pragma unroll
    for (int u = 0; u < U; ++u) asm volatile("" : "+v"(wl[u]));
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float vf[VEC];
      vv[u].unpack(vf);
      const float sc = ok[u] ? wl[u] * scale_log2e : -INFINITY;
      const float m_new = fmaxf(st.m, sc);
      const float alpha = (m_new == -INFINITY) ? 0.0f : exp2f(st.m - m_new);
      const float p = (m_new == -INFINITY) ? 0.0f : exp2f(sc - m_new);
      st.l = st.l * alpha + p;
#pragma unroll
      for (int e = 0; e < VEC; ++e) st.acc[e] = st.acc[e] * alpha + p * vf[e];
      st.m = m_new;
    }
  }
}

// Merges the lane groups of a wave, then the waves of the workgroup, and writes the workgroup's (m, l, acc[d])
// triple to pout[0 .. d + 2): thread t writes element t, and the first threads also the elements beyond the
// workgroup's thread count (d + 2 exceeds it for rows of 256 elements).
// red: [NW][2 + 256] floats of LDS.
template <int VEC, int NW>
__device__ __forceinline__ void attn_block_merge(AttnAcc<VEC>& st, int lpr_log2, int d, float (*red)[2 + 256],
                                                 float* __restrict__ pout) {
  const int lane = lane_id(), wave = wave_id();
  const int lpr = 1 << lpr_log2;
  const int sub = lane & (lpr - 1);
  const int grp = lane >> lpr_log2;
  for (int off = lpr; off < kWave; off <<= 1) {
    const float m_o = __shfl_xor(st.m, off, kWave);
    const float l_o = __shfl_xor(st.l, off, kWave);
    const float m_new = fmaxf(st.m, m_o);
    const float a = (m_new == -INFINITY) ? 0.0f : exp2f(st.m - m_new);
    const float b = (m_new == -INFINITY) ? 0.0f : exp2f(m_o - m_new);
    st.l = st.l * a + l_o * b;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float o = __shfl_xor(st.acc[e], off, kWave);
      st.acc[e] = st.acc[e] * a + o * b;
    }
    st.m = m_new;
  }
  if (grp == 0) {
    if (sub == 0) {
      red[wave][0] = st.m;
      red[wave][1] = st.l;
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) red[wave][2 + sub * VEC + e] = st.acc[e];
  }
  __syncthreads();
  float M = -INFINITY;
#pragma unroll
  for (int w = 0; w < NW; ++w) M = fmaxf(M, red[w][0]);
  float f[NW];
#pragma unroll
  for (int w = 0; w < NW; ++w) f[w] = (M == -INFINITY) ? 0.0f : exp2f(red[w][0] - M);
  const int c = threadIdx.x;
  if (c < d + 2) {
    float v = 0.0f;
#pragma unroll
    for (int w = 0; w < NW; ++w) v += red[w][c] * f[w];
    pout[c] = c == 0 ? M : v;
  }
  const int c2 = c + NW * kWave;
  if (c2 < d + 2) {  // (rows of 256 elements only)
    float v = 0.0f;
#pragma unroll
    for (int w = 0; w < NW; ++w) v += red[w][c2] * f[w];
    pout[c2] = v;
  }
}

template <typename T>
__device__ __forceinline__ void load_query(const T* q, int h, int d, int lpr_log2, float scale_log2e, float* qf) {
  constexpr int VEC = Vec16<T>::N;
  const int sub = lane_id() & ((1 << lpr_log2) - 1);
  Vec16<T> qv;
  qv.load(q + (int64_t)h * d + sub * VEC);
  qv.unpack(qf);
#pragma unroll
  for (int e = 0; e < VEC; ++e) qf[e] *= scale_log2e;
}

// Partial layout per (head, split): [m, l, acc[d]] fp32; `stride_s` triples per head.
// skip (optional): u8 [bh][k_skip], slots s < k_skip with skip != 0 are left out.
template <typename T, int U = 4>
__device__ __forceinline__ void attn_partial_body(const T* __restrict__ q, const T* __restrict__ K,
                                                  const T* __restrict__ V, int n_slots, int n_valid, int d,
                                                  int lpr_log2, float scale_log2e, float* __restrict__ part, int S,
                                                  int stride_s, const uint8_t* __restrict__ skip, int k_skip, int h,
                                                  int s, const float* __restrict__ w = nullptr) {
  constexpr int VEC = Vec16<T>::N;
  __shared__ float red[kAttnWaves][2 + 256];
  const int rows_per_split = (n_valid + S - 1) / S;
  const int r0 = s * rows_per_split;
  const int r1 = min(n_valid, r0 + rows_per_split);
  float qf[VEC];
  load_query<T>(q, h, d, lpr_log2, scale_log2e, qf);
  const T* Kh = K + (int64_t)h * n_slots * d;
  const T* Vh = V + (int64_t)h * n_slots * d;
  AttnAcc<VEC> st;
  st.init();
  if (skip && w) {
    // (decode step) the factor update's first kernel left K q of every slot, as the slots were before this
    // step's misses; the slots that are being replaced are skipped here anyway
    const uint8_t* sk = skip + (int64_t)h * k_skip;
    attn_scan_w<T, kAttnWaves, U>(w + (int64_t)h * n_slots, scale_log2e, Vh, d, lpr_log2, r0, r1, [&](int i, bool& valid) {
      valid = sk[min(i, k_skip - 1)] == 0 || i >= k_skip;
      return i;
    }, st);
  } else if (skip) {
    const uint8_t* sk = skip + (int64_t)h * k_skip;
    attn_scan<T, kAttnWaves, U>(qf, Kh, Vh, d, lpr_log2, r0, r1, [&](int i, bool& valid) {
      valid = sk[min(i, k_skip - 1)] == 0 || i >= k_skip;
      return i;
    }, st);
  } else {
    attn_scan<T, kAttnWaves, U>(qf, Kh, Vh, d, lpr_log2, r0, r1, [&](int i, bool& valid) {
      valid = true;
      return i;
    }, st);
  }
  attn_block_merge<VEC, kAttnWaves>(st, lpr_log2, d, red, part + ((int64_t)h * stride_s + s) * (d + 2));
}

template <typename T>
__global__ __launch_bounds__(kAttnThreads) void attn_partial_kernel(const T* __restrict__ q, const T* __restrict__ K,
                                                                    const T* __restrict__ V, int n_slots, int n_valid,
                                                                    int d, int lpr_log2, float scale_log2e,
                                                                    float* __restrict__ part, int S) {
  attn_partial_body<T>(q, K, V, n_slots, n_valid, d, lpr_log2, scale_log2e, part, S, S, nullptr, 0, blockIdx.y,
                       blockIdx.x);
}

// Fetch role of the decode step: like fetch_rows_body, and while a missed [K|V] row passes through
// the registers of its 2*cpr lanes (cpr K chunks, then cpr V chunks) the lanes also form the row's
// attention term, so the refetched slots never have to be read again.  The workgroup's rows are
// merged into one (max, sum, acc) triple at `pout` (an empty triple if it had no row).
template <typename T>
__device__ __forceinline__ void fetch_rows_attn_body(const uint4* __restrict__ store, int64_t cap,
                                                     uint4* __restrict__ k_act, uint4* __restrict__ v_act, int n_slots,
                                                     const int32_t* __restrict__ hit, int64_t hit_stride,
                                                     const int32_t* __restrict__ miss_slots,
                                                     const int32_t* __restrict__ miss_count, int hq, int hkv, int cpr,
                                                     int k, int h, int blk, int nblk, const T* __restrict__ q, int d,
                                                     float scale_log2e, float* __restrict__ pout,
                                                     const int32_t* __restrict__ miss_old, const VictimView& vic,
                                                     const int32_t* __restrict__ miss_new, uint4* __restrict__ evk,
                                                     int evk_rows) {
  constexpr int VEC = Vec16<T>::N;
  __shared__ float accs[8][256 + 2];               // [row group][m, l, acc[d]] (at most 8 groups are merged at a time)
  const int tid = threadIdx.x, lane = lane_id();
  const int cnt = miss_count[h];
  const int chunks = 2 * cpr;  // per store row; a power of two <= 64 here
  const int rpb = kAttnThreads / chunks;
  const int b = h / hq, head = h % hq;
  const int kvh = head / (hq / hkv);
  const int jl = tid / chunks, c = tid % chunks;
  const bool is_k = c < cpr;
  float qf[VEC];
  {
    Vec16<T> qv;
    qv.load(q + (int64_t)h * d + (is_k ? c : 0) * VEC);
    qv.unpack(qf);
#pragma unroll
    for (int e = 0; e < VEC; ++e) qf[e] *= scale_log2e;
  }
  AttnAcc<VEC> st;  // meaningful in the V lanes
  st.init();
  const int nv = vic.nv;  // uniform
  const int vbase = nv > 0 ? vic.base[h] : 0;
  // Every load is unconditional (clamped index, valid address) so that the loads of one stage go out
  // together: j -> (slot, token, previous token) -> FIFO positions -> row (+ FIFO tags) -> stores.
  // A lane group handles kFR rows per trip, stage by stage, so that one trip covers the usual number of misses.
  constexpr int kFR = 2;
  const int per_trip = kFR * nblk * rpb;
  for (int it = 0;; ++it) {
    int j[kFR], slot[kFR];
    int32_t tok[kFR], old[kFR];
#pragma unroll
    for (int u = 0; u < kFR; ++u) {
      j[u] = blk * rpb + jl + (it * kFR + u) * nblk * rpb;
      const int jc = min(j[u], k - 1);
      slot[u] = miss_slots[(int64_t)h * k + jc];
      tok[u] = miss_new ? miss_new[(int64_t)h * k + jc] : 0;
      old[u] = nv > 0 ? miss_old[(int64_t)h * k + jc] : -1;
    }
    const int trips = (cnt + per_trip - 1) / per_trip;  // uniform over the workgroup (first use of cnt)
    if (it >= trips) break;
    bool ok[kFR];
    int64_t dst[kFR];
    const uint4* host_src[kFR];
    const uint4* own[kFR];
#pragma unroll
    for (int u = 0; u < kFR; ++u) {
      ok[u] = j[u] < cnt && slot[u] >= 0 && slot[u] < k;
      slot[u] = ok[u] ? slot[u] : 0;
    }
    if (!miss_new) {
#pragma unroll
      for (int u = 0; u < kFR; ++u) tok[u] = hit[(int64_t)h * hit_stride + slot[u]];
    }
#pragma unroll
    for (int u = 0; u < kFR; ++u) {
      ok[u] = ok[u] && tok[u] >= 0 && tok[u] < cap;
      tok[u] = ok[u] ? tok[u] : 0;
      dst[u] = ((int64_t)h * n_slots + slot[u]) * cpr;
      host_src[u] = store + (((int64_t)b * hkv + kvh) * cap + tok[u]) * chunks + c;
      // a lane without a row reads a device address (its own slot), never the host store
      own[u] = is_k ? k_act + dst[u] + c : v_act + dst[u] + (c - cpr);
    }
    uint4 val[kFR];
    if (nv > 0) {
      // Victim cache.  The row that leaves the slot goes to FIFO position base + j (unless the
      // cache still holds it); the row that enters is taken from the FIFO if it is there and
      // not being replaced in this very step.  All reads of the metadata come before the writes,
      // and a row's lanes share one wave, so they decide alike.
      const int n_ins = min(cnt, nv);
      int p_ins[kFR], q_old[kFR], p_new[kFR];
      bool do_ins[kFR], old_cached[kFR], from_fifo[kFR];
#pragma unroll
      for (int u = 0; u < kFR; ++u) {
        p_ins[u] = (vbase + min(j[u], k - 1)) % nv;
        do_ins[u] = ok[u] && j[u] < nv && old[u] >= 0 && old[u] < vic.cap;
        q_old[u] = vic.pos[(int64_t)h * vic.cap + (do_ins[u] ? old[u] : 0)];
        p_new[u] = vic.pos[(int64_t)h * vic.cap + (tok[u] < vic.cap ? tok[u] : 0)];
      }
      uint4 old_val[kFR];
      int32_t tag_new[kFR], tag_old[kFR], prev[kFR];
#pragma unroll
      for (int u = 0; u < kFR; ++u) {
        old_cached[u] = do_ins[u] && q_old[u] >= 0 && q_old[u] < nv && !victim_slot_in_flight(q_old[u], vbase, n_ins, nv);
        from_fifo[u] = ok[u] && tok[u] < vic.cap && p_new[u] >= 0 && p_new[u] < nv &&
                       !victim_slot_in_flight(p_new[u], vbase, n_ins, nv);
        // the row is requested from where the position table points; the tags confirm it afterwards
        const uint4* src = from_fifo[u] ? vic.rows + ((int64_t)h * nv + p_new[u]) * chunks + c : (ok[u] ? host_src[u] : own[u]);
        val[u] = *src;
        old_val[u] = *own[u];
        tag_new[u] = vic.tok[(int64_t)h * nv + (from_fifo[u] ? p_new[u] : 0)];
        tag_old[u] = vic.tok[(int64_t)h * nv + (old_cached[u] ? q_old[u] : 0)];
        prev[u] = vic.tok[(int64_t)h * nv + p_ins[u]];
      }
      int prev_pos[kFR];
#pragma unroll
      for (int u = 0; u < kFR; ++u) {
        if (old_cached[u] && tag_old[u] == old[u]) do_ins[u] = false;
        if (from_fifo[u] && tag_new[u] != tok[u]) {  // (the table and the tags disagree: take the row from the store)
          from_fifo[u] = false;
          val[u] = *host_src[u];
        }
        prev_pos[u] = -1;
        if (do_ins[u] && prev[u] >= 0 && prev[u] < vic.cap) prev_pos[u] = vic.pos[(int64_t)h * vic.cap + prev[u]];
      }
#pragma unroll
      for (int u = 0; u < kFR; ++u) {
        if (do_ins[u]) {
          vic.rows[((int64_t)h * nv + p_ins[u]) * chunks + c] = old_val[u];
          if (c == 0) {
            if (prev_pos[u] == p_ins[u]) vic.pos[(int64_t)h * vic.cap + prev[u]] = -1;
            vic.tok[(int64_t)h * nv + p_ins[u]] = old[u];
            vic.pos[(int64_t)h * vic.cap + old[u]] = (int16_t)p_ins[u];
          }
        }
      }
      {  // statistics: rows taken from the host store (one addition per wave: additions to one line are served in turn)
        int n_host = 0;
#pragma unroll
        for (int u = 0; u < kFR; ++u) n_host += __popcll(__ballot(ok[u] && c == 0 && !from_fifo[u]));
        if (n_host && lane_id() == 0) atomicAdd(&vic.host_rows[h], n_host);
      }
      // the K rows that leave their slots, in the order of the miss list, for the kept sums of the factor update
      if (evk) {
#pragma unroll
        for (int u = 0; u < kFR; ++u)
          if (ok[u] && is_k && j[u] < evk_rows) evk[((int64_t)h * evk_rows + j[u]) * cpr + c] = old_val[u];
      }
    } else {
      uint4 old_val[kFR];
      if (evk) {  // (uniform)
#pragma unroll
        for (int u = 0; u < kFR; ++u) old_val[u] = *own[u];
      }
#pragma unroll
      for (int u = 0; u < kFR; ++u) val[u] = *(ok[u] ? host_src[u] : own[u]);
      if (evk) {
#pragma unroll
        for (int u = 0; u < kFR; ++u)
          if (ok[u] && is_k && j[u] < evk_rows) evk[((int64_t)h * evk_rows + j[u]) * cpr + c] = old_val[u];
      }
    }
#pragma unroll
    for (int u = 0; u < kFR; ++u) {
      if (ok[u]) {
        if (is_k) k_act[dst[u] + c] = val[u]; else v_act[dst[u] + (c - cpr)] = val[u];
      } else {
        val[u] = make_uint4(0, 0, 0, 0);
      }
      Vec16<T> vv;
      vv.raw = *reinterpret_cast<decltype(vv.raw)*>(&val[u]);
      float f[VEC];
      vv.unpack(f);
      float sc = 0.0f;
      if (is_k) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) sc = fmaf(f[e], qf[e], sc);
      }
      sc = group_sum(sc, cpr);  // K lanes: the row's score
      const float s_row = __shfl(sc, (lane & ~(chunks - 1)) | 0, kWave);           // first K lane of this row
      if (!is_k) {
        const float s_use = ok[u] ? s_row : -INFINITY;
        const float m_new = fmaxf(st.m, s_use);
        const float alpha = (m_new == -INFINITY) ? 0.0f : exp2f(st.m - m_new);
        const float p = (m_new == -INFINITY) ? 0.0f : exp2f(s_use - m_new);
        st.l = st.l * alpha + p;
#pragma unroll
        for (int e = 0; e < VEC; ++e) st.acc[e] = st.acc[e] * alpha + p * f[e];
        st.m = m_new;
      }
    }
  }
  // merge the row groups: V lane (jl, cv) owns columns cv*VEC .. of group jl
  const int groups = rpb;  // <= 8 for rows of >= 512 bytes; larger counts are merged in rounds of 8
  float M = -INFINITY, Lsum = 0.0f, col = 0.0f;  // thread t < d + 2 accumulates element t of the result
  for (int g0 = 0; g0 < groups; g0 += 8) {
    __syncthreads();
    if (!is_k && jl >= g0 && jl < g0 + 8 && jl < groups) {
      float* row = accs[jl - g0];
      if (c == cpr) {
        row[0] = st.m;
        row[1] = st.l;
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) row[2 + (c - cpr) * VEC + e] = st.acc[e];
    }
    __syncthreads();
    const int ng = min(8, groups - g0);
    float Mg = M;
    for (int g = 0; g < ng; ++g) Mg = fmaxf(Mg, accs[g][0]);
    const float a_old = (Mg == -INFINITY) ? 0.0f : exp2f(M - Mg);
    Lsum *= a_old;
    col *= a_old;
    for (int g = 0; g < ng; ++g) {
      const float fg = (Mg == -INFINITY || accs[g][0] == -INFINITY) ? 0.0f : exp2f(accs[g][0] - Mg);
      Lsum = fmaf(accs[g][1], fg, Lsum);
      if (tid >= 2 && tid < d + 2) col = fmaf(accs[g][tid], fg, col);
    }
    M = Mg;
  }
  if (tid < d + 2) pout[tid] = tid == 0 ? M : (tid == 1 ? Lsum : col);
  // Rows of 256 elements have two elements more than the workgroup has threads.  Such rows fill a wave, so the
  // workgroup has four row groups and the loop above made one round: the groups' triples are still in place.
  // (A second accumulator inside that loop cost the kernel 54 registers and half of its occupancy.)
  if (d + 2 > kAttnThreads && tid < d + 2 - kAttnThreads) {
    float c2 = 0.0f;
    for (int g = 0; g < groups; ++g) {
      const float fg = (M == -INFINITY || accs[g][0] == -INFINITY) ? 0.0f : exp2f(accs[g][0] - M);
      c2 = fmaf(accs[g][tid + kAttnThreads], fg, c2);
    }
    pout[tid + kAttnThreads] = c2;
  }
}

// Decode step: workgroups x < n_fetch copy this head's missed rows from the store into their
// slots; the next S run the partial attention over the slots that are not being replaced; one
// more (with_finish) runs the finish stage of this step's factor update, which nothing in this
// launch depends on, and after it one that encodes the appended row for the score index (if there
// is one).  The copy is bound by the host link, so the other roles ride along.
template <typename T>
__global__ __launch_bounds__(kAttnThreads, 4) void fetch_attn_partial_kernel(
    const uint4* __restrict__ store, int64_t cap, int32_t* __restrict__ hit, int64_t hit_stride,
    const int32_t* __restrict__ miss_slots, const int32_t* __restrict__ miss_count, const uint8_t* __restrict__ evict,
    int hq, int hkv, int cpr, int k, int n_fetch, const T* __restrict__ q, T* __restrict__ K, T* __restrict__ V,
    int n_slots, int d, int lpr_log2, float scale_log2e, float* __restrict__ part, int S, int with_finish,
    FinishArgs fa, const int32_t* __restrict__ miss_old, VictimView vic, const int32_t* __restrict__ miss_new,
    const float* __restrict__ kq, uint4* __restrict__ evk, int evk_rows, int32_t* __restrict__ count_copy) {
  const int h = blockIdx.y;
  // (the caller's copy of the miss counts, when the kernels keep them in the library's own block)
  if (count_copy && blockIdx.x == 0 && threadIdx.x == 0) count_copy[h] = miss_count[h];
  if (with_finish && (int)blockIdx.x >= n_fetch + S) {
    if ((int)blockIdx.x == n_fetch + S)
      als_finish_body<T>(fa, h);
    else
      als_index_append_body<T>(fa, h);  // (one wave) the appended row's entry in the score index
    return;
  }
  if ((int)blockIdx.x < n_fetch) {
    fetch_rows_attn_body<T>(store, cap, (uint4*)K, (uint4*)V, n_slots, hit, hit_stride, miss_slots, miss_count, hq, hkv,
                            cpr, k, h, blockIdx.x, n_fetch, q, d, scale_log2e,
                            part + ((int64_t)h * (S + n_fetch) + S + blockIdx.x) * (d + 2), miss_old, vic, miss_new, evk,
                            evk_rows);
    return;
  }
  // (eight row groups in flight per wave: the launch has few attention workgroups)
  attn_partial_body<T, 8>(q, K, V, n_slots, n_slots, d, lpr_log2, scale_log2e, part, S, S + n_fetch, evict, k, h,
                          (int)blockIdx.x - n_fetch, kq);
}

// One workgroup per head merges its S partial (max, sum, acc) triples (S <= kCombMaxS).
// d is a power of two <= 256: thread -> (column c, split group tg); all loads are issued up front.
constexpr int kCombMaxS = 128;
template <typename T>
__global__ __launch_bounds__(kCombThreads) void attn_combine_kernel(const float* __restrict__ part, int S, int d,
                                                                    T* __restrict__ out) {
  __shared__ float sc_s[kCombMaxS];  // weight exp2(m_t - M) of triple t (0 for an empty one)
  __shared__ float wred[2][4];
  __shared__ float comb[kCombThreads];
  const int h = blockIdx.x;
  const float* p = part + (int64_t)h * S * (d + 2);
  const int c = threadIdx.x & (d - 1);
  const int ntg = kCombThreads / d;  // >= 4
  const int tg = threadIdx.x / d;
  // only as many loads as there are triples for this thread (S, ntg are uniform): batches of 8
  const int per = (S - tg + ntg - 1) / ntg;
  constexpr int kPer = kCombMaxS / 4;  // triples per thread at most
  float x[kPer];
#pragma unroll
  for (int u0 = 0; u0 < kPer; u0 += 8) {
    if (u0 < per) {
#pragma unroll
      for (int u = u0; u < u0 + 8; ++u) x[u] = p[(int64_t)min(tg + u * ntg, S - 1) * (d + 2) + 2 + c];
    }
  }
  // the first two waves hold (m_t, l_t) of triple t = tid: block max, weights, weighted sum of l
  float mt = -INFINITY, lt = 0.0f;
  if (threadIdx.x < kCombMaxS) {
    const int t = min((int)threadIdx.x, S - 1);
    const float mv = p[(int64_t)t * (d + 2)], lv = p[(int64_t)t * (d + 2) + 1];
    if ((int)threadIdx.x < S) {
      mt = mv;
      lt = lv;
    }
    const float wm = wave_max(mt);
    if (lane_id() == 0) wred[0][wave_id()] = wm;
  }
  __syncthreads();
  const float Mh = fmaxf(wred[0][0], wred[0][1]);
  if (threadIdx.x < kCombMaxS) {
    const float w = (mt == -INFINITY) ? 0.0f : exp2f(mt - Mh);
    sc_s[threadIdx.x] = w;
    const float ws = wave_sum(lt * w);
    if (lane_id() == 0) wred[1][wave_id()] = ws;
  }
  __syncthreads();
  const float L = wred[1][0] + wred[1][1];
  float v = 0.0f;
#pragma unroll
  for (int u0 = 0; u0 < kPer; u0 += 8) {
    if (u0 < per) {
#pragma unroll
      for (int u = u0; u < u0 + 8; ++u) {
        const int t = tg + u * ntg;
        if (t < S) v = fmaf(x[u], sc_s[t], v);
      }
    }
  }
  comb[threadIdx.x] = v;
  __syncthreads();
  if (tg == 0) {
    float tot = 0.0f;
    for (int g = 0; g < ntg; ++g) tot += comb[g * d + c];
    st_f32<T>(out, (int64_t)h * d + c, L > 0.0f ? tot / L : 0.0f);
  }
}

static int attn_shape(int d, int vec, int* lpr_log2) {
  const int lpr = d / vec;
  int lg = 0;
  while ((1 << lg) < lpr) ++lg;
  LRQK_REQUIRE(d % vec == 0 && (1 << lg) == lpr && lpr <= kWave && d <= 256, LRQK_ELIMIT,
               "head_dim %d unsupported (need a power-of-two number of 16-byte chunks, <= 256 elements)", d);
  *lpr_log2 = lg;
  return LRQK_OK;
}

// Number of slot-axis splits of the stand-alone attention.
static int attn_splits(int n_valid) {
  int S = (n_valid + 63) / 64;
  if (S < 1) S = 1;
  if (S > 64) S = 64;
  return S;
}

// The two launches of the stand-alone attention; `part` holds bh * S * (d + 2) floats.  Every triple of
// `part` is written by the first launch (an empty split writes an empty triple), so it needs no clearing.
template <typename T>
static int attention_launch(const void* q, const void* k_act, const void* v_act, int n_slots, int n_valid, void* out,
                            int bh, int d, int lpr_log2, int S, float* part, hipStream_t st) {
  const float scale_log2e = (1.0f / sqrtf((float)d)) * 1.4426950408889634f;
  hipLaunchKernelGGL((attn_partial_kernel<T>), dim3((unsigned)S, (unsigned)bh), dim3(kAttnThreads), 0, st,
                     (const T*)q, (const T*)k_act, (const T*)v_act, n_slots, n_valid, d, lpr_log2, scale_log2e, part, S);
  LRQK_HIP_CHECK(hipGetLastError());
  hipLaunchKernelGGL((attn_combine_kernel<T>), dim3((unsigned)bh), dim3(kCombThreads), 0, st, (const float*)part, S, d,
                     (T*)out);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

template <typename T>
static int attention_impl(lrqk_ctx* ctx, const void* q, const void* k_act, const void* v_act, int n_slots, int n_valid,
                          void* out, int bh, int d, hipStream_t st) {
  int lpr_log2 = 0;
  int rc = attn_shape(d, Vec16<T>::N, &lpr_log2);
  if (rc) return rc;
  const int S = attn_splits(n_valid);
  if ((rc = ctx->attn_part.ensure((size_t)bh * S * (d + 2) * sizeof(float)))) return rc;
  return attention_launch<T>(q, k_act, v_act, n_slots, n_valid, out, bh, d, lpr_log2, S, (float*)ctx->attn_part.p, st);
}

// ----------------------------------------------------------------------------- attention without allocation
// Split partials of lrqk_attention_static: a fixed block in the code object's own device memory, one copy per
// GPU the library runs on, held until the process ends.
constexpr size_t kStaticPartFloats = (size_t)1 << 20;  // 4 MiB
static __device__ __align__(256) float g_attn_static_part[kStaticPartFloats];

constexpr int kMaxDevices = 64;
static std::mutex g_static_mu;
static float* g_static_part_ptr[kMaxDevices];  // device address of the block on each GPU (nullptr: not asked yet)

// Device address of g_attn_static_part on the current GPU (resolved once per device).
static int static_part(float** out) {
  int dev = 0;
  LRQK_HIP_CHECK(hipGetDevice(&dev));
  LRQK_REQUIRE(dev >= 0 && dev < kMaxDevices, LRQK_ELIMIT, "device ordinal %d beyond %d", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_static_mu);
  if (!g_static_part_ptr[dev]) {
    float* p = nullptr;
    LRQK_HIP_CHECK(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(g_attn_static_part)));
    LRQK_REQUIRE(p != nullptr, LRQK_EHIP, "hipGetSymbolAddress returned a null address");
    g_static_part_ptr[dev] = p;
  }
  *out = g_static_part_ptr[dev];
  return LRQK_OK;
}

template <typename T>
static int attention_static_impl(const void* q, const void* k_act, const void* v_act, int n_slots, int n_valid,
                                 void* out, int bh, int d, hipStream_t st) {
  int lpr_log2 = 0;
  int rc = attn_shape(d, Vec16<T>::N, &lpr_log2);
  if (rc) return rc;
  const int S = attn_splits(n_valid);
  const size_t need = (size_t)bh * S * (d + 2);
  LRQK_REQUIRE(need <= kStaticPartFloats, LRQK_ELIMIT,
               "bh=%d x %d splits x (d+2)=%d floats of partial results exceed the static block of %zu floats", bh, S, d + 2,
               kStaticPartFloats);
  float* part = nullptr;
  if ((rc = static_part(&part))) return rc;
  return attention_launch<T>(q, k_act, v_act, n_slots, n_valid, out, bh, d, lpr_log2, S, part, st);
}

template <typename T>
static int fetch_attention_impl(lrqk_ctx* ctx, const void* dev_store, int64_t cap, void* k_act, void* v_act,
                                int n_slots, int32_t* hit, int64_t hit_stride, const int32_t* miss_slots,
                                const int32_t* miss_count, const uint8_t* evict, int b, int hq, int hkv, int d, int k,
                                const void* q, void* out, hipStream_t st, const int32_t* miss_old,
                                const VictimView* vicp, const int32_t* miss_new, void* evk, int evk_rows,
                                int32_t* count_copy) {
  const int bh = b * hq;
  VictimView vic{};
  if (vicp && miss_old && vicp->nv > 0) vic = *vicp;
  int lpr_log2 = 0;
  int rc = attn_shape(d, Vec16<T>::N, &lpr_log2);
  if (rc) return rc;
  const int cpr = d * (int)sizeof(T) / 16;
  LRQK_REQUIRE(2 * cpr <= kWave, LRQK_ELIMIT, "row of %d bytes does not fit one wave", 2 * cpr * 16);
  // The launch should not hold more workgroups than the GPU does at a time (a second batch would only start when
  // the first has finished): 256 slots per attention workgroup, and as many fetch workgroups as still fit, between
  // 8 and the number that a miss rate of 1/8 keeps busy (with enough of them a head's misses take one trip).
  static std::atomic<int> slots_dev[kMaxDeviceSlots];
  std::atomic<int>& slots_a = slots_dev[per_device_slot()];
  int slots = slots_a;
  if (slots == 0) {
    int per_cu = 0, dev = 0, n_cu = 0;
    LRQK_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fetch_attn_partial_kernel<T>, kAttnThreads, 0));
    LRQK_HIP_CHECK(hipGetDevice(&dev));
    LRQK_HIP_CHECK(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev));
    slots = std::max(1, per_cu * n_cu);
    slots_a = slots;
  }
  const int rpb = kAttnThreads / (2 * cpr);
  const int want_fetch = std::max(1, std::min(32, (k / 8 + rpb - 1) / rpb));
  int S = (n_slots + 255) / 256;  // (128 slots per workgroup left the fetch role fewer workgroups: 0.3 .. 1.5 us slower)
  if (S > 64) S = 64;
  if (!out) S = 0;  // fetch only (the caller runs its own attention): no attention workgroups, nothing to merge
  const int room = slots / bh - S - 2;
  const int n_fetch = std::min(want_fetch, std::max(room, 8));
  if ((rc = ctx->attn_part.ensure((size_t)bh * (S + n_fetch) * (d + 2) * sizeof(float)))) return rc;
  const float scale_log2e = (1.0f / sqrtf((float)d)) * 1.4426950408889634f;
  static_assert(kAttnThreads == kFinThreads, "the finish stage rides in an attention-sized workgroup");
  int with_finish = 0;
  if (ctx->fin_pending) {
    if (ctx->fin.bh == bh && ctx->fin_dtype == (sizeof(T) == 4 ? LRQK_F32 : LRQK_BF16) && !ctx->qhat_pending) {
      with_finish = 1;
      ctx->fin_pending = false;
    } else if ((rc = flush_pending_finish(ctx, st))) {
      return rc;
    }
  }
  const int index_role = with_finish && ctx->fin.qa != nullptr && ctx->fin.append_row >= 0 ? 1 : 0;
  // K q of every slot, left by this step's Gram pass over the same buffers and query (else the role reads K)
  const float* kq = nullptr;
  if (out && ctx->kq_valid && ctx->kq_k_act == k_act && ctx->kq_q == q && ctx->kq_bh == bh && ctx->kq_n == n_slots)
    kq = (const float*)ctx->als_kq.p;
  ctx->kq_valid = false;
  hipLaunchKernelGGL((fetch_attn_partial_kernel<T>), dim3((unsigned)(n_fetch + S + with_finish + index_role), (unsigned)bh),
                     dim3(kAttnThreads), 0, st, (const uint4*)dev_store, cap, hit, hit_stride, miss_slots, miss_count,
                     evict, hq, hkv, cpr, k, n_fetch, (const T*)q, (T*)k_act, (T*)v_act, n_slots, d, lpr_log2,
                     scale_log2e, (float*)ctx->attn_part.p, S, with_finish, ctx->fin, miss_old, vic, miss_new, kq,
                     (uint4*)evk, evk_rows, count_copy);
  LRQK_HIP_CHECK(hipGetLastError());
  if (out) {
    hipLaunchKernelGGL((attn_combine_kernel<T>), dim3((unsigned)bh), dim3(kCombThreads), 0, st,
                       (const float*)ctx->attn_part.p, S + n_fetch, d, (T*)out);
    LRQK_HIP_CHECK(hipGetLastError());
  }
  return LRQK_OK;
}

// Miss fetch overlapped with the attention over the slots that stay resident, then the
// refetched slots and the merge.  Same result as lrqk_fetch_rows followed by lrqk_attention.
// out = NULL: the fetch alone (with the victim cache and the roles that ride along), for a caller
// that runs its own attention over the active set.
int fetch_attention(lrqk_ctx* ctx, const void* kv_store, int64_t cap, void* k_act, void* v_act, int n_slots,
                    int32_t* hit, int64_t hit_stride, const int32_t* miss_slots, const int32_t* miss_count,
                    const uint8_t* evict, int b, int hq, int hkv, int d, int k, const void* q, void* out, int dtype,
                    hipStream_t st, const int32_t* miss_old, const VictimView* vic, const int32_t* miss_new, void* evk,
                    int evk_rows, int32_t* count_copy) {
  const void* dev_store = nullptr;
  int rc = resolve_store(kv_store, &dev_store);
  if (rc) return rc;
  LRQK_REQUIRE(((uintptr_t)dev_store % 16 == 0) && ((uintptr_t)q % 16 == 0) && ((uintptr_t)k_act % 16 == 0) &&
                   ((uintptr_t)v_act % 16 == 0),
               LRQK_EINVAL, "pointers must be 16-byte aligned");
  if (dtype == LRQK_F32)
    return fetch_attention_impl<float>(ctx, dev_store, cap, k_act, v_act, n_slots, hit, hit_stride, miss_slots,
                                       miss_count, evict, b, hq, hkv, d, k, q, out, st, miss_old, vic, miss_new, evk,
                                       evk_rows, count_copy);
  return fetch_attention_impl<bf16_t>(ctx, dev_store, cap, k_act, v_act, n_slots, hit, hit_stride, miss_slots,
                                      miss_count, evict, b, hq, hkv, d, k, q, out, st, miss_old, vic, miss_new, evk,
                                      evk_rows, count_copy);
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

extern "C" int lrqk_attention_static(const void* q, const void* k_act, const void* v_act, int n_slots, int n_valid,
                                     void* out, int bh, int d, int dtype, void* stream) {
  LRQK_REQUIRE(q && k_act && v_act && out, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(dtype == LRQK_F32 || dtype == LRQK_BF16, LRQK_EINVAL, "dtype=%d", dtype);
  LRQK_REQUIRE(bh > 0 && bh <= 65535 && d > 0, LRQK_EINVAL, "bad sizes bh=%d d=%d", bh, d);
  LRQK_REQUIRE(n_valid > 0 && n_valid <= n_slots, LRQK_EINVAL, "n_valid=%d outside 1..%d", n_valid, n_slots);
  LRQK_REQUIRE(((uintptr_t)q % 16 == 0) && ((uintptr_t)k_act % 16 == 0) && ((uintptr_t)v_act % 16 == 0), LRQK_EINVAL,
               "pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == LRQK_F32) return attention_static_impl<float>(q, k_act, v_act, n_slots, n_valid, out, bh, d, st);
  return attention_static_impl<bf16_t>(q, k_act, v_act, n_slots, n_valid, out, bh, d, st);
}
