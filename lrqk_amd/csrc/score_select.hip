// Proxy-score scan q_hat . A_K^T and the per-head top-k selector.
//
// Score contract: fp32 fmaf chain over j = 0..r-1 starting at +0, optional rounding to
// bf16, -0 -> +0.  Selection order: (score descending, token index ascending); the
// result is written ascending by index.
//
// Decode-time structure (two launches, scores never reach HBM):
//   score_filter : streams A_K once; a row becomes a CANDIDATE if its key is >= the head's
//                  running lower bound t_low (the key that had rank ~2k at the previous
//                  call).  Candidates (key, index) are packed per workgroup in LDS and
//                  appended to a small per-head list.
//   select       : one workgroup per head.  If the list holds at least k (and not too many)
//                  candidates it provably contains the exact top-k including every tie at
//                  the threshold, and the exact radix select runs on the list alone.
//                  Otherwise (first call, distribution shift) the workgroup recomputes the
//                  head's scores itself and selects over all of them.  Either way it leaves
//                  the next t_low.  Results never depend on t_low, only speed does.
#include "common.hpp"
#include "ctx.hpp"

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

__global__ void init_select_state_kernel(uint32_t* t_low, int* cand_count, int* stats, int bh) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < bh) {
    t_low[i] = 0xffffffffu;
    cand_count[i] = 0;
  }
  if (i < 2) stats[i] = 0;
}

// --------------------------------------------------------------------------- score + filter
constexpr int kFiltThreads = 256;
constexpr int kFiltRPT = 8;  // rows per thread
constexpr int kFiltRows = kFiltThreads * kFiltRPT;

template <typename T, int R>
__global__ __launch_bounds__(kFiltThreads) void score_filter_kernel(const T* __restrict__ a_k, int64_t head_stride,
                                                                    const T* __restrict__ q_hat, int64_t m, int r,
                                                                    int round_bf16, const uint32_t* __restrict__ t_low,
                                                                    uint2* __restrict__ cand, int cand_cap,
                                                                    int* __restrict__ cand_count) {
  __shared__ uint2 lc[kFiltRows];
  __shared__ int l_count, g_base;
  const int h = blockIdx.y;
  const int tid = threadIdx.x;
  const T* A = a_k + (int64_t)h * head_stride;
  RowScorer<T, R> rs;
  rs.init(q_hat + (int64_t)h * r, r, round_bf16);
  const uint32_t tl = t_low[h];
  if (tid == 0) l_count = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kFiltRows;
#pragma unroll 4
  for (int it = 0; it < kFiltRPT; ++it) {
    const int64_t i = base + it * kFiltThreads + tid;
    const bool valid = i < m;
    const uint32_t key = valid ? score_key(rs.score(A, i)) : 0u;
    const bool pred = valid && key >= tl;
    int tot;
    const int rank = wave_rank(pred, tot);
    int wbase = 0;
    if (tot) {
      if (lane_id() == 0) wbase = atomicAdd(&l_count, tot);
      wbase = __shfl(wbase, 0, kWave);
      if (pred) lc[wbase + rank] = make_uint2(key, (uint32_t)i);
    }
  }
  __syncthreads();
  const int n = l_count;
  if (n == 0) return;
  if (tid == 0) g_base = atomicAdd(&cand_count[h], n);
  __syncthreads();
  const int gb = g_base;
  for (int j = tid; j < n; j += kFiltThreads) {
    const int p = gb + j;
    if (p < cand_cap) cand[(int64_t)h * cand_cap + p] = lc[j];
  }
}

// --------------------------------------------------------------------------- select
constexpr int kSelThreads = 1024;
constexpr int kChunkBits = 262144;            // token ids covered by one bitmap pass
constexpr int kChunkWords = kChunkBits / 32;  // 8192 words = 32 KB per bitmap

__device__ __forceinline__ int block_inclusive_sum_1024(int v, int* scratch, int& total) {
  int inc = wave_inclusive_sum(v);
  if (lane_id() == kWave - 1) scratch[wave_id()] = inc;
  __syncthreads();
  int base = 0, tot = 0;
  const int nw = blockDim.x >> 6;
  for (int w = 0; w < nw; ++w) {
    int c = scratch[w];
    if (w < wave_id()) base += c;
    tot += c;
  }
  __syncthreads();
  total = tot;
  return base + inc;
}

// Digit of the `need`-th largest element from a histogram of nb bins (nb = 4096 or 1024):
// the largest digit D with count(digit > D) < need <= count(digit >= D).  Every thread
// gets (D, need - count(digit > D)).  s_pair: 2 shared ints.
__device__ __forceinline__ int find_digit(const uint32_t* hist, int nb, int need, int* scratch, int* s_pair,
                                          int& need_out) {
  const int tid = threadIdx.x;
  const int per = nb / kSelThreads;  // 4 or 1
  int local = 0;
  for (int b = 0; b < per; ++b) local += (int)hist[tid * per + b];
  if (tid == 0) {
    s_pair[0] = 0;
    s_pair[1] = need;
  }
  int total;
  const int incl = block_inclusive_sum_1024(local, scratch, total);  // barriers order the init above
  const int above = total - incl;
  if (above < need && need <= above + local) {
    int c = above;
    for (int b = per - 1; b >= 0; --b) {
      const int cnt = (int)hist[tid * per + b];
      if (c + cnt >= need) {
        s_pair[0] = tid * per + b;
        s_pair[1] = need - c;
        break;
      }
      c += cnt;
    }
  }
  __syncthreads();
  const int d = s_pair[0];
  need_out = s_pair[1];
  __syncthreads();
  return d;
}

// mode: 0 = use the candidate list if valid, else compute the head's keys from A_K;
//       1 = keys[] already holds the head's keys (test hook / caller-provided scores).
template <typename T, int R>
__global__ __launch_bounds__(kSelThreads) void select_kernel(int mode, const uint2* __restrict__ cand_all, int cand_cap,
                                                             int* __restrict__ cand_count, uint32_t* __restrict__ t_low,
                                                             uint32_t* __restrict__ keys_all, int64_t key_stride,
                                                             const T* __restrict__ a_k, int64_t head_stride,
                                                             const T* __restrict__ q_hat, int64_t m, int r, int round_bf16,
                                                             int k, int32_t* __restrict__ out_all, int64_t out_stride,
                                                             int* __restrict__ stats) {
  extern __shared__ __align__(16) uint32_t bitmaps[];  // gt[kChunkWords] | eq[kChunkWords]
  __shared__ uint32_t hist[4096];
  __shared__ uint32_t hist_b[1024];
  __shared__ int scratch[kSelThreads / kWave + 1];
  __shared__ int s_pair[2];
  __shared__ int s_n;
  uint32_t* gt = bitmaps;
  uint32_t* eq = bitmaps + kChunkWords;
  const int tid = threadIdx.x;
  const int h = blockIdx.x;
  uint32_t* keys = keys_all + (int64_t)h * key_stride;
  const uint2* cand = cand_all + (int64_t)h * cand_cap;
  int32_t* out = out_all + (int64_t)h * out_stride;

  bool fast = false;
  int64_t N = m;
  if (mode == 0) {
    if (tid == 0) {
      s_n = cand_count[h];
      cand_count[h] = 0;  // re-arm for the next call
    }
    __syncthreads();
    const int n = s_n;
    fast = n >= k && n <= cand_cap;
    if (fast) {
      N = n;
    } else {
      const T* A = a_k + (int64_t)h * head_stride;
      RowScorer<T, R> rs;
      rs.init(q_hat + (int64_t)h * r, r, round_bf16);
      for (int64_t i = tid; i < m; i += kSelThreads) keys[i] = score_key(rs.score(A, i));
      __threadfence_block();
      __syncthreads();
    }
    if (tid == 0) atomicAdd(&stats[fast ? 0 : 1], 1);
  }
  // The candidate list is read once into registers (one batch of independent loads); the
  // rescan path walks the key array in batches of 8 independent loads per thread.
  constexpr int kRegCand = 8;
  const bool in_regs = fast && N <= (int64_t)kRegCand * kSelThreads;
  uint2 creg[kRegCand];
  if (in_regs) {
#pragma unroll
    for (int u = 0; u < kRegCand; ++u) {
      const int64_t j = tid + (int64_t)u * kSelThreads;
      creg[u] = j < N ? cand[j] : make_uint2(0u, 0u);
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
        for (int u = 0; u < 8; ++u) {
          const int64_t j = j0 + (int64_t)u * kSelThreads;
          kk[u] = j < N ? keys[j] : 0u;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int64_t j = j0 + (int64_t)u * kSelThreads;
          if (j < N) f(kk[u], j);
        }
      }
    }
  };

  const int k2 = (int)min((int64_t)2 * k, N);  // rank that defines the next t_low
  // ---- pass 1: top 12 bits, shared by both ranks
  for (int i = tid; i < 4096; i += kSelThreads) hist[i] = 0;
  __syncthreads();
  for_each([&](uint32_t key, int64_t) { atomicAdd(&hist[key >> 20], 1u); });
  __syncthreads();
  int need1, needE;
  const uint32_t D1 = (uint32_t)find_digit(hist, 4096, k, scratch, s_pair, need1);
  const uint32_t E1 = (uint32_t)find_digit(hist, 4096, k2, scratch, s_pair, needE);
  // ---- pass 2: next 10 bits under each prefix
  for (int i = tid; i < 1024; i += kSelThreads) {
    hist[i] = 0;
    hist_b[i] = 0;
  }
  __syncthreads();
  for_each([&](uint32_t key, int64_t) {
    const uint32_t top = key >> 20;
    if (top == D1) atomicAdd(&hist[(key >> 10) & 1023u], 1u);
    if (top == E1) atomicAdd(&hist_b[(key >> 10) & 1023u], 1u);
  });
  __syncthreads();
  int need2, needE2;
  const uint32_t D2 = (uint32_t)find_digit(hist, 1024, need1, scratch, s_pair, need2);
  const uint32_t E2 = (uint32_t)find_digit(hist_b, 1024, needE, scratch, s_pair, needE2);
  if (tid == 0) t_low[h] = (E1 << 20) | (E2 << 10);
  // ---- pass 3: last 10 bits
  const uint32_t pre22 = (D1 << 10) | D2;
  for (int i = tid; i < 1024; i += kSelThreads) hist[i] = 0;
  __syncthreads();
  for_each([&](uint32_t key, int64_t) {
    if ((key >> 10) == pre22) atomicAdd(&hist[key & 1023u], 1u);
  });
  __syncthreads();
  int need_eq;
  const uint32_t D3 = (uint32_t)find_digit(hist, 1024, need2, scratch, s_pair, need_eq);
  const uint32_t Tk = (pre22 << 10) | D3;

  // ---- ordered output through two bitmaps over the token ids: gt (key > T), eq (key == T).
  // Every index with key > T is emitted, plus the first need_eq indices with key == T.
  int out_pos = 0, eq_seen = 0;
  for (int64_t c0 = 0; c0 < m; c0 += kChunkBits) {
    const int span = (int)min((int64_t)kChunkBits, m - c0);
    const int words = (span + 31) >> 5;
    for (int i = tid; i < words; i += kSelThreads) {
      gt[i] = 0;
      eq[i] = 0;
    }
    __syncthreads();
    for_each([&](uint32_t key, int64_t idx) {
      const int64_t rel = idx - c0;
      if (key >= Tk && rel >= 0 && rel < span) atomicOr(key > Tk ? &gt[rel >> 5] : &eq[rel >> 5], 1u << (rel & 31));
    });
    __syncthreads();
    const int W = (words + kSelThreads - 1) / kSelThreads;
    const int w0 = tid * W;
    int cg = 0, ce = 0;
    for (int w = w0; w < min(words, w0 + W); ++w) {
      cg += __popc(gt[w]);
      ce += __popc(eq[w]);
    }
    int g_tot, e_tot;
    const int g_incl = block_inclusive_sum_1024(cg, scratch, g_tot);
    const int e_incl = block_inclusive_sum_1024(ce, scratch, e_tot);
    int e_run = eq_seen + e_incl - ce;  // equal keys before this thread's words (all chunks)
    int pos = out_pos + (g_incl - cg) + (min(e_run, need_eq) - min(eq_seen, need_eq));
    for (int w = w0; w < min(words, w0 + W); ++w) {
      const uint32_t gw = gt[w], ew = eq[w];
      uint32_t both = gw | ew;
      while (both) {
        const int bit = __ffs(both) - 1;
        both &= both - 1;
        const int32_t idx = (int32_t)(c0 + (int64_t)w * 32 + bit);
        if ((gw >> bit) & 1u) {
          out[pos++] = idx;
        } else {
          if (e_run < need_eq) out[pos++] = idx;
          ++e_run;
        }
      }
    }
    out_pos += g_tot + (min(eq_seen + e_tot, need_eq) - min(eq_seen, need_eq));
    eq_seen += e_tot;
    __syncthreads();
  }
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

constexpr size_t kSelSmem = (size_t)2 * kChunkWords * sizeof(uint32_t);

struct SelectBufs {
  uint2* cand;
  int cand_cap;
  int* cand_count;
  uint32_t* t_low;
  int* stats;
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
  sb->cand_cap = 4 * topk < 4096 ? 4096 : 4 * topk;
  if ((rc = ctx->cand.ensure((size_t)bh * sb->cand_cap * sizeof(uint2)))) return rc;
  sb->cand = (uint2*)ctx->cand.p;
  // layout: t_low u32 [bh] | cand_count i32 [bh] | stats i32 [2]
  void* before = ctx->cand_cnt.p;
  if ((rc = ctx->cand_cnt.ensure((size_t)(2 * bh + 2) * 4))) return rc;
  sb->t_low = (uint32_t*)ctx->cand_cnt.p;
  sb->cand_count = (int*)(sb->t_low + bh);
  sb->stats = sb->cand_count + bh;
  if (before != ctx->cand_cnt.p || ctx->sel_bh != bh) {
    hipLaunchKernelGGL(init_select_state_kernel, dim3((unsigned)((bh + 255) / 256)), dim3(256), 0, st, sb->t_low,
                       sb->cand_count, sb->stats, bh);
    LRQK_HIP_CHECK(hipGetLastError());
    ctx->sel_bh = bh;
  }
  return LRQK_OK;
}

template <typename T, int R>
static int launch_filter_select(lrqk_ctx* ctx, const SelectBufs& sb, const void* a_k, int64_t head_stride,
                                const void* q_hat, int bh, int64_t m, int r, int round_bf16, int topk, int32_t* out_idx,
                                int64_t out_stride, hipStream_t st) {
  static bool attr_done = false;
  if (!attr_done) {
    LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)select_kernel<T, R>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)kSelSmem));
    attr_done = true;
  }
  const bool timed = ctx->tev && ctx->tev_used < ctx->tev_pairs;
  if (timed) LRQK_HIP_CHECK(hipEventRecord(ctx->tev[2 * ctx->tev_used], st));
  dim3 grid((unsigned)((m + kFiltRows - 1) / kFiltRows), (unsigned)bh);
  hipLaunchKernelGGL((score_filter_kernel<T, R>), grid, dim3(kFiltThreads), 0, st, (const T*)a_k, head_stride,
                     (const T*)q_hat, m, r, round_bf16, sb.t_low, sb.cand, sb.cand_cap, sb.cand_count);
  LRQK_HIP_CHECK(hipGetLastError());
  if (timed) {
    LRQK_HIP_CHECK(hipEventRecord(ctx->tev[2 * ctx->tev_used + 1], st));
    ++ctx->tev_used;
  }
  hipLaunchKernelGGL((select_kernel<T, R>), dim3((unsigned)bh), dim3(kSelThreads), kSelSmem, st, 0, sb.cand, sb.cand_cap,
                     sb.cand_count, sb.t_low, sb.keys, sb.key_stride, (const T*)a_k, head_stride, (const T*)q_hat, m, r,
                     round_bf16, topk, out_idx, out_stride, sb.stats);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

template <typename T>
static int dispatch_filter_select(lrqk_ctx* ctx, const SelectBufs& sb, const void* a_k, int64_t head_stride,
                                  const void* q_hat, int bh, int64_t m, int r, int round_bf16, int topk,
                                  int32_t* out_idx, int64_t out_stride, hipStream_t st) {
  const bool vec_ok = ((uintptr_t)a_k % 16 == 0) && ((head_stride * sizeof(T)) % 16 == 0);
#define LRQK_FS_CASE(RR) \
  return launch_filter_select<T, RR>(ctx, sb, a_k, head_stride, q_hat, bh, m, r, round_bf16, topk, out_idx, out_stride, st)
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
  if (dtype == LRQK_F32)
    rc = dispatch_filter_select<float>(ctx, sb, a_k, head_stride, q_hat, bh, m, r, 0, topk, out_idx, out_stride, st);
  else
    rc = dispatch_filter_select<bf16_t>(ctx, sb, a_k, head_stride, q_hat, bh, m, r, round_bf16, topk, out_idx,
                                        out_stride, st);
  return rc ? rc : topk;
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
  static bool attr_done = false;
  if (!attr_done) {
    LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)select_kernel<float, 0>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)kSelSmem));
    attr_done = true;
  }
  hipLaunchKernelGGL((select_kernel<float, 0>), dim3((unsigned)bh), dim3(kSelThreads), kSelSmem, st, 1, sb.cand,
                     sb.cand_cap, sb.cand_count, sb.t_low, sb.keys, sb.key_stride, (const float*)nullptr, (int64_t)0,
                     (const float*)nullptr, m, 1, 0, topk, out_idx, out_stride, sb.stats);
  LRQK_HIP_CHECK(hipGetLastError());
  return topk;
}

extern "C" int lrqk_select_stats(lrqk_ctx* ctx, int* fast_heads, int* full_heads, int reset) {
  LRQK_REQUIRE(ctx && fast_heads && full_heads, LRQK_EINVAL, "null pointer");
  *fast_heads = *full_heads = 0;
  if (!ctx->cand_cnt.p || ctx->sel_bh <= 0) return LRQK_OK;
  int* stats = (int*)ctx->cand_cnt.p + 2 * ctx->sel_bh;
  int v[2];
  LRQK_HIP_CHECK(hipMemcpy(v, stats, sizeof(v), hipMemcpyDeviceToHost));
  *fast_heads = v[0];
  *full_heads = v[1];
  if (reset) LRQK_HIP_CHECK(hipMemset(stats, 0, sizeof(v)));
  return LRQK_OK;
}
