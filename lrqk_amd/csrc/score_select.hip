// Proxy-score scan q_hat . A_K^T and the per-head top-k selector.
//
// Score contract: fp32 fmaf chain over j = 0..r-1 starting at +0, optional rounding to
// bf16, -0 -> +0.  Selection order: (score descending, token index ascending); the
// result is written ascending by index.
#include "common.hpp"
#include "ctx.hpp"

namespace lrqk {

// --------------------------------------------------------------------------- scores
// One thread per cached token row.  R > 0: row of R elements fetched with 16-byte loads.
// R == 0: any r, scalar loads.
template <typename T, int R>
__global__ __launch_bounds__(256) void score_kernel(const T* __restrict__ a_k, int64_t head_stride,
                                                    const T* __restrict__ q_hat, int64_t m, int r,
                                                    int round_bf16, uint32_t* __restrict__ keys,
                                                    int64_t key_stride, float* __restrict__ scores) {
  const int h = blockIdx.y;
  const T* A = a_k + (int64_t)h * head_stride;
  const T* qh = q_hat + (int64_t)h * r;
  constexpr int VEC = Vec16<T>::N;
  float qf[R > 0 ? R : 1];
  if (R > 0) {
#pragma unroll
    for (int j = 0; j < R; ++j) qf[j] = ld_f32<T>(qh, j);
  }
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < m; i += (int64_t)gridDim.x * blockDim.x) {
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

// --------------------------------------------------------------------------- general select
// One workgroup of 1024 threads per head.  Three radix passes (12 + 10 + 10 bits, most
// significant first) over the head's keys find the k-th largest key T and how many keys
// equal to T must be taken; a final in-order pass emits every index with key > T and the
// first `need` indices with key == T.  Works for any key distribution (all-equal included).
constexpr int kSelThreads = 1024;

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

__global__ __launch_bounds__(kSelThreads) void select_general_kernel(const uint32_t* __restrict__ keys_all,
                                                                      int64_t key_stride, int64_t m, int k,
                                                                      int32_t* __restrict__ out_all,
                                                                      int64_t out_stride) {
  __shared__ uint32_t hist[4096];
  __shared__ int scratch[kSelThreads / kWave + 1];
  __shared__ uint32_t s_prefix;
  __shared__ int s_need;
  const int tid = threadIdx.x;
  const uint32_t* keys = keys_all + (int64_t)blockIdx.x * key_stride;
  int32_t* out = out_all + (int64_t)blockIdx.x * out_stride;

  uint32_t prefix = 0, mask = 0;
  int need = k;
  for (int pass = 0; pass < 3; ++pass) {
    const int shift = pass == 0 ? 20 : (pass == 1 ? 10 : 0);
    const int nb = pass == 0 ? 4096 : 1024;
    for (int i = tid; i < nb; i += kSelThreads) hist[i] = 0;
    if (tid == 0) {
      s_prefix = prefix;
      s_need = need;
    }
    __syncthreads();
    for (int64_t i = tid; i < m; i += kSelThreads) {
      uint32_t key = keys[i];
      if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & (uint32_t)(nb - 1)], 1u);
    }
    __syncthreads();
    const int per = nb / kSelThreads;  // 4 or 1
    int local = 0;
    for (int b = 0; b < per; ++b) local += (int)hist[tid * per + b];
    int total;
    int incl = block_inclusive_sum_1024(local, scratch, total);
    int above = total - incl;  // keys in bins above this thread's bins
    if (above < need && need <= above + local) {
      int c = above;
      for (int b = per - 1; b >= 0; --b) {
        int cnt = (int)hist[tid * per + b];
        if (c + cnt >= need) {
          s_prefix = prefix | ((uint32_t)(tid * per + b) << shift);
          s_need = need - c;
          break;
        }
        c += cnt;
      }
    }
    __syncthreads();
    prefix = s_prefix;
    need = s_need;
    mask |= (uint32_t)(nb - 1) << shift;
    __syncthreads();
  }

  const uint32_t T = prefix;
  const int need_eq = need;
  int out_pos = 0, eq_seen = 0;
  for (int64_t base = 0; base < m && out_pos < k; base += kSelThreads) {
    const int64_t i = base + tid;
    const bool valid = i < m;
    const uint32_t key = valid ? keys[i] : 0u;
    const bool gt = valid && key > T;
    const bool eq = valid && key == T;
    int eq_tot, sel_tot;
    const int eq_rank = block_rank(eq, scratch, eq_tot);
    const bool sel = gt || (eq && (eq_seen + eq_rank) < need_eq);
    const int pos = block_rank(sel, scratch, sel_tot);
    if (sel) out[out_pos + pos] = (int32_t)i;
    out_pos += sel_tot;
    eq_seen += eq_tot;
  }
}

static int run_select(lrqk_ctx* ctx, int bh, int64_t m, int64_t key_stride, int topk, int32_t* out_idx,
                      int64_t out_stride, hipStream_t st) {
  hipLaunchKernelGGL(select_general_kernel, dim3((unsigned)bh), dim3(kSelThreads), 0, st,
                     (const uint32_t*)ctx->keys.p, key_stride, m, topk, out_idx, out_stride);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
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
  if (m <= topk) {
    if (m > 0) {
      hipLaunchKernelGGL(arange_kernel, dim3((unsigned)((m + 255) / 256), (unsigned)bh), dim3(256), 0, st, out_idx,
                         out_stride, (int)m);
      LRQK_HIP_CHECK(hipGetLastError());
    }
    return (int)m;
  }
  const int64_t key_stride = (m + 63) & ~(int64_t)63;
  rc = ctx->keys.ensure((size_t)bh * key_stride * 4);
  if (rc) return rc;
  const bool timed = ctx->tev && ctx->tev_used < ctx->tev_pairs;
  if (timed) LRQK_HIP_CHECK(hipEventRecord(ctx->tev[2 * ctx->tev_used], st));
  if (dtype == LRQK_F32)
    rc = launch_scores<float>(a_k, head_stride, q_hat, bh, m, r, 0, (uint32_t*)ctx->keys.p, key_stride, nullptr, st);
  else
    rc = launch_scores<bf16_t>(a_k, head_stride, q_hat, bh, m, r, round_bf16, (uint32_t*)ctx->keys.p, key_stride,
                               nullptr, st);
  if (rc) return rc;
  if (timed) {
    LRQK_HIP_CHECK(hipEventRecord(ctx->tev[2 * ctx->tev_used + 1], st));
    ++ctx->tev_used;
  }
  rc = run_select(ctx, bh, m, key_stride, topk, out_idx, out_stride, st);
  return rc ? rc : topk;
}

extern "C" int lrqk_select_from_scores(lrqk_ctx* ctx, const float* scores, int bh, int64_t m, int topk,
                                       int32_t* out_idx, int64_t out_stride, void* stream) {
  int rc = check_select_args(ctx, bh, m, topk, out_idx, out_stride);
  if (rc) return rc;
  LRQK_REQUIRE(scores != nullptr, LRQK_EINVAL, "scores is null");
  hipStream_t st = (hipStream_t)stream;
  if (m <= topk) {
    if (m > 0) {
      hipLaunchKernelGGL(arange_kernel, dim3((unsigned)((m + 255) / 256), (unsigned)bh), dim3(256), 0, st, out_idx,
                         out_stride, (int)m);
      LRQK_HIP_CHECK(hipGetLastError());
    }
    return (int)m;
  }
  const int64_t key_stride = (m + 63) & ~(int64_t)63;
  rc = ctx->keys.ensure((size_t)bh * key_stride * 4);
  if (rc) return rc;
  int64_t blocks = (m + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  hipLaunchKernelGGL(keys_from_scores_kernel, dim3((unsigned)blocks, (unsigned)bh), dim3(256), 0, st, scores, m,
                     (uint32_t*)ctx->keys.p, key_stride);
  LRQK_HIP_CHECK(hipGetLastError());
  rc = run_select(ctx, bh, m, key_stride, topk, out_idx, out_stride, st);
  return rc ? rc : topk;
}
