/*
 * CPU oracle for the bit-exact (integer / byte / ordered-float) stages of the
 * LRQK decode step.  TEST INFRASTRUCTURE ONLY: this file is the checker that the
 * HIP path is compared against and the thing the CPU baseline times; the shipped
 * library never links or calls it.
 *
 * Every function restates one piece of the reference (paths relative to the
 * reference tree):
 *   oracle_proxy_scores      lrqk_attention.py:1260-1263  (A_K[:m] . q_hat^T)
 *   oracle_topk_sorted       lrqk_attention.py:1266-1273  (topk then ascending sort)
 *   oracle_only_indices      lrqk_attention.py:1303-1315  (hit/miss diff)
 *   oracle_linear_indices    lrqk_attention.py:91-98      (mask -> linear row ids)
 *   oracle_d0_indices_select cpp_kernel/take_along_dim_grouped.cpp:133-183
 *   oracle_take_along_dim_with_mask
 *                            cpp_kernel/take_along_dim_grouped.cpp:13-124
 *
 * Contract for the floating-point score (where the reference is silent):
 *   score(i) = fmaf-chain over j = 0..r-1 of fp32(A[i][j]) * fp32(q[j]), starting
 *   from +0.0f; a result of -0.0f is replaced by +0.0f; if round_bf16 != 0 the fp32
 *   sum is then rounded to bfloat16 (nearest-even) and widened again, which is what a
 *   bf16 x bf16 -> bf16 matmul returns.  Selection order: score descending, then
 *   token index ascending (the reference leaves ties to torch.topk).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t v) {
  uint32_t u = ((uint32_t)v) << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline float round_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) { /* NaN: keep quiet NaN */
    u |= 0x00400000u;
    u &= 0xffff0000u;
  } else {
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    u &= 0xffff0000u;
  }
  memcpy(&f, &u, 4);
  return f;
}

/* Monotone map float -> uint32 (larger float <=> larger key); -0 and +0 compare equal,
 * as they do for torch.topk, so they share one key. */
static inline uint32_t order_key(float f) {
  uint32_t u;
  if (f == 0.0f) f = 0.0f;
  memcpy(&u, &f, 4);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

/* dtype: 0 = float32, 1 = bfloat16 (raw uint16).  A is [m][r] row-major. */
int oracle_proxy_scores(const void* A, const void* q, int64_t m, int r, int dtype,
                        int round_bf16, float* out) {
  if (dtype != 0 && dtype != 1) return -1;
  float qf[1024];
  if (r > 1024 || r <= 0) return -2;
  for (int j = 0; j < r; ++j)
    qf[j] = dtype == 0 ? ((const float*)q)[j] : bf16_to_f32(((const uint16_t*)q)[j]);
  for (int64_t i = 0; i < m; ++i) {
    float acc = 0.0f;
    if (dtype == 0) {
      const float* row = (const float*)A + i * r;
      for (int j = 0; j < r; ++j) acc = fmaf(row[j], qf[j], acc);
    } else {
      const uint16_t* row = (const uint16_t*)A + i * r;
      for (int j = 0; j < r; ++j) acc = fmaf(bf16_to_f32(row[j]), qf[j], acc);
    }
    if (round_bf16) acc = round_to_bf16(acc);
    if (acc == 0.0f) acc = 0.0f; /* -0 -> +0 */
    out[i] = acc;
  }
  return 0;
}

typedef struct {
  uint32_t key;
  int32_t idx;
} kv_t;

static int cmp_desc_key_asc_idx(const void* a, const void* b) {
  const kv_t* x = (const kv_t*)a;
  const kv_t* y = (const kv_t*)b;
  if (x->key != y->key) return x->key > y->key ? -1 : 1;
  return x->idx < y->idx ? -1 : (x->idx > y->idx ? 1 : 0);
}

static int cmp_i32(const void* a, const void* b) {
  int32_t x = *(const int32_t*)a, y = *(const int32_t*)b;
  return x < y ? -1 : (x > y ? 1 : 0);
}

/* Full sort by (score desc, index asc), keep the first k, return them ascending.
 * m <= k returns arange(m) (lrqk_attention.py:1250-1258) and writes m entries. */
int64_t oracle_topk_sorted(const float* scores, int64_t m, int64_t k, int32_t* out_idx) {
  if (m <= k) {
    for (int64_t i = 0; i < m; ++i) out_idx[i] = (int32_t)i;
    return m;
  }
  kv_t* a = (kv_t*)malloc((size_t)m * sizeof(kv_t));
  if (!a) return -1;
  for (int64_t i = 0; i < m; ++i) {
    a[i].key = order_key(scores[i]);
    a[i].idx = (int32_t)i;
  }
  qsort(a, (size_t)m, sizeof(kv_t), cmp_desc_key_asc_idx);
  for (int64_t i = 0; i < k; ++i) out_idx[i] = a[i].idx;
  free(a);
  qsort(out_idx, (size_t)k, sizeof(int32_t), cmp_i32);
  return k;
}

/* The O(k^2) equality-matrix definition.  evict[i] = now[i] not in new;
 * missing[j] = new[j] not in now; updated = now with the evicted slots (ascending
 * slot) overwritten by the missing values (ascending position in new).
 * Returns the number of evicted slots, or -1 if the two counts differ (the
 * reference's boolean assignment would raise). */
int64_t oracle_only_indices(const int32_t* now, const int32_t* new_, int64_t k,
                            int32_t* updated, uint8_t* evict) {
  uint8_t* missing = (uint8_t*)malloc((size_t)k);
  if (!missing) return -2;
  int64_t n_evict = 0, n_missing = 0;
  for (int64_t i = 0; i < k; ++i) {
    int any = 0;
    for (int64_t j = 0; j < k; ++j) any |= (now[i] == new_[j]);
    evict[i] = (uint8_t)!any;
    n_evict += !any;
  }
  for (int64_t j = 0; j < k; ++j) {
    int any = 0;
    for (int64_t i = 0; i < k; ++i) any |= (now[i] == new_[j]);
    missing[j] = (uint8_t)!any;
    n_missing += !any;
  }
  if (n_evict != n_missing) {
    free(missing);
    return -1;
  }
  int64_t j = 0;
  for (int64_t i = 0; i < k; ++i) {
    updated[i] = now[i];
    if (evict[i]) {
      while (!missing[j]) ++j;
      updated[i] = new_[j++];
    }
  }
  free(missing);
  return n_evict;
}

/* indices/mask are [bsz][kv_heads][groups][k]; linear = (b*kv_heads + kv)*seq_len + idx
 * for the True entries in row-major order.  Returns the count. */
int64_t oracle_linear_indices(const int32_t* indices, const uint8_t* mask, int64_t bsz,
                              int64_t kv_heads, int64_t groups, int64_t k, int64_t seq_len,
                              int64_t* out) {
  int64_t n = 0;
  for (int64_t b = 0; b < bsz; ++b)
    for (int64_t h = 0; h < kv_heads; ++h)
      for (int64_t g = 0; g < groups; ++g)
        for (int64_t l = 0; l < k; ++l) {
          int64_t p = ((b * kv_heads + h) * groups + g) * k + l;
          if (mask[p]) out[n++] = (b * kv_heads + h) * seq_len + indices[p];
        }
  return n;
}

/* dst[i,:] = src[idx[i],:] with rows of row_bytes bytes. */
void oracle_d0_indices_select(void* dst, const void* src, const int64_t* idx, int64_t n,
                              int64_t row_bytes) {
  for (int64_t i = 0; i < n; ++i)
    memcpy((char*)dst + i * row_bytes, (const char*)src + idx[i] * row_bytes,
           (size_t)row_bytes);
}

/* src [bsz][kv_heads][seq_len][row], indices/mask [bsz][kv_heads][groups][k];
 * dst receives the masked rows in row-major mask order.  Returns the row count. */
int64_t oracle_take_along_dim_with_mask(const void* src, const int32_t* indices,
                                        const uint8_t* mask, int64_t bsz, int64_t kv_heads,
                                        int64_t groups, int64_t k, int64_t seq_len,
                                        int64_t row_bytes, void* dst) {
  int64_t n = 0;
  for (int64_t b = 0; b < bsz; ++b)
    for (int64_t h = 0; h < kv_heads; ++h) {
      const char* base = (const char*)src + (b * kv_heads + h) * seq_len * row_bytes;
      for (int64_t g = 0; g < groups; ++g)
        for (int64_t l = 0; l < k; ++l) {
          int64_t p = ((b * kv_heads + h) * groups + g) * k + l;
          if (mask[p]) {
            memcpy((char*)dst + n * row_bytes, base + (int64_t)indices[p] * row_bytes,
                   (size_t)row_bytes);
            ++n;
          }
        }
    }
  return n;
}
