// Hit/miss diff against the GPU-resident active set, miss fetch from the [K|V] store,
// on-device row gather, ring append and ring flush.
#include <algorithm>

#include "common.hpp"
#include "ctx.hpp"
#include "rows.hpp"

namespace lrqk {

// --------------------------------------------------------------------------- diff
// One workgroup per head.  new_idx is ascending and unique, so membership of a resident
// token is a binary search; a resident token that is found marks its position in new_idx
// as matched, which yields the missing tokens without sorting the resident set.  Both
// lists are then compacted in order, pairing the j-th evicted slot with the j-th missing
// token.
constexpr int kDiffThreads = 1024;

__global__ __launch_bounds__(kDiffThreads) void diff_kernel(const int32_t* __restrict__ new_all, int64_t new_stride,
                                                            int32_t* __restrict__ hit_all, int64_t hit_stride, int k,
                                                            uint8_t* __restrict__ evict_all,
                                                            int32_t* __restrict__ miss_slots_all,
                                                            int32_t* __restrict__ miss_count) {
  extern __shared__ __align__(16) unsigned char smem[];
  int32_t* new_s = reinterpret_cast<int32_t*>(smem);          // [k]
  int32_t* miss_s = new_s + k;                                 // [k] missing tokens, ascending
  uint8_t* matched = reinterpret_cast<uint8_t*>(miss_s + k);   // [k]
  uint8_t* evict_s = matched + k;                              // [k]
  __shared__ int scratch[kDiffThreads / kWave + 1];

  const int tid = threadIdx.x;
  const int h = blockIdx.x;
  const int32_t* nw = new_all + (int64_t)h * new_stride;
  int32_t* hit = hit_all + (int64_t)h * hit_stride;

  for (int i = tid; i < k; i += kDiffThreads) {
    new_s[i] = nw[i];
    matched[i] = 0;
  }
  __syncthreads();
  for (int s = tid; s < k; s += kDiffThreads) {
    const int32_t v = hit[s];
    int lo = 0, hi = k;
    while (lo < hi) {
      int mid = (lo + hi) >> 1;
      if (new_s[mid] < v) lo = mid + 1; else hi = mid;
    }
    const bool found = lo < k && new_s[lo] == v;
    if (found) matched[lo] = 1;
    evict_s[s] = found ? 0 : 1;
  }
  __syncthreads();
  // missing tokens in ascending order
  int n_missing = 0;
  for (int base = 0; base < k; base += kDiffThreads) {
    const int i = base + tid;
    const bool miss = i < k && matched[i] == 0;
    int tot;
    const int pos = block_rank(miss, scratch, tot);
    if (miss) miss_s[n_missing + pos] = new_s[i];
    n_missing += tot;
  }
  __syncthreads();
  // evicted slots in ascending order receive them
  int n_evict = 0;
  for (int base = 0; base < k; base += kDiffThreads) {
    const int s = base + tid;
    const bool ev = s < k && evict_s[s] != 0;
    int tot;
    const int pos = block_rank(ev, scratch, tot);
    const int j = n_evict + pos;
    if (ev && j < n_missing) {
      hit[s] = miss_s[j];
      if (miss_slots_all) miss_slots_all[(int64_t)h * k + j] = s;
    }
    if (s < k && evict_all) evict_all[(int64_t)h * k + s] = (ev && j < n_missing) ? 1 : 0;
    n_evict += tot;
  }
  if (tid == 0 && miss_count) miss_count[h] = n_evict < n_missing ? n_evict : n_missing;
}

// Ablation without the hit/miss bookkeeping: the resident set becomes the new selection
// (ascending) and every slot is refetched.
__global__ __launch_bounds__(256) void replace_all_kernel(const int32_t* __restrict__ new_all, int64_t new_stride,
                                                          int32_t* __restrict__ hit_all, int64_t hit_stride, int k,
                                                          uint8_t* __restrict__ evict_all,
                                                          int32_t* __restrict__ miss_slots_all,
                                                          int32_t* __restrict__ miss_count) {
  const int h = blockIdx.y;
  for (int s = blockIdx.x * blockDim.x + threadIdx.x; s < k; s += gridDim.x * blockDim.x) {
    hit_all[(int64_t)h * hit_stride + s] = new_all[(int64_t)h * new_stride + s];
    if (evict_all) evict_all[(int64_t)h * k + s] = 1;
    if (miss_slots_all) miss_slots_all[(int64_t)h * k + s] = s;
  }
  if (blockIdx.x == 0 && threadIdx.x == 0 && miss_count) miss_count[h] = k;
}

// --------------------------------------------------------------------------- row movers
// Rows are copied as 16-byte chunks; `cpr` chunks per K (or V) row.

__global__ __launch_bounds__(256) void fetch_rows_kernel(const uint4* __restrict__ store, int64_t cap,
                                                         uint4* __restrict__ k_act, uint4* __restrict__ v_act,
                                                         int n_slots, const int32_t* __restrict__ hit,
                                                         int64_t hit_stride, const int32_t* __restrict__ miss_slots,
                                                         const int32_t* __restrict__ miss_count, int hq, int hkv,
                                                         int cpr, int k) {
  fetch_rows_body(store, cap, k_act, v_act, n_slots, hit, hit_stride, miss_slots, miss_count, hq, hkv, cpr, k,
                  blockIdx.y, blockIdx.x, gridDim.x);
}

// dst[bh][j][:] = src[b][h/groups][idx[bh][j]][:]
__global__ __launch_bounds__(256) void gather_rows_kernel(const uint4* __restrict__ src, int64_t src_len,
                                                          const int32_t* __restrict__ idx, int64_t idx_stride,
                                                          int count, uint4* __restrict__ dst, int n_slots, int hq,
                                                          int hkv, int cpr) {
  const int h = blockIdx.y;
  const int b = h / hq, head = h % hq;
  const int kvh = head / (hq / hkv);
  const int64_t total = (int64_t)count * cpr;
  for (int64_t w = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; w < total; w += (int64_t)gridDim.x * blockDim.x) {
    const int j = (int)(w / cpr), c = (int)(w % cpr);
    const int32_t tok = idx[(int64_t)h * idx_stride + j];
    if (tok < 0 || tok >= src_len) continue;
    dst[((int64_t)h * n_slots + j) * cpr + c] = src[(((int64_t)b * hkv + kvh) * src_len + tok) * cpr + c];
  }
}

__global__ __launch_bounds__(256) void append_token_kernel(const uint4* __restrict__ k_new, const uint4* __restrict__ v_new,
                                                           uint4* __restrict__ k_act, uint4* __restrict__ v_act,
                                                           int n_slots, int slot, int32_t* __restrict__ active_idx,
                                                           int64_t idx_stride, int32_t token, int hq, int hkv, int cpr) {
  const int h = blockIdx.x;
  const int b = h / hq, head = h % hq;
  const int kvh = head / (hq / hkv);
  const int64_t src = ((int64_t)b * hkv + kvh) * cpr;
  const int64_t dst = ((int64_t)h * n_slots + slot) * cpr;
  for (int c = threadIdx.x; c < cpr; c += blockDim.x) {
    k_act[dst + c] = k_new[src + c];
    v_act[dst + c] = v_new[src + c];
  }
  if (threadIdx.x == 0 && active_idx) active_idx[(int64_t)h * idx_stride + slot] = token;
}

__global__ __launch_bounds__(256) void flush_ring_kernel(const uint4* __restrict__ k_act, const uint4* __restrict__ v_act,
                                                         int n_slots, int slot0, int count, uint4* __restrict__ store,
                                                         int64_t cap, int64_t row0, int hq, int hkv, int cpr) {
  const int bk = blockIdx.y;  // flattened (b, kv head)
  const int b = bk / hkv, kvh = bk % hkv;
  const int g = hq / hkv;
  const int64_t h = (int64_t)b * hq + (int64_t)kvh * g;  // first query head of the group
  const int chunks = 2 * cpr;
  const int64_t total = (int64_t)count * chunks;
  for (int64_t w = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; w < total; w += (int64_t)gridDim.x * blockDim.x) {
    const int s = (int)(w / chunks), c = (int)(w % chunks);
    const int64_t src = (h * n_slots + slot0 + s) * cpr;
    const uint4 val = c < cpr ? k_act[src + c] : v_act[src + c - cpr];
    store[((int64_t)bk * cap + row0 + s) * chunks + c] = val;
  }
}

static int check_rows(int b, int hq, int hkv, int d, int dtype, int* cpr) {
  LRQK_REQUIRE(dtype == LRQK_F32 || dtype == LRQK_BF16, LRQK_EINVAL, "dtype=%d", dtype);
  LRQK_REQUIRE(b > 0 && hq > 0 && hkv > 0 && hq % hkv == 0, LRQK_EINVAL, "bad heads b=%d hq=%d hkv=%d", b, hq, hkv);
  LRQK_REQUIRE((int64_t)b * hq <= 65535, LRQK_ELIMIT, "b*hq too large");
  const size_t row = (size_t)d * elem_size(dtype);
  LRQK_REQUIRE(d > 0 && row % 16 == 0, LRQK_EINVAL, "row of %zu bytes is not a multiple of 16", row);
  *cpr = (int)(row / 16);
  return LRQK_OK;
}

static bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

int resolve_store(const void* kv_store, const void** dev_store) {
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, kv_store) != hipSuccess) {
    (void)hipGetLastError();
    return set_error(LRQK_EINVAL, "kv_store is neither device memory nor pinned host memory");
  }
  *dev_store = kv_store;
  if (attr.type == hipMemoryTypeHost) {
    LRQK_REQUIRE(attr.devicePointer != nullptr, LRQK_EINVAL, "host store is not mapped into the device");
    *dev_store = attr.devicePointer;
  }
  return LRQK_OK;
}

}  // namespace lrqk

using namespace lrqk;

extern "C" int lrqk_diff(const int32_t* new_idx, int64_t new_stride, int32_t* hit, int64_t hit_stride, int bh, int k,
                         uint8_t* evict, int32_t* miss_slots, int32_t* miss_count, void* stream) {
  LRQK_REQUIRE(new_idx && hit, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(bh > 0 && bh <= 65535, LRQK_EINVAL, "bh=%d", bh);
  LRQK_REQUIRE(k > 0 && k <= LRQK_MAX_TOPK, LRQK_ELIMIT, "k=%d not in 1..%d", k, LRQK_MAX_TOPK);
  LRQK_REQUIRE(new_stride >= k && hit_stride >= k, LRQK_EINVAL, "stride smaller than k");
  const size_t smem = (size_t)k * 10;
  static std::atomic<bool> attr_set_dev[kMaxDeviceSlots];
  std::atomic<bool>& attr_set = attr_set_dev[per_device_slot()];
  if (smem > 48 * 1024 && !attr_set) {
    LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)diff_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       LRQK_MAX_TOPK * 10));
    attr_set = true;
  }
  hipLaunchKernelGGL(diff_kernel, dim3((unsigned)bh), dim3(kDiffThreads), smem, (hipStream_t)stream, new_idx,
                     new_stride, hit, hit_stride, k, evict, miss_slots, miss_count);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

extern "C" int lrqk_replace_all(const int32_t* new_idx, int64_t new_stride, int32_t* hit, int64_t hit_stride, int bh,
                                int k, uint8_t* evict, int32_t* miss_slots, int32_t* miss_count, void* stream) {
  LRQK_REQUIRE(new_idx && hit, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(bh > 0 && bh <= 65535 && k > 0, LRQK_EINVAL, "bad sizes bh=%d k=%d", bh, k);
  LRQK_REQUIRE(new_stride >= k && hit_stride >= k, LRQK_EINVAL, "stride smaller than k");
  hipLaunchKernelGGL(replace_all_kernel, dim3((unsigned)((k + 255) / 256), (unsigned)bh), dim3(256), 0,
                     (hipStream_t)stream, new_idx, new_stride, hit, hit_stride, k, evict, miss_slots, miss_count);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

extern "C" int lrqk_fetch_rows(const void* kv_store, int64_t cap, void* k_act, void* v_act, int n_slots,
                               const int32_t* hit, int64_t hit_stride, const int32_t* miss_slots,
                               const int32_t* miss_count, int b, int hq, int hkv, int d, int k, int dtype,
                               void* stream) {
  int cpr;
  int rc = check_rows(b, hq, hkv, d, dtype, &cpr);
  if (rc) return rc;
  LRQK_REQUIRE(kv_store && k_act && v_act && hit && miss_slots && miss_count, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(k > 0 && k <= n_slots && hit_stride >= k && cap > 0, LRQK_EINVAL, "bad sizes k=%d n_slots=%d", k, n_slots);
  const void* dev_store = nullptr;
  if ((rc = resolve_store(kv_store, &dev_store))) return rc;
  LRQK_REQUIRE(aligned16(dev_store) && aligned16(k_act) && aligned16(v_act), LRQK_EINVAL, "pointers must be 16-byte aligned");
  LRQK_REQUIRE(2 * cpr <= 256, LRQK_ELIMIT, "row of %d bytes too long", 2 * cpr * 16);
  const int rpb = 256 / (2 * cpr);
  dim3 grid((unsigned)std::min(256, (k + rpb - 1) / rpb), (unsigned)(b * hq));
  hipLaunchKernelGGL(fetch_rows_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const uint4*)dev_store, cap,
                     (uint4*)k_act, (uint4*)v_act, n_slots, hit, hit_stride, miss_slots, miss_count, hq, hkv, cpr, k);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

extern "C" int lrqk_gather_rows(const void* src, int64_t src_len, const int32_t* idx, int64_t idx_stride, int count,
                                void* dst, int n_slots, int b, int hq, int hkv, int d, int dtype, void* stream) {
  int cpr;
  int rc = check_rows(b, hq, hkv, d, dtype, &cpr);
  if (rc) return rc;
  LRQK_REQUIRE(src && idx && dst, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(count >= 0 && count <= n_slots && idx_stride >= count && src_len > 0, LRQK_EINVAL, "bad sizes");
  LRQK_REQUIRE(aligned16(src) && aligned16(dst), LRQK_EINVAL, "pointers must be 16-byte aligned");
  if (count == 0) return LRQK_OK;
  // src may be pinned host memory (the reference's host branch of fetch_by_hit): read through its mapping
  const void* dev_src = nullptr;
  rc = lrqk::resolve_store(src, &dev_src);
  if (rc) return rc;
  int64_t blocks = ((int64_t)count * cpr + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)blocks, (unsigned)(b * hq)), dim3(256), 0, (hipStream_t)stream,
                     (const uint4*)dev_src, src_len, idx, idx_stride, count, (uint4*)dst, n_slots, hq, hkv, cpr);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

extern "C" int lrqk_append_token(const void* k_new, const void* v_new, void* k_act, void* v_act, int n_slots, int slot,
                                 int32_t* active_idx, int64_t idx_stride, int32_t token, int b, int hq, int hkv, int d,
                                 int dtype, void* stream) {
  int cpr;
  int rc = check_rows(b, hq, hkv, d, dtype, &cpr);
  if (rc) return rc;
  LRQK_REQUIRE(k_new && v_new && k_act && v_act, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(slot >= 0 && slot < n_slots, LRQK_EINVAL, "slot=%d outside 0..%d", slot, n_slots);
  LRQK_REQUIRE(!active_idx || idx_stride > slot, LRQK_EINVAL, "idx_stride too small");
  LRQK_REQUIRE(aligned16(k_new) && aligned16(v_new) && aligned16(k_act) && aligned16(v_act), LRQK_EINVAL,
               "pointers must be 16-byte aligned");
  hipLaunchKernelGGL(append_token_kernel, dim3((unsigned)(b * hq)), dim3(64), 0, (hipStream_t)stream,
                     (const uint4*)k_new, (const uint4*)v_new, (uint4*)k_act, (uint4*)v_act, n_slots, slot, active_idx,
                     idx_stride, token, hq, hkv, cpr);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

extern "C" int lrqk_flush_ring(const void* k_act, const void* v_act, int n_slots, int slot0, int count, void* kv_store,
                               int64_t cap, int64_t row0, int b, int hq, int hkv, int d, int dtype, void* stream) {
  int cpr;
  int rc = check_rows(b, hq, hkv, d, dtype, &cpr);
  if (rc) return rc;
  LRQK_REQUIRE(k_act && v_act && kv_store, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(count > 0 && slot0 >= 0 && slot0 + count <= n_slots, LRQK_EINVAL, "slots %d..%d outside 0..%d", slot0,
               slot0 + count, n_slots);
  LRQK_REQUIRE(row0 >= 0 && row0 + count <= cap, LRQK_EINVAL, "rows %lld..%lld outside the store (cap %lld)",
               (long long)row0, (long long)(row0 + count), (long long)cap);
  void* dev_store = kv_store;
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, kv_store) == hipSuccess) {
    if (attr.type == hipMemoryTypeHost) {
      LRQK_REQUIRE(attr.devicePointer != nullptr, LRQK_EINVAL, "host store is not mapped into the device");
      dev_store = attr.devicePointer;
    }
  } else {
    (void)hipGetLastError();
    return set_error(LRQK_EINVAL, "kv_store is neither device memory nor pinned host memory");
  }
  LRQK_REQUIRE(aligned16(dev_store) && aligned16(k_act) && aligned16(v_act), LRQK_EINVAL, "pointers must be 16-byte aligned");
  int64_t blocks = ((int64_t)count * 2 * cpr + 255) / 256;
  if (blocks > 1024) blocks = 1024;
  hipLaunchKernelGGL(flush_ring_kernel, dim3((unsigned)blocks, (unsigned)(b * hkv)), dim3(256), 0, (hipStream_t)stream,
                     (const uint4*)k_act, (const uint4*)v_act, n_slots, slot0, count, (uint4*)dev_store, cap, row0, hq,
                     hkv, cpr);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}
