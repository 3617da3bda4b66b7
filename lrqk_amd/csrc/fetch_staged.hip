// Miss fetch through a staging buffer, the way the reference does it: the miss list is
// brought to the host, the host gathers the missed [K|V] rows of the pinned store into a
// pinned staging block, one hipMemcpyAsync on a side stream moves the block, and a kernel
// scatters it into the active-set slots.  The main stream waits on an event, not the host.
// (The default path lets the fetch kernel read the pinned store directly and needs none of
// this; the staged path exists for stores that are not mapped into the device and as the
// measured alternative.)
#include <string.h>

#include "common.hpp"
#include "ctx.hpp"
#include "hostpar.hpp"

namespace lrqk {

// tok[bh][k]: token of the j-th refetched slot (j < miss_count[h]), so that one copy tells the host everything
__global__ __launch_bounds__(256) void miss_tokens_kernel(const int32_t* __restrict__ hit, int64_t hit_stride,
                                                          const int32_t* __restrict__ miss_slots,
                                                          const int32_t* __restrict__ miss_count, int k,
                                                          int32_t* __restrict__ tok) {
  const int h = blockIdx.y;
  const int cnt = miss_count[h];
  for (int j = blockIdx.x * blockDim.x + threadIdx.x; j < cnt; j += gridDim.x * blockDim.x) {
    const int slot = miss_slots[(int64_t)h * k + j];
    tok[(int64_t)h * k + j] = (slot >= 0 && slot < k) ? hit[(int64_t)h * hit_stride + slot] : -1;
  }
}

// stage: rows of 2*cpr 16-byte chunks, head h's rows start at row offs[h]
__global__ __launch_bounds__(256) void scatter_rows_kernel(const uint4* __restrict__ stage,
                                                           const int32_t* __restrict__ offs,
                                                           const int32_t* __restrict__ miss_slots,
                                                           const int32_t* __restrict__ miss_count, int k, int cpr,
                                                           uint4* __restrict__ k_act, uint4* __restrict__ v_act,
                                                           int n_slots) {
  const int h = blockIdx.y;
  const int cnt = miss_count[h];
  const int chunks = 2 * cpr;
  const int64_t base = offs[h];
  for (int w = blockIdx.x * blockDim.x + threadIdx.x; w < cnt * chunks; w += gridDim.x * blockDim.x) {
    const int j = w / chunks, c = w % chunks;
    const int slot = miss_slots[(int64_t)h * k + j];
    if (slot < 0 || slot >= k) continue;
    const uint4 val = stage[(base + j) * chunks + c];
    const int64_t dst = ((int64_t)h * n_slots + slot) * cpr;
    if (c < cpr) k_act[dst + c] = val; else v_act[dst + (c - cpr)] = val;
  }
}

static int ensure_stage(lrqk_ctx* ctx, size_t bytes) {
  if (!ctx->side) LRQK_HIP_CHECK(hipStreamCreateWithFlags(&ctx->side, hipStreamNonBlocking));
  if (!ctx->stage_ev) LRQK_HIP_CHECK(hipEventCreateWithFlags(&ctx->stage_ev, hipEventDisableTiming));
  if (bytes > ctx->stage_host_bytes) {
    if (ctx->stage_host) {
      LRQK_HIP_CHECK(hipDeviceSynchronize());
      LRQK_HIP_CHECK(hipHostFree(ctx->stage_host));
      ctx->stage_host = nullptr;
      ctx->stage_host_bytes = 0;
    }
    const size_t want = bytes + bytes / 4;
    LRQK_HIP_CHECK(hipHostMalloc(&ctx->stage_host, want, hipHostMallocDefault));
    ctx->stage_host_bytes = want;
  }
  return ctx->stage_dev.ensure(bytes);
}

}  // namespace lrqk

using namespace lrqk;

extern "C" int lrqk_ctx_set_fetch_mode(lrqk_ctx* ctx, int mode, int host_threads) {
  LRQK_REQUIRE(ctx != nullptr, LRQK_EINVAL, "ctx is null");
  LRQK_REQUIRE(mode == 0 || mode == 1, LRQK_EINVAL, "mode=%d (0 = direct, 1 = staged)", mode);
  ctx->fetch_mode = mode;
  if (host_threads > 0) ctx->host_threads = host_threads;
  return LRQK_OK;
}

extern "C" int lrqk_fetch_rows_staged(lrqk_ctx* ctx, const void* kv_store, int64_t cap, void* k_act, void* v_act,
                                      int n_slots, const int32_t* hit, int64_t hit_stride, const int32_t* miss_slots,
                                      const int32_t* miss_count, int b, int hq, int hkv, int d, int k, int dtype,
                                      void* stream) {
  LRQK_REQUIRE(ctx && kv_store && k_act && v_act && hit && miss_slots && miss_count, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(dtype == LRQK_F32 || dtype == LRQK_BF16, LRQK_EINVAL, "dtype=%d", dtype);
  LRQK_REQUIRE(b > 0 && hq > 0 && hkv > 0 && hq % hkv == 0 && d > 0, LRQK_EINVAL, "bad heads b=%d hq=%d hkv=%d", b, hq, hkv);
  const size_t row_bytes = (size_t)2 * d * elem_size(dtype);
  LRQK_REQUIRE((d * elem_size(dtype)) % 16 == 0, LRQK_ELIMIT, "row of %zu bytes is not a multiple of 16", row_bytes / 2);
  LRQK_REQUIRE(k > 0 && k <= n_slots && hit_stride >= k && cap > 0, LRQK_EINVAL, "bad sizes k=%d n_slots=%d", k, n_slots);
  LRQK_REQUIRE(((uintptr_t)k_act % 16 == 0) && ((uintptr_t)v_act % 16 == 0), LRQK_EINVAL, "pointers must be 16-byte aligned");
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, kv_store) != hipSuccess || attr.type != hipMemoryTypeHost) {
    (void)hipGetLastError();
    return set_error(LRQK_EINVAL, "the staged fetch reads the store on the host: kv_store must be pinned host memory");
  }
  const char* host_store = (const char*)(attr.hostPointer ? attr.hostPointer : kv_store);
  hipStream_t st = (hipStream_t)stream;
  const int bh = b * hq;
  const int cpr = (int)(d * elem_size(dtype) / 16);
  // staging block: [bh] row offsets (padded to 16 B) then up to bh*k rows; host header: counts + tokens
  const size_t offs_bytes = ((size_t)bh * 4 + 15) & ~(size_t)15;
  const size_t rows_max = (size_t)bh * k * row_bytes;
  const size_t hdr_bytes = ((size_t)bh * 4 + (size_t)bh * k * 4 + 15) & ~(size_t)15;
  int rc = ensure_stage(ctx, hdr_bytes + offs_bytes + rows_max);
  if (rc) return rc;
  char* sh = (char*)ctx->stage_host;
  char* sd = (char*)ctx->stage_dev.p;
  int32_t* d_cnt = (int32_t*)sd;             // device copy area for the header (counts, tokens)
  int32_t* d_tok = d_cnt + bh;
  int32_t* h_cnt = (int32_t*)sh;
  int32_t* h_tok = h_cnt + bh;

  // 1. miss list to the host (one copy; the only host wait of the step)
  LRQK_HIP_CHECK(hipMemcpyAsync(d_cnt, miss_count, (size_t)bh * 4, hipMemcpyDeviceToDevice, st));
  hipLaunchKernelGGL(miss_tokens_kernel, dim3((unsigned)((k + 255) / 256), (unsigned)bh), dim3(256), 0, st, hit,
                     hit_stride, miss_slots, miss_count, k, d_tok);
  LRQK_HIP_CHECK(hipGetLastError());
  LRQK_HIP_CHECK(hipMemcpyAsync(h_cnt, d_cnt, (size_t)bh * 4 + (size_t)bh * k * 4, hipMemcpyDeviceToHost, st));
  LRQK_HIP_CHECK(hipStreamSynchronize(st));

  // 2. host gather into the pinned staging block (cpp_kernel/take_along_dim_grouped.cpp:13-124 in spirit)
  int32_t* h_offs = (int32_t*)(sh + hdr_bytes);
  char* h_rows = sh + hdr_bytes + offs_bytes;
  int64_t total = 0;
  for (int h = 0; h < bh; ++h) {
    LRQK_REQUIRE(h_cnt[h] >= 0 && h_cnt[h] <= k, LRQK_EINVAL, "miss_count[%d]=%d outside 0..%d", h, h_cnt[h], k);
    h_offs[h] = (int32_t)total;
    total += h_cnt[h];
  }
  bool bad = false;
  parallel_ranges(bh, ctx->host_threads, 1, [&](int64_t lo, int64_t hi) {
    for (int64_t h = lo; h < hi; ++h) {
      const int bb = (int)(h / hq), kvh = (int)((h % hq) / (hq / hkv));
      const char* src = host_store + ((int64_t)bb * hkv + kvh) * cap * row_bytes;
      char* dst = h_rows + (int64_t)h_offs[h] * row_bytes;
      for (int j = 0; j < h_cnt[h]; ++j) {
        const int32_t t = h_tok[h * (int64_t)k + j];
        if (t < 0 || t >= cap) {
          if (t >= cap) bad = true;
          memset(dst + (int64_t)j * row_bytes, 0, row_bytes);
          continue;
        }
        memcpy(dst + (int64_t)j * row_bytes, src + (int64_t)t * row_bytes, row_bytes);
      }
    }
  });
  LRQK_REQUIRE(!bad, LRQK_EINVAL, "a missed token id lies beyond the store capacity %lld", (long long)cap);

  // 3. one asynchronous copy on the side stream; the main stream waits for its event
  const size_t copy_bytes = offs_bytes + (size_t)total * row_bytes;
  LRQK_HIP_CHECK(hipMemcpyAsync(sd + hdr_bytes, sh + hdr_bytes, copy_bytes, hipMemcpyHostToDevice, ctx->side));
  LRQK_HIP_CHECK(hipEventRecord(ctx->stage_ev, ctx->side));
  LRQK_HIP_CHECK(hipStreamWaitEvent(st, ctx->stage_ev, 0));

  // 4. scatter into the slots
  if (total > 0) {
    hipLaunchKernelGGL(scatter_rows_kernel, dim3(16, (unsigned)bh), dim3(256), 0, st,
                       (const uint4*)(sd + hdr_bytes + offs_bytes), (const int32_t*)(sd + hdr_bytes), miss_slots,
                       miss_count, k, cpr, (uint4*)k_act, (uint4*)v_act, n_slots);
    LRQK_HIP_CHECK(hipGetLastError());
  }
  return LRQK_OK;
}
