// Host side of the victim cache: sizing, (re)initialisation, statistics.
#include <vector>

#include "common.hpp"
#include "ctx.hpp"

namespace lrqk {

__global__ __launch_bounds__(256) void victim_init_kernel(int32_t* tok, int64_t n_tok, int16_t* pos, int64_t n_pos,
                                                          int32_t* counters, int n_counters) {
  const int64_t i0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = i0; i < n_tok; i += stride) tok[i] = -1;
  for (int64_t i = i0; i < n_pos; i += stride) pos[i] = -1;
  for (int64_t i = i0; i < n_counters; i += stride) counters[i] = 0;
}

int victim_prepare(lrqk_ctx* ctx, int bh, int64_t cap, int chunks, hipStream_t st) {
  if (ctx->vic_req <= 0) {
    ctx->vic.nv = 0;
    return LRQK_OK;
  }
  const int nv = ctx->vic_req;
  const bool same = ctx->vic.nv == nv && ctx->vic_bh == bh && ctx->vic.cap == cap && ctx->vic_chunks == chunks;
  if (same && !ctx->vic_dirty) return LRQK_OK;
  int rc;
  if ((rc = ctx->vic_rows.ensure((size_t)bh * nv * chunks * sizeof(uint4)))) return rc;
  // meta: tok i32 [bh][nv] | counters i32 [3][bh] (ptr, base, host_rows) | pos i16 [bh][cap]
  const size_t n_tok = (size_t)bh * nv, n_cnt = (size_t)3 * bh, n_pos = (size_t)bh * cap;
  if ((rc = ctx->vic_meta.ensure((n_tok + n_cnt) * 4 + n_pos * 2 + 16))) return rc;
  VictimView v{};
  v.rows = (uint4*)ctx->vic_rows.p;
  v.tok = (int32_t*)ctx->vic_meta.p;
  v.ptr = v.tok + n_tok;
  v.base = v.ptr + bh;
  v.host_rows = v.base + bh;
  v.pos = (int16_t*)(v.host_rows + bh);
  v.nv = nv;
  v.cap = cap;
  hipLaunchKernelGGL(victim_init_kernel, dim3(512), dim3(256), 0, st, v.tok, (int64_t)n_tok, v.pos, (int64_t)n_pos, v.ptr,
                     (int)n_cnt);
  LRQK_HIP_CHECK(hipGetLastError());
  ctx->vic = v;
  ctx->vic_bh = bh;
  ctx->vic_chunks = chunks;
  ctx->vic_dirty = false;
  return LRQK_OK;
}

}  // namespace lrqk

using namespace lrqk;

extern "C" int lrqk_ctx_victim_cache(lrqk_ctx* ctx, int rows_per_head) {
  LRQK_REQUIRE(ctx != nullptr, LRQK_EINVAL, "ctx is null");
  LRQK_REQUIRE(rows_per_head >= 0 && rows_per_head <= 32767, LRQK_EINVAL, "rows_per_head=%d not in 0..32767",
               rows_per_head);
  ctx->vic_req = rows_per_head;
  ctx->vic_dirty = true;  // contents are dropped: the next step starts from an empty cache
  if (rows_per_head == 0) ctx->vic.nv = 0;
  return LRQK_OK;
}

extern "C" int lrqk_victim_stats(lrqk_ctx* ctx, int64_t* host_rows, int reset) {
  LRQK_REQUIRE(ctx && host_rows, LRQK_EINVAL, "null pointer");
  *host_rows = 0;
  if (ctx->vic.nv <= 0 || ctx->vic_dirty || ctx->vic_bh <= 0) return LRQK_OK;
  std::vector<int32_t> v((size_t)ctx->vic_bh);
  LRQK_HIP_CHECK(hipMemcpy(v.data(), ctx->vic.host_rows, v.size() * 4, hipMemcpyDeviceToHost));
  for (int32_t x : v) *host_rows += x;
  if (reset) LRQK_HIP_CHECK(hipMemset(ctx->vic.host_rows, 0, v.size() * 4));
  return LRQK_OK;
}
