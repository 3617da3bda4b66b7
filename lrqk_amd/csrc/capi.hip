// Host-only part of the C ABI: error text, workspace lifetime, and the multi-threaded
// host row gathers that carry the signatures of the reference's native extension.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <thread>
#include <vector>

#include "common.hpp"
#include "ctx.hpp"
#include "hostpar.hpp"

namespace lrqk {

static thread_local char g_err[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

}  // namespace lrqk

using namespace lrqk;

extern "C" int lrqk_version(void) { return 1; }

extern "C" const char* lrqk_last_error(void) { return g_err; }

extern "C" int lrqk_ctx_create(lrqk_ctx** out) {
  LRQK_REQUIRE(out != nullptr, LRQK_EINVAL, "out is null");
  *out = new lrqk_ctx();
  return LRQK_OK;
}

extern "C" int lrqk_ctx_destroy(lrqk_ctx* ctx) {
  if (!ctx) return LRQK_OK;
  (void)hipDeviceSynchronize();
  ctx->keys.release();
  ctx->hist.release();
  ctx->cand.release();
  ctx->cand_cnt.release();
  ctx->attn_part.release();
  ctx->als_part.release();
  ctx->als_pre.release();
  ctx->als_kq.release();
  ctx->als_iter.release();
  ctx->als_iter64.release();
  ctx->fstate.release();
  ctx->evk.release();
  ctx->prefill_ws.release();
  ctx->prefill_gd.release();
  ctx->new_idx.release();
  ctx->misc.release();
  ctx->stage_dev.release();
  ctx->vic_rows.release();
  ctx->sidx_qa.release();
  ctx->sidx_qs.release();
  ctx->sidx_wm.release();
  ctx->sidx_part.release();
  ctx->vic_meta.release();
  if (ctx->stage_host) (void)hipHostFree(ctx->stage_host);
  if (ctx->stage_ev) (void)hipEventDestroy(ctx->stage_ev);
  if (ctx->side) (void)hipStreamDestroy(ctx->side);
  if (ctx->tev) {
    for (int i = 0; i < 2 * ctx->tev_pairs; ++i) (void)hipEventDestroy(ctx->tev[i]);
    delete[] ctx->tev;
  }
  delete ctx;
  return LRQK_OK;
}

extern "C" int lrqk_ctx_reserve(lrqk_ctx* ctx, int bh, int64_t max_tokens, int topk, int n_active, int r, int d) {
  LRQK_REQUIRE(ctx != nullptr, LRQK_EINVAL, "ctx is null");
  LRQK_REQUIRE(bh > 0 && max_tokens >= 0 && topk > 0 && n_active > 0 && r > 0 && d > 0, LRQK_EINVAL, "bad sizes");
  int rc;
  const int64_t key_stride = (max_tokens + 63) & ~(int64_t)63;
  if ((rc = ctx->keys.ensure((size_t)bh * key_stride * 4))) return rc;
  if ((rc = ctx->attn_part.ensure((size_t)bh * 64 * (d + 2) * sizeof(float)))) return rc;
  // (partial sums of the factor update: up to 32 splits of r x r + r sums, r padded to one or two matrix-core tiles)
  const size_t tile_r = r > 32 ? 64 : 32;
  if ((rc = ctx->als_part.ensure((size_t)bh * 32 * (tile_r * tile_r + tile_r) * sizeof(float)))) return rc;
  if ((rc = ctx->als_kq.ensure((size_t)bh * n_active * sizeof(float)))) return rc;
  if ((rc = ctx->als_iter.ensure((size_t)bh * LRQK_MAX_DECODE_ITERS * (2 * r + 1) * sizeof(float)))) return rc;
  if ((rc = ctx->new_idx.ensure((size_t)bh * topk * sizeof(int32_t)))) return rc;
  if ((rc = ctx->misc.ensure((size_t)bh * topk * 13 + (size_t)bh * 4 + 64))) return rc;  // (as lrqk_decode_step sizes it)
  return LRQK_OK;
}

extern "C" int lrqk_select_stats_detail(lrqk_ctx* ctx, int* list_short, int* list_overflow) {
  LRQK_REQUIRE(ctx && list_short && list_overflow, LRQK_EINVAL, "null pointer");
  *list_short = ctx->last_short;
  *list_overflow = ctx->last_overflow;
  return LRQK_OK;
}

extern "C" int lrqk_timing_enable(lrqk_ctx* ctx, int max_launches) {
  LRQK_REQUIRE(ctx != nullptr && max_launches >= 0 && max_launches <= (1 << 20), LRQK_EINVAL, "bad arguments");
  if (ctx->tev) {
    LRQK_HIP_CHECK(hipDeviceSynchronize());
    for (int i = 0; i < 2 * ctx->tev_pairs; ++i) (void)hipEventDestroy(ctx->tev[i]);
    delete[] ctx->tev;
    ctx->tev = nullptr;
  }
  ctx->tev_pairs = ctx->tev_used = ctx->tev_seen = 0;
  if (max_launches == 0) return LRQK_OK;
  ctx->tev = new hipEvent_t[2 * (size_t)max_launches];
  for (int i = 0; i < 2 * max_launches; ++i) LRQK_HIP_CHECK(hipEventCreate(&ctx->tev[i]));
  ctx->tev_pairs = max_launches;
  return LRQK_OK;
}

extern "C" int lrqk_timing_stride(lrqk_ctx* ctx, int every) {
  LRQK_REQUIRE(ctx != nullptr && every >= 1, LRQK_EINVAL, "bad arguments");
  ctx->tev_every = every;
  ctx->tev_seen = 0;
  return LRQK_OK;
}

extern "C" int lrqk_timing_read(lrqk_ctx* ctx, double* total_ms, int* launches) {
  LRQK_REQUIRE(ctx && total_ms && launches, LRQK_EINVAL, "null pointer");
  double sum = 0.0;
  for (int i = 0; i < ctx->tev_used; ++i) {
    LRQK_HIP_CHECK(hipEventSynchronize(ctx->tev[2 * i + 1]));
    float ms = 0.0f;
    LRQK_HIP_CHECK(hipEventElapsedTime(&ms, ctx->tev[2 * i], ctx->tev[2 * i + 1]));
    sum += ms;
  }
  *total_ms = sum;
  *launches = ctx->tev_used;
  ctx->tev_used = 0;
  return LRQK_OK;
}

extern "C" int lrqk_d0_indices_select(void* dst, const void* src, const int64_t* idx, int64_t n, int64_t row_bytes,
                                      int64_t src_rows, int threads) {
  LRQK_REQUIRE(n >= 0 && row_bytes > 0, LRQK_EINVAL, "bad sizes n=%lld row_bytes=%lld", (long long)n, (long long)row_bytes);
  if (n == 0) return LRQK_OK;
  LRQK_REQUIRE(dst && src && idx, LRQK_EINVAL, "null pointer");
  for (int64_t i = 0; i < n; ++i)
    LRQK_REQUIRE(idx[i] >= 0 && idx[i] < src_rows, LRQK_EINVAL, "index %lld at %lld outside 0..%lld", (long long)idx[i],
                 (long long)i, (long long)src_rows);
  parallel_ranges(n, threads, 4096, [&](int64_t lo, int64_t hi) {
    for (int64_t i = lo; i < hi; ++i)
      memcpy((char*)dst + i * row_bytes, (const char*)src + idx[i] * row_bytes, (size_t)row_bytes);
  });
  return LRQK_OK;
}

extern "C" int64_t lrqk_take_along_dim_with_mask(void* dst, const void* src, const int64_t* indices,
                                                 const uint8_t* mask, int64_t b, int64_t hkv, int64_t groups, int64_t k,
                                                 int64_t seq, int64_t row_bytes, int threads) {
  LRQK_REQUIRE(b > 0 && hkv > 0 && groups > 0 && k > 0 && seq > 0 && row_bytes > 0, LRQK_EINVAL, "bad sizes");
  LRQK_REQUIRE(indices && mask, LRQK_EINVAL, "null pointer");
  const int64_t nbh = b * hkv, per = groups * k;
  std::vector<int64_t> offs((size_t)nbh + 1, 0);
  for (int64_t p = 0; p < nbh; ++p) {
    int64_t c = 0;
    for (int64_t e = 0; e < per; ++e) {
      if (mask[p * per + e]) {
        const int64_t t = indices[p * per + e];
        LRQK_REQUIRE(t >= 0 && t < seq, LRQK_EINVAL, "index %lld outside 0..%lld", (long long)t, (long long)seq);
        ++c;
      }
    }
    offs[(size_t)p + 1] = offs[(size_t)p] + c;
  }
  const int64_t total = offs[(size_t)nbh];
  if (!dst || total == 0) return total;
  LRQK_REQUIRE(src != nullptr, LRQK_EINVAL, "src is null");
  parallel_ranges(nbh, threads, 1, [&](int64_t lo, int64_t hi) {
    for (int64_t p = lo; p < hi; ++p) {
      char* out = (char*)dst + offs[(size_t)p] * row_bytes;
      const char* base = (const char*)src + p * seq * row_bytes;
      for (int64_t e = 0; e < per; ++e) {
        if (mask[p * per + e]) {
          memcpy(out, base + indices[p * per + e] * row_bytes, (size_t)row_bytes);
          out += row_bytes;
        }
      }
    }
  });
  return total;
}
