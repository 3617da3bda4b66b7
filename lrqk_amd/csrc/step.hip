// One decode step of one layer as a single host call: ring append (+ flush), factor
// update, proxy-score scan + top-k, hit/miss diff, miss fetch and (optionally) the exact
// attention over the active set.  Only launches; never synchronises.
#include "common.hpp"
#include "ctx.hpp"

using namespace lrqk;

extern "C" int lrqk_decode_step(lrqk_ctx* ctx, void* b_q, void* b_k, void* a_k, int64_t head_stride,
                                int32_t* active_idx, void* k_act, void* v_act, void* kv_store, int64_t cap,
                                const void* q, const void* k_new, const void* v_new, int b, int hq, int hkv, int r, int d,
                                int topk, int lite, int ring_slot, int32_t token, int64_t m, int64_t flush_row0,
                                int max_iter, float tol, int round_scores, int no_hit_miss, void* q_hat, void* k_hat,
                                void* attn_out, uint8_t* evict, int32_t* miss_count, int dtype, void* stream) {
  LRQK_REQUIRE(ctx != nullptr, LRQK_EINVAL, "ctx is null");
  LRQK_REQUIRE(topk > 0 && lite > 0 && ring_slot >= 0 && ring_slot < lite, LRQK_EINVAL, "bad ring slot %d of %d", ring_slot,
               lite);
  LRQK_REQUIRE(m >= topk, LRQK_EINVAL, "m=%lld < topk=%d: the main decode branch needs at least topk candidates",
               (long long)m, topk);
  const int bh = b * hq;
  const int n = topk + lite;
  int rc;
  ctx->fin_pending = ctx->qhat_pending = ctx->kq_valid = false;  // nothing survives a call that failed half-way
  ctx->sidx_rows_hint = token;                   // rows [0, token) of A_K exist before this step
  if ((rc = ctx->new_idx.ensure((size_t)bh * topk * sizeof(int32_t)))) return rc;
  // misc: miss_slots i32 [bh][topk] | miss_count i32 [bh] | miss_old i32 [bh][topk] | miss_new i32 [bh][topk] |
  // evict u8 [bh][topk]
  if ((rc = ctx->misc.ensure((size_t)bh * topk * 13 + (size_t)bh * 4 + 64))) return rc;
  int32_t* new_idx = (int32_t*)ctx->new_idx.p;
  int32_t* miss_slots = (int32_t*)ctx->misc.p;
  int32_t* mcount = miss_count ? miss_count : miss_slots + (size_t)bh * topk;
  int32_t* miss_old = miss_slots + (size_t)bh * topk + bh;
  int32_t* miss_new = miss_old + (size_t)bh * topk;
  uint8_t* ev = evict ? evict : (uint8_t*)(miss_new + (size_t)bh * topk);

  // The finish stage of the factor update (B update, outputs, A_K row) is off the critical path: when
  // the step ends with the fetch + attention launch it rides there, and the scan takes the proxy
  // query from the iterates directly.  Any path that cannot absorb it flushes it as its own launch.
  // (a [K|V] row must fit the lanes of one wave for the fetch role to form its attention term)
  // (without attn_out the same launch runs with its fetch, finish and index roles only)
  const bool fused_tail = !no_hit_miss && ctx->fetch_mode == 0 && 2 * (size_t)d * elem_size(dtype) / 16 <= (size_t)kWave;
  const bool defer_finish = fused_tail;
  // ring append folded into the first kernel of the factor update; the flush of a full ring
  // (which reads the slot just written) follows it
  if ((rc = als_decode_append(ctx, b_q, b_k, a_k, head_stride, active_idx, n, k_act, v_act, n, q, k_new, v_new, b, hq, hkv,
                              r, d, max_iter, tol, q_hat, k_hat, token, topk + ring_slot, token, defer_finish,
                              dtype, (hipStream_t)stream)))
    return rc;
  if (flush_row0 >= 0) {
    if ((rc = lrqk_flush_ring(k_act, v_act, n, topk, lite, kv_store, cap, flush_row0, b, hq, hkv, d, dtype, stream)))
      return rc;
  }
  // victim cache (only on the fused tail, and only while the diff runs inside the select kernel)
  const int row_chunks = (int)(2 * (size_t)d * elem_size(dtype) / 16);
  if (fused_tail) {
    if ((rc = victim_prepare(ctx, bh, cap, row_chunks, (hipStream_t)stream))) return rc;
  }
  const VictimView* vic = fused_tail && ctx->vic.nv > 0 && !ctx->vic_dirty ? &ctx->vic : nullptr;
  rc = score_select_diff(ctx, a_k, head_stride, q_hat, bh, m, r, topk, dtype, round_scores, new_idx, active_idx, n, ev,
                         miss_slots, mcount, no_hit_miss, (hipStream_t)stream, miss_old, vic, miss_new,
                         /*want_new_idx=*/false);
  const bool fused_diff = rc == 1;  // the select kernel also wrote miss_old / miss_new
  const bool vic_active = vic != nullptr && fused_diff;
  if (rc < 0) return rc;
  if (ctx->qhat_pending) {  // no scan took the iterate over (cannot happen on the paths above; kept as a guard)
    int rcf = flush_pending_finish(ctx, (hipStream_t)stream);
    if (rcf) return rcf;
  }
  if (rc == 0) {  // sizes outside the fused kernel's LDS budget: separate diff launch
    if (no_hit_miss)
      rc = lrqk_replace_all(new_idx, topk, active_idx, n, bh, topk, ev, miss_slots, mcount, stream);
    else
      rc = lrqk_diff(new_idx, topk, active_idx, n, bh, topk, ev, miss_slots, mcount, stream);
    if (rc) return rc;
  }
  if (!fused_tail) {
    int rcf = flush_pending_finish(ctx, (hipStream_t)stream);
    if (rcf) return rcf;
  }
  if (ctx->fetch_mode == 1) {
    if ((rc = lrqk_fetch_rows_staged(ctx, kv_store, cap, k_act, v_act, n, active_idx, n, miss_slots, mcount, b, hq, hkv,
                                     d, topk, dtype, stream)))
      return rc;
    if (attn_out) return lrqk_attention(ctx, q, k_act, v_act, n, n, attn_out, bh, d, dtype, stream);
    return LRQK_OK;
  }
  if (fused_tail) {
    // the fetch is bound by the host link: the attention over the resident slots runs beside it
    return fetch_attention(ctx, kv_store, cap, k_act, v_act, n, active_idx, n, miss_slots, mcount, ev, b, hq, hkv, d,
                           topk, q, attn_out, dtype, (hipStream_t)stream, miss_old, vic_active ? vic : nullptr,
                           fused_diff ? miss_new : nullptr);
  }
  if ((rc = lrqk_fetch_rows(kv_store, cap, k_act, v_act, n, active_idx, n, miss_slots, mcount, b, hq, hkv, d, topk, dtype,
                            stream)))
    return rc;
  if (attn_out) {
    if ((rc = lrqk_attention(ctx, q, k_act, v_act, n, n, attn_out, bh, d, dtype, stream))) return rc;
  }
  return LRQK_OK;
}
