// One decode step of one layer as a single host call: ring append (+ flush), factor
// update, proxy-score scan + top-k, hit/miss diff, miss fetch and (optionally) the exact
// attention over the active set.  Only launches; never synchronises.
#include "common.hpp"
#include <algorithm>

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
  // (the counts stay in the library's own block: a launch that reads them may run after the caller has let go
  // of its buffer; the caller's copy is written by the step's last launch, or the kernels use its buffer directly)
  int32_t* mcount_own = miss_slots + (size_t)bh * topk;
  int32_t* mcount = miss_count ? miss_count : mcount_own;
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
  // The factor update from kept state (als_state.hip, if the ctx has it switched on): one small launch before the
  // scan, and after the fetch one launch that brings the state up to date.  It needs the replaced tokens listed
  // (the select kernel's own diff) and the fused tail; every other path runs the update over the active rows, and
  // leaves the kept state invalid.
  const bool quick = fused_tail && ctx->fs_enabled && m > topk && topk <= kStepFusedDiffMaxK &&
                     factor_state_supported(r, d, dtype, max_iter) && (int64_t)b * hq <= 65535;
  if (quick) {
    mcount = mcount_own;
    const bool valid = ctx->fs_valid && ctx->fstate.p && ctx->fs_bq == b_q && ctx->fs_bk == b_k && ctx->fs_ak == a_k &&
                       ctx->fs_kact == k_act && ctx->fs_idx == active_idx && ctx->fs_head_stride == head_stride &&
                       ctx->fs_bh == bh && ctx->fs_r == r && ctx->fs_d == d && ctx->fs_dtype == dtype &&
                       ctx->fs_topk == topk && ctx->fs_n == n && ctx->fs_next_slot == topk + ring_slot &&
                       ctx->fs_next_token == token;
    ctx->fs_valid = false;  // until this step has brought it up to date
    const int evk_rows = std::min(topk, std::max(256, topk / 2));
    if ((rc = ctx->evk.ensure((size_t)bh * evk_rows * d * elem_size(dtype)))) return rc;
    ctx->evk_rows = evk_rows;
    if (!valid) {
      if ((rc = factor_state_rebuild(ctx, b_q, b_k, a_k, head_stride, active_idx, n, k_act, n, bh, r, d, topk,
                                     topk + ring_slot, dtype, (hipStream_t)stream)))
        return rc;
    }
    if ((rc = factor_state_quick(ctx, b_q, b_k, a_k, head_stride, active_idx, n, k_act, v_act, n, q, k_new, v_new, b, hq,
                                 hkv, r, d, max_iter, tol, q_hat, k_hat, token, topk + ring_slot, token, dtype,
                                 (hipStream_t)stream)))
      return rc;
  } else {
    ctx->fs_valid = false;
    // ring append folded into the first kernel of the factor update; the flush of a full ring
    // (which reads the slot just written) follows it
    if ((rc = als_decode_append(ctx, b_q, b_k, a_k, head_stride, active_idx, n, k_act, v_act, n, q, k_new, v_new, b, hq,
                                hkv, r, d, max_iter, tol, q_hat, k_hat, token, topk + ring_slot, token, defer_finish,
                                dtype, (hipStream_t)stream)))
      return rc;
  }
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
    const bool keep_state = quick && fused_diff;
    if ((rc = fetch_attention(ctx, kv_store, cap, k_act, v_act, n, active_idx, n, miss_slots, mcount, ev, b, hq, hkv, d,
                              topk, q, attn_out, dtype, (hipStream_t)stream, miss_old, vic_active ? vic : nullptr,
                              fused_diff ? miss_new : nullptr, keep_state ? ctx->evk.p : nullptr, ctx->evk_rows,
                              miss_count && mcount != miss_count ? miss_count : nullptr)))
      return rc;
    if (keep_state) {
      if ((rc = flush_pending_finish(ctx, (hipStream_t)stream))) return rc;  // (the fetch launch carried it, normally)
      const int next_slot = topk + (ring_slot + 1) % lite;
      if ((rc = factor_state_advance(ctx, b_q, b_k, a_k, head_stride, active_idx, n, k_act, n, miss_slots, miss_old,
                                     miss_new, mcount, cap, bh, r, d, topk, topk + ring_slot, token, next_slot, dtype,
                                     (hipStream_t)stream)))
        return rc;
      ctx->fs_bq = b_q;
      ctx->fs_bk = b_k;
      ctx->fs_ak = a_k;
      ctx->fs_kact = k_act;
      ctx->fs_idx = active_idx;
      ctx->fs_head_stride = head_stride;
      ctx->fs_bh = bh;
      ctx->fs_r = r;
      ctx->fs_d = d;
      ctx->fs_dtype = dtype;
      ctx->fs_topk = topk;
      ctx->fs_n = n;
      ctx->fs_next_slot = next_slot;
      ctx->fs_next_token = token + 1;
      ctx->fs_valid = true;
    }
    return LRQK_OK;
  }
  if ((rc = lrqk_fetch_rows(kv_store, cap, k_act, v_act, n, active_idx, n, miss_slots, mcount, b, hq, hkv, d, topk, dtype,
                            stream)))
    return rc;
  if (attn_out) {
    if ((rc = lrqk_attention(ctx, q, k_act, v_act, n, n, attn_out, bh, d, dtype, stream))) return rc;
  }
  return LRQK_OK;
}
