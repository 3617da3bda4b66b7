// Library-owned device workspace.
#pragma once
#include <atomic>
#include <hip/hip_runtime.h>

#include "common.hpp"
#include "als_finish.hpp"
#include "victim.hpp"

namespace lrqk {

struct DevBuf {
  void* p = nullptr;
  size_t bytes = 0;
  // Grows (never shrinks).  Growing frees the old block after a device sync, because
  // kernels of an earlier call may still be reading it.
  int ensure(size_t need) {
    if (need <= bytes) return LRQK_OK;
    size_t want = need + need / 4;
    void* np = nullptr;
    LRQK_HIP_CHECK(hipMalloc(&np, want));
    if (p) {
      LRQK_HIP_CHECK(hipDeviceSynchronize());
      LRQK_HIP_CHECK(hipFree(p));
    }
    p = np;
    bytes = want;
    return LRQK_OK;
  }
  // Same, and the block is zero-filled whenever it is (re)allocated.
  int ensure_zeroed(size_t need) {
    if (need <= bytes) return LRQK_OK;
    int rc = ensure(need);
    if (rc) return rc;
    LRQK_HIP_CHECK(hipMemset(p, 0, bytes));
    return LRQK_OK;
  }
  void release() {
    if (p) (void)hipFree(p);
    p = nullptr;
    bytes = 0;
  }
};

}  // namespace lrqk

struct lrqk_ctx {
  lrqk::DevBuf keys;        // u32 [bh][key_stride]   orderable score keys
  lrqk::DevBuf hist;        // u32 [bh][4096]         first-level radix histogram
  lrqk::DevBuf cand;        // candidate (key,idx) pairs for the fast select path
  lrqk::DevBuf cand_cnt;    // per-chunk counts / thresholds
  lrqk::DevBuf attn_part;   // f32 [bh][S][d+2]
  lrqk::DevBuf als_part;    // f32 [bh][S][32*32 + 32]
  lrqk::DevBuf als_kq;      // f32 [bh][n]: K q of every active slot, left by the step's Gram pass for its attention
  bool kq_valid = false;    //   set by that pass, consumed by the fetch + attention launch of the same step
  const void* kq_k_act = nullptr;
  const void* kq_q = nullptr;
  int kq_bh = 0, kq_n = 0;
  lrqk::DevBuf als_pre;     // f32 [bh][4*1024 + 65]: what the solve needs from B_Q, B_K, q, k (formed beside the Gram pass)
  lrqk::DevBuf als_iter;    // f32 [bh][MAX_IT][2r] + deltas
  lrqk::DevBuf als_iter64;  // f64 [bh][MAX_IT][2r]: the same iterates before rounding to fp32 (kept-state update only)
  int iter64_bh = 0, iter64_r = 0, iter64_iters = 0;
  int64_t iter64_token = -1;  // token whose step left them
  // Kept state of the decode step's factor update (als_state.hip): per head, fp64, the sums over the active slots
  // and the inverses / projections that the next step starts from.
  lrqk::DevBuf fstate;      // f64 [bh][3 d 32 + 3 * 1024]
  lrqk::DevBuf evk;         // storage dtype [bh][evk_rows][d]: K rows that the step's misses replaced
  int evk_rows = 0;
  bool fs_enabled = false;  // lrqk_ctx_factor_state
  bool fs_valid = false;    // fstate describes the buffers below as the next step (fs_next_*) will find them
  const void *fs_bq = nullptr, *fs_bk = nullptr, *fs_ak = nullptr, *fs_kact = nullptr, *fs_idx = nullptr;
  int64_t fs_head_stride = 0;
  int fs_bh = 0, fs_r = 0, fs_d = 0, fs_dtype = -1, fs_topk = 0, fs_n = 0, fs_next_slot = -1;
  int32_t fs_next_token = -1;
  lrqk::DevBuf prefill_ws;  // prefill ALS accumulators
  lrqk::DevBuf prefill_gd;  // prefill ALS on Gram matrices: X^T X sums, fp64 state
  lrqk::DevBuf new_idx;     // i32 [bh][k] selection result of the fused step
  lrqk::DevBuf misc;        // evict mask, miss lists, counters of the fused step
  // finish stage of the factor update deferred into later launches of the decode step
  lrqk::FinishArgs fin{};
  int fin_dtype = 0;
  bool fin_pending = false;   // B update / outputs / A_K row not done yet
  bool qhat_pending = false;  // q_hat not written yet
  // score index: 8-bit copy of the A_K rows for the scan (off unless lrqk_ctx_score_index enabled it)
  lrqk::DevBuf sidx_qa, sidx_qs, sidx_wm, sidx_part;
  bool sidx_enabled = false;
  const void* sidx_a_k = nullptr;   // A_K buffer the index was built from
  int64_t sidx_head_rows = 0, sidx_valid = 0;  // rows per head; rows [0, valid) are indexed
  int sidx_r = 0, sidx_dtype = -1, sidx_bh = 0;
  int64_t sidx_rows_hint = 0;  // rows of A_K known to be written (the decode step sets it); 0 = only the scanned ones
  // victim cache of the decode step (off unless lrqk_ctx_victim_cache asked for rows)
  lrqk::DevBuf vic_rows, vic_meta;
  lrqk::VictimView vic{};   // current view; nv == 0 while off or not yet built
  int vic_req = 0;          // FIFO rows per head asked for
  int vic_bh = 0, vic_chunks = 0;
  bool vic_dirty = true;    // (re)initialise before the next use
  // staged miss fetch: pinned host staging, its device twin, side stream and event (created on first use)
  lrqk::DevBuf stage_dev;
  void* stage_host = nullptr;
  size_t stage_host_bytes = 0;
  hipStream_t side = nullptr;
  hipEvent_t stage_ev = nullptr;
  int fetch_mode = 0;  // 0: the kernel reads the pinned store directly; 1: host gather + hipMemcpyAsync on the side stream
  int host_threads = 8;
  // optional event timing of the proxy-score kernel (two events per launch)
  hipEvent_t* tev = nullptr;
  int tev_pairs = 0;   // capacity in pairs
  int tev_used = 0;    // pairs recorded since the last read
  int tev_every = 1;   // only every n-th launch is bracketed (the event packets cost a few us each)
  int tev_seen = 0;    // launches seen since timing was enabled
  int sel_bh = 0;      // head count the selector state (t_low, counters) was initialised for
  int last_short = 0, last_overflow = 0;  // split of the rescans seen by the last lrqk_select_stats
  int scan_wgs = 0;        // workgroups of the last scan through the score index (0: the last scan read A_K itself)
  int64_t scan_rows = 0;   // rows that scan covered (all heads)
};

namespace lrqk {
// Launch set-up that is remembered between calls (function attributes raised so far, occupancy figures) belongs to
// a device: one slot per device ordinal, atomics because callers may come from several host threads (the set-up
// itself is idempotent, so a duplicate is harmless).
constexpr int kMaxDeviceSlots = 64;
inline int per_device_slot() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  return dev >= 0 && dev < kMaxDeviceSlots ? dev : 0;
}
// Proxy-score scan + top-k with the hit/miss diff fused into the select kernel when the
// sizes allow.  Returns 1 if the diff ran, 0 if the caller still has to, negative on error.
int score_select_diff(lrqk_ctx* ctx, const void* a_k, int64_t head_stride, const void* q_hat, int bh, int64_t m, int r,
                      int topk, int dtype, int round_bf16, int32_t* new_idx, int32_t* hit, int64_t hit_stride,
                      uint8_t* evict, int32_t* miss_slots, int32_t* miss_count, int replace_all, hipStream_t st,
                      int32_t* miss_old = nullptr, const VictimView* vic = nullptr, int32_t* miss_new = nullptr,
                      bool want_new_idx = true);
// Prefill iterations on Gram matrices (bf16 input, d = 128, r <= 32); see als_prefill_gram.hip.
int prefill_gram_domain(lrqk_ctx* ctx, const void* q, const void* k, const float* partQ, const float* partK, int S,
                        const float* a_q0, float* b_q, float* b_k, int b, int hq, int hkv, int64_t l, int r, int iters,
                        float tol, int* flags, float** mt_q, float** mt_k, hipStream_t st);
// A_K = K Mk with K read once per kv head (bf16 rows of 128); false: no kernel for this head grouping.
bool prefill_apply_shared(const void* k, const float* mt_k, float* a_k, int b, int hq, int hkv, int64_t l, int r,
                          hipStream_t st, int* rc_out);
// The factor update with the ring append of (k_new, v_new) at slot `slot` as token `token` folded
// into its first kernel.
int als_decode_append(lrqk_ctx* ctx, void* b_q, void* b_k, void* a_k, int64_t head_stride, int32_t* active_idx,
                      int64_t idx_stride, void* k_act, void* v_act, int n_slots, const void* q, const void* k_new,
                      const void* v_new, int b, int hq, int hkv, int r, int d, int max_iter, float tol, void* q_hat,
                      void* k_hat, int64_t append_row, int slot, int32_t token, bool defer_finish, int dtype,
                      hipStream_t st);
// Leaves the finish stage of a factor update whose iterates are in iter_out / deltas pending in the ctx (the
// step's later launches absorb it, flush_pending_finish otherwise).
int als_defer_finish(lrqk_ctx* ctx, void* b_q, void* b_k, void* a_k, int64_t head_stride, const void* q,
                     const void* k_new, int bh, int hq, int hkv, int r, int d, int max_iter, float tol, void* q_hat,
                     void* k_hat, int64_t append_row, float* iter_out, float* deltas, int dtype);
// The factor update from kept state (als_state.hip).
constexpr int kStepFusedDiffMaxK = 4096;  // the select kernel's in-kernel diff (it lists the replaced tokens)
bool factor_state_supported(int r, int d, int dtype, int max_iter);
int factor_state_rebuild(lrqk_ctx* ctx, const void* b_q, const void* b_k, const void* a_k, int64_t head_stride,
                         const int32_t* active_idx, int64_t idx_stride, const void* k_act, int n_slots, int bh, int r,
                         int d, int topk, int skip_slot, int dtype, hipStream_t st);
int factor_state_advance(lrqk_ctx* ctx, const void* b_q, const void* b_k, const void* a_k, int64_t head_stride,
                         const int32_t* active_idx, int64_t idx_stride, const void* k_act, int n_slots,
                         const int32_t* miss_slots, const int32_t* miss_old, const int32_t* miss_new,
                         const int32_t* miss_count, int64_t cap, int bh, int r, int d, int topk, int ring_slot,
                         int32_t ring_token, int skip_slot, int dtype, hipStream_t st);
int factor_state_quick(lrqk_ctx* ctx, void* b_q, void* b_k, void* a_k, int64_t head_stride, int32_t* active_idx,
                       int64_t idx_stride, void* k_act, void* v_act, int n_slots, const void* q, const void* k_new,
                       const void* v_new, int b, int hq, int hkv, int r, int d, int max_iter, float tol, void* q_hat,
                       void* k_hat, int64_t append_row, int slot, int32_t token, int dtype, hipStream_t st);
// Runs a deferred finish stage as its own launch (no-op if none is pending).
int flush_pending_finish(lrqk_ctx* ctx, hipStream_t st);
// Miss fetch overlapped with the attention over the slots that stay resident (one launch), then
// the attention over the refetched slots and the merge (second launch).
int fetch_attention(lrqk_ctx* ctx, const void* kv_store, int64_t cap, void* k_act, void* v_act, int n_slots,
                    int32_t* hit, int64_t hit_stride, const int32_t* miss_slots, const int32_t* miss_count,
                    const uint8_t* evict, int b, int hq, int hkv, int d, int k, const void* q, void* out, int dtype,
                    hipStream_t st, const int32_t* miss_old = nullptr, const VictimView* vic = nullptr,
                    const int32_t* miss_new = nullptr, void* evk = nullptr, int evk_rows = 0,
                    int32_t* count_copy = nullptr);
// Makes the score index cover rows [0, m) of a_k (building or extending it as needed).  Returns 1 and
// fills `view` if the scan may use it, 0 if the index is off or does not apply, negative on error.
int score_index_prepare(lrqk_ctx* ctx, const void* a_k, int64_t head_stride, int bh, int64_t m, int r, int dtype,
                        hipStream_t st, ScoreIndexView* view);
// Builds / resets the victim cache for the given geometry (no-op when it is current).
int victim_prepare(lrqk_ctx* ctx, int bh, int64_t cap, int chunks, hipStream_t st);
}  // namespace lrqk
