/*
 * C ABI of liblrqk_hip.so: the gfx950 (MI355X) kernels of the LRQK per-layer decode /
 * prefill path.  Plain pointers and sizes only; no torch types.  Every entry point
 * returns 0 on success and a negative LRQK_E* code on an argument error (the text is
 * available from lrqk_last_error()); nothing throws across the boundary.  All device
 * work is enqueued on the caller's stream (a hipStream_t passed as void*; NULL is the
 * default stream) and nothing synchronises unless the comment says so.
 *
 * Shapes: "bh" is batch * query-heads, flattened row-major (b, h).  Query head h reads
 * KV head h / groups.  dtype is the STORAGE type of factors and K/V rows; arithmetic is
 * fp32.  Token / slot indices on the device are int32.
 *
 * Each declaration cites the reference interface it replaces (paths relative to the
 * reference tree; "py" = lrqk_attention.py, "cpp" = cpp_kernel/take_along_dim_grouped.cpp).
 */
#ifndef LRQK_HIP_H
#define LRQK_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LRQK_F32 0
#define LRQK_BF16 1

#define LRQK_OK 0
#define LRQK_EINVAL (-1)   /* bad shape / size / dtype / null pointer */
#define LRQK_EHIP (-2)     /* a HIP runtime call failed */
#define LRQK_ELIMIT (-3)   /* size beyond what the kernels support */

#define LRQK_MAX_R 64          /* every entry; the factor updates (lrqk_als_*) are tuned for r <= 32 and run
                                * general kernels beyond (r (r + d) <= 12288 for the prefill) */
#define LRQK_MAX_TOPK 8192
#define LRQK_MAX_DECODE_ITERS 16

typedef struct lrqk_ctx lrqk_ctx;

int lrqk_version(void);
const char* lrqk_last_error(void);

/* Workspace (radix keys, histograms, split partials), sized on demand; growing it
 * synchronises the device once.  One ctx per engine; calls on one ctx must not overlap. */
int lrqk_ctx_create(lrqk_ctx** out);
int lrqk_ctx_destroy(lrqk_ctx* ctx);
/* Optional: pre-size the workspace so that later calls never allocate. */
int lrqk_ctx_reserve(lrqk_ctx* ctx, int bh, int64_t max_tokens, int topk, int n_active, int r, int d);

/* py:1260-1263 -- proxy scores A_K[:m] . q_hat^T as fp32 [bh][m].
 * a_k: [bh] heads of head_stride elements each, rows of r elements; q_hat: [bh][r].
 * score = fmaf chain over j = 0..r-1 from +0; -0 becomes +0; round_bf16 != 0 rounds the
 * fp32 sum to bfloat16 (nearest even), which is what a bf16 matmul returns. */
int lrqk_proxy_scores(const void* a_k, int64_t head_stride, const void* q_hat, int bh, int64_t m, int r,
                      int dtype, int round_bf16, float* out_scores, void* stream);

/* py:1235-1273 compute_hit_indices -- scores (as above, never materialised as floats)
 * + per-head top-k under the order (score descending, token index ascending), returned
 * ASCENDING by index in out_idx[bh][out_stride] (first min(k,m) entries).  m <= k yields
 * arange(m).  Returns min(k,m) (>= 0) on success.  The ctx remembers, per head, a lower
 * bound of the previous call's threshold to pre-filter the next scan; the result never
 * depends on it. */
int lrqk_score_select(lrqk_ctx* ctx, const void* a_k, int64_t head_stride, const void* q_hat, int bh,
                      int64_t m, int r, int topk, int dtype, int round_bf16, int32_t* out_idx,
                      int64_t out_stride, void* stream);

/* Same selection from caller-provided fp32 scores [bh][m] (test hook for tie cases). */
int lrqk_select_from_scores(lrqk_ctx* ctx, const float* scores, int bh, int64_t m, int topk,
                            int32_t* out_idx, int64_t out_stride, void* stream);

/* Which selector path the heads took since the last reset: `fast_heads` selected from the
 * candidate list of the streaming filter, `full_heads` rescanned their whole head (first
 * call, or the score distribution moved).  Copies two counters from the device
 * (synchronises).  No counterpart in the reference. */
int lrqk_select_stats(lrqk_ctx* ctx, int* fast_heads, int* full_heads, int reset);
/* Split of the full_heads reported by the last lrqk_select_stats call: lists that held fewer
 * than k candidates, lists that overflowed. */
int lrqk_select_stats_detail(lrqk_ctx* ctx, int* list_short, int* list_overflow);

/* Work of the last scan that went through the score index: rows it covered (all heads) and rows whose
 * bound reached the threshold and were rescored exactly from a_k (0 / 0 if the last scan read a_k itself).
 * Copies from the device (synchronises).  No counterpart in the reference. */
int lrqk_scan_stats(lrqk_ctx* ctx, int64_t* rows_scanned, int64_t* rows_rescored);

/* py:1275-1315 only_indices_in_cpu -- hit/miss diff, in place.
 * hit: [bh][hit_stride] current GPU-resident token ids (first k used), any order, unique.
 * new_idx: [bh][new_stride] ascending, unique.  On return the j-th evicted slot (ascending
 * slot) of each head holds the j-th smallest token of new \ hit; evict[bh][k] is 1 for
 * replaced slots; miss_slots[bh][k] lists the replaced slots ascending and miss_count[bh]
 * their number.  Any of evict / miss_slots / miss_count may be NULL only if all callers of
 * the result do not need it (miss_slots and miss_count are required by lrqk_fetch_rows). */
int lrqk_diff(const int32_t* new_idx, int64_t new_stride, int32_t* hit, int64_t hit_stride, int bh, int k,
              uint8_t* evict, int32_t* miss_slots, int32_t* miss_count, void* stream);

/* py:1235-1273 + py:1275-1315 in one pass -- lrqk_score_select followed by lrqk_diff, with the
 * diff done by the select kernel while the selection is still on chip (m >= topk required; with m == topk every row is selected).
 * new_idx: [bh][topk] receives the ascending selection; hit / evict / miss_slots / miss_count
 * as in lrqk_diff (evict may be NULL).  new_idx may be NULL: the caller then only gets what
 * changes (hit, evict, miss_slots, miss_count), and the selection is never put in order -- the
 * form lrqk_decode_step uses. */
int lrqk_score_select_diff(lrqk_ctx* ctx, const void* a_k, int64_t head_stride, const void* q_hat, int bh,
                           int64_t m, int r, int topk, int dtype, int round_bf16, int32_t* new_idx, int32_t* hit,
                           int64_t hit_stride, uint8_t* evict, int32_t* miss_slots, int32_t* miss_count,
                           void* stream);

/* py:1752, 1762-1773 (LightAttentionIndicesNoHitMiss) -- the ablation without hit/miss
 * bookkeeping: hit <- new_idx, every slot marked evicted (all k rows are refetched). */
int lrqk_replace_all(const int32_t* new_idx, int64_t new_stride, int32_t* hit, int64_t hit_stride, int bh, int k,
                     uint8_t* evict, int32_t* miss_slots, int32_t* miss_count, void* stream);

/* py:101-117 + cpp:133-183 (d0_indices_select) + py:1603-1608 -- fetch the missed rows of
 * the host [K|V] store straight into the active-set slots.
 * kv_store: [b][hkv][cap][2*d] (K row then V row), pinned host memory (or device memory);
 * k_act/v_act: [bh][n_slots][d].  For every head and every j < miss_count: slot =
 * miss_slots[j], token = hit[slot]; K/V slot rows are overwritten with the store row of
 * (b, h/groups, token).  The kernel reads the store through the GPU's host mapping. */
int lrqk_fetch_rows(const void* kv_store, int64_t cap, void* k_act, void* v_act, int n_slots,
                    const int32_t* hit, int64_t hit_stride, const int32_t* miss_slots,
                    const int32_t* miss_count, int b, int hq, int hkv, int d, int k, int dtype,
                    void* stream);

/* py:101-117 + py:1597-1608 as the reference stages it -- the same fetch through a staging block:
 * the miss list is copied to the host (the call waits for the stream once), the host gathers the
 * rows of the pinned store (cpp:13-124) into pinned staging memory owned by the ctx, one
 * hipMemcpyAsync on the ctx's side stream moves them, the caller's stream waits on an event and a
 * kernel scatters them into the slots.  kv_store must be pinned host memory. */
int lrqk_fetch_rows_staged(lrqk_ctx* ctx, const void* kv_store, int64_t cap, void* k_act, void* v_act, int n_slots,
                           const int32_t* hit, int64_t hit_stride, const int32_t* miss_slots,
                           const int32_t* miss_count, int b, int hq, int hkv, int d, int k, int dtype, void* stream);
/* Which fetch lrqk_decode_step uses: 0 (default) lrqk_fetch_rows, 1 lrqk_fetch_rows_staged with
 * host_threads gather threads (<= 0 keeps the current count).  No counterpart in the reference. */
int lrqk_ctx_set_fetch_mode(lrqk_ctx* ctx, int mode, int host_threads);

/* Score index for the scan (no counterpart in the reference; a new ctx has it off, the Python
 * engine switches it on).  The ctx keeps an
 * 8-bit copy of the A_K rows (one 16-bit scale per row, 34 instead of 64 bytes per row for r = 32) and the
 * scan of lrqk_score_select / lrqk_score_select_diff / lrqk_decode_step reads that copy: it bounds
 * every row's score and rescores exactly, from a_k itself, only the rows whose bound reaches the
 * filter threshold.  Results are identical.  The copy is built on demand for rows [0, m) and
 * extended by the factor update's appended row; it is derived state: after changing rows of a_k
 * in place call this again (any value) to drop it.  Applies to r = 16, 32, 64. */
int lrqk_ctx_score_index(lrqk_ctx* ctx, int enable);

/* Victim cache for lrqk_decode_step (no counterpart in the reference; a new ctx has it off, the
 * Python engine gives it 4 k rows per head).  K/V rows
 * that leave the top-k slots are kept in a per-head FIFO of rows_per_head rows on the device
 * (tokens near the selection threshold return within a few steps); a missed row that is still
 * there is copied from the FIFO instead of over the host link.  Results are identical: a token's
 * row never changes.  The cache belongs to ONE sequence: call this again (any value) to drop its
 * contents before the ctx is used for another prompt.  0 switches it off.  Memory: bh *
 * rows_per_head rows of 2*d elements plus 2 bytes per (head, store row). */
int lrqk_ctx_victim_cache(lrqk_ctx* ctx, int rows_per_head);
/* Rows that lrqk_decode_step fetched over the host link since the last reset (the other missed
 * rows came from the victim cache).  Synchronises.  Counts only while the victim cache is on. */
int lrqk_victim_stats(lrqk_ctx* ctx, int64_t* host_rows, int reset);

/* Kept state of the factor update inside lrqk_decode_step (no counterpart in the reference; a new ctx has it
 * off).  In py:555-609 everything but a few products with the step's q and k -- B_Q B_Q^T + A^T A, B_K B_K^T, their
 * inverses and K__^T A over the active slots -- depends only on what the previous step left, because the new
 * token's A_K row is zero while its update runs (py:888, 1560).  The ctx keeps those per head in fp64 and brings
 * them up to date after each step's fetch from the rows that the step replaced (one more launch at the end of the
 * step), so a step's update is one small launch in fp64: its iterates agree with an fp64 evaluation of py:555-609
 * to rounding, where the update over the active rows in fp32 is cond(G) * 2^-24 away (ranks <= 32, head widths 32,
 * 64, 128 or 256, at most 8 iterations; other shapes and every other entry point run the update over the active
 * rows in fp32).  The state describes the buffers that
 * the last lrqk_decode_step call was given, as its next call will find them: call this (any value) after changing
 * B_Q, B_K, the active ids, A_K rows or K rows of the active set in any other way, and the next step forms the
 * state from scratch.  0 switches the kept state off. */
int lrqk_ctx_factor_state(lrqk_ctx* ctx, int enable);
/* The iterates of the last lrqk_decode_step that ran from kept state, in fp64 as computed (before they are
 * rounded): out [bh][max_iter][2 r] = (q_hat, k_hat) of every iteration.  bh, max_iter, r receive the sizes and
 * token the id of the token whose step it was (-1: none yet); out may be NULL to ask for them.  Synchronises.
 * Test hook; no counterpart in the reference. */
int lrqk_last_iterates(lrqk_ctx* ctx, double* out, int64_t n_doubles, int* bh, int* max_iter, int* r,
                       int64_t* token);

/* py:1339-1351 fetch_by_hit (same-device branch) -- k_act[bh][j][:] = src[b][h/groups][idx[bh][j]][:]
 * for j < count, src: [b][hkv][src_len][d] on the device. */
int lrqk_gather_rows(const void* src, int64_t src_len, const int32_t* idx, int64_t idx_stride, int count,
                     void* dst, int n_slots, int b, int hq, int hkv, int d, int dtype, void* stream);

/* py:1133-1135, 1185-1188 -- write the new token's k,v ([b][hkv][d]) into ring slot `slot`
 * of every query head and record its token id in active_idx[bh][slot]. */
int lrqk_append_token(const void* k_new, const void* v_new, void* k_act, void* v_act, int n_slots, int slot,
                      int32_t* active_idx, int64_t idx_stride, int32_t token, int b, int hq, int hkv, int d,
                      int dtype, void* stream);

/* py:1192-1196 + 959-963 -- flush ring slots [slot0, slot0+count) of heads 0, g, 2g, ... to
 * store rows [row0, row0+count) as [K|V]. */
int lrqk_flush_ring(const void* k_act, const void* v_act, int n_slots, int slot0, int count, void* kv_store,
                    int64_t cap, int64_t row0, int b, int hq, int hkv, int d, int dtype, void* stream);

/* py:2326-2327 (flash_attn_with_kvcache, one query, scale 1/sqrt(d)) -- exact attention
 * over the first n_valid slots.  q,out: [bh][d]; k_act,v_act: [bh][n_slots][d]. */
int lrqk_attention(lrqk_ctx* ctx, const void* q, const void* k_act, const void* v_act, int n_slots,
                   int n_valid, void* out, int bh, int d, int dtype, void* stream);

/* No counterpart in the reference.  The same attention as lrqk_attention for callers that cannot
 * allocate device memory (code under HIP graph capture, serving loops and harnesses that forbid
 * hipMalloc): it takes no ctx and allocates nothing; its split partial results live in a fixed
 * 4 MiB block of the library's own device memory (one per GPU, held until the process ends).
 * Limit: bh * min(64, ceil(n_valid / 64)) * (d + 2) <= 1048576, else LRQK_ELIMIT.  All calls on one
 * GPU share that block: calls that overlap on one GPU (different streams or threads) race; calls on
 * one stream are ordered.  The block needs no clearing between calls (every entry that is read was
 * written by the same call).  The first call on a device looks up the block's address (and lets the
 * runtime load the kernels): make it outside a graph capture. */
int lrqk_attention_static(const void* q, const void* k_act, const void* v_act, int n_slots, int n_valid,
                          void* out, int bh, int d, int dtype, void* stream);

/* py:803-839 cast_lrqk_decode -> py:529-628 _lrqk_decode_inv_w1 + py:651-665 -- the per-step
 * factor update.  b_q,b_k: [bh][r][d] storage dtype, updated in place.  The active A_K rows
 * are gathered from a_k (heads of head_stride elements) at active_idx[bh][0..n) (py:1156-1171);
 * if active_idx is NULL rows 0..n-1 are used (the prefix branch, py:1526-1539).
 * k_prev: [bh][kprev_slots][d] (first n rows used); q: [bh][d]; k_new: [b][hkv][d].
 * Outputs q_hat,k_hat: [bh][r] storage dtype.  If append_row >= 0, k_hat is also written to
 * row append_row of every head of a_k (py:1560 sync_cache).  The stopping test
 * mean((k_hat - k_hat')^2) < tol is taken over all heads at once, on the device. */
int lrqk_als_decode(lrqk_ctx* ctx, void* b_q, void* b_k, void* a_k, int64_t head_stride,
                    const int32_t* active_idx, int64_t idx_stride, const void* k_prev, int kprev_slots, int n,
                    const void* q, const void* k_new, int b, int hq, int hkv, int r, int d, int max_iter,
                    float tol, void* q_hat, void* k_hat, int64_t append_row, int dtype, void* stream);

/* py:772-800 cast_lrqk_prefill -> py:319-423 _lrqk_prefill_inv_w1 -- joint rank-r ALS fit.
 * q: [b][hq][l][d], k: [b][hkv][l][d] storage dtype (query head h uses KV head h/groups);
 * a_q,a_k: [bh][l][r] fp32 work buffers holding the initial factors on entry and the
 * result on return; b_q,b_k out: [bh][r][d] fp32.  The stopping test (batch-wide mean squared
 * change of A_Q and A_K below tol) is evaluated on the device: once it fires the remaining
 * launches return at once, and the host never waits.  r <= 32: bf16 input with d <= 128 runs on
 * the bf16 matrix cores (fp32 operands as three bf16 pieces each, fp32 accumulation), fp32 input
 * or d = 256 on fp32 MFMA tiles, other shapes -- and ranks up to 64 (README.md:124-131 of the reference
 * names r = 64) -- on a general kernel, as long as r (r + d) <= 12288.  Returns 0. */
int lrqk_als_prefill(lrqk_ctx* ctx, const void* q, const void* k, float* a_q, float* a_k, float* b_q,
                     float* b_k, int b, int hq, int hkv, int64_t l, int r, int d, int max_iter, float tol,
                     int dtype, void* stream);

/* py:1506-1613 LightAttentionIndicesFactory.decode (main branch) + the attention call
 * site py:2326 -- one decode step of one layer as one host call that only enqueues
 * kernels.  State: b_q,b_k [bh][r][d]; a_k heads of head_stride elements (zero beyond the
 * rows written so far); active_idx [bh][topk+lite] = resident token ids then ring token
 * ids; k_act,v_act [bh][topk+lite][d]; kv_store [b][hkv][cap][2d].
 * Order: ring append of (k_new, v_new) at slot topk+ring_slot as token id `token`; if
 * flush_row0 >= 0 the whole ring is flushed to store rows flush_row0.. ; factor update
 * (k_hat appended as A_K row `token`); selection over candidates 0..m-1; diff (or
 * replace-all when no_hit_miss); miss fetch; if attn_out != NULL, attention of q over all
 * topk+lite slots.  evict ([bh][topk]) and miss_count ([bh]) are optional outputs. */
int lrqk_decode_step(lrqk_ctx* ctx, void* b_q, void* b_k, void* a_k, int64_t head_stride, int32_t* active_idx,
                     void* k_act, void* v_act, void* kv_store, int64_t cap, const void* q, const void* k_new,
                     const void* v_new, int b, int hq, int hkv, int r, int d, int topk, int lite, int ring_slot,
                     int32_t token, int64_t m, int64_t flush_row0, int max_iter, float tol, int round_scores,
                     int no_hit_miss, void* q_hat, void* k_hat, void* attn_out, uint8_t* evict,
                     int32_t* miss_count, int dtype, void* stream);

/* py:2031-2105 (WrapForwardTimer, the reference's only timing facility, wall clock around
 * forward) -- device-side timing of the dominant kernel instead: after
 * lrqk_timing_enable(ctx, n) the next n proxy-score kernel launches of lrqk_score_select /
 * lrqk_decode_step on this ctx are bracketed by HIP events on the launch stream;
 * lrqk_timing_read waits for them, returns the summed kernel time and the launch count, and
 * re-arms.  n = 0 switches timing off. */
int lrqk_timing_enable(lrqk_ctx* ctx, int max_launches);
/* Bracket only every `every`-th launch (default 1): the two event packets delay the kernels around
 * them by a few microseconds, which a sampled measurement keeps out of most steps. */
int lrqk_timing_stride(lrqk_ctx* ctx, int every);
int lrqk_timing_read(lrqk_ctx* ctx, double* total_ms, int* launches);

/* No counterpart in the reference.  Plain streaming kernels of known size on the caller's stream: `reps`
 * reads of src[0, bytes) and `reps` copies of it to dst, each series timed with HIP events; returns the
 * average milliseconds per pass (waits for the stream).  What the memory system delivers on the GPU at
 * hand, to read the scan's rate against, and a transfer of known size to scale hardware counters by.
 * src, dst: device memory, 16-byte aligned, bytes a multiple of 16. */
int lrqk_probe_bandwidth(const void* src, void* dst, int64_t bytes, int reps, double* read_ms, double* copy_ms,
                         void* stream);
/* Measurement helper (no counterpart in the reference): one variant of the plain read -- in_flight (4, 8 or 16)
 * 16-byte vectors per thread, plain or non-temporal loads, grid_per_cu workgroups of 256 threads per CU -- for a
 * sweep that looks for the best read rate of the GPU at hand.  slice_bytes = 0: every launch reads the whole buffer;
 * > 0: a launch reads one slice of that size and the launches take the slices in turn (the rate of a launch of a
 * given size whose data does not come from the last-level cache).  read_ms: per launch.  sink: 64 KB of device
 * memory (never written in practice).  Waits for the stream. */
int lrqk_probe_read_variant(const void* src, void* sink, int64_t bytes, int64_t slice_bytes, int reps, int in_flight,
                            int nontemporal, int grid_per_cu, double* read_ms, void* stream);
/* No counterpart in the reference.  What a pair of HIP events reads around `kernels` (1..16) launches that do nothing
 * (average microseconds over `reps` <= 256 pairs on the caller's stream, each pair between two other launches; waits
 * for the stream).  The reading with one launch less the difference between two launches and one is the part of an
 * event-bracketed kernel time (lrqk_timing_read) that is not the kernel. */
int lrqk_probe_event_pair(int reps, int kernels, double* pair_us, void* stream);

/* Host-side row gathers with the reference's native signatures (the staged fetch path
 * and API parity); multi-threaded memcpy.
 * cpp:133-183 d0_indices_select: dst[i,:] = src[idx[i],:]. */
int lrqk_d0_indices_select(void* dst, const void* src, const int64_t* idx, int64_t n, int64_t row_bytes,
                           int64_t src_rows, int threads);
/* cpp:13-124 take_along_dim_with_mask: src [b][hkv][seq][row], indices int64 / mask u8
 * [b][hkv][groups][k]; dst gets the masked rows in row-major mask order.  Returns the row
 * count (>= 0); dst may be NULL to only count. */
int64_t lrqk_take_along_dim_with_mask(void* dst, const void* src, const int64_t* indices, const uint8_t* mask,
                                      int64_t b, int64_t hkv, int64_t groups, int64_t k, int64_t seq,
                                      int64_t row_bytes, int threads);

#ifdef __cplusplus
}
#endif
#endif
