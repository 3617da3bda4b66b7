// Shared between the files that hold the per-step factor update (als_decode.hip: r <= 32 and the general
// form; als_decode_r64.hip: 32 < r <= 64 on the matrix cores).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ctx.hpp"

namespace lrqk {

// Ring append folded into the Gram pass: slot `slot` (>= 0) of every head is the new token.  The
// pass takes its K row from k_new and its token id from `token` instead of the buffers, and the
// wave that owns the slot writes k_new, v_new and the id into them.
struct GramAppend {
  const void* k_new;  // [b][hkv][d]
  const void* v_new;  // [b][hkv][d]
  void* v_act;        // [bh][kprev_slots][d]
  int32_t* idx_out;   // active_idx, writable
  int slot;           // -1: nothing to append
  int32_t token;
  int hq, hkv;
};

// Gram pass + solve of the factor update for bf16 storage, d = 128, 32 < r <= 64, r % 8 == 0 (16-byte aligned rows
// of A_K).  Leaves the iterates in iter_out ([bh][max_iter][2 r]) and their squared changes in deltas
// ([bh][max_iter]), like the kernels for r <= 32; kq_out (or null): K q of every slot, [bh][n].
bool als_r64_supported(int dtype, int r, int d, const void* a_k, int64_t head_stride);
int als_r64_update(lrqk_ctx* ctx, const void* b_q, const void* b_k, const void* a_k, int64_t head_stride,
                   const int32_t* active_idx, int64_t idx_stride, void* k_prev, int kprev_slots, int n, const void* q,
                   const void* k_new, int bh, int hq, int hkv, int r, int max_iter, float* iter_out, float* deltas,
                   const GramAppend& ap, float* kq_out, hipStream_t st);

}  // namespace lrqk
