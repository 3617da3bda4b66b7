// Device-side body of the miss fetch, shared by the stand-alone fetch kernel and the
// kernel that overlaps the fetch with the attention over the rows that stay resident.
#pragma once
#include "common.hpp"

namespace lrqk {

// Missed rows: store row (b, h/groups, token) = [K row | V row] -> active-set slot rows.
// Workgroup `blk` of `nblk` (per head) copies the missed rows blk*rpb .. , stepping nblk*rpb,
// rpb = blockDim.x / (2*cpr) rows at a time, one 16-byte chunk per thread.
__device__ __forceinline__ void fetch_rows_body(const uint4* __restrict__ store, int64_t cap, uint4* __restrict__ k_act,
                                                uint4* __restrict__ v_act, int n_slots,
                                                const int32_t* __restrict__ hit, int64_t hit_stride,
                                                const int32_t* __restrict__ miss_slots,
                                                const int32_t* __restrict__ miss_count, int hq, int hkv, int cpr, int k,
                                                int h, int blk, int nblk) {
  const int cnt = miss_count[h];
  const int chunks = 2 * cpr;  // per store row
  const int rpb = max(1, (int)blockDim.x / chunks);
  const int b = h / hq, head = h % hq;
  const int kvh = head / (hq / hkv);
  const int jl = threadIdx.x / chunks, c = threadIdx.x % chunks;
  if (jl >= rpb) return;
  for (int j = blk * rpb + jl; j < cnt; j += nblk * rpb) {
    const int slot = miss_slots[(int64_t)h * k + j];
    if (slot < 0 || slot >= k) continue;
    const int32_t tok = hit[(int64_t)h * hit_stride + slot];
    if (tok < 0 || tok >= cap) continue;
    const uint4 val = store[(((int64_t)b * hkv + kvh) * cap + tok) * chunks + c];
    const int64_t dst = ((int64_t)h * n_slots + slot) * cpr;
    if (c < cpr) k_act[dst + c] = val; else v_act[dst + (c - cpr)] = val;
  }
}

// Resolves a store pointer (device memory, or pinned host memory mapped into the device).
int resolve_store(const void* kv_store, const void** dev_store);

}  // namespace lrqk
