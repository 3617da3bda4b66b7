// Victim cache of the active set: K/V rows that leave the top-k slots are kept in a per-head FIFO
// on the device, because tokens near the selection threshold come back within a few steps.  A
// missed row that is still in the FIFO is copied from there instead of over the host link.
// Rows of a token never change, so a cached row can only be missing, never stale; the cache is
// tied to one sequence (the ctx owner resets it when a new prompt is factorised).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lrqk {

struct VictimView {
  uint4* rows;         // [bh][nv][chunks]  [K|V] rows, the store's row layout
  int32_t* tok;        // [bh][nv]          token of each FIFO position, -1 = empty
  int16_t* pos;        // [bh][cap]         FIFO position of a token, -1 = not cached
  int32_t* ptr;        // [bh]              next insert position (advanced by the diff)
  int32_t* base;       // [bh]              insert position of the current step's first victim
  int32_t* host_rows;  // [bh]              rows that had to come over the host link (cumulative)
  int nv;              // FIFO length per head, 0 = cache off
  int64_t cap;         // tokens covered by pos
};

// true if FIFO position q is (re)written during the current step: n victims go to base .. base+n-1
__device__ __forceinline__ bool victim_slot_in_flight(int q, int base, int n, int nv) {
  int rel = q - base;
  if (rel < 0) rel += nv;
  return rel < n;
}

}  // namespace lrqk
