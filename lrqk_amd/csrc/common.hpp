// Shared device helpers for the gfx950 kernels: storage-type loads, orderable score
// keys, wave64 / workgroup scans.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/lrqk_hip.h"

namespace lrqk {

constexpr int kWave = 64;

int set_error(int code, const char* fmt, ...);

#define LRQK_REQUIRE(cond, code, ...) \
  do {                                \
    if (!(cond)) return ::lrqk::set_error((code), __VA_ARGS__); \
  } while (0)

#define LRQK_HIP_CHECK(expr)                                                              \
  do {                                                                                    \
    hipError_t e_ = (expr);                                                               \
    if (e_ != hipSuccess)                                                                 \
      return ::lrqk::set_error(LRQK_EHIP, "%s failed: %s", #expr, hipGetErrorString(e_)); \
  } while (0)

static inline size_t elem_size(int dtype) { return dtype == LRQK_F32 ? 4 : 2; }

// ----------------------------------------------------------------------------- bf16
struct bf16_t {
  uint16_t v;
};

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

__device__ __forceinline__ float round_to_bf16_f32(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) {
    u = (u | 0x00400000u) & 0xffff0000u;
  } else {
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
  }
  return __uint_as_float(u);
}

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  return (uint16_t)(__float_as_uint(round_to_bf16_f32(f)) >> 16);
}

template <typename T>
__device__ __forceinline__ float ld_f32(const T* p, int64_t i);
template <>
__device__ __forceinline__ float ld_f32<float>(const float* p, int64_t i) {
  return p[i];
}
template <>
__device__ __forceinline__ float ld_f32<bf16_t>(const bf16_t* p, int64_t i) {
  return bf16_bits_to_f32(p[i].v);
}

template <typename T>
__device__ __forceinline__ void st_f32(T* p, int64_t i, float v);
template <>
__device__ __forceinline__ void st_f32<float>(float* p, int64_t i, float v) {
  p[i] = v;
}
template <>
__device__ __forceinline__ void st_f32<bf16_t>(bf16_t* p, int64_t i, float v) {
  p[i].v = f32_to_bf16_bits(v);
}

// 16-byte vector of storage elements, unpacked to floats.
template <typename T>
struct Vec16;
template <>
struct Vec16<float> {
  static constexpr int N = 4;
  float4 raw;
  __device__ __forceinline__ void load(const float* p) { raw = *reinterpret_cast<const float4*>(p); }
  __device__ __forceinline__ void unpack(float* f) const {
    f[0] = raw.x; f[1] = raw.y; f[2] = raw.z; f[3] = raw.w;
  }
};
template <>
struct Vec16<bf16_t> {
  static constexpr int N = 8;
  uint4 raw;
  __device__ __forceinline__ void load(const bf16_t* p) { raw = *reinterpret_cast<const uint4*>(p); }
  __device__ __forceinline__ void unpack(float* f) const {
    f[0] = __uint_as_float(raw.x << 16); f[1] = __uint_as_float(raw.x & 0xffff0000u);
    f[2] = __uint_as_float(raw.y << 16); f[3] = __uint_as_float(raw.y & 0xffff0000u);
    f[4] = __uint_as_float(raw.z << 16); f[5] = __uint_as_float(raw.z & 0xffff0000u);
    f[6] = __uint_as_float(raw.w << 16); f[7] = __uint_as_float(raw.w & 0xffff0000u);
  }
};

// ----------------------------------------------------------------------------- score keys
// Monotone map fp32 -> u32: larger score <=> larger key.  Scores are canonicalised so
// that -0 and +0 share one key.
__device__ __forceinline__ uint32_t score_key(float s) {
  if (s == 0.0f) s = 0.0f;
  uint32_t u = __float_as_uint(s);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_score(uint32_t k) {
  uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(u);
}

// ----------------------------------------------------------------------------- wave / block scans
__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }
__device__ __forceinline__ int wave_id() { return threadIdx.x >> 6; }

// number of set predicate bits in lanes below this one, and the wave total
__device__ __forceinline__ int wave_rank(bool pred, int& total) {
  unsigned long long mask = __ballot(pred);
  total = __popcll(mask);
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// inclusive wave scan (sum) via shuffles
__device__ __forceinline__ int wave_inclusive_sum(int v) {
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    int t = __shfl_up(v, off, kWave);
    if (lane_id() >= off) v += t;
  }
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Workgroup-wide rank of a predicate in thread order.  `scratch` needs blockDim/64 + 1
// ints of LDS.  Returns this thread's exclusive rank; block_total receives the sum.
// Contains two barriers; every thread of the block must call it.
__device__ __forceinline__ int block_rank(bool pred, int* scratch, int& block_total) {
  int wtotal;
  int r = wave_rank(pred, wtotal);
  const int nw = blockDim.x >> 6;
  if (lane_id() == 0) scratch[wave_id()] = wtotal;
  __syncthreads();
  int base = 0, tot = 0;
  for (int w = 0; w < nw; ++w) {
    int c = scratch[w];
    if (w < wave_id()) base += c;
    tot += c;
  }
  __syncthreads();
  block_total = tot;
  return base + r;
}

}  // namespace lrqk
