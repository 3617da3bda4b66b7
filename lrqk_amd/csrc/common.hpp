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
  __device__ __forceinline__ void pack(const float* f) { raw = make_float4(f[0], f[1], f[2], f[3]); }
  __device__ __forceinline__ void store(float* p) const { *reinterpret_cast<float4*>(p) = raw; }
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
  // rounds like st_f32 (to nearest even)
  __device__ __forceinline__ void pack(const float* f) {
    raw.x = (uint32_t)f32_to_bf16_bits(f[0]) | ((uint32_t)f32_to_bf16_bits(f[1]) << 16);
    raw.y = (uint32_t)f32_to_bf16_bits(f[2]) | ((uint32_t)f32_to_bf16_bits(f[3]) << 16);
    raw.z = (uint32_t)f32_to_bf16_bits(f[4]) | ((uint32_t)f32_to_bf16_bits(f[5]) << 16);
    raw.w = (uint32_t)f32_to_bf16_bits(f[6]) | ((uint32_t)f32_to_bf16_bits(f[7]) << 16);
  }
  __device__ __forceinline__ void store(bf16_t* p) const { *reinterpret_cast<uint4*>(p) = raw; }
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

// Cross-lane moves of the data-parallel-primitive kind (no LDS round trip, unlike a shuffle).
// Lanes that the row / bank mask disables, or whose source lies outside the row, receive 0.
template <int CTRL, int ROW_MASK, int BANK_MASK>
__device__ __forceinline__ int dpp_mov0(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, BANK_MASK, false);
}
constexpr int kDppQuadXor1 = 0xB1;     // quad_perm [1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;     // quad_perm [2,3,0,1]
constexpr int kDppRowShr1 = 0x111, kDppRowShr2 = 0x112, kDppRowShr3 = 0x113, kDppRowShr4 = 0x114, kDppRowShr8 = 0x118;
constexpr int kDppRowMirror = 0x140, kDppRowHalfMirror = 0x141;
constexpr int kDppRowBcast15 = 0x142, kDppRowBcast31 = 0x143;

// inclusive wave scan (sum): three shifted copies of the input, then doubling steps inside each
// row of 16 lanes, then the row totals are passed on (lane 15 -> next row, lane 31 -> rows 2, 3)
__device__ __forceinline__ int wave_inclusive_sum(int v) {
  int x = v + dpp_mov0<kDppRowShr1, 0xf, 0xf>(v);
  x += dpp_mov0<kDppRowShr2, 0xf, 0xf>(v);
  x += dpp_mov0<kDppRowShr3, 0xf, 0xf>(v);
  x += dpp_mov0<kDppRowShr4, 0xf, 0xe>(x);
  x += dpp_mov0<kDppRowShr8, 0xf, 0xc>(x);
  x += dpp_mov0<kDppRowBcast15, 0xa, 0xf>(x);
  x += dpp_mov0<kDppRowBcast31, 0xc, 0xf>(x);
  return x;
}

// Butterflies inside each row of 16 lanes; afterwards every lane of a row holds the row's result.
template <typename Op>
__device__ __forceinline__ float row_reduce(float v, Op op) {
  v = op(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), kDppQuadXor1, 0xf, 0xf, false)));
  v = op(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), kDppQuadXor2, 0xf, 0xf, false)));
  v = op(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), kDppRowHalfMirror, 0xf, 0xf, false)));
  v = op(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), kDppRowMirror, 0xf, 0xf, false)));
  return v;
}
__device__ __forceinline__ float lane_bcast(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// Sum over aligned groups of `n` adjacent lanes (n a power of two); every lane of a group gets
// the group's sum.  Steps inside a row of 16 lanes are register moves, wider ones shuffles.
template <int CTRL>
__device__ __forceinline__ float dpp_self(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float group_sum(float v, int n) {
  if (n > 1) v += dpp_self<kDppQuadXor1>(v);
  if (n > 2) v += dpp_self<kDppQuadXor2>(v);
  if (n > 4) v += dpp_self<kDppRowHalfMirror>(v);
  if (n > 8) v += dpp_self<kDppRowMirror>(v);
  if (n > 16) v += __shfl_xor(v, 16, kWave);
  if (n > 32) v += __shfl_xor(v, 32, kWave);
  return v;
}
// wave-wide reductions of unsigned values, result in every lane
template <typename Op>
__device__ __forceinline__ uint32_t wave_reduce_u32(uint32_t v, Op op) {
  v = op(v, (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, kDppQuadXor1, 0xf, 0xf, false));
  v = op(v, (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, kDppQuadXor2, 0xf, 0xf, false));
  v = op(v, (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, kDppRowHalfMirror, 0xf, 0xf, false));
  v = op(v, (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, kDppRowMirror, 0xf, 0xf, false));
  const uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), b = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
  const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), d = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
  return op(op(a, b), op(c, d));
}

// result in every lane
__device__ __forceinline__ float wave_sum(float v) {
  v = row_reduce(v, [](float a, float b) { return a + b; });
  return (lane_bcast(v, 0) + lane_bcast(v, 16)) + (lane_bcast(v, 32) + lane_bcast(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
  v = row_reduce(v, [](float a, float b) { return fmaxf(a, b); });
  return fmaxf(fmaxf(lane_bcast(v, 0), lane_bcast(v, 16)), fmaxf(lane_bcast(v, 32), lane_bcast(v, 48)));
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
