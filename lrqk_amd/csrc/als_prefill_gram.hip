// Prefill factorisation, iterations carried out on Gram matrices (bf16 input, d = 128, r <= 32).
//
// After the first half-step of lrqk_attention.py:359-421 every factor is a linear image of its input,
// A_Q = Q Mq and A_K = K Mk with Mq, Mk of size d x r.  Everything an iteration needs from the long axis
// is then a product with Sq = Q^T Q or Sk = K^T K (d x d):
//     A_Q^T A_Q = Mq^T Sq Mq,   A_Q^T Q = Mq^T Sq,   Q^T A_Q = Sq Mq   (likewise for K),
// and the change mse(A, A') that the stopping test looks at is
//     |A - A'|^2 = tr(A^T A) - 2 tr((A^T X) M') + tr(A'^T A').
// With (G, C) = (A^T A, A^T X) as the state of each side, one iteration is, in the reference's order
// (Gauss-Seidel: the A_K update sees the new A_Q),
//     B_Q = Gq^-1 Cq,  B_K = Gk^-1 Ck
//     Mq'^T = (Gk + B_Q B_Q^T)^-1 (Ck + B_Q)          T = Mq'^T Sq      Gq' = Mq'^T T^T     Cq' = T
//     Mk'^T = (Gq' + B_K B_K^T)^-1 (T + B_K)          U = Mk'^T Sk      Gk' = Mk'^T U^T     Ck' = U
// and this holds from the first iteration on (there G, C come from the given initial factors).  The long
// axis is read for Sq, Sk and the initial (G, C) before the loop and once more at the end, to form
// A_Q = Q Mq and A_K = K Mk: six passes whatever the iteration count, where the row-by-row formulation
// makes two per iteration plus two.
//
// Sq and Sk square the condition number of the inputs, so the d x d algebra is done in fp64 (vector
// ALU: these are 32 independent problems of a few MFLOP each); the sums Sq, Sk themselves are exact
// bf16 x bf16 products added in fp32 tile by tile and across tiles, then across splits in fp64.  Measured
// against the fp64 restatement the results are closer than the same iteration in fp32 LAPACK.
#include <algorithm>

#include "common.hpp"
#include "ctx.hpp"

namespace lrqk {

typedef float gd_floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 gd_bf16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ int gd_mfma_row(int lane, int v) { return ((v >> 2) << 3) + ((lane >> 5) << 2) + (v & 3); }

// ----------------------------------------------------------------------------- X^T X
// grid (S, x heads); 8 waves share the rows (128 per step, staged in LDS as they lie in memory); wave w owns
// the output blocks (w / 2, 2 (w % 2)) and (w / 2, 2 (w % 2) + 1) of 32 x 32.  A lane's operand for column
// block nb is eight rows of one column, which the transposing LDS read delivers four at a time; every 32-row
// tile is summed in a fresh accumulator and added to the running total in fp32 (the matrix cores do not round
// to nearest when they add to a large accumulator).
constexpr int kXtxWaves = 8, kXtxThreads = kXtxWaves * kWave, kXtxRows = 128, kXtxD = 128;
constexpr int kXtxLd = kXtxD + 16;  // bf16 elements per staged row: 288 bytes, so four successive rows start 8 banks apart

__global__ __launch_bounds__(kXtxThreads) void pf_xtx_kernel(const bf16_t* __restrict__ X, int64_t l,
                                                             float* __restrict__ part, int S) {
  __shared__ __align__(16) uint16_t x_s[kXtxRows * kXtxLd];
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int col = lane & 31, half = lane >> 5;
  const int xh = blockIdx.y, s = blockIdx.x;
  const bf16_t* Xh = X + (int64_t)xh * l * kXtxD;
  const int nb1 = wave >> 1, nb2 = 2 * (wave & 1);
  constexpr int NL = kXtxRows * kXtxD / (kXtxThreads * 8);  // 16-byte loads per thread and step
  // One step ahead is all that pays: with two steps of rows in flight per workgroup the kernel is slower
  // (65 against 54 us at 32 heads x 32K rows).
  uint4 pre_a[NL];
  auto issue = [&](int64_t t0, uint4 (&dst)[NL]) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int e = (i * kXtxThreads + tid) * 8;  // element of the 128 x 128 step
      const int64_t row = t0 + e / kXtxD;
      dst[i] = *reinterpret_cast<const uint4*>(Xh + min(row, l - 1) * kXtxD + e % kXtxD);
    }
  };
  gd_floatx16 acc0, acc1;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc0[v] = acc1[v] = 0.0f;
  // An operand of the 32x32x16 product, lane (col, half): rows row0 + 8 half .. + 7 of column 32 nb + col.  The
  // transposing LDS read hands a lane four successive rows of its column: within 16 lanes, lane s points at
  // row s / 4, columns 4 (s % 4) .. + 3, and lane t receives column t of the four rows.
  auto operand = [&](int row0, int nb) {
    const int s16 = lane & 15;
    const uint16_t* p = &x_s[(row0 + 8 * half + (s16 >> 2)) * kXtxLd + 32 * nb + (col & 16) + 4 * (s16 & 3)];
    typedef short gd_v4s __attribute__((ext_vector_type(4)));
    typedef gd_v4s __attribute__((address_space(3))) * gd_lds_v4s;
    const gd_v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((gd_lds_v4s)p);
    const gd_v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((gd_lds_v4s)(p + 4 * kXtxLd));
    return __builtin_bit_cast(gd_bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  // split s takes the steps s, s + S, ...: the workgroups of a head walk the head's rows side by side
  const int64_t stride = (int64_t)S * kXtxRows;
  // one step: stage `cur` (the rows from t0 on), ask for the next step into `cur`, multiply
  auto step = [&](int64_t t0, uint4 (&cur)[NL]) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int e = (i * kXtxThreads + tid) * 8;
      const int row = e / kXtxD;
      *reinterpret_cast<uint4*>(&x_s[row * kXtxLd + e % kXtxD]) = t0 + row < l ? cur[i] : make_uint4(0, 0, 0, 0);
    }
    __syncthreads();
    if (t0 + stride < l) issue(t0 + stride, cur);
    const int tiles = (int)min((int64_t)4, (l - t0 + 31) / 32);
    for (int tile = 0; tile < tiles; ++tile) {
      gd_floatx16 t0a, t1a;
#pragma unroll
      for (int v = 0; v < 16; ++v) t0a[v] = t1a[v] = 0.0f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const int row0 = 32 * tile + 16 * kb;
        const gd_bf16x8 a = operand(row0, nb1);
        const gd_bf16x8 b0 = operand(row0, nb2), b1 = operand(row0, nb2 + 1);
        t0a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b0, t0a, 0, 0, 0);
        t1a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b1, t1a, 0, 0, 0);
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        acc0[v] += t0a[v];
        acc1[v] += t1a[v];
      }
    }
    __syncthreads();
  };
  const int64_t first = (int64_t)s * kXtxRows;
  if (first < l) issue(first, pre_a);
  for (int64_t t0 = first; t0 < l; t0 += stride) step(t0, pre_a);
  float* out = part + ((int64_t)xh * S + s) * kXtxD * kXtxD;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int i = 32 * nb1 + gd_mfma_row(lane, v);
    out[i * kXtxD + 32 * nb2 + col] = acc0[v];
    out[i * kXtxD + 32 * (nb2 + 1) + col] = acc1[v];
  }
}

// ----------------------------------------------------------------------------- X^T X and the sums over given factors
// One reading of X for both (the Q side, where every head has rows of its own): the workgroup stages 128 rows of X
// per step as pf_xtx_kernel does and its waves form, besides their two blocks of X^T X, the sums (A^T A, A^T X)
// over the given factors A (fp32, [head][l][r]).  Wave (a, ch) = (w / 2, w % 2) takes the 32-row group a of the
// step and the column blocks 2 ch, 2 ch + 1 of A^T X; of A^T A it takes the products of k block ch (the two
// waves' halves are added at the end).  The rows of A are read in the accumulator layout (element v of lane l: row
// gd_mfma_row(l, v), column l % 32) and split into three bf16 pieces (8 + 8 + 8 mantissa bits, exact); taken
// eight at a time these are an operand's k elements, and X's come out of LDS in the same order by the transposing
// read.  Products per 32 rows as in the row-by-row pass: all piece pairs of A^T A except lo x lo, three pieces of
// A times X; every 32-row group in a fresh accumulator.  part: [head][S][r][r + d] like the row-by-row pass
// writes them; xtx_part: [head][S][d][d].
// (Several heads that share their X -- the K side -- in one workgroup were tried and are slower: a wave then works
// through its heads' row groups one after the other, and their rows of A in flight together do not fit the
// registers.  Requesting the rows of A a step ahead also made this kernel slower: 142 against 126 us at 32 heads
// x 32K rows.)
__device__ __forceinline__ void gd_split3(float x, uint32_t& hi, uint32_t& mid, uint32_t& lo) {
  hi = __float_as_uint(x) & 0xffff0000u;
  const float r1 = x - __uint_as_float(hi);  // exact
  mid = __float_as_uint(r1) & 0xffff0000u;
  const float r2 = r1 - __uint_as_float(mid);  // exact, at most 8 significant bits
  lo = __float_as_uint(r2) & 0xffff0000u;
}
__device__ __forceinline__ uint32_t gd_pack2(uint32_t a, uint32_t b) { return (a >> 16) | (b & 0xffff0000u); }

__global__ __launch_bounds__(kXtxThreads) void pf_sums_kernel(const bf16_t* __restrict__ X, int64_t l,
                                                              const float* __restrict__ A, int r,
                                                              float* __restrict__ part, float* __restrict__ xtx_part,
                                                              int S) {
  // the tile of X; at the end the waves' sums pass through it
  __shared__ __align__(16) uint16_t x_s[kXtxRows * kXtxLd];
  static_assert(sizeof(x_s) >= kXtxWaves * 1024 * sizeof(float), "the reduction uses the tile's LDS");
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int col = lane & 31, half = lane >> 5;
  const int xh = blockIdx.y, s = blockIdx.x;
  const bf16_t* Xh = X + (int64_t)xh * l * kXtxD;
  const int wa = wave >> 1, ch = wave & 1;
  const int nb1 = wa, nb2 = 2 * ch;  // blocks of X^T X
  const float* Ah = A + (int64_t)xh * l * r;
  constexpr int NL = kXtxRows * kXtxD / (kXtxThreads * 8);
  uint4 pre_a[NL];
  auto issue = [&](int64_t t0, uint4 (&dst)[NL]) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int e = (i * kXtxThreads + tid) * 8;
      const int64_t row = t0 + e / kXtxD;
      dst[i] = *reinterpret_cast<const uint4*>(Xh + min(row, l - 1) * kXtxD + e % kXtxD);
    }
  };
  gd_floatx16 acc0, acc1, gAA, gAX[2];
#pragma unroll
  for (int v = 0; v < 16; ++v) acc0[v] = acc1[v] = gAA[v] = gAX[0][v] = gAX[1][v] = 0.0f;
  typedef short gd_v4s __attribute__((ext_vector_type(4)));
  typedef gd_v4s __attribute__((address_space(3))) * gd_lds_v4s;
  auto operand = [&](int row0, int nb) {  // rows row0 + 8 half .. + 7 of column 32 nb + col
    const int s16 = lane & 15;
    const uint16_t* p = &x_s[(row0 + 8 * half + (s16 >> 2)) * kXtxLd + 32 * nb + (col & 16) + 4 * (s16 & 3)];
    const gd_v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((gd_lds_v4s)p);
    const gd_v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((gd_lds_v4s)(p + 4 * kXtxLd));
    return __builtin_bit_cast(gd_bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  auto operand_acc = [&](int row0, int nb) {  // rows row0 + 4 half .. + 3 and the same + 8: the accumulator's order
    const int s16 = lane & 15;
    const uint16_t* p = &x_s[(row0 + 4 * half + (s16 >> 2)) * kXtxLd + 32 * nb + (col & 16) + 4 * (s16 & 3)];
    const gd_v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((gd_lds_v4s)p);
    const gd_v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((gd_lds_v4s)(p + 8 * kXtxLd));
    return __builtin_bit_cast(gd_bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  const int64_t stride = (int64_t)S * kXtxRows;
  float arow[16];  // this wave's rows of A of the step being multiplied, requested at the start of the step
  auto step = [&](int64_t t0, uint4 (&cur)[NL]) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {  // (requested first, consumed after the blocks of X^T X below)
      const int64_t row = min(t0 + 32 * wa + gd_mfma_row(lane, v), l - 1);
      arow[v] = Ah[row * r + min(col, r - 1)];
    }
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int e = (i * kXtxThreads + tid) * 8;
      const int row = e / kXtxD;
      *reinterpret_cast<uint4*>(&x_s[row * kXtxLd + e % kXtxD]) = t0 + row < l ? cur[i] : make_uint4(0, 0, 0, 0);
    }
    __syncthreads();
    if (t0 + stride < l) issue(t0 + stride, cur);
    const int tiles = (int)min((int64_t)4, (l - t0 + 31) / 32);
    for (int tile = 0; tile < tiles; ++tile) {
      gd_floatx16 t0a, t1a;
#pragma unroll
      for (int v = 0; v < 16; ++v) t0a[v] = t1a[v] = 0.0f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const int row0 = 32 * tile + 16 * kb;
        const gd_bf16x8 a = operand(row0, nb1);
        const gd_bf16x8 b0 = operand(row0, nb2), b1 = operand(row0, nb2 + 1);
        t0a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b0, t0a, 0, 0, 0);
        t1a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b1, t1a, 0, 0, 0);
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        acc0[v] += t0a[v];
        acc1[v] += t1a[v];
      }
    }
    if (t0 + 32 * wa < l) {  // (wave-uniform)
      // the three pieces of the group's rows of A, eight rows (one k block) at a time
      gd_bf16x8 cp[3][2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        uint32_t pc[3][8];
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          const int v = 8 * kb + q;
          const bool valid = t0 + 32 * wa + gd_mfma_row(lane, v) < l && col < r;
          gd_split3(valid ? arow[v] : 0.0f, pc[0][q], pc[1][q], pc[2][q]);
        }
#pragma unroll
        for (int pp = 0; pp < 3; ++pp)
          cp[pp][kb] = __builtin_bit_cast(gd_bf16x8, make_uint4(gd_pack2(pc[pp][0], pc[pp][1]), gd_pack2(pc[pp][2], pc[pp][3]),
                                                                gd_pack2(pc[pp][4], pc[pp][5]), gd_pack2(pc[pp][6], pc[pp][7])));
      }
      {
        gd_floatx16 t;
#pragma unroll
        for (int v = 0; v < 16; ++v) t[v] = 0.0f;
        // k block ch of A^T A, smallest pieces first
        const gd_bf16x8 c0 = ch ? cp[0][1] : cp[0][0], c1 = ch ? cp[1][1] : cp[1][0], c2 = ch ? cp[2][1] : cp[2][0];
        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(c1, c2, t, 0, 0, 0);
        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(c2, c1, t, 0, 0, 0);
        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(c0, c2, t, 0, 0, 0);
        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(c2, c0, t, 0, 0, 0);
        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(c1, c1, t, 0, 0, 0);
        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(c0, c1, t, 0, 0, 0);
        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(c1, c0, t, 0, 0, 0);
        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(c0, c0, t, 0, 0, 0);
#pragma unroll
        for (int v = 0; v < 16; ++v) gAA[v] += t[v];
      }
#pragma unroll
      for (int nbi = 0; nbi < 2; ++nbi) {
        gd_bf16x8 xb[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) xb[kb] = operand_acc(32 * wa + 16 * kb, 2 * ch + nbi);
        gd_floatx16 t;
#pragma unroll
        for (int v = 0; v < 16; ++v) t[v] = 0.0f;
#pragma unroll
        for (int pp = 2; pp >= 0; --pp)
#pragma unroll
          for (int kb = 0; kb < 2; ++kb) t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cp[pp][kb], xb[kb], t, 0, 0, 0);
#pragma unroll
        for (int v = 0; v < 16; ++v) gAX[nbi][v] += t[v];
      }
    }
    __syncthreads();
  };
  const int64_t first = (int64_t)s * kXtxRows;
  if (first < l) issue(first, pre_a);
  for (int64_t t0 = first; t0 < l; t0 += stride) step(t0, pre_a);
  {
    float* out = xtx_part + ((int64_t)xh * S + s) * kXtxD * kXtxD;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int i = 32 * nb1 + gd_mfma_row(lane, v);
      out[i * kXtxD + 32 * nb2 + col] = acc0[v];
      out[i * kXtxD + 32 * (nb2 + 1) + col] = acc1[v];
    }
  }
  // the waves' sums: pass 0 is A^T A (all waves), passes 1, 2 the column blocks 2 ch + 0 / + 1 of A^T X (the waves
  // with the same ch)
  float* sm = reinterpret_cast<float*>(x_s);
  const int ne = r * (r + kXtxD);
  float* outp = part + ((int64_t)xh * S + s) * ne;
#pragma unroll 1
  for (int blk = 0; blk < 3; ++blk) {
    float* mine = sm + wave * 1024;
#pragma unroll
    for (int v = 0; v < 16; ++v)
      mine[gd_mfma_row(lane, v) * 32 + col] = blk == 0 ? gAA[v] : (blk == 1 ? gAX[0][v] : gAX[1][v]);
    __syncthreads();
    const int n_out = (blk == 0 ? 1 : 2) * 1024;
    for (int o = tid; o < n_out; o += kXtxThreads) {
      const int e = o & 1023, c_half = blk == 0 ? -1 : (o >> 10);
      float v = 0.0f;
#pragma unroll
      for (int w = 0; w < kXtxWaves; ++w)
        if (c_half < 0 || (w & 1) == c_half) v += sm[w * 1024 + e];
      const int m = e >> 5, n = e & 31;
      if (blk == 0) {
        if (m < r && n < r) outp[m * (r + kXtxD) + n] = v;
      } else {
        const int cx = 32 * (2 * c_half + (blk - 1)) + n;
        if (m < r) outp[m * (r + kXtxD) + r + cx] = v;
      }
    }
    __syncthreads();
  }
}

// ----------------------------------------------------------------------------- A = X Mt^T for heads that share X
// The K side's last pass: the NH query heads of a kv head take their rows of A_K from the same rows of K, so one
// workgroup stages 128 rows of K per step (as pf_xtx_kernel does) and applies the NH heads' Mt to them: K is read
// once per kv head instead of once per query head.  Mt (fp32) lies in LDS as three bf16 pieces per head, X as it
// is; wave w takes head w / (8 / NH) and NH / 2 of the step's four 32-row groups; 24 products of 32x32x16 per
// group (X times the three pieces), fp32 accuracy as in the row-by-row pass.  grid (S, kv heads); split s takes
// the steps s, s + S, ...
constexpr int kApLd = kXtxD + 8;  // bf16 elements per staged row: 16-byte operand reads want rows 4 banks apart
template <int NH>
__global__ __launch_bounds__(kXtxThreads) void pf_apply_shared_kernel(const bf16_t* __restrict__ X, int64_t l,
                                                                      const float* __restrict__ Mt, int r,
                                                                      float* __restrict__ A, int S) {
  static_assert(NH == 2 || NH == 4, "query heads per kv head");
  extern __shared__ __align__(16) uint16_t ap_s[];
  uint16_t* x_s = ap_s;                          // [128][kApLd]
  uint16_t* mt_s = ap_s + kXtxRows * kApLd;      // [NH][3][32][kApLd]
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int col = lane & 31, half = lane >> 5;
  const int xh = blockIdx.y, s = blockIdx.x;
  const bf16_t* Xh = X + (int64_t)xh * l * kXtxD;
  constexpr int WPH = kXtxWaves / NH, GPW = 4 / WPH;  // waves per head, row groups per wave and step
  const int hl = wave / WPH, g0 = (wave % WPH) * GPW;
  float* Ah = A + ((int64_t)xh * NH + hl) * l * r;
  for (int e = tid; e < NH * 32 * kXtxD; e += kXtxThreads) {
    const int hh = e / (32 * kXtxD), n = (e / kXtxD) % 32, k = e % kXtxD;
    const float v = n < r ? Mt[(((int64_t)xh * NH + hh) * r + n) * kXtxD + k] : 0.0f;
    uint32_t p0, p1, p2;
    gd_split3(v, p0, p1, p2);
    mt_s[((hh * 3 + 0) * 32 + n) * kApLd + k] = (uint16_t)(p0 >> 16);
    mt_s[((hh * 3 + 1) * 32 + n) * kApLd + k] = (uint16_t)(p1 >> 16);
    mt_s[((hh * 3 + 2) * 32 + n) * kApLd + k] = (uint16_t)(p2 >> 16);
  }
  constexpr int NL = kXtxRows * kXtxD / (kXtxThreads * 8);
  static_assert(NL == 4, "four 16-byte loads per thread and step");
  uint4 pre0 = make_uint4(0, 0, 0, 0), pre1 = pre0, pre2 = pre0, pre3 = pre0;
  auto issue = [&](int64_t t0) {
    auto ld = [&](int i) {
      const int e = (i * kXtxThreads + tid) * 8;
      const int64_t row = t0 + e / kXtxD;
      return *reinterpret_cast<const uint4*>(Xh + min(row, l - 1) * kXtxD + e % kXtxD);
    };
    pre0 = ld(0);
    pre1 = ld(1);
    pre2 = ld(2);
    pre3 = ld(3);
  };
  auto stage = [&](int i, const uint4& v) {
    const int e = (i * kXtxThreads + tid) * 8;
    *reinterpret_cast<uint4*>(&x_s[(e / kXtxD) * kApLd + e % kXtxD]) = v;  // (rows beyond l are never stored from)
  };
  const int64_t stride = (int64_t)S * kXtxRows;
  const int64_t first = (int64_t)s * kXtxRows;
  if (first < l) issue(first);
  for (int64_t t0 = first; t0 < l; t0 += stride) {
    stage(0, pre0);
    stage(1, pre1);
    stage(2, pre2);
    stage(3, pre3);
    __syncthreads();  // (the first one also covers the staging of Mt)
    if (t0 + stride < l) issue(t0 + stride);
#pragma unroll
    for (int j = 0; j < GPW; ++j) {
      const int g = g0 + j;
      if (t0 + 32 * g >= l) continue;  // (wave-uniform)
      gd_floatx16 c;
#pragma unroll
      for (int v = 0; v < 16; ++v) c[v] = 0.0f;
#pragma unroll
      for (int kb = 0; kb < kXtxD / 16; ++kb) {
        const gd_bf16x8 xa = *reinterpret_cast<const gd_bf16x8*>(&x_s[(32 * g + col) * kApLd + kb * 16 + 8 * half]);
#pragma unroll
        for (int pp = 0; pp < 3; ++pp) {
          const gd_bf16x8 m =
              *reinterpret_cast<const gd_bf16x8*>(&mt_s[((hl * 3 + pp) * 32 + col) * kApLd + kb * 16 + 8 * half]);
          c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa, m, c, 0, 0, 0);
        }
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int64_t row = t0 + 32 * g + gd_mfma_row(lane, v);
        if (row < l && col < r) Ah[row * r + col] = c[v];
      }
    }
    __syncthreads();
  }
}

// A_K = K Mk for all query heads, reading K once per kv head.  Returns false if this grouping of heads has no
// kernel here (the caller then runs its row-by-row pass).
bool prefill_apply_shared(const void* k, const float* mt_k, float* a_k, int b, int hq, int hkv, int64_t l, int r,
                          hipStream_t st, int* rc_out) {
  *rc_out = LRQK_OK;
  const int nh = hq / hkv, bkv = b * hkv;
  if (nh != 2 && nh != 4) return false;
  const int S = (int)std::max<int64_t>(1, std::min<int64_t>(std::max(1, 256 / bkv), (l + kXtxRows - 1) / kXtxRows));
  const size_t smem = (size_t)(kXtxRows + nh * 3 * 32) * kApLd * sizeof(uint16_t);
  auto kern = nh == 2 ? pf_apply_shared_kernel<2> : pf_apply_shared_kernel<4>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  if (e != hipSuccess) {
    *rc_out = set_error(LRQK_EHIP, "hipFuncSetAttribute failed: %s", hipGetErrorString(e));
    return true;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)S, (unsigned)bkv), dim3(kXtxThreads), smem, st, (const bf16_t*)k, l, mt_k, r,
                     a_k, S);
  e = hipGetLastError();
  if (e != hipSuccess) *rc_out = set_error(LRQK_EHIP, "launch failed: %s", hipGetErrorString(e));
  return true;
}

// ----------------------------------------------------------------------------- d x d algebra, fp64
constexpr int kGdThreads = 256;   // four waves: 32 of the 128 right-hand columns each (one wave per SIMD: 512 registers)
constexpr int kGdD = 128;
constexpr int kGdLd = 34;         // doubles per row of a transposed r x d matrix in LDS ([d][34], 16-byte rows)
constexpr int kGdLg = 33;         // doubles per row of an r x r matrix in LDS

// ---- two systems [W | RHS] (W 32 x 32 symmetric positive definite up to rounding, rows/columns beyond r the
// identity; RHS 32 x 128) solved side by side by block Gauss-Jordan elimination on the fp64 matrix cores, four
// pivots per step.  The matrices live in the accumulator layout of 16 x 16 tiles (element v of lane l = row
// 16 rt + l / 16 + 4 v, column 16 u + l % 16 of tile (rt, u)): each of the four waves holds W itself (every wave
// eliminates its own copy: no wave waits for another, the solve has no barrier) and 32 columns of RHS.
// Step m, with P the pivot columns 4 m .. 4 m + 3 (32 x 4) and D its rows 4 m .. 4 m + 3:
//     X <- X - (P D^-1) X[4 m .. 4 m + 3, :] outside the pivot rows,   X[pivot rows] <- D^-1 X[pivot rows]
// (one product: the pivot rows' accumulators are cleared and their left operand is D^-1 itself), which clears the
// pivot columns elsewhere.  The right-hand
// operand, four rows of X, is element m % 4 of the lane's own tile in row tile m / 4: no data moves for it.  The
// left operand needs P by rows: the lanes that hold the pivot columns put them into the wave's own LDS slot, the
// two pivot blocks are inverted side by side in the two halves of the wave (by 2 x 2 blocks, no pivoting) and
// handed round through the same slot.  The products on W come first (the next step waits for them only); those on
// RHS run on the matrix cores while the next step's inverse is computed.
typedef double gd_v4d __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void gd_wave_sync() {  // orders one wave's LDS writes and reads
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// 1 / x to ~1e-14: the hardware estimate (2^-23) and one Newton step.  The pivot blocks' inverses need no more
// (their error enters the solution once, scaled by the condition number, far below the rounding of the fp32 sums
// the systems are built from), and every operation here is on the solve's dependent chain.
__device__ __forceinline__ double gd_rcp(double x) {
  const double inv = __builtin_amdgcn_rcp(x);
  return fma(fma(-x, inv, 1.0), inv, inv);
}

// R = D^-1 for a 4 x 4 matrix with positive definite symmetric part, by 2 x 2 blocks (no pivoting):
// D = [[A, B], [C, E]], S = E - C A^-1 B, D^-1 = [[A^-1 + Y S^-1 Z, -Y S^-1], [-S^-1 Z, S^-1]], Y = A^-1 B, Z = C A^-1.
// D is taken as it is, not as symmetric: the Gram sums it comes from are symmetric only up to their rounding, and
// the elimination around it uses both triangles.
__device__ __forceinline__ void gd_inv4(const double (&D)[4][4], double (&R)[4][4]) {
  const double ia = gd_rcp(fma(D[0][0], D[1][1], -D[0][1] * D[1][0]));
  const double a00 = D[1][1] * ia, a01 = -D[0][1] * ia, a10 = -D[1][0] * ia, a11 = D[0][0] * ia;  // A^-1
  // Y = A^-1 B  (B = D[0..1][2..3]),  Z = C A^-1  (C = D[2..3][0..1])
  const double y00 = fma(a00, D[0][2], a01 * D[1][2]), y01 = fma(a00, D[0][3], a01 * D[1][3]);
  const double y10 = fma(a10, D[0][2], a11 * D[1][2]), y11 = fma(a10, D[0][3], a11 * D[1][3]);
  const double z00 = fma(D[2][0], a00, D[2][1] * a10), z01 = fma(D[2][0], a01, D[2][1] * a11);
  const double z10 = fma(D[3][0], a00, D[3][1] * a10), z11 = fma(D[3][0], a01, D[3][1] * a11);
  // S = E - C Y
  const double s00 = D[2][2] - fma(D[2][0], y00, D[2][1] * y10), s01 = D[2][3] - fma(D[2][0], y01, D[2][1] * y11);
  const double s10 = D[3][2] - fma(D[3][0], y00, D[3][1] * y10), s11 = D[3][3] - fma(D[3][0], y01, D[3][1] * y11);
  const double is = gd_rcp(fma(s00, s11, -s01 * s10));
  const double t00 = s11 * is, t01 = -s01 * is, t10 = -s10 * is, t11 = s00 * is;  // S^-1
  // U = Y S^-1 (upper right, negated), V = S^-1 Z (lower left, negated)
  const double u00 = fma(y00, t00, y01 * t10), u01 = fma(y00, t01, y01 * t11);
  const double u10 = fma(y10, t00, y11 * t10), u11 = fma(y10, t01, y11 * t11);
  const double v00 = fma(t00, z00, t01 * z10), v01 = fma(t00, z01, t01 * z11);
  const double v10 = fma(t10, z00, t11 * z10), v11 = fma(t10, z01, t11 * z11);
  R[0][0] = a00 + fma(u00, z00, u01 * z10);
  R[0][1] = a01 + fma(u00, z01, u01 * z11);
  R[1][0] = a10 + fma(u10, z00, u11 * z10);
  R[1][1] = a11 + fma(u10, z01, u11 * z11);
  R[0][2] = -u00; R[0][3] = -u01; R[1][2] = -u10; R[1][3] = -u11;
  R[2][0] = -v00; R[2][1] = -v01; R[3][0] = -v10; R[3][1] = -v11;
  R[2][2] = t00; R[2][3] = t01; R[3][2] = t10; R[3][3] = t11;
}

struct GdSys {
  gd_v4d w[2][2];  // W: [row tile][column tile]
  gd_v4d x[2][2];  // this wave's columns of RHS: [row tile][column tile 2 wave + u]
};
constexpr int kGdSlot = 2 * 128 + 32;                    // per wave: P of both systems, the two inverses
constexpr int kGdPivDoubles = (kGdThreads / 64) * kGdSlot;
__device__ __forceinline__ void gd_solve_pair(GdSys (&s)[2], double* __restrict__ piv) {
  const int lane = lane_id(), wave = wave_id();
  const int li = lane & 15, lk = lane >> 4;
  double* pb = piv + wave * kGdSlot;
  double* xch = pb + 256;
#pragma unroll
  for (int m = 0; m < 8; ++m) {
    const int tp = m >> 2, vp = m & 3;  // the pivots' tile (row tile of the pivot rows, column tile of W) and element
    {
      const int kk = li - 4 * vp;
      if (kk >= 0 && kk < 4) {
#pragma unroll
        for (int sy = 0; sy < 2; ++sy)
#pragma unroll
          for (int rt = 0; rt < 2; ++rt)
#pragma unroll
            for (int v = 0; v < 4; ++v) pb[sy * 128 + (16 * rt + lk + 4 * v) * 4 + kk] = s[sy].w[rt][tp][v];
      }
    }
    gd_wave_sync();
    {
      const int mine = lane >> 5;
      const double* P = pb + mine * 128;
      double D[4][4], R[4][4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const double2 lo = *reinterpret_cast<const double2*>(&P[(4 * m + i) * 4]);
        const double2 hi = *reinterpret_cast<const double2*>(&P[(4 * m + i) * 4 + 2]);
        D[i][0] = lo.x; D[i][1] = lo.y; D[i][2] = hi.x; D[i][3] = hi.y;
      }
      gd_inv4(D, R);
      if ((lane & 31) == 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          *reinterpret_cast<double2*>(&xch[mine * 16 + i * 4]) = make_double2(R[i][0], R[i][1]);
          *reinterpret_cast<double2*>(&xch[mine * 16 + i * 4 + 2]) = make_double2(R[i][2], R[i][3]);
        }
      }
      gd_wave_sync();
    }
    double aop[2][2];
#pragma unroll
    for (int sy = 0; sy < 2; ++sy) {
      const double* P = pb + sy * 128;
      double ic[4];  // column l / 16 of the inverse
#pragma unroll
      for (int k = 0; k < 4; ++k) ic[k] = xch[sy * 16 + k * 4 + lk];
#pragma unroll
      for (int rt = 0; rt < 2; ++rt) {
        const int row = 16 * rt + li;
        const double2 lo = *reinterpret_cast<const double2*>(&P[row * 4]);
        const double2 hi = *reinterpret_cast<const double2*>(&P[row * 4 + 2]);
        // pivot rows: the rows of D^-1 themselves (their accumulators are cleared below, so they come out as
        // D^-1 X and not as X - (I - D^-1) X, which cancels in its leading digits when D is far from unit size:
        // with a diagonal of 1e12 solutions were off by 5e-3 where the conditioning allowed 1e-11)
        const double own = xch[sy * 16 + (row & 3) * 4 + lk];
        const double oth = -fma(lo.x, ic[0], fma(lo.y, ic[1], fma(hi.x, ic[2], hi.y * ic[3])));
        aop[sy][rt] = (row >> 2) == m ? own : oth;
      }
    }
    gd_wave_sync();  // (the reads of the slot precede the next step's writes)
    // W: the column tiles from the pivots' on (those before hold finished unit columns: zero in the pivot rows)
#pragma unroll
    for (int sy = 0; sy < 2; ++sy)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        if (u < tp) continue;
        const double bop = s[sy].w[tp][u][vp];
        s[sy].w[tp][u][vp] = 0.0;
#pragma unroll
        for (int rt = 0; rt < 2; ++rt)
          s[sy].w[rt][u] = __builtin_amdgcn_mfma_f64_16x16x4f64(aop[sy][rt], bop, s[sy].w[rt][u], 0, 0, 0);
      }
#pragma unroll
    for (int sy = 0; sy < 2; ++sy)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const double bop = s[sy].x[tp][u][vp];
        s[sy].x[tp][u][vp] = 0.0;
#pragma unroll
        for (int rt = 0; rt < 2; ++rt)
          s[sy].x[rt][u] = __builtin_amdgcn_mfma_f64_16x16x4f64(aop[sy][rt], bop, s[sy].x[rt][u], 0, 0, 0);
      }
  }
}

// One system filled from fw(row, column of W) and fx(row, column of RHS) / its solution handed to g(row, column
// of RHS, value).
template <typename FW, typename FX>
__device__ __forceinline__ void gd_fill(GdSys& t, FW&& fw, FX&& fx) {
  const int lane = lane_id(), wave = wave_id();
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int i = 16 * rt + (lane >> 4) + 4 * v;
        t.w[rt][u][v] = fw(i, 16 * u + (lane & 15));
        t.x[rt][u][v] = fx(i, 16 * (2 * wave + u) + (lane & 15));
      }
}
template <typename G>
__device__ __forceinline__ void gd_drain(const gd_v4d (&x)[2][2], G&& g) {
  const int lane = lane_id(), wave = wave_id();
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int v = 0; v < 4; ++v) g(16 * rt + (lane >> 4) + 4 * v, 16 * (2 * wave + u) + (lane & 15), x[rt][u][v]);
}

// out[i][j] = sum over c < 128 of PT[c][i] * RT[c][j]   (two r x d matrices, stored transposed) on the fp64 matrix
// cores, by waves 0..3: wave w owns the 16 x 16 tile (w / 2, w % 2) and runs its 32 products of depth 4 in a row.
// Element v of a thread is out[gd_outer_row(v)][gd_outer_col()].  Rows/columns beyond r come out as what the zero
// padding of PT, RT gives.
__device__ __forceinline__ int gd_outer_row(int v) { return 16 * (wave_id() >> 1) + (lane_id() >> 4) + 4 * v; }
__device__ __forceinline__ int gd_outer_col() { return 16 * (wave_id() & 1) + (lane_id() & 15); }
__device__ __forceinline__ void gd_outer(const double* __restrict__ PT, const double* __restrict__ RT, double (&o)[4]) {
  o[0] = o[1] = o[2] = o[3] = 0.0;
  if (threadIdx.x < 256) {
    const int lane = lane_id(), wave = wave_id();
    const int li = lane & 15, lk = lane >> 4;
    const double* pa = PT + lk * kGdLd + 16 * (wave >> 1) + li;
    const double* pb = RT + lk * kGdLd + 16 * (wave & 1) + li;
    gd_v4d acc = gd_v4d{0.0, 0.0, 0.0, 0.0};
#pragma unroll 8
    for (int c = 0; c < kGdD; c += 4)
      acc = __builtin_amdgcn_mfma_f64_16x16x4f64(pa[c * kGdLd], pb[c * kGdLd], acc, 0, 0, 0);
#pragma unroll
    for (int v = 0; v < 4; ++v) o[v] = acc[v];
  }
}

// TT[c][i] = sum over k of MT[k][i] * S[k][c]   (the transposed form of Mt S, S symmetric d x d in global
// memory) on the fp64 matrix cores: 16 x 16 x 4 tiles, A operand lane l = Mt[i0 + l % 16][k0 + l / 16] (from the
// LDS copy), B operand lane l = S[k0 + l / 16][c0 + l % 16] (16 independent loads per lane in flight), result
// element v of lane l = row l / 16 + 4 v, column l % 16 of the tile.  Waves 0..3 take 32 columns each.
// One barrier.
__device__ __forceinline__ void gd_times_s(const double* __restrict__ MT, const double* __restrict__ S,
                                           double* __restrict__ TT) {
  const int lane = lane_id(), wave = wave_id();
  if (wave < 4) {
    const int li = lane & 15, lk = lane >> 4;
    const int c0 = 32 * wave;
    gd_v4d acc[2][2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int ct = 0; ct < 2; ++ct) acc[rt][ct] = gd_v4d{0.0, 0.0, 0.0, 0.0};
    for (int kb = 0; kb < kGdD; kb += 32) {
      double bv[8][2];
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) bv[u][ct] = S[(int64_t)(kb + 4 * u + lk) * kGdD + c0 + 16 * ct + li];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int k = kb + 4 * u + lk;
        const double a0 = MT[k * kGdLd + li], a1 = MT[k * kGdLd + 16 + li];
        acc[0][0] = __builtin_amdgcn_mfma_f64_16x16x4f64(a0, bv[u][0], acc[0][0], 0, 0, 0);
        acc[0][1] = __builtin_amdgcn_mfma_f64_16x16x4f64(a0, bv[u][1], acc[0][1], 0, 0, 0);
        acc[1][0] = __builtin_amdgcn_mfma_f64_16x16x4f64(a1, bv[u][0], acc[1][0], 0, 0, 0);
        acc[1][1] = __builtin_amdgcn_mfma_f64_16x16x4f64(a1, bv[u][1], acc[1][1], 0, 0, 0);
      }
    }
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int ct = 0; ct < 2; ++ct)
#pragma unroll
        for (int v = 0; v < 4; ++v) TT[(c0 + 16 * ct + li) * kGdLd + 16 * rt + lk + 4 * v] = acc[rt][ct][v];
  }
  __syncthreads();
}

// sum of v over the workgroup, result in every thread.  red: kGdThreads / 64 doubles.  Two barriers.
__device__ __forceinline__ double gd_block_sum(double v, double* red) {
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  if (lane_id() == 0) red[wave_id()] = v;
  __syncthreads();
  double t = 0.0;
  for (int w = 0; w < kGdThreads / kWave; ++w) t += red[w];
  __syncthreads();
  return t;
}

struct GdArgs {
  // initial (G, C) of the two sides as the first Gram passes left them: S partial sums of [r][r + d] floats per head
  const float* partQ;
  const float* partK;
  int S;                // splits of partQ
  int S_k;              // splits of partK
  const double* Sq;     // [bh][d][d]
  const double* Sk;     // [b * hkv][d][d]
  double* G;            // [2][bh][32][32]  (side 0: Q, 1: K), padded with the identity
  double* C;            // [2][bh][32][d]   zero rows beyond r
  double* BqT;          // [bh][d][32]      B_Q of the state, transposed (written by an iteration for the next)
  double* delta;        // [iters][2][bh]   squared changes |A - A'|^2 per head
  int* flags;           // [iters + 1]
  float* Mt_q;          // [bh][r][d]  Mq^T, Mk^T for the final row-by-row pass
  float* Mt_k;
  float* b_q;           // [bh][r][d] outputs
  float* b_k;
  int bh, hq, hkv, r;
  int64_t l;
  float tol;
};

// One launch for everything that only adds partial sums up, in fp64:
//   blocks [0, nq)        Sq[x][e] = sum over the Sx splits of xq_part[x][s][e]   (nq = bh * d * d / 256)
//   blocks [nq, nq + nk)  Sk likewise over the bkv distinct K heads
//   the rest              the state (G, C) of both sides from the first Gram passes: S partial sums of [G | C]
//                         packed as [r][r + d] floats per head; G padded with the identity, C with zero rows
//                         (20 blocks per head and side).
constexpr int kGdInitBlocks = (32 * (32 + kGdD) + 255) / 256;
__global__ __launch_bounds__(256) void pf_gramdom_init_kernel(GdArgs a, const float* __restrict__ xq_part, int Sx,
                                                              const float* __restrict__ xk_part, int Sxk, int bkv,
                                                              double* __restrict__ Sq, double* __restrict__ Sk) {
  constexpr int dd = kGdD * kGdD, per = dd / 256;
  int blk = blockIdx.x;
  const int nq = a.bh * per, nk = bkv * per;
  if (blk < nq + nk) {
    const bool k_side = blk >= nq;
    if (k_side) blk -= nq;
    const int x = blk / per, e = (blk % per) * 256 + threadIdx.x;
    const int S = k_side ? Sxk : Sx;
    const float* part = (k_side ? xk_part : xq_part) + (int64_t)x * S * dd + e;
    double v = 0.0;
#pragma unroll 4
    for (int s = 0; s < S; ++s) v += (double)part[(int64_t)s * dd];
    (k_side ? Sk : Sq)[(int64_t)x * dd + e] = v;
    return;
  }
  blk -= nq + nk;
  const int h = blk / (2 * kGdInitBlocks), side = (blk / kGdInitBlocks) & 1;
  const int r = a.r, d = kGdD;
  const int e = (blk % kGdInitBlocks) * 256 + threadIdx.x;
  if (e >= 32 * (32 + d)) return;
  const int ne = r * (r + d);
  const int Sn = side ? a.S_k : a.S;
  const float* part = (side ? a.partK : a.partQ) + (int64_t)h * Sn * ne;
  const int i = e / (32 + d), j = e % (32 + d);
  double v = 0.0;
  if (i < r && (j >= 32 || j < r)) {
    const int src = i * (r + d) + (j < 32 ? j : r + (j - 32));
    for (int s = 0; s < Sn; ++s) v += (double)part[(int64_t)s * ne + src];
  } else if (j < 32) {
    v = i == j ? 1.0 : 0.0;
  }
  if (j < 32)
    a.G[((int64_t)side * a.bh + h) * 1024 + i * 32 + j] = v;
  else
    a.C[((int64_t)side * a.bh + h) * 32 * d + i * d + (j - 32)] = v;
}

// stage 0: one iteration `it`; stage 2: the final B_Q, B_K from the state.
__global__ __launch_bounds__(kGdThreads) void pf_gramdom_kernel(int stage, int it, GdArgs a) {
  extern __shared__ __align__(16) double gsm[];
  double* MT = gsm;                         // [128][34]  Mq'^T, later Mk'^T (transposed storage)
  double* TT = MT + kGdD * kGdLd;           // [128][34]  T, later U
  double* BT = TT + kGdD * kGdLd;           // [128][34]  B_Q, later B_K
  double* Gs = BT + kGdD * kGdLd;           // [3][32][33]
  double* piv = Gs + 3 * 32 * kGdLg;        // [2 buffers][2 systems][32][4]
  double* red = piv + kGdPivDoubles;        // [8]
  const int tid = threadIdx.x;
  const int h = blockIdx.x;
  const int r = a.r, d = kGdD, bh = a.bh;
  const int b = h / a.hq, kvh = (h % a.hq) / (a.hq / a.hkv);
  const double* Sq = a.Sq + (int64_t)h * d * d;
  const double* Sk = a.Sk + ((int64_t)b * a.hkv + kvh) * d * d;
  double* Gq = a.G + (int64_t)h * 1024;
  double* Gk = a.G + ((int64_t)bh + h) * 1024;
  double* Cq = a.C + (int64_t)h * 32 * d;
  double* Ck = a.C + ((int64_t)bh + h) * 32 * d;

  // ---- what an iteration reads of its state is requested before anything else: the handed-over B_Q and this
  // wave's tiles of Ck and Cq (Cq is rewritten only at the end of the Q side's step, Ck at the end of the iteration)
  const bool fresh = stage == 2 || it == 0;
  constexpr int kBqPer = 32 * kGdD / kGdThreads;
  double bq_pre[kBqPer];
  gd_v4d ckt[2][2], cqt[2][2];
  if (!fresh) {
    const double* src = a.BqT + (int64_t)h * 32 * d;  // [32][d]
#pragma unroll
    for (int u = 0; u < kBqPer; ++u) bq_pre[u] = src[tid + u * kGdThreads];
  }
  if (stage == 0) {
    const int lane = lane_id(), wave = wave_id();
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int e = (16 * rt + (lane >> 4) + 4 * v) * d + 16 * (2 * wave + u) + (lane & 15);
          ckt[rt][u][v] = Ck[e];
          cqt[rt][u][v] = Cq[e];
        }
  }
  if (stage == 0) {
    // ---- the stopping test of the previous iteration (batch-wide, as the reference takes it)
    int done = 0;
    if (it > 0) {
      done = a.flags[it - 1];
      if (!done) {
        const double* dq = a.delta + ((int64_t)(it - 1) * 2 + 0) * bh;
        const double* dk = a.delta + ((int64_t)(it - 1) * 2 + 1) * bh;
        double sq = 0.0, sk = 0.0;
        for (int i = tid; i < bh; i += kGdThreads) {
          sq += dq[i];
          sk += dk[i];
        }
        sq = gd_block_sum(sq, red);
        sk = gd_block_sum(sk, red);
        const double n = (double)bh * (double)a.l * (double)r;
        done = fmax(sq / n, sk / n) < (double)a.tol;
      }
    }
    if (h == 0 && tid == 0) a.flags[it] = done;
    if (done) return;
  }

  // Of an iteration's r x r systems only two follow each other: B_K = Gk^-1 Ck does not depend on the Q side's
  // step and is solved beside it, and the next iteration's B_Q = Gq'^-1 Cq' is solved beside the K side's step
  // and handed over in `BqT`.  Iteration 0 (and the final stage) start from the state alone: B_Q and B_K side by side.
  GdSys sy[2];
  gd_v4d bk[2][2];  // B_K in the layout of the right-hand sides
  double* BqT = a.BqT + (int64_t)h * 32 * d;  // [32][d]
  if (fresh) {
    gd_fill(sy[0], [&](int i, int j) { return Gq[i * 32 + j]; }, [&](int i, int cc) { return Cq[i * d + cc]; });
    if (stage == 2)
      gd_fill(sy[1], [&](int i, int j) { return Gk[i * 32 + j]; }, [&](int i, int cc) { return Ck[i * d + cc]; });
    else
      gd_fill(sy[1], [&](int i, int j) { return i == j ? 1.0 : 0.0; }, [&](int, int) { return 0.0; });
    gd_solve_pair(sy, piv);
    if (stage == 2) {
      float* oq = a.b_q + (int64_t)h * r * d;
      float* ok = a.b_k + (int64_t)h * r * d;
      gd_drain(sy[0].x, [&](int i, int cc, double v) { if (i < r) oq[i * d + cc] = (float)v; });
      gd_drain(sy[1].x, [&](int i, int cc, double v) { if (i < r) ok[i * d + cc] = (float)v; });
      return;
    }
    gd_drain(sy[0].x, [&](int i, int cc, double v) { BT[cc * kGdLd + i] = v; });
  } else {
#pragma unroll
    for (int u = 0; u < kBqPer; ++u) {
      const int e = tid + u * kGdThreads;
      BT[(e % d) * kGdLd + e / d] = bq_pre[u];
    }
  }
  __syncthreads();
  // ---- W1 = Gk + B_Q B_Q^T
  {
    double o[4];
    gd_outer(BT, BT, o);
    const int j = gd_outer_col();
#pragma unroll
    for (int u = 0; u < 4; ++u) Gs[gd_outer_row(u) * kGdLg + j] = Gk[gd_outer_row(u) * 32 + j] + o[u];
  }
  __syncthreads();
  // ---- Mq'^T = W1^-1 (Ck + B_Q) beside B_K = Gk^-1 Ck
  gd_fill(sy[0], [&](int i, int j) { return Gs[i * kGdLg + j]; }, [&](int i, int cc) { return BT[cc * kGdLd + i]; });
  gd_fill(sy[1], [&](int i, int j) { return Gk[i * 32 + j]; }, [&](int, int) { return 0.0; });
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      sy[0].x[rt][u] += ckt[rt][u];
      sy[1].x[rt][u] = ckt[rt][u];
    }
  __syncthreads();  // (every read of B_Q precedes the rewriting of the B tile below)
  gd_solve_pair(sy, piv);
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int u = 0; u < 2; ++u) bk[rt][u] = sy[1].x[rt][u];
  // ---- the B tile now holds B_K; Mq'^T goes to its tile and to the caller, with the sum of Cq (the old one) . Mq'^T
  gd_drain(bk, [&](int i, int cc, double v) { BT[cc * kGdLd + i] = v; });
  double part_q = 0.0;
  {
    float* mt = a.Mt_q + (int64_t)h * r * d;
    gd_drain(sy[0].x, [&](int i, int cc, double v) {
      MT[cc * kGdLd + i] = v;
      if (i < r) mt[i * d + cc] = (float)v;
    });
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int v = 0; v < 4; ++v) part_q = fma(cqt[rt][u][v], sy[0].x[rt][u][v], part_q);
  }
  double tr_old = 0.0;
  if (tid < 32) tr_old = tid < r ? Gq[tid * 32 + tid] : 0.0;
  __syncthreads();
  {
    double o[4];
    gd_outer(BT, BT, o);
    if (tid < 256) {
      const int j = gd_outer_col();
#pragma unroll
      for (int u = 0; u < 4; ++u) Gs[32 * kGdLg + gd_outer_row(u) * kGdLg + j] = o[u];
    }
  }
  // ---- T = Mq'^T Sq, Gq' = Mq'^T T^T
  gd_times_s(MT, Sq, TT);
  {
    double o[4];
    gd_outer(MT, TT, o);
    double tr_new = 0.0;
    if (tid < 256) {
      const int j = gd_outer_col();
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = gd_outer_row(u);
        const double v = (i < r && j < r) ? o[u] : (i == j ? 1.0 : 0.0);
        Gs[2 * 32 * kGdLg + i * kGdLg + j] = v;
        Gq[i * 32 + j] = v;
        if (i == j && i < r) tr_new += v;
      }
    }
    const double dq = gd_block_sum(tr_old - 2.0 * part_q + tr_new, red);
    if (tid == 0) a.delta[((int64_t)it * 2 + 0) * bh + h] = dq;
  }
  // Cq' = T (rows beyond r stay zero: Mq'^T has zero rows there)
  if (tid < d) {
#pragma unroll
    for (int i = 0; i < 32; ++i) Cq[i * d + tid] = TT[tid * kGdLd + i];
  }
  // ---- Mk'^T = (Gq' + B_K B_K^T)^-1 (T + B_K) beside the next B_Q = Gq'^-1 T
  {
    const double* Gn = Gs + 2 * 32 * kGdLg;
    const double* Gb = Gs + 32 * kGdLg;
    gd_fill(sy[0], [&](int i, int j) { return Gn[i * kGdLg + j]; }, [&](int i, int cc) { return TT[cc * kGdLd + i]; });
    gd_fill(sy[1], [&](int i, int j) { return Gn[i * kGdLg + j] + Gb[i * kGdLg + j]; },
            [&](int i, int cc) { return TT[cc * kGdLd + i]; });
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int u = 0; u < 2; ++u) sy[1].x[rt][u] += bk[rt][u];
  }
  __syncthreads();
  gd_solve_pair(sy, piv);
  gd_drain(sy[0].x, [&](int i, int cc, double v) { BqT[i * d + cc] = v; });
  double part_k = 0.0;
  {
    float* mt = a.Mt_k + (int64_t)h * r * d;
    gd_drain(sy[1].x, [&](int i, int cc, double v) {
      MT[cc * kGdLd + i] = v;
      if (i < r) mt[i * d + cc] = (float)v;
    });
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int v = 0; v < 4; ++v) part_k = fma(ckt[rt][u][v], sy[1].x[rt][u][v], part_k);
  }
  double trk_old = 0.0;
  if (tid < 32) trk_old = tid < r ? Gk[tid * 32 + tid] : 0.0;
  __syncthreads();
  // ---- U = Mk'^T Sk, Gk' = Mk'^T U^T, Ck' = U
  gd_times_s(MT, Sk, TT);
  {
    double o[4];
    gd_outer(MT, TT, o);
    double tr_new = 0.0;
    if (tid < 256) {
      const int j = gd_outer_col();
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = gd_outer_row(u);
        const double v = (i < r && j < r) ? o[u] : (i == j ? 1.0 : 0.0);
        Gk[i * 32 + j] = v;
        if (i == j && i < r) tr_new += v;
      }
    }
    const double dk = gd_block_sum(trk_old - 2.0 * part_k + tr_new, red);
    if (tid == 0) a.delta[((int64_t)it * 2 + 1) * bh + h] = dk;
  }
  if (tid < d) {
#pragma unroll
    for (int i = 0; i < 32; ++i) Ck[i * d + tid] = TT[tid * kGdLd + i];
  }
}

// Workspace (bytes) of the Gram-domain iteration for bh heads over bkv distinct K heads.
static size_t gramdom_bytes(int bh, int bkv, int Sx, int Sxk, int iters, size_t own_part_floats) {
  const size_t dd = (size_t)kGdD * kGdD;
  return ((size_t)bh * Sx + (size_t)bkv * Sxk) * dd * sizeof(float)      // X^T X partial sums
         + own_part_floats * sizeof(float)                                // (G, C) partial sums of the fused kernel
         + ((size_t)bh + bkv) * dd * sizeof(double)                       // Sq, Sk
         + (size_t)2 * bh * (1024 + 32 * kGdD) * sizeof(double)           // G, C
         + (size_t)bh * 32 * kGdD * sizeof(double)                        // B_Q handed from iteration to iteration
         + (size_t)std::max(iters, 1) * 2 * bh * sizeof(double)           // squared changes
         + (size_t)2 * bh * 32 * kGdD * sizeof(float) + 256;              // Mq^T, Mk^T
}

// Runs all iterations on the Gram matrices.  On return Mt_q / Mt_k (device pointers written to *mt_q, *mt_k)
// hold Mq^T, Mk^T of the last iteration that ran, and b_q, b_k the final B factors; the caller applies
// A_Q = Q Mq, A_K = K Mk.  The initial [G | C] sums: partK (and partQ) with S splits from the row-by-row pass; with
// a_q0 (the given A_Q, [bh][l][r]) the Q side's are formed here together with Q^T Q and partQ is not read.
int prefill_gram_domain(lrqk_ctx* ctx, const void* q, const void* k, const float* partQ, const float* partK, int S,
                        const float* a_q0, float* b_q, float* b_k, int b, int hq, int hkv, int64_t l, int r, int iters,
                        float tol, int* flags, float** mt_q, float** mt_k, hipStream_t st) {
  const int bh = b * hq, bkv = b * hkv;
  const int d = kGdD;
  const bool fused = a_q0 != nullptr;
  LRQK_REQUIRE(partK && (fused || partQ), LRQK_EINVAL, "neither partial sums nor initial factors");
  // splits of the long axis for the X^T X sums: about two workgroups per CU for Q, one for K (with 64 splits of 8
  // heads the partial sums are 33 MB to write and to add up: 25.6 + 18.5 us against 19.7 + 11.1 with 32).  The
  // fused kernel: one workgroup per CU (registers), at most 4096 rows per split (its fp32 sums), at least one step each.
  int Sx = (int)std::max<int64_t>(1, std::min<int64_t>(std::max(1, 512 / bh), (l + 511) / 512));
  const int Sxk = (int)std::max<int64_t>(1, std::min<int64_t>(std::max(1, 256 / bkv), (l + 511) / 512));
  int Spq = S;
  if (fused) {
    int64_t v = std::max<int64_t>(std::max(1, 256 / bh), (l + 4095) / 4096);
    v = std::min<int64_t>(v, 64);
    Sx = Spq = (int)std::max<int64_t>(1, std::min<int64_t>(v, (l + kXtxRows - 1) / kXtxRows));
  }
  const size_t ne = (size_t)r * (r + d);
  const size_t own_part = fused ? (size_t)bh * Spq * ne : 0;
  int rc = ctx->prefill_gd.ensure(gramdom_bytes(bh, bkv, Sx, Sxk, iters, own_part));
  if (rc) return rc;
  const size_t dd = (size_t)d * d;
  char* p = (char*)ctx->prefill_gd.p;
  double* Sq = (double*)p;                  p += (size_t)bh * dd * sizeof(double);
  double* Sk = (double*)p;                  p += (size_t)bkv * dd * sizeof(double);
  double* G = (double*)p;                   p += (size_t)2 * bh * 1024 * sizeof(double);
  double* C = (double*)p;                   p += (size_t)2 * bh * 32 * d * sizeof(double);
  double* BqT = (double*)p;                 p += (size_t)bh * 32 * d * sizeof(double);
  double* delta = (double*)p;               p += (size_t)std::max(iters, 1) * 2 * bh * sizeof(double);
  float* Mtq = (float*)p;                   p += (size_t)bh * 32 * d * sizeof(float);
  float* Mtk = (float*)p;                   p += (size_t)bh * 32 * d * sizeof(float);
  float* xq_part = (float*)p;               p += (size_t)bh * Sx * dd * sizeof(float);
  float* xk_part = (float*)p;               p += (size_t)bkv * Sxk * dd * sizeof(float);
  if (fused) {
    float* pq = (float*)p;
    LRQK_REQUIRE((uintptr_t)q % 16 == 0, LRQK_EINVAL, "rows must be 16-byte aligned");
    hipLaunchKernelGGL(pf_sums_kernel, dim3((unsigned)Spq, (unsigned)bh), dim3(kXtxThreads), 0, st, (const bf16_t*)q, l,
                       a_q0, r, pq, xq_part, Spq);
    partQ = pq;
  } else {
    hipLaunchKernelGGL(pf_xtx_kernel, dim3((unsigned)Sx, (unsigned)bh), dim3(kXtxThreads), 0, st, (const bf16_t*)q, l,
                       xq_part, Sx);
  }
  hipLaunchKernelGGL(pf_xtx_kernel, dim3((unsigned)Sxk, (unsigned)bkv), dim3(kXtxThreads), 0, st, (const bf16_t*)k, l,
                     xk_part, Sxk);
  LRQK_HIP_CHECK(hipGetLastError());
  const size_t smem = ((size_t)3 * kGdD * kGdLd + 3 * 32 * kGdLg + kGdPivDoubles + 8) * sizeof(double);
  static std::atomic<bool> attr_dev[kMaxDeviceSlots];
  std::atomic<bool>& attr = attr_dev[per_device_slot()];
  if (!attr) {
    LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)pf_gramdom_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem));
    attr = true;
  }
  GdArgs a{partQ, partK, Spq, S, Sq, Sk, G, C, BqT, delta, flags, Mtq, Mtk, b_q, b_k, bh, hq, hkv, r, l, tol};
  const unsigned init_blocks = (unsigned)(((size_t)bh + bkv) * (dd / 256) + (size_t)2 * bh * kGdInitBlocks);
  hipLaunchKernelGGL(pf_gramdom_init_kernel, dim3(init_blocks), dim3(256), 0, st, a, (const float*)xq_part, Sx,
                     (const float*)xk_part, Sxk, bkv, Sq, Sk);
  for (int it = 0; it < iters; ++it)
    hipLaunchKernelGGL(pf_gramdom_kernel, dim3((unsigned)bh), dim3(kGdThreads), smem, st, 0, it, a);
  hipLaunchKernelGGL(pf_gramdom_kernel, dim3((unsigned)bh), dim3(kGdThreads), smem, st, 2, iters, a);
  LRQK_HIP_CHECK(hipGetLastError());
  *mt_q = Mtq;
  *mt_k = Mtk;
  return LRQK_OK;
}

}  // namespace lrqk
