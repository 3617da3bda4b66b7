// Per-step factor update for ranks 33..64 on the matrix cores (bf16 storage, d = 128, r % 8 == 0): the
// reference's "accuracy-focused" setting is r = 64 (README.md:124-131 of the reference); the update itself is
// _lrqk_decode_inv_w1 (lrqk_attention.py:555-609).
//
//   gram  : grid (S, heads).  A^T A (64 x 64: three 32 x 32 tiles, the fourth is a transpose), A^T w and w = K q over
//           the active rows, as in the pass for r <= 32: 16-byte loads, a wave-private LDS tile that turns the rows into
//           the operand layout of the bf16 matrix cores (bf16 x bf16 products are exact in fp32), the next chunk's rows
//           in flight while a chunk is multiplied.  Per-workgroup partial sums go to HBM.
//   solve : one workgroup of 512 threads per head.  Adds the partial sums; B_Q B_Q^T, B_K B_K^T, q B_Q^T and k B_K^T on
//           the bf16 matrix cores straight from the stored rows (a lane's operand is 16 contiguous bytes of a row); each
//           64 x 64 matrix is then inverted by ONE wave as 32 symmetric sweeps on pairs of pivots, on 2 x 2 accumulator
//           tiles of the fp32 matrix cores (four rank-2 updates per pair, no barrier), G_Q and G_K side by side on two
//           waves; one wave runs the alternating rank-1 (Sherman-Morrison) iterations with a vector per lane.
// Same outputs as the kernels for r <= 32 (iter_out, deltas), so the finish stage and the scan take over unchanged.
#include <algorithm>
#include <atomic>

#include "common.hpp"
#include "ctx.hpp"
#include "als_gram.hpp"
#include "small_inverse.hpp"

namespace lrqk {

typedef __bf16 r64_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 r64_bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kG64Threads = 256;
constexpr int kG64Waves = kG64Threads / kWave;
constexpr int kG64Chunk = 32;           // tokens per wave and chunk
constexpr int kG64Ld = 72;              // 16-bit elements per staged row of A: 144 bytes, see the operand gather below
constexpr int kG64Ne = 64 * 64 + 64;    // floats of a partial result: A^T A (row stride 64), then A^T w
constexpr int kG64Red = 3 * 1024 + 64;  // floats a wave contributes to the cross-wave sum: tiles (0,0), (0,1), (1,1), A^T w
static_assert(kG64Waves * (kG64Chunk * kG64Ld / 2 + kG64Chunk) <= kG64Waves * kG64Red, "the tiles fit the shared block");

__device__ __forceinline__ void r64_wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__global__ __launch_bounds__(kG64Threads, 2) void als_gram64_bf16_kernel(
    const bf16_t* __restrict__ a_k, int64_t head_stride, int64_t a_rows, const int32_t* __restrict__ active_idx,
    int64_t idx_stride, bf16_t* k_prev, int kprev_slots, int n, const bf16_t* __restrict__ q, int r,
    float* __restrict__ part, int S, GramAppend ap, float* __restrict__ kq_out) {
  constexpr int d = 128, VEC = 8, lpr_log2 = 4, lpr = 16, gpw = kWave / lpr;  // 16 lanes per K row, 4 rows per load
  constexpr int KL = kG64Chunk / gpw;                                          // K loads per lane and chunk
  constexpr int AL = kG64Chunk * 8 / kWave;                                    // A loads per lane and chunk (8 pieces per row)
  __shared__ __align__(16) float gsm[kG64Waves * kG64Red];
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int h = blockIdx.y, s = blockIdx.x;
  // wave-private: the chunk's A rows as bf16 [32][kG64Ld], and its 32 products K q
  uint16_t* At = reinterpret_cast<uint16_t*>(gsm) + wave * (kG64Chunk * kG64Ld);
  float* w_s = gsm + kG64Waves * (kG64Chunk * kG64Ld / 2) + wave * kG64Chunk;

  const int sub = lane & (lpr - 1), grp = lane >> lpr_log2;
  const int arow = lane >> 3, aq = lane & 7;  // A loads: tokens arow + 8 j of the chunk, piece aq of the row
  const int lpa = r >> 3;
  const int aqc = min(aq, lpa - 1);
  const int rows_per_split = (n + S - 1) / S;
  const int s0 = s * rows_per_split;
  const int s1 = min(n, s0 + rows_per_split);
  const int rows_per_wave = (rows_per_split + kG64Waves - 1) / kG64Waves;
  const int w0 = s0 + wave * rows_per_wave;
  const int w1 = min(s1, w0 + rows_per_wave);
  const int n_chunks = (rows_per_wave + kG64Chunk - 1) / kG64Chunk;
  const bf16_t* A = a_k + (int64_t)h * head_stride;
  const bf16_t* Kp = k_prev + (int64_t)h * kprev_slots * d;
  const int col = lane & 31, khalf = lane >> 5;
  const bf16_t* knew_h = Kp;
  if (ap.slot >= 0) {
    const int bb = h / ap.hq, kvh = (h % ap.hq) / (ap.hq / ap.hkv);
    knew_h = (const bf16_t*)ap.k_new + ((int64_t)bb * ap.hkv + kvh) * d;
  }
  uint32_t qw[4];  // this lane's eight elements of q, as stored
  {
    const uint4 qv = *reinterpret_cast<const uint4*>(q + (int64_t)h * d + sub * VEC);
    qw[0] = qv.x;
    qw[1] = qv.y;
    qw[2] = qv.z;
    qw[3] = qv.w;
  }
  // every load is unconditional: indices are clamped into range and the results masked afterwards
  auto load_ids = [&](int c0, int32_t (&tok)[AL]) {
#pragma unroll
    for (int j = 0; j < AL; ++j) {
      const int t = min(c0 + arow + 8 * j, n - 1);
      const int32_t id = active_idx ? active_idx[(int64_t)h * idx_stride + t] : t;
      tok[j] = t == ap.slot ? ap.token : id;
    }
  };
  auto load_a = [&](const int32_t (&tok)[AL], uint4 (&av)[AL]) {
#pragma unroll
    for (int j = 0; j < AL; ++j) {
      const int64_t sr = min(max((int64_t)tok[j], (int64_t)0), a_rows - 1);
      av[j] = *reinterpret_cast<const uint4*>(A + sr * r + aqc * 8);
    }
  };
  auto load_k = [&](int c0, uint4 (&kv)[KL]) {
#pragma unroll
    for (int u = 0; u < KL; ++u) {
      const int row = min(c0 + u * gpw + grp, n - 1);
      kv[u] = *reinterpret_cast<const uint4*>((row == ap.slot ? knew_h : Kp + (int64_t)row * d) + sub * VEC);
    }
  };

  v16f acc00, acc01, acc11;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc00[v] = acc01[v] = acc11[v] = 0.0f;
  float racc0 = 0.0f, racc1 = 0.0f;
  int32_t tok_cur[AL], tok_nxt[AL];
  uint4 a_cur[AL];
  uint4 kv[KL];
  load_ids(w0, tok_cur);
  load_k(w0, kv);
  load_ids(w0 + kG64Chunk, tok_nxt);
  load_a(tok_cur, a_cur);

  for (int ch = 0; ch < n_chunks; ++ch) {
    const int c0 = w0 + ch * kG64Chunk;
    // K q of the chunk's rows: products of bf16 pairs summed in fp32 (q stays in its storage form)
#pragma unroll
    for (int u = 0; u < KL; ++u) {
      const int row = u * gpw + grp;
      const uint32_t kw[4] = {kv[u].x, kv[u].y, kv[u].z, kv[u].w};
      float wv = 0.0f;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        wv = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(r64_bf16x2, kw[e]), __builtin_bit_cast(r64_bf16x2, qw[e]),
                                             wv, false);
      wv = group_sum(wv, lpr);
      if (sub == 0) w_s[row] = (c0 + row < w1) ? wv : 0.0f;
    }
    // the next chunk's rows and the ids of the one after it (wave-uniform conditions)
    uint4 a_nxt[AL];
    int32_t tok_nn[AL];
#pragma unroll
    for (int j = 0; j < AL; ++j) {
      a_nxt[j] = a_cur[j];
      tok_nn[j] = 0;
    }
    if (ch + 1 < n_chunks) {
      load_k(c0 + kG64Chunk, kv);
      load_a(tok_nxt, a_nxt);
    }
    if (ch + 2 < n_chunks) load_ids(c0 + 2 * kG64Chunk, tok_nn);
    // this chunk's A rows into the tile (rows that do not count, and columns >= r, as zeros)
#pragma unroll
    for (int j = 0; j < AL; ++j) {
      const bool ok = (c0 + arow + 8 * j < w1) && tok_cur[j] >= 0 && (int64_t)tok_cur[j] < a_rows && aq < lpa;
      const uint4 v = ok ? a_cur[j] : make_uint4(0, 0, 0, 0);
      *reinterpret_cast<uint4*>(At + (arow + 8 * j) * kG64Ld + aq * 8) = v;
    }
    r64_wave_sync();
    if (kq_out && lane < kG64Chunk && c0 + lane < w1) kq_out[(int64_t)h * n + c0 + lane] = w_s[lane];
    // Lane (col, khalf) takes eight tokens of a group of 16 as the k elements of one bf16 MFMA: tokens
    // 0..3 and 8..11 (+ 4 khalf).  Both operands of every product use the same assignment, so the order is
    // immaterial; this one puts the two halves of the wave 4 rows = 576 bytes = 16 LDS banks apart.
#pragma unroll
    for (int mm = 0; mm < kG64Chunk / 16; ++mm) {
      uint32_t e0[8], e1[8];
      float wv[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int t = 16 * mm + (j & 3) + 8 * (j >> 2) + 4 * khalf;
        e0[j] = At[t * kG64Ld + col];
        e1[j] = At[t * kG64Ld + 32 + col];
        wv[j] = w_s[t];
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        racc0 = fmaf(wv[j], __uint_as_float(e0[j] << 16), racc0);
        racc1 = fmaf(wv[j], __uint_as_float(e1[j] << 16), racc1);
      }
      const r64_bf16x8 op0 = __builtin_bit_cast(
          r64_bf16x8, make_uint4(e0[0] | (e0[1] << 16), e0[2] | (e0[3] << 16), e0[4] | (e0[5] << 16), e0[6] | (e0[7] << 16)));
      const r64_bf16x8 op1 = __builtin_bit_cast(
          r64_bf16x8, make_uint4(e1[0] | (e1[1] << 16), e1[2] | (e1[3] << 16), e1[4] | (e1[5] << 16), e1[6] | (e1[7] << 16)));
      acc00 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(op0, op0, acc00, 0, 0, 0);
      acc01 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(op0, op1, acc01, 0, 0, 0);
      acc11 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(op1, op1, acc11, 0, 0, 0);
    }
    r64_wave_sync();  // the tile and w_s are rewritten by the next chunk
#pragma unroll
    for (int j = 0; j < AL; ++j) {
      a_cur[j] = a_nxt[j];
      tok_cur[j] = tok_nxt[j];
      tok_nxt[j] = tok_nn[j];
    }
  }
  racc0 += __shfl_xor(racc0, 32, kWave);
  racc1 += __shfl_xor(racc1, 32, kWave);
  if (ap.slot >= w0 && ap.slot < w1 && lane < lpr) {  // this wave owns the new token's slot
    const int bb = h / ap.hq, kvh = (h % ap.hq) / (ap.hq / ap.hkv);
    const int64_t so = ((int64_t)bb * ap.hkv + kvh) * d + lane * VEC;
    const int64_t dof = ((int64_t)h * kprev_slots + ap.slot) * d + lane * VEC;
    const uint4 kx = *reinterpret_cast<const uint4*>((const bf16_t*)ap.k_new + so);
    const uint4 vx = *reinterpret_cast<const uint4*>((const bf16_t*)ap.v_new + so);
    *reinterpret_cast<uint4*>(k_prev + dof) = kx;
    *reinterpret_cast<uint4*>((bf16_t*)ap.v_act + dof) = vx;
    if (lane == 0) ap.idx_out[(int64_t)h * idx_stride + ap.slot] = ap.token;
  }
  // ---- cross-wave reduction through the same block of LDS
  __syncthreads();
  float* red = gsm + wave * kG64Red;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int e = mfma_row(lane, v) * 32 + col;
    red[e] = acc00[v];
    red[1024 + e] = acc01[v];
    red[2048 + e] = acc11[v];
  }
  if (lane < 32) {
    red[3072 + col] = racc0;
    red[3072 + 32 + col] = racc1;
  }
  __syncthreads();
  float* pout = part + ((int64_t)h * S + s) * kG64Ne;
  for (int e = tid; e < kG64Ne; e += kG64Threads) {
    int src;
    if (e < 64 * 64) {
      const int i = e >> 6, j = e & 63;
      if (i < 32)
        src = j < 32 ? i * 32 + j : 1024 + i * 32 + (j - 32);
      else
        src = j < 32 ? 1024 + j * 32 + (i - 32) : 2048 + (i - 32) * 32 + (j - 32);
    } else {
      src = 3072 + (e - 64 * 64);
    }
    float v = 0.0f;
#pragma unroll
    for (int wv = 0; wv < kG64Waves; ++wv) v += gsm[wv * kG64Red + src];
    pout[e] = v;
  }
}

// ----------------------------------------------------------------------------- solve
constexpr int kS64Threads = 512;
constexpr int kS64Ld = 65;  // row stride of a 64 x 64 matrix in LDS

// In-place inverse of one SPD matrix of even order r <= 64 held in LDS ([64][kS64Ld]; only the leading r x r block
// is read), by one wave: the scheme of invert_sweep_mfma -- symmetric sweeps on the matrix scaled to unit diagonal,
// the sweeps on p and p + 1 as the two k elements of one rank-2 MFMA update, the 2 that every sweep leaves on its
// diagonal entry taken off at the end -- on the accumulators of 2 x 2 tiles: row p (and p + 1) of both column
// blocks makes the operands, A_i = B_i / d for the rows of either block.  Rows and columns >= r form an identity
// block.  sbuf: 64 floats.
__device__ __forceinline__ void invert64_sweep_mfma(float* G, int r, float* sbuf) {
  const int lane = lane_id();
  const int col = lane & 31, half = lane >> 5;
  v16f acc[2][2];
#pragma unroll
  for (int I = 0; I < 2; ++I)
#pragma unroll
    for (int J = 0; J < 2; ++J)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int i = 32 * I + mfma_row(lane, v), j = 32 * J + col;
        const float x = G[i * kS64Ld + j];
        acc[I][J][v] = (i < r && j < r) ? x : (i == j ? 1.0f : 0.0f);
      }
  const float s_lane = lane < r ? __builtin_amdgcn_rsqf(G[lane * kS64Ld + lane]) : 1.0f;
  sbuf[lane] = s_lane;
  r64_wave_sync();
  const float sc0 = sbuf[col], sc1 = sbuf[32 + col];
#pragma unroll
  for (int I = 0; I < 2; ++I)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const float4 s4 = reinterpret_cast<const float4*>(sbuf)[8 * I + 2 * a + half];  // rows 32 I + 8 a + 4 half + 0..3
      const float sr[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[I][0][4 * a + e] *= sr[e] * sc0;
        acc[I][1][4 * a + e] *= sr[e] * sc1;
      }
    }
  // (lane-dependent cases by weights of 0 and 1, not by selects between expressions, which compile to divergent
  // branches; the matrix is finite, so a product with a weight of 0 is 0)
  const float in0 = half == 0 ? 1.0f : 0.0f, in1 = 1.0f - in0;
#pragma unroll
  for (int p = 0; p < 64; p += 2) {
    if (p < r) {  // (wave-uniform)
      const int P = p >> 5, pl = p & 31;
      const int v = ((pl >> 3) << 2) + (pl & 3), hp = (pl >> 2) & 1;  // rows p, p + 1: elements v, v + 1 of half hp
      const float r0P = acc[P][P][v], r1P = acc[P][P][v + 1];
      const float r0X = acc[P][1 - P][v], r1X = acc[P][1 - P][v + 1];
      const float da = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(r0P), pl + 32 * hp));
      const float db = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(r0P), pl + 1 + 32 * hp));
      const float dc = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(r1P), pl + 1 + 32 * hp));
      float rc0 = __builtin_amdgcn_rcpf(da);
      rc0 = fmaf(fmaf(-da, rc0, 1.0f), rc0, rc0);
      const float brc = db * rc0;
      const float c1 = fmaf(-db, brc, dc);  // the second pivot as the first sweep leaves it
      float rc1 = __builtin_amdgcn_rcpf(c1);
      rc1 = fmaf(fmaf(-c1, rc1, 1.0f), rc1, rc1);
      const float rck = half ? rc1 : rc0;
      const float wp0 = col == pl ? 1.0f : 0.0f, wp1 = col == pl + 1 ? 1.0f : 0.0f;
      float Av[2], Bv[2];
      {  // the pivots' own block of columns
        const float U = half_pair(r0P, r1P, hp), V = half_pair(r1P, r0P, hp);  // [row p | row p + 1], [row p + 1 | row p]
        const float B1 = (half ? V : U) - wp0;     // the first sweep's B, in every lane
        const float B2 = fmaf(-brc, B1, U) - wp1;  // (upper half) the second sweep's B
        Bv[P] = half ? B2 : B1;
        Av[P] = Bv[P] * rck;
      }
      {  // the other block of columns
        const float U = half_pair(r0X, r1X, hp), V = half_pair(r1X, r0X, hp);
        const float B1 = half ? V : U;
        const float B2 = fmaf(-brc, B1, U);
        Bv[1 - P] = half ? B2 : B1;
        Av[1 - P] = Bv[1 - P] * rck;
      }
      // the tiles that hold the next pivots' rows first: the other two run while those rows are being read
      const int Pn = (p + 2) >> 5 < 2 ? (p + 2) >> 5 : P;
      acc[Pn][Pn] = __builtin_amdgcn_mfma_f32_32x32x2f32(-Av[Pn], Bv[Pn], acc[Pn][Pn], 0, 0, 0);
      acc[Pn][1 - Pn] = __builtin_amdgcn_mfma_f32_32x32x2f32(-Av[Pn], Bv[1 - Pn], acc[Pn][1 - Pn], 0, 0, 0);
      acc[1 - Pn][Pn] = __builtin_amdgcn_mfma_f32_32x32x2f32(-Av[1 - Pn], Bv[Pn], acc[1 - Pn][Pn], 0, 0, 0);
      acc[1 - Pn][1 - Pn] = __builtin_amdgcn_mfma_f32_32x32x2f32(-Av[1 - Pn], Bv[1 - Pn], acc[1 - Pn][1 - Pn], 0, 0, 0);
    }
  }
#pragma unroll
  for (int I = 0; I < 2; ++I)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const float4 s4 = reinterpret_cast<const float4*>(sbuf)[8 * I + 2 * a + half];
      const float sr[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = 32 * I + mfma_row(lane, 4 * a + e);
#pragma unroll
        for (int J = 0; J < 2; ++J) {
          const int j = 32 * J + col;
          const float fix = i == j ? 2.0f : 0.0f;  // (the 2 I left in every pivot block)
          const float x = -(acc[I][J][4 * a + e] - fix) * sr[e] * (J ? sc1 : sc0);
          G[i * kS64Ld + j] = (i < r && j < r) ? x : (i == j ? 1.0f : 0.0f);
        }
      }
    }
}

__global__ __launch_bounds__(kS64Threads) void als_solve64_bf16_kernel(
    const float* __restrict__ part, int S, const bf16_t* __restrict__ b_q, const bf16_t* __restrict__ b_k,
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_new, int hq, int hkv, int r, int max_iter,
    float* __restrict__ iter_out, float* __restrict__ deltas) {
  constexpr int d = 128;
  __shared__ __align__(16) float GQ[64 * kS64Ld];
  __shared__ __align__(16) float GK[64 * kS64Ld];
  __shared__ __align__(16) float aw_s[64], rhs_s[64], kb_s[64], sbuf[2][64];
  __shared__ float sqk_s;
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int h = blockIdx.x;
  const int b = h / hq, kvh = (h % hq) / (hq / hkv);
  const int col = lane & 31, khalf = lane >> 5;
  const bf16_t* BQ = b_q + (int64_t)h * r * d;
  const bf16_t* BK = b_k + (int64_t)h * r * d;
  const bf16_t* qh = q + (int64_t)h * d;
  const bf16_t* kh = k_new + ((int64_t)b * hkv + kvh) * d;

  // ---- operands of B B^T: wave -> (matrix, tile); a lane's operand for step kk is 16 contiguous bytes of its row
  const int mat = wave >> 2, TI = (wave >> 1) & 1, TJ = wave & 1;  // mat 0: B_K, 1: B_Q
  const bf16_t* Bm = mat ? BQ : BK;
  uint4 opi[8], opj[8];
  {
    const int ri = 32 * TI + col, rj = 32 * TJ + col;
    const bf16_t* pi = Bm + (int64_t)min(ri, r - 1) * d + 8 * khalf;
    const bf16_t* pj = Bm + (int64_t)min(rj, r - 1) * d + 8 * khalf;
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
      opi[kk] = *reinterpret_cast<const uint4*>(pi + 16 * kk);
      opj[kk] = *reinterpret_cast<const uint4*>(pj + 16 * kk);
    }
    if (ri >= r) {
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) opi[kk] = make_uint4(0, 0, 0, 0);
    }
    if (rj >= r) {
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) opj[kk] = make_uint4(0, 0, 0, 0);
    }
  }
  // ---- the partial sums of A^T A and A^T w: 1040 16-byte vectors per partial result, three per thread
  {
    constexpr int NV = kG64Ne / 4;
    const float4* pin = reinterpret_cast<const float4*>(part + (int64_t)h * S * kG64Ne);
    float4 ps[3];
    int f[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      ps[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      f[i] = tid + kS64Threads * i;
    }
#pragma unroll 1
    for (int s0 = 0; s0 < S; s0 += 8) {
      float4 t[8][3];
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int i = 0; i < 3; ++i) t[u][i] = pin[(int64_t)min(s0 + u, S - 1) * NV + min(f[i], NV - 1)];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float wgt = s0 + u < S ? 1.0f : 0.0f;  // (finite values: a weight of 0 drops the repeated load)
#pragma unroll
        for (int i = 0; i < 3; ++i) {
          ps[i].x = fmaf(wgt, t[u][i].x, ps[i].x);
          ps[i].y = fmaf(wgt, t[u][i].y, ps[i].y);
          ps[i].z = fmaf(wgt, t[u][i].z, ps[i].z);
          ps[i].w = fmaf(wgt, t[u][i].w, ps[i].w);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      const float v4[4] = {ps[i].x, ps[i].y, ps[i].z, ps[i].w};
      if (f[i] < 1024) {
        const int e = 4 * f[i], row = e >> 6, c = e & 63;
#pragma unroll
        for (int x = 0; x < 4; ++x) GQ[row * kS64Ld + c + x] = v4[x];
      } else if (f[i] < NV) {
#pragma unroll
        for (int x = 0; x < 4; ++x) aw_s[4 * (f[i] - 1024) + x] = v4[x];
      }
    }
  }
  // ---- the tile of B B^T
  v16f acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
#pragma unroll
  for (int kk = 0; kk < 8; ++kk)
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(r64_bf16x8, opi[kk]),
                                                  __builtin_bit_cast(r64_bf16x8, opj[kk]), acc, 0, 0, 0);
  if (mat == 0) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int i = 32 * TI + mfma_row(lane, v), j = 32 * TJ + col;
      GK[i * kS64Ld + j] = acc[v];
    }
  }
  // ---- q B_Q^T and k B_K^T: the waves of the first tile row multiply once more, with the vector as row 0 of the
  // left operand (all other rows zero) and the operands of B they already hold; row 0 of the result is the product
  if (TI == 0) {
    const bf16_t* vec = mat ? qh : kh;
    v16f vacc;
#pragma unroll
    for (int v = 0; v < 16; ++v) vacc[v] = 0.0f;
    uint4 vop[8];
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) vop[kk] = *reinterpret_cast<const uint4*>(vec + 16 * kk + 8 * khalf);
    if (col != 0) {
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) vop[kk] = make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int kk = 0; kk < 8; ++kk)
      vacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(r64_bf16x8, vop[kk]),
                                                     __builtin_bit_cast(r64_bf16x8, opj[kk]), vacc, 0, 0, 0);
    if (khalf == 0) (mat ? rhs_s : kb_s)[32 * TJ + col] = vacc[0];  // (rows >= r of B are zero operands)
  }
  // ---- q . k
  if (wave == kS64Threads / kWave - 1) {
    float v = 0.0f;
    if (lane < d / 8) {
      const uint4 a = *reinterpret_cast<const uint4*>(qh + 8 * lane), c = *reinterpret_cast<const uint4*>(kh + 8 * lane);
      const uint32_t a4[4] = {a.x, a.y, a.z, a.w}, b4[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
      for (int e = 0; e < 4; ++e)
        v = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(r64_bf16x2, a4[e]), __builtin_bit_cast(r64_bf16x2, b4[e]), v, false);
    }
    v = wave_sum(v);
    if (lane == 0) sqk_s = v;
  }
  __syncthreads();
  // ---- G_Q = B_Q B_Q^T + A^T A;  q B_Q^T + (q K^T) A
  if (mat == 1) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int i = 32 * TI + mfma_row(lane, v), j = 32 * TJ + col;
      GQ[i * kS64Ld + j] += acc[v];
    }
  }
  if (tid < 64) rhs_s[tid] += tid < r ? aw_s[tid] : 0.0f;
  __syncthreads();
  // ---- both inverses, side by side
  if (wave == 0) invert64_sweep_mfma(GQ, r, sbuf[0]);
  if (wave == 1) invert64_sweep_mfma(GK, r, sbuf[1]);
  __syncthreads();
  if (wave != 0) return;
  // ---- the alternating iterations, lane c <-> element c of every vector (zeros beyond r)
  // out[c] = sum_i in[i] G[i][c]
  auto vecmat = [&](float in_lane, const float* G) {
    float v = 0.0f;
#pragma unroll
    for (int i = 0; i < 64; ++i)
      v = fmaf(__int_as_float(__builtin_amdgcn_readlane(__float_as_int(in_lane), i)), G[i * kS64Ld + lane], v);
    return v;
  };
  const float sqk = sqk_s;
  const float hk0 = vecmat(kb_s[lane], GK);    // k_hat_0 = k B_K^T G_K^-1
  const float yq0 = vecmat(rhs_s[lane], GQ);   // rhs_q G_Q^-1
  float hk = hk0;
  // x = b (G + v^T v)^-1 with b = b0 + s v, from G^-1 (Sherman-Morrison): z = v G^-1, y = y0 + s z,
  // x = y - (y . v / (1 + z . v)) z
  auto rank1 = [&](float y0, float v, const float* G) {
    const float z = vecmat(v, G);
    const float y = fmaf(sqk, z, y0);
    const float yv = wave_sum(y * v);
    const float zv = wave_sum(z * v);
    const float alpha = yv / (1.0f + zv);
    return fmaf(-alpha, z, y);
  };
  for (int it = 0; it < max_iter; ++it) {
    const float hqv = rank1(yq0, hk, GQ);   // q_hat (G_Q + k_hat^T k_hat) = rhs_q + s k_hat
    const float hkn = rank1(hk0, hqv, GK);  // k_hat' (G_K + q_hat^T q_hat) = k B_K^T + s q_hat
    float df = hk - hkn;
    df = wave_sum(df * df);
    if (lane == 0) deltas[(int64_t)h * max_iter + it] = df;
    float* o = iter_out + ((int64_t)h * max_iter + it) * 2 * r;
    if (lane < r) {
      o[lane] = hqv;
      o[r + lane] = hkn;
    }
    hk = hkn;
  }
}

bool als_r64_supported(int dtype, int r, int d, const void* a_k, int64_t head_stride) {
  return dtype == LRQK_BF16 && d == 128 && r > 32 && r <= 64 && r % 8 == 0 && ((uintptr_t)a_k % 16 == 0) &&
         (head_stride * 2) % 16 == 0;
}

int als_r64_update(lrqk_ctx* ctx, const void* b_q, const void* b_k, const void* a_k, int64_t head_stride,
                   const int32_t* active_idx, int64_t idx_stride, void* k_prev, int kprev_slots, int n, const void* q,
                   const void* k_new, int bh, int hq, int hkv, int r, int max_iter, float* iter_out, float* deltas,
                   const GramAppend& ap, float* kq_out, hipStream_t st) {
  // two chunks per wave where the launch still fits the GPU at one time (two workgroups per CU)
  static std::atomic<int> slots_dev[kMaxDeviceSlots];
  std::atomic<int>& slots_a = slots_dev[per_device_slot()];
  int slots = slots_a;
  if (slots == 0) {
    int per_cu = 0, dev = 0, n_cu = 0;
    LRQK_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, als_gram64_bf16_kernel, kG64Threads, 0));
    LRQK_HIP_CHECK(hipGetDevice(&dev));
    LRQK_HIP_CHECK(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev));
    slots = std::max(1, per_cu * n_cu);
    slots_a = slots;
  }
  int S = (n + 2 * kG64Waves * kG64Chunk - 1) / (2 * kG64Waves * kG64Chunk);
  S = std::max(1, std::min(std::min(S, 32), std::max(1, slots / bh)));
  int rc = ctx->als_part.ensure((size_t)bh * S * kG64Ne * sizeof(float));
  if (rc) return rc;
  hipLaunchKernelGGL(als_gram64_bf16_kernel, dim3((unsigned)S, (unsigned)bh), dim3(kG64Threads), 0, st,
                     (const bf16_t*)a_k, head_stride, head_stride / r, active_idx, idx_stride, (bf16_t*)k_prev, kprev_slots,
                     n, (const bf16_t*)q, r, (float*)ctx->als_part.p, S, ap, kq_out);
  LRQK_HIP_CHECK(hipGetLastError());
  hipLaunchKernelGGL(als_solve64_bf16_kernel, dim3((unsigned)bh), dim3(kS64Threads), 0, st,
                     (const float*)ctx->als_part.p, S, (const bf16_t*)b_q, (const bf16_t*)b_k, (const bf16_t*)q,
                     (const bf16_t*)k_new, hq, hkv, r, max_iter, iter_out, deltas);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

}  // namespace lrqk
