// Per-step factor update (the decode half of the alternating least squares), r <= 32.
//
//   gram   : grid (S, heads).  Each wave streams its share of the active rows once: w = K_prev q
//            on the vector ALUs and A^T A / A^T w on the matrix cores (fp32 MFMA 32x32x2; both
//            operands of A^T A are the same registers), A = the gathered active A_K rows.
//            Per-workgroup partial sums go to HBM.
//   solve  : one workgroup per head: adds the S partials in a fixed order, forms
//            G_K = B_K B_K^T and G_Q = B_Q B_Q^T + A^T A (MFMA again), inverts both once and runs
//            every alternating iteration as a rank-one (Sherman-Morrison) update of them,
//            recording each iterate and its squared change.
//   finish : per head: pick the iterate at which the batch-wide stopping test fired, take the
//            exact line-search step on B_Q, B_K, round and store.
//
// One CU retires 64 fp32 lane-operations per clock and a global load costs about a
// microsecond, so the per-head kernels avoid integer division, keep every batch of loads
// independent, and never walk a chain of dependent loads.  (A single launch in which the
// last-arriving workgroup continues was measured slower: the device-scope fence it needs
// costs ~15 us per workgroup because each XCD has its own L2.)
#include <algorithm>
#include <stdlib.h>

#include "common.hpp"
#include "ctx.hpp"
#include "als_finish.hpp"
#include "als_gram.hpp"
#include "small_inverse.hpp"

namespace lrqk {

constexpr int kGramThreads = 256;
constexpr int kGramWaves = kGramThreads / kWave;
constexpr int kGramChunk = 32;  // tokens per wave per chunk = 16 MFMA steps
constexpr int kGramNe = 32 * 32 + 32;
constexpr int kSolveThreads = 256;


// Everything the solve needs from B_Q, B_K, q and the new k -- B_Q B_Q^T and B_K B_K^T (four 32 x 32
// MFMA tiles: matrix x half of the d axis), q B_Q^T, k B_K^T and q . k -- does not depend on the Gram
// pass over the active rows, so two more workgroups per head of that launch form it beside them.
// out (kPreNe floats per head): tiles [4][1024] | q B_Q^T [32] | k B_K^T [32] | q . k.
constexpr int kPreNe = 4 * 1024 + 32 + 32 + 1;
template <typename T>
__device__ __forceinline__ void als_bgram_body(const T* __restrict__ b_q, const T* __restrict__ b_k,
                                               const T* __restrict__ q, const T* __restrict__ k_new, int h, int hq,
                                               int hkv, int r, int d, int vshift, float* __restrict__ out,
                                               float* __restrict__ sm, int which) {
  // Two workgroups per head, one per matrix (which = 0: B_Q with q, 1: B_K with k): waves 0 and 1 form the
  // two half-sums of B B^T, waves 2 and 3 the 32 products with the vector, wave 0 of the first also q . k.
  constexpr int VEC = Vec16<T>::N;
  constexpr int kMaxVec = 8;  // 16-byte vectors per thread: r * d / VEC <= 2048
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int b = h / hq, head = h % hq;
  const int kvh = head / (hq / hkv);
  const int ld = d + 1;
  float* B = sm;            // [32][d+1]  (rows >= r are zero)
  float* vec = B + 32 * ld;  // [d]
  float* oth = vec + d;      // [d] the other vector (for q . k)
  const T* bsrc = which ? b_k : b_q;
  const int vpr = 1 << vshift;
  const int nvec = r << vshift;
  Vec16<T> vb[kMaxVec];
#pragma unroll
  for (int u = 0; u < kMaxVec; ++u) {
    const int vi = min(tid + u * kGramThreads, nvec - 1);
    vb[u].load(bsrc + (int64_t)h * r * d + (int64_t)vi * VEC);
  }
  {
    const int c = min(tid, d - 1);
    const float qx = ld_f32<T>(q, (int64_t)h * d + c);
    const float kx = ld_f32<T>(k_new, ((int64_t)b * hkv + kvh) * d + c);
    if (tid < d) {
      vec[tid] = which ? kx : qx;
      oth[tid] = which ? qx : kx;
    }
  }
  for (int e = tid; e < (32 - r) * ld; e += kGramThreads) B[r * ld + e] = 0.0f;
#pragma unroll
  for (int u = 0; u < kMaxVec; ++u) {
    const int vi = tid + u * kGramThreads;
    if (vi < nvec) {
      const int row = vi >> vshift, c0 = (vi & (vpr - 1)) * VEC;
      float f[VEC];
      vb[u].unpack(f);
#pragma unroll
      for (int e = 0; e < VEC; ++e) B[row * ld + c0 + e] = f[e];
    }
  }
  __syncthreads();
  if (wave < 2) {
    // B B^T on the matrix cores: wave -> half of the d axis
    const int col = lane & 31, khalf = lane >> 5;
    const int half = wave;
    const float* Bp = B + col * ld + khalf;
    v16f acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
    const int k1 = (half + 1) * (d / 2);
#pragma unroll 8
    for (int kk = half * (d / 2); kk < k1; kk += 2)  // d >= 8 is a power of two
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(Bp[kk], Bp[kk], acc, 0, 0, 0);
    float* mine = out + (which * 2 + half) * 1024;
#pragma unroll
    for (int v = 0; v < 16; ++v) mine[mfma_row(lane, v) * 32 + col] = acc[v];
    if (which == 0 && wave == 0) {
      float v = 0.0f;
      for (int c = lane; c < d; c += kWave) v = fmaf(vec[c], oth[c], v);
      v = wave_sum(v);
      if (lane == 0) out[4 * 1024 + 64] = v;
    }
  } else {
    // vec B^T : thread -> (row = (tid - 128) >> 2, quarter of d)
    const int i = (tid - 128) >> 2, qtr = tid & 3;
    const float* Br = B + i * ld;
    float v = 0.0f;
#pragma unroll 8
    for (int c = qtr; c < d; c += 4) v = fmaf(vec[c], Br[c], v);
    v = group_sum(v, 4);
    if (qtr == 0) out[4 * 1024 + which * 32 + i] = v;
  }
}

// Partial layout per (head, split): 32*32 floats of A^T A (row stride 32) then 32 floats of
// A^T w.  Rows/columns >= r are zero.
template <typename T>
__global__ __launch_bounds__(kGramThreads) void als_gram_kernel(const T* __restrict__ a_k, int64_t head_stride,
                                                                int64_t a_rows, const int32_t* __restrict__ active_idx,
                                                                int64_t idx_stride, T* k_prev,
                                                                int kprev_slots, int n, const T* __restrict__ q, int r,
                                                                int d, int lpr_log2, float* __restrict__ part, int S,
                                                                GramAppend ap, const T* __restrict__ b_q,
                                                                const T* __restrict__ b_k, const T* __restrict__ k_new,
                                                                int hq, int hkv, float* __restrict__ pre,
                                                                float* __restrict__ kq_out) {
  constexpr int VEC = Vec16<T>::N;
  extern __shared__ __align__(16) float gram_dyn[];  // used by the extra workgroup only
  __shared__ float w_all[kGramWaves][kGramChunk];
  __shared__ float red[kGramWaves][kGramNe];
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int h = blockIdx.y, s = blockIdx.x;
  if (s >= S) {  // two workgroups per head beside the S splits
    als_bgram_body<T>(b_q, b_k, q, k_new, h, hq, hkv, r, d, lpr_log2, pre + (int64_t)h * kPreNe, gram_dyn, s - S);
    return;
  }
  float* w_s = w_all[wave];

  const int lpr = 1 << lpr_log2;
  const int sub = lane & (lpr - 1), grp = lane >> lpr_log2, gpw = kWave >> lpr_log2;
  const int rows_per_split = (n + S - 1) / S;
  const int s0 = s * rows_per_split;
  const int s1 = min(n, s0 + rows_per_split);
  const int rows_per_wave = (rows_per_split + kGramWaves - 1) / kGramWaves;
  const int w0 = s0 + wave * rows_per_wave;
  const int w1 = min(s1, w0 + rows_per_wave);
  const int n_chunks = (rows_per_wave + kGramChunk - 1) / kGramChunk;  // uniform over waves
  const T* A = a_k + (int64_t)h * head_stride;
  const T* Kp = k_prev + (int64_t)h * kprev_slots * d;
  const int col = lane & 31, khalf = lane >> 5;
  const T* knew_h = Kp;
  if (ap.slot >= 0) {
    const int bb = h / ap.hq, kvh = (h % ap.hq) / (ap.hq / ap.hkv);
    knew_h = (const T*)ap.k_new + ((int64_t)bb * ap.hkv + kvh) * d;
  }

  float qf[VEC];
  {
    Vec16<T> qv;
    qv.load(q + (int64_t)h * d + sub * VEC);
    qv.unpack(qf);
  }
  v16f acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
  float racc = 0.0f;

  for (int ch = 0; ch < n_chunks; ++ch) {
    const int c0 = w0 + ch * kGramChunk;
    // Loads are unconditional (indices clamped into range, results masked afterwards): a
    // conditional load compiles to a branch with a full wait, which would serialise them.
    // token ids this lane needs: tokens c0 + 2g + khalf, g = 0..15
    int src[kGramChunk / 2];
#pragma unroll
    for (int g = 0; g < kGramChunk / 2; ++g) {
      const int t = min(c0 + 2 * g + khalf, n - 1);
      const int id = active_idx ? active_idx[(int64_t)h * idx_stride + t] : t;
      src[g] = t == ap.slot ? ap.token : id;
    }
    // K rows of the chunk -> w
    for (int base0 = 0; base0 < kGramChunk; base0 += 8 * gpw) {
      Vec16<T> kv[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int row = min(c0 + base0 + u * gpw + grp, n - 1);
        kv[u].load((row == ap.slot ? knew_h : Kp + (int64_t)row * d) + sub * VEC);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int row = base0 + u * gpw + grp;
        float kf[VEC];
        kv[u].unpack(kf);
        float wv = 0.0f;
#pragma unroll
        for (int e = 0; e < VEC; ++e) wv = fmaf(kf[e], qf[e], wv);
        wv = group_sum(wv, lpr);
        if (sub == 0 && row < kGramChunk) w_s[row] = (c0 + row < w1) ? wv : 0.0f;
      }
    }
    // A elements of the chunk: lane (col, khalf) holds A[token 2g + khalf][col]
    float a0[kGramChunk / 2];
    const int colc = min(col, r - 1);
#pragma unroll
    for (int g = 0; g < kGramChunk / 2; ++g) {
      const int64_t sr = min(max((int64_t)src[g], (int64_t)0), a_rows - 1);
      a0[g] = ld_f32<T>(A, sr * r + colc);
    }
#pragma unroll
    for (int g = 0; g < kGramChunk / 2; ++g) {
      const bool ok = (c0 + 2 * g + khalf < w1) && src[g] >= 0 && (int64_t)src[g] < a_rows && col < r;
      a0[g] = ok ? a0[g] : 0.0f;
    }
    __syncthreads();  // w_s of this chunk is complete (every wave runs the same number of chunks)
    // K q of the wave's rows for the attention that ends the step (it then reads only V)
    if (kq_out && lane < kGramChunk && c0 + lane < w1) kq_out[(int64_t)h * n + c0 + lane] = w_s[lane];
#pragma unroll
    for (int g = 0; g < kGramChunk / 2; ++g) {
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[g], a0[g], acc, 0, 0, 0);
      racc = fmaf(w_s[2 * g + khalf], a0[g], racc);
    }
    __syncthreads();  // before the next chunk overwrites w_s
  }
  racc += __shfl_xor(racc, 32, kWave);
  if (ap.slot >= w0 && ap.slot < w1 && lane < lpr) {  // this wave owns the new token's slot
    const int bb = h / ap.hq, kvh = (h % ap.hq) / (ap.hq / ap.hkv);
    const int64_t so = ((int64_t)bb * ap.hkv + kvh) * d + lane * VEC;
    const int64_t dof = ((int64_t)h * kprev_slots + ap.slot) * d + lane * VEC;
    Vec16<T> kx, vx;
    kx.load((const T*)ap.k_new + so);
    vx.load((const T*)ap.v_new + so);
    *reinterpret_cast<decltype(kx.raw)*>(k_prev + dof) = kx.raw;
    *reinterpret_cast<decltype(vx.raw)*>((T*)ap.v_act + dof) = vx.raw;
    if (lane == 0) ap.idx_out[(int64_t)h * idx_stride + ap.slot] = ap.token;
  }
  // ---- cross-wave reduction through LDS
#pragma unroll
  for (int v = 0; v < 16; ++v) red[wave][mfma_row(lane, v) * 32 + col] = acc[v];
  if (lane < 32) red[wave][32 * 32 + col] = racc;
  __syncthreads();
  float* pout = part + ((int64_t)h * S + s) * kGramNe;
  for (int e = tid; e < kGramNe; e += kGramThreads) {
    float v = 0.0f;
#pragma unroll
    for (int wv = 0; wv < kGramWaves; ++wv) v += red[wv][e];
    pout[e] = v;
  }
}

// The same pass for bf16 storage with d = 128 and r a multiple of 8, built for throughput when many heads are
// stepped together: the active A_K rows come in as 16-byte pieces (two loads per lane and chunk instead of
// sixteen 2-byte ones) and reach the operand layout of the bf16 matrix cores through a wave-private LDS tile
// (bf16 x bf16 products are exact in fp32, so A^T A is the same sum as on the fp32 pipe, at a sixteenth of its
// cost); a wave walks its rows chunk by chunk with the next chunk's K and A rows and the ids of the chunk after
// it already requested, and no workgroup barrier inside the loop; all LDS is one static block shared by the
// roles, so the launch is bounded by registers (4 workgroups per CU), not by the extra workgroups' B tile.
typedef __bf16 gram_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 gram_bf16x2 __attribute__((ext_vector_type(2)));
constexpr int kGramSmemFloats = 32 * (128 + 1) + 2 * 128;  // the extra workgroups' need at d = 128 (>= 4 * kGramNe)
static_assert(kGramSmemFloats >= kGramWaves * kGramNe, "the cross-wave reduction fits the shared block");

__device__ __forceinline__ void gram_wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__global__ __launch_bounds__(kGramThreads, 4) void als_gram_bf16_kernel(
    const bf16_t* __restrict__ a_k, int64_t head_stride, int64_t a_rows, const int32_t* __restrict__ active_idx,
    int64_t idx_stride, bf16_t* k_prev, int kprev_slots, int n, const bf16_t* __restrict__ q, int r,
    float* __restrict__ part, int S, GramAppend ap, const bf16_t* __restrict__ b_q, const bf16_t* __restrict__ b_k,
    const bf16_t* __restrict__ k_new, int hq, int hkv, float* __restrict__ pre, float* __restrict__ kq_out) {
  constexpr int d = 128, VEC = 8, lpr_log2 = 4, lpr = 16, gpw = kWave / lpr;  // 16 lanes per K row, 4 rows per load
  constexpr int KL = kGramChunk / gpw;                                          // K loads per lane and chunk
  __shared__ __align__(16) float gsm[kGramSmemFloats];
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int h = blockIdx.y, s = blockIdx.x;
  if (s >= S) {
    als_bgram_body<bf16_t>(b_q, b_k, q, k_new, h, hq, hkv, r, d, lpr_log2, pre + (int64_t)h * kPreNe, gsm, s - S);
    return;
  }
  // wave-private: the chunk's A rows as bf16 [32][32] (64-byte rows), and its 32 products K q
  uint16_t* At = reinterpret_cast<uint16_t*>(gsm) + wave * (kGramChunk * 32);
  float* w_s = gsm + kGramWaves * (kGramChunk * 32 / 2) + wave * kGramChunk;

  const int sub = lane & (lpr - 1), grp = lane >> lpr_log2;
  const int arow = lane >> 2, aq = lane & 3;  // A loads: tokens arow and arow + 16 of the chunk, piece aq of the row
  const int lpa = r >> 3;
  const int aqc = min(aq, lpa - 1);
  const int rows_per_split = (n + S - 1) / S;
  const int s0 = s * rows_per_split;
  const int s1 = min(n, s0 + rows_per_split);
  const int rows_per_wave = (rows_per_split + kGramWaves - 1) / kGramWaves;
  const int w0 = s0 + wave * rows_per_wave;
  const int w1 = min(s1, w0 + rows_per_wave);
  const int n_chunks = (rows_per_wave + kGramChunk - 1) / kGramChunk;
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
    Vec16<bf16_t> qv;
    qv.load(q + (int64_t)h * d + sub * VEC);
    qw[0] = qv.raw.x;
    qw[1] = qv.raw.y;
    qw[2] = qv.raw.z;
    qw[3] = qv.raw.w;
  }
  // every load is unconditional: indices are clamped into range and the results masked afterwards
  auto load_ids = [&](int c0, int32_t (&tok)[2]) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int t = min(c0 + arow + 16 * j, n - 1);
      const int32_t id = active_idx ? active_idx[(int64_t)h * idx_stride + t] : t;
      tok[j] = t == ap.slot ? ap.token : id;
    }
  };
  auto load_a = [&](const int32_t (&tok)[2], uint4 (&av)[2]) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t sr = min(max((int64_t)tok[j], (int64_t)0), a_rows - 1);
      av[j] = *reinterpret_cast<const uint4*>(A + sr * r + aqc * 8);
    }
  };
  auto load_k = [&](int c0, Vec16<bf16_t> (&kv)[KL]) {
#pragma unroll
    for (int u = 0; u < KL; ++u) {
      const int row = min(c0 + u * gpw + grp, n - 1);
      kv[u].load((row == ap.slot ? knew_h : Kp + (int64_t)row * d) + sub * VEC);
    }
  };

  v16f acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
  float racc = 0.0f;
  int32_t tok_cur[2], tok_nxt[2];
  uint4 a_cur[2];
  Vec16<bf16_t> kv[KL];
  load_ids(w0, tok_cur);
  load_k(w0, kv);
  load_ids(w0 + kGramChunk, tok_nxt);
  load_a(tok_cur, a_cur);

  for (int ch = 0; ch < n_chunks; ++ch) {
    const int c0 = w0 + ch * kGramChunk;
    // K q of the chunk's rows: products of bf16 pairs summed in fp32 (q stays in its storage form)
#pragma unroll
    for (int u = 0; u < KL; ++u) {
      const int row = u * gpw + grp;
      const uint32_t kw[4] = {kv[u].raw.x, kv[u].raw.y, kv[u].raw.z, kv[u].raw.w};
      float wv = 0.0f;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        wv = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(gram_bf16x2, kw[e]), __builtin_bit_cast(gram_bf16x2, qw[e]),
                                             wv, false);
      wv = group_sum(wv, lpr);
      if (sub == 0) w_s[row] = (c0 + row < w1) ? wv : 0.0f;
    }
    // the next chunk's rows and the ids of the one after it (wave-uniform conditions)
    uint4 a_nxt[2] = {a_cur[0], a_cur[1]};
    int32_t tok_nn[2] = {0, 0};
    if (ch + 1 < n_chunks) {
      load_k(c0 + kGramChunk, kv);
      load_a(tok_nxt, a_nxt);
    }
    if (ch + 2 < n_chunks) load_ids(c0 + 2 * kGramChunk, tok_nn);
    // this chunk's A rows into the tile (rows that do not count, and columns >= r, as zeros)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const bool ok = (c0 + arow + 16 * j < w1) && tok_cur[j] >= 0 && (int64_t)tok_cur[j] < a_rows && aq < lpa;
      const uint4 v = ok ? a_cur[j] : make_uint4(0, 0, 0, 0);
      *reinterpret_cast<uint4*>(At + (arow + 16 * j) * 32 + aq * 8) = v;
    }
    gram_wave_sync();
    if (kq_out && lane < kGramChunk && c0 + lane < w1) kq_out[(int64_t)h * n + c0 + lane] = w_s[lane];
    // lane (col, khalf) takes tokens 16 mm + 8 khalf .. + 7 of its column: the k elements of one bf16 MFMA (both
    // operands are the same registers, so their order is immaterial)
#pragma unroll
    for (int mm = 0; mm < kGramChunk / 16; ++mm) {
      const int t0 = 16 * mm + 8 * khalf;
      uint32_t e[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) e[j] = At[(t0 + j) * 32 + col];
      const float4 wa = *reinterpret_cast<const float4*>(w_s + t0);
      const float4 wb = *reinterpret_cast<const float4*>(w_s + t0 + 4);
      const float wv[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
#pragma unroll
      for (int j = 0; j < 8; ++j) racc = fmaf(wv[j], __uint_as_float(e[j] << 16), racc);
      const gram_bf16x8 op = __builtin_bit_cast(
          gram_bf16x8, make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)));
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(op, op, acc, 0, 0, 0);
    }
    gram_wave_sync();  // the tile and w_s are rewritten by the next chunk
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      a_cur[j] = a_nxt[j];
      tok_cur[j] = tok_nxt[j];
      tok_nxt[j] = tok_nn[j];
    }
  }
  racc += __shfl_xor(racc, 32, kWave);
  if (ap.slot >= w0 && ap.slot < w1 && lane < lpr) {  // this wave owns the new token's slot
    const int bb = h / ap.hq, kvh = (h % ap.hq) / (ap.hq / ap.hkv);
    const int64_t so = ((int64_t)bb * ap.hkv + kvh) * d + lane * VEC;
    const int64_t dof = ((int64_t)h * kprev_slots + ap.slot) * d + lane * VEC;
    Vec16<bf16_t> kx, vx;
    kx.load((const bf16_t*)ap.k_new + so);
    vx.load((const bf16_t*)ap.v_new + so);
    *reinterpret_cast<decltype(kx.raw)*>(k_prev + dof) = kx.raw;
    *reinterpret_cast<decltype(vx.raw)*>((bf16_t*)ap.v_act + dof) = vx.raw;
    if (lane == 0) ap.idx_out[(int64_t)h * idx_stride + ap.slot] = ap.token;
  }
  // ---- cross-wave reduction through the same block of LDS
  __syncthreads();
  float* red = gsm;
#pragma unroll
  for (int v = 0; v < 16; ++v) red[wave * kGramNe + mfma_row(lane, v) * 32 + col] = acc[v];
  if (lane < 32) red[wave * kGramNe + 32 * 32 + col] = racc;
  __syncthreads();
  float* pout = part + ((int64_t)h * S + s) * kGramNe;
  for (int e = tid; e < kGramNe; e += kGramThreads) {
    float v = 0.0f;
#pragma unroll
    for (int wv = 0; wv < kGramWaves; ++wv) v += red[wv * kGramNe + e];
    pout[e] = v;
  }
}

// Everything in the solve kernel works on 32 x 32 tiles padded with an identity block (rows
// and columns >= r), so every loop has a compile-time trip count and its LDS reads pipeline.
// Sum of x over lanes 0..31 of the wave (the first two rows of 16 lanes); every lane must call it.
__device__ __forceinline__ float sum_lanes_0_31(float x) {
  x = row_reduce(x, [](float a, float b) { return a + b; });
  return lane_bcast(x, 0) + lane_bcast(x, 16);
}

// iter_out per head: [max_iter][2r] (q_hat then k_hat of each iteration);
// deltas: [bh][max_iter] sum over r of (k_hat - k_hat')^2.
// KS: compile-time bound of the number of Gram splits S (S <= KS): that many 16-byte loads per thread
// are in flight for the partial sums, so the bound follows S closely.
// (Two workgroups per CU as the launch bound where the partial sums leave room: with at most 256 registers per
// lane the matrix cores take their accumulators in ordinary registers, and a sweep reads its pivot row without
// copying the whole tile out of the accumulation registers.)
template <int KS>
__global__ __launch_bounds__(kSolveThreads, KS <= 16 ? 2 : 1) void als_solve_kernel(const float* __restrict__ pre,
                                                                  const float* __restrict__ part, int S, int r,
                                                                  int max_iter, float* __restrict__ iter_out,
                                                                  float* __restrict__ deltas) {
  static_assert(kGramNe % 4 == 0 && kGramNe / 4 - kSolveThreads <= kWave && kGramNe / 4 > kSolveThreads,
                "a partial is one 16-byte vector per thread plus a few more for the first wave");
  extern __shared__ __align__(16) float sm[];
  __shared__ float s_qk;
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int h = blockIdx.x;
  float* G = sm;                    // [kGramNe] summed A^T [A | w]
  float* Mx = G + kGramNe;          // [2][32] row scales of the two inversions (16-byte aligned)
  float* GKi = Mx + 2 * 32;         // [32][kLdi]
  float* GQi = GKi + 32 * kLdi;     // [32][kLdi]
  float* rhs_q = GQi + 32 * kLdi;   // 6 vectors of 32
  float* kB = rhs_q + 32;
  float* hat_k = kB + 32;
  float* hat_q = hat_k + 32;
  float* new_k = hat_q + 32;
  float* tmp = new_k + 32;
  float* cred = tmp + 32;           // [2 matrices][2 halves of d][32*32] MFMA tiles of B B^T (from the Gram launch)
  (void)hat_k; (void)hat_q; (void)new_k; (void)tmp;

  // ---- every global load of the kernel is issued here, back to back
  const float* pin = part + (int64_t)h * S * kGramNe;
  const float* pr = pre + (int64_t)h * kPreNe;
  {
    // a partial is kGramNe / 4 = 264 vectors: one per thread, the last 8 (the A^T w column) in the first wave
    constexpr int kVec = kGramNe / 4;
    const float4* pin4 = reinterpret_cast<const float4*>(pin);
    float4 x[KS], y[KS];
#pragma unroll
    for (int t = 0; t < KS; ++t) x[t] = pin4[(int64_t)min(t, S - 1) * kVec + tid];
    if (wave == 0) {
#pragma unroll
      for (int t = 0; t < KS; ++t) y[t] = pin4[(int64_t)min(t, S - 1) * kVec + min(kSolveThreads + tid, kVec - 1)];
    }
    float4 tl4[4];  // the four B B^T tiles: 4096 floats, 16 per thread
#pragma unroll
    for (int u = 0; u < 4; ++u) tl4[u] = reinterpret_cast<const float4*>(pr)[tid + u * kSolveThreads];
    const float pv = pr[4 * 1024 + min(tid, 64)];  // q B_Q^T [32] | k B_K^T [32] | q . k
#pragma unroll
    for (int u = 0; u < 4; ++u) reinterpret_cast<float4*>(cred)[tid + u * kSolveThreads] = tl4[u];
    auto sum_splits = [&](const float4 (&v)[KS]) {  // fixed order 0..S-1, element-wise
      float4 a = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
      for (int t = 0; t < KS; ++t) {
        a.x += (t < S) ? v[t].x : 0.0f;
        a.y += (t < S) ? v[t].y : 0.0f;
        a.z += (t < S) ? v[t].z : 0.0f;
        a.w += (t < S) ? v[t].w : 0.0f;
      }
      return a;
    };
    reinterpret_cast<float4*>(G)[tid] = sum_splits(x);
    if (wave == 0 && kSolveThreads + tid < kVec) reinterpret_cast<float4*>(G)[kSolveThreads + tid] = sum_splits(y);
    // rhs_q = q B_Q^T + (q K^T) A: the second term (G[1024 + i]) is added after the barrier; kB = k B_K^T
    if (tid < 32) rhs_q[tid] = pv;
    else if (tid < 64) kB[tid - 32] = pv;
    else if (tid == 64) s_qk = pv;
  }
  __syncthreads();
  if (tid < 32) rhs_q[tid] += G[32 * 32 + tid];  // (read again only after the barriers of the inversion)
  // G_K = B_K B_K^T (first wave) and G_Q = B_Q B_Q^T + A^T A (second wave), each inverted by its wave
  if (wave < 2) {
    const float* c0 = cred + (wave ? 0 : 2048);
    const float gsel = wave ? 1.0f : 0.0f;
    auto elem = [&](int i, int j) { return fmaf(gsel, G[i * 32 + j], c0[i * 32 + j] + c0[1024 + i * 32 + j]); };
    invert_sweep_mfma(elem, r, Mx + 32 * wave, wave ? GQi : GKi);
  }
  __syncthreads();
  // ---- k_hat_0 and the alternating rank-1 solves, all inside the first wave: lane c (and c + 32)
  // holds column c of both inverses and element c of every vector; a vector element is
  // broadcast with readlane, so the chain of small solves needs no barrier and no LDS round trip.
  if (wave == 0) {
    const int c = lane & 31;
    float cK[32], cQ[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      cK[i] = GKi[i * kLdi + c];
      cQ[i] = GQi[i * kLdi + c];
    }
    const float rq = rhs_q[c], kb = kB[c], sqk = s_qk;
    // y_c = sum_i b_i col[i]  (b lane-distributed)
    auto vecmat = [&](float bvec, const float (&col)[32]) {
      float y0 = 0.0f, y1 = 0.0f;
#pragma unroll
      for (int i = 0; i < 32; i += 2) {
        y0 = fmaf(__int_as_float(__builtin_amdgcn_readlane(__float_as_int(bvec), i)), col[i], y0);
        y1 = fmaf(__int_as_float(__builtin_amdgcn_readlane(__float_as_int(bvec), i + 1)), col[i + 1], y1);
      }
      return y0 + y1;
    };
    auto dot32 = [&](float a, float bb) { return sum_lanes_0_31(a * bb); };
    // x = b (G + v^T v)^-1 from G^-1 (Sherman-Morrison): x = y - (y.v / (1 + z.v)) z, y = b G^-1, z = v G^-1.
    // Both right-hand sides have the form b = b0 + s v, so y = b0 G^-1 + s z: b0 G^-1 is formed once
    // (for the k side it is k_hat_0 itself) and every solve costs one vector-matrix product.
    auto rank1 = [&](float y0, float v, const float (&col)[32]) {
      const float z = vecmat(v, col);
      const float y = fmaf(sqk, z, y0);
      const float alpha = dot32(y, v) / (1.0f + dot32(z, v));
      return fmaf(-alpha, z, y);
    };
    const float hk0 = vecmat(kb, cK);  // k_hat_0 = kB G_K^-1
    const float yq0 = vecmat(rq, cQ);  // rhs_q G_Q^-1
    float hk = hk0;
    for (int it = 0; it < max_iter; ++it) {
      const float hq = rank1(yq0, hk, cQ);  // q_hat (G_Q + k_hat^T k_hat) = rhs_q + s k_hat
      const float nk = rank1(hk0, hq, cK);  // k_hat' (G_K + q_hat^T q_hat) = kB + s q_hat
      const float df = c < r ? hk - nk : 0.0f;
      const float dsq = dot32(df, df);
      if (lane == 0) deltas[(int64_t)h * max_iter + it] = dsq;
      float* o = iter_out + ((int64_t)h * max_iter + it) * 2 * r;
      if (lane < r) {
        o[lane] = hq;
        o[r + lane] = nk;
      }
      hk = nk;
    }
  }
}

// ----------------------------------------------------------------------------- ranks beyond one matrix-core tile
// 32 < r <= 64 (the reference's "accuracy-focused" setting is r = 64, README.md:126) for the shapes that the
// matrix-core kernels of als_decode_r64.hip do not take (fp32 storage, rows other than 128 elements, ranks that are
// not multiples of 8): the same two launches in plain fp32 arithmetic, not tuned -- sums over the active rows, then one workgroup per head that forms G_K, G_Q, inverts
// them (Gauss-Jordan on the matrix scaled to unit diagonal, no pivoting: symmetric positive definite) and runs the
// alternating rank-1 solves with the formulas of als_solve_kernel.  Same outputs (iter_out, deltas), so the finish
// stage and the scan take over from there unchanged.
constexpr int kWideThreads = 256;
constexpr int kWideTile = 32;   // active rows per step
constexpr int kWideMaxR = 64;

// part per (head, split): r * r sums A^T A, then r sums A^T w.
// A tile of 32 active rows at a time: their A_K rows (as 16-byte pieces, zero-padded to 64 columns) and K rows go
// through LDS; thread (ti, tj) of a 16 x 16 grid keeps the 4 x 4 block (4 ti.., 4 tj..) of A^T A in registers.
// Every load is unconditional (clamped index, masked value).  r % 8 == 0 and 16-byte aligned rows for the vector
// loads of A_K (r = 40, 48, 56, 64 with bf16; multiples of 4 with fp32); other ranks take one element at a time.
template <typename T>
__global__ __launch_bounds__(kWideThreads) void als_gram_wide_kernel(
    const T* __restrict__ a_k, int64_t head_stride, int64_t a_rows, const int32_t* __restrict__ active_idx,
    int64_t idx_stride, T* k_prev, int kprev_slots, int n, const T* __restrict__ q, int r, int d,
    float* __restrict__ part, int S, GramAppend ap) {
  constexpr int VEC = Vec16<T>::N;
  constexpr int lda = kWideMaxR + 4;           // floats per staged row of A (16-byte aligned rows, 4 banks apart)
  extern __shared__ __align__(16) float wsm[];
  float* a_s = wsm;                            // [kWideTile][lda]
  float* w_s = a_s + kWideTile * lda;          // [kWideTile]
  float* q_s = w_s + kWideTile;                // [d]
  __shared__ int32_t tok_s[kWideTile];
  const int tid = threadIdx.x;
  const int h = blockIdx.y, s = blockIdx.x;
  const T* A = a_k + (int64_t)h * head_stride;
  const T* Kp = k_prev + (int64_t)h * kprev_slots * d;
  const T* knew_h = Kp;
  if (ap.slot >= 0) {
    const int bb = h / ap.hq, kvh = (h % ap.hq) / (ap.hq / ap.hkv);
    knew_h = (const T*)ap.k_new + ((int64_t)bb * ap.hkv + kvh) * d;
  }
  for (int c = tid; c < d; c += kWideThreads) q_s[c] = ld_f32<T>(q, (int64_t)h * d + c);
  const bool vec_a = r % VEC == 0 && ((uintptr_t)A % 16 == 0) && (head_stride * sizeof(T)) % 16 == 0;
  const int rows_per_split = (n + S - 1) / S;
  const int s0 = s * rows_per_split, s1 = min(n, s0 + rows_per_split);
  const int ti = tid >> 4, tj = tid & 15;
  float acc[4][4], racc = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;
  const int vpr = d / VEC;  // 16-byte pieces per K row (a power of two <= 64)
  for (int t0 = s0; t0 < s1; t0 += kWideTile) {
    const int rows = min(kWideTile, s1 - t0);
    if (tid < kWideTile) {
      const int t = min(t0 + tid, n - 1);
      const int32_t id = active_idx ? active_idx[(int64_t)h * idx_stride + t] : t;
      tok_s[tid] = t == ap.slot ? ap.token : id;
    }
    __syncthreads();
    // the rows of A_K of the tile's tokens (zero where the slot holds no token, and beyond column r)
    if (vec_a) {
      const int pieces = kWideMaxR / VEC;  // per staged row
      for (int e = tid; e < kWideTile * pieces; e += kWideThreads) {
        const int row = e / pieces, pc = e % pieces;
        const int32_t tok = tok_s[row];
        const bool ok = row < rows && tok >= 0 && (int64_t)tok < a_rows && pc * VEC < r;
        const int64_t sr = min(max((int64_t)tok, (int64_t)0), a_rows - 1);
        Vec16<T> v;
        v.load(A + sr * r + min(pc * VEC, r - VEC));
        float f[VEC];
        v.unpack(f);
#pragma unroll
        for (int x = 0; x < VEC; ++x) a_s[row * lda + pc * VEC + x] = ok ? f[x] : 0.0f;
      }
    } else {
      for (int e = tid; e < kWideTile * kWideMaxR; e += kWideThreads) {
        const int row = e / kWideMaxR, j = e % kWideMaxR;
        const int32_t tok = tok_s[row];
        const bool ok = row < rows && tok >= 0 && (int64_t)tok < a_rows && j < r;
        const int64_t sr = min(max((int64_t)tok, (int64_t)0), a_rows - 1);
        const float v = ld_f32<T>(A, sr * r + min(j, r - 1));
        a_s[row * lda + j] = ok ? v : 0.0f;
      }
    }
    // w = K q of the tile's rows: eight lanes per row, 16-byte pieces
    {
      const int row = tid >> 3, sub = tid & 7;
      const int t = min(t0 + row, n - 1);
      const T* kr = t == ap.slot ? knew_h : Kp + (int64_t)t * d;
      float wv = 0.0f;
      for (int pc = sub; pc < vpr; pc += 8) {
        Vec16<T> v;
        v.load(kr + pc * VEC);
        float f[VEC];
        v.unpack(f);
#pragma unroll
        for (int x = 0; x < VEC; ++x) wv = fmaf(f[x], q_s[pc * VEC + x], wv);
      }
      wv = group_sum(wv, 8);
      if (sub == 0) w_s[row] = row < rows ? wv : 0.0f;
    }
    __syncthreads();
#pragma unroll 4
    for (int row = 0; row < kWideTile; ++row) {  // (rows beyond the tile are zero)
      const float4 ai = *reinterpret_cast<const float4*>(a_s + row * lda + 4 * ti);
      const float4 aj = *reinterpret_cast<const float4*>(a_s + row * lda + 4 * tj);
      const float av[4] = {ai.x, ai.y, ai.z, ai.w}, bv[4] = {aj.x, aj.y, aj.z, aj.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
    }
    if (tid < kWideMaxR)
      for (int row = 0; row < kWideTile; ++row) racc = fmaf(w_s[row], a_s[row * lda + tid], racc);
    __syncthreads();
  }
  if (ap.slot >= s0 && ap.slot < s1) {  // this workgroup owns the new token's slot: the ring append
    const int bb = h / ap.hq, kvh = (h % ap.hq) / (ap.hq / ap.hkv);
    const T* ks = (const T*)ap.k_new + ((int64_t)bb * ap.hkv + kvh) * d;
    const T* vs = (const T*)ap.v_new + ((int64_t)bb * ap.hkv + kvh) * d;
    T* kd = k_prev + ((int64_t)h * kprev_slots + ap.slot) * d;
    T* vd = (T*)ap.v_act + ((int64_t)h * kprev_slots + ap.slot) * d;
    for (int c = tid; c < d; c += kWideThreads) {
      kd[c] = ks[c];
      vd[c] = vs[c];
    }
    if (tid == 0) ap.idx_out[(int64_t)h * idx_stride + ap.slot] = ap.token;
  }
  float* pout = part + ((int64_t)h * S + s) * (r * r + r);
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int a = 4 * ti + i, b2 = 4 * tj + j;
      if (a < r && b2 < r) pout[a * r + b2] = acc[i][j];
    }
  if (tid < r) pout[r * r + tid] = racc;
}

// One workgroup per head.  Thread (ti, tj) of a 16 x 16 grid keeps the 4 x 4 block (4 ti.., 4 tj..) of G_K and of
// G_Q in registers from the moment they are formed (B B^T from transposed copies of B_Q, B_K in LDS, plus the
// partial sums of A^T A) until their inverses are complete: Gauss-Jordan without pivoting on the matrices scaled
// to unit diagonal (symmetric positive definite), both at once, one barrier per pivot -- the owners of column p and
// row p publish them in LDS (two buffers in turn), every thread updates its blocks.  Rows and columns beyond r are
// an identity block.  Then the alternating rank-1 solves with the formulas of als_solve_kernel.
template <typename T>
__global__ __launch_bounds__(kWideThreads) void als_solve_wide_kernel(
    const float* __restrict__ part, int S, const T* __restrict__ b_q, const T* __restrict__ b_k,
    const T* __restrict__ q, const T* __restrict__ k_new, int hq, int hkv, int r, int d, int max_iter,
    float* __restrict__ iter_out, float* __restrict__ deltas) {
  extern __shared__ __align__(16) float wsm[];
  constexpr int R = kWideMaxR, ldt = R + 4, ldg = R + 1;
  float* BtQ = wsm;                // [d][ldt]  B_Q transposed (columns beyond r zero)
  float* BtK = BtQ + d * ldt;      // [d][ldt]
  float* GQ = BtK + d * ldt;       // [R][ldg]  inverses
  float* GK = GQ + R * ldg;        // [R][ldg]
  float* qv = GK + R * ldg;        // [d]
  float* kv = qv + d;              // [d]
  float* vec = kv + d;             // vectors of R
  float* rhs_q = vec, *kB = vec + R, *hk0 = vec + 2 * R, *yq0 = vec + 3 * R, *hk = vec + 4 * R, *hqv = vec + 5 * R;
  float* z = vec + 6 * R, *y = vec + 7 * R;
  float* pub = vec + 8 * R;        // [2 buffers][colQ, rowQ, colK, rowK][R]
  float* scq = pub + 8 * R, *sck = scq + R;
  __shared__ float s_red[4];
  const int tid = threadIdx.x;
  const int ti = tid >> 4, tj = tid & 15;
  const int h = blockIdx.x;
  const int b = h / hq, kvh = (h % hq) / (hq / hkv);
  const int ne = r * r + r;
  for (int e = tid; e < R * d; e += kWideThreads) {
    const int row = e / d, c = e % d;  // (d is a power of two)
    const bool ok = row < r;
    const int64_t src = (int64_t)h * r * d + (int64_t)min(row, r - 1) * d + c;
    const float vq = ld_f32<T>(b_q, src), vk = ld_f32<T>(b_k, src);
    BtQ[c * ldt + row] = ok ? vq : 0.0f;
    BtK[c * ldt + row] = ok ? vk : 0.0f;
  }
  for (int c = tid; c < d; c += kWideThreads) {
    qv[c] = ld_f32<T>(q, (int64_t)h * d + c);
    kv[c] = ld_f32<T>(k_new, ((int64_t)b * hkv + kvh) * d + c);
  }
  __syncthreads();
  // ---- G_K = B_K B_K^T, G_Q = B_Q B_Q^T + A^T A
  float gq[4][4], gk[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) gq[i][j] = gk[i][j] = 0.0f;
#pragma unroll 4
  for (int c = 0; c < d; ++c) {
    const float4 qi = *reinterpret_cast<const float4*>(BtQ + c * ldt + 4 * ti);
    const float4 qj = *reinterpret_cast<const float4*>(BtQ + c * ldt + 4 * tj);
    const float4 ki = *reinterpret_cast<const float4*>(BtK + c * ldt + 4 * ti);
    const float4 kj = *reinterpret_cast<const float4*>(BtK + c * ldt + 4 * tj);
    const float a[4] = {qi.x, qi.y, qi.z, qi.w}, bb[4] = {qj.x, qj.y, qj.z, qj.w};
    const float e[4] = {ki.x, ki.y, ki.z, ki.w}, f[4] = {kj.x, kj.y, kj.z, kj.w};
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        gq[i][j] = fmaf(a[i], bb[j], gq[i][j]);
        gk[i][j] = fmaf(e[i], f[j], gk[i][j]);
      }
  }
  const float* pin = part + (int64_t)h * S * ne;
  for (int s = 0; s < S; ++s) {  // (split order; the block's sixteen loads of a split go out together)
    float t[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        t[i][j] = pin[(int64_t)s * ne + min(4 * ti + i, r - 1) * r + min(4 * tj + j, r - 1)];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) gq[i][j] += t[i][j];
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int row = 4 * ti + i, col = 4 * tj + j;
      if (row >= r || col >= r) gq[i][j] = gk[i][j] = row == col ? 1.0f : 0.0f;
    }
  if (tid < r) {
    float rq = 0.0f, kb = 0.0f, aw = 0.0f;
    for (int c = 0; c < d; ++c) {
      rq = fmaf(qv[c], BtQ[c * ldt + tid], rq);
      kb = fmaf(kv[c], BtK[c * ldt + tid], kb);
    }
    for (int s0 = 0; s0 < S; s0 += 8) {
      float t[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) t[u] = pin[(int64_t)min(s0 + u, S - 1) * ne + r * r + tid];
#pragma unroll
      for (int u = 0; u < 8; ++u) aw += s0 + u < S ? t[u] : 0.0f;
    }
    rhs_q[tid] = rq + aw;   // q B_Q^T + (q K^T) A
    kB[tid] = kb;           // k B_K^T
  }
  if (tid >= kWideThreads - kWave) {  // (the last wave: the first is busy with the products above)
    float v = 0.0f;
    for (int c = tid - (kWideThreads - kWave); c < d; c += kWave) v = fmaf(qv[c], kv[c], v);
    v = wave_sum(v);
    if (tid == kWideThreads - kWave) s_red[0] = v;  // q . k
  }
  // ---- scale to unit diagonal
  if (ti == tj) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      scq[4 * ti + i] = rsqrtf(gq[i][i]);
      sck[4 * ti + i] = rsqrtf(gk[i][i]);
    }
  }
  __syncthreads();
  float sqr[4], sqc[4], skr[4], skc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    sqr[i] = scq[4 * ti + i];
    sqc[i] = scq[4 * tj + i];
    skr[i] = sck[4 * ti + i];
    skc[i] = sck[4 * tj + i];
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      gq[i][j] *= sqr[i] * sqc[j];
      gk[i][j] *= skr[i] * skc[j];
    }
  // ---- Gauss-Jordan, both matrices, one barrier per pivot
  for (int p = 0; p < r; ++p) {
    float* pb = pub + (p & 1) * 4 * R;
    const int pt = p >> 2, pe = p & 3;
    if (tj == pt) {  // this thread holds column p of rows 4 ti ..
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float cqv = gq[i][0], ckv = gk[i][0];
#pragma unroll
        for (int j = 1; j < 4; ++j) {
          cqv = pe == j ? gq[i][j] : cqv;
          ckv = pe == j ? gk[i][j] : ckv;
        }
        pb[4 * ti + i] = cqv;
        pb[2 * R + 4 * ti + i] = ckv;
      }
    }
    if (ti == pt) {  // row p of columns 4 tj ..
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float rqv = gq[0][j], rkv = gk[0][j];
#pragma unroll
        for (int i = 1; i < 4; ++i) {
          rqv = pe == i ? gq[i][j] : rqv;
          rkv = pe == i ? gk[i][j] : rkv;
        }
        pb[R + 4 * tj + j] = rqv;
        pb[3 * R + 4 * tj + j] = rkv;
      }
    }
    __syncthreads();
    const float pq_ = 1.0f / pb[p], pk_ = 1.0f / pb[2 * R + p];
    const float4 cq4 = *reinterpret_cast<const float4*>(pb + 4 * ti), rq4 = *reinterpret_cast<const float4*>(pb + R + 4 * tj);
    const float4 ck4 = *reinterpret_cast<const float4*>(pb + 2 * R + 4 * ti), rk4 = *reinterpret_cast<const float4*>(pb + 3 * R + 4 * tj);
    const float cq[4] = {cq4.x, cq4.y, cq4.z, cq4.w}, rq[4] = {rq4.x, rq4.y, rq4.z, rq4.w};
    const float ck[4] = {ck4.x, ck4.y, ck4.z, ck4.w}, rk[4] = {rk4.x, rk4.y, rk4.z, rk4.w};
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool rp = 4 * ti + i == p, cp = 4 * tj + j == p;
        const float uq = fmaf(-cq[i] * pq_, rq[j], gq[i][j]), uk = fmaf(-ck[i] * pk_, rk[j], gk[i][j]);
        const float vq = rp ? (cp ? pq_ : rq[j] * pq_) : (cp ? -cq[i] * pq_ : uq);
        const float vk = rp ? (cp ? pk_ : rk[j] * pk_) : (cp ? -ck[i] * pk_ : uk);
        gq[i][j] = vq;
        gk[i][j] = vk;
      }
  }
  // ---- scale back; the inverses go to LDS
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      GQ[(4 * ti + i) * ldg + 4 * tj + j] = gq[i][j] * sqr[i] * sqc[j];
      GK[(4 * ti + i) * ldg + 4 * tj + j] = gk[i][j] * skr[i] * skc[j];
    }
  __syncthreads();
  const float sqk = s_red[0];
  // out[c] = sum_i in[i] G[i][c]
  auto vecmat = [&](const float* in, const float* G, float* out) {
    if (tid < r) {
      float v = 0.0f;
      for (int i = 0; i < r; ++i) v = fmaf(in[i], G[i * ldg + tid], v);
      out[tid] = v;
    }
    __syncthreads();
  };
  // (a . b) over r elements, in every thread; s_red[1 + slot] is the scratch cell
  auto dot = [&](const float* a, const float* bb, int slot) {
    if (tid < kWave) {
      float v = tid < r ? a[tid] * bb[tid] : 0.0f;
      v = wave_sum(v);
      if (tid == 0) s_red[1 + slot] = v;
    }
    __syncthreads();
    const float v = s_red[1 + slot];
    return v;
  };
  // x = b (G + v^T v)^-1 with b = b0 + s v, from G^-1 (Sherman-Morrison): z = v G^-1, y = y0 + s z,
  // x = y - (y . v / (1 + z . v)) z
  auto rank1 = [&](const float* y0, const float* v, const float* G, float* out) {
    vecmat(v, G, z);
    if (tid < r) y[tid] = fmaf(sqk, z[tid], y0[tid]);
    __syncthreads();
    const float yv = dot(y, v, 0);
    const float zv = dot(z, v, 1);
    const float alpha = yv / (1.0f + zv);
    __syncthreads();  // (both cells read before the next call writes them)
    if (tid < r) out[tid] = fmaf(-alpha, z[tid], y[tid]);
    __syncthreads();
  };
  vecmat(kB, GK, hk0);      // k_hat_0 = kB G_K^-1
  vecmat(rhs_q, GQ, yq0);   // rhs_q G_Q^-1
  if (tid < r) hk[tid] = hk0[tid];
  __syncthreads();
  for (int it = 0; it < max_iter; ++it) {
    rank1(yq0, hk, GQ, hqv);   // q_hat (G_Q + k_hat^T k_hat) = rhs_q + s k_hat
    rank1(hk0, hqv, GK, y);    // k_hat' (G_K + q_hat^T q_hat) = kB + s q_hat   (the result takes y's place)
    float df = 0.0f;
    if (tid < r) {
      df = hk[tid] - y[tid];
      df *= df;
    }
    if (tid < kWave) {
      const float t = wave_sum(df);
      if (tid == 0) deltas[(int64_t)h * max_iter + it] = t;
    }
    float* o = iter_out + ((int64_t)h * max_iter + it) * 2 * r;
    if (tid < r) {
      o[tid] = hqv[tid];
      o[r + tid] = y[tid];
    }
    __syncthreads();
    if (tid < r) hk[tid] = y[tid];
    __syncthreads();
  }
}

template <typename T>
__global__ __launch_bounds__(kFinThreads) void als_finish_kernel(FinishArgs fa) {
  // workgroups [bh, 2 bh), if launched, encode the appended rows for the score index
  if ((int)blockIdx.x < fa.bh)
    als_finish_body<T>(fa, blockIdx.x);
  else
    als_index_append_body<T>(fa, (int)blockIdx.x - fa.bh);
}
static inline unsigned finish_grid(const FinishArgs& fa) {
  return (unsigned)fa.bh * (fa.qa != nullptr && fa.append_row >= 0 ? 2u : 1u);
}

// The finish stage of a factor update whose iterates are in iter_out / deltas: launched, or handed to the step's
// later launches.
template <typename T>
static int als_decode_finish(lrqk_ctx* ctx, void* b_q, void* b_k, void* a_k, int64_t head_stride, const void* q,
                             const void* k_new, int bh, int hq, int hkv, int r, int d, int lpr_log2, int max_iter,
                             float tol, void* q_hat, void* k_hat, int64_t append_row, float* iter_out, float* deltas,
                             bool defer_finish, hipStream_t st) {
  FinishArgs fa{b_q, b_k, q, k_new, iter_out, deltas, bh, hq, hkv, r, d, lpr_log2, max_iter, tol, q_hat, k_hat, a_k,
                head_stride, append_row, nullptr, nullptr, nullptr, 0};
  if (ctx->sidx_enabled && ctx->sidx_a_k == a_k && ctx->sidx_bh == bh && ctx->sidx_r == r && append_row >= 0 &&
      ctx->sidx_head_rows == head_stride / r && ctx->sidx_dtype == (sizeof(T) == 4 ? LRQK_F32 : LRQK_BF16)) {
    // the appended row also goes into the score index; rows stay contiguous as long as rows are appended in order
    fa.qa = (uint8_t*)ctx->sidx_qa.p;
    fa.qs = (uint16_t*)ctx->sidx_qs.p;
    fa.qw = (const float*)ctx->sidx_wm.p;
    fa.q_head_rows = ctx->sidx_head_rows;
    if (append_row == ctx->sidx_valid) ctx->sidx_valid = append_row + 1;  // (a gap is indexed on demand later)
  }
  if (defer_finish) {
    // the caller lets later launches of the step absorb the finish stage (flush_pending_finish otherwise)
    ctx->fin = fa;
    ctx->fin_dtype = sizeof(T) == 4 ? LRQK_F32 : LRQK_BF16;
    ctx->fin_pending = true;   // B update, outputs and the A_K row still to be done
    ctx->qhat_pending = true;  // q_hat has not been written yet: consumers take the iterate from iter_out
    return LRQK_OK;
  }
  hipLaunchKernelGGL((als_finish_kernel<T>), dim3(finish_grid(fa)), dim3(kFinThreads), 0, st, fa);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

template <typename T>
static int als_decode_impl(lrqk_ctx* ctx, void* b_q, void* b_k, void* a_k, int64_t head_stride,
                           const int32_t* active_idx, int64_t idx_stride, const void* k_prev, int kprev_slots, int n,
                           const void* q, const void* k_new, int b, int hq, int hkv, int r, int d, int max_iter,
                           float tol, void* q_hat, void* k_hat, int64_t append_row, GramAppend ap, bool defer_finish,
                           hipStream_t st) {
  constexpr int VEC = Vec16<T>::N;
  ctx->kq_valid = false;
  const int bh = b * hq;
  const int lpr = d / VEC;
  int lpr_log2 = 0;
  while ((1 << lpr_log2) < lpr) ++lpr_log2;
  LRQK_REQUIRE(d % VEC == 0 && (1 << lpr_log2) == lpr && lpr <= kWave && d <= 256 && d >= 8, LRQK_ELIMIT,
               "head_dim %d unsupported (need a power of two in 8..256 with at least one 16-byte chunk)", d);
  LRQK_REQUIRE(((uintptr_t)b_q % 16 == 0) && ((uintptr_t)b_k % 16 == 0) && ((int64_t)r * d * sizeof(T)) % 16 == 0,
               LRQK_EINVAL, "b_q/b_k must be 16-byte aligned");
  if (r > kAlsMaxR) {
    // ranks beyond one matrix-core tile: the general kernels
    const int S = std::min(32, std::max(1, (n + 255) / 256));
    const int ne = r * r + r;
    int rc = ctx->als_part.ensure((size_t)bh * S * ne * sizeof(float));
    if (rc) return rc;
    if ((rc = ctx->als_iter.ensure((size_t)bh * max_iter * (2 * r + 1) * sizeof(float)))) return rc;
    float* iter_out = (float*)ctx->als_iter.p;
    float* deltas = iter_out + (size_t)bh * max_iter * 2 * r;
    if (als_r64_supported(sizeof(T) == 2 ? LRQK_BF16 : LRQK_F32, r, d, a_k, head_stride)) {
      // bf16 rows of 128 elements: both launches on the matrix cores
      float* kq_out = nullptr;
      if (defer_finish && ap.slot >= 0 && n == kprev_slots) {
        if ((rc = ctx->als_kq.ensure((size_t)bh * n * sizeof(float)))) return rc;
        kq_out = (float*)ctx->als_kq.p;
      }
      if ((rc = als_r64_update(ctx, b_q, b_k, a_k, head_stride, active_idx, idx_stride, (void*)k_prev, kprev_slots, n, q,
                               k_new, bh, hq, hkv, r, max_iter, iter_out, deltas, ap, kq_out, st)))
        return rc;
      if (kq_out) {
        ctx->kq_valid = true;
        ctx->kq_k_act = k_prev;
        ctx->kq_q = q;
        ctx->kq_bh = bh;
        ctx->kq_n = n;
      }
      return als_decode_finish<T>(ctx, b_q, b_k, a_k, head_stride, q, k_new, bh, hq, hkv, r, d, lpr_log2, max_iter, tol,
                                  q_hat, k_hat, append_row, iter_out, deltas, defer_finish, st);
    }
    float* part = (float*)ctx->als_part.p;
    const size_t smem_g = ((size_t)kWideTile * (kWideMaxR + 4) + kWideTile + d) * sizeof(float);
    const size_t smem_s = ((size_t)2 * d * (kWideMaxR + 4) + (size_t)2 * kWideMaxR * (kWideMaxR + 1) + 2 * d + 18 * kWideMaxR) * sizeof(float);
    LRQK_REQUIRE(smem_s <= (size_t)160 * 1024 - 256, LRQK_ELIMIT, "r=%d with rows of %d elements needs too much LDS", r, d);
    static std::atomic<size_t> wide_allowed_dev[kMaxDeviceSlots];
    std::atomic<size_t>& wide_allowed = wide_allowed_dev[per_device_slot()];
    if (smem_s > std::max<size_t>(wide_allowed, 48 * 1024)) {
      LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)als_solve_wide_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)smem_s));
      wide_allowed = smem_s;
    }
    hipLaunchKernelGGL((als_gram_wide_kernel<T>), dim3((unsigned)S, (unsigned)bh), dim3(kWideThreads), smem_g, st,
                       (const T*)a_k, head_stride, head_stride / r, active_idx, idx_stride, (T*)k_prev, kprev_slots, n,
                       (const T*)q, r, d, part, S, ap);
    LRQK_HIP_CHECK(hipGetLastError());
    hipLaunchKernelGGL((als_solve_wide_kernel<T>), dim3((unsigned)bh), dim3(kWideThreads), smem_s, st, (const float*)part,
                       S, (const T*)b_q, (const T*)b_k, (const T*)q, (const T*)k_new, hq, hkv, r, d, max_iter, iter_out,
                       deltas);
    LRQK_HIP_CHECK(hipGetLastError());
    return als_decode_finish<T>(ctx, b_q, b_k, a_k, head_stride, q, k_new, bh, hq, hkv, r, d, lpr_log2, max_iter, tol, q_hat,
                                k_hat, append_row, iter_out, deltas, defer_finish, st);
  }
  // one 32-token chunk per wave where possible: a workgroup then pays two memory latencies
  int S = (n + kGramWaves * kGramChunk - 1) / (kGramWaves * kGramChunk);
  if (S < 1) S = 1;
  if (S > 32) S = 32;
  // bf16, d = 128, r in {8, 16, 24, 32}, 16-byte aligned rows: the pipelined pass on the bf16 matrix cores
  const bool fast_bf16 = sizeof(T) == 2 && d == 128 && r % 8 == 0 && ((uintptr_t)a_k % 16 == 0) &&
                         (head_stride * sizeof(T)) % 16 == 0 && !getenv("LRQK_GRAM_OLD");
  // (the pipelined pass: two chunks per wave measured best at 1, 4 and 8 sequences of the Llama-3-8B shape)
  if (fast_bf16) S = std::min(32, std::max(1, (n + 2 * kGramWaves * kGramChunk - 1) / (2 * kGramWaves * kGramChunk)));
  int rc = ctx->als_part.ensure((size_t)bh * S * kGramNe * sizeof(float));
  if (rc) return rc;
  if ((rc = ctx->als_iter.ensure((size_t)bh * max_iter * (2 * r + 1) * sizeof(float)))) return rc;
  float* part = (float*)ctx->als_part.p;
  float* iter_out = (float*)ctx->als_iter.p;
  float* deltas = iter_out + (size_t)bh * max_iter * 2 * r;
  const int64_t a_rows = head_stride / r;

  const size_t smem_solve = ((size_t)kGramNe + 2 * 32 + 2 * 32 * kLdi + 6 * 32 + 4 * 1024) * sizeof(float);
  static_assert(((size_t)kGramNe + 2 * 32 + 2 * 32 * kLdi + 6 * 32 + 4 * 1024) * sizeof(float) <= 48 * 1024,
                "the solve kernel's LDS fits the default dynamic limit");
  // the Gram launch carries two more workgroups per head, each with B_Q or B_K (fp32, padded rows) in LDS
  const size_t smem_gram = ((size_t)32 * (d + 1) + 2 * d) * sizeof(float);
  static std::atomic<size_t> gram_allowed_dev[kMaxDeviceSlots];
  std::atomic<size_t>& gram_allowed = gram_allowed_dev[per_device_slot()];
  if (smem_gram > std::max<size_t>(gram_allowed, 48 * 1024)) {
    LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)als_gram_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem_gram));
    gram_allowed = smem_gram;
  }
  if ((rc = ctx->als_pre.ensure((size_t)bh * kPreNe * sizeof(float)))) return rc;
  float* pre = (float*)ctx->als_pre.p;
  // With the ring append folded in, the pass sees every slot as the attention of this step will (except the
  // slots that the misses replace): it leaves K q per slot for that attention.
  float* kq_out = nullptr;
  if (defer_finish && ap.slot >= 0 && n == kprev_slots) {
    if ((rc = ctx->als_kq.ensure((size_t)bh * n * sizeof(float)))) return rc;
    kq_out = (float*)ctx->als_kq.p;
  }
  if (fast_bf16) {
    hipLaunchKernelGGL(als_gram_bf16_kernel, dim3((unsigned)S + 2, (unsigned)bh), dim3(kGramThreads), 0, st,
                       (const bf16_t*)a_k, head_stride, a_rows, active_idx, idx_stride, (bf16_t*)k_prev, kprev_slots, n,
                       (const bf16_t*)q, r, part, S, ap, (const bf16_t*)b_q, (const bf16_t*)b_k, (const bf16_t*)k_new,
                       hq, hkv, pre, kq_out);
  } else {
    hipLaunchKernelGGL((als_gram_kernel<T>), dim3((unsigned)S + 2, (unsigned)bh), dim3(kGramThreads), smem_gram, st,
                       (const T*)a_k, head_stride, a_rows, active_idx, idx_stride, (T*)k_prev, kprev_slots, n,
                       (const T*)q, r, d, lpr_log2, part, S, ap, (const T*)b_q, (const T*)b_k, (const T*)k_new, hq, hkv,
                       pre, kq_out);
  }
  LRQK_HIP_CHECK(hipGetLastError());
  if (kq_out) {
    ctx->kq_valid = true;
    ctx->kq_k_act = k_prev;
    ctx->kq_q = q;
    ctx->kq_bh = bh;
    ctx->kq_n = n;
  }
#define LRQK_SOLVE_CASE(KS)                                                                                     \
  hipLaunchKernelGGL((als_solve_kernel<KS>), dim3((unsigned)bh), dim3(kSolveThreads), smem_solve, st, (const float*)pre, \
                     (const float*)part, S, r, max_iter, iter_out, deltas)
  switch ((S + 3) / 4) {
    case 1: LRQK_SOLVE_CASE(4); break;
    case 2: LRQK_SOLVE_CASE(8); break;
    case 3: LRQK_SOLVE_CASE(12); break;
    case 4: LRQK_SOLVE_CASE(16); break;
    case 5: LRQK_SOLVE_CASE(20); break;
    case 6: LRQK_SOLVE_CASE(24); break;
    case 7: LRQK_SOLVE_CASE(28); break;
    default: LRQK_SOLVE_CASE(32); break;
  }
#undef LRQK_SOLVE_CASE
  LRQK_HIP_CHECK(hipGetLastError());
  return als_decode_finish<T>(ctx, b_q, b_k, a_k, head_stride, q, k_new, bh, hq, hkv, r, d, lpr_log2, max_iter, tol, q_hat,
                              k_hat, append_row, iter_out, deltas, defer_finish, st);
}

static int als_decode_checked(lrqk_ctx* ctx, void* b_q, void* b_k, void* a_k, int64_t head_stride,
                              const int32_t* active_idx, int64_t idx_stride, const void* k_prev, int kprev_slots, int n,
                              const void* q, const void* k_new, int b, int hq, int hkv, int r, int d, int max_iter,
                              float tol, void* q_hat, void* k_hat, int64_t append_row, GramAppend ap, bool defer_finish,
                              int dtype, hipStream_t st) {
  LRQK_REQUIRE(ctx && b_q && b_k && a_k && k_prev && q && k_new && q_hat && k_hat, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(dtype == LRQK_F32 || dtype == LRQK_BF16, LRQK_EINVAL, "dtype=%d", dtype);
  LRQK_REQUIRE(b > 0 && hq > 0 && hkv > 0 && hq % hkv == 0 && (int64_t)b * hq <= 65535, LRQK_EINVAL,
               "bad heads b=%d hq=%d hkv=%d", b, hq, hkv);
  LRQK_REQUIRE(r > 0 && r <= kWideMaxR, LRQK_ELIMIT, "r=%d not in 1..%d (the factor update supports rank <= %d)", r,
               kWideMaxR, kWideMaxR);
  LRQK_REQUIRE((int64_t)r * d * (int64_t)elem_size(dtype) / 16 <= 2048, LRQK_ELIMIT,
               "r=%d x d=%d: B_Q, B_K exceed the 32 KB each that the finish stage holds in registers", r, d);
  LRQK_REQUIRE(n > 0 && n <= kprev_slots, LRQK_EINVAL, "n=%d outside 1..%d", n, kprev_slots);
  LRQK_REQUIRE(!active_idx || idx_stride >= n, LRQK_EINVAL, "idx_stride < n");
  LRQK_REQUIRE(head_stride >= r && head_stride % r == 0, LRQK_EINVAL, "head_stride must be a multiple of r");
  LRQK_REQUIRE(active_idx || (int64_t)n * r <= head_stride, LRQK_EINVAL, "n rows exceed the A_K head");
  LRQK_REQUIRE(append_row < head_stride / r, LRQK_EINVAL, "append_row beyond the A_K capacity");
  if (max_iter < 1) max_iter = 1;
  LRQK_REQUIRE(max_iter <= LRQK_MAX_DECODE_ITERS, LRQK_ELIMIT, "max_iter=%d > %d", max_iter, LRQK_MAX_DECODE_ITERS);
  LRQK_REQUIRE(((uintptr_t)q % 16 == 0) && ((uintptr_t)k_prev % 16 == 0), LRQK_EINVAL, "pointers must be 16-byte aligned");
  if (dtype == LRQK_F32)
    return als_decode_impl<float>(ctx, b_q, b_k, a_k, head_stride, active_idx, idx_stride, k_prev, kprev_slots, n, q,
                                  k_new, b, hq, hkv, r, d, max_iter, tol, q_hat, k_hat, append_row, ap, defer_finish, st);
  return als_decode_impl<bf16_t>(ctx, b_q, b_k, a_k, head_stride, active_idx, idx_stride, k_prev, kprev_slots, n, q,
                                 k_new, b, hq, hkv, r, d, max_iter, tol, q_hat, k_hat, append_row, ap, defer_finish, st);
}

// The factor update with the ring append of (k_new, v_new) at slot `slot` as token `token` folded
// into its first kernel (same result as lrqk_append_token followed by lrqk_als_decode).
int als_decode_append(lrqk_ctx* ctx, void* b_q, void* b_k, void* a_k, int64_t head_stride, int32_t* active_idx,
                      int64_t idx_stride, void* k_act, void* v_act, int n_slots, const void* q, const void* k_new,
                      const void* v_new, int b, int hq, int hkv, int r, int d, int max_iter, float tol, void* q_hat,
                      void* k_hat, int64_t append_row, int slot, int32_t token, bool defer_finish, int dtype,
                      hipStream_t st) {
  LRQK_REQUIRE(active_idx && v_act && v_new, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(slot >= 0 && slot < n_slots, LRQK_EINVAL, "slot=%d outside 0..%d", slot, n_slots);
  LRQK_REQUIRE(((uintptr_t)k_new % 16 == 0) && ((uintptr_t)v_new % 16 == 0) && ((uintptr_t)v_act % 16 == 0), LRQK_EINVAL,
               "pointers must be 16-byte aligned");
  GramAppend ap{k_new, v_new, v_act, active_idx, slot, token, hq, hkv};
  return als_decode_checked(ctx, b_q, b_k, a_k, head_stride, active_idx, idx_stride, k_act, n_slots, n_slots, q, k_new, b,
                            hq, hkv, r, d, max_iter, tol, q_hat, k_hat, append_row, ap, defer_finish, dtype, st);
}

int als_defer_finish(lrqk_ctx* ctx, void* b_q, void* b_k, void* a_k, int64_t head_stride, const void* q,
                     const void* k_new, int bh, int hq, int hkv, int r, int d, int max_iter, float tol, void* q_hat,
                     void* k_hat, int64_t append_row, float* iter_out, float* deltas, int dtype) {
  const int vec = dtype == LRQK_F32 ? 4 : 8;
  int lpr_log2 = 0;
  while ((1 << lpr_log2) < d / vec) ++lpr_log2;
  if (dtype == LRQK_F32)
    return als_decode_finish<float>(ctx, b_q, b_k, a_k, head_stride, q, k_new, bh, hq, hkv, r, d, lpr_log2, max_iter, tol,
                                    q_hat, k_hat, append_row, iter_out, deltas, true, nullptr);
  return als_decode_finish<bf16_t>(ctx, b_q, b_k, a_k, head_stride, q, k_new, bh, hq, hkv, r, d, lpr_log2, max_iter, tol,
                                   q_hat, k_hat, append_row, iter_out, deltas, true, nullptr);
}

// Runs a deferred finish stage as its own launch (when no later launch of the step took it over).
int flush_pending_finish(lrqk_ctx* ctx, hipStream_t st) {
  if (!ctx->fin_pending) return LRQK_OK;
  ctx->fin_pending = false;
  ctx->qhat_pending = false;
  if (ctx->fin_dtype == LRQK_F32)
    hipLaunchKernelGGL((als_finish_kernel<float>), dim3(finish_grid(ctx->fin)), dim3(kFinThreads), 0, st, ctx->fin);
  else
    hipLaunchKernelGGL((als_finish_kernel<bf16_t>), dim3(finish_grid(ctx->fin)), dim3(kFinThreads), 0, st, ctx->fin);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

}  // namespace lrqk

using namespace lrqk;

extern "C" int lrqk_als_decode(lrqk_ctx* ctx, void* b_q, void* b_k, void* a_k, int64_t head_stride,
                               const int32_t* active_idx, int64_t idx_stride, const void* k_prev, int kprev_slots,
                               int n, const void* q, const void* k_new, int b, int hq, int hkv, int r, int d,
                               int max_iter, float tol, void* q_hat, void* k_hat, int64_t append_row, int dtype,
                               void* stream) {
  GramAppend ap{nullptr, nullptr, nullptr, nullptr, -1, 0, hq, hkv};
  if (ctx) ctx->fs_valid = false;  // B_Q, B_K change behind the kept state of the decode step
  return als_decode_checked(ctx, b_q, b_k, a_k, head_stride, active_idx, idx_stride, k_prev, kprev_slots, n, q, k_new, b,
                            hq, hkv, r, d, max_iter, tol, q_hat, k_hat, append_row, ap, false, dtype, (hipStream_t)stream);
}
