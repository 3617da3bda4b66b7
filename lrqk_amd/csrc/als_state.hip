// Per-step factor update of the decode step with everything that does not depend on the step's (q, k)
// taken out of its critical path (r <= 32).
//
// With all weights 1 the update of lrqk_attention.py:555-609 is
//   k_hat_0 = (k B_K^T) G_K^-1,                                            G_K = B_K B_K^T
//   q_hat   = (q B_Q^T + (q K__^T) A + s k_hat)(G_Q + k_hat^T k_hat)^-1,    G_Q = B_Q B_Q^T + A^T A,  s = q . k
//   k_hat'  = (k B_K^T + s q_hat)(G_K + q_hat^T q_hat)^-1
// where A are the A_K rows of the active slots and K__ their K rows.  The new token's A_K row is zero while
// its update runs (it is appended afterwards), so B_Q, B_K, A^T A and M = K__^T A (d x r) are all functions of
// the state that the previous step left.  They are kept per head in fp64:
//   M, GA = A^T A        sums over the active slots, kept up to date from the rows that a step replaces
//                        (bf16 x bf16 and fp32 x fp32 products are exact in fp64, so adding and later removing a
//                        row's term leaves roundings of 2^-53: nothing that matters against fp32 sums formed from
//                        scratch, however many steps pass)
//   N = B_Q^T + M (d x r),  GQi = G_Q^-1,  GKi = G_K^-1
// A step then needs  q N,  k B_K^T,  s = q . k, two products with the inverses and their rank-one
// (Sherman-Morrison) updates per iteration: one small launch in fp64 (als_quick_kernel), which also appends the
// new token to the ring.  After the step's fetch one more launch (als_state_tail_kernel) brings the state up to
// date; nothing waits for it except the same layer's next step.
#include <algorithm>
#include <atomic>

#include "common.hpp"
#include "ctx.hpp"
#include "als_finish.hpp"

namespace lrqk {

constexpr int kQsThreads = 256;
constexpr int kFsTerms = 256;  // rows staged per pass of the tail kernel's sums (one per thread)
typedef double fs_v4d __attribute__((ext_vector_type(4)));


// per head (doubles): N [d][32] | GQi [32][32] | GKi [32][32] | M [d][32] | GA [32][32]
static __host__ __device__ constexpr int64_t fs_stride(int d) { return (int64_t)2 * d * 32 + 3 * 1024; }

// ----------------------------------------------------------------------------- fp64 across the lanes of a wave
__device__ __forceinline__ double bcast_f64(double v, int lane) {
  const int lo = __builtin_amdgcn_readlane(__double2loint(v), lane);
  const int hi = __builtin_amdgcn_readlane(__double2hiint(v), lane);
  return __hiloint2double(hi, lo);
}
template <int CTRL>
__device__ __forceinline__ double dpp_f64(double v) {
  const int lo = __builtin_amdgcn_update_dpp(__double2loint(v), __double2loint(v), CTRL, 0xf, 0xf, false);
  const int hi = __builtin_amdgcn_update_dpp(__double2hiint(v), __double2hiint(v), CTRL, 0xf, 0xf, false);
  return __hiloint2double(hi, lo);
}
// sum over lanes 0..31 (two rows of 16 lanes); every lane of the wave must call it, result in every lane
__device__ __forceinline__ double sum_lanes_0_31_f64(double x) {
  x += dpp_f64<kDppQuadXor1>(x);
  x += dpp_f64<kDppQuadXor2>(x);
  x += dpp_f64<kDppRowHalfMirror>(x);
  x += dpp_f64<kDppRowMirror>(x);
  return bcast_f64(x, 0) + bcast_f64(x, 16);
}
__device__ __forceinline__ double wave_sum_f64(double x) {
  x += dpp_f64<kDppQuadXor1>(x);
  x += dpp_f64<kDppQuadXor2>(x);
  x += dpp_f64<kDppRowHalfMirror>(x);
  x += dpp_f64<kDppRowMirror>(x);
  return (bcast_f64(x, 0) + bcast_f64(x, 16)) + (bcast_f64(x, 32) + bcast_f64(x, 48));
}
// 1 / x to full precision for a finite, normal x (the pivots of a matrix scaled to unit diagonal)
__device__ __forceinline__ double recip_f64(double x) {
  double y = __builtin_amdgcn_rcp(x);
  y = fma(fma(-x, y, 1.0), y, y);
  y = fma(fma(-x, y, 1.0), y, y);
  return y;
}

// ----------------------------------------------------------------------------- the step's own launch
// One workgroup per head.  Ring append (slot `slot` <- k_new, v_new, token), then the iterations from the kept
// state.  Outputs in the layout of als_solve_kernel: iter_out [bh][max_iter][2r] (q_hat, then k_hat of every
// iteration), deltas [bh][max_iter]; iter64 the same iterates before they are rounded to fp32.
template <typename T, int D>
__global__ __launch_bounds__(kQsThreads) void als_quick_kernel(const double* __restrict__ state,
                                                               const T* __restrict__ q, const T* __restrict__ k_new,
                                                               const T* __restrict__ v_new, T* __restrict__ k_act,
                                                               T* __restrict__ v_act, int n_slots,
                                                               int32_t* __restrict__ active_idx, int64_t idx_stride,
                                                               int slot, int32_t token, const T* __restrict__ b_k,
                                                               int hq, int hkv, int r, int max_iter,
                                                               float* __restrict__ iter_out, float* __restrict__ deltas,
                                                               double* __restrict__ iter64) {
  constexpr int VEC = Vec16<T>::N;
  constexpr int EPT = D / 8;  // elements of a B_K row per thread
  __shared__ double qs[D], ks[D];
  __shared__ double redq[8][32], kbs[32];
  __shared__ double s_qk;
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const int h = blockIdx.x;
  const int b = h / hq, kvh = (h % hq) / (hq / hkv);
  const double* st = state + (int64_t)h * fs_stride(D);
  const double* N = st;
  const double* GQi = st + (int64_t)D * 32;
  const double* GKi = GQi + 1024;
  const int c = tid & 31, g = tid >> 5;
  // ---- every global load goes out here: the inverses' columns (for the wave that iterates), N, B_K, q, k
  double cK[32], cQ[32];
  if (wave == 0) {
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      cK[i] = GKi[i * 32 + c];
      cQ[i] = GQi[i * 32 + c];
    }
  }
  double pn[D / 8];
#pragma unroll
  for (int u = 0; u < D / 8; ++u) pn[u] = N[(int64_t)(g + 8 * u) * 32 + c];
  const int brow = tid >> 3, part = tid & 7;
  float bkf[EPT];
  {
    const T* src = b_k + ((int64_t)h * r + min(brow, r - 1)) * D + part * EPT;
    if constexpr (EPT % VEC == 0) {
#pragma unroll
      for (int v = 0; v < EPT / VEC; ++v) {
        Vec16<T> x;
        x.load(src + v * VEC);
        x.unpack(bkf + v * VEC);
      }
    } else {
#pragma unroll
      for (int e = 0; e < EPT; ++e) bkf[e] = ld_f32<T>(src, e);
    }
  }
  const int64_t src_row = ((int64_t)b * hkv + kvh) * D;
  {
    const int cc = min(tid, D - 1);
    const double qx = (double)ld_f32<T>(q, (int64_t)h * D + cc);
    const double kx = (double)ld_f32<T>(k_new, src_row + cc);
    if (tid < D) {
      qs[tid] = qx;
      ks[tid] = kx;
    }
  }
  // ring append: the first lanes copy the K row, the next ones the V row, 16 bytes each
  {
    constexpr int cpr = D / VEC;  // <= 64
    if (tid < 2 * cpr) {
      const bool is_k = tid < cpr;
      const int ch = is_k ? tid : tid - cpr;
      Vec16<T> x;
      x.load((is_k ? k_new : v_new) + src_row + ch * VEC);
      x.store((is_k ? k_act : v_act) + ((int64_t)h * n_slots + slot) * D + ch * VEC);
    }
    if (tid == kQsThreads - 1) active_idx[(int64_t)h * idx_stride + slot] = token;
  }
  __syncthreads();
  // q N: thread (column c, row group g) takes rows g, g + 8, ...;  k B_K^T: eight threads per row of B_K
  double aq = 0.0, ak = 0.0;
#pragma unroll
  for (int u = 0; u < D / 8; ++u) aq = fma(qs[g + 8 * u], pn[u], aq);
#pragma unroll
  for (int e = 0; e < EPT; ++e) ak = fma(ks[part * EPT + e], (double)bkf[e], ak);
  ak += dpp_f64<kDppQuadXor1>(ak);
  ak += dpp_f64<kDppQuadXor2>(ak);
  ak += dpp_f64<kDppRowHalfMirror>(ak);
  redq[g][c] = aq;
  if (part == 0) kbs[brow] = brow < r ? ak : 0.0;
  if (wave == 1) {
    double v = 0.0;
    for (int j = lane; j < D; j += kWave) v = fma(qs[j], ks[j], v);
    v = wave_sum_f64(v);
    if (lane == 0) s_qk = v;
  }
  __syncthreads();
  if (wave != 0) return;
  double rq = 0.0;
#pragma unroll
  for (int u = 0; u < 8; ++u) rq += redq[u][c];
  const double kb = kbs[c];
  const double sqk = s_qk;
  // y_c = sum_i b_i col[i]  (b lane-distributed; lanes 32..63 mirror lanes 0..31)
  auto vecmat = [&](double bvec, const double (&col)[32]) {
    double y0 = 0.0, y1 = 0.0;
#pragma unroll
    for (int i = 0; i < 32; i += 2) {
      y0 = fma(bcast_f64(bvec, i), col[i], y0);
      y1 = fma(bcast_f64(bvec, i + 1), col[i + 1], y1);
    }
    return y0 + y1;
  };
  // x = (y0 + s v)(G + v^T v)^-1 from G^-1 (Sherman-Morrison): z = v G^-1, y = y0 + s z, x = y - (y.v / (1 + z.v)) z
  auto rank1 = [&](double y0, double v, const double (&col)[32]) {
    const double z = vecmat(v, col);
    const double y = fma(sqk, z, y0);
    const double alpha = sum_lanes_0_31_f64(y * v) / (1.0 + sum_lanes_0_31_f64(z * v));
    return fma(-alpha, z, y);
  };
  const double hk0 = vecmat(kb, cK);  // k_hat_0 = (k B_K^T) G_K^-1
  const double yq0 = vecmat(rq, cQ);  // (q B_Q^T + q K__^T A) G_Q^-1
  double hk = hk0;
  for (int it = 0; it < max_iter; ++it) {
    const double hqv = rank1(yq0, hk, cQ);  // q_hat (G_Q + k_hat^T k_hat) = rhs_q + s k_hat
    const double nk = rank1(hk0, hqv, cK);  // k_hat' (G_K + q_hat^T q_hat) = k B_K^T + s q_hat
    const double df = c < r ? hk - nk : 0.0;
    const double dsq = sum_lanes_0_31_f64(df * df);
    if (lane == 0) deltas[(int64_t)h * max_iter + it] = (float)dsq;
    const int64_t o = ((int64_t)h * max_iter + it) * 2 * r;
    if (lane < r) {
      iter_out[o + lane] = (float)hqv;
      iter_out[o + r + lane] = (float)nk;
      iter64[o + lane] = hqv;
      iter64[o + r + lane] = nk;
    }
    hk = nk;
  }
}

// ----------------------------------------------------------------------------- the kept state
struct TailArgs {
  double* state;
  const void* a_k;
  int64_t head_stride, a_rows;
  const int32_t* active_idx;
  int64_t idx_stride;
  const void* k_act;
  int n_slots;
  const void* evk;            // [bh][evk_rows][d]: K rows that this step's misses replaced (written by the fetch)
  int evk_rows;
  const int32_t* miss_slots;  // [bh][k]
  const int32_t* miss_old;    // [bh][k]
  const int32_t* miss_new;    // [bh][k]
  const int32_t* miss_count;  // [bh]
  int k;
  int64_t cap;                // rows of the host store (a miss beyond it was not fetched)
  int ring_slot;              // slot of the token that this step appended (its A_K row exists now); -1: none
  int32_t ring_token;
  int skip_slot;              // slot that the next step overwrites: not part of its sums
  int rebuild;                // != 0: every head's sums are formed from scratch
  int r;
  const void* b_q;
  const void* b_k;
};

// One 32 x 32 block of the sums of the next step's view (all slots but skip_slot, each with the A_K row of the
// token it holds): block blk < D / 32 is rows 32 blk .. of M, block D / 32 is GA.  A pass stages up to 256
// terms -- a row of 32 "left" elements (a K row's part, or the A_K row itself for GA) and the signed A_K row --
// in LDS as they are stored (bf16 and fp32 values are fp32 values), one term per thread; then the four waves each
// add the terms' products to one 16 x 16 tile on the fp64 matrix cores (16 x 16 x 4: four terms per instruction,
// operands widened on the way in, four accumulators in turn because a product waits ~100 cycles for the one
// before it).  Terms: the appended token's row (+), the row that the next step overwrites (-), and for every
// miss the row that came in (+) and the row it replaced (-, from evk); or, from scratch, every slot.  A head
// with more misses than evk holds rows is formed from scratch.
// Element v of lane l of wave w: row 16 (w >> 1) + (l >> 4) + 4 v, column 16 (w & 1) + (l & 15).
// mid() runs once, after the first pass's row loads have been requested and before they are waited for.
// Returns true if the block was formed from scratch (its value replaces the kept one).
constexpr int kFsLdf = 36;  // floats per staged row (16-byte aligned rows, 16-byte stores spread over all banks)
template <typename T, int D, typename Mid>
__device__ __forceinline__ bool fs_block_sums(const TailArgs& ta, int h, int blk, float* __restrict__ Lb,
                                              float* __restrict__ Ab, fs_v4d& acc, Mid&& mid) {
  constexpr int VEC = Vec16<T>::N;
  constexpr int NV = 32 / VEC;  // 16-byte pieces per block of 32 elements
  const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
  const bool ga_role = blk == D / 32;
  const int r = ta.r, k = ta.k;
  const T* A = (const T*)ta.a_k + (int64_t)h * ta.head_stride;
  const T* Kh = (const T*)ta.k_act + (int64_t)h * ta.n_slots * D;
  const T* Eh = (const T*)ta.evk + (int64_t)h * ta.evk_rows * D;
  const int32_t* ids = ta.active_idx + (int64_t)h * ta.idx_stride;
  // every list entry that a thread may need is requested before the head's miss count is looked at: the terms are
  // the appended token's row (e = 0), the row that the next step overwrites (e = 1), then for every miss j the row
  // that came in (e = 2 + 2 j) and the row it replaced (e = 3 + 2 j) -- indices that do not depend on the count
  const int skip_c = min(max(ta.skip_slot, 0), ta.n_slots - 1);
  const int ring_c = min(max(ta.ring_slot, 0), ta.n_slots - 1);
  const int32_t skip_id = ids[skip_c];
  const bool lists = ta.miss_slots != nullptr;
  int32_t ms0 = 0, mn0 = 0, mo0 = 0, id0 = ids[min(tid, ta.n_slots - 1)];
  {
    const int jc = min(max(tid - 2, 0) >> 1, k - 1);
    if (lists) {  // (uniform)
      ms0 = ta.miss_slots[(int64_t)h * k + jc];
      mn0 = ta.miss_new[(int64_t)h * k + jc];
      mo0 = ta.miss_old[(int64_t)h * k + jc];
    }
  }
  const int cnt_raw = ta.miss_count ? ta.miss_count[h] : 0;
  const int cnt = min(max(cnt_raw, 0), k);
  const bool scratch = ta.rebuild != 0 || cnt > ta.evk_rows || !lists;
  const int nterms = scratch ? ta.n_slots : 2 * cnt + 2;
  const bool vec_a = r % VEC == 0 && ((uintptr_t)A % 16 == 0) && (ta.head_stride * sizeof(T)) % 16 == 0;
  const int li = lane & 15, lk = lane >> 4, rt = wave >> 1, ct = wave & 1;
  fs_v4d acc4[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) acc4[u] = fs_v4d{0.0, 0.0, 0.0, 0.0};
  for (int e0 = 0; e0 < nterms; e0 += kFsTerms) {
    const int e = e0 + tid;
    // ---- which row this thread stages (every load unconditional: clamped index, masked value)
    int slot, j = 0;
    int32_t id;
    bool ok, from_evk = false;
    float sign = 1.0f;
    if (scratch) {
      slot = min(e, ta.n_slots - 1);
      id = e0 == 0 ? id0 : ids[slot];
      ok = e < ta.n_slots && slot != ta.skip_slot;
    } else {
      j = max(e - 2, 0) >> 1;
      const int jc = min(j, k - 1);
      int32_t ms = ms0, mn = mn0, mo = mo0;
      if (e0 > 0) {  // (uniform)
        ms = ta.miss_slots[(int64_t)h * k + jc];
        mn = ta.miss_new[(int64_t)h * k + jc];
        mo = ta.miss_old[(int64_t)h * k + jc];
      }
      const bool fetched = ms >= 0 && ms < k && mn >= 0 && mn < ta.cap;  // what the fetch role requires of a miss
      if (e >= 2) {
        const bool plus = ((e - 2) & 1) == 0;
        slot = fetched ? ms : 0;
        id = plus ? mn : mo;
        ok = fetched && j < cnt;
        from_evk = !plus;
        sign = plus ? 1.0f : -1.0f;
      } else if (e == 0) {
        slot = ring_c;
        id = ta.ring_token;
        ok = ta.ring_slot >= 0;
      } else {
        slot = skip_c;
        id = skip_id;
        ok = ta.skip_slot >= 0;
        sign = -1.0f;
      }
    }
    const bool a_ok = ok && id >= 0 && (int64_t)id < ta.a_rows;
    const int64_t arow = a_ok ? (int64_t)id : 0;
    // ---- the A_K row (elements >= r are zero) and the left row: requested together
    Vec16<T> av[NV], kv[NV];
    float af[32];
    if (vec_a) {
#pragma unroll
      for (int v = 0; v < NV; ++v) av[v].load(A + arow * r + min(v * VEC, r - VEC));
    } else {
#pragma unroll
      for (int u = 0; u < 32; ++u) af[u] = ld_f32<T>(A, arow * r + min(u, r - 1));
    }
    if (!ga_role) {
      const T* krow = (from_evk ? Eh + (int64_t)min(j, ta.evk_rows - 1) * D : Kh + (int64_t)slot * D) + 32 * blk;
#pragma unroll
      for (int v = 0; v < NV; ++v) kv[v].load(krow + v * VEC);
    }
    if (e0 == 0) mid();
    if (vec_a) {
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        float f[VEC];
        av[v].unpack(f);
#pragma unroll
        for (int u = 0; u < VEC; ++u) af[v * VEC + u] = (a_ok && v * VEC < r) ? f[u] : 0.0f;
      }
    } else {
#pragma unroll
      for (int u = 0; u < 32; ++u) af[u] = (a_ok && u < r) ? af[u] : 0.0f;
    }
    float4* lrow = reinterpret_cast<float4*>(Lb + tid * kFsLdf);
    float4* arow_s = reinterpret_cast<float4*>(Ab + tid * kFsLdf);
#pragma unroll
    for (int u = 0; u < 8; ++u)
      arow_s[u] = make_float4(sign * af[4 * u], sign * af[4 * u + 1], sign * af[4 * u + 2], sign * af[4 * u + 3]);
    if (ga_role) {
#pragma unroll
      for (int u = 0; u < 8; ++u) lrow[u] = make_float4(af[4 * u], af[4 * u + 1], af[4 * u + 2], af[4 * u + 3]);
    } else {
      float kf[32];
#pragma unroll
      for (int v = 0; v < NV; ++v) kv[v].unpack(kf + v * VEC);
#pragma unroll
      for (int u = 0; u < 8; ++u)
        lrow[u] = ok ? make_float4(kf[4 * u], kf[4 * u + 1], kf[4 * u + 2], kf[4 * u + 3]) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    __syncthreads();
    // (rows beyond the last term were staged as zeros, so whole groups of four terms are added, eight at a time)
    const int groups = (min(kFsTerms, nterms - e0) + 3) >> 2;
    const float* pa = Lb + lk * kFsLdf + 16 * rt + li;
    const float* pb = Ab + lk * kFsLdf + 16 * ct + li;
    for (int s0 = 0; s0 < groups; s0 += 8) {
      float fa[8], fb[8];
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        fa[s] = pa[(s0 + s) * 4 * kFsLdf];
        fb[s] = pb[(s0 + s) * 4 * kFsLdf];
      }
#pragma unroll
      for (int s = 0; s < 8; ++s)
        acc4[s & 3] = __builtin_amdgcn_mfma_f64_16x16x4f64((double)fa[s], (double)fb[s], acc4[s & 3], 0, 0, 0);
    }
    __syncthreads();
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) acc[v] = (acc4[0][v] + acc4[1][v]) + (acc4[2][v] + acc4[3][v]);
  return scratch;
}

// acc += B B^T for one 16 x 16 tile per wave, B as stored values in LDS [32][ldb] floats (rows >= r zero).
template <int D>
__device__ __forceinline__ void fs_bbt_tile(const float* __restrict__ Bs, int ldb, fs_v4d& acc) {
  const int lane = lane_id(), wave = wave_id();
  const int li = lane & 15, lk = lane >> 4, rt = wave >> 1, ct = wave & 1;
  const float* pa = Bs + (16 * rt + li) * ldb + lk;
  const float* pb = Bs + (16 * ct + li) * ldb + lk;
  fs_v4d a2[2] = {acc, fs_v4d{0.0, 0.0, 0.0, 0.0}};
#pragma unroll 8
  for (int k0 = 0; k0 < D; k0 += 8) {
    a2[0] = __builtin_amdgcn_mfma_f64_16x16x4f64((double)pa[k0], (double)pb[k0], a2[0], 0, 0, 0);
    a2[1] = __builtin_amdgcn_mfma_f64_16x16x4f64((double)pa[k0 + 4], (double)pb[k0 + 4], a2[1], 0, 0, 0);
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) acc[v] = a2[0][v] + a2[1][v];
}

// B (storage type, [r][D]) -> LDS [32][D + 1] floats, rows >= r zero.  16-byte loads, held in registers
// between request and store so that the caller can put other work between the two.
template <typename T, int D>
struct FsBRows {
  static constexpr int VEC = Vec16<T>::N;
  static constexpr int vpr = D / VEC;  // vectors per row
  static constexpr int NB = (32 * vpr + kQsThreads - 1) / kQsThreads;
  Vec16<T> v[NB];
  __device__ __forceinline__ void request(const T* __restrict__ B, int r) {
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      const int vi = min((int)threadIdx.x + u * kQsThreads, 32 * vpr - 1);
      v[u].load(B + (int64_t)min(vi / vpr, r - 1) * D + (vi % vpr) * VEC);
    }
  }
  __device__ __forceinline__ void store(int r, float* __restrict__ Bs) const {
    constexpr int ldb = D + 1;
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      const int vi = (int)threadIdx.x + u * kQsThreads;
      if (vi < 32 * vpr) {
        const int row = vi / vpr, c0 = (vi % vpr) * VEC;
        float f[VEC];
        v[u].unpack(f);
#pragma unroll
        for (int e = 0; e < VEC; ++e) Bs[row * ldb + c0 + e] = row < r ? f[e] : 0.0f;
      }
    }
  }
};

// Inverse of the symmetric positive definite matrix in Gs ([32][33] fp64 in LDS; rows and columns >= r count as an
// identity block), by ONE wave, as r symmetric sweeps on the fp64 matrix cores.  The wave holds the matrix as
// four 16 x 16 tiles in the accumulator layout of the 16 x 16 x 4 product (tile (rt, ct), element v of lane l:
// row 16 rt + (l >> 4) + 4 v, column 16 ct + (l & 15)).  A sweep on pivot p (d = a_pp) maps
//   a_ij -> a_ij - a_ip a_pj / d,   a_ip -> a_ip / d,   a_pj -> a_pj / d,   a_pp -> -1 / d
// and leaves -G^-1 after all p.  All four cases are one update acc -= A B of depth 2: the lanes that hold row p
// (one group of 16 lanes, one register, per tile column -- by symmetry also column p) supply A_i = a_pi / d,
// B_j = a_pj, except A_p = 1 - 1/d and B_p = d - 1; the next group of lanes supplies 2 and 1 at p, which takes the
// remaining 2 off the pivot.  B_p = d - 1 cancels for large d, so the matrix is scaled to unit diagonal first
// (every pivot is then <= 1) and the scaling is undone on the way out.  out: [32][32] in global memory.
__device__ __forceinline__ void fs_invert_wave(const double* __restrict__ Gs, int r, double* __restrict__ scl,
                                               double* __restrict__ out) {
  const int lane = lane_id();
  const int li = lane & 15, lk = lane >> 4;
  if (lane < 32) scl[lane] = lane < r ? 1.0 / sqrt(Gs[lane * 33 + lane]) : 1.0;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  fs_v4d t[2][2];
  double sc[2][2][4];
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int ct = 0; ct < 2; ++ct)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int i = 16 * rt + lk + 4 * v, j = 16 * ct + li;
        sc[rt][ct][v] = scl[i] * scl[j];
        const double x = Gs[i * 33 + j];
        t[rt][ct][v] = (i < r && j < r) ? x * sc[rt][ct][v] : (i == j ? 1.0 : 0.0);
      }
#pragma unroll
  for (int p = 0; p < 32; ++p) {
    if (p < r) {  // (wave-uniform)
      const int rtp = p >> 4, pp = p & 15, lkp = pp & 3, vp = pp >> 2, lk2 = (lkp + 1) & 3;
      const double s0 = t[rtp][0][vp], s1 = t[rtp][1][vp];  // row p, columns 0..15 / 16..31, in the lanes of group lkp
      const double d = bcast_f64(rtp ? s1 : s0, 16 * lkp + pp);
      const double rinv = recip_f64(d);
      const bool grp = lk == lkp, grp2 = lk == lk2, atp = li == pp;
      // operands per 16-row / 16-column half: h2 = 0, 1
      double Aop[2], Bop[2];
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const double src = h2 ? s1 : s0;
        const bool isp = atp && h2 == rtp;
        const double a_main = isp ? 1.0 - rinv : src * rinv;
        const double b_main = isp ? d - 1.0 : src;
        Aop[h2] = grp ? a_main : ((grp2 && isp) ? 2.0 : 0.0);
        Bop[h2] = grp ? b_main : ((grp2 && isp) ? 1.0 : 0.0);
      }
      // the tiles that hold the next pivot's row first: the next sweep's operands are then prepared while the
      // other two products are still in the matrix pipe
      const int rn = ((p + 1) >> 4) & 1;
#pragma unroll
      for (int o = 0; o < 2; ++o) {
        const int rt = o ? 1 - rn : rn;
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
          t[rt][ct] = __builtin_amdgcn_mfma_f64_16x16x4f64(-Aop[rt], Bop[ct], t[rt][ct], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int ct = 0; ct < 2; ++ct)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int i = 16 * rt + lk + 4 * v, j = 16 * ct + li;
        out[i * 32 + j] = (i < r && j < r) ? -t[rt][ct][v] * sc[rt][ct][v] : (i == j ? 1.0 : 0.0);
      }
}

// Workgroups x < D / 32 of a head: rows 32 x .. of M (and of N = B_Q^T + M).  x == D / 32: GA, then
// G_Q = B_Q B_Q^T + GA and its inverse.  x == D / 32 + 1: G_K = B_K B_K^T and its inverse.  Reads B_Q, B_K as the
// step's finish stage left them.
template <typename T, int D>
__global__ __launch_bounds__(kQsThreads) void als_state_tail_kernel(TailArgs ta) {
  extern __shared__ __align__(16) float fs_dynf[];
  float* Lb = fs_dynf;                      // [kFsTerms][kFsLdf]
  float* Ab = Lb + kFsTerms * kFsLdf;       // [kFsTerms][kFsLdf]
  float* Bs = Ab + kFsTerms * kFsLdf;       // [32][D + 1]
  double* Gs = reinterpret_cast<double*>(Bs + ((32 * (D + 1) + 3) & ~3));  // [32][33]
  double* scl = Gs + 32 * 33;               // [32]
  const int h = blockIdx.y, blk = blockIdx.x;
  const int lane = lane_id(), wave = wave_id();
  const int li = lane & 15, lk = lane >> 4, rt = wave >> 1, ct = wave & 1;
  const int r = ta.r;
  double* st = ta.state + (int64_t)h * fs_stride(D);
  double* N = st;
  double* GQi = st + (int64_t)D * 32;
  double* GKi = GQi + 1024;
  double* M = GKi + 1024;
  double* GA = M + (int64_t)D * 32;
  fs_v4d acc = fs_v4d{0.0, 0.0, 0.0, 0.0};
  if (blk < D / 32) {
    // (what the block's result is combined with is requested before the sums are formed)
    const T* bq = (const T*)ta.b_q + (int64_t)h * r * D;
    const int col = 16 * ct + li;
    float bv[4];
    double mo[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      bv[v] = ld_f32<T>(bq, (int64_t)min(col, r - 1) * D + 32 * blk + 16 * rt + lk + 4 * v);
      mo[v] = M[(32 * blk + 16 * rt + lk + 4 * v) * 32 + col];
    }
    const bool scratch = fs_block_sums<T, D>(ta, h, blk, Lb, Ab, acc, [] {});
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int idx = (32 * blk + 16 * rt + lk + 4 * v) * 32 + col;
      const double m = scratch ? acc[v] : mo[v] + acc[v];
      M[idx] = m;
      N[idx] = col < r ? m + (double)bv[v] : 0.0;
    }
    return;
  }
  const bool q_side = blk == D / 32;
  FsBRows<T, D> brows;
  brows.request((const T*)(q_side ? ta.b_q : ta.b_k) + (int64_t)h * r * D, r);
  fs_v4d bbt = fs_v4d{0.0, 0.0, 0.0, 0.0};
  // B B^T while the first pass's rows are on their way (the K side has nothing else to wait for)
  auto form_bbt = [&] {
    brows.store(r, Bs);
    __syncthreads();
    fs_bbt_tile<D>(Bs, D + 1, bbt);
  };
  if (q_side) {
    double go[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) go[v] = GA[(16 * rt + lk + 4 * v) * 32 + 16 * ct + li];
    const bool scratch = fs_block_sums<T, D>(ta, h, blk, Lb, Ab, acc, form_bbt);
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int idx = (16 * rt + lk + 4 * v) * 32 + 16 * ct + li;
      const double x = scratch ? acc[v] : go[v] + acc[v];
      GA[idx] = x;
      acc[v] = x;
    }
  } else {
    form_bbt();
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) Gs[(16 * rt + lk + 4 * v) * 33 + 16 * ct + li] = acc[v] + bbt[v];
  __syncthreads();
  if (wave == 0) fs_invert_wave(Gs, r, scl, q_side ? GQi : GKi);
}

// ----------------------------------------------------------------------------- host side
bool factor_state_supported(int r, int d, int dtype, int max_iter) {
  (void)dtype;
  return r >= 1 && r <= kAlsMaxR && (d == 32 || d == 64 || d == 128 || d == 256) && max_iter <= 8;
}

template <typename T, int D>
static int fs_launch_tail_d(const TailArgs& ta, int bh, hipStream_t st) {
  const size_t smem = ((size_t)2 * kFsTerms * kFsLdf + ((32 * (D + 1) + 3) & ~3)) * sizeof(float) +
                      ((size_t)32 * 33 + 32) * sizeof(double);
  static std::atomic<bool> attr_dev[kMaxDeviceSlots];
  std::atomic<bool>& attr = attr_dev[per_device_slot()];
  if (!attr) {
    LRQK_HIP_CHECK(hipFuncSetAttribute((const void*)als_state_tail_kernel<T, D>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    attr = true;
  }
  hipLaunchKernelGGL((als_state_tail_kernel<T, D>), dim3((unsigned)(D / 32 + 2), (unsigned)bh), dim3(kQsThreads), smem, st,
                     ta);
  LRQK_HIP_CHECK(hipGetLastError());
  return LRQK_OK;
}

template <typename T>
static int fs_launch_tail(const TailArgs& ta, int bh, int d, hipStream_t st) {
  switch (d) {
    case 32: return fs_launch_tail_d<T, 32>(ta, bh, st);
    case 64: return fs_launch_tail_d<T, 64>(ta, bh, st);
    case 128: return fs_launch_tail_d<T, 128>(ta, bh, st);
    default: return fs_launch_tail_d<T, 256>(ta, bh, st);
  }
}

static TailArgs fs_tail_args(lrqk_ctx* ctx, const void* b_q, const void* b_k, const void* a_k, int64_t head_stride,
                             const int32_t* active_idx, int64_t idx_stride, const void* k_act, int n_slots, int r,
                             int topk) {
  TailArgs ta{};
  ta.state = (double*)ctx->fstate.p;
  ta.a_k = a_k;
  ta.head_stride = head_stride;
  ta.a_rows = head_stride / r;
  ta.active_idx = active_idx;
  ta.idx_stride = idx_stride;
  ta.k_act = k_act;
  ta.n_slots = n_slots;
  ta.evk = k_act;  // (a valid address for the clamped loads when nothing was kept)
  ta.evk_rows = 1;
  ta.k = topk;
  ta.ring_slot = -1;
  ta.r = r;
  ta.b_q = b_q;
  ta.b_k = b_k;
  return ta;
}

// State from scratch for the view of a step whose new token goes to slot `skip_slot`.
int factor_state_rebuild(lrqk_ctx* ctx, const void* b_q, const void* b_k, const void* a_k, int64_t head_stride,
                         const int32_t* active_idx, int64_t idx_stride, const void* k_act, int n_slots, int bh, int r,
                         int d, int topk, int skip_slot, int dtype, hipStream_t st) {
  int rc = ctx->fstate.ensure((size_t)bh * fs_stride(d) * sizeof(double));
  if (rc) return rc;
  TailArgs ta = fs_tail_args(ctx, b_q, b_k, a_k, head_stride, active_idx, idx_stride, k_act, n_slots, r, topk);
  ta.skip_slot = skip_slot;
  ta.rebuild = 1;
  if (dtype == LRQK_F32) return fs_launch_tail<float>(ta, bh, d, st);
  return fs_launch_tail<bf16_t>(ta, bh, d, st);
}

// After a step's fetch and finish stage: the sums follow the rows that the step replaced, then the inverses.
int factor_state_advance(lrqk_ctx* ctx, const void* b_q, const void* b_k, const void* a_k, int64_t head_stride,
                         const int32_t* active_idx, int64_t idx_stride, const void* k_act, int n_slots,
                         const int32_t* miss_slots, const int32_t* miss_old, const int32_t* miss_new,
                         const int32_t* miss_count, int64_t cap, int bh, int r, int d, int topk, int ring_slot,
                         int32_t ring_token, int skip_slot, int dtype, hipStream_t st) {
  TailArgs ta = fs_tail_args(ctx, b_q, b_k, a_k, head_stride, active_idx, idx_stride, k_act, n_slots, r, topk);
  ta.evk = ctx->evk.p;
  ta.evk_rows = ctx->evk_rows;
  ta.miss_slots = miss_slots;
  ta.miss_old = miss_old;
  ta.miss_new = miss_new;
  ta.miss_count = miss_count;
  ta.cap = cap;
  ta.ring_slot = ring_slot;
  ta.ring_token = ring_token;
  ta.skip_slot = skip_slot;
  ta.rebuild = 0;
  if (dtype == LRQK_F32) return fs_launch_tail<float>(ta, bh, d, st);
  return fs_launch_tail<bf16_t>(ta, bh, d, st);
}

template <typename T, int D>
static void fs_launch_quick(lrqk_ctx* ctx, void* b_k, int32_t* active_idx, int64_t idx_stride, void* k_act, void* v_act,
                            int n_slots, const void* q, const void* k_new, const void* v_new, int bh, int hq, int hkv,
                            int r, int max_iter, int slot, int32_t token, float* iter_out, float* deltas, hipStream_t st) {
  hipLaunchKernelGGL((als_quick_kernel<T, D>), dim3((unsigned)bh), dim3(kQsThreads), 0, st, (const double*)ctx->fstate.p,
                     (const T*)q, (const T*)k_new, (const T*)v_new, (T*)k_act, (T*)v_act, n_slots, active_idx, idx_stride,
                     slot, token, (const T*)b_k, hq, hkv, r, max_iter, iter_out, deltas, (double*)ctx->als_iter64.p);
}

// The step's own launch: ring append + iterations; the finish stage is left pending (the scan reads the
// iterates, the fetch launch carries the finish).
int factor_state_quick(lrqk_ctx* ctx, void* b_q, void* b_k, void* a_k, int64_t head_stride, int32_t* active_idx,
                       int64_t idx_stride, void* k_act, void* v_act, int n_slots, const void* q, const void* k_new,
                       const void* v_new, int b, int hq, int hkv, int r, int d, int max_iter, float tol, void* q_hat,
                       void* k_hat, int64_t append_row, int slot, int32_t token, int dtype, hipStream_t st) {
  const int bh = b * hq;
  if (max_iter < 1) max_iter = 1;
  LRQK_REQUIRE(slot >= 0 && slot < n_slots, LRQK_EINVAL, "slot=%d outside 0..%d", slot, n_slots);
  LRQK_REQUIRE(((uintptr_t)k_new % 16 == 0) && ((uintptr_t)v_new % 16 == 0) && ((uintptr_t)v_act % 16 == 0) &&
                   ((uintptr_t)k_act % 16 == 0) && ((uintptr_t)q % 16 == 0),
               LRQK_EINVAL, "pointers must be 16-byte aligned");
  LRQK_REQUIRE(((uintptr_t)b_q % 16 == 0) && ((uintptr_t)b_k % 16 == 0) && ((int64_t)r * d * (int64_t)elem_size(dtype)) % 16 == 0,
               LRQK_EINVAL, "b_q/b_k must be 16-byte aligned");
  LRQK_REQUIRE(append_row < head_stride / r, LRQK_EINVAL, "append_row beyond the A_K capacity");
  int rc = ctx->als_iter.ensure((size_t)bh * max_iter * (2 * r + 1) * sizeof(float));
  if (rc) return rc;
  if ((rc = ctx->als_iter64.ensure((size_t)bh * max_iter * 2 * r * sizeof(double)))) return rc;
  float* iter_out = (float*)ctx->als_iter.p;
  float* deltas = iter_out + (size_t)bh * max_iter * 2 * r;
  ctx->iter64_bh = bh;
  ctx->iter64_r = r;
  ctx->iter64_iters = max_iter;
  ctx->iter64_token = token;
#define LRQK_QUICK_CASE(TT, DD)                                                                                       \
  fs_launch_quick<TT, DD>(ctx, b_k, active_idx, idx_stride, k_act, v_act, n_slots, q, k_new, v_new, bh, hq, hkv, r,     \
                          max_iter, slot, token, iter_out, deltas, st)
  if (dtype == LRQK_F32) {
    switch (d) {
      case 32: LRQK_QUICK_CASE(float, 32); break;
      case 64: LRQK_QUICK_CASE(float, 64); break;
      case 128: LRQK_QUICK_CASE(float, 128); break;
      default: LRQK_QUICK_CASE(float, 256); break;
    }
  } else {
    switch (d) {
      case 32: LRQK_QUICK_CASE(bf16_t, 32); break;
      case 64: LRQK_QUICK_CASE(bf16_t, 64); break;
      case 128: LRQK_QUICK_CASE(bf16_t, 128); break;
      default: LRQK_QUICK_CASE(bf16_t, 256); break;
    }
  }
#undef LRQK_QUICK_CASE
  LRQK_HIP_CHECK(hipGetLastError());
  return als_defer_finish(ctx, b_q, b_k, a_k, head_stride, q, k_new, bh, hq, hkv, r, d, max_iter, tol, q_hat, k_hat,
                          append_row, iter_out, deltas, dtype);
}

}  // namespace lrqk

using namespace lrqk;

extern "C" int lrqk_ctx_factor_state(lrqk_ctx* ctx, int enable) {
  LRQK_REQUIRE(ctx != nullptr, LRQK_EINVAL, "ctx is null");
  ctx->fs_enabled = enable != 0;
  ctx->fs_valid = false;
  return LRQK_OK;
}

extern "C" int lrqk_last_iterates(lrqk_ctx* ctx, double* out, int64_t n_doubles, int* bh, int* max_iter, int* r,
                                  int64_t* token) {
  LRQK_REQUIRE(ctx && bh && max_iter && r && token, LRQK_EINVAL, "null pointer");
  *token = ctx->iter64_token;
  *bh = ctx->iter64_bh;
  *max_iter = ctx->iter64_iters;
  *r = ctx->iter64_r;
  const int64_t need = (int64_t)ctx->iter64_bh * ctx->iter64_iters * 2 * ctx->iter64_r;
  if (!out || need == 0) return LRQK_OK;
  LRQK_REQUIRE(n_doubles >= need, LRQK_EINVAL, "out holds %lld doubles, %lld needed", (long long)n_doubles, (long long)need);
  LRQK_HIP_CHECK(hipDeviceSynchronize());
  LRQK_HIP_CHECK(hipMemcpy(out, ctx->als_iter64.p, (size_t)need * sizeof(double), hipMemcpyDeviceToHost));
  return LRQK_OK;
}
