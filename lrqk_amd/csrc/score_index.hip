// Host side of the score index (8-bit copy of the A_K rows used by the scan): binding to an A_K
// buffer, building / extending it, and the quantisation kernel.
#include <algorithm>

#include "common.hpp"
#include "ctx.hpp"

namespace lrqk {

// W of one head from a strided sample of at most kSidxSample of the rows [0, rows): second-moment
// matrix S of the sample (plus a small ridge), Cholesky factor S = L L^T, W = L^-T.  Two launches:
// kSidxParts workgroups per head sum their share of the sample (fixed order: reproducible), then
// one workgroup per head adds the parts and factors.  Anything degenerate (no rows, zero or
// non-finite S, a non-positive pivot) gives W = I.
constexpr int kSidxSample = 4096;
constexpr int kSidxTile = 64;   // sample rows per LDS tile
constexpr int kSidxParts = 16;  // workgroups per head in the first launch
template <typename T, int R>
__global__ __launch_bounds__(256) void score_index_moments_kernel(const T* __restrict__ a_k, int64_t head_stride,
                                                                  int64_t rows, float* __restrict__ part) {
  constexpr int LD = R + 1;
  constexpr int EPT = (R * R + 255) / 256;  // entries of S per thread
  __shared__ float tile[kSidxTile][LD];
  const int h = blockIdx.y, p = blockIdx.x, tid = threadIdx.x;
  const T* A = a_k + (int64_t)h * head_stride;
  const int64_t step = rows > 0 ? (rows + kSidxSample - 1) / kSidxSample : 1;
  const int64_t n = rows > 0 ? (rows + step - 1) / step : 0;  // sample size
  const int64_t per = (n + kSidxParts - 1) / kSidxParts;
  const int64_t n0 = min(n, p * per), n1 = min(n, n0 + per);
  float acc[EPT];
#pragma unroll
  for (int e = 0; e < EPT; ++e) acc[e] = 0.0f;
  for (int64_t t0 = n0; t0 < n1; t0 += kSidxTile) {
    const int cnt = (int)min((int64_t)kSidxTile, n1 - t0);
    __syncthreads();
    for (int x = tid; x < kSidxTile * R; x += 256) {
      const int rr = x / R, c = x % R;
      tile[rr][c] = rr < cnt ? ld_f32<T>(A, (t0 + rr) * step * R + c) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int x = tid + e * 256;
      if (x < R * R) {
        const int i = x / R, j = x % R;
        float sum = acc[e];
        for (int rr = 0; rr < kSidxTile; ++rr) sum = fmaf(tile[rr][i], tile[rr][j], sum);
        acc[e] = sum;
      }
    }
  }
  float* out = part + ((int64_t)h * kSidxParts + p) * R * R;
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int x = tid + e * 256;
    if (x < R * R) out[x] = acc[e];
  }
}

template <int R>
__global__ __launch_bounds__(256) void score_index_factor_kernel(const float* __restrict__ part, int64_t rows,
                                                                 float* __restrict__ wm) {
  constexpr int LD = R + 1;
  __shared__ float S[R][LD];
  __shared__ float X[R][LD];
  __shared__ int bad;
  const int h = blockIdx.x, tid = threadIdx.x;
  float* W = wm + (int64_t)h * (R * R + R);
  const int64_t step = rows > 0 ? (rows + kSidxSample - 1) / kSidxSample : 1;
  const int64_t n = rows > 0 ? (rows + step - 1) / step : 0;
  if (tid == 0) bad = 0;
  for (int x = tid; x < R * R; x += 256) {
    float sum = 0.0f;
    for (int p = 0; p < kSidxParts; ++p) sum += part[((int64_t)h * kSidxParts + p) * R * R + x];
    S[x / R][x % R] = n > 0 ? sum / (float)n : 0.0f;
  }
  __syncthreads();
  float tr = 0.0f;
  for (int i = 0; i < R; ++i) tr += S[i][i];
  // (1 % of the mean diagonal: directions that hold next to nothing are not blown up to unit size, where their
  // quantisation step would only add slack to the bound; 12 % fewer rows to rescore than with 0.01 % on the 128K stream)
  const float ridge = 1e-2f * tr / (float)R;
  if (!(tr > 0.0f && tr < INFINITY) && tid == 0) bad = 1;
  __syncthreads();
  if (tid < R) S[tid][tid] += ridge;
  // Cholesky, column by column (lower triangle of S becomes L)
  for (int c = 0; c < R; ++c) {
    __syncthreads();
    const float piv = S[c][c];
    if (!(piv > 0.0f && piv < INFINITY)) {
      if (tid == 0) bad = 1;
      break;  // uniform: every thread reads the same pivot
    }
    const float d = sqrtf(piv);
    __syncthreads();
    if (tid == 0) S[c][c] = d;
    if (tid > c && tid < R) S[tid][c] /= d;
    __syncthreads();
    for (int x = tid; x < R * R; x += 256) {
      const int i = x / R, j = x % R;
      if (j > c && i >= j) S[i][j] -= S[i][c] * S[j][c];
    }
  }
  __syncthreads();
  // X = L^-1 by forward substitution, one column per thread
  if (!bad && tid < R) {
    const int c = tid;
    for (int i = 0; i < R; ++i) X[i][c] = 0.0f;
    X[c][c] = 1.0f / S[c][c];
    for (int i = c + 1; i < R; ++i) {
      float sum = 0.0f;
      for (int k = c; k < i; ++k) sum = fmaf(S[i][k], X[k][c], sum);
      X[i][c] = -sum / S[i][i];
    }
    for (int i = c; i < R; ++i)
      if (!(fabsf(X[i][c]) < INFINITY)) bad = 1;
    if (!(X[c][c] > 0.0f)) bad = 1;
  }
  __syncthreads();
  const bool ident = bad != 0;
  // W[i][j] = X[j][i] for i <= j, zero below the diagonal; then 1 / W_jj
  for (int x = tid; x < R * R; x += 256) {
    const int i = x / R, j = x % R;
    W[x] = ident ? (i == j ? 1.0f : 0.0f) : (i <= j ? X[j][i] : 0.0f);
  }
  if (tid < R) W[R * R + tid] = ident ? 1.0f : 1.0f / X[tid][tid];
}

// One wave per row: lane i holds element i of the row, and column `lane` of W stays in registers.
template <typename T, int R>
__global__ __launch_bounds__(256) void score_index_build_kernel(const T* __restrict__ a_k, int64_t head_stride,
                                                                int64_t row0, int64_t row1, uint8_t* __restrict__ qa,
                                                                uint16_t* __restrict__ qs, const float* __restrict__ wm,
                                                                int64_t head_rows) {
  const int h = blockIdx.y;
  const int lane = lane_id();
  const int64_t wave0 = (int64_t)blockIdx.x * (blockDim.x / kWave) + wave_id();
  const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x / kWave);
  float wcol[R];
  score_index_load_wcol<R>(wm + (int64_t)h * (R * R + R), lane, wcol);
  for (int64_t row = row0 + wave0; row < row1; row += nwaves) {
    const float v = lane < R ? ld_f32<T>(a_k, (int64_t)h * head_stride + row * R + lane) : 0.0f;
    float scale;
    const uint8_t u = score_index_encode_row<R>(v, wcol, &scale);
    if (lane < R) qa[((int64_t)h * head_rows + row) * R + lane] = u;
    if (lane == 0) qs[(int64_t)h * head_rows + row] = sidx_scale_bits(scale);
  }
}

// r = 32: the transform of 32 rows is one 32x32x32 product on the fp32 matrix pipe (16 steps of
// mfma 32x32x2), and a second one on absolute values gives g.  Lane (m, kh) = (lane & 31, lane >> 5)
// feeds A[m][2 kk + kh] (row m of the group) and B[2 kk + kh][m] (W); it receives, for v = 0..15,
// C[row(v)][m] with row(v) = (v / 4) * 8 + kh * 4 + v % 4.  Any summation order inside the pipe
// stays within the rounding bound the scale charges for.
typedef float sidx_v16f __attribute__((ext_vector_type(16)));
template <typename T>
__global__ __launch_bounds__(256) void score_index_build32_kernel(const T* __restrict__ a_k, int64_t head_stride,
                                                                  int64_t row0, int64_t row1, uint8_t* __restrict__ qa,
                                                                  uint16_t* __restrict__ qs, const float* __restrict__ wm,
                                                                  int64_t head_rows) {
  constexpr int R = 32, VEC = Vec16<T>::N;
  const int h = blockIdx.y;
  const int lane = lane_id(), m = lane & 31, kh = lane >> 5;
  const int64_t ngroups = (row1 - row0 + 31) / 32;
  const int64_t wave0 = (int64_t)blockIdx.x * (blockDim.x / kWave) + wave_id();
  const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x / kWave);
  const T* A = a_k + (int64_t)h * head_stride;
  const float* W = wm + (int64_t)h * (R * R + R);
  float wb[16], wba[16];
#pragma unroll
  for (int kk = 0; kk < 16; ++kk) {
    wb[kk] = W[(2 * kk + kh) * R + m];
    wba[kk] = fabsf(wb[kk]);
  }
  for (int64_t grp = wave0; grp < ngroups; grp += nwaves) {
    const int64_t r0 = row0 + grp * 32;
    const int64_t row = min(r0 + m, row1 - 1);
    float f[R];
    {
      Vec16<T> v[R / VEC];
#pragma unroll
      for (int c = 0; c < R / VEC; ++c) v[c].load(A + row * R + c * VEC);
#pragma unroll
      for (int c = 0; c < R / VEC; ++c) v[c].unpack(f + c * VEC);
    }
    sidx_v16f acc, accg;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = accg[v] = 0.0f;
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      const float a = kh ? f[2 * kk + 1] : f[2 * kk];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, wb[kk], acc, 0, 0, 0);
      accg = __builtin_amdgcn_mfma_f32_32x32x2f32(fabsf(a), wba[kk], accg, 0, 0, 0);
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      // maxima over the 32 columns of this half-wave's row
      float mx = row_reduce(fabsf(acc[v]), [](float x, float y) { return fmaxf(x, y); });
      float gx = row_reduce(accg[v], [](float x, float y) { return fmaxf(x, y); });
      mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
      gx = fmaxf(gx, __shfl_xor(gx, 16, kWave));
      const unsigned long long okm = __ballot(accg[v] < INFINITY);  // false for NaN and infinity
      const bool ok = (uint32_t)(kh ? okm >> 32 : okm) == 0xffffffffu;
      const float scale = score_index_scale(mx, ok ? gx : INFINITY, R);
      const uint8_t u = score_index_code(acc[v], 1.0f / scale);
      const int64_t orow = r0 + (v >> 2) * 8 + kh * 4 + (v & 3);
      if (orow < row1) {
        qa[((int64_t)h * head_rows + orow) * R + m] = u;
        if (m == 0) qs[(int64_t)h * head_rows + orow] = sidx_scale_bits(scale);
      }
    }
  }
}

template <typename T, int R>
static void launch_build(lrqk_ctx* ctx, const void* a_k, int64_t head_stride, int bh, int64_t from, int64_t upto,
                         int64_t head_rows, hipStream_t st) {
  float* wm = (float*)ctx->sidx_wm.p;
  if (from == 0) {  // first rows of this binding: they set W
    float* part = (float*)ctx->sidx_part.p;
    hipLaunchKernelGGL((score_index_moments_kernel<T, R>), dim3(kSidxParts, (unsigned)bh), dim3(256), 0, st,
                       (const T*)a_k, head_stride, upto, part);
    hipLaunchKernelGGL((score_index_factor_kernel<R>), dim3((unsigned)bh), dim3(256), 0, st, (const float*)part, upto, wm);
  }
  if (R == 32 && upto - from >= 32) {
    const unsigned blocks = (unsigned)std::min<int64_t>(1024, (upto - from + 127) / 128);
    hipLaunchKernelGGL((score_index_build32_kernel<T>), dim3(blocks, (unsigned)bh), dim3(256), 0, st, (const T*)a_k,
                       head_stride, from, upto, (uint8_t*)ctx->sidx_qa.p, (uint16_t*)ctx->sidx_qs.p, wm, head_rows);
    return;
  }
  const unsigned blocks = (unsigned)std::min<int64_t>(2048, (upto - from + 3) / 4);
  hipLaunchKernelGGL((score_index_build_kernel<T, R>), dim3(blocks, (unsigned)bh), dim3(256), 0, st, (const T*)a_k,
                     head_stride, from, upto, (uint8_t*)ctx->sidx_qa.p, (uint16_t*)ctx->sidx_qs.p, wm, head_rows);
}

int score_index_prepare(lrqk_ctx* ctx, const void* a_k, int64_t head_stride, int bh, int64_t m, int r, int dtype,
                        hipStream_t st, ScoreIndexView* view) {
  if (!ctx->sidx_enabled) return 0;
  if (!(r == 16 || r == 32 || r == 64) || head_stride % r != 0 || ((uintptr_t)a_k % 16 != 0)) return 0;
  const int64_t head_rows = head_stride / r;
  if (m > head_rows) return 0;
  const bool bound = ctx->sidx_a_k == a_k && ctx->sidx_head_rows == head_rows && ctx->sidx_r == r &&
                     ctx->sidx_dtype == dtype && ctx->sidx_bh == bh;
  if (!bound) {
    int rc;
    if ((rc = ctx->sidx_qa.ensure((size_t)bh * head_rows * r))) return rc;
    if ((rc = ctx->sidx_qs.ensure((size_t)bh * head_rows * sizeof(uint16_t)))) return rc;
    if ((rc = ctx->sidx_wm.ensure((size_t)bh * (r * r + r) * sizeof(float)))) return rc;
    if ((rc = ctx->sidx_part.ensure((size_t)bh * kSidxParts * r * r * sizeof(float)))) return rc;
    ctx->sidx_a_k = a_k;
    ctx->sidx_head_rows = head_rows;
    ctx->sidx_r = r;
    ctx->sidx_dtype = dtype;
    ctx->sidx_bh = bh;
    ctx->sidx_valid = 0;
  }
  if (ctx->sidx_valid < m) {
    // index everything that is known to exist, so that the rows appended from now on stay contiguous
    const int64_t upto = std::min(head_rows, std::max(m, ctx->sidx_rows_hint));
    const int64_t from = ctx->sidx_valid;
#define LRQK_SIDX_BUILD(TT)                                                                   \
  (r == 16 ? launch_build<TT, 16>(ctx, a_k, head_stride, bh, from, upto, head_rows, st)       \
   : r == 32 ? launch_build<TT, 32>(ctx, a_k, head_stride, bh, from, upto, head_rows, st)     \
             : launch_build<TT, 64>(ctx, a_k, head_stride, bh, from, upto, head_rows, st))
    if (dtype == LRQK_F32)
      LRQK_SIDX_BUILD(float);
    else
      LRQK_SIDX_BUILD(bf16_t);
#undef LRQK_SIDX_BUILD
    LRQK_HIP_CHECK(hipGetLastError());
    ctx->sidx_valid = upto;
  }
  view->qa = (const uint8_t*)ctx->sidx_qa.p;
  view->qs = (const uint16_t*)ctx->sidx_qs.p;
  view->wm = (const float*)ctx->sidx_wm.p;
  view->head_rows = head_rows;
  return 1;
}

}  // namespace lrqk

using namespace lrqk;

extern "C" int lrqk_ctx_score_index(lrqk_ctx* ctx, int enable) {
  LRQK_REQUIRE(ctx != nullptr, LRQK_EINVAL, "ctx is null");
  ctx->sidx_enabled = enable != 0;
  ctx->sidx_a_k = nullptr;  // whatever was indexed is dropped; the next scan rebuilds what it needs
  ctx->sidx_valid = 0;
  ctx->sel_bh = 0;  // the bound a scan carries to the next one is in the units of the scan that made it
  return LRQK_OK;
}
