// Plain streaming kernels of known size: a read of `bytes` and a copy of `bytes`, timed with HIP events on
// the caller's stream.  They measure what the memory system of the GPU at hand delivers, next to which the
// rates of the scan kernels can be read, and give hardware counters a transfer of known size to be scaled by.
#include "common.hpp"

namespace lrqk {

constexpr int kProbeThreads = 256;
constexpr int kProbeUnroll = 4;

// Every thread reads 16-byte vectors, kProbeUnroll in flight, grid-stride.  The folded value is stored only if
// it equals a value that it never takes in practice, which keeps the loads alive without write traffic.
__global__ __launch_bounds__(kProbeThreads) void probe_read_kernel(const uint4* __restrict__ src, int64_t n_vec,
                                                                   uint32_t* __restrict__ sink) {
  const int64_t stride = (int64_t)gridDim.x * kProbeThreads;
  uint32_t acc = 0;
  for (int64_t i = (int64_t)blockIdx.x * kProbeThreads + threadIdx.x; i < n_vec; i += stride * kProbeUnroll) {
    uint4 v[kProbeUnroll];
#pragma unroll
    for (int u = 0; u < kProbeUnroll; ++u) v[u] = src[min(i + u * stride, n_vec - 1)];
#pragma unroll
    for (int u = 0; u < kProbeUnroll; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  if (acc == 0x9e3779b9u && threadIdx.x == 1023) sink[blockIdx.x] = acc;
}

// The same read with U vectors in flight per thread, plain or non-temporal loads: the variants of the sweep that
// looks for the best read rate the GPU at hand delivers to a streaming kernel.
template <int U, bool NT>
__global__ __launch_bounds__(kProbeThreads) void probe_read_variant_kernel(const uint4* __restrict__ src, int64_t n_vec,
                                                                           uint32_t* __restrict__ sink) {
  const int64_t stride = (int64_t)gridDim.x * kProbeThreads;
  uint32_t acc = 0;
  for (int64_t i = (int64_t)blockIdx.x * kProbeThreads + threadIdx.x; i < n_vec; i += stride * U) {
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint4* p = src + min(i + u * stride, n_vec - 1);
      if constexpr (NT) {
        const uint32_t* w = reinterpret_cast<const uint32_t*>(p);
        v[u] = make_uint4(__builtin_nontemporal_load(w), __builtin_nontemporal_load(w + 1),
                          __builtin_nontemporal_load(w + 2), __builtin_nontemporal_load(w + 3));
      } else {
        v[u] = *p;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  if (acc == 0x9e3779b9u && threadIdx.x == 1023) sink[blockIdx.x] = acc;
}

__global__ __launch_bounds__(kProbeThreads) void probe_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                                   int64_t n_vec) {
  const int64_t stride = (int64_t)gridDim.x * kProbeThreads;
  for (int64_t i = (int64_t)blockIdx.x * kProbeThreads + threadIdx.x; i < n_vec; i += stride * kProbeUnroll) {
    uint4 v[kProbeUnroll];
#pragma unroll
    for (int u = 0; u < kProbeUnroll; ++u) v[u] = src[min(i + u * stride, n_vec - 1)];
#pragma unroll
    for (int u = 0; u < kProbeUnroll; ++u)
      if (i + u * stride < n_vec) dst[i + u * stride] = v[u];
  }
}

// Does nothing: what a pair of events around a launch reads when the kernel itself takes no time.
__global__ void probe_empty_kernel() {}

}  // namespace lrqk

using namespace lrqk;

extern "C" int lrqk_probe_event_pair(int reps, int kernels, double* pair_us, void* stream) {
  LRQK_REQUIRE(pair_us != nullptr && reps > 0 && reps <= 256 && kernels >= 1 && kernels <= 16, LRQK_EINVAL,
               "bad arguments reps=%d kernels=%d", reps, kernels);
  hipStream_t st = (hipStream_t)stream;
  hipEvent_t* ev = new hipEvent_t[2 * (size_t)reps];
  int made = 0, rc = LRQK_OK;
  for (; made < 2 * reps; ++made) {
    if (hipEventCreate(&ev[made]) != hipSuccess) {
      rc = LRQK_EHIP;
      break;
    }
  }
  double sum = 0.0;
  if (rc == LRQK_OK) {
    // as in the timed step: a kernel before the pair, the bracketed launch, a kernel after it
    for (int i = 0; i < reps && rc == LRQK_OK; ++i) {
      hipLaunchKernelGGL(probe_empty_kernel, dim3(1), dim3(64), 0, st);
      if (hipEventRecord(ev[2 * i], st) != hipSuccess) rc = LRQK_EHIP;
      for (int k = 0; k < kernels; ++k) hipLaunchKernelGGL(probe_empty_kernel, dim3(1), dim3(64), 0, st);
      if (hipEventRecord(ev[2 * i + 1], st) != hipSuccess) rc = LRQK_EHIP;
      hipLaunchKernelGGL(probe_empty_kernel, dim3(1), dim3(64), 0, st);
    }
    if (rc == LRQK_OK && hipStreamSynchronize(st) != hipSuccess) rc = LRQK_EHIP;
    for (int i = 0; i < reps && rc == LRQK_OK; ++i) {
      float ms = 0.0f;
      if (hipEventElapsedTime(&ms, ev[2 * i], ev[2 * i + 1]) != hipSuccess) rc = LRQK_EHIP;
      sum += ms;
    }
  }
  for (int i = 0; i < made; ++i) (void)hipEventDestroy(ev[i]);
  delete[] ev;
  (void)hipGetLastError();
  LRQK_REQUIRE(rc == LRQK_OK, LRQK_EHIP, "HIP event calls failed");
  *pair_us = sum * 1e3 / reps;
  return LRQK_OK;
}

extern "C" int lrqk_probe_bandwidth(const void* src, void* dst, int64_t bytes, int reps, double* read_ms,
                                    double* copy_ms, void* stream) {
  LRQK_REQUIRE(src && dst && read_ms && copy_ms, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(bytes >= 16 && bytes % 16 == 0 && reps > 0 && reps <= 1000, LRQK_EINVAL, "bad sizes bytes=%lld reps=%d",
               (long long)bytes, reps);
  LRQK_REQUIRE(((uintptr_t)src % 16 == 0) && ((uintptr_t)dst % 16 == 0), LRQK_EINVAL, "pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  int dev = 0, n_cu = 0;
  LRQK_HIP_CHECK(hipGetDevice(&dev));
  LRQK_HIP_CHECK(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev));
  const int64_t n_vec = bytes / 16;
  const unsigned grid = (unsigned)std::max<int64_t>(1, std::min<int64_t>((int64_t)n_cu * 8, (n_vec + kProbeThreads - 1) / kProbeThreads));
  hipEvent_t ev[3];
  for (auto& e : ev) LRQK_HIP_CHECK(hipEventCreate(&e));
  // one untimed pass of each, then `reps` timed ones
  hipLaunchKernelGGL(probe_read_kernel, dim3(grid), dim3(kProbeThreads), 0, st, (const uint4*)src, n_vec, (uint32_t*)dst);
  hipLaunchKernelGGL(probe_copy_kernel, dim3(grid), dim3(kProbeThreads), 0, st, (const uint4*)src, (uint4*)dst, n_vec);
  LRQK_HIP_CHECK(hipEventRecord(ev[0], st));
  for (int i = 0; i < reps; ++i)
    hipLaunchKernelGGL(probe_read_kernel, dim3(grid), dim3(kProbeThreads), 0, st, (const uint4*)src, n_vec, (uint32_t*)dst);
  LRQK_HIP_CHECK(hipEventRecord(ev[1], st));
  for (int i = 0; i < reps; ++i)
    hipLaunchKernelGGL(probe_copy_kernel, dim3(grid), dim3(kProbeThreads), 0, st, (const uint4*)src, (uint4*)dst, n_vec);
  LRQK_HIP_CHECK(hipEventRecord(ev[2], st));
  LRQK_HIP_CHECK(hipGetLastError());
  LRQK_HIP_CHECK(hipEventSynchronize(ev[2]));
  float a = 0.0f, b = 0.0f;
  LRQK_HIP_CHECK(hipEventElapsedTime(&a, ev[0], ev[1]));
  LRQK_HIP_CHECK(hipEventElapsedTime(&b, ev[1], ev[2]));
  for (auto& e : ev) (void)hipEventDestroy(e);
  *read_ms = a / reps;
  *copy_ms = b / reps;
  return LRQK_OK;
}

extern "C" int lrqk_probe_read_variant(const void* src, void* sink, int64_t bytes, int64_t slice_bytes, int reps,
                                       int in_flight, int nontemporal, int grid_per_cu, double* read_ms, void* stream) {
  LRQK_REQUIRE(src && sink && read_ms, LRQK_EINVAL, "null pointer");
  LRQK_REQUIRE(bytes >= 16 && bytes % 16 == 0 && reps > 0 && reps <= 1000, LRQK_EINVAL, "bad sizes bytes=%lld reps=%d",
               (long long)bytes, reps);
  LRQK_REQUIRE(slice_bytes == 0 || (slice_bytes >= 16 && slice_bytes % 16 == 0 && slice_bytes <= bytes), LRQK_EINVAL,
               "slice_bytes=%lld not a multiple of 16 within the buffer", (long long)slice_bytes);
  LRQK_REQUIRE((in_flight == 4 || in_flight == 8 || in_flight == 16) && grid_per_cu >= 1 && grid_per_cu <= 64, LRQK_EINVAL,
               "in_flight=%d (4, 8 or 16), grid_per_cu=%d (1..64)", in_flight, grid_per_cu);
  LRQK_REQUIRE((uintptr_t)src % 16 == 0, LRQK_EINVAL, "src must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  int dev = 0, n_cu = 0;
  LRQK_HIP_CHECK(hipGetDevice(&dev));
  LRQK_HIP_CHECK(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev));
  // a launch reads the whole buffer, or (slice_bytes > 0) one slice of it, the launches taking the slices in turn
  const int64_t n_vec = (slice_bytes ? slice_bytes : bytes) / 16;
  const int64_t n_slices = slice_bytes ? bytes / slice_bytes : 1;
  int64_t turn = 0;
  const unsigned grid = (unsigned)std::max<int64_t>(1, std::min<int64_t>((int64_t)n_cu * grid_per_cu,
                                                                        (n_vec + kProbeThreads - 1) / kProbeThreads));
  auto launch = [&]() {
    const uint4* from = (const uint4*)src + (turn++ % n_slices) * n_vec;
#define LRQK_PROBE_CASE(UU, NTT)                                                                           \
  hipLaunchKernelGGL((probe_read_variant_kernel<UU, NTT>), dim3(grid), dim3(kProbeThreads), 0, st, from, n_vec, \
                     (uint32_t*)sink)
    if (nontemporal) {
      if (in_flight == 4) LRQK_PROBE_CASE(4, true);
      else if (in_flight == 8) LRQK_PROBE_CASE(8, true);
      else LRQK_PROBE_CASE(16, true);
    } else {
      if (in_flight == 4) LRQK_PROBE_CASE(4, false);
      else if (in_flight == 8) LRQK_PROBE_CASE(8, false);
      else LRQK_PROBE_CASE(16, false);
    }
#undef LRQK_PROBE_CASE
  };
  hipEvent_t ev[2];
  for (auto& e : ev) LRQK_HIP_CHECK(hipEventCreate(&e));
  launch();  // untimed
  LRQK_HIP_CHECK(hipEventRecord(ev[0], st));
  for (int i = 0; i < reps; ++i) launch();
  LRQK_HIP_CHECK(hipEventRecord(ev[1], st));
  LRQK_HIP_CHECK(hipGetLastError());
  LRQK_HIP_CHECK(hipEventSynchronize(ev[1]));
  float a = 0.0f;
  LRQK_HIP_CHECK(hipEventElapsedTime(&a, ev[0], ev[1]));
  for (auto& e : ev) (void)hipEventDestroy(e);
  *read_ms = a / reps;
  return LRQK_OK;
}
