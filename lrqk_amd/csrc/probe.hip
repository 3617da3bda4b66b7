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

}  // namespace lrqk

using namespace lrqk;

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
