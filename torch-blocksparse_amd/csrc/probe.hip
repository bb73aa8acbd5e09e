// Streaming probes for the benchmark's calibration mode (not part of the operator library: built into its own small
// shared object, libbsp_probe.so, and loaded by `bench.py --calibrate` only).  Each probe moves a known number of
// bytes with 16-byte accesses in address order, grid-stride, which is the access pattern an ideal HBM-bound kernel
// would have; their rates are what the operator kernels' GB/s figures are compared with.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

namespace {
constexpr int kThreads = 256;

// Every lane keeps U independent 16-byte accesses in flight per round (a workgroup walks U * 4 KiB of consecutive
// addresses per round), as the operator kernels do with their prefetch rings.
constexpr int U = 8;

// mode 0: read only (the xor of everything read is written by one lane that can never exist, so that the loads stay)
__global__ void __launch_bounds__(kThreads) k_probe_read(const u32x4 *src, u32x4 *sink, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * kThreads * U;
  u32x4 acc = {0u, 0u, 0u, 0u};
  for (int64_t i = (int64_t)blockIdx.x * kThreads * U + threadIdx.x; i < n; i += stride) {
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) v[u] = src[i + u * kThreads < n ? i + u * kThreads : i];
#pragma unroll
    for (int u = 0; u < U; u++) acc ^= v[u];
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u && n < 0) sink[0] = acc;
}
// mode 1: write only
__global__ void __launch_bounds__(kThreads) k_probe_write(u32x4 *dst, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * kThreads * U;
  for (int64_t i = (int64_t)blockIdx.x * kThreads * U + threadIdx.x; i < n; i += stride) {
#pragma unroll
    for (int u = 0; u < U; u++)
      if (i + u * kThreads < n) dst[i + u * kThreads] = u32x4{(uint32_t)i, 1u, 2u, 3u};
  }
}
// mode 2: copy (1 read : 1 write); mode 3: in place (read, modify, write back); mode 4: 1 read : 2 writes
__global__ void __launch_bounds__(kThreads) k_probe_copy(const u32x4 *src, u32x4 *dst, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * kThreads * U;
  for (int64_t i = (int64_t)blockIdx.x * kThreads * U + threadIdx.x; i < n; i += stride) {
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) v[u] = src[i + u * kThreads < n ? i + u * kThreads : i];
#pragma unroll
    for (int u = 0; u < U; u++)
      if (i + u * kThreads < n) dst[i + u * kThreads] = v[u];
  }
}
__global__ void __launch_bounds__(kThreads) k_probe_inplace(u32x4 *buf, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * kThreads * U;
  for (int64_t i = (int64_t)blockIdx.x * kThreads * U + threadIdx.x; i < n; i += stride) {
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) v[u] = buf[i + u * kThreads < n ? i + u * kThreads : i];
#pragma unroll
    for (int u = 0; u < U; u++)
      if (i + u * kThreads < n) buf[i + u * kThreads] = v[u] + 1u;
  }
}
__global__ void __launch_bounds__(kThreads) k_probe_r1w2(const u32x4 *src, u32x4 *dst0, u32x4 *dst1, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * kThreads * U;
  for (int64_t i = (int64_t)blockIdx.x * kThreads * U + threadIdx.x; i < n; i += stride) {
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) v[u] = src[i + u * kThreads < n ? i + u * kThreads : i];
#pragma unroll
    for (int u = 0; u < U; u++)
      if (i + u * kThreads < n) { dst0[i + u * kThreads] = v[u]; dst1[i + u * kThreads] = v[u]; }
  }
}
}  // namespace

// bytes = size of each buffer (a multiple of 16).  Moves: mode 0 bytes, 1 bytes, 2 2*bytes, 3 2*bytes, 4 3*bytes.
// Returns 0, or -1 on a bad argument / failed launch.
extern "C" int bsp_probe_stream(int mode, void *a, void *b, void *c, int64_t bytes, int groups, void *stream) {
  if (!a || bytes <= 0 || bytes % 16 || groups <= 0) return -1;
  const int64_t n = bytes / 16;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)groups), wg(kThreads);
  switch (mode) {
    case 0: if (!b) return -1; hipLaunchKernelGGL(k_probe_read, grid, wg, 0, st, (const u32x4 *)a, (u32x4 *)b, n); break;
    case 1: hipLaunchKernelGGL(k_probe_write, grid, wg, 0, st, (u32x4 *)a, n); break;
    case 2: if (!b) return -1; hipLaunchKernelGGL(k_probe_copy, grid, wg, 0, st, (const u32x4 *)a, (u32x4 *)b, n); break;
    case 3: hipLaunchKernelGGL(k_probe_inplace, grid, wg, 0, st, (u32x4 *)a, n); break;
    case 4: if (!b || !c) return -1; hipLaunchKernelGGL(k_probe_r1w2, grid, wg, 0, st, (const u32x4 *)a, (u32x4 *)b, (u32x4 *)c, n); break;
    default: return -1;
  }
  return hipGetLastError() == hipSuccess ? 0 : -1;
}
