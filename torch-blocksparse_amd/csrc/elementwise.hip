// The two dense utility ops of the reference package, for gfx950: the fused scale-bias-residual ReLU
// (relu.py:8-58) and the NCHW <-> CHWN permutation (permute.py:5-30).  Both are plain HBM streams.
#include "bsp_common.h"

namespace bsp {
namespace {

constexpr int kThreads = 256;
constexpr int kMaxGroups = 4096;   // workgroups of a ReLU launch = partial sums the backward pass leaves behind

template <typename T, int VE> struct Chunk;
template <typename T> struct Chunk<T, 1> { T e[1]; };
template <> struct Chunk<f16, 8> { union { u32x4 raw; f16 e[8]; }; };
template <> struct Chunk<bf16, 8> { union { u32x4 raw; bf16 e[8]; }; };
template <> struct Chunk<float, 4> { union { u32x4 raw; float e[4]; }; };

template <typename T, int VE> __device__ __forceinline__ Chunk<T, VE> load_chunk(const T *p) {
  Chunk<T, VE> c;
  if constexpr (VE == 1) c.e[0] = *p;
  else c.raw = *reinterpret_cast<const u32x4 *>(p);
  return c;
}
template <typename T, int VE> __device__ __forceinline__ void store_chunk(T *p, const Chunk<T, VE> &c) {
  if constexpr (VE == 1) *p = c.e[0];
  else *reinterpret_cast<u32x4 *>(p) = c.raw;
}

// y = max(x * scale + bias + res, 0) over n elements of identically laid out tensors (relu.py:13-27); scale and bias
// are read from device memory, so the launch needs no host synchronisation.  VE elements per lane and step; the
// n % VE last elements go one by one.
template <typename T, int VE>
__global__ void __launch_bounds__(kThreads) k_relu_fwd(const T *x, const T *res, T *y, const T *scale, const T *bias, int64_t n) {
  const float s = to_float(*scale), b = to_float(*bias);
  const int64_t nv = n / VE, stride = (int64_t)gridDim.x * kThreads, t = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  for (int64_t i = t; i < nv; i += stride) {
    const Chunk<T, VE> cx = load_chunk<T, VE>(x + i * VE), cr = load_chunk<T, VE>(res + i * VE);
    Chunk<T, VE> cy;
#pragma unroll
    for (int e = 0; e < VE; e++) {
      const float v = fmaf(to_float(cx.e[e]), s, b) + to_float(cr.e[e]);
      cy.e[e] = from_float<T>(v > 0.f ? v : 0.f);
    }
    store_chunk<T, VE>(y + i * VE, cy);
  }
  for (int64_t i = nv * VE + t; i < n; i += stride) {
    const float v = fmaf(to_float(x[i]), s, b) + to_float(res[i]);
    y[i] = from_float<T>(v > 0.f ? v : 0.f);
  }
}

// du = (y > 0) ? dy : 0; dx = du * scale; dres = du; per-workgroup sums of du and du * x (relu.py:30-55).  The
// reference adds them up with floating-point atomics; here every workgroup writes its two partial sums and
// k_relu_finish adds them in a fixed order, so the result does not depend on scheduling.
template <typename T, int VE>
__global__ void __launch_bounds__(kThreads) k_relu_bwd(const T *x, const T *y, const T *dy, T *dx, T *dres, const T *scale,
                                                        float *partial, int64_t n) {
  const float s = to_float(*scale);
  const int64_t nv = n / VE, stride = (int64_t)gridDim.x * kThreads, t = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  float sum_b = 0.f, sum_s = 0.f;
  for (int64_t i = t; i < nv; i += stride) {
    const Chunk<T, VE> cx = load_chunk<T, VE>(x + i * VE), cy = load_chunk<T, VE>(y + i * VE), cd = load_chunk<T, VE>(dy + i * VE);
    Chunk<T, VE> ox, orr;
#pragma unroll
    for (int e = 0; e < VE; e++) {
      const float du = to_float(cy.e[e]) > 0.f ? to_float(cd.e[e]) : 0.f;
      ox.e[e] = from_float<T>(du * s);
      orr.e[e] = from_float<T>(du);
      sum_b += du;
      sum_s = fmaf(du, to_float(cx.e[e]), sum_s);
    }
    store_chunk<T, VE>(dx + i * VE, ox);
    store_chunk<T, VE>(dres + i * VE, orr);
  }
  for (int64_t i = nv * VE + t; i < n; i += stride) {
    const float du = to_float(y[i]) > 0.f ? to_float(dy[i]) : 0.f;
    dx[i] = from_float<T>(du * s);
    dres[i] = from_float<T>(du);
    sum_b += du;
    sum_s = fmaf(du, to_float(x[i]), sum_s);
  }
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) {
    sum_b += __shfl_xor(sum_b, d);
    sum_s += __shfl_xor(sum_s, d);
  }
  __shared__ float red[2][kThreads / 64];
  if ((threadIdx.x & 63) == 0) { red[0][threadIdx.x >> 6] = sum_b; red[1][threadIdx.x >> 6] = sum_s; }
  __syncthreads();
  if (threadIdx.x == 0) {
    float b = 0.f, sc = 0.f;
    for (int w = 0; w < kThreads / 64; w++) { b += red[0][w]; sc += red[1][w]; }
    partial[2 * blockIdx.x + 0] = b;
    partial[2 * blockIdx.x + 1] = sc;
  }
}

__global__ void __launch_bounds__(64) k_relu_finish(const float *partial, int groups, float *dscale, float *dbias) {
  // one wavefront, fixed order: lane l adds groups l, l + 64, ...; then a butterfly
  float b = 0.f, s = 0.f;
  for (int g = threadIdx.x; g < groups; g += 64) { b += partial[2 * g]; s += partial[2 * g + 1]; }
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) { b += __shfl_xor(b, d); s += __shfl_xor(s, d); }
  if (threadIdx.x == 0) { *dbias = b; *dscale = s; }
}

// y[c][r] = x[r][c] for a rows x cols matrix: 64 x 64 tiles through LDS, reads and writes both along the
// contiguous dimension of their tensor (permute.py:5-30 does the same with 32-wide tiles).
template <typename T>
__global__ void __launch_bounds__(kThreads) k_transpose(const T *x, T *y, int64_t rows, int64_t cols) {
  __shared__ T tile[64][64 + 4 / sizeof(T)];   // odd number of 32-bit words per row: column reads spread over all banks
  const int64_t tiles_c = (cols + 63) / 64;
  const int64_t r0 = (blockIdx.x / tiles_c) * 64, c0 = (blockIdx.x % tiles_c) * 64;
  const int lx = threadIdx.x & 63, ly = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 16; i++) {
    const int64_t r = r0 + ly + 4 * i, c = c0 + lx;
    if (r < rows && c < cols) tile[ly + 4 * i][lx] = x[r * cols + c];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; i++) {
    const int64_t c = c0 + ly + 4 * i, r = r0 + lx;
    if (r < rows && c < cols) y[c * rows + r] = tile[lx][ly + 4 * i];
  }
}

int relu_groups(int64_t n, int ve) {
  const int64_t g = (n / ve + kThreads - 1) / kThreads;
  return (int)(g < 1 ? 1 : (g > kMaxGroups ? kMaxGroups : g));
}
bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename T> int relu_fwd_t(const void *x, const void *res, void *y, const void *scale, const void *bias, int64_t n, hipStream_t st) {
  constexpr int VE = 16 / sizeof(T);
  const T *px = (const T *)x, *pr = (const T *)res, *ps = (const T *)scale, *pb = (const T *)bias;
  if (aligned16(x) && aligned16(res) && aligned16(y))
    hipLaunchKernelGGL((k_relu_fwd<T, VE>), dim3(relu_groups(n, VE)), dim3(kThreads), 0, st, px, pr, (T *)y, ps, pb, n);
  else
    hipLaunchKernelGGL((k_relu_fwd<T, 1>), dim3(relu_groups(n, 1)), dim3(kThreads), 0, st, px, pr, (T *)y, ps, pb, n);
  return BSP_OK;
}
template <typename T> int relu_bwd_t(const void *x, const void *y, const void *dy, void *dx, void *dres, const void *scale,
                                     float *partial, int *groups, int64_t n, hipStream_t st) {
  constexpr int VE = 16 / sizeof(T);
  const T *px = (const T *)x, *py = (const T *)y, *pd = (const T *)dy, *ps = (const T *)scale;
  if (aligned16(x) && aligned16(y) && aligned16(dy) && aligned16(dx) && aligned16(dres)) {
    *groups = relu_groups(n, VE);
    hipLaunchKernelGGL((k_relu_bwd<T, VE>), dim3(*groups), dim3(kThreads), 0, st, px, py, pd, (T *)dx, (T *)dres, ps, partial, n);
  } else {
    *groups = relu_groups(n, 1);
    hipLaunchKernelGGL((k_relu_bwd<T, 1>), dim3(*groups), dim3(kThreads), 0, st, px, py, pd, (T *)dx, (T *)dres, ps, partial, n);
  }
  return BSP_OK;
}

}  // namespace
}  // namespace bsp

using namespace bsp;

extern "C" int64_t bsp_relu_workspace_bytes(void) { return 2 * (int64_t)kMaxGroups * (int64_t)sizeof(float); }

extern "C" int bsp_relu_fwd(int dtype, const void *x, const void *res, void *y, const void *d_scale, const void *d_bias, int64_t n,
                            void *stream) {
  if (!x || !res || !y || !d_scale || !d_bias || n < 0) return BSP_ERR_ARG;
  if (n == 0) return BSP_OK;
  hipStream_t st = as_stream(stream);
  switch (dtype) {
    case BSP_F16: relu_fwd_t<f16>(x, res, y, d_scale, d_bias, n, st); break;
    case BSP_BF16: relu_fwd_t<bf16>(x, res, y, d_scale, d_bias, n, st); break;
    case BSP_F32: relu_fwd_t<float>(x, res, y, d_scale, d_bias, n, st); break;
    default: return BSP_ERR_UNSUPPORTED;
  }
  BSP_LAUNCH_CHECK();
  return BSP_OK;
}

extern "C" int bsp_relu_bwd(int dtype, const void *x, const void *y, const void *dy, void *dx, void *dres, const void *d_scale,
                            float *d_dscale, float *d_dbias, void *d_ws, int64_t ws_bytes, int64_t n, void *stream) {
  if (!x || !y || !dy || !dx || !dres || !d_scale || !d_dscale || !d_dbias || !d_ws || n < 0) return BSP_ERR_ARG;
  if (ws_bytes < bsp_relu_workspace_bytes()) return BSP_ERR_CAPACITY;
  hipStream_t st = as_stream(stream);
  float *partial = (float *)d_ws;
  int groups = 0;
  if (n > 0) {
    switch (dtype) {
      case BSP_F16: relu_bwd_t<f16>(x, y, dy, dx, dres, d_scale, partial, &groups, n, st); break;
      case BSP_BF16: relu_bwd_t<bf16>(x, y, dy, dx, dres, d_scale, partial, &groups, n, st); break;
      case BSP_F32: relu_bwd_t<float>(x, y, dy, dx, dres, d_scale, partial, &groups, n, st); break;
      default: return BSP_ERR_UNSUPPORTED;
    }
  }
  hipLaunchKernelGGL(k_relu_finish, dim3(1), dim3(64), 0, st, partial, groups, d_dscale, d_dbias);
  BSP_LAUNCH_CHECK();
  return BSP_OK;
}

extern "C" int bsp_transpose(int dtype, const void *x, void *y, int64_t rows, int64_t cols, void *stream) {
  if (!x || !y || rows < 0 || cols < 0) return BSP_ERR_ARG;
  if (rows == 0 || cols == 0) return BSP_OK;
  const int64_t tiles = ((rows + 63) / 64) * ((cols + 63) / 64);
  if (tiles >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  hipStream_t st = as_stream(stream);
  if (dtype == BSP_F32) hipLaunchKernelGGL((k_transpose<float>), dim3((unsigned)tiles), dim3(kThreads), 0, st, (const float *)x, (float *)y, rows, cols);
  else if (dtype == BSP_F16 || dtype == BSP_BF16)   // a permutation only moves bits: both 16-bit types share the kernel
    hipLaunchKernelGGL((k_transpose<uint16_t>), dim3((unsigned)tiles), dim3(kThreads), 0, st, (const uint16_t *)x, (uint16_t *)y, rows, cols);
  else return BSP_ERR_UNSUPPORTED;
  BSP_LAUNCH_CHECK();
  return BSP_OK;
}
