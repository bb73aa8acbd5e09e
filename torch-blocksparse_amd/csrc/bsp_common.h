// Shared declarations for the gfx950 block-sparse kernels: status helpers, 16-bit types, MFMA wrappers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/bsp.h"

#define BSP_HIP_CHECK(expr)                       \
  do {                                            \
    hipError_t e__ = (expr);                      \
    if (e__ != hipSuccess) return BSP_ERR_HIP;    \
  } while (0)

// Launch check: asynchronous launches only report configuration errors here.
#define BSP_LAUNCH_CHECK()                                 \
  do {                                                     \
    if (hipGetLastError() != hipSuccess) return BSP_ERR_HIP; \
  } while (0)

namespace bsp {

typedef _Float16 f16;
typedef __bf16 bf16;

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

static inline int cdiv(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }
static inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2).  Re-number them so that the
// workgroups that land on one XCD cover one contiguous range of work items.
__device__ __forceinline__ int64_t xcd_remap(int64_t wg, int64_t n_wg) {
  const int64_t per = n_wg >> 3;
  const int64_t full = per << 3;
  if (wg >= full) return wg;            // ragged tail keeps its position
  return (wg & 7) * per + (wg >> 3);
}

// Look-up tables are read-only for every kernel that consumes them.  Reading them through the constant address
// space lets the compiler use scalar loads for wave-uniform entries even after a barrier (a plain global pointer
// falls back to vector loads there, and waiting for such a load means waiting for every prefetch issued before it).
typedef const int32_t __attribute__((address_space(4))) *table_ptr;
__device__ __forceinline__ table_ptr as_table(const int32_t *p) { return (table_ptr)p; }

template <typename T> struct TypeInfo;
template <> struct TypeInfo<f16> { static constexpr int kVec = 8; static constexpr bool k16 = true; };
template <> struct TypeInfo<bf16> { static constexpr int kVec = 8; static constexpr bool k16 = true; };
template <> struct TypeInfo<float> { static constexpr int kVec = 4; static constexpr bool k16 = false; };

__device__ __forceinline__ float to_float(f16 v) { return (float)v; }
__device__ __forceinline__ float to_float(bf16 v) { return (float)v; }
__device__ __forceinline__ float to_float(float v) { return v; }
template <typename T> __device__ __forceinline__ T from_float(float v) { return (T)v; }

}  // namespace bsp
