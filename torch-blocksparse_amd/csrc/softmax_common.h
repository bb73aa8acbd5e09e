// Shared pieces of the block-sparse softmax kernels (softmax.hip: a few lanes per row, the row in registers;
// softmax_row.hip: one wavefront per row, for rows too long for that).
#ifndef BSP_SOFTMAX_COMMON_H
#define BSP_SOFTMAX_COMMON_H
#include "bsp_common.h"

namespace bsp {

template <typename T, int EV> struct RawVec;
template <> struct RawVec<f16, 8> { typedef u32x4 type; };
template <> struct RawVec<bf16, 8> { typedef u32x4 type; };
template <> struct RawVec<f16, 4> { typedef u32x2 type; };
template <> struct RawVec<bf16, 4> { typedef u32x2 type; };
template <> struct RawVec<float, 4> { typedef u32x4 type; };

template <typename T, int EV> struct Pack {
  typedef typename RawVec<T, EV>::type raw_t;
  union { raw_t raw; T e[EV]; };
  __device__ __forceinline__ void load(const T *p) { raw = *reinterpret_cast<const raw_t *>(p); }
  __device__ __forceinline__ void store(T *p) const { *reinterpret_cast<raw_t *>(p) = raw; }
  // for data nobody reads again soon: leaves the caches to what the next kernels need
  __device__ __forceinline__ void load_stream(const T *p) { raw = __builtin_nontemporal_load(reinterpret_cast<const raw_t *>(p)); }
};

template <int LPR> __device__ __forceinline__ float row_max(float v) {
#pragma unroll
  for (int d = 1; d < LPR; d <<= 1) v = fmaxf(v, __shfl_xor(v, d));
  return v;
}
template <int LPR> __device__ __forceinline__ float row_sum(float v) {
#pragma unroll
  for (int d = 1; d < LPR; d <<= 1) v += __shfl_xor(v, d);
  return v;
}

// 16-bit types work in the log2 domain: the logits are built as x * (scale * log2 e) + mask * log2 e, so that the
// exponential is a bare v_exp_f32 of a difference.  fp32 keeps the natural domain and the accurate expf.
constexpr float kLog2e = 1.44269504088896340736f;
template <typename T> __device__ __forceinline__ float logit_unit() { return sizeof(T) == 4 ? 1.f : kLog2e; }
template <typename T> __device__ __forceinline__ float exp_sub(float x, float mx) {
  if constexpr (sizeof(T) == 4) return expf(x - mx);
  else return __builtin_amdgcn_exp2f(x - mx);
}

// Dropout on the softmax result (no counterpart in the reference, which refuses dropout: attention.py:223-224).
// Element i of the [Z, nnz, block, block] tensor (i = its linear offset, z * stride_z + ...) is kept iff
// u(i) >= p, where u(i) = (w >> 8) * 2^-24 and w is word i % 4 of Philox4x32-10(counter = (i / 4, offset), key = seed);
// kept elements are scaled by 1 / (1 - p).  The mask is a pure function of (seed, offset, i): the backward pass
// re-creates it instead of reading it from memory.
struct DropArgs {
  float p = 0.f, inv_keep = 1.f;
  uint32_t seed_lo = 0, seed_hi = 0, off_lo = 0, off_hi = 0;
  void *yd = nullptr; int64_t yd_sz = 0;   // forward: where the dropped result goes (x keeps the softmax itself)
};

__device__ __forceinline__ u32x4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; r++) {
    const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
    c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  return u32x4{c0, c1, c2, c3};
}

// m[e] = 1 / (1 - p) if element idx + e is kept, else 0; idx is a multiple of 4, EV is 4 or 8
template <int EV> __device__ __forceinline__ void keep_scale(const DropArgs &d, int64_t idx, float (&m)[EV]) {
#pragma unroll
  for (int e4 = 0; e4 < EV; e4 += 4) {
    const uint64_t q = (uint64_t)(idx + e4) >> 2;
    const u32x4 w = philox4x32_10((uint32_t)q, (uint32_t)(q >> 32), d.off_lo, d.off_hi, d.seed_lo, d.seed_hi);
#pragma unroll
    for (int e = 0; e < 4; e++) m[e4 + e] = (float)(w[e] >> 8) * 5.9604644775390625e-08f >= d.p ? d.inv_keep : 0.f;
  }
}

struct FwdArgs {
  void *x; float scale; const int32_t *lut;
  const void *rpe; int64_t rpe_sz, rpe_sh, rpe_sr;
  const void *kpm; int64_t kpm_sz; int kpm_mul;
  const void *attn; int64_t attn_sr; int attn_mul;
  int Z, H, R; int64_t x_sz; int64_t n_units;
  DropArgs drop;
};

struct BwdArgs {
  const void *y; void *dy; float scale; const int32_t *lut;
  int Z, H, R; int64_t y_sz, dy_sz; int64_t n_units;
  DropArgs drop;
};


// One wavefront per matrix row (softmax_row.hip): 1 = launched, 0 = not this kernel's case (the caller takes another)
int softmax_row_fwd(int dtype, const FwdArgs &a, int block, int maxlut, hipStream_t st);
int softmax_row_bwd(int dtype, const BwdArgs &a, int block, int maxlut, hipStream_t st);

}  // namespace bsp
#endif
