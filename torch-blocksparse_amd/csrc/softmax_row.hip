// Block-sparse softmax for long rows: one wavefront per matrix row.
//
// The kernels of softmax.hip give a row a few lanes (8 at block 64) and keep it in registers, which stops at 32 blocks
// per row; beyond that they fall back to a variant that re-reads x and works a row of a hundred blocks with one
// eighth of a wavefront.  Rows that long come with dense-ish layouts (the reference's own softmax benchmark: "sparse
// GPT-2 / BERT" at sequence 8192 are a full and a triangular matrix of blocks of 64, tests/test_softmax.py:92-128; the
// 'fixed' layout at the default block of 16 has 67 blocks per row at sequence 4096), and there the row, not the block,
// is the natural unit: here the 64 lanes of a wavefront walk the row's blocks side by side, each lane one 16-byte piece of
// a block's row per step (block 64, fp16: 8 lanes per block, 8 blocks per step), NI steps, everything in registers,
// each element read once and written once (forward) or read twice and written once (backward).  Same semantics as
// softmax.py:7-138, 144-194; same table.  Rows of up to 64 * NI pieces (8192 elements of a 16-bit type at NI = 16).
#include "softmax_common.h"

namespace bsp {
namespace {

template <typename T> struct RowGeo {
  static constexpr int EV = 16 / (int)sizeof(T);                 // elements per lane and step
};

template <typename T, int BLOCK, int NI>
__global__ void __launch_bounds__(256) k_softmax_row_fwd(FwdArgs a) {
  constexpr int EV = RowGeo<T>::EV, LPB = BLOCK / EV, BPS = 64 / LPB;     // blocks per step
  typedef Pack<T, EV> P;
  const int lane = threadIdx.x & 63;
  const int64_t n_rows = (int64_t)a.Z * a.H * a.R * BLOCK;
  const int64_t row = ((int64_t)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6));
  if (row >= n_rows) return;
  // rows of a block-row are neighbours (they share the table and the masks' columns), block-rows from the last one down
  const int rxm = (int)(row % BLOCK);
  const int64_t t = row / BLOCK;
  const int HR = a.H * a.R;
  const int hr = HR - 1 - (int)(t % HR);
  const int z = (int)(t / HR);
  const table_ptr lut = as_table(a.lut);
  const int size = lut[2 * hr + 0], offset = lut[2 * hr + 1];
  if (size <= 0) return;
  const int head = hr / a.R, brow = hr % a.R;
  const int32_t *core = a.lut + offset;                          // (blockid, col, row, head) per block: read per lane
  const int sub = lane / LPB, col = (lane % LPB) * EV;           // this lane's block inside a step, first column inside the block
  const float unit = logit_unit<T>();
  const float sc = a.scale * unit;
  T *xz = reinterpret_cast<T *>(a.x) + (int64_t)z * a.x_sz + rxm * BLOCK + col;
  const int64_t grow = (int64_t)brow * BLOCK + rxm;
  const T *kz = reinterpret_cast<const T *>(a.kpm) + (int64_t)z * a.kpm_sz + col;
  const T *rz = reinterpret_cast<const T *>(a.rpe) + (int64_t)z * a.rpe_sz + (int64_t)head * a.rpe_sh + grow * a.rpe_sr + col;
  const T *az = reinterpret_cast<const T *>(a.attn) + grow * a.attn_sr + col;
  P px[NI];
  float l[NI][EV];
  // all loads of the row first (tables, then x and the masks), then the arithmetic
  int32_t bid[NI], bcol[NI];
#pragma unroll
  for (int i = 0; i < NI; i++) {
    const int b = i * BPS + sub;
    const int bb = b < size ? b : 0;
    bid[i] = core[4 * bb + 0];
    bcol[i] = core[4 * bb + 1];
  }
#pragma unroll
  for (int i = 0; i < NI; i++) px[i].load(xz + (int64_t)bid[i] * (BLOCK * BLOCK));
#pragma unroll
  for (int i = 0; i < NI; i++) {
    const bool live = i * BPS + sub < size;
#pragma unroll
    for (int e = 0; e < EV; e++) l[i][e] = live ? to_float(px[i].e[e]) * sc : -INFINITY;      // softmax.py:112-116
  }
  if (a.kpm) {                                                    // :122-124, 'mul' mode :104-106
#pragma unroll
    for (int i = 0; i < NI; i++) {
      P pk;
      pk.load(kz + (int64_t)bcol[i] * BLOCK);
#pragma unroll
      for (int e = 0; e < EV; e++) {
        const float m = to_float(pk.e[e]);
        l[i][e] += a.kpm_mul ? (m == 0.f ? -INFINITY : 0.f) : m * unit;
      }
    }
  }
  if (a.rpe) {                                                    // :118-120
#pragma unroll
    for (int i = 0; i < NI; i++) {
      P pr;
      pr.load(rz + (int64_t)bcol[i] * BLOCK);
#pragma unroll
      for (int e = 0; e < EV; e++) l[i][e] = fmaf(to_float(pr.e[e]), unit, l[i][e]);
    }
  }
  if (a.attn) {                                                   // :126-128, 'mul' mode :108-110
#pragma unroll
    for (int i = 0; i < NI; i++) {
      P pa;
      pa.load(az + (int64_t)bcol[i] * BLOCK);
#pragma unroll
      for (int e = 0; e < EV; e++) {
        const float m = to_float(pa.e[e]);
        l[i][e] += a.attn_mul ? (m == 0.f ? -INFINITY : 0.f) : m * unit;
      }
    }
  }
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < NI; i++)
#pragma unroll
    for (int e = 0; e < EV; e++) mx = fmaxf(mx, l[i][e]);
  mx = row_max<64>(mx);                                           // :130
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < NI; i++)
#pragma unroll
    for (int e = 0; e < EV; e++) { l[i][e] = exp_sub<T>(l[i][e], mx); sum += l[i][e]; }   // :131-132 (a fully masked row: NaN, as there)
  sum = row_sum<64>(sum);
  const float inv = 1.f / sum;
#pragma unroll
  for (int i = 0; i < NI; i++)
    if (i * BPS + sub < size) {
      P out;
#pragma unroll
      for (int e = 0; e < EV; e++) out.e[e] = from_float<T>(l[i][e] * inv);               // :137
      out.store(xz + (int64_t)bid[i] * (BLOCK * BLOCK));
    }
}

template <typename T, int BLOCK, int NI>
__global__ void __launch_bounds__(256) k_softmax_row_bwd(BwdArgs a) {
  constexpr int EV = RowGeo<T>::EV, LPB = BLOCK / EV, BPS = 64 / LPB;
  typedef Pack<T, EV> P;
  const int lane = threadIdx.x & 63;
  const int64_t n_rows = (int64_t)a.Z * a.H * a.R * BLOCK;
  const int64_t row = ((int64_t)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6));
  if (row >= n_rows) return;
  const int rxm = (int)(row % BLOCK);
  const int64_t t = row / BLOCK;
  const int HR = a.H * a.R;
  const int hr = HR - 1 - (int)(t % HR);
  const int z = (int)(t / HR);
  const table_ptr lut = as_table(a.lut);
  const int size = lut[2 * hr + 0], offset = lut[2 * hr + 1];
  if (size <= 0) return;
  const int32_t *core = a.lut + offset;
  const int sub = lane / LPB, col = (lane % LPB) * EV;
  const T *yz = reinterpret_cast<const T *>(a.y) + (int64_t)z * a.y_sz + rxm * BLOCK + col;
  T *dz = reinterpret_cast<T *>(a.dy) + (int64_t)z * a.dy_sz + rxm * BLOCK + col;
  int32_t bid[NI];
  P py[NI], pd[NI];
#pragma unroll
  for (int i = 0; i < NI; i++) {
    const int b = i * BPS + sub;
    bid[i] = core[4 * (b < size ? b : 0)];
  }
#pragma unroll
  for (int i = 0; i < NI; i++) {
    py[i].load_stream(yz + (int64_t)bid[i] * (BLOCK * BLOCK));    // y is not read again after the backward pass
    pd[i].load(dz + (int64_t)bid[i] * (BLOCK * BLOCK));
  }
  float dot = 0.f;
#pragma unroll
  for (int i = 0; i < NI; i++)
    if (i * BPS + sub < size) {
#pragma unroll
      for (int e = 0; e < EV; e++) dot += to_float(py[i].e[e]) * to_float(pd[i].e[e]);     // softmax.py:187-188
    }
  dot = row_sum<64>(dot);
#pragma unroll
  for (int i = 0; i < NI; i++)
    if (i * BPS + sub < size) {
      P out;
#pragma unroll
      for (int e = 0; e < EV; e++) out.e[e] = from_float<T>(to_float(py[i].e[e]) * (to_float(pd[i].e[e]) - dot) * a.scale);   // :189
      out.store(dz + (int64_t)bid[i] * (BLOCK * BLOCK));
    }
}

// the smallest number of steps (1, 2, 4, 8 or 16) that holds a row of maxlut blocks; 0 = too long for these kernels
template <typename T, int BLOCK> int steps_for(int maxlut) {
  constexpr int BPS = 64 / (BLOCK / RowGeo<T>::EV);
  for (int ni : {1, 2, 4, 8, 16})
    if (maxlut <= ni * BPS) return ni;
  return 0;
}

template <typename T, int BLOCK> int row_fwd_b(const FwdArgs &a, int maxlut, hipStream_t st) {
  const int64_t n_rows = (int64_t)a.Z * a.H * a.R * BLOCK, n_wg = (n_rows + 3) / 4;
  if (n_wg >= ((int64_t)1 << 31)) return 0;
  const dim3 grid((unsigned)n_wg), wg(256);
  switch (steps_for<T, BLOCK>(maxlut)) {
    case 1: hipLaunchKernelGGL((k_softmax_row_fwd<T, BLOCK, 1>), grid, wg, 0, st, a); return 1;
    case 2: hipLaunchKernelGGL((k_softmax_row_fwd<T, BLOCK, 2>), grid, wg, 0, st, a); return 1;
    case 4: hipLaunchKernelGGL((k_softmax_row_fwd<T, BLOCK, 4>), grid, wg, 0, st, a); return 1;
    case 8: hipLaunchKernelGGL((k_softmax_row_fwd<T, BLOCK, 8>), grid, wg, 0, st, a); return 1;
    case 16: hipLaunchKernelGGL((k_softmax_row_fwd<T, BLOCK, 16>), grid, wg, 0, st, a); return 1;
    default: return 0;
  }
}
template <typename T, int BLOCK> int row_bwd_b(const BwdArgs &a, int maxlut, hipStream_t st) {
  const int64_t n_rows = (int64_t)a.Z * a.H * a.R * BLOCK, n_wg = (n_rows + 3) / 4;
  if (n_wg >= ((int64_t)1 << 31)) return 0;
  const dim3 grid((unsigned)n_wg), wg(256);
  switch (steps_for<T, BLOCK>(maxlut)) {
    case 1: hipLaunchKernelGGL((k_softmax_row_bwd<T, BLOCK, 1>), grid, wg, 0, st, a); return 1;
    case 2: hipLaunchKernelGGL((k_softmax_row_bwd<T, BLOCK, 2>), grid, wg, 0, st, a); return 1;
    case 4: hipLaunchKernelGGL((k_softmax_row_bwd<T, BLOCK, 4>), grid, wg, 0, st, a); return 1;
    case 8: hipLaunchKernelGGL((k_softmax_row_bwd<T, BLOCK, 8>), grid, wg, 0, st, a); return 1;
    case 16: hipLaunchKernelGGL((k_softmax_row_bwd<T, BLOCK, 16>), grid, wg, 0, st, a); return 1;
    default: return 0;
  }
}
template <typename T> int row_fwd_t(const FwdArgs &a, int block, int maxlut, hipStream_t st) {
  switch (block) {
    case 16: return row_fwd_b<T, 16>(a, maxlut, st);
    case 32: return row_fwd_b<T, 32>(a, maxlut, st);
    case 64: return row_fwd_b<T, 64>(a, maxlut, st);
    case 128: return row_fwd_b<T, 128>(a, maxlut, st);
    default: return 0;
  }
}
template <typename T> int row_bwd_t(const BwdArgs &a, int block, int maxlut, hipStream_t st) {
  switch (block) {
    case 16: return row_bwd_b<T, 16>(a, maxlut, st);
    case 32: return row_bwd_b<T, 32>(a, maxlut, st);
    case 64: return row_bwd_b<T, 64>(a, maxlut, st);
    case 128: return row_bwd_b<T, 128>(a, maxlut, st);
    default: return 0;
  }
}

}  // namespace

// (dropout stays with the kernels of softmax.hip)
int softmax_row_fwd(int dtype, const FwdArgs &a, int block, int maxlut, hipStream_t st) {
  if (a.drop.yd != nullptr) return 0;
  switch (dtype) {
    case BSP_F16: return row_fwd_t<f16>(a, block, maxlut, st);
    case BSP_BF16: return row_fwd_t<bf16>(a, block, maxlut, st);
    case BSP_F32: return row_fwd_t<float>(a, block, maxlut, st);
    default: return 0;
  }
}
int softmax_row_bwd(int dtype, const BwdArgs &a, int block, int maxlut, hipStream_t st) {
  if (a.drop.p > 0.f) return 0;
  switch (dtype) {
    case BSP_F16: return row_bwd_t<f16>(a, block, maxlut, st);
    case BSP_BF16: return row_bwd_t<bf16>(a, block, maxlut, st);
    case BSP_F32: return row_bwd_t<float>(a, block, maxlut, st);
    default: return 0;
  }
}

}  // namespace bsp
