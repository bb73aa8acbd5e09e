// General block-sparse matmul kernels for gfx950: every block size (16/32/64/128), fp16 / bf16 / fp32,
// every trans_a / trans_b / trans_c combination.
//
// Replaces the reference's single Triton-C kernel with its SDD / DSD / DDS branches (matmul.py:6-205).
// Structure: a workgroup of four wavefronts owns one output tile; both operand tiles are staged through LDS
// in a reduction-contiguous layout (rows of TK elements plus padding) so that every MFMA operand is one
// 16-byte LDS read whatever the operand's orientation in memory; an operand stored with the reduction
// dimension strided is transposed while it is written to LDS.  Global loads for step s+1 are issued before
// the MFMAs of step s (two LDS buffers, one barrier per step).  fp32 accumulation in 16x16 MFMA tiles.
//
// "xsd" is the kernel behind both dsd and dds: dds is dsd with the roles of rows and columns exchanged
// (C^T = B_sparse^T . A^T), which only changes the three orientation flags.
#pragma once
#include "bsp_common.h"

namespace bsp {

// ---------------------------------------------------------------------------------------------------------
// 16x16 MFMA per element type.  Lane l supplies row (l % 16) of its operand, reduction indices
// (l / 16) * KV .. + KV - 1; the result tile has row 4 * (l / 16) + e, column l % 16 in element e.
// ---------------------------------------------------------------------------------------------------------
template <typename T> struct Mma16;
template <> struct Mma16<f16> {
  static constexpr int KSTEP = 32, KV = 8;
  typedef f16x8 frag_t;
  static __device__ __forceinline__ f32x4 run(frag_t a, frag_t b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};
template <> struct Mma16<bf16> {
  static constexpr int KSTEP = 32, KV = 8;
  typedef bf16x8 frag_t;
  static __device__ __forceinline__ f32x4 run(frag_t a, frag_t b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Mma16<float> {
  static constexpr int KSTEP = 4, KV = 1;
  typedef float frag_t;
  static __device__ __forceinline__ f32x4 run(frag_t a, frag_t b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
};

template <typename T> struct TileK { static constexpr int TK = 64 / sizeof(T), PAD = 16 / sizeof(T); };  // 64-byte rows + 16 bytes

// ---------------------------------------------------------------------------------------------------------
// One operand tile: ROWS x TK, fetched by NT threads in 16-byte chunks, kept in registers until the LDS
// buffer is free.  View::ptr_k(row, k) -> address of elements (row, k..k+VE-1) or nullptr (zero fill);
// View::ptr_r(row, k) -> address of elements (row..row+VE-1, k) or nullptr.
// ---------------------------------------------------------------------------------------------------------
template <typename T, int ROWS, int NT, bool KCONTIG> struct TileLoader {
  static constexpr int TK = TileK<T>::TK, LDK = TK + TileK<T>::PAD;
  static constexpr int VE = 16 / sizeof(T);
  static constexpr int NCH = ROWS * TK / VE;
  static constexpr int ITER = (NCH + NT - 1) / NT;
  static constexpr int CPR = TK / VE;    // chunks per row when the reduction is contiguous
  static constexpr int RCH = ROWS / VE;  // chunks per reduction index otherwise
  u32x4 reg[ITER];

  template <class View> __device__ __forceinline__ void load(const View &v, int k0, int tid) {
#pragma unroll
    for (int it = 0; it < ITER; it++) {
      const int c = tid + it * NT;
      const T *p = nullptr;
      if (NCH % NT == 0 || c < NCH) {
        if constexpr (KCONTIG) p = v.ptr_k(c / CPR, k0 + (c % CPR) * VE);
        else p = v.ptr_r((c % RCH) * VE, k0 + c / RCH);
      }
      u32x4 z = {0u, 0u, 0u, 0u};
      reg[it] = p ? *reinterpret_cast<const u32x4 *>(p) : z;
    }
  }
  __device__ __forceinline__ void store(T *S, int tid) const {
#pragma unroll
    for (int it = 0; it < ITER; it++) {
      const int c = tid + it * NT;
      if (NCH % NT == 0 || c < NCH) {
        if constexpr (KCONTIG) {
          *reinterpret_cast<u32x4 *>(S + (c / CPR) * LDK + (c % CPR) * VE) = reg[it];
        } else {
          union { u32x4 raw; T e[VE]; } u;
          u.raw = reg[it];
          const int row0 = (c % RCH) * VE, k = c / RCH;
#pragma unroll
          for (int e = 0; e < VE; e++) S[(row0 + e) * LDK + k] = u.e[e];
        }
      }
    }
  }
};

// ---------------------------------------------------------------------------------------------------------
// The tile product.  X supplies TM rows ("m"), Y supplies TN rows ("n"); out(m, n) = sum_k X(m,k) * Y(n,k).
// WGM x WGN wavefronts, each RM x RN MFMA tiles.  OUT_NCONTIG chooses which index the four values of a lane
// run along, so that the epilogue writes 4 consecutive elements whatever the output orientation.
// ---------------------------------------------------------------------------------------------------------
template <typename T, int TM, int TN, int WGM, int WGN, bool X_KCONTIG, bool Y_KCONTIG, bool OUT_NCONTIG> struct TileGemm {
  static constexpr int NT = 64 * WGM * WGN;
  static constexpr int TK = TileK<T>::TK, LDK = TK + TileK<T>::PAD;
  static constexpr int RM = TM / (16 * WGM), RN = TN / (16 * WGN);
  static constexpr int X_ELEMS = TM * LDK, Y_ELEMS = TN * LDK;
  static constexpr int SMEM_BYTES = 2 * (X_ELEMS + Y_ELEMS) * (int)sizeof(T);
  typedef Mma16<T> M;
  typedef TileLoader<T, TM, NT, X_KCONTIG> XL;
  typedef TileLoader<T, TN, NT, Y_KCONTIG> YL;

  // ksteps = number of TK-wide reduction steps.  Store(m, n, vals): vals[4] run along n (OUT_NCONTIG) or m.
  template <class XView, class YView, class Store>
  static __device__ __forceinline__ void run(const XView &xv, const YView &yv, int ksteps, T *smem, const Store &store) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    T *Xs[2] = {smem, smem + X_ELEMS + Y_ELEMS};
    T *Ys[2] = {smem + X_ELEMS, smem + 2 * X_ELEMS + Y_ELEMS};
    f32x4 acc[RM][RN];
#pragma unroll
    for (int i = 0; i < RM; i++)
#pragma unroll
      for (int j = 0; j < RN; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    XL xl;
    YL yl;
    if (ksteps > 0) {
      xl.load(xv, 0, tid);
      yl.load(yv, 0, tid);
      xl.store(Xs[0], tid);
      yl.store(Ys[0], tid);
    }
    __syncthreads();
    for (int s = 0; s < ksteps; s++) {
      const int cur = s & 1;
      if (s + 1 < ksteps) {
        xl.load(xv, (s + 1) * TK, tid);
        yl.load(yv, (s + 1) * TK, tid);
      }
      const T *xs = Xs[cur] + (wm * RM * 16 + (lane & 15)) * LDK + (lane >> 4) * M::KV;
      const T *ys = Ys[cur] + (wn * RN * 16 + (lane & 15)) * LDK + (lane >> 4) * M::KV;
#pragma unroll
      for (int kk = 0; kk < TK / M::KSTEP; kk++) {
        typename M::frag_t xf[RM], yf[RN];
#pragma unroll
        for (int i = 0; i < RM; i++) xf[i] = *reinterpret_cast<const typename M::frag_t *>(xs + i * 16 * LDK + kk * M::KSTEP);
#pragma unroll
        for (int j = 0; j < RN; j++) yf[j] = *reinterpret_cast<const typename M::frag_t *>(ys + j * 16 * LDK + kk * M::KSTEP);
#pragma unroll
        for (int i = 0; i < RM; i++)
#pragma unroll
          for (int j = 0; j < RN; j++) {
            if constexpr (OUT_NCONTIG) acc[i][j] = M::run(yf[j], xf[i], acc[i][j]);   // result rows = n, column = m
            else acc[i][j] = M::run(xf[i], yf[j], acc[i][j]);                          // result rows = m, column = n
          }
      }
      if (s + 1 < ksteps) {
        xl.store(Xs[cur ^ 1], tid);   // the other buffer was last read before the previous barrier
        yl.store(Ys[cur ^ 1], tid);
      }
      __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < RM; i++)
#pragma unroll
      for (int j = 0; j < RN; j++) {
        const int m0 = (wm * RM + i) * 16, n0 = (wn * RN + j) * 16;
        if constexpr (OUT_NCONTIG) store(m0 + (lane & 15), n0 + 4 * (lane >> 4), acc[i][j]);
        else store(m0 + 4 * (lane >> 4), n0 + (lane & 15), acc[i][j]);
      }
  }
};

template <typename T> __device__ __forceinline__ void store4(T *p, f32x4 v) {
  if constexpr (sizeof(T) == 4) {
    *reinterpret_cast<f32x4 *>(p) = v;
  } else {
    union { u32x2 raw; T e[4]; } u;
#pragma unroll
    for (int e = 0; e < 4; e++) u.e[e] = from_float<T>(v[e]);
    *reinterpret_cast<u32x2 *>(p) = u.raw;
  }
}

// ---------------------------------------------------------------------------------------------------------
// sdd: C[z, blockid] = op(A)[z,h, i-th block-row, :K] . op(B)[z,h, :K, j-th block-col]
// One workgroup per super-block of PACK x PACK blocks of the sdd table (reference kernel matmul.py:30-54,
// 163-176: rows come from the table entries (bm, 0), columns from (0, bn), the head from entry (0, 0), the
// output block from entry (bm, bn)).
// ---------------------------------------------------------------------------------------------------------
struct SddArgs {
  const void *a, *b; void *c;
  int Z, K;
  int64_t a_sz, a_sh, lda, b_sz, b_sh, ldb, c_sz;
  const int32_t *lut; const uint8_t *valid;
  int64_t n_groups;
  const int32_t *gplan; int n_pgroups; int lines;   // optional group plan (by rows), its groups, block-rows per head
};

template <typename T, int BLOCK, int PACK, bool KCONTIG> struct SddView {
  const T *base; int64_t ld; int K; int idx[PACK];
  __device__ __forceinline__ int blk(int row) const {
    int r = idx[0];
#pragma unroll
    for (int p = 1; p < PACK; p++) r = (row / BLOCK == p) ? idx[p] : r;
    return r * BLOCK + row % BLOCK;
  }
  __device__ __forceinline__ const T *ptr_k(int row, int k) const { return k < K ? base + (int64_t)blk(row) * ld + k : nullptr; }
  __device__ __forceinline__ const T *ptr_r(int row, int k) const { return k < K ? base + (int64_t)k * ld + blk(row) : nullptr; }
};

template <int T_> struct SddShape { static constexpr int WG = T_ >= 32 ? 2 : 1; };

template <typename T, int BLOCK, int PACK, bool A_KCONTIG, bool B_KCONTIG>
__global__ void __launch_bounds__(64 * SddShape<BLOCK * PACK>::WG * SddShape<BLOCK * PACK>::WG) k_sdd(SddArgs g) {
  constexpr int TT = BLOCK * PACK, WG = SddShape<TT>::WG;
  typedef TileGemm<T, TT, TT, WG, WG, A_KCONTIG, B_KCONTIG, true> G;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int64_t n_wg = g.n_groups * g.Z;
  const int64_t w = xcd_remap(blockIdx.x, n_wg);
  const int z = (int)(w / g.n_groups);
  const int64_t grp = w % g.n_groups;
  const int32_t *e = g.lut + grp * (PACK * PACK * 4);
  const int h = e[0];
  SddView<T, BLOCK, PACK, A_KCONTIG> av;
  SddView<T, BLOCK, PACK, B_KCONTIG> bv;
  av.base = reinterpret_cast<const T *>(g.a) + z * g.a_sz + h * g.a_sh; av.ld = g.lda; av.K = g.K;
  bv.base = reinterpret_cast<const T *>(g.b) + z * g.b_sz + h * g.b_sh; bv.ld = g.ldb; bv.K = g.K;
#pragma unroll
  for (int p = 0; p < PACK; p++) {
    av.idx[p] = e[(p * PACK) * 4 + 1];   // block-row of entries (p, 0)
    bv.idx[p] = e[p * 4 + 2];            // block-col of entries (0, p)
  }
  T *cz = reinterpret_cast<T *>(g.c) + z * g.c_sz;
  const uint8_t *valid = g.valid ? g.valid + grp * (PACK * PACK) : nullptr;
  auto store = [&](int m, int n, f32x4 v) {
    const int ent = (m / BLOCK) * PACK + n / BLOCK;
    if (valid && !valid[ent]) return;
    const int64_t bk = e[ent * 4 + 3];
    store4<T>(cz + bk * (BLOCK * BLOCK) + (m % BLOCK) * BLOCK + n % BLOCK, v);
  };
  G::run(av, bv, (g.K + G::TK - 1) / G::TK, reinterpret_cast<T *>(smem_raw), store);
}

// ---------------------------------------------------------------------------------------------------------
// xsd: out[col*BLOCK + m, n] = sum over the blocks t of one table segment  S_t(m, :) . D(n, pos_t + :)
// (dsd: S = op(A) blocks, D = op(B)^T rows; dds: S = op(B)^T blocks, D = op(A) rows).
// One workgroup per (segment, 64-wide tile of the dense free dimension, batch).  Reads the segment header
// of the reference table (offset, length, column, depth; matmul.py:57-63) and the per-block positions.
// ---------------------------------------------------------------------------------------------------------
struct XsdArgs {
  const void *sp, *dn; void *out;
  int Z, NF;                            // batch, size of the dense free dimension
  int64_t sp_sz, dn_sz, dn_sh, ldd, out_sz, out_sh, ldo;
  const int32_t *lut; const int32_t *plan; int width; int div2;   // div2 = 2 * block / step of the table
  int n_tiles;
  const int32_t *gplan; int n_pgroups; int lines;   // optional group plan, its groups, lines (block-rows or -columns) per head
};

template <typename T, int BLOCK, bool TRANS> struct SparseView {   // element (m, k) of the segment's blocks
  const T *base; const int32_t *plan; int nblk;
  __device__ __forceinline__ const T *blk(int k) const {
    const int ord = k / BLOCK;
    return ord < nblk ? base + (int64_t)plan[2 * ord + 1] * (BLOCK * BLOCK) : nullptr;
  }
  __device__ __forceinline__ const T *ptr_k(int row, int k) const {   // stored [m][k]
    const T *b = blk(k);
    return b ? b + row * BLOCK + k % BLOCK : nullptr;
  }
  __device__ __forceinline__ const T *ptr_r(int row, int k) const {   // stored [k][m]
    const T *b = blk(k);
    return b ? b + (k % BLOCK) * BLOCK + row : nullptr;
  }
};

template <typename T, int BLOCK> struct DenseView {                   // element (n, k): dense row/col n, reduction position k
  const T *base; const int32_t *plan; int nblk; int64_t ld; int n0, NF;
  __device__ __forceinline__ int64_t pos(int k) const { return (int64_t)plan[2 * (k / BLOCK)] + k % BLOCK; }
  __device__ __forceinline__ const T *ptr_k(int row, int k) const {   // stored [n][k]
    return (n0 + row < NF && k / BLOCK < nblk) ? base + (int64_t)(n0 + row) * ld + pos(k) : nullptr;
  }
  __device__ __forceinline__ const T *ptr_r(int row, int k) const {   // stored [k][n]
    return (n0 + row < NF && k / BLOCK < nblk) ? base + pos(k) * ld + n0 + row : nullptr;
  }
};

template <int BLOCK> struct XsdShape {
  static constexpr int TN = 64;
  static constexpr int WGM = BLOCK >= 32 ? 2 : 1;
  static constexpr int WGN = 4 / WGM;
};

template <typename T, int BLOCK, bool SP_TRANS, bool DN_KCONTIG, bool OUT_NCONTIG>
__global__ void __launch_bounds__(256) k_xsd(XsdArgs g) {
  typedef XsdShape<BLOCK> S;
  typedef TileGemm<T, BLOCK, S::TN, S::WGM, S::WGN, !SP_TRANS, DN_KCONTIG, OUT_NCONTIG> G;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int64_t per_z = (int64_t)g.width * g.n_tiles;
  const int64_t w = xcd_remap(blockIdx.x, per_z * g.Z);
  const int z = (int)(w / per_z);
  const int seg = (int)((w % per_z) / g.n_tiles);
  const int nt = (int)(w % g.n_tiles);
  const int32_t *hd = g.lut + 6 * (int64_t)seg;
  const int offset = hd[0], seglen = hd[1], column = hd[2], depth = hd[3];
  const int nblk = seglen / BLOCK;
  if (nblk == 0) {
    // The table carries zero-length segments.  One that stands alone is an empty row/column of the layout and
    // must zero-fill its output tile; one that follows a real segment of the same row/column must not touch it.
    if (seg > 0 && hd[-6 + 2] == column && hd[-6 + 3] == depth) return;
  }
  const int t0 = (offset - 6 * g.width) / g.div2;   // first block of the segment in table order
  SparseView<T, BLOCK, SP_TRANS> sv;
  sv.base = reinterpret_cast<const T *>(g.sp) + z * g.sp_sz; sv.plan = g.plan + 2 * (int64_t)t0; sv.nblk = nblk;
  DenseView<T, BLOCK> dv;
  dv.base = reinterpret_cast<const T *>(g.dn) + z * g.dn_sz + depth * g.dn_sh; dv.plan = sv.plan; dv.nblk = nblk; dv.ld = g.ldd;
  dv.n0 = nt * S::TN; dv.NF = g.NF;
  T *oz = reinterpret_cast<T *>(g.out) + z * g.out_sz + depth * g.out_sh;
  const int NF = g.NF, n0 = nt * S::TN;
  const int64_t ldo = g.ldo;
  auto store = [&](int m, int n, f32x4 v) {
    if (n0 + n >= NF) return;
    if constexpr (OUT_NCONTIG) store4<T>(oz + ((int64_t)column * BLOCK + m) * ldo + n0 + n, v);
    else store4<T>(oz + (int64_t)(n0 + n) * ldo + column * BLOCK + m, v);
  };
  G::run(sv, dv, (nblk * BLOCK + G::TK - 1) / G::TK, reinterpret_cast<T *>(smem_raw), store);
}

// ---------------------------------------------------------------------------------------------------------
// host-side launch helpers shared by the per-type translation units
// ---------------------------------------------------------------------------------------------------------
template <typename T, int BLOCK, int PACK> int launch_sdd_tp(const SddArgs &g, bool a_kc, bool b_kc, hipStream_t st) {
  constexpr int TT = BLOCK * PACK, WG = SddShape<TT>::WG;
  const int64_t n_wg = g.n_groups * g.Z;
  if (n_wg <= 0) return BSP_OK;
  if (n_wg >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  dim3 grid((unsigned)n_wg), blockdim(64 * WG * WG);
#define BSP_SDD_LAUNCH(AK, BK)                                                                                   \
  hipLaunchKernelGGL((k_sdd<T, BLOCK, PACK, AK, BK>), grid, blockdim,                                           \
                     (TileGemm<T, TT, TT, WG, WG, AK, BK, true>::SMEM_BYTES), st, g)
  if (a_kc && b_kc) BSP_SDD_LAUNCH(true, true);
  else if (a_kc && !b_kc) BSP_SDD_LAUNCH(true, false);
  else if (!a_kc && b_kc) BSP_SDD_LAUNCH(false, true);
  else BSP_SDD_LAUNCH(false, false);
#undef BSP_SDD_LAUNCH
  return BSP_OK;
}

template <typename T> int launch_sdd(const SddArgs &g, int block, int pack, bool a_kc, bool b_kc, hipStream_t st) {
  if (block == 16 && pack == 4) return launch_sdd_tp<T, 16, 4>(g, a_kc, b_kc, st);
  if (block == 16 && pack == 2) return launch_sdd_tp<T, 16, 2>(g, a_kc, b_kc, st);
  if (block == 16 && pack == 1) return launch_sdd_tp<T, 16, 1>(g, a_kc, b_kc, st);
  if (block == 32 && pack == 2) return launch_sdd_tp<T, 32, 2>(g, a_kc, b_kc, st);
  if (block == 32 && pack == 1) return launch_sdd_tp<T, 32, 1>(g, a_kc, b_kc, st);
  if (block == 64 && pack == 1) return launch_sdd_tp<T, 64, 1>(g, a_kc, b_kc, st);
  if (block == 128 && pack == 1) return launch_sdd_tp<T, 128, 1>(g, a_kc, b_kc, st);
  return BSP_ERR_UNSUPPORTED;
}

template <typename T, int BLOCK> int launch_xsd_b(const XsdArgs &g, bool sp_trans, bool dn_kc, bool out_nc, hipStream_t st) {
  typedef XsdShape<BLOCK> S;
  const int64_t n_wg = (int64_t)g.width * g.n_tiles * g.Z;
  if (n_wg <= 0) return BSP_OK;
  if (n_wg >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  dim3 grid((unsigned)n_wg), blockdim(256);
#define BSP_XSD_LAUNCH(ST, DK, ON)                                                                               \
  hipLaunchKernelGGL((k_xsd<T, BLOCK, ST, DK, ON>), grid, blockdim,                                             \
                     (TileGemm<T, BLOCK, S::TN, S::WGM, S::WGN, !ST, DK, ON>::SMEM_BYTES), st, g)
  const int key = (sp_trans ? 4 : 0) | (dn_kc ? 2 : 0) | (out_nc ? 1 : 0);
  switch (key) {
    case 0: BSP_XSD_LAUNCH(false, false, false); break;
    case 1: BSP_XSD_LAUNCH(false, false, true); break;
    case 2: BSP_XSD_LAUNCH(false, true, false); break;
    case 3: BSP_XSD_LAUNCH(false, true, true); break;
    case 4: BSP_XSD_LAUNCH(true, false, false); break;
    case 5: BSP_XSD_LAUNCH(true, false, true); break;
    case 6: BSP_XSD_LAUNCH(true, true, false); break;
    default: BSP_XSD_LAUNCH(true, true, true); break;
  }
#undef BSP_XSD_LAUNCH
  return BSP_OK;
}

template <typename T> int launch_xsd(const XsdArgs &g, int block, bool sp_trans, bool dn_kc, bool out_nc, hipStream_t st) {
  switch (block) {
    case 16: return launch_xsd_b<T, 16>(g, sp_trans, dn_kc, out_nc, st);
    case 32: return launch_xsd_b<T, 32>(g, sp_trans, dn_kc, out_nc, st);
    case 64: return launch_xsd_b<T, 64>(g, sp_trans, dn_kc, out_nc, st);
    case 128: return launch_xsd_b<T, 128>(g, sp_trans, dn_kc, out_nc, st);
    default: return BSP_ERR_UNSUPPORTED;
  }
}

// implemented once per element type (matmul_f16.hip, matmul_bf16.hip, matmul_f32.hip)
int sdd_generic_f16(const SddArgs &g, int block, int pack, bool a_kc, bool b_kc, hipStream_t st);
int sdd_generic_bf16(const SddArgs &g, int block, int pack, bool a_kc, bool b_kc, hipStream_t st);
int sdd_generic_f32(const SddArgs &g, int block, int pack, bool a_kc, bool b_kc, hipStream_t st);
int xsd_generic_f16(const XsdArgs &g, int block, bool sp_trans, bool dn_kc, bool out_nc, hipStream_t st);
int xsd_generic_bf16(const XsdArgs &g, int block, bool sp_trans, bool dn_kc, bool out_nc, hipStream_t st);
int xsd_generic_f32(const XsdArgs &g, int block, bool sp_trans, bool dn_kc, bool out_nc, hipStream_t st);


// specialised block-64 16-bit kernels (matmul_fast64.hip): 1 = launched, 0 = not applicable, < 0 = error
int sdd_fast64(int dtype, const SddArgs &g, int block, int pack, bool a_kc, bool b_kc, hipStream_t st);
int xsd_fast64(int dtype, const XsdArgs &g, int block, bool sp_trans, bool dn_kc, bool out_nc, hipStream_t st);

}  // namespace bsp
