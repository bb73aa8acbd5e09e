// Bandwidth-oriented kernels for the attention shapes: fp16 / bf16, dense operands with a unit stride along the
// head dimension (64 or 128).  At head_dim 64 every product of the sdd -> softmax -> dsd chain moves ~400 MB for
// 17 GFLOP (43 flop/byte), i.e. it is bound by HBM, not by the matrix cores; these kernels are organised around
// keeping many 16-byte loads in flight and touching every byte once.  (The file began with block 64 only, hence its
// name; blocks 16 and 32 have their own kernels below.)
//
//   row-group kernels (need a group plan, see bsp_group_plan_build):
//   k_sdd64_rg, k_xsd64_rg        : block 64.  A workgroup owns 4 consecutive block-rows (or -columns) of a head; each
//                                   wavefront computes 16 rows of every member; chains split over the wavefronts.
//   k_sdd_rg_small, k_xsd_rg_small: blocks 16 and 32.  Same plan, one wavefront per member.
//
//   without a plan (block 64):
//   k_sdd64_nt : C_blk = A[i-rows, :K] . B[j-rows, :K]^T.  One wavefront per output block.  Both operands
//                have the reduction dimension contiguous, which is exactly the MFMA operand layout (a lane
//                owns one row and 8 consecutive reduction indices), so they go from global memory straight
//                into the operand registers: no LDS, no barrier.
//   k_xsd64    : out[64 rows of one table segment, 64 columns] = sum over the segment's blocks
//                S_t . D[pos_t : pos_t + 64, n0 : n0 + 64].  D is stored with the reduction dimension strided,
//                and so is S when it is read transposed (the dV / dK products); those tiles are staged in LDS
//                as they lie in memory and read back with the transposing LDS load of gfx950
//                (ds_read_b64_tr_b16), which hands each lane 4 reduction-consecutive values of its column.
//                Four wavefronts per workgroup, each owning 16 output rows; global loads run four blocks
//                ahead of the MFMAs in a register ring.
#include "matmul_generic.h"
#include <type_traits>

namespace bsp {
namespace {

template <typename T> struct Mma32;   // 32x32x16: lane l supplies row l % 32, reduction indices 8 * (l / 32) + j
template <> struct Mma32<f16> {
  typedef f16x8 frag_t;
  static __device__ __forceinline__ f32x16 run(frag_t a, frag_t b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};
template <> struct Mma32<bf16> {
  typedef bf16x8 frag_t;
  static __device__ __forceinline__ f32x16 run(frag_t a, frag_t b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};

constexpr int kLdsRow = 72;     // elements per LDS tile row: 64 + 8 (144 bytes, keeps 16-byte alignment)
constexpr int kRing = 4;        // blocks in flight per workgroup

template <typename T> __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  union { T h[2]; uint32_t u; } p;
  p.h[0] = from_float<T>(lo);
  p.h[1] = from_float<T>(hi);
  return p.u;
}

// ---------------------------------------------------------------------------------------------------------
// sdd, block 64, A and B both with the reduction dimension contiguous ("NT"), K a multiple of 64
// ---------------------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256) k_sdd64_nt(SddArgs g) {
  typedef Mma32<T> M;
  typedef typename M::frag_t frag_t;
  const int64_t n_items = g.n_groups * g.Z;
  const int64_t n_wg = (n_items + 3) >> 2;
  const int64_t item = xcd_remap(blockIdx.x, n_wg) * 4 + (threadIdx.x >> 6);
  if (item >= n_items) return;
  const int lane = threadIdx.x & 63;
  const int z = (int)(item / g.n_groups);
  const int64_t grp = item % g.n_groups;
  if (g.valid && !g.valid[grp]) return;
  const int32_t *e = g.lut + grp * 4;
  const int h = e[0], bi = e[1], bj = e[2];
  const int64_t bk = e[3];
  // lane's operand rows: r and r + 32 of the block-row (A) / block-column (B); its reduction offset inside a step
  const int r = lane & 31, kq = (lane >> 5) * 8;
  const T *pa = reinterpret_cast<const T *>(g.a) + z * g.a_sz + h * g.a_sh + ((int64_t)bi * 64 + r) * g.lda + kq;
  const T *pb = reinterpret_cast<const T *>(g.b) + z * g.b_sz + h * g.b_sh + ((int64_t)bj * 64 + r) * g.ldb + kq;
  const int64_t a32 = 32 * g.lda, b32 = 32 * g.ldb;
  f32x16 acc[2][2];   // [tn][tm]: rows n of the 32x32 result come from B, columns m from A
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;
  for (int k0 = 0; k0 < g.K; k0 += 64) {
    frag_t fa[2][4], fb[2][4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
      fa[0][s] = *reinterpret_cast<const frag_t *>(pa + k0 + 16 * s);
      fa[1][s] = *reinterpret_cast<const frag_t *>(pa + a32 + k0 + 16 * s);
      fb[0][s] = *reinterpret_cast<const frag_t *>(pb + k0 + 16 * s);
      fb[1][s] = *reinterpret_cast<const frag_t *>(pb + b32 + k0 + 16 * s);
    }
#pragma unroll
    for (int s = 0; s < 4; s++)
#pragma unroll
      for (int tn = 0; tn < 2; tn++)
#pragma unroll
        for (int tm = 0; tm < 2; tm++) acc[tn][tm] = M::run(fb[tn][s], fa[tm][s], acc[tn][tm]);
  }
  // Result element v = 4*gq + e of tile (tn, tm) is C[m = 32*tm + r][n = 32*tn + 8*gq + 4*(lane/32) + e].
  // Exchanging the upper half-wave's values of group gq = 2a with the lower half-wave's of gq = 2a+1 leaves every
  // lane with 8 consecutive n (16 bytes).  The tile then goes through a wave-private LDS buffer so that each store
  // instruction writes 8 whole rows of the block: 1 KiB of consecutive addresses instead of 32-byte pieces.
  __shared__ __attribute__((aligned(16))) T Cs[4][64 * kLdsRow];
  T *cs = Cs[threadIdx.x >> 6];
#pragma unroll
  for (int tn = 0; tn < 2; tn++)
#pragma unroll
    for (int tm = 0; tm < 2; tm++)
#pragma unroll
      for (int a = 0; a < 2; a++) {
        const f32x16 &c = acc[tn][tm];
        uint32_t p0 = pack2<T>(c[8 * a + 0], c[8 * a + 1]), p1 = pack2<T>(c[8 * a + 2], c[8 * a + 3]);
        uint32_t q0 = pack2<T>(c[8 * a + 4], c[8 * a + 5]), q1 = pack2<T>(c[8 * a + 6], c[8 * a + 7]);
        auto x = __builtin_amdgcn_permlane32_swap(p0, q0, false, false);
        auto y = __builtin_amdgcn_permlane32_swap(p1, q1, false, false);
        u32x4 out = {x[0], y[0], x[1], y[1]};
        *reinterpret_cast<u32x4 *>(cs + (32 * tm + r) * kLdsRow + 32 * tn + 16 * a + (lane >> 5) * 8) = out;
      }
  __builtin_amdgcn_wave_barrier();   // LDS operations of one wavefront complete in order; this only pins the code order
  T *pc = reinterpret_cast<T *>(g.c) + z * g.c_sz + bk * 4096 + lane * 8;
  const T *rs = cs + (lane >> 3) * kLdsRow + (lane & 7) * 8;
#pragma unroll
  for (int i = 0; i < 8; i++)
    *reinterpret_cast<u32x4 *>(pc + i * 512) = *reinterpret_cast<const u32x4 *>(rs + i * 8 * kLdsRow);
}

// ---------------------------------------------------------------------------------------------------------
// xsd, block 64, dense operand and output with the free dimension contiguous
// ---------------------------------------------------------------------------------------------------------
template <typename T> __device__ __forceinline__ typename Mma16<T>::frag_t tr_frag(const T *p_lo, const T *p_hi) {
  // two transposing reads: reduction indices 0..3 and 4..7 of this lane's column
  typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)p_lo);
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)p_hi);
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(typename Mma16<T>::frag_t, v);
}

template <typename T, bool SP_TRANS>
__global__ void __launch_bounds__(256) k_xsd64(XsdArgs g) {
  typedef Mma16<T> M;
  typedef typename M::frag_t frag_t;
  constexpr int TILE = 64 * kLdsRow;
  __shared__ __attribute__((aligned(16))) T Ys[2][TILE];
  __shared__ __attribute__((aligned(16))) T Xs[SP_TRANS ? 2 : 1][SP_TRANS ? TILE : 8];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t per_z = (int64_t)g.width * g.n_tiles;
  const int64_t w = xcd_remap(blockIdx.x, per_z * g.Z);
  const int z = (int)(w / per_z);
  const int seg = (int)((w % per_z) / g.n_tiles);
  const int n0 = (int)(w % g.n_tiles) * 64;
  const table_ptr hd = as_table(g.lut) + 6 * (int64_t)seg;
  const int offset = hd[0], seglen = hd[1], column = hd[2], depth = hd[3];
  const int nblk = seglen >> 6;
  if (nblk == 0 && seg > 0 && hd[-4] == column && hd[-3] == depth) return;   // see k_xsd: empty twin of a real segment
  const table_ptr plan = as_table(g.plan) + 2 * (int64_t)((offset - 6 * g.width) / g.div2);
  const T *sp = reinterpret_cast<const T *>(g.sp) + z * g.sp_sz;
  const T *dn = reinterpret_cast<const T *>(g.dn) + z * g.dn_sz + depth * g.dn_sh + n0;
  const int64_t ldd = g.ldd;

  // cooperative tile loads: thread handles 16-byte chunks (row tid/8, column-chunk tid%8) and the same 32 rows below
  const int ck = tid >> 3, cc = (tid & 7) * 8;
  // direct X operand (not transposed): lane owns row 16*wave + lane%16 of the block, reduction offset 8*(lane/16)
  const int xr = wave * 16 + (lane & 15), xq = (lane >> 4) * 8;

  struct Stage { u32x4 y[2]; u32x4 x[2]; };
  Stage ring[kRing];
  auto issue = [&](Stage &st, int b) {
    const int64_t pos = plan[2 * b];
    const T *blk = sp + (int64_t)plan[2 * b + 1] * 4096;
    const T *py = dn + (pos + ck) * ldd + cc;
    st.y[0] = *reinterpret_cast<const u32x4 *>(py);
    st.y[1] = *reinterpret_cast<const u32x4 *>(py + 32 * ldd);
    if constexpr (SP_TRANS) {
      st.x[0] = *reinterpret_cast<const u32x4 *>(blk + ck * 64 + cc);
      st.x[1] = *reinterpret_cast<const u32x4 *>(blk + (ck + 32) * 64 + cc);
    } else {
      st.x[0] = *reinterpret_cast<const u32x4 *>(blk + xr * 64 + xq);
      st.x[1] = *reinterpret_cast<const u32x4 *>(blk + xr * 64 + 32 + xq);
    }
  };

  f32x4 acc[4];
#pragma unroll
  for (int j = 0; j < 4; j++) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
  for (int u = 0; u < kRing; u++)
    if (u < nblk) issue(ring[u], u);

  // transposing-read addresses: within a 16-lane group, lane t points at row (t / 4), 4-element piece (t % 4);
  // the group then receives, per lane i, the 4 rows' values of column i.
  const int tr_row = (lane >> 4) * 8 + ((lane & 15) >> 2), tr_col = (lane & 3) * 4;

  for (int b0 = 0; b0 < nblk; b0 += kRing) {
#pragma unroll
    for (int u = 0; u < kRing; u++) {
      const int b = b0 + u;
      if (b < nblk) {
        const int buf = b & 1;
        Stage &st = ring[u];
        *reinterpret_cast<u32x4 *>(&Ys[buf][ck * kLdsRow + cc]) = st.y[0];
        *reinterpret_cast<u32x4 *>(&Ys[buf][(ck + 32) * kLdsRow + cc]) = st.y[1];
        frag_t xf[2];
        if constexpr (SP_TRANS) {
          *reinterpret_cast<u32x4 *>(&Xs[buf][ck * kLdsRow + cc]) = st.x[0];
          *reinterpret_cast<u32x4 *>(&Xs[buf][(ck + 32) * kLdsRow + cc]) = st.x[1];
        } else {
          xf[0] = __builtin_bit_cast(frag_t, st.x[0]);
          xf[1] = __builtin_bit_cast(frag_t, st.x[1]);
        }
        if (b + kRing < nblk) issue(st, b + kRing);
        __syncthreads();
#pragma unroll
        for (int s = 0; s < 2; s++) {
          const T *yrow = &Ys[buf][(32 * s + tr_row) * kLdsRow + tr_col];
          if constexpr (SP_TRANS) {
            const T *xrow = &Xs[buf][(32 * s + tr_row) * kLdsRow + 16 * wave + tr_col];
            xf[s] = tr_frag<T>(xrow, xrow + 4 * kLdsRow);
          }
#pragma unroll
          for (int j = 0; j < 4; j++) {
            frag_t yf = tr_frag<T>(yrow + 16 * j, yrow + 16 * j + 4 * kLdsRow);
            acc[j] = M::run(yf, xf[s], acc[j]);   // result rows = n (16*j + 4*(lane/16) + e), column = m (lane%16)
          }
        }
      }
    }
  }
  // Epilogue through LDS (each wavefront its own 16 rows of the first tile buffer, free after the last barrier
  // below): lanes then store 16 bytes each, 8 lanes per output row, whole 128-byte lines.
  __syncthreads();
  T *cs = &Ys[0][(wave * 16) * kLdsRow];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    union { u32x2 raw; T e[4]; } pk;
#pragma unroll
    for (int e = 0; e < 4; e++) pk.e[e] = from_float<T>(acc[j][e]);
    *reinterpret_cast<u32x2 *>(cs + (lane & 15) * kLdsRow + 16 * j + 4 * (lane >> 4)) = pk.raw;
  }
  __builtin_amdgcn_wave_barrier();
  T *po = reinterpret_cast<T *>(g.out) + z * g.out_sz + depth * g.out_sh + ((int64_t)column * 64 + wave * 16 + (lane >> 3)) * g.ldo +
          n0 + (lane & 7) * 8;
  const T *rs = cs + (lane >> 3) * kLdsRow + (lane & 7) * 8;
#pragma unroll
  for (int i = 0; i < 2; i++)
    *reinterpret_cast<u32x4 *>(po + (int64_t)i * 8 * g.ldo) = *reinterpret_cast<const u32x4 *>(rs + i * 8 * kLdsRow);
}

// ---------------------------------------------------------------------------------------------------------
// Row-group kernels.  A workgroup owns BSP_GROUP consecutive block-rows (or block-columns) of one head and walks
// the entries of its group plan: every entry is one dense tile that at least one member needs.  The tile is
// fetched once, with whole-line loads, into LDS and serves all members, so the L2-level reads of the shared
// operand drop by the average number of members per entry (3.4x on the fixed attention layout) and each LDS
// operand read feeds up to four MFMAs.  Each wavefront computes 16 rows of every member.
// Workgroup w: batch z = w % Z (one batch per XCD when Z = 8), plan group w / Z in the plan's
// longest-first order.
// ---------------------------------------------------------------------------------------------------------
constexpr int G = BSP_GROUP;
constexpr int kGroupRing = 2;   // register stages of k_xsd64_rg (three were measured 5-8 % slower)

// Plans over 64 x 64 tiles of a block-16 / block-32 layout (SUBS = 64 / block per side): an entry is (position, G tile
// flags, G x SUBS*SUBS ids of the small blocks, -1 where absent).  The kernels below then fetch a tile's rows from the
// small blocks that hold them: `ids` = the SUBS ids of one row of small blocks (scalar), sc = the lane's column of
// small blocks, (r_in, c_in) = the element inside the small block.  An absent block reads zeros.
__device__ __attribute__((aligned(16))) const uint32_t kZeroChunk[4] = {0u, 0u, 0u, 0u};
template <int SUBS> constexpr int plan_entry_ints() { return SUBS == 1 ? G + 1 : 1 + G + G * SUBS * SUBS; }
template <typename T, int SUBS>
__device__ __forceinline__ const T *sub_block_ptr(const T *sp, table_ptr ids, int sc, int r_in, int c_in) {
  constexpr int BLKF = 64 / SUBS;
  int id = ids[0];
#pragma unroll
  for (int k = 1; k < SUBS; k++) id = sc == k ? ids[k] : id;
  const T *p = sp + (int64_t)id * (BLKF * BLKF) + r_in * BLKF + c_in;
  return id >= 0 ? p : reinterpret_cast<const T *>(kZeroChunk);
}

// STREAM: the slice belongs to a dense result, which nothing in the sparse chain reads again: written with streaming
// stores it does not displace the sparse tensors that the next launches re-read from the memory-side cache
// (measured on the attention step: 8-9 us less for two of the four dsd/dds launches, 1-2 us for the others; the same
// hint on the sparse result of sdd, which the next launch does read, costs 10-25 % of the sdd).
template <typename T, bool STREAM = false> __device__ __forceinline__ void store_slice(T *cs, T *dst, int64_t ld, const f32x4 (&acc)[4], int lane) {
  // acc[j][e] = out[row lane%16][col 16*j + 4*(lane/16) + e] of a 16 x 64 slice -> LDS -> two stores of 8 whole rows
#pragma unroll
  for (int j = 0; j < 4; j++) {
    union { u32x2 raw; T e[4]; } pk;
#pragma unroll
    for (int e = 0; e < 4; e++) pk.e[e] = from_float<T>(acc[j][e]);
    *reinterpret_cast<u32x2 *>(cs + (lane & 15) * kLdsRow + 16 * j + 4 * (lane >> 4)) = pk.raw;
  }
  __builtin_amdgcn_wave_barrier();
  const T *rs = cs + (lane >> 3) * kLdsRow + (lane & 7) * 8;
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const u32x4 v = *reinterpret_cast<const u32x4 *>(rs + i * 8 * kLdsRow);
    u32x4 *o = reinterpret_cast<u32x4 *>(dst + ((lane >> 3) + 8 * i) * ld + (lane & 7) * 8);
    if constexpr (STREAM) __builtin_nontemporal_store(v, o);
    else *o = v;
  }
  __builtin_amdgcn_wave_barrier();
}

// The same slice scattered to the four small blocks (16 x 16) of one row of a tile: ids = their block ids (-1: absent,
// nothing stored); a store instruction writes 8 rows = 256 contiguous bytes of each.
template <typename T> __device__ __forceinline__ void store_slice_sub16(T *cs, T *c, table_ptr ids, const f32x4 (&acc)[4], int lane) {
#pragma unroll
  for (int j = 0; j < 4; j++) {
    union { u32x2 raw; T e[4]; } pk;
#pragma unroll
    for (int e = 0; e < 4; e++) pk.e[e] = from_float<T>(acc[j][e]);
    *reinterpret_cast<u32x2 *>(cs + (lane & 15) * kLdsRow + 16 * j + 4 * (lane >> 4)) = pk.raw;
  }
  __builtin_amdgcn_wave_barrier();
  const int sc = (lane & 7) >> 1;
  int id = ids[0];
#pragma unroll
  for (int k = 1; k < 4; k++) id = sc == k ? ids[k] : id;
  const T *rs = cs + (lane >> 3) * kLdsRow + (lane & 7) * 8;
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const u32x4 v = *reinterpret_cast<const u32x4 *>(rs + i * 8 * kLdsRow);
    if (id >= 0) *reinterpret_cast<u32x4 *>(c + (int64_t)id * 256 + ((lane >> 3) + 8 * i) * 16 + (lane & 1) * 8) = v;
  }
  __builtin_amdgcn_wave_barrier();
}

// sdd, K = KD (64 or 128): members = block-rows of A (their 16-row slices stay in registers), entries = block-columns
// (B tiles of 64 rows x KD)
template <typename T, int KD, bool STREAM, int SUBS = 1>
__device__ __forceinline__ void sdd64_rg_body(const SddArgs &g, T *smem) {
  typedef Mma16<T> M;
  typedef typename M::frag_t frag_t;
  constexpr int ENT = plan_entry_ints<SUBS>();   // SUBS = 4: a plan over 64 x 64 tiles of a block-16 layout, the result tile is scattered
  static_assert(SUBS == 1 || SUBS == 4, "tiles of whole blocks or of 4 x 4 blocks of 16");
  constexpr int NK = KD / 32;                    // MFMA steps along the reduction
  constexpr int LDK = KD + 8;                    // LDS row of a B tile
  constexpr int TILE = 64 * LDK;
  constexpr int CPR = KD / 8, NL = 64 * CPR / 256;   // 16-byte chunks per row, loads per thread and tile
  T (*Ks)[TILE] = reinterpret_cast<T (*)[TILE]>(smem);                              // two B tiles
  T (*Cs)[16 * kLdsRow] = reinterpret_cast<T (*)[16 * kLdsRow]>(smem + 2 * TILE);   // a 16-row staging slice per wavefront
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int z = blockIdx.x % g.Z;
  const table_ptr hd = as_table(g.gplan) + 4 * (int64_t)(blockIdx.x / g.Z);
  const int e0 = hd[0], ne = hd[1], h = hd[2], lg = hd[3] & 0xffffff;
  const table_ptr ent = as_table(g.gplan) + 4 * (int64_t)g.n_pgroups + (int64_t)ENT * e0;
  const int r = lane & 15, kq = (lane >> 4) * 8;
  const T *pa = reinterpret_cast<const T *>(g.a) + z * g.a_sz + h * g.a_sh;
  const T *pb = reinterpret_cast<const T *>(g.b) + z * g.b_sz + h * g.b_sh;
  T *pc = reinterpret_cast<T *>(g.c) + z * g.c_sz;
  frag_t xq[G][NK];
#pragma unroll
  for (int m = 0; m < G; m++) {
    const int row = lg * G + m;
    if (row < g.lines) {
      const T *p = pa + ((int64_t)row * 64 + wave * 16 + r) * g.lda + kq;
#pragma unroll
      for (int s2 = 0; s2 < NK; s2++) xq[m][s2] = *reinterpret_cast<const frag_t *>(p + 32 * s2);
    }
  }
  struct Stage { u32x4 y[NL]; };
  Stage ring[kRing];
  auto issue = [&](Stage &st, int e) {
    const T *py = pb + (int64_t)ent[ENT * e] * 64 * g.ldb;
#pragma unroll
    for (int i = 0; i < NL; i++) {
      const int c = tid + 256 * i;
      // streaming loads where the plan says so: tiles that few groups want, kept out of the memory-side cache, leave
      // it to the sparse result that the next launch reads (measured: 3-4 us per launch on the fixed attention layout)
      const u32x4 *pt = reinterpret_cast<const u32x4 *>(py + (int64_t)(c / CPR) * g.ldb + (c % CPR) * 8);
      if constexpr (STREAM) st.y[i] = __builtin_nontemporal_load(pt);
      else st.y[i] = *pt;
    }
  };
#pragma unroll
  for (int u = 0; u < kRing; u++)
    if (u < ne) issue(ring[u], u);
  for (int e0i = 0; e0i < ne; e0i += kRing) {
#pragma unroll
    for (int u = 0; u < kRing; u++) {
      const int e = e0i + u;
      if (e < ne) {
        const int buf = e & 1;
#pragma unroll
        for (int i = 0; i < NL; i++) {
          const int c = tid + 256 * i;
          *reinterpret_cast<u32x4 *>(&Ks[buf][(c / CPR) * LDK + (c % CPR) * 8]) = ring[u].y[i];
        }
        if (e + kRing < ne) issue(ring[u], e + kRing);
        __syncthreads();
        frag_t yf[4][NK];
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
          for (int s2 = 0; s2 < NK; s2++) yf[j][s2] = *reinterpret_cast<const frag_t *>(&Ks[buf][(16 * j + r) * LDK + 32 * s2 + kq]);
#pragma unroll
        for (int m = 0; m < G; m++) {
          const int bid = ent[ENT * e + 1 + m];
          if (bid >= 0) {
            f32x4 acc[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
              acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
              for (int s2 = 0; s2 < NK; s2++) acc[j] = M::run(yf[j][s2], xq[m][s2], acc[j]);   // rows n = 16j + 4*(lane/16) + e, column m-row = lane%16
            }
            if constexpr (SUBS == 1) store_slice<T>(Cs[wave], pc + (int64_t)bid * 4096 + wave * 1024, 64, acc, lane);
            else store_slice_sub16<T>(Cs[wave], pc, ent + ENT * e + 1 + G + m * 16 + wave * 4, acc, lane);
          }
        }
      }
    }
  }
}

// The streaming hint is a property of the whole plan (bit 28 of every group's index field), so all workgroups of a
// launch take the same side of this branch.  Two copies of the body rather than a condition at the load: the
// compiler merges two loads of one address that differ only in the hint, and drops the hint.
template <typename T, int KD, int SUBS = 1>
__global__ void __launch_bounds__(256) k_sdd64_rg(SddArgs g) {
  __shared__ __attribute__((aligned(16))) T smem[2 * 64 * (KD + 8) + 4 * 16 * kLdsRow];
  const int code = as_table(g.gplan)[4 * (int64_t)(blockIdx.x / g.Z) + 3];
  if ((code >> 28) & 1) sdd64_rg_body<T, KD, true, SUBS>(g, smem);
  else sdd64_rg_body<T, KD, false, SUBS>(g, smem);
}

// A chain = one output line with many blocks (the plan builder takes such lines out of their groups).  Walking its
// entries one after the other would make this workgroup the last to finish by far, so the four wavefronts split
// the reduction instead: wavefront w takes entries w, w+4, ... and computes all 64 rows of the line for them, in its
// own piece of LDS and without workgroup barriers; the four partial results are added through LDS at the end.
template <typename T, bool SP_TRANS, int SUBS = 1>
__device__ __forceinline__ void xsd_chain(const XsdArgs &g, T *smem, int z, int n0, int depth, int line, table_ptr ent, int ne,
                                          int part, int parts, int seq) {
  constexpr int ENT = plan_entry_ints<SUBS>(), BLKF = 64 / SUBS;
  typedef Mma16<T> M;
  typedef typename M::frag_t frag_t;
  constexpr int TILE = 64 * kLdsRow;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const T *sp = reinterpret_cast<const T *>(g.sp) + z * g.sp_sz;
  const T *dn = reinterpret_cast<const T *>(g.dn) + z * g.dn_sz + depth * g.dn_sh + n0;
  const int64_t ldd = g.ldd;
  T *Yw = smem + wave * TILE;
  T *Xw = smem + (4 + wave) * TILE;              // used only when the sparse operand is read transposed
  const int lr = lane >> 3, lc = (lane & 7) * 8;  // a lane's row (of 8) and 16-byte column chunk in a 64 x 64 tile
  u32x4 y[8], x[8];
  auto issue = [&](int e) {
    const table_ptr en = ent + ENT * e;
    const T *py = dn + ((int64_t)en[0] * 64 + lr) * ldd + lc;
#pragma unroll
    for (int i = 0; i < 8; i++) y[i] = *reinterpret_cast<const u32x4 *>(py + (int64_t)i * 8 * ldd);
    if constexpr (SUBS == 1) {
      const T *blk = sp + (int64_t)en[1] * 4096;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        if constexpr (SP_TRANS) x[i] = *reinterpret_cast<const u32x4 *>(blk + (i * 8 + lr) * 64 + lc);   // as stored, [k][m]
        else x[i] = *reinterpret_cast<const u32x4 *>(blk + ((i >> 1) * 16 + (lane & 15)) * 64 + 32 * (i & 1) + (lane >> 4) * 8);   // operand layout
      }
    } else {
      const table_ptr ids = en + 1 + G;            // member 0 = the line
#pragma unroll
      for (int i = 0; i < 8; i++) {
        // the same elements of the tile as above (whole rows of 8 lanes when transposed: 256 contiguous bytes per small
        // block and load; else the operand layout, which walks a small block with consecutive lanes); the row of
        // small blocks is the same for all lanes of a load
        const int row0 = SP_TRANS ? i * 8 : (i >> 1) * 16;                       // the part of the row all lanes share
        const int row = SP_TRANS ? row0 + lr : row0 + (lane & 15);
        const int col = SP_TRANS ? lc : 32 * (i & 1) + (lane >> 4) * 8;
        x[i] = *reinterpret_cast<const u32x4 *>(sub_block_ptr<T, SUBS>(sp, ids + (row0 / BLKF) * SUBS, col / BLKF, row % BLKF, col % BLKF));
      }
    }
  };
  f32x4 acc[4][4];
#pragma unroll
  for (int mt = 0; mt < 4; mt++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[mt][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int tr_row = (lane >> 4) * 8 + ((lane & 15) >> 2), tr_col = (lane & 3) * 4;
  const int mine = (ne - wave + 3) / 4;          // entries wave, wave + 4, ...
  if (mine > 0) issue(wave);
  for (int k = 0; k < mine; k++) {
#pragma unroll
    for (int i = 0; i < 8; i++) *reinterpret_cast<u32x4 *>(&Yw[(i * 8 + lr) * kLdsRow + lc]) = y[i];
    frag_t xf[4][2];
    if constexpr (SP_TRANS) {
#pragma unroll
      for (int i = 0; i < 8; i++) *reinterpret_cast<u32x4 *>(&Xw[(i * 8 + lr) * kLdsRow + lc]) = x[i];
    } else {
#pragma unroll
      for (int i = 0; i < 8; i++) xf[i >> 1][i & 1] = __builtin_bit_cast(frag_t, x[i]);
    }
    // the LDS operations of one wavefront complete in order: no barrier between its own stores and loads
    __builtin_amdgcn_wave_barrier();
    frag_t yf[2][4];
#pragma unroll
    for (int s2 = 0; s2 < 2; s2++) {
      const T *yrow = &Yw[(32 * s2 + tr_row) * kLdsRow + tr_col];
#pragma unroll
      for (int j = 0; j < 4; j++) yf[s2][j] = tr_frag<T>(yrow + 16 * j, yrow + 16 * j + 4 * kLdsRow);
      if constexpr (SP_TRANS) {
#pragma unroll
        for (int mt = 0; mt < 4; mt++) {
          const T *xrow = &Xw[(32 * s2 + tr_row) * kLdsRow + 16 * mt + tr_col];
          xf[mt][s2] = tr_frag<T>(xrow, xrow + 4 * kLdsRow);
        }
      }
    }
    if (k + 1 < mine) issue(wave + 4 * (k + 1));   // the stage's registers are free again
#pragma unroll
    for (int mt = 0; mt < 4; mt++)
#pragma unroll
      for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[mt][j] = M::run(yf[s2][j], xf[mt][s2], acc[mt][j]);
    __builtin_amdgcn_wave_barrier();
  }
  // add the four partial results: two rounds of 32 floats per lane and wavefront through LDS, after which wavefront w
  // holds rows 16w.. of the line
  float *red = reinterpret_cast<float *>(smem);   // [wavefront][32][lane], 32 KiB
  f32x4 fin[4];
#pragma unroll
  for (int half = 0; half < 2; half++) {
    __syncthreads();
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int j = 0; j < 4; j++)
#pragma unroll
        for (int c = 0; c < 4; c++) red[(wave * 32 + (t * 4 + j) * 4 + c) * 64 + lane] = acc[2 * half + t][j][c];
    __syncthreads();
    if ((wave >> 1) == half) {
      const int t = wave & 1;
#pragma unroll
      for (int j = 0; j < 4; j++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
          float v = 0.f;
#pragma unroll
          for (int w = 0; w < 4; w++) v += red[(w * 32 + (t * 4 + j) * 4 + c) * 64 + lane];
          fin[j][c] = v;
        }
    }
  }
  __syncthreads();
  if (parts > 1) {
    // One part of a split chain: its sums go to the workspace as fp32, 16 bytes per lane in address order;
    // k_xsd_chain_sum, launched behind this kernel, adds the parts in part order and writes the line.
    const int64_t slot = ((int64_t)seq * g.n_tiles + n0 / 64) * g.Z + z;
    f32x4 *ws = reinterpret_cast<f32x4 *>(g.partials) + (slot * BSP_CHAIN_PARTS + part) * 1024;   // 1024 f32x4 = one 64 x 64 tile
#pragma unroll
    for (int j = 0; j < 4; j++) ws[(wave * 4 + j) * 64 + lane] = fin[j];
    return;
  }
  T *po = reinterpret_cast<T *>(g.out) + z * g.out_sz + depth * g.out_sh + n0;
  store_slice<T, true>(smem + (wave * 16) * kLdsRow, po + ((int64_t)line * 64 + wave * 16) * g.ldo, g.ldo, fin, lane);
}

// Second pass over the split chains of a plan: one workgroup per (header row, tile of the free dimension, batch); the
// rows that are part 0 of a split chain add the chain's partial tiles in part order and write the output line, all
// others leave at once.  A kernel of its own rather than a last-arriver epilogue: the kernel boundary orders the
// partial sums before their use without device-wide fences inside the product kernel (which cost more than this
// launch: a release fence writes the whole L2 of its XCD back), and the sum has one fixed order.
template <typename T>
__global__ void __launch_bounds__(256) k_xsd_chain_sum(XsdArgs g) {
  __shared__ __attribute__((aligned(16))) T stage[4 * 16 * kLdsRow];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int z = blockIdx.x % g.Z;
  const int64_t rest = blockIdx.x / g.Z;
  const int tile = (int)(rest % g.n_tiles);
  const table_ptr hd = as_table(g.gplan) + 4 * (rest / g.n_tiles);
  const int cnt = hd[1], code = hd[3];
  const int part = (cnt >> 20) & 63, parts = ((cnt >> 26) & 31) + 1;
  if (code >= 0 || parts == 1 || part != 0) return;
  const int depth = hd[2] & 0xffff, seq = hd[2] >> 16, line = -(code + 1);
  const int64_t slot = ((int64_t)seq * g.n_tiles + tile) * g.Z + z;
  const f32x4 *ws = reinterpret_cast<const f32x4 *>(g.partials) + (slot * BSP_CHAIN_PARTS) * 1024;
  f32x4 fin[4];
#pragma unroll
  for (int j = 0; j < 4; j++) fin[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int p = 0; p < parts; p++) {
#pragma unroll
    for (int j = 0; j < 4; j++) fin[j] += __builtin_nontemporal_load(ws + (int64_t)p * 1024 + (wave * 4 + j) * 64 + lane);
  }
  T *po = reinterpret_cast<T *>(g.out) + z * g.out_sz + depth * g.out_sh + tile * 64;
  store_slice<T, true>(stage + (wave * 16) * kLdsRow, po + ((int64_t)line * 64 + wave * 16) * g.ldo, g.ldo, fin, lane);
}

// dsd / dds: members = output lines (block-rows of the result), entries = positions of the reduction
template <typename T, bool SP_TRANS, bool STREAM, int SUBS = 1>
__device__ __forceinline__ void xsd64_rg_body(const XsdArgs &g, T *smem) {
  typedef Mma16<T> M;
  typedef typename M::frag_t frag_t;
  constexpr int TILE = 64 * kLdsRow;
  constexpr int ENT = plan_entry_ints<SUBS>(), BLKF = 64 / SUBS;
  constexpr int RING = kGroupRing;
  T (*Ys)[TILE] = reinterpret_cast<T (*)[TILE]>(smem);
  T (*Xs)[TILE] = reinterpret_cast<T (*)[TILE]>(smem + 2 * TILE);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  T *Xw = smem + 2 * TILE + wave * TILE;   // untransposed groups: this wavefront's slices, member m at Xw + m * 16 * kLdsRow
  const int z = blockIdx.x % g.Z;
  const int64_t rest = blockIdx.x / g.Z;
  const int n0 = (int)(rest % g.n_tiles) * 64;
  const table_ptr hd = as_table(g.gplan) + 4 * (rest / g.n_tiles);
  const int e0 = hd[0], ne = hd[1], depth = hd[2], code = hd[3];
  const table_ptr ent = as_table(g.gplan) + 4 * (int64_t)g.n_pgroups + (int64_t)ENT * e0;
  if (code < 0) {   // a chain: the line -(code + 1) on its own, or one part of it (see bsp_group_plan_build)
    xsd_chain<T, SP_TRANS, SUBS>(g, smem, z, n0, depth & 0xffff, -(code + 1), ent, ne & 0xfffff, (ne >> 20) & 63, ((ne >> 26) & 31) + 1,
                                 depth >> 16);
    return;
  }
  const int lg = code & 0xffffff, skip = (code >> 24) & 0xf;   // members whose line is a chain are left to that chain
  const T *sp = reinterpret_cast<const T *>(g.sp) + z * g.sp_sz;
  const T *dn = reinterpret_cast<const T *>(g.dn) + z * g.dn_sz + depth * g.dn_sh + n0;
  const int64_t ldd = g.ldd;
  const int ck = tid >> 3, cc = (tid & 7) * 8;
  const int xq = (lane >> 4) * 8;
  struct Stage { u32x4 y[2]; u32x4 x[G][2]; };
  Stage ring[RING];
  auto issue = [&](Stage &st, int e) {
    const table_ptr en = ent + ENT * e;
    const T *py = dn + ((int64_t)en[0] * 64 + ck) * ldd + cc;
    // streaming loads for the dense tiles where the plan says so (kept out of the memory-side cache: 6 us per launch
    // on the fixed attention layout)
    const u32x4 *q0 = reinterpret_cast<const u32x4 *>(py), *q1 = reinterpret_cast<const u32x4 *>(py + 32 * ldd);
    if constexpr (STREAM) { st.y[0] = __builtin_nontemporal_load(q0); st.y[1] = __builtin_nontemporal_load(q1); }
    else { st.y[0] = *q0; st.y[1] = *q1; }
    // A fixed number of loads per stage whatever the entry holds, so that the wait before a stage is consumed can
    // count exactly the loads issued after it (a data-dependent count would force a wait for everything in flight).
    // Absent members read one cache line at the start of the sparse tensor instead.
#pragma unroll
    for (int m = 0; m < G; m++) {
      const int bid = en[1 + m];
      const T *p0, *p1;
      if constexpr (SUBS == 1) {
        const T *blk = sp + (int64_t)(bid >= 0 ? bid : 0) * 4096;
        if constexpr (SP_TRANS) { p0 = blk + ck * 64 + cc; p1 = p0 + 32 * 64; }
        else { p0 = blk + (wave * 16 + (lane >> 3)) * 64 + (lane & 7) * 8; p1 = p0 + 8 * 64; }   // whole rows: 8 lanes per 128-byte line
      } else {
        // the same elements of the tile, from the small blocks that hold them (8 rows of a small block are 256
        // contiguous bytes at block 16); the row of small blocks is the same for a wavefront
        const table_ptr ids = en + 1 + G + m * (SUBS * SUBS);
        if constexpr (SP_TRANS) {
          const int r0 = __builtin_amdgcn_readfirstlane(ck / BLKF);
          p0 = sub_block_ptr<T, SUBS>(sp, ids + r0 * SUBS, cc / BLKF, ck % BLKF, cc % BLKF);
          p1 = sub_block_ptr<T, SUBS>(sp, ids + (r0 + 32 / BLKF) * SUBS, cc / BLKF, ck % BLKF, cc % BLKF);
        } else {
          const int c = (lane & 7) * 8;
          p0 = sub_block_ptr<T, SUBS>(sp, ids + ((wave * 16) / BLKF) * SUBS, c / BLKF, (wave * 16) % BLKF + (lane >> 3), c % BLKF);
          p1 = p0 + (p0 == reinterpret_cast<const T *>(kZeroChunk) ? 0 : 8 * BLKF);
        }
      }
      if (bid < 0) { p0 = sp; p1 = sp; }
      st.x[m][0] = *reinterpret_cast<const u32x4 *>(p0);
      st.x[m][1] = *reinterpret_cast<const u32x4 *>(p1);
    }
  };
  f32x4 acc[G][4];
#pragma unroll
  for (int m = 0; m < G; m++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[m][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int tr_row = (lane >> 4) * 8 + ((lane & 15) >> 2), tr_col = (lane & 3) * 4;
  if (ne > 0) {
    // Every vector-memory operation below is unconditional: the loop runs a whole number of ring rounds, prefetches
    // past the end re-read the last entry, and the padding steps mark all members absent.
    const int last = ne - 1;
#pragma unroll
    for (int u = 0; u < RING; u++) issue(ring[u], u < last ? u : last);
    const int steps = (ne + RING - 1) / RING * RING;
    for (int e0i = 0; e0i < steps; e0i += RING) {
#pragma unroll
      for (int u = 0; u < RING; u++) {
        const int e = e0i + u;
        const bool live = e < ne;
        const int buf = e & 1;
        Stage &st = ring[u];
        const table_ptr en = ent + ENT * (live ? e : last);
        int bid[G];
#pragma unroll
        for (int m = 0; m < G; m++) bid[m] = live ? en[1 + m] : -1;
        *reinterpret_cast<u32x4 *>(&Ys[buf][ck * kLdsRow + cc]) = st.y[0];
        *reinterpret_cast<u32x4 *>(&Ys[buf][(ck + 32) * kLdsRow + cc]) = st.y[1];
        frag_t xf[G][2];
        if constexpr (SP_TRANS) {
          // Two barriers per step: one tile per member, all written, then all read.  The first barrier keeps this
          // step's tile stores behind the previous step's reads (the dense tile has two buffers for that, the four
          // sparse tiles have not), the second one orders the stores before the reads.
          __syncthreads();
#pragma unroll
          for (int m = 0; m < G; m++)
            if (bid[m] >= 0) {
              *reinterpret_cast<u32x4 *>(&Xs[m][ck * kLdsRow + cc]) = st.x[m][0];
              *reinterpret_cast<u32x4 *>(&Xs[m][(ck + 32) * kLdsRow + cc]) = st.x[m][1];
            }
          __syncthreads();
#pragma unroll
          for (int m = 0; m < G; m++)
            if (bid[m] >= 0) {
#pragma unroll
              for (int s2 = 0; s2 < 2; s2++) {
                const T *xrow = &Xs[m][(32 * s2 + tr_row) * kLdsRow + 16 * wave + tr_col];
                xf[m][s2] = tr_frag<T>(xrow, xrow + 4 * kLdsRow);
              }
            }
        } else {
          // The wavefront's 16 rows of each block were fetched line by line (operand layout, one row per lane, costs
          // 7 % of the launch: neighbouring lanes then never share a cache line); its own piece of LDS turns them into
          // operand layout.  The LDS operations of one wavefront complete in order: no barrier of its own.
#pragma unroll
          for (int m = 0; m < G; m++)
            if (bid[m] >= 0) {
              T *xm = Xw + m * 16 * kLdsRow;
              *reinterpret_cast<u32x4 *>(xm + (lane >> 3) * kLdsRow + (lane & 7) * 8) = st.x[m][0];
              *reinterpret_cast<u32x4 *>(xm + (8 + (lane >> 3)) * kLdsRow + (lane & 7) * 8) = st.x[m][1];
            }
          __syncthreads();
#pragma unroll
          for (int m = 0; m < G; m++)
            if (bid[m] >= 0) {
              const T *xm = Xw + m * 16 * kLdsRow + (lane & 15) * kLdsRow + xq;
              xf[m][0] = *reinterpret_cast<const frag_t *>(xm);
              xf[m][1] = *reinterpret_cast<const frag_t *>(xm + 32);
            }
        }
        frag_t yf[2][4];
#pragma unroll
        for (int s2 = 0; s2 < 2; s2++) {
          const T *yrow = &Ys[buf][(32 * s2 + tr_row) * kLdsRow + tr_col];
#pragma unroll
          for (int j = 0; j < 4; j++) yf[s2][j] = tr_frag<T>(yrow + 16 * j, yrow + 16 * j + 4 * kLdsRow);
        }
#pragma unroll
        for (int m = 0; m < G; m++)
          if (bid[m] >= 0) {
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
              for (int j = 0; j < 4; j++) acc[m][j] = M::run(yf[s2][j], xf[m][s2], acc[m][j]);
          }
        // refill this ring slot only now: its old contents are dead, so the loads can land in the same registers
        // (issued earlier, the compiler would rotate registers at the loop edge and wait for every load to do so)
        issue(st, e + RING < last ? e + RING : last);
      }
    }
  }
  __syncthreads();
  T *cs = &Ys[0][(wave * 16) * kLdsRow];
  T *po = reinterpret_cast<T *>(g.out) + z * g.out_sz + depth * g.out_sh + n0;
#pragma unroll
  for (int m = 0; m < G; m++) {
    const int line = lg * G + m;
    if (line < g.lines && !((skip >> m) & 1)) store_slice<T, true>(cs, po + ((int64_t)line * 64 + wave * 16) * g.ldo, g.ldo, acc[m], lane);
  }
}

// (two copies of the body, chosen by the plan's streaming hint: see k_sdd64_rg)
template <typename T, bool SP_TRANS, int SUBS = 1>
__global__ void __launch_bounds__(256) k_xsd64_rg(XsdArgs g) {
  // groups: two dense tiles + two sparse tiles when read transposed, else a 16-row slice of each member's block per
  // wavefront (4 x 4 quarter tiles); chains: one dense and one sparse tile per wavefront
  __shared__ __attribute__((aligned(16))) T smem[(SP_TRANS ? 8 : 6) * 64 * kLdsRow];
  const int code = as_table(g.gplan)[4 * ((int64_t)(blockIdx.x / g.Z) / g.n_tiles) + 3];
  if (code >= 0 && ((code >> 28) & 1)) xsd64_rg_body<T, SP_TRANS, true, SUBS>(g, smem);
  else xsd64_rg_body<T, SP_TRANS, false, SUBS>(g, smem);
}

// ---------------------------------------------------------------------------------------------------------
// Row groups for blocks of 16 and 32 (16-bit types, 64-wide tile of the dense free dimension).  Same plan as the
// block-64 kernel above, other division of labour: a line is only 16 or 32 rows, so each of the four wavefronts
// takes one MEMBER of the group (all rows of its line), and an entry is one block of the reduction: its dense rows
// (BLOCK x 64) go through LDS once for all four members, each wavefront fetches its own sparse block straight into
// operand registers (through its own piece of LDS and the transposing read when the block is read transposed).
// Against one workgroup per line this moves 2.5x fewer bytes between L2, LDS and the registers per line and
// needs half the barriers.  Block 16 multiplies with the 16x16x16 MFMA (one block = one reduction step).
// ---------------------------------------------------------------------------------------------------------
template <typename T, int K> struct LineMma;
template <typename T> struct LineMma<T, 32> : Mma16<T> {};
template <> struct LineMma<f16, 16> {
  typedef f16x4 frag_t;
  static __device__ __forceinline__ f32x4 run(frag_t a, frag_t b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0); }
};
template <> struct LineMma<bf16, 16> {
  typedef s16x4 frag_t;
  static __device__ __forceinline__ f32x4 run(frag_t a, frag_t b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0); }
};
// operand of the line kernels from an LDS tile stored [k][column]: K consecutive reduction indices of this lane's column
template <typename T, int K> __device__ __forceinline__ typename LineMma<T, K>::frag_t line_tr_frag(const T *tile, int ld, int col0, int lane) {
  const int q = lane >> 4, t = lane & 15;
  if constexpr (K == 32) {
    const T *p = tile + (8 * q + (t >> 2)) * ld + col0 + 4 * (t & 3);
    return tr_frag<T>(p, p + 4 * ld);
  } else {
    typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
    const T *p = tile + (4 * q + (t >> 2)) * ld + col0 + 4 * (t & 3);
    return __builtin_bit_cast(typename LineMma<T, K>::frag_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)p));
  }
}

// A chain at blocks 16 / 32: the four wavefronts take every fourth entry of the line each, with their own dense rows
// in their own piece of LDS (no workgroup barrier in the loop), and the four partial results are added through LDS at
// the end, one 16-row tile at a time.  Ys: four tiles of BLOCK x kLdsRow, Xs: four sparse blocks (transposed variant),
// red: 16 KiB for the reduction (may overlap Ys and Xs: used after a barrier that ends the loop).
template <typename T, int BLOCK, bool SP_TRANS>
__device__ __forceinline__ void xsd_chain_small(const XsdArgs &g, T *Ys, T *Xs, T *Cs, float *red, int z, int n0, int depth, int line,
                                                table_ptr ent, int ne) {
  typedef LineMma<T, BLOCK> M;
  typedef typename M::frag_t frag_t;
  constexpr int MT = BLOCK / 16, LDX = BLOCK + 8, YT = BLOCK * kLdsRow, XT = BLOCK * LDX;
  constexpr int NY = BLOCK / 8;                   // 16-byte loads per lane for BLOCK rows of 64 columns
  constexpr int XB = BLOCK * BLOCK * 2 / 64;
  constexpr int NX = XB / 16 > 0 ? XB / 16 : 1;
  typedef typename std::conditional<XB == 8, u32x2, u32x4>::type xreg_t;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int q = lane >> 4, t = lane & 15;
  const T *sp = reinterpret_cast<const T *>(g.sp) + z * g.sp_sz;
  const T *dn = reinterpret_cast<const T *>(g.dn) + z * g.dn_sz + depth * g.dn_sh + n0;
  const int64_t ldd = g.ldd;
  T *Yw = Ys + wave * YT, *Xw = Xs + wave * XT;
  const int lr = lane >> 3, lc = (lane & 7) * 8;
  u32x4 y[NY];
  xreg_t x[NX];
  auto issue = [&](int e) {
    const table_ptr en = ent + (G + 1) * e;
    const T *py = dn + ((int64_t)en[0] * BLOCK + lr) * ldd + lc;
#pragma unroll
    for (int i = 0; i < NY; i++) y[i] = *reinterpret_cast<const u32x4 *>(py + (int64_t)i * 8 * ldd);
    const T *blk = sp + (int64_t)en[1] * (BLOCK * BLOCK);
#pragma unroll
    for (int i = 0; i < NX; i++) {
      if constexpr (SP_TRANS) x[i] = *reinterpret_cast<const xreg_t *>(blk + (XB == 8 ? lane * 4 : (64 * i + lane) * 8));
      else x[i] = *reinterpret_cast<const xreg_t *>(XB == 8 ? blk + t * BLOCK + 4 * q : blk + (16 * i + t) * BLOCK + 8 * q);
    }
  };
  f32x4 acc[MT][4];
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int count = (ne - wave + 3) / 4;          // entries wave, wave + 4, ...
  if (count > 0) issue(wave);
  for (int k = 0; k < count; k++) {
#pragma unroll
    for (int i = 0; i < NY; i++) *reinterpret_cast<u32x4 *>(&Yw[(8 * i + lr) * kLdsRow + lc]) = y[i];
    frag_t xf[MT];
    if constexpr (SP_TRANS) {
#pragma unroll
      for (int i = 0; i < NX; i++) {
        const int c = 64 * i + lane;
        constexpr int CPR = BLOCK * 2 / (int)sizeof(xreg_t), CE = (int)sizeof(xreg_t) / 2;
        *reinterpret_cast<xreg_t *>(&Xw[(c / CPR) * LDX + (c % CPR) * CE]) = x[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < MT; i++) xf[i] = __builtin_bit_cast(frag_t, x[i]);
    }
    __builtin_amdgcn_wave_barrier();              // the LDS operations of one wavefront complete in order
    frag_t yf[4];
#pragma unroll
    for (int j = 0; j < 4; j++) yf[j] = line_tr_frag<T, BLOCK>(Yw, kLdsRow, 16 * j, lane);
    if constexpr (SP_TRANS) {
#pragma unroll
      for (int i = 0; i < MT; i++) xf[i] = line_tr_frag<T, BLOCK>(Xw, LDX, 16 * i, lane);
    }
    if (k + 1 < count) issue(wave + 4 * (k + 1));  // the registers of this entry are free again
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) acc[i][j] = M::run(yf[j], xf[i], acc[i][j]);
    __builtin_amdgcn_wave_barrier();
  }
  T *po = reinterpret_cast<T *>(g.out) + z * g.out_sz + depth * g.out_sh + n0;
#pragma unroll
  for (int i = 0; i < MT; i++) {
    __syncthreads();                               // the loop's tiles (first round) or the previous sums are no longer read
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int c = 0; c < 4; c++) red[((wave * 4 + j) * 4 + c) * 64 + lane] = acc[i][j][c];
    __syncthreads();
    if (wave == (i & 3)) {
      f32x4 fin[4];
#pragma unroll
      for (int j = 0; j < 4; j++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
          float v = 0.f;
#pragma unroll
          for (int w = 0; w < 4; w++) v += red[((w * 4 + j) * 4 + c) * 64 + lane];
          fin[j][c] = v;
        }
      asm volatile("" ::: "memory");   // the staging rows lie over the sums just read (as floats): keep the order
      store_slice<T, true>(Cs + wave * (16 * kLdsRow), po + ((int64_t)line * BLOCK + 16 * i) * g.ldo, g.ldo, fin, lane);
    }
  }
}

// LDS of k_xsd_rg_small.  groups: two dense tiles (double buffer); chains: one per wavefront.  The chain's reduction
// buffer (16 KiB of floats) lies over the tiles (the front part is as large as the larger of the two) and is only
// used after a barrier that ends the chain's loop.  The staging rows Cs (one 16-row slice per wavefront) lie over the
// front of all that as well: they are written after a barrier that ends the loop, or by the one wavefront that has
// just read the sums (6 -> 7 workgroups per CU at block 16: the untransposed products 3 % faster).
template <typename T, int BLOCK, bool SP_TRANS> struct SmallXsdLds {
  static constexpr int LDX = BLOCK + 8;
  static constexpr int YT = BLOCK * kLdsRow, XT = SP_TRANS ? BLOCK * LDX : 0, CT = 16 * kLdsRow;
  static constexpr int TILES = 4 * YT + 4 * XT, RED = 16 * 64 * 4 * (int)sizeof(float) / (int)sizeof(T);
  static constexpr int FRONT = TILES > RED ? TILES : RED;
  static constexpr int ELEMS = FRONT;
  static_assert(FRONT >= 4 * CT, "the staging rows lie over the tiles");
};

template <typename T, int BLOCK, bool SP_TRANS, bool STREAM>
__device__ __forceinline__ void xsd_rg_small_body(const XsdArgs &g, T *smem) {
  typedef LineMma<T, BLOCK> M;
  typedef typename M::frag_t frag_t;
  constexpr int MT = BLOCK / 16;                 // 16-row tiles of a line
  constexpr int XB = BLOCK * BLOCK * 2 / 64;     // bytes of a sparse block per lane: 8 (block 16) or 32
  constexpr int NX = XB / 16 > 0 ? XB / 16 : 1;  // loads per lane: one of 8 bytes, or two of 16
  typedef typename std::conditional<XB == 8, u32x2, u32x4>::type xreg_t;
  typedef SmallXsdLds<T, BLOCK, SP_TRANS> LD;
  constexpr int LDX = LD::LDX, YT = LD::YT, XT = LD::XT, CT = LD::CT;
  T (*Ys)[YT] = reinterpret_cast<T (*)[YT]>(smem);
  T (*Xs)[XT > 0 ? XT : 8] = reinterpret_cast<T (*)[XT > 0 ? XT : 8]>(smem + 4 * YT);
  T (*Cs)[CT] = reinterpret_cast<T (*)[CT]>(smem);
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int z = blockIdx.x % g.Z;
  const int64_t rest = blockIdx.x / g.Z;
  const int n0 = (int)(rest % g.n_tiles) * 64;
  const table_ptr hd = as_table(g.gplan) + 4 * (rest / g.n_tiles);
  const int e0 = hd[0], ne = hd[1], depth = hd[2], code = hd[3];
  const table_ptr ent = as_table(g.gplan) + 4 * (int64_t)g.n_pgroups + (int64_t)(G + 1) * e0;
  if (code < 0) {   // a chain: the line -(code + 1) on its own
    xsd_chain_small<T, BLOCK, SP_TRANS>(g, smem, smem + 4 * YT, smem, reinterpret_cast<float *>(smem), z, n0, depth, -(code + 1), ent, ne);
    return;
  }
  const int line = (code & 0xffffff) * G + wave;
  const bool mine = line < g.lines && !(((code >> 24) >> wave) & 1);
  const T *sp = reinterpret_cast<const T *>(g.sp) + z * g.sp_sz;
  const T *dn = reinterpret_cast<const T *>(g.dn) + z * g.dn_sz + depth * g.dn_sh + n0;
  const int64_t ldd = g.ldd;
  const int yc = tid % (BLOCK * 8), yrow = yc >> 3, ycol = (yc & 7) * 8;   // this thread's 16-byte chunk of the dense rows
  const bool ywrite = tid < BLOCK * 8;
  const int q = lane >> 4, t = lane & 15;
  struct Stage { u32x4 y; xreg_t x[NX]; };
  // Stages in flight (even: a stage's LDS buffer is its parity).  Measured: the untransposed products are 3-6 % faster
  // with 2 than with 4 (fewer registers, one more workgroup per CU), the transposed ones at block 32 6-8 % slower;
  // 6 and 8 are 5-20 % slower everywhere.
  constexpr int RING = (!SP_TRANS || BLOCK == 16) ? 2 : 4;
  Stage ring[RING];
  // A fixed number of loads per stage whatever the entry holds (the wait in front of a stage is then exact): an
  // absent block reads one line at the start of the sparse tensor.
  auto issue = [&](Stage &st, int e) {
    const table_ptr en = ent + (G + 1) * e;
    // (streaming loads of the dense rows where the plan says so: 4-6 us less at block 32 on the fixed attention
    // layout, 3-5 us more at block 16, where four times as many groups ask for each row)
    const u32x4 *py = reinterpret_cast<const u32x4 *>(dn + ((int64_t)en[0] * BLOCK + yrow) * ldd + ycol);
    if constexpr (STREAM) st.y = __builtin_nontemporal_load(py);
    else st.y = *py;
    const int bid = en[1 + wave];
    const T *blk = sp + (int64_t)(bid >= 0 ? bid : 0) * (BLOCK * BLOCK);
#pragma unroll
    for (int i = 0; i < NX; i++) {
      const T *px;
      if constexpr (SP_TRANS) px = blk + (XB == 8 ? lane * 4 : (64 * i + lane) * 8);        // as stored: consecutive lanes, consecutive chunks
      else px = XB == 8 ? blk + t * BLOCK + 4 * q : blk + (16 * i + t) * BLOCK + 8 * q;   // operand layout
      if (bid < 0) px = sp;
      st.x[i] = *reinterpret_cast<const xreg_t *>(px);
    }
  };
  f32x4 acc[MT][4];
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  if (ne > 0) {
    const int last = ne - 1;
#pragma unroll
    for (int u = 0; u < RING; u++) issue(ring[u], u < last ? u : last);
    const int steps = (ne + RING - 1) / RING * RING;
    for (int e0i = 0; e0i < steps; e0i += RING) {
#pragma unroll
      for (int u = 0; u < RING; u++) {
        const int e = e0i + u;
        const bool live = e < ne;
        const int buf = e & 1;
        Stage &st = ring[u];
        const int bid0 = ent[(G + 1) * min(e, last) + 1 + wave];
        const int bid = live ? bid0 : -1;
        if (ywrite) *reinterpret_cast<u32x4 *>(&Ys[buf][yrow * kLdsRow + ycol]) = st.y;
        frag_t xf[MT];
        if constexpr (SP_TRANS) {
#pragma unroll
          for (int i = 0; i < NX; i++) {
            const int c = 64 * i + lane;                       // chunk of xreg_t: row c / (chunks per row)
            constexpr int CPR = BLOCK * 2 / (int)sizeof(xreg_t), CE = (int)sizeof(xreg_t) / 2;
            *reinterpret_cast<xreg_t *>(&Xs[wave][(c / CPR) * LDX + (c % CPR) * CE]) = st.x[i];
          }
        } else {
#pragma unroll
          for (int i = 0; i < MT; i++) xf[i] = __builtin_bit_cast(frag_t, st.x[i]);
        }
        __syncthreads();
        if (bid >= 0) {
          frag_t yf[4];
#pragma unroll
          for (int j = 0; j < 4; j++) yf[j] = line_tr_frag<T, BLOCK>(Ys[buf], kLdsRow, 16 * j, lane);
          if constexpr (SP_TRANS) {
#pragma unroll
            for (int i = 0; i < MT; i++) xf[i] = line_tr_frag<T, BLOCK>(Xs[wave], LDX, 16 * i, lane);
          }
#pragma unroll
          for (int i = 0; i < MT; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[i][j] = M::run(yf[j], xf[i], acc[i][j]);   // rows n = 16j + 4*(lane/16) + e, column m = lane % 16
        }
        issue(st, e + RING < last ? e + RING : last);
      }
    }
  }
  __syncthreads();   // the staging rows lie over the tiles: nobody reads those any more
  if (mine) {
    T *po = reinterpret_cast<T *>(g.out) + z * g.out_sz + depth * g.out_sh + n0;
#pragma unroll
    for (int i = 0; i < MT; i++)
      store_slice<T, true>(Cs[wave], po + ((int64_t)line * BLOCK + 16 * i) * g.ldo, g.ldo, acc[i], lane);
  }
}

// (two copies of the body, chosen by the plan's streaming hint: see k_sdd64_rg)
template <typename T, int BLOCK, bool SP_TRANS>
__global__ void __launch_bounds__(256) k_xsd_rg_small(XsdArgs g) {
  __shared__ __attribute__((aligned(16))) T smem[SmallXsdLds<T, BLOCK, SP_TRANS>::ELEMS];
  const int code = as_table(g.gplan)[4 * ((int64_t)(blockIdx.x / g.Z) / g.n_tiles) + 3];
  // (block 16 ignores the hint: with four times as many groups per dense row as block 64, streaming loads were
  // measured 3-15 % slower there whatever the plan says)
  if (BLOCK != 16 && code >= 0 && ((code >> 28) & 1)) xsd_rg_small_body<T, BLOCK, SP_TRANS, true>(g, smem);
  else xsd_rg_small_body<T, BLOCK, SP_TRANS, false>(g, smem);
}

// sdd at blocks 16 / 32, K = 64 or 128, both operands with the reduction contiguous: one wavefront per member of a row
// group.  The member's rows of A stay in operand registers; per entry (a block-column that some member needs) the
// BLOCK rows of B are fetched once by the whole workgroup with whole-line loads, pass through LDS (two buffers, one
// barrier per 64 rows: four entries at block 16, two at block 32) and serve all four members; a wavefront whose member has a block there multiplies and writes
// it through its own piece of LDS, 16 bytes per lane in address order.  (Fetching the rows of B straight into operand layout, one row per lane, was measured 15-55 %
// slower than the general kernel: neighbouring lanes then never share a cache line.)
template <typename T, int BLOCK, int KD>
__global__ void __launch_bounds__(256) k_sdd_rg_small(SddArgs g) {
  typedef Mma16<T> M;
  typedef typename M::frag_t frag_t;
  constexpr int MT = BLOCK / 16, NK = KD / 32;
  constexpr int EB = 64 / BLOCK;                 // entries per step: 64 rows of B per barrier, as at block 64
  constexpr int RING = 2;
  constexpr int LDK = KD + 8, YT = EB * BLOCK * LDK;
  constexpr int CPR = KD / 8, CHUNKS = EB * BLOCK * CPR, NL = CHUNKS / 256;   // 16-byte chunks per row and step, loads per thread
  static_assert(CHUNKS % 256 == 0, "a step's rows of B divide evenly among the threads");
  constexpr int LDC = BLOCK + 8;                 // staging row of a result block
  __shared__ __attribute__((aligned(16))) T Ks[2][YT];
  __shared__ __attribute__((aligned(16))) T Cs[4][EB * BLOCK * LDC];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int z = blockIdx.x % g.Z;
  const table_ptr hd = as_table(g.gplan) + 4 * (int64_t)(blockIdx.x / g.Z);
  const int e0 = hd[0], ne = hd[1], h = hd[2], code = hd[3];
  if (ne <= 0) return;
  const table_ptr ent = as_table(g.gplan) + 4 * (int64_t)g.n_pgroups + (int64_t)(G + 1) * e0;
  // (a plan with chains: a chain is a group whose only member is member 0)
  const int line = code < 0 ? -(code + 1) + wave : (code & 0xffffff) * G + wave;
  const bool mine = code < 0 ? wave == 0 : (line < g.lines && !(((code >> 24) >> wave) & 1));
  const int t = lane & 15, q = lane >> 4;
  const T *pa = reinterpret_cast<const T *>(g.a) + z * g.a_sz + h * g.a_sh;
  const T *pb = reinterpret_cast<const T *>(g.b) + z * g.b_sz + h * g.b_sh;
  T *pc = reinterpret_cast<T *>(g.c) + z * g.c_sz;
  frag_t xq[MT][NK];
#pragma unroll
  for (int i = 0; i < MT; i++) {
    const T *p = pa + ((int64_t)(mine ? line : 0) * BLOCK + 16 * i + t) * g.lda + 8 * q;
#pragma unroll
    for (int s2 = 0; s2 < NK; s2++) xq[i][s2] = *reinterpret_cast<const frag_t *>(p + 32 * s2);
  }
  struct Stage { u32x4 y[NL]; };
  Stage ring[RING];
  const int last = ne - 1;
  // step s = entries EB * s ..; entries past the end repeat the last one (loaded, not used): a fixed number of loads
  auto issue = [&](Stage &st, int s) {
#pragma unroll
    for (int i = 0; i < NL; i++) {
      const int c = tid + 256 * i, r = c / CPR;              // row of the step's EB * BLOCK rows
      const int e = min(EB * s + r / BLOCK, last);
      st.y[i] = *reinterpret_cast<const u32x4 *>(pb + ((int64_t)ent[(G + 1) * e] * BLOCK + r % BLOCK) * g.ldb + (c % CPR) * 8);
    }
  };
  const int nsteps = (ne + EB - 1) / EB, slast = nsteps - 1;
#pragma unroll
  for (int u = 0; u < RING; u++) issue(ring[u], u < slast ? u : slast);
  const int steps = (nsteps + RING - 1) / RING * RING;
  for (int s0 = 0; s0 < steps; s0 += RING) {
#pragma unroll
    for (int u = 0; u < RING; u++) {
      const int s = s0 + u;
      const int buf = s & 1;
#pragma unroll
      for (int i = 0; i < NL; i++) {
        const int c = tid + 256 * i;
        *reinterpret_cast<u32x4 *>(&Ks[buf][(c / CPR) * LDK + (c % CPR) * 8]) = ring[u].y[i];
      }
      issue(ring[u], s + RING < slast ? s + RING : slast);
      __syncthreads();
      // The step's blocks of this member are computed into the wavefront's own piece of LDS (a lane holds 8 bytes of a
      // row, neighbouring lanes different rows) and leave from there in address order, 1 KiB per store instruction:
      // a block of 32 as two stores, two blocks of 16 as one (measured at block 32: 94 -> 77 us against storing from
      // the accumulators).
      int bids[EB];
#pragma unroll
      for (int k = 0; k < EB; k++) {
        const int e = EB * s + k;
        const int bid0 = ent[(G + 1) * min(e, last) + 1 + wave];
        bids[k] = (e < ne && mine) ? bid0 : -1;
        if (bids[k] >= 0) {
          T *cw = Cs[wave] + k * (BLOCK * LDC);
#pragma unroll
          for (int j = 0; j < MT; j++) {
            frag_t yf[NK];
#pragma unroll
            for (int s2 = 0; s2 < NK; s2++) yf[s2] = *reinterpret_cast<const frag_t *>(&Ks[buf][(k * BLOCK + 16 * j + t) * LDK + 32 * s2 + 8 * q]);
#pragma unroll
            for (int i = 0; i < MT; i++) {
              f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
              for (int s2 = 0; s2 < NK; s2++) acc = M::run(yf[s2], xq[i][s2], acc);   // rows n = 16j + 4q + c, column m = 16i + t
              union { u32x2 raw; T e[4]; } pk;
#pragma unroll
              for (int c = 0; c < 4; c++) pk.e[c] = from_float<T>(acc[c]);
              *reinterpret_cast<u32x2 *>(cw + (16 * i + t) * LDC + 16 * j + 4 * q) = pk.raw;
            }
          }
        }
      }
      __builtin_amdgcn_wave_barrier();                 // the LDS operations of one wavefront complete in order
      constexpr int CPB = BLOCK * BLOCK / 8, RC = BLOCK / 8;   // 16-byte chunks per block and per row
      constexpr int BPI = CPB >= 64 ? 1 : 64 / CPB;            // blocks per store instruction
#pragma unroll
      for (int k0 = 0; k0 < EB; k0 += BPI)
#pragma unroll
        for (int i = 0; i < (CPB * BPI) / 64; i++) {
          const int c = lane + 64 * i;                  // chunk among the BPI blocks k0 ..
          int bid = bids[k0];
#pragma unroll
          for (int p = 1; p < BPI; p++) bid = (c / CPB == p) ? bids[k0 + p] : bid;
          const int cb = c % CPB;
          const T *src = Cs[wave] + (k0 + c / CPB) * (BLOCK * LDC) + (cb / RC) * LDC + (cb % RC) * 8;
          if (bid >= 0) *reinterpret_cast<u32x4 *>(pc + (int64_t)bid * (BLOCK * BLOCK) + cb * 8) = *reinterpret_cast<const u32x4 *>(src);
        }
      __builtin_amdgcn_wave_barrier();
    }
  }
}

bool fast_ok_sdd(const SddArgs &g, int block, int pack, bool a_kc, bool b_kc) {
  return block == 64 && pack == 1 && a_kc && b_kc && g.K % 64 == 0;
}
bool fast_ok_xsd(const XsdArgs &g, int block, bool dn_kc, bool out_nc) {
  return block == 64 && !dn_kc && out_nc && g.NF % 64 == 0;
}

// The member-per-wavefront kernel pays while the free dimension is short; with many 64-wide tiles the general kernel's
// 256-wide tile reuses each sparse block four times.
bool small_ok_xsd(const XsdArgs &g, int block, bool dn_kc, bool out_nc) {
  return (block == 16 || block == 32) && g.gplan && g.n_pgroups > 0 && g.n_split == 0 && !dn_kc && out_nc && g.NF % 64 == 0 && g.NF <= 128;
}
template <typename T> int xsd_small_t(const XsdArgs &g, int block, bool sp_trans, hipStream_t st) {
  const int64_t n = (int64_t)g.n_pgroups * g.n_tiles * g.Z;
  if (n >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)n), wg(256);
  if (block == 16) {
    if (sp_trans) hipLaunchKernelGGL((k_xsd_rg_small<T, 16, true>), grid, wg, 0, st, g);
    else hipLaunchKernelGGL((k_xsd_rg_small<T, 16, false>), grid, wg, 0, st, g);
  } else {
    if (sp_trans) hipLaunchKernelGGL((k_xsd_rg_small<T, 32, true>), grid, wg, 0, st, g);
    else hipLaunchKernelGGL((k_xsd_rg_small<T, 32, false>), grid, wg, 0, st, g);
  }
  return BSP_OK;
}

bool small_ok_sdd(const SddArgs &g, int block, bool a_kc, bool b_kc) {
  return (block == 16 || block == 32) && g.gplan && g.n_pgroups > 0 && a_kc && b_kc && (g.K == 64 || g.K == 128);
}
template <typename T> int sdd_small_t(const SddArgs &g, int block, hipStream_t st) {
  const int64_t n = (int64_t)g.n_pgroups * g.Z;
  if (n >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)n), wg(256);
  if (block == 16 && g.K == 64) hipLaunchKernelGGL((k_sdd_rg_small<T, 16, 64>), grid, wg, 0, st, g);
  else if (block == 16) hipLaunchKernelGGL((k_sdd_rg_small<T, 16, 128>), grid, wg, 0, st, g);
  else if (g.K == 64) hipLaunchKernelGGL((k_sdd_rg_small<T, 32, 64>), grid, wg, 0, st, g);
  else hipLaunchKernelGGL((k_sdd_rg_small<T, 32, 128>), grid, wg, 0, st, g);
  return BSP_OK;
}

// -> 2: the plan kernel wrote the whole layout; BSP_OK: the per-block kernel took this pack level; 1: nothing applies
template <typename T> int sdd_fast_t(const SddArgs &g, hipStream_t st) {
  if (g.gplan && g.n_pgroups > 0 && (g.K == 64 || g.K == 128) && !g.valid) {
    const int64_t n = (int64_t)g.n_pgroups * g.Z;
    if (n >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
    if (g.K == 64) hipLaunchKernelGGL((k_sdd64_rg<T, 64>), dim3((unsigned)n), dim3(256), 0, st, g);
    else hipLaunchKernelGGL((k_sdd64_rg<T, 128>), dim3((unsigned)n), dim3(256), 0, st, g);
    return 2;
  }
  if (!g.lut) return 1;
  const int64_t n_wg = (g.n_groups * g.Z + 3) / 4;
  if (n_wg <= 0) return BSP_OK;
  if (n_wg >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(k_sdd64_nt<T>, dim3((unsigned)n_wg), dim3(256), 0, st, g);
  return BSP_OK;
}
template <typename T> int xsd_fast_t(const XsdArgs &g, bool sp_trans, hipStream_t st) {
  if (g.gplan && g.n_pgroups > 0) {
    const int64_t n = (int64_t)g.n_pgroups * g.n_tiles * g.Z;
    if (n >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
    if (sp_trans) hipLaunchKernelGGL((k_xsd64_rg<T, true>), dim3((unsigned)n), dim3(256), 0, st, g);
    else hipLaunchKernelGGL((k_xsd64_rg<T, false>), dim3((unsigned)n), dim3(256), 0, st, g);
    if (g.n_split > 0) hipLaunchKernelGGL((k_xsd_chain_sum<T>), dim3((unsigned)n), dim3(256), 0, st, g);
    return BSP_OK;
  }
  const int64_t n_wg = (int64_t)g.width * g.n_tiles * g.Z;
  if (n_wg <= 0) return BSP_OK;
  if (n_wg >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  if (sp_trans) hipLaunchKernelGGL((k_xsd64<T, true>), dim3((unsigned)n_wg), dim3(256), 0, st, g);
  else hipLaunchKernelGGL((k_xsd64<T, false>), dim3((unsigned)n_wg), dim3(256), 0, st, g);
  return BSP_OK;
}

}  // namespace

// Returns 1 if a specialised kernel took the launch (2: through the group plan, which covers every pack level of the
// layout), 0 if the caller should use the general kernel, < 0 on error.
int sdd_fast64(int dtype, const SddArgs &g0, int block, int pack, bool a_kc, bool b_kc, hipStream_t st) {
  SddArgs g = g0;
  if (g.gplan && g.lines < 0) {
    // a plan over 64 x 64 tiles of a block-16 layout: the block-64 row-group kernel, scattering each result tile to
    // its small blocks; covers the whole layout
    const bool ok = dtype != BSP_F32 && block == 16 && g.n_pgroups > 0 && a_kc && b_kc && (g.K == 64 || g.K == 128);
    if (!ok) return 0;
    g.lines = -g.lines;
    const int64_t n = (int64_t)g.n_pgroups * g.Z;
    if (n >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)n), wg(256);
    if (dtype == BSP_F16) {
      if (g.K == 64) hipLaunchKernelGGL((k_sdd64_rg<f16, 64, 4>), grid, wg, 0, st, g);
      else hipLaunchKernelGGL((k_sdd64_rg<f16, 128, 4>), grid, wg, 0, st, g);
    } else {
      if (g.K == 64) hipLaunchKernelGGL((k_sdd64_rg<bf16, 64, 4>), grid, wg, 0, st, g);
      else hipLaunchKernelGGL((k_sdd64_rg<bf16, 128, 4>), grid, wg, 0, st, g);
    }
    return 2;
  }
  if (dtype != BSP_F32 && small_ok_sdd(g, block, a_kc, b_kc)) {
    int rc = dtype == BSP_F16 ? sdd_small_t<f16>(g, block, st) : sdd_small_t<bf16>(g, block, st);
    return rc == BSP_OK ? 2 : rc;
  }
  // (a call without the table, with the plan alone: pack is unknown, the plan kernel covers every pack level anyway)
  if (dtype == BSP_F32 || !fast_ok_sdd(g, block, g.lut ? pack : 1, a_kc, b_kc)) return 0;
  int rc = dtype == BSP_F16 ? sdd_fast_t<f16>(g, st) : sdd_fast_t<bf16>(g, st);
  return rc == BSP_OK ? 1 : rc == 1 ? 0 : rc;
}
// a plan over 64 x 64 tiles of a block-16 / block-32 layout (negative line count): the block-64 row-group kernel,
// gathering each tile from its small blocks
template <typename T, int SUBS> int xsd_coarse_t(const XsdArgs &g, bool sp_trans, hipStream_t st) {
  const int64_t n = (int64_t)g.n_pgroups * g.n_tiles * g.Z;
  if (n >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  if (sp_trans) hipLaunchKernelGGL((k_xsd64_rg<T, true, SUBS>), dim3((unsigned)n), dim3(256), 0, st, g);
  else hipLaunchKernelGGL((k_xsd64_rg<T, false, SUBS>), dim3((unsigned)n), dim3(256), 0, st, g);
  if (g.n_split > 0) hipLaunchKernelGGL((k_xsd_chain_sum<T>), dim3((unsigned)n), dim3(256), 0, st, g);
  return BSP_OK;
}
int xsd_fast64(int dtype, const XsdArgs &g0, int block, bool sp_trans, bool dn_kc, bool out_nc, hipStream_t st) {
  XsdArgs g = g0;
  if (g.gplan && g.lines < 0) {
    const bool ok = dtype != BSP_F32 && block == 16 && g.n_pgroups > 0 && !dn_kc && out_nc && g.NF % 64 == 0;
    if (!ok) return 0;                              // such a plan serves nothing else: the general kernels take the launch
    g.lines = -g.lines;
    const int rc = dtype == BSP_F16 ? xsd_coarse_t<f16, 4>(g, sp_trans, st) : xsd_coarse_t<bf16, 4>(g, sp_trans, st);
    return rc == BSP_OK ? 1 : rc;
  }
  if (dtype != BSP_F32 && small_ok_xsd(g, block, dn_kc, out_nc)) {
    int rc = dtype == BSP_F16 ? xsd_small_t<f16>(g, block, sp_trans, st) : xsd_small_t<bf16>(g, block, sp_trans, st);
    return rc == BSP_OK ? 1 : rc;
  }
  if (dtype == BSP_F32 || !fast_ok_xsd(g, block, dn_kc, out_nc)) return 0;
  int rc = dtype == BSP_F16 ? xsd_fast_t<f16>(g, sp_trans, st) : xsd_fast_t<bf16>(g, sp_trans, st);
  return rc == BSP_OK ? 1 : rc;
}

}  // namespace bsp
