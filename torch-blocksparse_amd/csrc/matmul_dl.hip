// dsd / dds for a wide free dimension (a few hundred dense rows or more), blocks of 64 and 128, fp16 / bf16: the
// products that are bound by the matrix cores and by how fast tiles travel from L2 into the CUs, not by HBM
// (a block-sparse linear layer: 8192 tokens against a 4096 x 4096 weight in blocks of 128).
//
// Same work decomposition as the general kernel k_xsd (one workgroup per table segment and 256-wide tile of the free
// dimension, tables and semantics of the reference's DSD / DDS branches, matmul.py:56-99), other pipeline:
//   * operand tiles go from global memory straight into LDS (global_load_lds_dwordx4: 16 bytes per lane, 1 KiB of
//     consecutive LDS per wavefront-level load): no staging registers, no LDS store instructions, and the only wait
//     for memory is the one in front of the barrier of a reduction step;
//   * a ring of three LDS stages, loads two reduction steps (of 32) ahead of their use, one barrier per step;
//   * conflict-free LDS reads through an XOR swizzle of the 16-byte chunks, applied by choosing which global chunk
//     each lane fetches (the data lands where the swizzled layout wants it);
//   * all eight orientations (sparse operand as stored / transposed, dense operand with the reduction contiguous or
//     strided, result written along either index): a tile whose reduction index is strided in memory is kept as it
//     lies and read with the transposing LDS load.
// A standalone dense probe of this pipeline (128 x 256 x 32 tiles) reaches 0.9 PFLOP/s on an 8192 x 4096 x 4096
// product where the register-staged general kernel reaches 0.75.
#include "matmul_generic.h"
#include <atomic>

namespace bsp {
namespace {

// The kernels of this file use more dynamic LDS than a launch may ask for by default: the limit of a kernel is raised
// once per device (a bit per device; devices past the 64th set it at every launch), from whichever thread gets there.
inline bool raise_lds_limit(const void *kernel, int bytes, std::atomic<uint64_t> &done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  const uint64_t bit = dev < 64 ? uint64_t(1) << dev : 0;
  if (bit && (done.load(std::memory_order_acquire) & bit)) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return false;
  done.fetch_or(bit, std::memory_order_release);
  return true;
}

#define BSP_GLOBAL_PTR(p) ((const void __attribute__((address_space(1))) *)(p))
#define BSP_LDS_PTR(p) ((void __attribute__((address_space(3))) *)(p))
// Wait until at most n vector-memory operations of this wavefront are outstanding and all of its LDS reads have
// returned.  It stands before the barrier of a reduction step, behind which other wavefronts start the direct-to-LDS
// loads that overwrite the stage read last: a read still in flight then could return the new bytes.  (In these
// kernels the matrix instructions that consume a step's reads come before the barrier in the compiled code, so the
// reads have returned anyway; the explicit wait does not leave that to the instruction scheduler.)
#define BSP_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | (0x7 << 4) | (0x0 << 8))

constexpr int kTK = 32;          // reduction step (elements)
constexpr int kTN = 256;         // tile of the dense free dimension
constexpr int kStages = 3;

// ---- LDS tile layouts (byte offsets) ------------------------------------------------------------------------
// Reduction contiguous: [row][4 chunks of 16 bytes]; chunk c of row r sits at chunk slot c ^ ((r >> 2) & 3).  A 128-bit
// read is served sixteen lanes (rows) per clock from 64 banks: rows r, r + 4, r + 8, r + 12 start in the same bank and
// get four different slots.  (Measured: with the slot c ^ ((r >> 1) & 3), which suits 32 banks, half of the LDS-active
// cycles were bank conflicts; with this one 7-17 %.)
__device__ __forceinline__ int kc_swz(int row) { return (row >> 2) & 3; }
__device__ __forceinline__ int kc_offset(int row, int chunk) { return row * 64 + ((chunk ^ kc_swz(row)) << 4); }
// Reduction strided: [32 reduction indices][R elements], as in memory.  The transposing read of a 16-lane group takes
// 32 contiguous bytes (a pair of chunks) from each of four consecutive reduction rows, and two such groups (neighbouring
// pairs p, p + 1 of the same four rows) are served together: eight pieces of 32 bytes that should cover the 64 banks
// once.  R >= 128 (a row is a multiple of 256 bytes: every row starts in bank 0): pair p of row k sits at pair slot
// p ^ 2 (k & 3), so the even pair lands on the four even slots and the odd pair on the four odd ones (with p ^ (k & 3)
// the two groups met in the same four slots: half of the LDS cycles of the kernels that read both operands this way
// were bank conflicts).  R = 64 (128-byte rows: two rows per bank period): p ^ (k & 3).  R = 32 (a row is 2 pairs,
// rows k and k + 2 start in the same bank): p ^ ((k >> 1) & 1).
template <int R> __device__ __forceinline__ int ks_swz(int k) { return R >= 128 ? ((k & 3) << 1) : R >= 64 ? (k & 3) : ((k >> 1) & 1); }
template <int R> __device__ __forceinline__ int ks_offset(int k, int col) {   // col in elements, multiple of 4
  const int chunk = col >> 3, pair = (chunk >> 1) ^ ks_swz<R>(k);
  return k * (R * 2) + (((pair << 1) | (chunk & 1)) << 4) + ((col & 7) << 1);
}

// One operand tile of a stage: ROWS rows of the tile index (m or n) by kTK reduction indices.
template <typename T, int ROWS, bool KCONTIG> struct DlTile {
  static constexpr int BYTES = ROWS * kTK * 2;
  static constexpr int LOADS = BYTES / 1024;          // wavefront-level loads per stage
  static_assert(KCONTIG || ROWS >= 32, "a reduction row holds at least two pairs of chunks");
  // Global element offset (relative to the tile's origin) of the chunk that lane `lane` of load `ld` fetches, as
  // (row index, reduction index): rows advance by `row_stride` elements, reduction indices by `k_stride`.
  __device__ __forceinline__ static int64_t lane_offset(int ld, int lane, int64_t row_stride, int64_t k_stride) {
    if constexpr (KCONTIG) {
      const int row = ld * 16 + (lane >> 2), slot = lane & 3;
      const int chunk = slot ^ kc_swz(row);      // the global chunk that belongs into this LDS slot
      return row * row_stride + chunk * 8 * k_stride;
    } else {
      constexpr int CPR = ROWS / 8;                    // chunks per reduction row
      const int j = ld * 64 + lane, k = j / CPR, slot = j % CPR;
      const int pair = (slot >> 1) ^ ks_swz<ROWS>(k);
      return k * k_stride + (((pair << 1) | (slot & 1)) * 8) * row_stride;
    }
  }
  // MFMA operand (32 x 16 slice): rows row0 .. row0 + 31 of the tile, reduction indices 16 * kk ..; lane l supplies row
  // l % 32, indices 8 * (l / 32) .. + 7
  __device__ __forceinline__ static typename Mma<T, 32>::frag_t frag(const unsigned char *tile, int row0, int kk, int lane) {
    typedef typename Mma<T, 32>::frag_t frag_t;
    if constexpr (KCONTIG) {
      return *reinterpret_cast<const frag_t *>(tile + kc_offset(row0 + (lane & 31), kk * 2 + (lane >> 5)));
    } else {
      typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
      const int t = lane & 15, gi = lane >> 4;
      const int k = kk * 16 + 8 * (gi >> 1) + (t >> 2), col = row0 + 16 * (gi & 1) + 4 * (t & 3);
      s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(tile + ks_offset<ROWS>(k, col)));
      s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(tile + ks_offset<ROWS>(k + 4, col)));
      typedef short s16x8 __attribute__((ext_vector_type(8)));
      s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(frag_t, v);
    }
  }
};

template <typename T, int BLOCK, bool SP_TRANS, bool DN_KC, bool OUT_NC>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) k_xsd_dl(XsdArgs g) {
  typedef Mma<T, 32> M;
  typedef typename M::frag_t frag_t;
  typedef DlTile<T, BLOCK, !SP_TRANS> XT;             // sparse block: rows m
  typedef DlTile<T, kTN, DN_KC> YT;                   // dense tile: rows n
  constexpr int STAGE = XT::BYTES + YT::BYTES;
  constexpr int WGM = BLOCK >= 128 ? 2 : 1, WGN = 4 / WGM;          // wavefronts along m and n
  constexpr int RM = BLOCK / (32 * WGM), RN = kTN / (32 * WGN);     // 32 x 32 MFMA tiles per wavefront
  constexpr int XL = XT::LOADS / 4, YL = YT::LOADS / 4, L = XL + YL; // loads per wavefront and stage
  static_assert(XT::LOADS % 4 == 0 && YT::LOADS % 4 == 0, "the loads of a stage divide evenly among four wavefronts");
  constexpr int SPB = BLOCK / kTK;                    // reduction steps per block
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;

  const int n_tiles = (g.NF + kTN - 1) / kTN;
  int z, nt, seg0;
  xsd_work_item(g, n_tiles, z, nt, seg0);
  const int seg = g.order ? as_table(g.order)[seg0] : seg0;
  const table_ptr hd = as_table(g.lut) + 6 * (int64_t)seg;
  const int offset = hd[0], seglen = hd[1], column = hd[2], depth = hd[3];
  const int nblk = seglen / BLOCK;
  // a zero-length segment that follows a real one of the same line must not touch the output; one that stands alone
  // is an empty line and zero-fills its tile (as in k_xsd)
  if (nblk == 0 && seg > 0 && hd[-6 + 2] == column && hd[-6 + 3] == depth) return;
  const table_ptr plan = as_table(g.plan) + 2 * (int64_t)((offset - 6 * g.width) / g.div2);
  const int n0 = nt * kTN, NF = g.NF;
  const int64_t ldd = g.ldd, ldo = g.ldo;
  const T *sp = reinterpret_cast<const T *>(g.sp) + z * g.sp_sz;
  const T *dn = reinterpret_cast<const T *>(g.dn) + z * g.dn_sz + depth * g.dn_sh;
  T *oz = reinterpret_cast<T *>(g.out) + z * g.out_sz + depth * g.out_sh;

  // Per-lane part of every load address, computed once.  Sparse block element (m, k): stored [m][k] or, transposed,
  // [k][m], rows of BLOCK elements.  Dense element (n, k): [n][k] (reduction contiguous) or [k][n], rows of ldd; dense
  // rows past the free dimension read row NF - 1 instead (their results are not stored).
  int64_t xoff[XL], yoff[YL];
#pragma unroll
  for (int i = 0; i < XL; i++)
    xoff[i] = SP_TRANS ? XT::lane_offset(wave * XL + i, lane, 1, BLOCK) : XT::lane_offset(wave * XL + i, lane, BLOCK, 1);
#pragma unroll
  for (int i = 0; i < YL; i++) {
    if constexpr (DN_KC) {
      const int ld = wave * YL + i, row = ld * 16 + (lane >> 2), chunk = (lane & 3) ^ kc_swz(row);
      const int n = n0 + row < NF ? n0 + row : NF - 1;
      yoff[i] = (int64_t)n * ldd + chunk * 8;
    } else {
      constexpr int CPR = kTN / 8;
      const int j = (wave * YL + i) * 64 + lane, k = j / CPR, slot = j % CPR;
      const int chunk = (((slot >> 1) ^ ks_swz<kTN>(k)) << 1) | (slot & 1);
      const int n = n0 + chunk * 8 < NF ? n0 + chunk * 8 : (NF - 8 > 0 ? NF - 8 : 0);   // whole chunks: NF is a multiple of 8
      yoff[i] = (int64_t)k * ldd + n;
    }
  }
  typename M::acc_t acc[RM][RN];
#pragma unroll
  for (int i = 0; i < RM; i++)
#pragma unroll
    for (int j = 0; j < RN; j++)
#pragma unroll
      for (int v = 0; v < M::NACC; v++) acc[i][j][v] = 0.f;

  const int ksteps = nblk * SPB;
  // table values of a step: (position of its block in the dense operand, storage index of the block).  Steps past the
  // end repeat the last one: every stage issues the same number of loads, so the wait in front of a step counts
  // exactly the loads issued after it.
  auto lookup = [&](int s, int &pos, int &bid) {
    const int b = (s < ksteps ? s : ksteps - 1) / SPB;
    pos = plan[2 * b];
    bid = plan[2 * b + 1];
  };
  auto issue = [&](int s, int pos, int bid) {
    const int kin = ((s < ksteps ? s : ksteps - 1) % SPB) * kTK;
    const T *xb = sp + (int64_t)bid * (BLOCK * BLOCK) + (SP_TRANS ? kin * BLOCK : kin);
    const T *yb = dn + (DN_KC ? (int64_t)pos + kin : ((int64_t)pos + kin) * ldd);
    unsigned char *st = smem + (s % kStages) * STAGE;
#pragma unroll
    for (int i = 0; i < XL; i++)
      __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(xb + xoff[i]), BSP_LDS_PTR(st + (wave * XL + i) * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < YL; i++)
      __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(yb + yoff[i]), BSP_LDS_PTR(st + XT::BYTES + (wave * YL + i) * 1024), 16, 0, 0);
  };
  if (nblk > 0) {
    int pos, bid;
#pragma unroll
    for (int s = 0; s < kStages - 1; s++) {
      lookup(s, pos, bid);
      issue(s, pos, bid);
    }
    lookup(kStages - 1, pos, bid);                     // the table runs one step ahead of the loads that use it: its
    for (int s = 0; s < ksteps; s++) {                 // (scalar) latency is not between the barrier and the loads
      // this wavefront's loads of step s have landed: all but those of the one step issued after them, or, at the
      // last step, all (no load is issued for steps past the end)
      if (s + 1 < ksteps) BSP_WAIT_VM(L * (kStages - 2));
      else BSP_WAIT_VM(0);
      asm volatile("" ::: "memory");                   // (the compiler must not move LDS accesses across the barrier)
      __builtin_amdgcn_s_barrier();                    // everybody's have, and everybody is done reading step s - 1
      asm volatile("" ::: "memory");
      if (s + kStages - 1 < ksteps) issue(s + kStages - 1, pos, bid);   // into the stage that step s - 1 used
      lookup(s + kStages, pos, bid);
      const unsigned char *st = smem + (s % kStages) * STAGE;
      // operands of the second half of the step are fetched from LDS before the matrix instructions of the first
      frag_t xf[kTK / 16][RM], yf[kTK / 16][RN];
#pragma unroll
      for (int kk = 0; kk < kTK / 16; kk++) {
#pragma unroll
        for (int i = 0; i < RM; i++) xf[kk][i] = XT::frag(st, (wm * RM + i) * 32, kk, lane);
#pragma unroll
        for (int j = 0; j < RN; j++) yf[kk][j] = YT::frag(st + XT::BYTES, (wn * RN + j) * 32, kk, lane);
      }
#pragma unroll
      for (int kk = 0; kk < kTK / 16; kk++)
#pragma unroll
        for (int i = 0; i < RM; i++)
#pragma unroll
          for (int j = 0; j < RN; j++) {
            if constexpr (OUT_NC) acc[i][j] = M::run(yf[kk][j], xf[kk][i], acc[i][j]);   // 4 consecutive values run along n
            else acc[i][j] = M::run(xf[kk][i], yf[kk][j], acc[i][j]);                    // ... along m
          }
    }
    BSP_WAIT_VM(0);                                    // (nothing is in flight any more unless the segment had a single step)
  }
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  // Epilogue: the whole tile through LDS (the ring is free now), then 16-byte stores along the output's contiguous
  // index, consecutive lanes on consecutive chunks.  Staged as [row][CW + 8] with CW = the contiguous extent: 256 (n)
  // or BLOCK (m).  acc[i][j][4g + e]: the A operand's row 8g + 4 * (lane / 32) + e, the B operand's row lane % 32.
  constexpr int CW = OUT_NC ? kTN : BLOCK, NR = OUT_NC ? BLOCK : kTN, LDR = CW + 8;
  static_assert(NR * LDR * 2 <= kStages * STAGE, "the staged tile fits into the ring");
  T *stage = reinterpret_cast<T *>(smem);
#pragma unroll
  for (int i = 0; i < RM; i++)
#pragma unroll
    for (int j = 0; j < RN; j++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        const int m0 = (wm * RM + i) * 32, nn0 = (wn * RN + j) * 32;
        const int fast = 8 * g4 + 4 * (lane >> 5), slow = lane & 31;
        const int row = OUT_NC ? m0 + slow : nn0 + slow, col = OUT_NC ? nn0 + fast : m0 + fast;
        union { u32x2 raw; T e[4]; } u;
#pragma unroll
        for (int e = 0; e < 4; e++) u.e[e] = from_float<T>(acc[i][j][4 * g4 + e]);
        *reinterpret_cast<u32x2 *>(stage + row * LDR + col) = u.raw;
      }
  __syncthreads();
  constexpr int CHUNKS = NR * CW / 8;
#pragma unroll 4
  for (int c = tid; c < CHUNKS; c += 256) {
    const int row = c / (CW / 8), col = (c % (CW / 8)) * 8;
    const u32x4 v = *reinterpret_cast<const u32x4 *>(stage + row * LDR + col);
    if constexpr (OUT_NC) {
      if (n0 + col < NF) __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(oz + ((int64_t)column * BLOCK + row) * ldo + n0 + col));
    } else {
      if (n0 + row < NF) __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(oz + (int64_t)(n0 + row) * ldo + column * BLOCK + col));
    }
  }
}

// ---------------------------------------------------------------------------------------------------------
// Blocks of 32 with a wide free dimension.  A 32-row line is too little work per byte fetched: with one line per
// workgroup every dense tile (32 reduction rows x 256 columns, 16 KiB) serves 32 output rows, and the launch is bound
// by the feed from L2 at a seventh of the matrix peak.  Here a workgroup owns a group of BSP_GROUP consecutive lines
// (the group plan of bsp_group_plan_build) and walks the union of their blocks: per entry one dense tile, fetched
// once, serves every member that has a block there.  Each wavefront owns 64 of the tile's 256 columns for all four
// members (its dense operands are read from LDS once per entry and used by up to four blocks) and loads one member's
// block; absent members load block 0 instead (a fixed number of loads per stage keeps the waits exact).
// Chains of the plan (long lines taken out of their groups) are groups with a single member here.
// ---------------------------------------------------------------------------------------------------------
template <typename T, bool SP_TRANS, bool DN_KC, bool OUT_NC>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) k_xsd_rg_dl(XsdArgs g) {
  typedef Mma<T, 32> M;
  typedef typename M::frag_t frag_t;
  constexpr int B = 32, G = BSP_GROUP;
  static_assert(G == 4, "one member block per wavefront");
  typedef DlTile<T, B, !SP_TRANS> XT;                 // a member's block: 2 KiB
  typedef DlTile<T, kTN, DN_KC> YT;                   // dense tile: 16 KiB
  constexpr int STAGE = G * XT::BYTES + YT::BYTES;
  constexpr int XL = XT::LOADS, YL = YT::LOADS / 4, L = XL + YL;   // loads per wavefront and stage
  constexpr int RN = kTN / (32 * 4);                  // 32-column tiles per wavefront
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n_tiles = (g.NF + kTN - 1) / kTN;
  const int64_t per_z = (int64_t)g.n_pgroups * n_tiles;
  const int64_t w = xcd_remap(blockIdx.x, per_z * g.Z);
  const int z = (int)(w / per_z);
  const int nt = (int)((w % per_z) / g.n_pgroups);
  const table_ptr hd = as_table(g.gplan) + 4 * ((w % per_z) % g.n_pgroups);
  const int e0 = hd[0], ne = hd[1], depth = hd[2], code = hd[3];
  const table_ptr ent = as_table(g.gplan) + 4 * (int64_t)g.n_pgroups + (int64_t)(G + 1) * e0;
  const bool chain = code < 0;
  const int line0 = chain ? -(code + 1) : (code & 0xffffff) * G;
  const int absent = chain ? 0xe : ((code >> 24) & 0xf);            // members that are not this group's to compute
  const int n0 = nt * kTN, NF = g.NF;
  const int64_t ldd = g.ldd, ldo = g.ldo;
  const T *sp = reinterpret_cast<const T *>(g.sp) + z * g.sp_sz;
  const T *dn = reinterpret_cast<const T *>(g.dn) + z * g.dn_sz + depth * g.dn_sh;
  T *oz = reinterpret_cast<T *>(g.out) + z * g.out_sz + depth * g.out_sh;

  int64_t xoff[XL], yoff[YL];
#pragma unroll
  for (int i = 0; i < XL; i++) xoff[i] = SP_TRANS ? XT::lane_offset(i, lane, 1, B) : XT::lane_offset(i, lane, B, 1);
#pragma unroll
  for (int i = 0; i < YL; i++) {
    if constexpr (DN_KC) {
      const int ld = wave * YL + i, row = ld * 16 + (lane >> 2), chunk = (lane & 3) ^ kc_swz(row);
      const int n = n0 + row < NF ? n0 + row : NF - 1;
      yoff[i] = (int64_t)n * ldd + chunk * 8;
    } else {
      constexpr int CPR = kTN / 8;
      const int j = (wave * YL + i) * 64 + lane, k = j / CPR, slot = j % CPR;
      const int chunk = (((slot >> 1) ^ ks_swz<kTN>(k)) << 1) | (slot & 1);
      const int n = n0 + chunk * 8 < NF ? n0 + chunk * 8 : (NF - 8 > 0 ? NF - 8 : 0);
      yoff[i] = (int64_t)k * ldd + n;
    }
  }
  typename M::acc_t acc[G][RN];
#pragma unroll
  for (int m = 0; m < G; m++)
#pragma unroll
    for (int j = 0; j < RN; j++)
#pragma unroll
      for (int v = 0; v < M::NACC; v++) acc[m][j][v] = 0.f;

  // an entry of the plan: (position of the reduction block, block id of each member or -1); entries past the end repeat
  // the last one with every member absent
  // (the ids are a vector, not an array: an array member that is copied around makes the compiler keep the entries in
  // scratch memory, and every access to scratch is a vector-memory operation that the loop would wait for)
  typedef int ids_t __attribute__((ext_vector_type(4)));
  struct Entry { int pos; ids_t id; };
  auto lookup = [&](int e) {
    const table_ptr en = ent + (G + 1) * (e < ne ? e : ne - 1);
    Entry r;
    r.pos = en[0];
    const bool live = e < ne;
#pragma unroll
    for (int m = 0; m < G; m++) {
      const int id = en[1 + m];                        // read unconditionally: one wait for the whole entry
      r.id[m] = (live && !((absent >> m) & 1)) ? id : -1;
    }
    return r;
  };
  auto issue = [&](int e, const Entry &en) {
    int bid = en.id[0];
#pragma unroll
    for (int m = 1; m < G; m++) bid = wave == m ? en.id[m] : bid;
    // an absent member still issues its loads (the count per stage is fixed), but all lanes fetch one and the same
    // chunk: a single cache line instead of sixteen
    const T *xb = sp + (int64_t)(bid > 0 ? bid : 0) * (B * B);
    const T *yb = dn + (DN_KC ? (int64_t)en.pos * B : (int64_t)en.pos * B * ldd);
    unsigned char *st = smem + (e % kStages) * STAGE;
#pragma unroll
    for (int i = 0; i < XL; i++)
      __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(xb + (bid >= 0 ? xoff[i] : 0)), BSP_LDS_PTR(st + wave * XT::BYTES + i * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < YL; i++)
      __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(yb + yoff[i]), BSP_LDS_PTR(st + G * XT::BYTES + (wave * YL + i) * 1024), 16, 0, 0);
  };
  if (ne > 0) {
    // entries s, s + 1 and s + 2 are in flight at step s (their table values in registers: the table is read one step
    // before the loads that need it are issued)
    Entry cur = lookup(0), nx1 = lookup(1), nx2 = lookup(2);
    issue(0, cur);
    issue(1, nx1);
    for (int s = 0; s < ne; s++) {
      BSP_WAIT_VM(L * (kStages - 2));
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      issue(s + 2, nx2);
      const Entry nx3 = lookup(s + 3);
      const unsigned char *st = smem + (s % kStages) * STAGE;
#pragma unroll
      for (int kk = 0; kk < kTK / 16; kk++) {
        frag_t yf[RN];
#pragma unroll
        for (int j = 0; j < RN; j++) yf[j] = YT::frag(st + G * XT::BYTES, (wave * RN + j) * 32, kk, lane);
#pragma unroll
        for (int m = 0; m < G; m++)
          if (cur.id[m] >= 0) {
            const frag_t xf = XT::frag(st + m * XT::BYTES, 0, kk, lane);
#pragma unroll
            for (int j = 0; j < RN; j++) {
              if constexpr (OUT_NC) acc[m][j] = M::run(yf[j], xf, acc[m][j]);
              else acc[m][j] = M::run(xf, yf[j], acc[m][j]);
            }
          }
      }
      cur = nx1; nx1 = nx2; nx2 = nx3;
    }
    BSP_WAIT_VM(0);
  }
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  // epilogue: the 128 x 256 tile of the group through LDS, then 16-byte stores along the contiguous output index
  constexpr int TM = G * B;
  constexpr int CW = OUT_NC ? kTN : TM, NR = OUT_NC ? TM : kTN, LDR = CW + 8;
  static_assert(NR * LDR * 2 <= kStages * STAGE, "the staged tile fits into the ring");
  T *stage = reinterpret_cast<T *>(smem);
#pragma unroll
  for (int m = 0; m < G; m++)
#pragma unroll
    for (int j = 0; j < RN; j++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        const int m0 = m * 32, nn0 = (wave * RN + j) * 32;
        const int fast = 8 * g4 + 4 * (lane >> 5), slow = lane & 31;
        const int row = OUT_NC ? m0 + slow : nn0 + slow, col = OUT_NC ? nn0 + fast : m0 + fast;
        union { u32x2 raw; T e[4]; } u;
#pragma unroll
        for (int e = 0; e < 4; e++) u.e[e] = from_float<T>(acc[m][j][4 * g4 + e]);
        *reinterpret_cast<u32x2 *>(stage + row * LDR + col) = u.raw;
      }
  __syncthreads();
  // lines of this group that exist and are its own (a line that became a chain is written by that chain)
  int own = 0;
#pragma unroll
  for (int m = 0; m < G; m++) own |= (line0 + m < g.lines && !((absent >> m) & 1)) ? 1 << m : 0;
  constexpr int CHUNKS = NR * CW / 8;
#pragma unroll 4
  for (int c = tid; c < CHUNKS; c += 256) {
    const int row = c / (CW / 8), col = (c % (CW / 8)) * 8;
    const u32x4 v = *reinterpret_cast<const u32x4 *>(stage + row * LDR + col);
    if constexpr (OUT_NC) {   // row = m (member row / 32), col = n
      if (((own >> (row >> 5)) & 1) && n0 + col < NF)
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(oz + ((int64_t)line0 * B + row) * ldo + n0 + col));
    } else {                  // row = n, col = m: a chunk of 8 lies inside one member
      if (((own >> (col >> 5)) & 1) && n0 + row < NF)
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(oz + (int64_t)(n0 + row) * ldo + line0 * B + col));
    }
  }
}

template <typename T> int launch_rg_dl(const XsdArgs &g, bool sp_trans, bool dn_kc, bool out_nc, hipStream_t st) {
  const int64_t n_wg = (int64_t)g.n_pgroups * ((g.NF + kTN - 1) / kTN) * g.Z;
  if (n_wg <= 0) return BSP_OK;
  if (n_wg >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  constexpr int SMEM = kStages * (BSP_GROUP * 32 + kTN) * kTK * 2;
  dim3 grid((unsigned)n_wg), wg(256);
#define BSP_RG_LAUNCH(ST, DK, ON)                                                                                       \
  do {                                                                                                                  \
    static std::atomic<uint64_t> done{0};                                                                               \
    if (!raise_lds_limit((const void *)k_xsd_rg_dl<T, ST, DK, ON>, SMEM, done)) return BSP_ERR_HIP;                     \
    hipLaunchKernelGGL((k_xsd_rg_dl<T, ST, DK, ON>), grid, wg, SMEM, st, g);                                           \
  } while (0)
  const int key = (sp_trans ? 4 : 0) | (dn_kc ? 2 : 0) | (out_nc ? 1 : 0);
  switch (key) {
    case 0: BSP_RG_LAUNCH(false, false, false); break;
    case 1: BSP_RG_LAUNCH(false, false, true); break;
    case 2: BSP_RG_LAUNCH(false, true, false); break;
    case 3: BSP_RG_LAUNCH(false, true, true); break;
    case 4: BSP_RG_LAUNCH(true, false, false); break;
    case 5: BSP_RG_LAUNCH(true, false, true); break;
    case 6: BSP_RG_LAUNCH(true, true, false); break;
    default: BSP_RG_LAUNCH(true, true, true); break;
  }
#undef BSP_RG_LAUNCH
  return BSP_OK;
}

// ---------------------------------------------------------------------------------------------------------
// sdd with a long reduction (hundreds of elements or more), blocks of 32, fp16 / bf16.  One output block is a 32 x 32
// product: a workgroup per block (or per 2 x 2 pack of the reference's table) fetches 2 + 2 KiB per 65 kflop and is bound
// by the feed from L2 at a thirteenth of the matrix peak.  Here a workgroup takes a group of four consecutive block-rows
// (128 rows of A, the group plan of bsp_group_plan_build) and eight of the block-columns in which any of them has a
// block (256 rows of B, gathered), and runs the dense 128 x 256 product over the whole reduction with the pipeline
// of k_xsd_dl; only the blocks that exist are written.  Computing the absent ones as well costs matrix time that the
// launch has to spare (it waits for operands either way) and removes all bookkeeping from the reduction loop: no
// table is read in it.  Operand bytes per useful flop drop by 2 at a quarter of the blocks kept.
// ---------------------------------------------------------------------------------------------------------
constexpr int kSddColsElems = 256;   // columns of the gathered B tile: 8 block-columns of 32, 16 of 16

// BLOCK = 32: the group plan of the layout itself, entries (position, id of each member's block or -1).
// BLOCK = 16: the same 128 x 256 product from blocks of 16.  The plan is over PAIRS of block-rows (a member = two
// consecutive block-rows = 32 rows of A, present at a block-column if either has a block there), so that a group is
// still 128 consecutive rows of A; a workgroup gathers sixteen block-columns of 16; an entry is (position, 4 member
// flags, then the ids of the two blocks of each member, -1 where absent): 13 ints.
template <typename T, bool A_KC, bool B_KC, int BLOCK>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) k_sdd_rg_dl(SddArgs g, int chunks) {
  typedef Mma<T, 32> M;
  typedef typename M::frag_t frag_t;
  constexpr int B = 32, G = BSP_GROUP, CB = BLOCK, J = kSddColsElems / CB, TM = G * B, TN = J * CB;
  constexpr int SUB = B / CB;                         // block-rows per member: 1 or 2
  constexpr int ENT = SUB == 1 ? G + 1 : G + 1 + G * SUB;
  static_assert(BLOCK == 16 || BLOCK == 32, "blocks of 16 or 32");
  static_assert(TN == kTN, "the gathered B tile is the dense tile of the other kernels");
  typedef DlTile<T, TM, A_KC> XT;
  typedef DlTile<T, TN, B_KC> YT;
  constexpr int STAGE = XT::BYTES + YT::BYTES;
  constexpr int XL = XT::LOADS / 4, YL = YT::LOADS / 4, L = XL + YL;
  constexpr int RM = 2, RN = 4;                       // 2 x 2 wavefronts of 64 x 128
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t per_z = (int64_t)g.n_pgroups * chunks;
  const int64_t w = xcd_remap(blockIdx.x, per_z * g.Z);
  const int z = (int)(w / per_z);
  const int chunk = (int)((w % per_z) % chunks);      // chunk fastest: the chunks of a group share its rows of A in L2
  const table_ptr hd = as_table(g.gplan) + 4 * ((w % per_z) / chunks);
  const int e0 = hd[0], ne = hd[1], h = hd[2], code = hd[3];
  if (chunk * J >= ne) return;                        // (the grid is sized for the longest possible group)
  static_assert(J == kSddColsElems / BLOCK, "launch_sdd_rg_dl sizes the grid with the same J");
  const int left = ne - chunk * J;                    // entries of this chunk: min(left, J)
  const int line0 = (code & 0xffffff) * G;
  const int rows_a = g.lines * B;                     // rows of op(A) per head
  const int64_t lda = g.lda, ldb = g.ldb;
  const T *pa = reinterpret_cast<const T *>(g.a) + z * g.a_sz + h * g.a_sh;
  const T *pb = reinterpret_cast<const T *>(g.b) + z * g.b_sz + h * g.b_sh;

  // Loop-invariant part of every load address.  A: rows line0 * 32 .. + 127 (rows past the end of the matrix read its
  // last rows; their blocks do not exist).  B: row n of the tile is row n % 32 of block-column pos[n / 32].
  int64_t xoff[XL], yoff[YL];
#pragma unroll
  for (int i = 0; i < XL; i++) {
    const int ld = wave * XL + i;
    if constexpr (A_KC) {
      const int row = ld * 16 + (lane >> 2), chunk16 = (lane & 3) ^ kc_swz(row);
      const int r = line0 * B + row < rows_a ? line0 * B + row : rows_a - 1;
      xoff[i] = (int64_t)r * lda + chunk16 * 8;
    } else {
      constexpr int CPR = TM / 8;
      const int j = ld * 64 + lane, k = j / CPR, slot = j % CPR;
      const int c = (((slot >> 1) ^ ks_swz<TM>(k)) << 1) | (slot & 1);
      const int r = line0 * B + c * 8 < rows_a ? line0 * B + c * 8 : rows_a - 8;
      xoff[i] = (int64_t)k * lda + r;
    }
  }
#pragma unroll
  for (int i = 0; i < YL; i++) {
    const int ld = wave * YL + i;
    if constexpr (B_KC) {
      const int row = ld * 16 + (lane >> 2), chunk16 = (lane & 3) ^ kc_swz(row);
      const int jj = row / CB;
      const int pos = as_table(g.gplan)[4 * (int64_t)g.n_pgroups + (int64_t)ENT * (e0 + chunk * J + (jj < left ? jj : left - 1))];
      yoff[i] = ((int64_t)pos * CB + (row % CB)) * ldb + chunk16 * 8;
    } else {
      constexpr int CPR = TN / 8;
      const int j = ld * 64 + lane, k = j / CPR, slot = j % CPR;
      const int c = (((slot >> 1) ^ ks_swz<TN>(k)) << 1) | (slot & 1);
      const int jj = c / (CB / 8);                    // CB / 8 chunks of 8 columns per block-column
      const int pos = as_table(g.gplan)[4 * (int64_t)g.n_pgroups + (int64_t)ENT * (e0 + chunk * J + (jj < left ? jj : left - 1))];
      yoff[i] = (int64_t)k * ldb + (int64_t)pos * CB + (c % (CB / 8)) * 8;
    }
  }
  typename M::acc_t acc[RM][RN];
#pragma unroll
  for (int i = 0; i < RM; i++)
#pragma unroll
    for (int j = 0; j < RN; j++)
#pragma unroll
      for (int v = 0; v < M::NACC; v++) acc[i][j][v] = 0.f;
  // which of this wavefront's 2 x 4 blocks exist: the others are neither multiplied nor (if a whole row or column of
  // them is absent) read from LDS.  The loads into LDS stay dense: their count per stage is fixed.
  unsigned present = 0;
  {
    const table_ptr ids = as_table(g.gplan) + 4 * (int64_t)g.n_pgroups + (int64_t)ENT * (e0 + chunk * J);
#pragma unroll
    for (int i = 0; i < RM; i++)
#pragma unroll
      for (int j = 0; j < RN; j++) {
        // a 32 x 32 tile of the product covers one member and 32 / CB entries; the member's flag of an entry says
        // whether any of its blocks exists there
        const int m = wm * RM + i;
        bool any = false;
#pragma unroll
        for (int t = 0; t < B / CB; t++) {
          const int jj = (wn * RN + j) * (B / CB) + t;
          any = any || (jj < left && ids[ENT * (jj < left ? jj : left - 1) + 1 + m] >= 0);
        }
        present |= any ? 1u << (i * RN + j) : 0u;
      }
  }
  const int ksteps = g.K / kTK;
  auto issue = [&](int s) {
    const int64_t k0 = (int64_t)(s < ksteps ? s : ksteps - 1) * kTK;
    const T *xb = pa + (A_KC ? k0 : k0 * lda);
    const T *yb = pb + (B_KC ? k0 : k0 * ldb);
    unsigned char *st = smem + (s % kStages) * STAGE;
#pragma unroll
    for (int i = 0; i < XL; i++)
      __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(xb + xoff[i]), BSP_LDS_PTR(st + (wave * XL + i) * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < YL; i++)
      __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(yb + yoff[i]), BSP_LDS_PTR(st + XT::BYTES + (wave * YL + i) * 1024), 16, 0, 0);
  };
#pragma unroll
  for (int s = 0; s < kStages - 1; s++) issue(s);
  for (int s = 0; s < ksteps; s++) {
    BSP_WAIT_VM(L * (kStages - 2));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    issue(s + kStages - 1);
    const unsigned char *st = smem + (s % kStages) * STAGE;
#pragma unroll
    for (int kk = 0; kk < kTK / 16; kk++) {
      frag_t xf[RM] = {}, yf[RN] = {};
#pragma unroll
      for (int i = 0; i < RM; i++)
        if ((present >> (i * RN)) & ((1u << RN) - 1)) xf[i] = XT::frag(st, (wm * RM + i) * 32, kk, lane);
#pragma unroll
      for (int j = 0; j < RN; j++)
        if ((present >> j) & 0x11u) yf[j] = YT::frag(st + XT::BYTES, (wn * RN + j) * 32, kk, lane);
      static_assert(RM == 2 && RN == 4, "the column test above reads bits j and j + RN");
#pragma unroll
      for (int i = 0; i < RM; i++)
#pragma unroll
        for (int j = 0; j < RN; j++)
          if ((present >> (i * RN + j)) & 1u) acc[i][j] = M::run(yf[j], xf[i], acc[i][j]);   // 4 consecutive values run along the block's columns
    }
  }
  BSP_WAIT_VM(0);
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  // epilogue: the 128 x 256 tile through LDS, then the blocks that exist, each 2 KiB of consecutive addresses
  constexpr int LDR = TN + 8;
  static_assert(TM * LDR * 2 <= kStages * STAGE, "the staged tile fits into the ring");
  T *stage = reinterpret_cast<T *>(smem);
#pragma unroll
  for (int i = 0; i < RM; i++)
#pragma unroll
    for (int j = 0; j < RN; j++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        const int row = (wm * RM + i) * 32 + (lane & 31), col = (wn * RN + j) * 32 + 8 * g4 + 4 * (lane >> 5);
        union { u32x2 raw; T e[4]; } u;
#pragma unroll
        for (int e = 0; e < 4; e++) u.e[e] = from_float<T>(acc[i][j][4 * g4 + e]);
        *reinterpret_cast<u32x2 *>(stage + row * LDR + col) = u.raw;
      }
  __syncthreads();
  T *pc = reinterpret_cast<T *>(g.c) + z * g.c_sz;
  const int32_t *ids = g.gplan + 4 * (int64_t)g.n_pgroups + (int64_t)ENT * (e0 + chunk * J);   // vector loads: the id differs from lane to lane
  constexpr int CPB = CB * CB / 8;                    // 16-byte chunks per block
  constexpr int MR = G * SUB;                         // block-rows of the tile
#pragma unroll 4
  for (int c = tid; c < MR * J * CPB; c += 256) {
    const int blk = c / CPB, within = c % CPB;
    const int mr = blk / J, jj = blk % J;             // block-row of the tile (member mr / SUB, its block-row mr % SUB), entry
    const int id = jj < left ? ids[ENT * jj + (SUB == 1 ? 1 + mr : 1 + G + mr)] : -1;
    if (id >= 0) {
      const int r = within / (CB / 8), cc = (within % (CB / 8)) * 8;
      *reinterpret_cast<u32x4 *>(pc + (int64_t)id * (CB * CB) + within * 8) = *reinterpret_cast<const u32x4 *>(stage + (mr * CB + r) * LDR + jj * CB + cc);
    }
  }
}

template <typename T, int BLOCK> int launch_sdd_rg_dl(const SddArgs &g, bool a_kc, bool b_kc, hipStream_t st) {
  constexpr int J = kSddColsElems / BLOCK;
  const int chunks = (g.cols + J - 1) / J;
  const int64_t n_wg = (int64_t)g.n_pgroups * chunks * g.Z;
  if (n_wg <= 0) return BSP_OK;
  if (n_wg >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  constexpr int SMEM = kStages * (BSP_GROUP * 32 + kTN) * kTK * 2;
  dim3 grid((unsigned)n_wg), wg(256);
#define BSP_SDD_RG_LAUNCH(AK, BK)                                                                                       \
  do {                                                                                                                  \
    static std::atomic<uint64_t> done{0};                                                                               \
    if (!raise_lds_limit((const void *)k_sdd_rg_dl<T, AK, BK, BLOCK>, SMEM, done)) return BSP_ERR_HIP;                  \
    hipLaunchKernelGGL((k_sdd_rg_dl<T, AK, BK, BLOCK>), grid, wg, SMEM, st, g, chunks);                                \
  } while (0)
  if (a_kc && b_kc) BSP_SDD_RG_LAUNCH(true, true);
  else if (a_kc) BSP_SDD_RG_LAUNCH(true, false);
  else if (b_kc) BSP_SDD_RG_LAUNCH(false, true);
  else BSP_SDD_RG_LAUNCH(false, false);
#undef BSP_SDD_RG_LAUNCH
  return BSP_OK;
}

// ---------------------------------------------------------------------------------------------------------
// sdd over a long reduction into few blocks of 128 (the weight gradient of a block-sparse linear layer: 102 blocks,
// reduction over 8192 tokens).  One workgroup per block leaves most of the chip idle, four 64 x 64 workgroups per block
// fetch every operand row twice.  Here a workgroup computes a whole 128 x 128 block over a PART of the reduction with
// the pipeline of k_xsd_dl (128 x 128 x 32 steps, three LDS stages of 16 KiB, three workgroups per CU) and leaves an
// fp32 partial block in the caller's workspace; k_sdd_splitk_sum adds the parts of a block in part order and writes
// it.  Deterministic, no locks, no atomics: this is what the reference's split-K lock path (matmul.py:186-203, dead
// there) was meant for.  With a single part the block is written directly.
// Work item w: block fastest, then part, then batch: the workgroups that start together on an XCD (a contiguous range
// of w) then work on the same part of the reduction, and blocks of one block-row (neighbours in the table) find the
// rows of A they share in L2, as blocks of one block-column do with B.
// ---------------------------------------------------------------------------------------------------------
struct SplitK { int parts; int steps_per_part; float *ws; };

template <typename T, bool A_KC, bool B_KC>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 3))) k_sdd128_splitk(SddArgs g, SplitK sk) {
  typedef Mma<T, 32> M;
  typedef typename M::frag_t frag_t;
  constexpr int BL = 128;
  typedef DlTile<T, BL, A_KC> XT;
  typedef DlTile<T, BL, B_KC> YT;
  constexpr int STAGE = XT::BYTES + YT::BYTES;
  constexpr int XL = XT::LOADS / 4, YL = YT::LOADS / 4, L = XL + YL;
  constexpr int RM = 2, RN = 2;                       // 2 x 2 wavefronts of 64 x 64
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t per_z = g.n_groups * sk.parts;
  const int64_t w = xcd_remap(blockIdx.x, per_z * g.Z);
  const int z = (int)(w / per_z);
  const int64_t grp = (w % per_z) % g.n_groups;
  const int part = (int)((w % per_z) / g.n_groups);
  if (g.valid && !g.valid[grp]) return;
  const table_ptr e = as_table(g.lut) + grp * 4;
  const int h = e[0], bi = e[1], bj = e[2], id = e[3];
  const int64_t lda = g.lda, ldb = g.ldb;
  const int ksteps_all = g.K / kTK;
  const int s0 = part * sk.steps_per_part;
  const int ksteps = min(sk.steps_per_part, ksteps_all - s0);
  // (a part past the end of the reduction has nothing to add: it leaves a zero block, so that the sum reads no garbage)
  const T *pa = reinterpret_cast<const T *>(g.a) + z * g.a_sz + h * g.a_sh + (A_KC ? (int64_t)bi * BL * lda : (int64_t)bi * BL);
  const T *pb = reinterpret_cast<const T *>(g.b) + z * g.b_sz + h * g.b_sh + (B_KC ? (int64_t)bj * BL * ldb : (int64_t)bj * BL);
  int64_t xoff[XL], yoff[YL];
#pragma unroll
  for (int i = 0; i < XL; i++) xoff[i] = A_KC ? XT::lane_offset(wave * XL + i, lane, lda, 1) : XT::lane_offset(wave * XL + i, lane, 1, lda);
#pragma unroll
  for (int i = 0; i < YL; i++) yoff[i] = B_KC ? YT::lane_offset(wave * YL + i, lane, ldb, 1) : YT::lane_offset(wave * YL + i, lane, 1, ldb);
  typename M::acc_t acc[RM][RN];
#pragma unroll
  for (int i = 0; i < RM; i++)
#pragma unroll
    for (int j = 0; j < RN; j++)
#pragma unroll
      for (int v = 0; v < M::NACC; v++) acc[i][j][v] = 0.f;
  auto issue = [&](int s) {
    const int64_t k0 = (int64_t)(s0 + (s < ksteps ? s : ksteps - 1)) * kTK;
    const T *xb = pa + (A_KC ? k0 : k0 * lda);
    const T *yb = pb + (B_KC ? k0 : k0 * ldb);
    unsigned char *st = smem + (s % kStages) * STAGE;
#pragma unroll
    for (int i = 0; i < XL; i++)
      __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(xb + xoff[i]), BSP_LDS_PTR(st + (wave * XL + i) * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < YL; i++)
      __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(yb + yoff[i]), BSP_LDS_PTR(st + XT::BYTES + (wave * YL + i) * 1024), 16, 0, 0);
  };
  if (ksteps > 0) {
#pragma unroll
    for (int s = 0; s < kStages - 1; s++) issue(s);
    for (int s = 0; s < ksteps; s++) {
      BSP_WAIT_VM(L * (kStages - 2));
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      issue(s + kStages - 1);                          // (past the end: the last step again, a fixed number of loads per step)
      const unsigned char *st = smem + (s % kStages) * STAGE;
      frag_t xf[kTK / 16][RM], yf[kTK / 16][RN];
#pragma unroll
      for (int kk = 0; kk < kTK / 16; kk++) {
#pragma unroll
        for (int i = 0; i < RM; i++) xf[kk][i] = XT::frag(st, (wm * RM + i) * 32, kk, lane);
#pragma unroll
        for (int j = 0; j < RN; j++) yf[kk][j] = YT::frag(st + XT::BYTES, (wn * RN + j) * 32, kk, lane);
      }
#pragma unroll
      for (int kk = 0; kk < kTK / 16; kk++)
#pragma unroll
        for (int i = 0; i < RM; i++)
#pragma unroll
          for (int j = 0; j < RN; j++) acc[i][j] = M::run(yf[kk][j], xf[kk][i], acc[i][j]);   // 4 consecutive values run along the block's columns
    }
    BSP_WAIT_VM(0);
  }
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  // acc[i][j][4 * g4 + e] = C[row (wm * RM + i) * 32 + lane % 32][col (wn * RN + j) * 32 + 8 * g4 + 4 * (lane / 32) + e]
  if (sk.parts > 1) {
    // fp32 partial block, 16 bytes per lane (the parts of a block are summed by k_sdd_splitk_sum)
    float *ws = sk.ws + (((int64_t)z * g.n_groups + grp) * sk.parts + part) * (BL * BL);
#pragma unroll
    for (int i = 0; i < RM; i++)
#pragma unroll
      for (int j = 0; j < RN; j++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          const int row = (wm * RM + i) * 32 + (lane & 31), col = (wn * RN + j) * 32 + 8 * g4 + 4 * (lane >> 5);
          const f32x4 v = {acc[i][j][4 * g4 + 0], acc[i][j][4 * g4 + 1], acc[i][j][4 * g4 + 2], acc[i][j][4 * g4 + 3]};
          *reinterpret_cast<f32x4 *>(ws + row * BL + col) = v;
        }
    return;
  }
  constexpr int LDR = BL + 8;
  static_assert(BL * LDR * 2 <= kStages * STAGE, "the staged block fits into the ring");
  T *stage = reinterpret_cast<T *>(smem);
#pragma unroll
  for (int i = 0; i < RM; i++)
#pragma unroll
    for (int j = 0; j < RN; j++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        const int row = (wm * RM + i) * 32 + (lane & 31), col = (wn * RN + j) * 32 + 8 * g4 + 4 * (lane >> 5);
        union { u32x2 raw; T e[4]; } u;
#pragma unroll
        for (int e2 = 0; e2 < 4; e2++) u.e[e2] = from_float<T>(acc[i][j][4 * g4 + e2]);
        *reinterpret_cast<u32x2 *>(stage + row * LDR + col) = u.raw;
      }
  __syncthreads();
  T *pc = reinterpret_cast<T *>(g.c) + z * g.c_sz + (int64_t)id * (BL * BL);
#pragma unroll 4
  for (int c = tid; c < BL * BL / 8; c += 256) {
    const int row = c >> 4, cc = (c & 15) * 8;
    *reinterpret_cast<u32x4 *>(pc + row * BL + cc) = *reinterpret_cast<const u32x4 *>(stage + row * LDR + cc);
  }
}

// c[z, id] = sum over the parts, in part order, of the fp32 partial blocks; one thread per 8 elements
template <typename T>
__global__ void __launch_bounds__(256) k_sdd_splitk_sum(SddArgs g, SplitK sk) {
  constexpr int BB = 128 * 128;
  const int64_t chunk = (int64_t)blockIdx.x * 256 + threadIdx.x;      // 8 consecutive elements of one block
  const int64_t blk = chunk / (BB / 8);                               // z * n_groups + grp
  if (blk >= g.n_groups * g.Z) return;
  const int64_t grp = blk % g.n_groups, z = blk / g.n_groups;
  if (g.valid && !g.valid[grp]) return;
  const int within = (int)(chunk % (BB / 8)) * 8;
  const float *ws = sk.ws + blk * sk.parts * BB + within;
  f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
  for (int p = 0; p < sk.parts; p++) {
    lo += __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(ws + (int64_t)p * BB));
    hi += __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(ws + (int64_t)p * BB + 4));
  }
  union { u32x4 raw; T e[8]; } u;
#pragma unroll
  for (int k = 0; k < 4; k++) { u.e[k] = from_float<T>(lo[k]); u.e[4 + k] = from_float<T>(hi[k]); }
  const int id = as_table(g.lut)[grp * 4 + 3];
  *reinterpret_cast<u32x4 *>(reinterpret_cast<T *>(g.c) + z * g.c_sz + (int64_t)id * BB + within) = u.raw;
}

template <typename T> int launch_sdd128_splitk(const SddArgs &g, const SplitK &sk, bool a_kc, bool b_kc, hipStream_t st) {
  const int64_t n_wg = g.n_groups * g.Z * sk.parts;
  if (n_wg <= 0) return BSP_OK;
  if (n_wg >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  constexpr int SMEM = kStages * 2 * 128 * kTK * 2;
  dim3 grid((unsigned)n_wg), wg(256);
#define BSP_SPLITK_LAUNCH(AK, BK)                                                                                       \
  do {                                                                                                                  \
    static std::atomic<uint64_t> done{0};                                                                               \
    if (!raise_lds_limit((const void *)k_sdd128_splitk<T, AK, BK>, SMEM, done)) return BSP_ERR_HIP;                     \
    hipLaunchKernelGGL((k_sdd128_splitk<T, AK, BK>), grid, wg, SMEM, st, g, sk);                                       \
  } while (0)
  if (a_kc && b_kc) BSP_SPLITK_LAUNCH(true, true);
  else if (a_kc) BSP_SPLITK_LAUNCH(true, false);
  else if (b_kc) BSP_SPLITK_LAUNCH(false, true);
  else BSP_SPLITK_LAUNCH(false, false);
#undef BSP_SPLITK_LAUNCH
  if (sk.parts > 1) {
    const int64_t chunks = g.n_groups * g.Z * (128 * 128 / 8);
    hipLaunchKernelGGL((k_sdd_splitk_sum<T>), dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, st, g, sk);
  }
  return BSP_OK;
}

template <typename T, int BLOCK> int launch_dl(const XsdArgs &g0, bool sp_trans, bool dn_kc, bool out_nc, hipStream_t st) {
  const int64_t n_wg = (int64_t)g0.width * ((g0.NF + kTN - 1) / kTN) * g0.Z;
  if (n_wg <= 0) return BSP_OK;
  if (n_wg >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  XsdArgs g = g0;
  if (n_wg > 16 * 256) g.order = nullptr;            // longest segments first only in short launches (see launch_xsd_bw)
  constexpr int SMEM = kStages * (BLOCK + kTN) * kTK * 2;
  dim3 grid((unsigned)n_wg), wg(256);
#define BSP_DL_LAUNCH(ST, DK, ON)                                                                                       \
  do {                                                                                                                  \
    static std::atomic<uint64_t> done{0};                                                                               \
    if (!raise_lds_limit((const void *)k_xsd_dl<T, BLOCK, ST, DK, ON>, SMEM, done)) return BSP_ERR_HIP;                 \
    hipLaunchKernelGGL((k_xsd_dl<T, BLOCK, ST, DK, ON>), grid, wg, SMEM, st, g);                                       \
  } while (0)
  const int key = (sp_trans ? 4 : 0) | (dn_kc ? 2 : 0) | (out_nc ? 1 : 0);
  switch (key) {
    case 0: BSP_DL_LAUNCH(false, false, false); break;
    case 1: BSP_DL_LAUNCH(false, false, true); break;
    case 2: BSP_DL_LAUNCH(false, true, false); break;
    case 3: BSP_DL_LAUNCH(false, true, true); break;
    case 4: BSP_DL_LAUNCH(true, false, false); break;
    case 5: BSP_DL_LAUNCH(true, false, true); break;
    case 6: BSP_DL_LAUNCH(true, true, false); break;
    default: BSP_DL_LAUNCH(true, true, true); break;
  }
#undef BSP_DL_LAUNCH
  return BSP_OK;
}

}  // namespace

// 1 = launched, 0 = not applicable (the caller takes another kernel), < 0 = error
int xsd_dl(int dtype, const XsdArgs &g, int block, bool sp_trans, bool dn_kc, bool out_nc, hipStream_t st) {
  if (dtype == BSP_F32 || g.NF < 256) return 0;
  if (block == 32) {   // needs the group plan (whole blocks, no split chains)
    // Measured on 2048^3 products at a quarter of the blocks (8 x 16 of them): with the dense operand's reduction
    // contiguous 1.60-1.83 ms against 1.89-2.05 for the general kernel; with it strided the general kernel's 1.47-1.58 ms
    // stand against 1.70-1.73 (also with the conflict-free layout of the strided tiles), so those stay where they were.
    if (!dn_kc) return 0;
    if (!g.gplan || g.n_pgroups <= 0 || g.lines <= 0 || g.n_split != 0) return 0;
    const int rc = dtype == BSP_F16 ? launch_rg_dl<f16>(g, sp_trans, dn_kc, out_nc, st) : launch_rg_dl<bf16>(g, sp_trans, dn_kc, out_nc, st);
    return rc == BSP_OK ? 1 : rc;
  }
  if (block != 64 && block != 128) return 0;
  // (sparse operand transposed and dense operand with the reduction contiguous, the dX product of a sparse linear layer:
  // measured 0.064 ms here against 0.059 ms for the general kernel at block 128, 0.0595 against 0.0596 once the strided
  // tiles were free of bank conflicts, equal at block 64: left where it was)
  if (sp_trans && dn_kc) return 0;
  int rc;
  if (dtype == BSP_F16) rc = block == 128 ? launch_dl<f16, 128>(g, sp_trans, dn_kc, out_nc, st) : launch_dl<f16, 64>(g, sp_trans, dn_kc, out_nc, st);
  else rc = block == 128 ? launch_dl<bf16, 128>(g, sp_trans, dn_kc, out_nc, st) : launch_dl<bf16, 64>(g, sp_trans, dn_kc, out_nc, st);
  return rc == BSP_OK ? 1 : rc;
}

// sdd at blocks of 128 over a reduction cut into `parts` parts (pack-1 table rows; ws: parts fp32 blocks per table row and
// batch, may be null when parts == 1): BSP_OK = launched, BSP_ERR_UNSUPPORTED = not this kernel's case
int sdd128_splitk(int dtype, const SddArgs &g, int parts, float *ws, bool a_kc, bool b_kc, hipStream_t st) {
  if (dtype == BSP_F32 || parts < 1 || g.K % kTK || (parts > 1 && !ws)) return BSP_ERR_UNSUPPORTED;
  const int steps = g.K / kTK;
  SplitK sk;
  sk.parts = parts; sk.steps_per_part = (steps + parts - 1) / parts; sk.ws = ws;
  return dtype == BSP_F16 ? launch_sdd128_splitk<f16>(g, sk, a_kc, b_kc, st) : launch_sdd128_splitk<bf16>(g, sk, a_kc, b_kc, st);
}

// sdd with a long reduction at blocks of 32 from the group plan alone: 2 = launched (every block of the layout is
// written), 0 = not applicable, < 0 = error
int sdd_dl(int dtype, const SddArgs &g, int block, bool rowpair_plan, bool a_kc, bool b_kc, hipStream_t st) {
  if (dtype == BSP_F32 || (block != 32 && block != 16) || !g.gplan || g.n_pgroups <= 0 || g.lines <= 0 || g.cols <= 0) return 0;
  if ((block == 16) != rowpair_plan) return 0;        // blocks of 16 come with the plan over pairs of block-rows, and only they
  if (g.K < 256 || g.K % kTK) return 0;
  int rc;
  if (block == 32) rc = dtype == BSP_F16 ? launch_sdd_rg_dl<f16, 32>(g, a_kc, b_kc, st) : launch_sdd_rg_dl<bf16, 32>(g, a_kc, b_kc, st);
  else rc = dtype == BSP_F16 ? launch_sdd_rg_dl<f16, 16>(g, a_kc, b_kc, st) : launch_sdd_rg_dl<bf16, 16>(g, a_kc, b_kc, st);
  return rc == BSP_OK ? 2 : rc;
}

}  // namespace bsp
