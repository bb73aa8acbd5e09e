// General block-sparse matmul kernels for gfx950: every block size (16/32/64/128), fp16 / bf16 / fp32,
// every trans_a / trans_b / trans_c combination.
//
// Replaces the reference's single Triton-C kernel with its SDD / DSD / DDS branches (matmul.py:6-205).
// Structure: a workgroup of four wavefronts owns one output tile; both operand tiles are staged through LDS
// An operand whose reduction dimension is contiguous in memory sits in LDS as rows of TK elements plus padding
// and every MFMA operand is one 16-byte LDS read; an operand stored with the reduction dimension strided sits in
// LDS as it lies in memory and is read with the transposing LDS load (16-bit types; 32-bit ones are transposed
// while they are written).  Global loads for step s+1 are issued before
// the MFMAs of step s (two LDS buffers, one barrier per step).  fp32 accumulation in 16x16 MFMA tiles.
//
// "xsd" is the kernel behind both dsd and dds: dds is dsd with the roles of rows and columns exchanged
// (C^T = B_sparse^T . A^T), which only changes the three orientation flags.
#pragma once
#include "bsp_common.h"

namespace bsp {

// ---------------------------------------------------------------------------------------------------------
// MFMA per element type and tile size MS (16 or 32).  Lane l supplies row (l % MS) of its operand, reduction
// indices (l / MS) * KV .. + KV - 1.  Result: MS = 16 -> element e is (row 4*(l/16) + e, column l % 16);
// MS = 32 -> element 4*g + e is (row 8*g + 4*(l/32) + e, column l % 32).
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

template <typename T, int MS> struct Mma;
template <typename T> struct Mma<T, 16> : Mma16<T> {
  static constexpr int NACC = 4;
  typedef f32x4 acc_t;
};
template <> struct Mma<f16, 32> {
  static constexpr int KSTEP = 16, KV = 8, NACC = 16;
  typedef f16x8 frag_t;
  typedef f32x16 acc_t;
  static __device__ __forceinline__ acc_t run(frag_t a, frag_t b, acc_t c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};
template <> struct Mma<bf16, 32> {
  static constexpr int KSTEP = 16, KV = 8, NACC = 16;
  typedef bf16x8 frag_t;
  typedef f32x16 acc_t;
  static __device__ __forceinline__ acc_t run(frag_t a, frag_t b, acc_t c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Mma<float, 32> {
  static constexpr int KSTEP = 2, KV = 1, NACC = 16;
  typedef float frag_t;
  typedef f32x16 acc_t;
  static __device__ __forceinline__ acc_t run(frag_t a, frag_t b, acc_t c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
};

template <typename T> struct TileK { static constexpr int TK = 64 / sizeof(T), PAD = 16 / sizeof(T); };  // 64-byte rows + 16 bytes

// ---------------------------------------------------------------------------------------------------------
// One operand tile: ROWS x TK, fetched by NT threads in 16-byte chunks, kept in registers until the LDS
// buffer is free.  The address of a chunk is split into the part that never changes for a thread (computed once, before
// the reduction loop) and the part that is the same for all threads of a step (scalar arithmetic on the step's table
// values): a load costs one 64-bit add, not the multiplications and selects of a full index computation.
//   View::part_k(row, k) / part_r(row, k) -> Part{off, ok, sel, k}: element offset of chunk (row, k..k+VE-1) resp.
//     (row..row+VE-1, k) inside the step, whether the rows exist, which of the step's blocks it belongs to
//   View::step(k0) -> Step{..., live[NB], klim}: raw table values of the reduction step starting at k0
//   View::scalar_k(step, i) / scalar_r(step, i) -> element offset of block i of the step
// ---------------------------------------------------------------------------------------------------------
struct Part { int64_t off; bool ok; int sel; int k; };

template <typename T, int ROWS, int NT, bool KCONTIG> struct TileLoader {
  static constexpr int TK = TileK<T>::TK, LDK = TK + TileK<T>::PAD;
  static constexpr int VE = 16 / sizeof(T);
  static constexpr int NCH = ROWS * TK / VE;
  static constexpr int ITER = (NCH + NT - 1) / NT;
  static constexpr int CPR = TK / VE;    // chunks per row when the reduction is contiguous
  static constexpr int RCH = ROWS / VE;  // chunks per reduction index otherwise
  // An operand stored with the reduction dimension strided is kept in LDS as it lies in memory, [TK][ROWS + 8].  A
  // 16-bit one is handed to the MFMA through the transposing LDS read; a 32-bit one needs no transposition at all:
  // its MFMA operand is a single element per lane, (row lane % MS, reduction index lane / MS), read where it lies.
  static constexpr bool ASIS = !KCONTIG;
  static constexpr bool TR = ASIS && sizeof(T) == 2;
  // Padding of a row of the as-is layout.  16-bit: the transposing read of a 16-lane group takes 32 contiguous bytes from
  // each of four consecutive reduction rows, and two groups half a row block apart are served together; with rows of
  // 64 bytes more than a multiple of 256 these eight pieces fall into different banks (the LDS serves 256 bytes per
  // clock: measured, bank-conflict cycles 46-50 % -> 10-20 % of the LDS-active cycles against a padding of 16 bytes).
  static constexpr int LDR = ROWS + (sizeof(T) == 2 ? 32 : 8);
  static constexpr int ELEMS = ASIS ? TK * LDR : ROWS * LDK;
  u32x4 reg[ITER];
  bool ok[ITER];

  __device__ __forceinline__ void store(T *S, int tid) const {
#pragma unroll
    for (int it = 0; it < ITER; it++) {
      const int c = tid + it * NT;
      if (NCH % NT == 0 || c < NCH) {
        const u32x4 z = {0u, 0u, 0u, 0u};
        const u32x4 val = ok[it] ? reg[it] : z;
        if constexpr (KCONTIG) {
          *reinterpret_cast<u32x4 *>(S + (c / CPR) * LDK + (c % CPR) * VE) = val;
        } else {
          *reinterpret_cast<u32x4 *>(S + (c / RCH) * LDR + (c % RCH) * VE) = val;
        }
      }
    }
  }
  // operand fragment of an MS-row MFMA tile starting at tile row `row0`, reduction step kk (KSTEP wide)
  template <int MS, class M> __device__ __forceinline__ static typename M::frag_t frag(const T *S, int row0, int kk, int lane) {
    if constexpr (TR) {
      typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
      const int t = lane & 15, gi = lane >> 4;
      // MS 16: the four 16-lane groups are the four reduction groups; MS 32: two row halves x two reduction groups
      const int kq = (MS == 16) ? gi : (gi >> 1), rh = (MS == 16) ? 0 : 16 * (gi & 1);
      const T *p = S + (kk * M::KSTEP + 8 * kq + (t >> 2)) * LDR + row0 + rh + 4 * (t & 3);
      s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)p);
      s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 4 * LDR));
      typedef short s16x8 __attribute__((ext_vector_type(8)));
      s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(typename M::frag_t, v);
    } else if constexpr (ASIS) {
      static_assert(M::KV == 1, "32-bit operands: one element per lane");
      return S[(kk * M::KSTEP + lane / MS) * LDR + row0 + lane % MS];
    } else {
      return *reinterpret_cast<const typename M::frag_t *>(S + (row0 + lane % MS) * LDK + (lane / MS) * M::KV + kk * M::KSTEP);
    }
  }
};

// The thread-invariant half of a loader's addressing (one per operand, shared by all ring stages).
template <typename T, int ROWS, int NT, bool KCONTIG> struct TileAddr {
  typedef TileLoader<T, ROWS, NT, KCONTIG> L;
  Part part[L::ITER];
  template <class View> __device__ __forceinline__ void init(const View &v, int tid) {
#pragma unroll
    for (int it = 0; it < L::ITER; it++) {
      int c = tid + it * NT;
      if (L::NCH % NT != 0 && c >= L::NCH) c = L::NCH - 1;
      if constexpr (KCONTIG) part[it] = v.part_k(c / L::CPR, (c % L::CPR) * L::VE);
      else part[it] = v.part_r((c % L::RCH) * L::VE, c / L::RCH);
    }
  }
  // Every thread issues exactly ITER loads whatever the tile holds (chunks outside the operand read a dummy line
  // and are zeroed afterwards): with a fixed count the wait before a stage is consumed is exact.
  template <class View> __device__ __forceinline__ void load(L &dst, const View &v, const typename View::Step &st) const {
    constexpr int NB = View::NB;
    int64_t so[NB];
#pragma unroll
    for (int i = 0; i < NB; i++) so[i] = KCONTIG ? v.scalar_k(st, i) : v.scalar_r(st, i);
#pragma unroll
    for (int it = 0; it < L::ITER; it++) {
      int64_t o = so[0];
      bool live = st.live[0];
#pragma unroll
      for (int i = 1; i < NB; i++) {
        o = part[it].sel == i ? so[i] : o;
        live = part[it].sel == i ? st.live[i] : live;
      }
      const bool good = part[it].ok && live && part[it].k < st.klim;
      dst.ok[it] = good;                // zero-filling happens when the stage is consumed, not here: a use of the loaded
      dst.reg[it] = *reinterpret_cast<const u32x4 *>(good ? v.base + part[it].off + o : v.base);   // value right away would make the wait for it immediate
    }
  }
};

// ---------------------------------------------------------------------------------------------------------
// The tile product.  X supplies TM rows ("m"), Y supplies TN rows ("n"); out(m, n) = sum_k X(m,k) * Y(n,k).
// WGM x WGN wavefronts, each RM x RN MFMA tiles.  OUT_NCONTIG chooses which index the four values of a lane
// run along, so that the epilogue writes 4 consecutive elements whatever the output orientation.
// ---------------------------------------------------------------------------------------------------------
constexpr int stage_tiles(int nc, int ms, int ve, int bytes_per_elem_all_waves, int limit) {
  int cg = nc;
  while (cg > 1 && ms * (cg * ms + ve) * bytes_per_elem_all_waves > limit) cg /= 2;
  return cg;
}

template <typename T, int TM, int TN, int WGM, int WGN, bool X_KCONTIG, bool Y_KCONTIG, bool OUT_NCONTIG> struct TileGemm {
  static constexpr int NT = 64 * WGM * WGN;
  static constexpr int TK = TileK<T>::TK, LDK = TK + TileK<T>::PAD;
  // 32x32 MFMA tiles when a wavefront's region allows it (half the LDS operand traffic per flop), 16x16 otherwise
  static constexpr int MS = (TM / WGM >= 32 && TN / WGN >= 32) ? 32 : 16;
  static constexpr int RM = TM / (MS * WGM), RN = TN / (MS * WGN);
  typedef Mma<T, MS> M;
  typedef TileLoader<T, TM, NT, X_KCONTIG> XL;
  typedef TileLoader<T, TN, NT, Y_KCONTIG> YL;
  static constexpr int X_ELEMS = (XL::ELEMS + 7) & ~7, Y_ELEMS = (YL::ELEMS + 7) & ~7;
  static constexpr int SMEM_BYTES = 2 * (X_ELEMS + Y_ELEMS) * (int)sizeof(T);

  // ksteps = number of TK-wide reduction steps.  Store(m, n, vals): vals[4] run along n (OUT_NCONTIG) or m.
  // SUB > 0: the output consists of SUB x SUB blocks that are each contiguous in memory (the sparse result of sdd);
  // the epilogue then writes block by block.  SUB == 0: the output is a matrix with long rows.
  template <int SUB = 0, class XView, class YView, class Store>
  static __device__ __forceinline__ void run(const XView &xv, const YView &yv, int ksteps, T *smem, const Store &store) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    T *Xs[2] = {smem, smem + X_ELEMS + Y_ELEMS};
    T *Ys[2] = {smem + X_ELEMS, smem + 2 * X_ELEMS + Y_ELEMS};
    typename M::acc_t acc[RM][RN];
#pragma unroll
    for (int i = 0; i < RM; i++)
#pragma unroll
      for (int j = 0; j < RN; j++)
#pragma unroll
        for (int v = 0; v < M::NACC; v++) acc[i][j][v] = 0.f;
    // Register ring of NS stages (two: deeper rings were measured slower or equal, the loop is not waiting for its
    // loads): global loads run NS - 1 reduction steps ahead of their use; two LDS buffers, one
    // barrier per step.  Step s first writes stage s + 1 to the other LDS buffer, then reads stage s and issues its
    // MFMAs, then refills the ring slot it has just emptied, and only then meets the barrier: the LDS write and the
    // barrier wait pass while the matrix pipe works instead of in front of it.  The loop runs whole rounds of NS
    // steps; steps past the end hold zeros.
    constexpr int NS = 2;
    static_assert(NS % 2 == 0, "the LDS buffer of a step is chosen by the ring slot's parity");
    XL xl[NS];
    YL yl[NS];
    TileAddr<T, TM, NT, X_KCONTIG> xa;
    TileAddr<T, TN, NT, Y_KCONTIG> ya;
    xa.init(xv, tid);
    ya.init(yv, tid);
#pragma unroll
    for (int u = 0; u < NS; u++) {
      xa.load(xl[u], xv, xv.step(u * TK));
      ya.load(yl[u], yv, yv.step(u * TK));
    }
    xl[0].store(Xs[0], tid);
    yl[0].store(Ys[0], tid);
    xa.load(xl[0], xv, xv.step(NS * TK));
    ya.load(yl[0], yv, yv.step(NS * TK));
    // The table look-ups run one step ahead of the refill that uses them: started a whole step before they are needed,
    // their (scalar) latency is not in front of the loads.
    auto xst = xv.step((NS + 1) * TK);
    auto yst = yv.step((NS + 1) * TK);
    __syncthreads();
    for (int s0 = 0; s0 < ksteps; s0 += NS) {
#pragma unroll
      for (int u = 0; u < NS; u++) {
        const int s = s0 + u;
        const int cur = u & 1, nxt = cur ^ 1, u1 = (u + 1) % NS;
        xl[u1].store(Xs[nxt], tid);   // stage s + 1; this buffer was last read in step s - 1, before the previous barrier
        yl[u1].store(Ys[nxt], tid);
        // (steps past the end multiply zeros: cheaper than a branch, which would copy the accumulators around)
#pragma unroll
        for (int kk = 0; kk < TK / M::KSTEP; kk++) {
          typename M::frag_t xf[RM], yf[RN];
#pragma unroll
          for (int i = 0; i < RM; i++) xf[i] = XL::template frag<MS, M>(Xs[cur], (wm * RM + i) * MS, kk, lane);
#pragma unroll
          for (int j = 0; j < RN; j++) yf[j] = YL::template frag<MS, M>(Ys[cur], (wn * RN + j) * MS, kk, lane);
#pragma unroll
          for (int i = 0; i < RM; i++)
#pragma unroll
            for (int j = 0; j < RN; j++) {
              if constexpr (OUT_NCONTIG) acc[i][j] = M::run(yf[j], xf[i], acc[i][j]);   // result rows = n, column = m
              else acc[i][j] = M::run(xf[i], yf[j], acc[i][j]);                          // result rows = m, column = n
            }
        }
        const auto xnext = xv.step((s + NS + 2) * TK);
        const auto ynext = yv.step((s + NS + 2) * TK);
        xa.load(xl[u1], xv, xst);   // stage s + 1 + NS into the slot emptied above
        ya.load(yl[u1], yv, yst);
        xst = xnext;
        yst = ynext;
        __syncthreads();
      }
    }
    // Epilogue.  A lane's values come in groups of 4 consecutive positions along the output's contiguous index
    // (4*(lane/16) for MS 16, 8*g + 4*(lane/32) for MS 32) at row lane % MS of a tile, so a direct store would write
    // 8- or 16-byte pieces of 32 different rows per instruction.  Each wavefront instead passes one row of tiles at a
    // time through its own piece of LDS (free after the last barrier) and writes whole 16-byte chunks, consecutive
    // lanes along a row.  store(r, c, chunk): r = row (m if OUT_NCONTIG, else n), c = first of VE consecutive columns.
    constexpr int VE = 16 / (int)sizeof(T);
    if constexpr (SUB > 0 && OUT_NCONTIG && TM * (TN + VE) * (int)sizeof(T) <= SMEM_BYTES) {
      // Blocked output: the whole TM x TN tile is staged (all wavefronts, two barriers) and then written block by
      // block, consecutive lanes on consecutive 16-byte chunks of one block: 512 contiguous bytes per 32 lanes at
      // block 16, where row-wise stores would write 32-byte pieces.
      constexpr int LDS_ROW = TN + VE, CPB = SUB * SUB / VE, BPR = TN / SUB, CHUNKS = TM * TN / VE;
      const int cc = lane % MS;
#pragma unroll
      for (int i = 0; i < RM; i++)
#pragma unroll
        for (int j = 0; j < RN; j++)
#pragma unroll
          for (int g4 = 0; g4 < M::NACC / 4; g4++) {
            const int rr = (MS == 16) ? 4 * (lane >> 4) : 8 * g4 + 4 * (lane >> 5);
            T *dst = smem + ((wm * RM + i) * MS + cc) * LDS_ROW + (wn * RN + j) * MS + rr;
            if constexpr (sizeof(T) == 4) {
              *reinterpret_cast<f32x4 *>(dst) = f32x4{acc[i][j][4 * g4 + 0], acc[i][j][4 * g4 + 1], acc[i][j][4 * g4 + 2], acc[i][j][4 * g4 + 3]};
            } else {
              union { u32x2 raw; T e[4]; } u;
#pragma unroll
              for (int e = 0; e < 4; e++) u.e[e] = from_float<T>(acc[i][j][4 * g4 + e]);
              *reinterpret_cast<u32x2 *>(dst) = u.raw;
            }
          }
      __syncthreads();
#pragma unroll
      for (int it = 0; it < (CHUNKS + NT - 1) / NT; it++) {
        const int idx = it * NT + tid;
        if (CHUNKS % NT == 0 || idx < CHUNKS) {
          const int blk = idx / CPB, within = idx % CPB;
          const int m = (blk / BPR) * SUB + within / (SUB / VE), n = (blk % BPR) * SUB + (within % (SUB / VE)) * VE;
          store(m, n, *reinterpret_cast<const u32x4 *>(smem + m * LDS_ROW + n));
        }
      }
      return;
    }
    constexpr int NR = OUT_NCONTIG ? RM : RN, NC = OUT_NCONTIG ? RN : RM;   // tiles along the row / contiguous index
    // tiles staged per pass: all NC of them if that fits the tile buffers, else half, a quarter ...
    constexpr int CG = stage_tiles(NC, MS, VE, (int)sizeof(T) * WGM * WGN, SMEM_BYTES);
    constexpr int CW = CG * MS, LDS_ROW = CW + VE;                            // staged row, padded by one chunk
    static_assert(MS * LDS_ROW * (int)sizeof(T) * WGM * WGN <= SMEM_BYTES, "epilogue staging must fit the tile buffers");
    T *stage = smem + wave * (MS * LDS_ROW);
    const int cc = lane % MS;
    const int r_wave = OUT_NCONTIG ? wm * RM * MS : wn * RN * MS, c_wave = OUT_NCONTIG ? wn * RN * MS : wm * RM * MS;
#pragma unroll
    for (int pass = 0; pass < NR * (NC / CG); pass++) {
      const int rt = pass / (NC / CG), c0 = (pass % (NC / CG)) * CG;
#pragma unroll
      for (int ct = 0; ct < CG; ct++)
#pragma unroll
        for (int g4 = 0; g4 < M::NACC / 4; g4++) {
          const typename M::acc_t &t = OUT_NCONTIG ? acc[rt][c0 + ct] : acc[c0 + ct][rt];
          const int rr = (MS == 16) ? 4 * (lane >> 4) : 8 * g4 + 4 * (lane >> 5);
          T *dst = stage + cc * LDS_ROW + ct * MS + rr;
          if constexpr (sizeof(T) == 4) {
            *reinterpret_cast<f32x4 *>(dst) = f32x4{t[4 * g4 + 0], t[4 * g4 + 1], t[4 * g4 + 2], t[4 * g4 + 3]};
          } else {
            union { u32x2 raw; T e[4]; } u;
#pragma unroll
            for (int e = 0; e < 4; e++) u.e[e] = from_float<T>(t[4 * g4 + e]);
            *reinterpret_cast<u32x2 *>(dst) = u.raw;
          }
        }
      __builtin_amdgcn_wave_barrier();   // the LDS operations of one wavefront complete in order
      constexpr int CHUNKS = MS * CW / VE;
#pragma unroll
      for (int it = 0; it < (CHUNKS + 63) / 64; it++) {
        const int idx = it * 64 + lane;
        if (CHUNKS % 64 == 0 || idx < CHUNKS) {
          const int row = idx / (CW / VE), ch = idx % (CW / VE);
          store(r_wave + rt * MS + row, c_wave + c0 * MS + ch * VE, *reinterpret_cast<const u32x4 *>(stage + row * LDS_ROW + ch * VE));
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
};

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
  int cols = 0;                                       // block-columns per head when known (a call with the plan alone), else 0
};

template <typename T, int BLOCK, int PACK, bool KCONTIG> struct SddView {
  // idx is a vector, not an array: an array member makes the compiler keep the view in scratch memory and turn the
  // selection in blk() into an indexed scratch load, a full memory round trip before a workgroup's first load
  typedef int idx_t __attribute__((ext_vector_type(PACK == 1 ? 2 : PACK)));
  const T *base; int64_t ld; int K; idx_t idx;   // base doubles as the dummy address of out-of-range chunks
  int off = 0;                                        // first row of the tile inside its block (tiles smaller than a block)
  static constexpr int NB = 1;
  struct Step { int k0; bool live[1]; int klim; };
  __device__ __forceinline__ Step step(int k0) const { return Step{k0, {true}, K - k0}; }
  __device__ __forceinline__ int blk(int row) const {
    int r = idx[0];
#pragma unroll
    for (int p = 1; p < PACK; p++) r = (row / BLOCK == p) ? idx[p] : r;
    return r * BLOCK + off + row % BLOCK;
  }
  __device__ __forceinline__ Part part_k(int row, int k) const { return Part{(int64_t)blk(row) * ld + k, true, 0, k}; }
  __device__ __forceinline__ Part part_r(int row, int k) const { return Part{(int64_t)k * ld + blk(row), true, 0, k}; }
  __device__ __forceinline__ int64_t scalar_k(const Step &st, int) const { return st.k0; }
  __device__ __forceinline__ int64_t scalar_r(const Step &st, int) const { return (int64_t)st.k0 * ld; }
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
  const table_ptr e = as_table(g.lut) + grp * (PACK * PACK * 4);
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
  // The entry differs from lane to lane here, so the output block is looked up through an ordinary pointer (a vector
  // load): through the constant address space the compiler fetches all PACK * PACK entries with scalar loads and
  // indexes them per lane in scratch memory.
  const int32_t *eg = g.lut + grp * (PACK * PACK * 4);
  auto store = [&](int m, int n, u32x4 v) {
    const int ent = (m / BLOCK) * PACK + n / BLOCK;
    if (valid && !valid[ent]) return;
    const int64_t bk = eg[ent * 4 + 3];
    *reinterpret_cast<u32x4 *>(cz + bk * (BLOCK * BLOCK) + (m % BLOCK) * BLOCK + n % BLOCK) = v;
  };
  G::template run<BLOCK>(av, bv, (g.K + G::TK - 1) / G::TK, reinterpret_cast<T *>(smem_raw), store);
}

// sdd with SPLIT x SPLIT workgroups per block (pack 1): for layouts with so few blocks that one workgroup per block
// would leave most of the chip idle (a 10 % dense 32 x 32 layout of 128-blocks has 100 blocks for 256 CUs).  The
// sub-tiles of a block are neighbours in the grid, so that they meet their shared operand rows in L2.
template <typename T, int BLOCK, int SPLIT, bool A_KCONTIG, bool B_KCONTIG>
__global__ void __launch_bounds__(64 * SddShape<BLOCK / SPLIT>::WG * SddShape<BLOCK / SPLIT>::WG) k_sdd_split(SddArgs g) {
  constexpr int TT = BLOCK / SPLIT, WG = SddShape<TT>::WG;
  typedef TileGemm<T, TT, TT, WG, WG, A_KCONTIG, B_KCONTIG, true> G;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int64_t n_wg = g.n_groups * g.Z * (SPLIT * SPLIT);
  const int64_t w = xcd_remap(blockIdx.x, n_wg);
  const int sub = (int)(w % (SPLIT * SPLIT));
  const int z = (int)(w / (SPLIT * SPLIT) / g.n_groups);
  const int64_t grp = w / (SPLIT * SPLIT) % g.n_groups;
  const table_ptr e = as_table(g.lut) + grp * 4;
  if (g.valid && !g.valid[grp]) return;
  SddView<T, BLOCK, 1, A_KCONTIG> av;
  SddView<T, BLOCK, 1, B_KCONTIG> bv;
  av.base = reinterpret_cast<const T *>(g.a) + z * g.a_sz + e[0] * g.a_sh; av.ld = g.lda; av.K = g.K;
  bv.base = reinterpret_cast<const T *>(g.b) + z * g.b_sz + e[0] * g.b_sh; bv.ld = g.ldb; bv.K = g.K;
  av.idx[0] = e[1]; av.off = (sub / SPLIT) * TT;
  bv.idx[0] = e[2]; bv.off = (sub % SPLIT) * TT;
  T *cb = reinterpret_cast<T *>(g.c) + z * g.c_sz + (int64_t)e[3] * (BLOCK * BLOCK) + av.off * BLOCK + bv.off;
  auto store = [&](int m, int n, u32x4 v) { *reinterpret_cast<u32x4 *>(cb + m * BLOCK + n) = v; };
  G::run(av, bv, (g.K + G::TK - 1) / G::TK, reinterpret_cast<T *>(smem_raw), store);
}

// ---------------------------------------------------------------------------------------------------------
// xsd: out[col*BLOCK + m, n] = sum over the blocks t of one table segment  S_t(m, :) . D(n, pos_t + :)
// (dsd: S = op(A) blocks, D = op(B)^T rows; dds: S = op(B)^T blocks, D = op(A) rows).
// One workgroup per (segment, tile of the dense free dimension, batch).  Reads the segment header
// of the reference table (offset, length, column, depth; matmul.py:57-63) and the per-block positions.
// ---------------------------------------------------------------------------------------------------------
struct XsdArgs {
  const void *sp, *dn; void *out;
  int Z, NF;                            // batch, size of the dense free dimension
  int64_t sp_sz, dn_sz, dn_sh, ldd, out_sz, out_sh, ldo;
  const int32_t *lut; const int32_t *plan; int width; int div2;   // div2 = 2 * block / step of the table
  const int32_t *order;                 // order[p] = segment dispatched p-th (head by head, longest first inside a head), or null
  int n_tiles;                          // 64-wide tiles of the free dimension (specialised kernels)
  const int32_t *gplan; int n_pgroups; int lines;   // optional group plan, its groups, lines (block-rows or -columns) per head
  int n_split = 0;                      // split chains of the plan; their fp32 partial tiles (caller's workspace)
  float *partials = nullptr;
};

// A reduction step of TK elements lies inside one block (BLOCK >= TK) or covers TK / BLOCK whole blocks.
template <typename T, int BLOCK> struct StepBlocks { static constexpr int TK = TileK<T>::TK, NB = TK > BLOCK ? TK / BLOCK : 1; };

// The Step of a view holds the raw table values only; all arithmetic on them happens when the addresses are formed,
// so that a look-up started one step ahead is not waited for before it is needed.
template <typename T, int BLOCK, bool TRANS> struct SparseView {   // element (m, k) of the segment's blocks
  const T *base; table_ptr plan; int nblk;
  static constexpr int NB = StepBlocks<T, BLOCK>::NB;
  struct Step { int32_t bid[NB]; bool live[NB]; int kin; int klim; };   // storage index of each block, whether it exists, offset inside
  __device__ __forceinline__ Step step(int k0) const {
    Step st;
    st.kin = k0 % BLOCK;
    st.klim = 1 << 30;
#pragma unroll
    for (int i = 0; i < NB; i++) {
      const int ord = k0 / BLOCK + i;
      // unconditional read of a clamped index (nblk >= 1): a load under a branch could not be started early
      st.bid[i] = plan[2 * (ord < nblk ? ord : nblk - 1) + 1];
      st.live[i] = ord < nblk;
    }
    return st;
  }
  // stored [m][k] (part_k) or [k][m] (part_r); k / BLOCK picks the block when a step spans several
  __device__ __forceinline__ Part part_k(int row, int k) const { return Part{(int64_t)row * BLOCK + k % BLOCK, true, k / BLOCK, k}; }
  __device__ __forceinline__ Part part_r(int row, int k) const { return Part{(int64_t)(k % BLOCK) * BLOCK + row, true, k / BLOCK, k}; }
  __device__ __forceinline__ int64_t scalar_k(const Step &st, int i) const { return (int64_t)st.bid[i] * (BLOCK * BLOCK) + st.kin; }
  __device__ __forceinline__ int64_t scalar_r(const Step &st, int i) const { return (int64_t)st.bid[i] * (BLOCK * BLOCK) + st.kin * BLOCK; }
};

template <typename T, int BLOCK> struct DenseView {                   // element (n, k): dense row/col n, reduction position k
  const T *base; table_ptr plan; int nblk; int64_t ld; int n0, NF;
  static constexpr int NB = StepBlocks<T, BLOCK>::NB;
  struct Step { int32_t pos[NB]; bool live[NB]; int kin; int klim; };  // position of each block in the dense operand, whether it exists
  __device__ __forceinline__ Step step(int k0) const {
    Step st;
    st.kin = k0 % BLOCK;
    st.klim = 1 << 30;
#pragma unroll
    for (int i = 0; i < NB; i++) {
      const int ord = k0 / BLOCK + i;
      st.pos[i] = plan[2 * (ord < nblk ? ord : nblk - 1)];
      st.live[i] = ord < nblk;
    }
    return st;
  }
  // stored [n][k] (part_k) or [k][n] (part_r); rows past the free dimension are zero-filled
  __device__ __forceinline__ Part part_k(int row, int k) const { return Part{(int64_t)(n0 + row) * ld + k % BLOCK, n0 + row < NF, k / BLOCK, k}; }
  __device__ __forceinline__ Part part_r(int row, int k) const { return Part{(int64_t)(k % BLOCK) * ld + n0 + row, n0 + row < NF, k / BLOCK, k}; }
  __device__ __forceinline__ int64_t scalar_k(const Step &st, int i) const { return (int64_t)st.pos[i] + st.kin; }
  __device__ __forceinline__ int64_t scalar_r(const Step &st, int i) const { return ((int64_t)st.pos[i] + st.kin) * ld; }
};

template <int BLOCK, bool WIDE> struct XsdShape {
  // Tile of the dense free dimension.  Wide tiles for block 32 and 128: a wavefront then reuses each fragment of the
  // sparse block for two or four MFMAs (LDS reads per MFMA are what bounds these kernels); measured +13 % at block 32.
  // The narrow shape serves free dimensions up to 64 (the head dimension of an attention product), where a wide
  // tile would be mostly padding.
  static constexpr int TN = !WIDE ? 64 : BLOCK == 64 ? 128 : BLOCK >= 32 ? 256 : 64;
  // wide: 32 -> 1x4 wavefronts of 32x64; 64 -> 2x2 of 32x64; 128 -> 2x2 of 64x128.  narrow: 16 -> 1x4 of 16x16;
  // 32 -> 2x2 of 16x32; 64 -> 2x2 of 32x32; 128 -> 2x2 of 64x32
  static constexpr int WGM = (WIDE ? BLOCK >= 64 : BLOCK >= 32) ? 2 : 1;
  static constexpr int WGN = 4 / WGM;
};

// Which (batch, tile of the free dimension, position in the dispatch order) a workgroup of the dsd / dds kernels takes.
// Segment index fastest: consecutive workgroups (same XCD after the re-numbering) walk the segments of a head against one
// slab of columns of the dense operand, which then stays in L2 between its uses.  With a dispatch order (g.order:
// longest segments first, short launches only) "first" has to mean first on every XCD: an XCD works on a contiguous
// eighth of the launch, so inside its eighth the position in the order is the slow index and the tile the fast one.
// One batch with a number of tiles that divides by 8: every XCD gets all segments for its own tiles; a batch that
// divides by 8: every XCD gets whole batches.
__device__ __forceinline__ void xsd_work_item(const XsdArgs &g, int n_tiles, int &z, int &nt, int &seg0) {
  const int64_t per_z = (int64_t)g.width * n_tiles, total = per_z * g.Z;
  const int64_t w = xcd_remap(blockIdx.x, total);
  z = (int)(w / per_z);
  nt = (int)((w % per_z) / g.width);
  seg0 = (int)((w % per_z) % g.width);
  if (g.order && total % 8 == 0) {
    const int64_t chunk = total / 8, p = w % chunk;
    const int x = (int)(w / chunk);
    if (g.Z == 1 && n_tiles % 8 == 0) {
      const int tpx = n_tiles / 8;
      seg0 = (int)(p / tpx);
      nt = x * tpx + (int)(p % tpx);
    } else if (g.Z % 8 == 0) {
      const int64_t q = p % per_z;
      z = x * (g.Z / 8) + (int)(p / per_z);
      seg0 = (int)(q / n_tiles);
      nt = (int)(q % n_tiles);
    }
  }
}

// (at least two wavefronts per SIMD: the 128 x 256 tile of block 128 would otherwise take 266 registers and run alone)
template <typename T, int BLOCK, bool WIDE, bool SP_TRANS, bool DN_KCONTIG, bool OUT_NCONTIG>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) k_xsd(XsdArgs g) {
  typedef XsdShape<BLOCK, WIDE> S;
  typedef TileGemm<T, BLOCK, S::TN, S::WGM, S::WGN, !SP_TRANS, DN_KCONTIG, OUT_NCONTIG> G;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int n_tiles = (g.NF + S::TN - 1) / S::TN;
  int z, nt, seg0;
  xsd_work_item(g, n_tiles, z, nt, seg0);
  const int seg = g.order ? as_table(g.order)[seg0] : seg0;   // longest first only where the launch is short (see the dispatcher)
  const table_ptr hd = as_table(g.lut) + 6 * (int64_t)seg;
  const int offset = hd[0], seglen = hd[1], column = hd[2], depth = hd[3];
  const int nblk = seglen / BLOCK;
  if (nblk == 0) {
    // The table carries zero-length segments.  One that stands alone is an empty row/column of the layout and
    // must zero-fill its output tile; one that follows a real segment of the same row/column must not touch it.
    if (seg > 0 && hd[-6 + 2] == column && hd[-6 + 3] == depth) return;
  }
  const int t0 = (offset - 6 * g.width) / g.div2;   // first block of the segment in table order
  SparseView<T, BLOCK, SP_TRANS> sv;
  sv.base = reinterpret_cast<const T *>(g.sp) + z * g.sp_sz; sv.plan = as_table(g.plan) + 2 * (int64_t)t0; sv.nblk = nblk;
  DenseView<T, BLOCK> dv;
  dv.base = reinterpret_cast<const T *>(g.dn) + z * g.dn_sz + depth * g.dn_sh; dv.plan = sv.plan; dv.nblk = nblk; dv.ld = g.ldd;
  dv.n0 = nt * S::TN; dv.NF = g.NF;
  T *oz = reinterpret_cast<T *>(g.out) + z * g.out_sz + depth * g.out_sh;
  const int NF = g.NF, n0 = nt * S::TN;
  const int64_t ldo = g.ldo;
  // r, c = (m, n) when the output has n contiguous, (n, m) otherwise; c is the first of a 16-byte chunk
  // streaming stores: the dense result is not read again by the sparse chain and should not displace what is
  auto store = [&](int r, int c, u32x4 v) {
    if constexpr (OUT_NCONTIG) {
      if (n0 + c < NF) __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(oz + ((int64_t)column * BLOCK + r) * ldo + n0 + c));
    } else {
      if (n0 + r < NF) __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(oz + (int64_t)(n0 + r) * ldo + column * BLOCK + c));
    }
  };
  if (nblk == 0) {   // nothing to read (the views below assume at least one block): write the zeros and leave
    const u32x4 zero = {0u, 0u, 0u, 0u};
    constexpr int VE = 16 / (int)sizeof(T), CW = OUT_NCONTIG ? S::TN : BLOCK;   // chunks run along the contiguous index
    for (int i = threadIdx.x; i < BLOCK * S::TN / VE; i += 256) store(i / (CW / VE), (i % (CW / VE)) * VE, zero);
    return;
  }
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

template <typename T, int BLOCK, int SPLIT> int launch_sdd_split(const SddArgs &g, bool a_kc, bool b_kc, hipStream_t st) {
  constexpr int TT = BLOCK / SPLIT, WG = SddShape<TT>::WG;
  const int64_t n_wg = g.n_groups * g.Z * (SPLIT * SPLIT);
  if (n_wg <= 0) return BSP_OK;
  dim3 grid((unsigned)n_wg), blockdim(64 * WG * WG);
#define BSP_SDD_LAUNCH(AK, BK)                                                                                   \
  hipLaunchKernelGGL((k_sdd_split<T, BLOCK, SPLIT, AK, BK>), grid, blockdim,                                    \
                     (TileGemm<T, TT, TT, WG, WG, AK, BK, true>::SMEM_BYTES), st, g)
  if (a_kc && b_kc) BSP_SDD_LAUNCH(true, true);
  else if (a_kc && !b_kc) BSP_SDD_LAUNCH(true, false);
  else if (!a_kc && b_kc) BSP_SDD_LAUNCH(false, true);
  else BSP_SDD_LAUNCH(false, false);
#undef BSP_SDD_LAUNCH
  return BSP_OK;
}

template <typename T> int launch_sdd(const SddArgs &g, int block, int pack, bool a_kc, bool b_kc, hipStream_t st) {
  // fewer than two workgroups per CU: four 64 x 64 workgroups per 128-block instead of one
  if (block == 128 && pack == 1 && g.n_groups * g.Z < 512) return launch_sdd_split<T, 128, 2>(g, a_kc, b_kc, st);
  if (block == 16 && pack == 4) return launch_sdd_tp<T, 16, 4>(g, a_kc, b_kc, st);
  if (block == 16 && pack == 2) return launch_sdd_tp<T, 16, 2>(g, a_kc, b_kc, st);
  if (block == 16 && pack == 1) return launch_sdd_tp<T, 16, 1>(g, a_kc, b_kc, st);
  if (block == 32 && pack == 2) return launch_sdd_tp<T, 32, 2>(g, a_kc, b_kc, st);
  if (block == 32 && pack == 1) return launch_sdd_tp<T, 32, 1>(g, a_kc, b_kc, st);
  if (block == 64 && pack == 1) return launch_sdd_tp<T, 64, 1>(g, a_kc, b_kc, st);
  if (block == 128 && pack == 1) return launch_sdd_tp<T, 128, 1>(g, a_kc, b_kc, st);
  return BSP_ERR_UNSUPPORTED;
}

template <typename T, int BLOCK, bool WIDE> int launch_xsd_bw(const XsdArgs &g0, bool sp_trans, bool dn_kc, bool out_nc, hipStream_t st) {
  typedef XsdShape<BLOCK, WIDE> S;
  const int64_t n_wg = (int64_t)g0.width * ((g0.NF + S::TN - 1) / S::TN) * g0.Z;
  if (n_wg <= 0) return BSP_OK;
  if (n_wg >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  // Longest segments first only in short launches (a few workgroups per CU), where the last workgroups to start
  // decide when the launch ends: 7 % on an 8192 x 4096 x 4096 linear layer at block 128 and 10 % density (1024
  // workgroups).  A long launch balances by itself and reads the sparse blocks in storage order without it (1 %
  // faster at 65536 workgroups).
  XsdArgs g = g0;
  if (n_wg > 16 * 256) g.order = nullptr;
  dim3 grid((unsigned)n_wg), blockdim(256);
#define BSP_XSD_LAUNCH(ST, DK, ON)                                                                               \
  hipLaunchKernelGGL((k_xsd<T, BLOCK, WIDE, ST, DK, ON>), grid, blockdim,                                       \
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

template <typename T, int BLOCK> int launch_xsd_b(const XsdArgs &g, bool sp_trans, bool dn_kc, bool out_nc, hipStream_t st) {
  if (g.NF > 64 && XsdShape<BLOCK, true>::TN > 64) return launch_xsd_bw<T, BLOCK, true>(g, sp_trans, dn_kc, out_nc, st);
  return launch_xsd_bw<T, BLOCK, false>(g, sp_trans, dn_kc, out_nc, st);
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
// dsd / dds for a wide free dimension at blocks 64 / 128, 16-bit (matmul_dl.hip): same return convention
int xsd_dl(int dtype, const XsdArgs &g, int block, bool sp_trans, bool dn_kc, bool out_nc, hipStream_t st);
// sdd with a long reduction at blocks of 32, from the group plan alone (matmul_dl.hip): 2 = launched and every block written
int sdd_dl(int dtype, const SddArgs &g, int block, bool rowpair_plan, bool a_kc, bool b_kc, hipStream_t st);
int sdd128_splitk(int dtype, const SddArgs &g, int parts, float *ws, bool a_kc, bool b_kc, hipStream_t st);

}  // namespace bsp
