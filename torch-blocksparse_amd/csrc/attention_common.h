// Shared pieces of the fused attention kernels (attention_core.hip: rows of up to 8 tiles, the row's scores in
// registers; attention_long.hip: rows of any length, block after block): the LDS tile ring of direct global -> LDS
// loads, its swizzles, the transposing operand reads, the result stores, the tile tables of small blocks.
#ifndef BSP_ATTENTION_COMMON_H
#define BSP_ATTENTION_COMMON_H
#include "matmul_generic.h"
#include "softmax_common.h"
#include <type_traits>

namespace bsp {

struct AttnArgs {
  const void *x, *y1, *y2;   // forward: q, k, v; backward: do, v, k
  const void *p_in;          // backward: the saved softmax
  void *p_out, *o;           // forward: p, o; backward: ds, dq
  const void *o_in;          // backward: the forward result o
  float *delta;              // backward: sum_d do . o of every row, [Z][H] rows delta_sh apart (row kernels write it when given, the column kernel reads it)
  int64_t delta_sh;
  void *o2;                  // column kernel of the backward pass: dv (o is dk)
  int64_t o2_sz, o2_sh, o2_ld;
  float *partial;            // ... the slots of the long columns' parts, [Z][n_slots][dk, dv][64][D]
  const int32_t *split_lut;  // ... per long column (head, column, first slot, parts)
  int n_slots, n_split;
  int64_t oin_sz, oin_sh, oin_ld;
  int64_t x_sz, x_sh, x_ld, y1_sz, y1_sh, y1_ld, y2_sz, y2_sh, y2_ld, o_sz, o_sh, o_ld, pin_sz, pout_sz;
  float scale;
  const int32_t *lut;        // the softmax table (softmax.py:201-221): per block-row (size, offset), per block (id, col, row, head)
  const void *rpe; int64_t rpe_sz, rpe_sh, rpe_sr;
  const void *kpm; int64_t kpm_sz; int kpm_mul;
  const void *attn; int64_t attn_sr; int attn_mul;
  int Z, H, R;
};

namespace {

// LDS stages of the tile ring: loads run (stages - 1) tiles ahead of their use; three at head dimension 128, where a
// tile is 16 KiB and a launch may ask for 64 KiB of dynamic LDS without further ado
template <int D> constexpr int ring_stages() { return D == 64 ? 4 : 3; }

// cache-policy argument of the direct-to-LDS load for data that is read once (the tiles of p in the backward kernels): the
// non-temporal bit, so that the lines do not displace the dense tiles that the workgroups of a (batch, head) share
#define BSP_LOAD_ONCE 2
#define BSP_GLOBAL_PTR(p) ((const void __attribute__((address_space(1))) *)(p))
#define BSP_LDS_PTR(p) ((void __attribute__((address_space(3))) *)(p))
// Wait until at most n vector-memory operations of this wavefront are outstanding AND all of its LDS reads have returned.
// The second half matters before the barrier of a ring step: the barrier lets other wavefronts start the direct-to-LDS
// load that overwrites the stage this wavefront read last, and a read that is still in flight then can return the new
// tile's bytes (the compiler is free to leave the wait for a read's data behind the barrier, next to its first use;
// seen as one wrong block in 150000 at full occupancy).
#define BSP_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | (0x7 << 4) | (0x0 << 8))

// Tiles of 64 rows x D elements travel from global memory straight into LDS (global_load_lds_dwordx4: 16 bytes per
// lane, 1 KiB of consecutive LDS per wavefront-level load), so their rows lie unpadded, 2 D bytes apart, and the bank
// conflicts of the reads are avoided by an XOR swizzle of the 16-byte chunks inside a row, applied by choosing which
// global chunk each lane fetches.  Two swizzles, one per way a tile is read:
//   tiles of the first product (16-byte reads, sixteen lanes per clock, the lanes' rows differ in bits 0, 1, 3, 4):
//     D = 64 (rows r, r + 2 start in the same bank): chunk c of row r at slot c ^ (bit 1 | bit 3 << 1 | bit 4 << 2);
//     D = 128 (every row starts in bank 0): slot c ^ (bits 0, 1 | bits 3, 4 << 2);
//   tiles of the second product (transposing reads: a 16-lane group takes 32 bytes, a pair of chunks, from each of four
//     consecutive rows; the group served with it reads rows 8 further on): pair p of row r at pair slot
//     p ^ (r & 3) ^ (bit 3) for D = 64, p ^ 2 (r & 3) ^ (bit 3) for D = 128.
template <int D> __device__ __forceinline__ int swz_first(int r) {
  return D == 64 ? (((r >> 1) & 1) | (((r >> 3) & 3) << 1)) : ((r & 3) | (((r >> 3) & 3) << 2));
}
template <int D> __device__ __forceinline__ int swz_second(int r) {
  return D == 64 ? ((r & 3) ^ ((r >> 3) & 1)) : (((r & 3) << 1) ^ ((r >> 3) & 1));
}
// byte offsets inside a tile
template <int D> __device__ __forceinline__ int first_offset(int r, int chunk) { return r * (2 * D) + ((chunk ^ swz_first<D>(r)) << 4); }
template <int D> __device__ __forceinline__ int second_offset(int r, int col) {   // col in elements, a multiple of 4
  const int chunk = col >> 3, pair = (chunk >> 1) ^ swz_second<D>(r);
  return r * (2 * D) + (((pair << 1) | (chunk & 1)) << 4) + ((col & 7) << 1);
}



// Four operand fragments of the second product through the transposing LDS read: for each of four LDS addresses, rows
// 0..3 (reduction indices 0..3 of the lane's column) at the address and rows 4..7 at the address + HI bytes.  Written as
// one assembly block with its own wait: the compiler would otherwise, before every such read, wait for all direct-to-LDS
// loads in flight (it cannot tell that they fill other stages of the ring), which would undo the prefetch.
template <typename T, int HI>
__device__ __forceinline__ void tr_frags4(typename Mma16<T>::frag_t (&f)[4], uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3) {
  s16x4 lo0, hi0, lo1, hi1, lo2, hi2, lo3, hi3;
  asm volatile(
      "ds_read_b64_tr_b16 %0, %8\n\t"
      "ds_read_b64_tr_b16 %1, %8 offset:%12\n\t"
      "ds_read_b64_tr_b16 %2, %9\n\t"
      "ds_read_b64_tr_b16 %3, %9 offset:%12\n\t"
      "ds_read_b64_tr_b16 %4, %10\n\t"
      "ds_read_b64_tr_b16 %5, %10 offset:%12\n\t"
      "ds_read_b64_tr_b16 %6, %11\n\t"
      "ds_read_b64_tr_b16 %7, %11 offset:%12\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(lo0), "=&v"(hi0), "=&v"(lo1), "=&v"(hi1), "=&v"(lo2), "=&v"(hi2), "=&v"(lo3), "=&v"(hi3)
      : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "n"(HI));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  typedef typename Mma16<T>::frag_t frag_t;
  f[0] = __builtin_bit_cast(frag_t, (s16x8)__builtin_shufflevector(lo0, hi0, 0, 1, 2, 3, 4, 5, 6, 7));
  f[1] = __builtin_bit_cast(frag_t, (s16x8)__builtin_shufflevector(lo1, hi1, 0, 1, 2, 3, 4, 5, 6, 7));
  f[2] = __builtin_bit_cast(frag_t, (s16x8)__builtin_shufflevector(lo2, hi2, 0, 1, 2, 3, 4, 5, 6, 7));
  f[3] = __builtin_bit_cast(frag_t, (s16x8)__builtin_shufflevector(lo3, hi3, 0, 1, 2, 3, 4, 5, 6, 7));
}

// acc[j][e] = out[row lane % 16][column 16j + 4 * (lane / 16) + e] of a 16 x D slice -> the wavefront's piece of LDS ->
// stores of whole rows (16 bytes per lane, a row = D / 8 consecutive lanes)
template <typename T, int D> __device__ __forceinline__ void store_rows(T *cs, T *dst, int64_t ld, const f32x4 (&acc)[D / 16], int lane) {
  constexpr int LDK = D + 8, CPR = D / 8;
#pragma unroll
  for (int j = 0; j < D / 16; j++) {
    union { u32x2 raw; T e[4]; } pk;
#pragma unroll
    for (int e = 0; e < 4; e++) pk.e[e] = from_float<T>(acc[j][e]);
    *reinterpret_cast<u32x2 *>(cs + (lane & 15) * LDK + 16 * j + 4 * (lane >> 4)) = pk.raw;
  }
  __builtin_amdgcn_wave_barrier();   // LDS operations of one wavefront complete in order; this only pins the code order
#pragma unroll
  for (int i = 0; i < CPR / 4; i++) {
    const int c = lane + 64 * i;
    const u32x4 v = *reinterpret_cast<const u32x4 *>(cs + (c / CPR) * LDK + (c % CPR) * 8);
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(dst + (int64_t)(c / CPR) * ld + (c % CPR) * 8));
  }
  __builtin_amdgcn_wave_barrier();
}

// The wavefront's 16 rows of a 64 x 64 block of the sparse tensor (2 KiB of consecutive addresses), a lane holding
// columns 8 * (lane / 16) .. + 7 (c0) and 32 + 8 * (lane / 16) .. (c1) of row lane % 16: through the wavefront's piece of
// LDS (rows of 72 elements), then two stores of 1 KiB of consecutive addresses.  (Stored straight from the registers,
// every store instruction writes sixteen separate 64-byte pieces: measured, the forward kernel then takes 170 us
// instead of 107 without the stores.)
// The stores are non-temporal: p is 336 MB in the benchmark configuration, more than the caches hold, and is next read
// by the backward pass.  Stored the ordinary way its lines are allocated in L2 on their way out and the forward kernel
// moves its bytes at 3.8 TB/s (144 us); streamed out, at 4.8 TB/s (112 us).
template <typename T> __device__ __forceinline__ void store_block_rows(T *cs, T *dst, const u32x4 &c0, const u32x4 &c1, int lane) {
  T *w = cs + (lane & 15) * 72 + 8 * (lane >> 4);
  *reinterpret_cast<u32x4 *>(w) = c0;
  *reinterpret_cast<u32x4 *>(w + 32) = c1;
  __builtin_amdgcn_wave_barrier();   // LDS operations of one wavefront complete in order; this only pins the code order
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int c = lane + 64 * i;
    __builtin_nontemporal_store(*reinterpret_cast<const u32x4 *>(cs + (c >> 3) * 72 + (c & 7) * 8), reinterpret_cast<u32x4 *>(dst + c * 8));
  }
  __builtin_amdgcn_wave_barrier();
}

// Blocks of 16 and 32 (SUBS = 64 / block > 1): the kernels work on 64 x 64 tiles formed from SUBS x SUBS small blocks
// (SUBS consecutive block-rows by SUBS gathered block-columns, or the other way round in the column kernel); the table
// lists the tiles of each line, each with the ids of its blocks row by row, -1 where absent.  A
// wavefront's 16 rows lie in one row of small blocks (rs) and a lane's chunk of 8 columns in one small block: its id, or -1.
// t = the ids of the wavefront's row of small blocks in the tile (scalars, fetched once per block of the row; kept as a
// vector type: an array indexed in a select chain ends up in scratch memory, whose loads count as vector-memory
// operations and stall every wait of the tile ring)
typedef int i32x4 __attribute__((ext_vector_type(4)));
template <int SUBS> __device__ __forceinline__ int chunk_block_id(const i32x4 &t, int s, int q) {
  if constexpr (SUBS == 2) return s ? t[1] : t[0];           // columns 32s + 8q .. of the tile: small block column s
  else if constexpr (SUBS == 4) return s ? ((q >> 1) ? t[3] : t[2]) : ((q >> 1) ? t[1] : t[0]);   // small block column 2s + q / 2
  else return 0;
}
// the ids of the blocks of the tile's row rs of small blocks, from the tile's table entry (see entry_ints)
template <int SUBS> __device__ __forceinline__ i32x4 entry_ids(table_ptr e, int rs) {
  i32x4 t = {0, 0, 0, 0};
  if constexpr (SUBS > 1) {
#pragma unroll
    for (int c = 0; c < SUBS; c++) t[c] = e[8 + rs * SUBS + c];
  }
  return t;
}
// Table entries.  Blocks of 64: four ints (block id, block-column [the column kernel: block-row], ., .).  Smaller
// blocks: 8 + S * S ints, S = SUBS: (., ., ., ., the S block-columns [block-rows] gathered into the tile, then the ids of
// the tile's blocks, [block-row of the line][gathered block-column], -1 where absent): the tile's 64 columns [rows] are
// S groups of 64 / S consecutive ones, each group anywhere in the matrix.  Everything a tile needs is in its entry: one
// round of scalar loads, which the kernels issue a step ahead of the tile's loads.
template <int SUBS> constexpr int entry_ints() { return SUBS == 1 ? 4 : 8 + SUBS * SUBS; }
template <int SUBS> __device__ __forceinline__ int entry_group(table_ptr e, int g) { return SUBS == 1 ? e[1] : e[4 + g]; }
template <int SUBS> __device__ __forceinline__ i32x4 entry_groups(table_ptr e) {
  i32x4 t = i32x4{0, 0, 0, 0};
  if constexpr (SUBS == 1) {
    t[0] = e[1];
  } else {
#pragma unroll
    for (int g = 0; g < SUBS; g++) t[g] = e[4 + g];
  }
  return t;
}
// position (in elements) of the lane's chunk (columns 32s + 8q .. + 7 of the tile) in the matrix, from the tile's groups
template <int SUBS> __device__ __forceinline__ int64_t chunk_position(const i32x4 &groups, int s, int q) {
  constexpr int B = 64 / SUBS;
  if constexpr (SUBS == 1) return (int64_t)groups[0] * 64 + 32 * s + 8 * q;
  else return (int64_t)chunk_block_id<SUBS>(groups, s, q) * B + (32 * s + 8 * q) % B;
}
// position of element j (0 .. 63, any lane) of the tile
template <int SUBS> __device__ __forceinline__ int64_t element_position(const i32x4 &groups, int j) {
  constexpr int B = 64 / SUBS;
  int grp = groups[0];
#pragma unroll
  for (int g = 1; g < SUBS; g++) grp = (j / B == g) ? groups[g] : grp;
  return (int64_t)grp * B + j % B;
}
// the lane's chunk (row 16 * wave + lane % 16 of the tile, columns 32s + 8q ..) inside its small block, in elements
template <int SUBS> __device__ __forceinline__ int chunk_in_block(int wave, int qrow, int s, int q) {
  constexpr int B = 64 / SUBS;
  return ((16 * wave + qrow) % B) * B + (32 * s + 8 * q) % B;
}

// wait until at most c (0 .. 16; more is treated as 16) vector-memory operations are outstanding, exactly
__device__ __forceinline__ void wait_vm_exact(int c) {
  switch (c < 16 ? c : 16) {
    case 0: BSP_WAIT_VM(0); break;
    case 1: BSP_WAIT_VM(1); break;
    case 2: BSP_WAIT_VM(2); break;
    case 3: BSP_WAIT_VM(3); break;
    case 4: BSP_WAIT_VM(4); break;
    case 5: BSP_WAIT_VM(5); break;
    case 6: BSP_WAIT_VM(6); break;
    case 7: BSP_WAIT_VM(7); break;
    case 8: BSP_WAIT_VM(8); break;
    case 9: BSP_WAIT_VM(9); break;
    case 10: BSP_WAIT_VM(10); break;
    case 11: BSP_WAIT_VM(11); break;
    case 12: BSP_WAIT_VM(12); break;
    case 13: BSP_WAIT_VM(13); break;
    case 14: BSP_WAIT_VM(14); break;
    case 15: BSP_WAIT_VM(15); break;
    default: BSP_WAIT_VM(16); break;
  }
}

// wait until at most c (0, 2, 4, 6 or 8) vector-memory operations are outstanding; the instruction takes an immediate
__device__ __forceinline__ void wait_vm(int c) {
  if (c >= 8) BSP_WAIT_VM(8);
  else if (c >= 6) BSP_WAIT_VM(6);
  else if (c >= 4) BSP_WAIT_VM(4);
  else if (c >= 2) BSP_WAIT_VM(2);
  else BSP_WAIT_VM(0);
}


// Two fragments of the same kind (see tr_frags4).
template <typename T, int HI>
__device__ __forceinline__ void tr_frags2(typename Mma16<T>::frag_t (&f)[2], uint32_t a0, uint32_t a1) {
  s16x4 lo0, hi0, lo1, hi1;
  asm volatile(
      "ds_read_b64_tr_b16 %0, %4\n\t"
      "ds_read_b64_tr_b16 %1, %4 offset:%6\n\t"
      "ds_read_b64_tr_b16 %2, %5\n\t"
      "ds_read_b64_tr_b16 %3, %5 offset:%6\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(lo0), "=&v"(hi0), "=&v"(lo1), "=&v"(hi1)
      : "v"(a0), "v"(a1), "n"(HI));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  typedef typename Mma16<T>::frag_t frag_t;
  f[0] = __builtin_bit_cast(frag_t, (s16x8)__builtin_shufflevector(lo0, hi0, 0, 1, 2, 3, 4, 5, 6, 7));
  f[1] = __builtin_bit_cast(frag_t, (s16x8)__builtin_shufflevector(lo1, hi1, 0, 1, 2, 3, 4, 5, 6, 7));
}

// A tile that is read both ways (16-byte reads along a row and transposing reads): the swizzle of the second product
// with the two halves of a pair exchanged in rows with bit 4 set.  The transposing reads take whole pairs and do not
// notice; of the sixteen rows of a 16-byte read (bits 0, 1, 3, 4 differ) the pair swizzle separates four and the
// exchanged halves the other two, so that these are free of bank conflicts as well.
template <int D> __device__ __forceinline__ int dual_slot(int r, int chunk) {
  return ((((chunk >> 1) ^ swz_second<D>(r)) << 1) | ((chunk & 1) ^ ((r >> 4) & 1)));
}
template <int D> __device__ __forceinline__ int dual_offset(int r, int col) {   // col in elements
  return r * (2 * D) + (dual_slot<D>(r, col >> 3) << 4) + ((col & 7) << 1);
}

}  // namespace
// rows of more than BSP_ATTENTION_MAX_ROW_BLOCKS tiles (attention_long.hip)
int attention_long(int dtype, const AttnArgs &a, int D, int block, bool bwd, hipStream_t st);
// dk and dv, one workgroup per column of tiles (attention_kv.hip)
int attention_kv(int dtype, const AttnArgs &a, int D, int block, hipStream_t st);
}  // namespace bsp
#endif
