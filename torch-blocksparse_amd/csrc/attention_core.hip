// The attention chain of one block-row in one kernel, blocks of 64 (and, on tiles of 64 x 64 formed from them, of 32
// and 16), fp16 / bf16, for gfx950.
//
// The reference's attention modules run three operators per call: scores = sdd(q, k^T), softmax in place, context =
// dsd(p, v) (deepspeedsparseselfattention.py:152-157; attention.py:190-202), and autograd adds five more launches for
// the backward pass.  Every one of them streams the [Z, nnz, 64, 64] sparse tensor through HBM: at head_dim 64 the
// chain is bound by that traffic, not by arithmetic.  Here a workgroup owns one block-row of one (batch, head); each
// of its four wavefronts keeps 16 rows of ALL nonzero blocks of that block-row in MFMA accumulators, so the scores
// never leave the registers between the three steps:
//
//   forward  : s = q . k^T  ->  p = softmax(s * scale + rpe + key-padding mask + attention mask)  ->  o = p . v
//              p is written once (the backward pass needs it), o once; the scores are never stored.
//   backward : dp = do . v^T  ->  ds = p * (dp - sum(p * dp)) * scale  ->  dq = ds . k
//              p is read once; ds is written only if the caller wants it (dk = ds^T . q and dv = p^T . do then are
//              ordinary dsd products; otherwise the column kernel of attention_kv.hip computes both from p).
//
// Arithmetic mirrors the separate operators: the scores (and dp) are rounded to the storage type before the softmax
// sees them, as they are when sdd stores them; the softmax is computed in fp32 (log2 domain) and rounded before the
// second product consumes it.
//
// Register layout.  The first product is computed transposed, s^T = k_tile . q^T, with the MFMA 16x16x32: its A operand
// (rows of the result) is a k tile read from LDS, its B operand the wavefront's 16 q rows, loaded once from global
// memory straight into operand registers.  A lane then holds, for q row lane % 16, four result rows 4 * (lane / 16) + e
// of each 16-row sub-tile.  The k rows are dealt to the sub-tiles so that these are keys 32s + 8 * (lane / 16) + 0..7
// of the block (s = 0, 1): eight consecutive keys, which is at once a 16-byte piece of a row of p (stored as it is) and
// the B-operand fragment of the second product o^T = v^T . p^T (no shuffle, no LDS round trip).  v^T comes from the v
// tile in LDS through the transposing LDS read.
//
// Blocks of 32 / 16 (SUBS = 2 / 4): a tile is SUBS consecutive block-rows by SUBS block-columns gathered from anywhere in
// those rows (the tile's table entry names them): its 64 k / v rows are SUBS groups of consecutive rows, a wavefront
// loads 16 rows, which lie in one group, and the lane's 8-key chunk lies in one small block, whose id (-1: absent) comes
// from the tile table.
#include "attention_common.h"

namespace bsp {
namespace {

// D = head dimension (64 or 128); NB = most blocks a block-row may hold (the host picks the bucket from the table's
// longest row); EXTRA = a relative position embedding or an attention mask is present.
template <typename T, int D, int NB, bool EXTRA, int SUBS = 1>
__global__ void __launch_bounds__(256, (EXTRA || D > 64) ? 2 : 3) k_attn64_fwd(AttnArgs a) {
  typedef Mma16<T> M;
  typedef typename M::frag_t frag_t;
  typedef Pack<T, 8> P8;
  constexpr int NK = D / 32;            // MFMA steps along the head dimension in the first product
  constexpr int ND = D / 16;            // 16-column sub-tiles of the result of the second product
  constexpr int LDK = D + 8;            // row of the staging slice of the result (16 bytes of padding)
  constexpr int TB = 64 * D * 2;        // bytes of a tile
  constexpr int LW = TB / 1024 / 4;     // wavefront-level loads per wavefront and tile
  constexpr int CPR = D / 8;            // 16-byte chunks per tile row
  constexpr int kStages = ring_stages<D>();
  // dynamic LDS: the tile ring (at the end it stages the results: per wavefront a slice of the dense and one of the
  // sparse result), then the key-padding terms
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  unsigned char *ring = smem;
  T *stage_out = reinterpret_cast<T *>(smem);
  float *kpm_s = reinterpret_cast<float *>(smem + kStages * TB);
  static_assert(4 * 16 * (LDK + 72) * 2 <= kStages * TB, "the staged results fit into the ring");
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t n_wg = (int64_t)a.Z * a.H * a.R;
  const int64_t wg = xcd_remap(blockIdx.x, n_wg);
  // block-rows from the last one down (the longest rows of a causal layout first), all rows of a (batch, head) in a
  // row: its k and v tiles stay in the L2 of the XCD that works on it
  // (with per-element masks, which the batches share: the batches of a block-row next to each other, so that the second
  // one finds the row's mask values in L2)
  int br, h, z;
  if constexpr (EXTRA) {
    z = (int)(wg % a.Z);
    br = a.R - 1 - (int)((wg / a.Z) % a.R);
    h = (int)(wg / a.Z / a.R);
  } else {
    br = a.R - 1 - (int)(wg % a.R);
    const int zh = (int)(wg / a.R);
    h = zh % a.H, z = zh / a.H;
  }
  const table_ptr lut = as_table(a.lut);
  const int size = lut[2 * (h * a.R + br) + 0];   // header (size, offset), softmax.py:30-32
  const int offset = lut[2 * (h * a.R + br) + 1];
  const int qrow = lane & 15, q = lane >> 4;
  const int64_t row = (int64_t)br * 64 + wave * 16 + qrow;   // the lane's row of the dense matrices (first product)
  T *cs = stage_out + wave * 16 * LDK;
  T *stage_p = stage_out + 4 * 16 * LDK + wave * (16 * 72);
  T *po = reinterpret_cast<T *>(a.o) + z * a.o_sz + h * a.o_sh + ((int64_t)br * 64 + wave * 16) * a.o_ld;
  f32x4 o[ND];
#pragma unroll
  for (int j = 0; j < ND; j++) o[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  if (size <= 0) {   // an empty block-row: its rows of the dense result are zero, as the dsd operator leaves them
    store_rows<T, D>(cs, po, a.o_ld, o, lane);
    return;
  }
  const table_ptr core = lut + offset;
  constexpr int ES = entry_ints<SUBS>();
  const int wgroup = (16 * wave) / (64 / SUBS);   // the group of the tile's rows (k, v: of the gathered columns) that the wavefront's 16 lie in
  int32_t bid[NB];
#pragma unroll
  for (int b = 0; b < NB; b++) bid[b] = core[ES * (b < size ? b : 0)];   // blocks past the end repeat the first one (valid to read, never used)
  i32x4 tid_[NB];   // small blocks: the ids of the wavefront's row of small blocks in each tile
#pragma unroll
  for (int b = 0; b < NB; b++) tid_[b] = entry_ids<SUBS>(core + ES * (b < size ? b : 0), wgroup);
  const T *px = reinterpret_cast<const T *>(a.x) + z * a.x_sz + h * a.x_sh + row * a.x_ld + 8 * q;
  frag_t xq[NK];
#pragma unroll
  for (int s2 = 0; s2 < NK; s2++) xq[s2] = *reinterpret_cast<const frag_t *>(px + 32 * s2);
  const T *py1 = reinterpret_cast<const T *>(a.y1) + z * a.y1_sz + h * a.y1_sh;
  const T *py2 = reinterpret_cast<const T *>(a.y2) + z * a.y2_sz + h * a.y2_sh;
  // The unified tile sequence of the workgroup: y1 tiles of blocks 0 .. size - 1, then y2 tiles of the same blocks.
  // Tile n lives in ring stage n % kStages.  Per-lane part of the addresses: load i of this wavefront covers rows
  // (wave * LW + i) * (64 / CPR) .. of the tile, lane l its row l / CPR and the chunk that belongs into slot l % CPR.
  int64_t off1[LW], off2[LW];
#pragma unroll
  for (int i = 0; i < LW; i++) {
    const int r = (wave * LW + i) * (64 / CPR) + lane / CPR, slot = lane % CPR;
    off1[i] = (int64_t)r * a.y1_ld + ((slot ^ swz_first<D>(r)) << 3);
    off2[i] = (int64_t)r * a.y2_ld + (((((slot >> 1) ^ swz_second<D>(r)) << 1) | (slot & 1)) << 3);
  }
  const int total = 2 * size;
  int next_col;
  // the block-column of tile n, from the table (a scalar load; clamped past the end)
  // (small blocks: the block-column of the group that this wavefront loads; off1 / off2 count rows from the tile's first)
  auto tile_col = [&](int n) {
    const int m = n < size ? n : n - size;
    return entry_group<SUBS>(core + ES * (m < size ? m : size - 1), wgroup) - wgroup;
  };
  auto issue = [&](int n, int col) {
    unsigned char *st = ring + (n % kStages) * TB + wave * LW * 1024;
    if (n < size) {
      const T *base = py1 + (int64_t)col * (64 / SUBS) * a.y1_ld;
#pragma unroll
      for (int i = 0; i < LW; i++) __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(base + off1[i]), BSP_LDS_PTR(st + i * 1024), 16, 0, 0);
    } else {
      const T *base = py2 + (int64_t)col * (64 / SUBS) * a.y2_ld;
#pragma unroll
      for (int i = 0; i < LW; i++) __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(base + off2[i]), BSP_LDS_PTR(st + i * 1024), 16, 0, 0);
    }
  };
  // Before tile n is read: this wavefront's loads of it have landed (all but those of the tiles issued after it,
  // kStages - 2 of them or fewer near the end), then the barrier (everybody's have, and everybody is done reading tile n - 1), then the
  // load of tile n + kStages - 1 into the stage that tile n - 1 used.
  // With per-element masks (EXTRA) the mask values of block b + 1 are fetched into registers while block b is worked on:
  // four loads per lane and block (two masks, two chunks of eight columns; a mask that is not given is replaced by the
  // other one, so that the count is fixed), issued right before the tile load of a step, the first ones (block 0)
  // before the last tile of the prologue.  They share the counter of the tile loads and complete in order with them, so
  // the wait for tile n also counts the mask loads issued after it: those of blocks max(0, n - kStages + 3) .. n, as far
  // as they were issued (blocks 0 .. size).
  constexpr int MASK_LOADS = 4;
  auto arrive = [&](int n) {
    if constexpr (EXTRA) {
      int tiles = total - 1 - n;
      tiles = tiles < kStages - 2 ? (tiles < 0 ? 0 : tiles) : kStages - 2;
      const int first = n - kStages + 3 > 0 ? n - kStages + 3 : 0, last = n < size ? n : size;
      wait_vm_exact(LW * tiles + MASK_LOADS * (last >= first ? last - first + 1 : 0));
    } else {
      const int rem = total - 1 - n;
      if (rem >= kStages - 2) BSP_WAIT_VM(LW * (kStages - 2));
      else if (kStages > 3 && rem == 1) BSP_WAIT_VM(LW);
      else BSP_WAIT_VM(0);
    }
    asm volatile("" ::: "memory");                     // (the compiler must not move LDS accesses across the barrier)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  auto advance = [&](int n) {
    if (n + kStages - 1 < total) issue(n + kStages - 1, next_col);
    next_col = tile_col(n + kStages);                  // the table runs one step ahead of the load that uses it
  };
  auto step = [&](int n) {
    arrive(n);
    advance(n);
  };
  // the mask values of the lane's two chunks of block b (address: softmax.py:50-55, 67-70)
  auto load_masks = [&](int b, P8 (&pr)[2], P8 (&pa)[2]) {
    const i32x4 groups = entry_groups<SUBS>(core + ES * (b < size ? b : 0));   // the block-column(s) of the tile
#pragma unroll
    for (int s = 0; s < 2; s++) {
      const int64_t gcol = chunk_position<SUBS>(groups, s, q);
      const T *attn = reinterpret_cast<const T *>(a.attn) + row * a.attn_sr + gcol;
      const T *rpe = reinterpret_cast<const T *>(a.rpe) + z * a.rpe_sz + h * a.rpe_sh + row * a.rpe_sr + gcol;
      pr[s].load(a.rpe ? rpe : attn);
      pa[s].load(a.attn ? attn : rpe);
    }
  };
  // The key-padding term of every column of the block-row (softmax.py:104-106, 122-124), fetched once per workgroup
  // and kept in LDS as the value that is added to the logits; the first barrier below orders it before its readers.
  P8 kp;
  const bool kpm_lane = a.kpm && tid < NB * 8;
  {
    if (kpm_lane) {
      // the lane's eight columns of tile b: in one group of the tile; its block-column from the table
      constexpr int B = 64 / SUBS;
      const int b = tid >> 3, j = (tid & 7) * 8;
      const int col = core[ES * (b < size ? b : 0) + (SUBS == 1 ? 1 : 4 + j / B)];
      kp.load(reinterpret_cast<const T *>(a.kpm) + z * a.kpm_sz + (int64_t)col * B + j % B);
    }
  }
  // the first two tiles always exist (a row has at least one block); in a straight line, so that the wait for the
  // key-padding values counts exactly the loads issued after them
  issue(0, tile_col(0));
  issue(1, tile_col(1));
  {
    if (kpm_lane) {
      const float unit = logit_unit<T>();
#pragma unroll
      for (int e4 = 0; e4 < 8; e4 += 4) {
        f32x4 add;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const float m = to_float(kp.e[e4 + e]);
          add[e] = a.kpm_mul ? (m == 0.f ? -INFINITY : 0.f) : m * unit;
        }
        *reinterpret_cast<f32x4 *>(&kpm_s[tid * 8 + e4]) = add;
      }
    }
  }
  P8 pr[EXTRA ? NB + 1 : 1][2], pa[EXTRA ? NB + 1 : 1][2];
  if constexpr (EXTRA) load_masks(0, pr[0], pa[0]);
#pragma unroll
  for (int n = 2; n < kStages - 1; n++)
    if (n < total) issue(n, tile_col(n));
  next_col = tile_col(kStages - 1);

  // ---- first product: acc[b][jt][e] = (x . y1_b^T)[row lane % 16][key 32 * (jt / 2) + 8 * (lane / 16) + 4 * (jt % 2) + e]
  f32x4 acc[NB][4];
  // the k row that supplies result row m of sub-tile jt (see the file comment)
  const int krow0 = 8 * (qrow >> 2) + (qrow & 3);
  float mx = -INFINITY;
  int any_block = SUBS == 1;                           // small blocks: does the lane's row of small blocks hold any block?
#pragma unroll
  for (int b = 0; b < NB; b++)
    if (b < size) {
      if constexpr (EXTRA) {
        arrive(b);
        load_masks(b + 1, pr[b + 1], pa[b + 1]);       // (past the row's end: the last block's again, never used)
        advance(b);
      } else {
        step(b);
      }
      const unsigned char *tile = ring + (b % kStages) * TB;
      frag_t kf[4][NK];
#pragma unroll
      for (int jt = 0; jt < 4; jt++)
#pragma unroll
        for (int s2 = 0; s2 < NK; s2++)
          kf[jt][s2] = *reinterpret_cast<const frag_t *>(tile + first_offset<D>(32 * (jt >> 1) + 4 * (jt & 1) + krow0, 4 * s2 + q));
#pragma unroll
      for (int jt = 0; jt < 4; jt++) {
        acc[b][jt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s2 = 0; s2 < NK; s2++) acc[b][jt] = M::run(kf[jt][s2], xq[s2], acc[b][jt]);
      }
      if constexpr (EXTRA) {
        // the block's logits right away, with the mask values that were fetched during the previous block
        const float unit = logit_unit<T>(), sc = a.scale * unit;
#pragma unroll
        for (int s = 0; s < 2; s++) {
          float add[8];
          if (a.kpm != nullptr) {
#pragma unroll
            for (int e4 = 0; e4 < 8; e4 += 4)
              *reinterpret_cast<f32x4 *>(&add[e4]) = *reinterpret_cast<const f32x4 *>(&kpm_s[b * 64 + 32 * s + 8 * q + e4]);
          } else {
#pragma unroll
            for (int i = 0; i < 8; i++) add[i] = 0.f;
          }
          if constexpr (SUBS > 1) {                    // a chunk in an absent small block takes no part in the row
            const bool here = chunk_block_id<SUBS>(tid_[b], s, q) >= 0;
            any_block |= here;
            if (!here) {
#pragma unroll
              for (int i = 0; i < 8; i++) add[i] = -INFINITY;
            }
          }
#pragma unroll
          for (int i = 0; i < 8; i++) {
            float fx = fmaf(to_float(from_float<T>(acc[b][2 * s + (i >> 2)][i & 3])), sc, add[i]);   // softmax.py:112-116, 122-124
            if (a.rpe) fx = fmaf(to_float(pr[b][s].e[i]), unit, fx);                                 // :118-120
            if (a.attn) {                                                                            // :126-128, 'mul' mode :108-110
              const float m = to_float(pa[b][s].e[i]);
              fx += a.attn_mul ? (m == 0.f ? -INFINITY : 0.f) : m * unit;
            }
            acc[b][2 * s + (i >> 2)][i & 3] = fx;
            mx = fmaxf(mx, fx);
          }
        }
      }
    }

  // ---- between the products: the softmax on the wavefront's 16 rows.  A lane's
  // values of block b: two chunks (s = 0, 1) of eight consecutive columns 32s + 8 * (lane / 16) + i, i = 4t + e in
  // acc[b][2s + t][e].  The reductions over a row run over the lane's values, then over the four lanes that share it.
  frag_t pf[NB][2];
  T *pout = reinterpret_cast<T *>(a.p_out) + z * a.pout_sz + wave * 1024;   // the wavefront's 16 rows of block 0
  {
    const float unit = logit_unit<T>(), sc = a.scale * unit;
    const bool has_kpm = a.kpm != nullptr;
    if constexpr (!EXTRA) {
#pragma unroll
      for (int b = 0; b < NB; b++)
        if (b < size) {
#pragma unroll
          for (int s = 0; s < 2; s++) {
            float add[8];
            if (has_kpm) {
#pragma unroll
              for (int e4 = 0; e4 < 8; e4 += 4)
                *reinterpret_cast<f32x4 *>(&add[e4]) = *reinterpret_cast<const f32x4 *>(&kpm_s[b * 64 + 32 * s + 8 * q + e4]);
            } else {
#pragma unroll
              for (int i = 0; i < 8; i++) add[i] = 0.f;
            }
            if constexpr (SUBS > 1) {                    // a chunk in an absent small block takes no part in the row
              const bool here = chunk_block_id<SUBS>(tid_[b], s, q) >= 0;
              any_block |= here;
              if (!here) {
#pragma unroll
                for (int i = 0; i < 8; i++) add[i] = -INFINITY;
              }
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
              const float fx = fmaf(to_float(from_float<T>(acc[b][2 * s + (i >> 2)][i & 3])), sc, add[i]);   // softmax.py:112-116, 122-124
              acc[b][2 * s + (i >> 2)][i & 3] = fx;
              mx = fmaxf(mx, fx);
            }
          }
        }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16));                                  // :130
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    float sum = 0.f;
#pragma unroll
    for (int b = 0; b < NB; b++)
      if (b < size) {
#pragma unroll
        for (int jt = 0; jt < 4; jt++)
#pragma unroll
          for (int e = 0; e < 4; e++) { acc[b][jt][e] = exp_sub<T>(acc[b][jt][e], mx); sum += acc[b][jt][e]; }   // :131-132
      }
    sum += __shfl_xor(sum, 16);
    sum += __shfl_xor(sum, 32);
    const float inv = 1.f / sum;
    if constexpr (SUBS > 1) {   // rows of a small block-row without blocks (inside a tile-row that others keep alive): zeros for p . v
      any_block |= __shfl_xor(any_block, 16);
      any_block |= __shfl_xor(any_block, 32);
    }
#pragma unroll
    for (int b = 0; b < NB; b++)
      if (b < size) {
#pragma unroll
        for (int s = 0; s < 2; s++) {
          P8 y;
#pragma unroll
          for (int i = 0; i < 8; i++) {
            const float v = acc[b][2 * s + (i >> 2)][i & 3] * inv;                                    // :137
            y.e[i] = from_float<T>(SUBS > 1 && !any_block ? 0.f : v);
          }
          pf[b][s] = __builtin_bit_cast(frag_t, y.raw);
        }
      }
  }

  // ---- second product: o^T[d][row] += y2_b^T[d][key] . pf_b[key][row]; the y2 tiles continue the ring
  // a lane's part of the LDS addresses of its transposing reads: rows 8 * (lane / 16) + (lane % 16) / 4 (+ 4, + 32 as
  // immediate offsets: neither changes the swizzle), columns 16j + 4 * (lane % 4)
  const int tr_row = q * 8 + (qrow >> 2), tr_col = (qrow & 3) * 4;
  const uint32_t ring_lds = (uint32_t)(uintptr_t)BSP_LDS_PTR(ring);
  uint32_t tr_off[ND];
#pragma unroll
  for (int j = 0; j < ND; j++) tr_off[j] = second_offset<D>(tr_row, 16 * j + tr_col);
#pragma unroll
  for (int b = 0; b < NB; b++)
    if (b < size) {
      step(size + b);
      const uint32_t tile_lds = ring_lds + ((size + b) % kStages) * TB;
#pragma unroll
      for (int s = 0; s < 2; s++)
#pragma unroll
        for (int j4 = 0; j4 < ND; j4 += 4) {
          frag_t vf[4];
          const uint32_t t0 = tile_lds + s * (32 * 2 * D);
          tr_frags4<T, 4 * 2 * D>(vf, t0 + tr_off[j4], t0 + tr_off[j4 + 1], t0 + tr_off[j4 + 2], t0 + tr_off[j4 + 3]);
#pragma unroll
          for (int j = 0; j < 4; j++) o[j4 + j] = M::run(vf[j], pf[b][s], o[j4 + j]);
        }
    }
  // The sparse result leaves only now, although it has been ready since the softmax: on this architecture loads and
  // stores share one counter of outstanding operations, so stores issued before the second product would have to be
  // acknowledged by memory before the wait for its next tile could end (measured: the stores then cost their full
  // 50 us on top of the rest instead of overlapping with other workgroups).  The values are the operand registers pf.
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();                        // the ring is free: everybody is done reading the last tile
  asm volatile("" ::: "memory");
  store_rows<T, D>(cs, po, a.o_ld, o, lane);
  if (a.p_out == nullptr) return;   // p is not asked for (a forward pass without a backward pass to follow)
#pragma unroll
  for (int b = 0; b < NB; b++)
    if (b < size) {
      if constexpr (SUBS == 1) {
        store_block_rows<T>(stage_p, pout + (int64_t)bid[b] * 4096, __builtin_bit_cast(u32x4, pf[b][0]), __builtin_bit_cast(u32x4, pf[b][1]), lane);
      } else {
        // small blocks: a wavefront's rows of a block are contiguous (512 bytes at block 16, 1 KiB at block 32), so its
        // lanes store their chunks directly, block by block; nothing is stored for an absent block
        T *pz = reinterpret_cast<T *>(a.p_out) + z * a.pout_sz;
#pragma unroll
        for (int s = 0; s < 2; s++) {
          const int id = chunk_block_id<SUBS>(tid_[b], s, q);
          if (id >= 0)
            __builtin_nontemporal_store(__builtin_bit_cast(u32x4, pf[b][s]), reinterpret_cast<u32x4 *>(pz + (int64_t)id * ((64 / SUBS) * (64 / SUBS)) + chunk_in_block<SUBS>(wave, qrow, s, q)));
        }
      }
    }
}

// The backward chain.  x = do, y1 = v, y2 = k.  Unlike the forward chain it needs no second look at a row before its
// values can be finished: the sum over the row in the softmax gradient, sum_j p_j dp_j, equals sum_d do_d o_d (o = p . v,
// dp = do . v^T), which the wavefront computes up front from its 16 rows of do and of the forward result.  So block
// after block goes through dp = do . v_b^T -> ds_b = p_b * (dp - delta) * scale at once: the tile sequence is
// v_0, p_0, v_1, p_1, ... (the block of p is one more 8 KiB tile of the ring: no register-staged loads inside the
// loop, whose waits the compiler would place after all direct-to-LDS loads in flight), then k_0, k_1, ... for
// dq = ds . k.  Only the packed ds (the operand of the second product) stays in registers.
template <typename T, int D, int NB, int SUBS = 1>
__global__ void __launch_bounds__(256, 2) k_attn64_bwd(AttnArgs a) {
  typedef Mma16<T> M;
  typedef typename M::frag_t frag_t;
  typedef Pack<T, 8> P8;
  constexpr int NK = D / 32, ND = D / 16, LDK = D + 8;
  constexpr int TB = 64 * D * 2;        // bytes of a ring stage (a v or k tile; a block of p fills the first 8 KiB)
  constexpr int LW = TB / 1024 / 4;     // wavefront-level loads per wavefront and v / k tile
  constexpr int LWP = 2;                // ... and block of p
  constexpr int CPR = D / 8;
  constexpr int kStages = ring_stages<D>();
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  unsigned char *ring = smem;
  T *stage_out = reinterpret_cast<T *>(smem);
  static_assert(4 * 16 * (LDK + 72) * 2 <= kStages * TB, "the staged results fit into the ring");
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t n_wg = (int64_t)a.Z * a.H * a.R;
  const int64_t wg = xcd_remap(blockIdx.x, n_wg);
  const int br = a.R - 1 - (int)(wg % a.R);          // as in the forward kernel
  const int zh = (int)(wg / a.R);
  const int h = zh % a.H, z = zh / a.H;
  const table_ptr lut = as_table(a.lut);
  const int size = lut[2 * (h * a.R + br) + 0];
  const int offset = lut[2 * (h * a.R + br) + 1];
  const int qrow = lane & 15, q = lane >> 4;
  const int64_t row = (int64_t)br * 64 + wave * 16 + qrow;
  T *cs = stage_out + wave * 16 * LDK;
  T *stage_p = stage_out + 4 * 16 * LDK + wave * (16 * 72);
  T *po = reinterpret_cast<T *>(a.o) + z * a.o_sz + h * a.o_sh + ((int64_t)br * 64 + wave * 16) * a.o_ld;
  f32x4 o[ND];
#pragma unroll
  for (int j = 0; j < ND; j++) o[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  if (size <= 0) {   // an empty block-row: zero rows of dq
    store_rows<T, D>(cs, po, a.o_ld, o, lane);
    return;
  }
  const table_ptr core = lut + offset;
  constexpr int ES = entry_ints<SUBS>();
  const int wgroup = (16 * wave) / (64 / SUBS);   // as in the forward kernel
  int32_t bid[NB];
#pragma unroll
  for (int b = 0; b < NB; b++) bid[b] = core[ES * (b < size ? b : 0)];
  // small blocks: the ids of the wavefront's row of small blocks in each tile.  At head dimension 128 they are read from
  // the tile table where they are needed instead: kept for all tiles of the row, they and the arguments do not fit into
  // the scalar registers there.
  constexpr bool KEEP_IDS = D == 64;
  i32x4 tid_[KEEP_IDS ? NB : 1];
  if constexpr (KEEP_IDS) {
#pragma unroll
    for (int b = 0; b < NB; b++) tid_[b] = entry_ids<SUBS>(core + ES * (b < size ? b : 0), wgroup);
  }
  auto ids_of = [&](int b) {
    if constexpr (KEEP_IDS) return tid_[b];
    else return entry_ids<SUBS>(core + ES * (b < size ? b : 0), wgroup);
  };
  const T *px = reinterpret_cast<const T *>(a.x) + z * a.x_sz + h * a.x_sh + row * a.x_ld + 8 * q;
  const T *pof = reinterpret_cast<const T *>(a.o_in) + z * a.oin_sz + h * a.oin_sh + row * a.oin_ld + 8 * q;
  frag_t xq[NK], oq[NK];
#pragma unroll
  for (int s2 = 0; s2 < NK; s2++) {
    xq[s2] = *reinterpret_cast<const frag_t *>(px + 32 * s2);
    oq[s2] = *reinterpret_cast<const frag_t *>(pof + 32 * s2);
  }
  const T *py1 = reinterpret_cast<const T *>(a.y1) + z * a.y1_sz + h * a.y1_sh;
  const T *py2 = reinterpret_cast<const T *>(a.y2) + z * a.y2_sz + h * a.y2_sh;
  const T *pin = reinterpret_cast<const T *>(a.p_in) + z * a.pin_sz;
  // Tile n < 2 size: block n / 2, its v tile (n even) or its block of p (n odd); then the k tiles.  Stage n % kStages.
  int64_t off1[LW], off2[LW];
  int offp[LWP];
#pragma unroll
  for (int i = 0; i < LW; i++) {
    const int r = (wave * LW + i) * (64 / CPR) + lane / CPR, slot = lane % CPR;
    off1[i] = (int64_t)r * a.y1_ld + ((slot ^ swz_first<D>(r)) << 3);
    off2[i] = (int64_t)r * a.y2_ld + (((((slot >> 1) ^ swz_second<D>(r)) << 1) | (slot & 1)) << 3);
  }
  // a block of p: rows of 128 bytes; a lane reads 16 bytes of row 16 * wave + lane % 16, sixteen consecutive rows per
  // clock: chunk c of row r at slot c ^ ((r >> 1) & 7)
  // (small blocks: the chunk's offset inside its small block, and which small block column it lies in)
  int colp[LWP];
#pragma unroll
  for (int i = 0; i < LWP; i++) {
    const int r = (wave * LWP + i) * 8 + (lane >> 3), slot = lane & 7, chunk = slot ^ ((r >> 1) & 7);
    if constexpr (SUBS == 1) {
      offp[i] = r * 64 + (chunk << 3);
      colp[i] = 0;
    } else {
      constexpr int B = 64 / SUBS;
      offp[i] = (r % B) * B + (chunk * 8) % B;
      colp[i] = (chunk * 8) / B;
    }
  }
  const int total = 3 * size;
  auto loads_of = [&](int n) { return n >= total ? 0 : (n < 2 * size && (n & 1)) ? LWP : LW; };
  // block-column (v and k tiles) or block id (p) of tile n, from the table (a scalar load; clamped past the end)
  auto tile_key = [&](int n) {
    const int m = n < 2 * size ? (n >> 1) : n - 2 * size;
    const table_ptr e = core + ES * (m < size ? m : size - 1);
    return (n < 2 * size && (n & 1)) ? e[0] : entry_group<SUBS>(e, wgroup) - wgroup;
  };
  int next_key;
  auto issue = [&](int n, int key) {
    unsigned char *st = ring + (n % kStages) * TB;
    if (n < 2 * size && (n & 1)) {
      if constexpr (SUBS == 1) {
        const T *base = pin + (int64_t)key * 4096;
#pragma unroll
        for (int i = 0; i < LWP; i++)
          __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(base + offp[i]), BSP_LDS_PTR(st + (wave * LWP + i) * 1024), 16, 0, BSP_LOAD_ONCE);
      } else {
        // the tile of p gathered from its small blocks; chunks of absent blocks fetch the start of the tensor instead
        // (every load is issued: the waits count them) and are replaced by zeros when they are read
        i32x4 ids;
        if constexpr (KEEP_IDS) {
          const int m = n >> 1;
          ids = tid_[0];
#pragma unroll
          for (int b2 = 1; b2 < NB; b2++) ids = (m == b2) ? tid_[b2] : ids;
        } else {
          const int m = n >> 1;
          ids = entry_ids<SUBS>(core + ES * (m < size ? m : size - 1), wgroup);
        }
#pragma unroll
        for (int i = 0; i < LWP; i++) {
          int id = ids[0];
#pragma unroll
          for (int c = 1; c < SUBS; c++) id = (colp[i] == c) ? ids[c] : id;
          const T *src = id >= 0 ? pin + (int64_t)id * ((64 / SUBS) * (64 / SUBS)) + offp[i] : pin;
          __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(src), BSP_LDS_PTR(st + (wave * LWP + i) * 1024), 16, 0, BSP_LOAD_ONCE);
        }
      }
    } else if (n < 2 * size) {
      const T *base = py1 + (int64_t)key * (64 / SUBS) * a.y1_ld;
#pragma unroll
      for (int i = 0; i < LW; i++)
        __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(base + off1[i]), BSP_LDS_PTR(st + (wave * LW + i) * 1024), 16, 0, 0);
    } else {
      const T *base = py2 + (int64_t)key * (64 / SUBS) * a.y2_ld;
#pragma unroll
      for (int i = 0; i < LW; i++)
        __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(base + off2[i]), BSP_LDS_PTR(st + (wave * LW + i) * 1024), 16, 0, 0);
    }
  };
  // as in the forward kernel; the tiles issued after tile n differ in their number of loads
  auto step = [&](int n) {
    wait_vm(loads_of(n + 1) + (kStages > 3 ? loads_of(n + 2) : 0));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (n + kStages - 1 < total) issue(n + kStages - 1, next_key);
    next_key = tile_key(n + kStages);
  };
#pragma unroll
  for (int n = 0; n < kStages - 1; n++) issue(n, tile_key(n));   // (a row has at least one block: three tiles)
  next_key = tile_key(kStages - 1);
  // delta = sum_d do[row][d] * o[row][d]: sixteen products per lane, then over the four lanes of the row
  float delta = 0.f;
#pragma unroll
  for (int s2 = 0; s2 < NK; s2++)
#pragma unroll
    for (int i = 0; i < 8; i++) delta = fmaf(to_float(xq[s2][i]), to_float(oq[s2][i]), delta);
  delta += __shfl_xor(delta, 16);
  delta += __shfl_xor(delta, 32);
  if (a.delta != nullptr && q == 0) a.delta[((int64_t)z * a.H + h) * a.delta_sh + row] = delta;   // for the column kernel

  frag_t pf[NB][2];
  const int krow0 = 8 * (qrow >> 2) + (qrow & 3);
  const int prow = wave * 16 + qrow, pswz = (prow >> 1) & 7;
#pragma unroll
  for (int b = 0; b < NB; b++)
    if (b < size) {
      const i32x4 ids_b = ids_of(b);
      step(2 * b);
      const unsigned char *tile = ring + ((2 * b) % kStages) * TB;
      frag_t kf[4][NK];
#pragma unroll
      for (int jt = 0; jt < 4; jt++)
#pragma unroll
        for (int s2 = 0; s2 < NK; s2++)
          kf[jt][s2] = *reinterpret_cast<const frag_t *>(tile + first_offset<D>(32 * (jt >> 1) + 4 * (jt & 1) + krow0, 4 * s2 + q));
      f32x4 acc[4];
#pragma unroll
      for (int jt = 0; jt < 4; jt++) {
        acc[jt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s2 = 0; s2 < NK; s2++) acc[jt] = M::run(kf[jt][s2], xq[s2], acc[jt]);
      }
      step(2 * b + 1);
      const unsigned char *pt = ring + ((2 * b + 1) % kStages) * TB + prow * 128;
#pragma unroll
      for (int s = 0; s < 2; s++) {
        P8 y, d;
        y.raw = *reinterpret_cast<const u32x4 *>(pt + (((q + 4 * s) ^ pswz) << 4));
        bool here = true;
        if constexpr (SUBS > 1) here = chunk_block_id<SUBS>(ids_b, s, q) >= 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
          const float dp = to_float(from_float<T>(acc[2 * s + (i >> 2)][i & 3]));   // dp as the sdd operator would have stored it
          const float v = to_float(y.e[i]) * (dp - delta) * a.scale;                  // softmax.py:189
          d.e[i] = from_float<T>(here ? v : 0.f);
        }
        pf[b][s] = __builtin_bit_cast(frag_t, d.raw);
      }
    }

  // ---- second product: dq^T[d][row] += k_b^T[d][key] . ds_b[key][row]
  const int tr_row = q * 8 + (qrow >> 2), tr_col = (qrow & 3) * 4;
  const uint32_t ring_lds = (uint32_t)(uintptr_t)BSP_LDS_PTR(ring);
  uint32_t tr_off[ND];
#pragma unroll
  for (int j = 0; j < ND; j++) tr_off[j] = second_offset<D>(tr_row, 16 * j + tr_col);
#pragma unroll
  for (int b = 0; b < NB; b++)
    if (b < size) {
      step(2 * size + b);
      const uint32_t tile_lds = ring_lds + ((2 * size + b) % kStages) * TB;
#pragma unroll
      for (int s = 0; s < 2; s++)
#pragma unroll
        for (int j4 = 0; j4 < ND; j4 += 4) {
          frag_t vf[4];
          const uint32_t t0 = tile_lds + s * (32 * 2 * D);
          tr_frags4<T, 4 * 2 * D>(vf, t0 + tr_off[j4], t0 + tr_off[j4 + 1], t0 + tr_off[j4 + 2], t0 + tr_off[j4 + 3]);
#pragma unroll
          for (int j = 0; j < 4; j++) o[j4 + j] = M::run(vf[j], pf[b][s], o[j4 + j]);
        }
    }
  // ds leaves at the end, for the reason given in the forward kernel
  T *pout = reinterpret_cast<T *>(a.p_out) + z * a.pout_sz + wave * 1024;
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  store_rows<T, D>(cs, po, a.o_ld, o, lane);
  if (a.p_out == nullptr) return;   // ds is not asked for (the column kernel computes it again)
#pragma unroll
  for (int b = 0; b < NB; b++)
    if (b < size) {
      if constexpr (SUBS == 1) {
        store_block_rows<T>(stage_p, pout + (int64_t)bid[b] * 4096, __builtin_bit_cast(u32x4, pf[b][0]), __builtin_bit_cast(u32x4, pf[b][1]), lane);
      } else {
        T *pz = reinterpret_cast<T *>(a.p_out) + z * a.pout_sz;
        const i32x4 ids_b = ids_of(b);
#pragma unroll
        for (int s = 0; s < 2; s++) {
          const int id = chunk_block_id<SUBS>(ids_b, s, q);
          if (id >= 0)
            __builtin_nontemporal_store(__builtin_bit_cast(u32x4, pf[b][s]), reinterpret_cast<u32x4 *>(pz + (int64_t)id * ((64 / SUBS) * (64 / SUBS)) + chunk_in_block<SUBS>(wave, qrow, s, q)));
        }
      }
    }
}

template <int D, int NB> constexpr int lds_bytes(bool bwd) { return ring_stages<D>() * 64 * D * 2 + (bwd ? 0 : NB * 64 * 4); }

template <typename T, int D, int NB, int SUBS> void launch_nb(const AttnArgs &a, bool bwd, hipStream_t st) {
  const dim3 grid((unsigned)((int64_t)a.Z * a.H * a.R)), wg(256);
  constexpr int LDS = lds_bytes<D, NB>(false), LDS_BWD = lds_bytes<D, NB>(true);
  static_assert(LDS <= 64 * 1024, "within what a launch may ask for without raising the kernel's limit");
  if (bwd) hipLaunchKernelGGL((k_attn64_bwd<T, D, NB, SUBS>), grid, wg, LDS_BWD, st, a);
  else if (a.rpe || a.attn) hipLaunchKernelGGL((k_attn64_fwd<T, D, NB, true, SUBS>), grid, wg, LDS, st, a);
  else hipLaunchKernelGGL((k_attn64_fwd<T, D, NB, false, SUBS>), grid, wg, LDS, st, a);
}

template <typename T, int D, int SUBS> int launch_d(const AttnArgs &a, int maxlut, bool bwd, hipStream_t st) {
  if (maxlut <= 4) launch_nb<T, D, 4, SUBS>(a, bwd, st);
  else if (maxlut <= 8) launch_nb<T, D, 8, SUBS>(a, bwd, st);
  else return BSP_ERR_ROW_TOO_LONG;
  return BSP_OK;
}

template <typename T, int SUBS> int launch_s(const AttnArgs &a, int D, int maxlut, bool bwd, hipStream_t st) {
  if (D == 64) return launch_d<T, 64, SUBS>(a, maxlut, bwd, st);
  if (D == 128) return launch_d<T, 128, SUBS>(a, maxlut, bwd, st);
  return BSP_ERR_UNSUPPORTED;
}

template <typename T> int launch_t(const AttnArgs &a, int D, int block, int maxlut, bool bwd, hipStream_t st) {
  if (block == 64) return launch_s<T, 1>(a, D, maxlut, bwd, st);
  if (block == 32) return launch_s<T, 2>(a, D, maxlut, bwd, st);
  if (block == 16) return launch_s<T, 4>(a, D, maxlut, bwd, st);
  return BSP_ERR_UNSUPPORTED;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int run(int dtype, AttnArgs &a, int D, int block, int maxlut, bool bwd, void *stream) {
  if (!a.x || !a.y1 || !a.y2 || !a.o || !a.lut || (bwd && (!a.p_in || !a.o_in)) || a.Z <= 0 || a.H <= 0 || a.R <= 0 || maxlut < 0)
    return BSP_ERR_ARG;
  if ((block != 64 && block != 32 && block != 16) || (dtype != BSP_F16 && dtype != BSP_BF16) || (D != 64 && D != 128)) return BSP_ERR_UNSUPPORTED;
  if ((int64_t)maxlut * 64 >= 32768) return BSP_ERR_ROW_TOO_LONG;   // the softmax operator's bound on a row (softmax.py:225-227)
  const bool is_long = maxlut > BSP_ATTENTION_MAX_ROW_BLOCKS;         // longer rows: streamed
  // 16-byte vector accesses everywhere: every pointer and every stride a multiple of 8 elements
  const void *ptrs[] = {a.x, a.y1, a.y2, a.p_in, a.o_in, a.p_out, a.o, a.rpe, a.kpm, a.attn};
  for (const void *p : ptrs)
    if (!aligned16(p)) return BSP_ERR_ARG;
  const int64_t strides[] = {a.x_sz, a.x_sh, a.x_ld, a.y1_sz, a.y1_sh, a.y1_ld, a.y2_sz, a.y2_sh, a.y2_ld, a.o_sz, a.o_sh, a.o_ld,
                             a.pin_sz, a.pout_sz, a.rpe_sz, a.rpe_sh, a.rpe_sr, a.kpm_sz, a.attn_sr, a.oin_sz, a.oin_sh, a.oin_ld};
  for (int64_t s : strides)
    if (s % 8) return BSP_ERR_ARG;
  if (a.x_ld < D || a.y1_ld < D || a.y2_ld < D || a.o_ld < D || (bwd && a.oin_ld < D)) return BSP_ERR_ARG;
  if (a.delta != nullptr && ((reinterpret_cast<uintptr_t>(a.delta) & 3) || a.delta_sh < (int64_t)a.R * 64)) return BSP_ERR_ARG;
  if ((int64_t)a.Z * a.H * a.R >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  int rc;
  if (is_long) rc = attention_long(dtype, a, D, block, bwd, as_stream(stream));
  else if (dtype == BSP_F16) rc = launch_t<f16>(a, D, block, maxlut, bwd, as_stream(stream));
  else rc = launch_t<bf16>(a, D, block, maxlut, bwd, as_stream(stream));
  if (rc != BSP_OK) return rc;
  BSP_LAUNCH_CHECK();
  return BSP_OK;
}

}  // namespace
}  // namespace bsp

using namespace bsp;

extern "C" int bsp_attention_fwd(int dtype, const void *q, const void *k, const void *v, void *p, void *o, int Z, int H, int R,
                                 int D, int64_t q_stride_z, int64_t q_stride_h, int64_t ldq, int64_t k_stride_z, int64_t k_stride_h,
                                 int64_t ldk, int64_t v_stride_z, int64_t v_stride_h, int64_t ldv, int64_t o_stride_z,
                                 int64_t o_stride_h, int64_t ldo, int64_t p_stride_z, int block, float scale, const int32_t *d_lut,
                                 int maxlut, const void *rpe, int64_t rpe_stride_z, int64_t rpe_stride_h, int64_t rpe_stride_r,
                                 const void *kpm, int64_t kpm_stride_z, int kpm_mul, const void *attn, int64_t attn_stride_r,
                                 int attn_mul, void *stream) {
  AttnArgs a{};
  a.x = q; a.y1 = k; a.y2 = v; a.p_in = nullptr; a.p_out = p; a.o = o;
  a.x_sz = q_stride_z; a.x_sh = q_stride_h; a.x_ld = ldq;
  a.y1_sz = k_stride_z; a.y1_sh = k_stride_h; a.y1_ld = ldk;
  a.y2_sz = v_stride_z; a.y2_sh = v_stride_h; a.y2_ld = ldv;
  a.o_sz = o_stride_z; a.o_sh = o_stride_h; a.o_ld = ldo;
  a.pin_sz = 0; a.pout_sz = p_stride_z;
  a.scale = scale; a.lut = d_lut;
  a.rpe = rpe; a.rpe_sz = rpe_stride_z; a.rpe_sh = rpe_stride_h; a.rpe_sr = rpe_stride_r;
  a.kpm = kpm; a.kpm_sz = kpm_stride_z; a.kpm_mul = kpm_mul;
  a.attn = attn; a.attn_sr = attn_stride_r; a.attn_mul = attn_mul;
  a.Z = Z; a.H = H; a.R = R;
  return run(dtype, a, D, block, maxlut, false, stream);
}

extern "C" int bsp_attention_bwd(int dtype, const void *d_o, const void *v, const void *k, const void *p, const void *o, void *ds,
                                 void *dq, int Z, int H, int R, int D, int64_t do_stride_z, int64_t do_stride_h, int64_t lddo,
                                 int64_t v_stride_z, int64_t v_stride_h, int64_t ldv, int64_t k_stride_z, int64_t k_stride_h,
                                 int64_t ldk, int64_t o_stride_z, int64_t o_stride_h, int64_t ldo, int64_t dq_stride_z,
                                 int64_t dq_stride_h, int64_t lddq, int64_t p_stride_z, int64_t ds_stride_z, int block, float scale,
                                 const int32_t *d_lut, int maxlut, float *delta, int64_t delta_stride_h,
                                 void *stream) {
  AttnArgs a{};
  a.x = d_o; a.y1 = v; a.y2 = k; a.p_in = p; a.p_out = ds; a.o = dq;
  a.delta = delta; a.delta_sh = delta_stride_h;
  a.o_in = o; a.oin_sz = o_stride_z; a.oin_sh = o_stride_h; a.oin_ld = ldo;
  a.x_sz = do_stride_z; a.x_sh = do_stride_h; a.x_ld = lddo;
  a.y1_sz = v_stride_z; a.y1_sh = v_stride_h; a.y1_ld = ldv;
  a.y2_sz = k_stride_z; a.y2_sh = k_stride_h; a.y2_ld = ldk;
  a.o_sz = dq_stride_z; a.o_sh = dq_stride_h; a.o_ld = lddq;
  a.pin_sz = p_stride_z; a.pout_sz = ds_stride_z;
  a.scale = scale; a.lut = d_lut;
  a.Z = Z; a.H = H; a.R = R;
  return run(dtype, a, D, block, maxlut, true, stream);
}

extern "C" int bsp_attention_bwd_kv(int dtype, const void *d_o, const void *q, const void *v, const void *p, const float *delta,
                                    void *dk, void *dv, int Z, int H, int C, int D, int64_t do_stride_z, int64_t do_stride_h,
                                    int64_t lddo, int64_t q_stride_z, int64_t q_stride_h, int64_t ldq, int64_t v_stride_z,
                                    int64_t v_stride_h, int64_t ldv, int64_t dk_stride_z, int64_t dk_stride_h, int64_t lddk,
                                    int64_t dv_stride_z, int64_t dv_stride_h, int64_t lddv, int64_t p_stride_z,
                                    int64_t delta_stride_h, int block, float scale, const int32_t *d_col_lut, int n_items,
                                    float *partial, int n_slots, const int32_t *d_split_lut, int n_split, void *stream) {
  if (!d_o || !q || !v || !p || !delta || !dk || !dv || !d_col_lut || Z <= 0 || H <= 0 || C <= 0 || delta_stride_h < 0 || n_items < H * C)
    return BSP_ERR_ARG;
  if (n_slots < 0 || n_split < 0 || (n_slots > 0) != (n_split > 0) || (n_slots > 0 && (!partial || !d_split_lut)) || n_items > H * C + n_slots)
    return BSP_ERR_ARG;
  if (reinterpret_cast<uintptr_t>(partial) & 15) return BSP_ERR_ARG;
  if ((block != 64 && block != 32 && block != 16) || (dtype != BSP_F16 && dtype != BSP_BF16) || (D != 64 && D != 128)) return BSP_ERR_UNSUPPORTED;
  const void *ptrs[] = {d_o, q, v, p, dk, dv};
  for (const void *ptr : ptrs)
    if ((reinterpret_cast<uintptr_t>(ptr) & 15) != 0) return BSP_ERR_ARG;
  if (reinterpret_cast<uintptr_t>(delta) & 3) return BSP_ERR_ARG;
  const int64_t strides[] = {do_stride_z, do_stride_h, lddo, q_stride_z, q_stride_h, ldq, v_stride_z, v_stride_h, ldv,
                             dk_stride_z, dk_stride_h, lddk, dv_stride_z, dv_stride_h, lddv, p_stride_z};
  for (int64_t s : strides)
    if (s % 8) return BSP_ERR_ARG;
  if (lddo < D || ldq < D || ldv < D || lddk < D || lddv < D) return BSP_ERR_ARG;
  if ((int64_t)Z * n_items >= ((int64_t)1 << 31) || (int64_t)Z * n_split * 4 >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  AttnArgs a{};
  a.x = v; a.y1 = d_o; a.y2 = q; a.p_in = p; a.o = dk; a.o2 = dv;
  a.partial = partial; a.n_slots = n_slots; a.split_lut = d_split_lut; a.n_split = n_split;
  a.delta = const_cast<float *>(delta); a.delta_sh = delta_stride_h;
  a.x_sz = v_stride_z; a.x_sh = v_stride_h; a.x_ld = ldv;
  a.y1_sz = do_stride_z; a.y1_sh = do_stride_h; a.y1_ld = lddo;
  a.y2_sz = q_stride_z; a.y2_sh = q_stride_h; a.y2_ld = ldq;
  a.o_sz = dk_stride_z; a.o_sh = dk_stride_h; a.o_ld = lddk;
  a.o2_sz = dv_stride_z; a.o2_sh = dv_stride_h; a.o2_ld = lddv;
  a.pin_sz = p_stride_z;
  a.scale = scale; a.lut = d_col_lut;
  a.Z = Z; a.H = H; a.R = n_items;
  const int rc = attention_kv(dtype, a, D, block, as_stream(stream));
  if (rc != BSP_OK) return rc;
  BSP_LAUNCH_CHECK();
  return BSP_OK;
}
