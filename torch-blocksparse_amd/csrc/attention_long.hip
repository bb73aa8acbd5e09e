// The fused attention chain for rows of any length (more than 8 tiles of 64 x 64): the kernels of attention_core.hip
// keep a row's scores (forward) or its packed gradient (backward) in registers, which bounds the row; these walk the
// row block after block with a few registers of state and runtime loops.
//
//   backward: already streams in attention_core.hip (the row sum of the softmax gradient is known up front as
//             sum_d do_d o_d); here dq is accumulated as the blocks go by instead of after them, so nothing per block
//             is kept: tiles v_b, p_b, k_b per block.
//   forward : two sweeps.  The first computes the scores of every block and keeps only the running maximum and the
//             running sum of exponentials of each row (rescaled when the maximum grows); the second computes the
//             scores again (the k tiles come from L2 a second time, the matrix instructions are cheap), writes
//             p = exp(s - max) / sum and accumulates p . v.  Twice the exponentials of the kernel that holds the row.
// The key-padding mask of a block is one more 128-byte load of a k tile's stage; the values of a relative position
// embedding and of an attention mask are fetched into registers in the step of the block's k tile (in both sweeps).
#include "attention_common.h"

namespace bsp {
namespace {

template <typename T, int D, int SUBS>
__global__ void __launch_bounds__(256, 3) k_attn64_bwd_long(AttnArgs a) {
  typedef Mma16<T> M;
  typedef typename M::frag_t frag_t;
  typedef Pack<T, 8> P8;
  constexpr int NK = D / 32, ND = D / 16, LDK = D + 8;
  constexpr int TB = 64 * D * 2, LW = TB / 1024 / 4, LWP = 2, CPR = D / 8;
  constexpr int kStages = ring_stages<D>();
  // dynamic LDS: the tile ring (at the end it stages dq), then a staging slice of ds per wavefront
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  unsigned char *ring = smem;
  static_assert(4 * 16 * LDK * 2 <= kStages * TB, "the staged result fits into the ring");
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t n_wg = (int64_t)a.Z * a.H * a.R;
  const int64_t wg = xcd_remap(blockIdx.x, n_wg);
  const int br = a.R - 1 - (int)(wg % a.R);
  const int zh = (int)(wg / a.R);
  const int h = zh % a.H, z = zh / a.H;
  const table_ptr lut = as_table(a.lut);
  const int size = lut[2 * (h * a.R + br) + 0];
  const int offset = lut[2 * (h * a.R + br) + 1];
  const int qrow = lane & 15, q = lane >> 4;
  const int64_t row = (int64_t)br * 64 + wave * 16 + qrow;
  T *cs = reinterpret_cast<T *>(smem) + wave * 16 * LDK;
  T *stage_p = reinterpret_cast<T *>(smem + kStages * TB) + wave * (16 * 72);
  T *po = reinterpret_cast<T *>(a.o) + z * a.o_sz + h * a.o_sh + ((int64_t)br * 64 + wave * 16) * a.o_ld;
  f32x4 o[ND];
#pragma unroll
  for (int j = 0; j < ND; j++) o[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  if (size <= 0) {
    store_rows<T, D>(cs, po, a.o_ld, o, lane);
    return;
  }
  const table_ptr core = lut + offset;
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
  int64_t off1[LW], off2[LW];
  int offp[LWP], colp[LWP];
#pragma unroll
  for (int i = 0; i < LW; i++) {
    const int r = (wave * LW + i) * (64 / CPR) + lane / CPR, slot = lane % CPR;
    off1[i] = (int64_t)r * a.y1_ld + ((slot ^ swz_first<D>(r)) << 3);
    off2[i] = (int64_t)r * a.y2_ld + (((((slot >> 1) ^ swz_second<D>(r)) << 1) | (slot & 1)) << 3);
  }
#pragma unroll
  for (int i = 0; i < LWP; i++) {   // a tile of p, as in k_attn64_bwd
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
  const int rs = (16 * wave) / (64 / SUBS);
  constexpr int ES = entry_ints<SUBS>();
  // tile n: block n / 3; its v tile, its tile of p, its k tile
  const int total = 3 * size;
  auto loads_of = [&](int n) { return n >= total ? 0 : (n % 3 == 1) ? LWP : LW; };
  // block-column (v, k; small blocks: of the group of rows that this wavefront loads) or tile id (p), from the table;
  // clamped past the end
  auto tile_key = [&](int n) {
    const int m = n / 3;
    const table_ptr e = core + ES * (m < size ? m : size - 1);
    return n % 3 == 1 ? e[0] : entry_group<SUBS>(e, rs) - rs;
  };
  // (small blocks, with the key of a tile of p: the ids of the blocks it is gathered from)
  auto tile_vec = [&](int n) {
    const int m = n / 3;
    return entry_ids<SUBS>(core + ES * (m < size ? m : size - 1), rs);
  };
  int next_key;
  i32x4 next_vec;
  auto issue = [&](int n, int key, const i32x4 &ids) {
    unsigned char *st = ring + (n % kStages) * TB;
    const int kind = n % 3;
    if (kind == 1) {
      if constexpr (SUBS == 1) {
        const T *base = pin + (int64_t)key * 4096;
#pragma unroll
        for (int i = 0; i < LWP; i++)
          __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(base + offp[i]), BSP_LDS_PTR(st + (wave * LWP + i) * 1024), 16, 0, BSP_LOAD_ONCE);
      } else {
#pragma unroll
        for (int i = 0; i < LWP; i++) {
          int id = ids[0];
#pragma unroll
          for (int c = 1; c < SUBS; c++) id = (colp[i] == c) ? ids[c] : id;
          const T *src = id >= 0 ? pin + (int64_t)id * ((64 / SUBS) * (64 / SUBS)) + offp[i] : pin;
          __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(src), BSP_LDS_PTR(st + (wave * LWP + i) * 1024), 16, 0, BSP_LOAD_ONCE);
        }
      }
    } else if (kind == 0) {
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
  // The wait counts the loads of the tiles issued after tile n.  The stores of ds issued in between are not counted:
  // operations complete in order, so a count that leaves them out only waits for a little more than it must.
  auto step = [&](int n) {
    wait_vm(loads_of(n + 1) + (kStages > 3 ? loads_of(n + 2) : 0));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (n + kStages - 1 < total) issue(n + kStages - 1, next_key, next_vec);
    next_key = tile_key(n + kStages);
    next_vec = tile_vec(n + kStages);
  };
#pragma unroll
  for (int n = 0; n < kStages - 1; n++) issue(n, tile_key(n), tile_vec(n));   // (a row has at least one block: three tiles)
  next_key = tile_key(kStages - 1);
  next_vec = tile_vec(kStages - 1);
  float delta = 0.f;
#pragma unroll
  for (int s2 = 0; s2 < NK; s2++)
#pragma unroll
    for (int i = 0; i < 8; i++) delta = fmaf(to_float(xq[s2][i]), to_float(oq[s2][i]), delta);
  delta += __shfl_xor(delta, 16);
  delta += __shfl_xor(delta, 32);
  if (a.delta != nullptr && q == 0) a.delta[((int64_t)z * a.H + h) * a.delta_sh + row] = delta;   // for the column kernel

  const int krow0 = 8 * (qrow >> 2) + (qrow & 3);
  const int prow = wave * 16 + qrow, pswz = (prow >> 1) & 7;
  const int tr_row = q * 8 + (qrow >> 2), tr_col = (qrow & 3) * 4;
  const uint32_t ring_lds = (uint32_t)(uintptr_t)BSP_LDS_PTR(ring);
  uint32_t tr_off[ND];
#pragma unroll
  for (int j = 0; j < ND; j++) tr_off[j] = second_offset<D>(tr_row, 16 * j + tr_col);
  T *pz = reinterpret_cast<T *>(a.p_out) + z * a.pout_sz;
  for (int b = 0; b < size; b++) {
    const int tile_id = core[ES * b];
    const i32x4 ids = entry_ids<SUBS>(core + ES * b, rs);
    step(3 * b);
    const unsigned char *tile = ring + ((3 * b) % kStages) * TB;
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
    step(3 * b + 1);
    const unsigned char *pt = ring + ((3 * b + 1) % kStages) * TB + prow * 128;
    frag_t pf[2];
#pragma unroll
    for (int s = 0; s < 2; s++) {
      P8 y, d;
      y.raw = *reinterpret_cast<const u32x4 *>(pt + (((q + 4 * s) ^ pswz) << 4));
      bool here = true;
      if constexpr (SUBS > 1) here = chunk_block_id<SUBS>(ids, s, q) >= 0;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const float dp = to_float(from_float<T>(acc[2 * s + (i >> 2)][i & 3]));   // dp as the sdd operator would have stored it
        const float v = to_float(y.e[i]) * (dp - delta) * a.scale;                  // softmax.py:189
        d.e[i] = from_float<T>(here ? v : 0.f);
      }
      pf[s] = __builtin_bit_cast(frag_t, d.raw);
    }
    step(3 * b + 2);
    const uint32_t tile_lds = ring_lds + ((3 * b + 2) % kStages) * TB;
#pragma unroll
    for (int s = 0; s < 2; s++)
#pragma unroll
      for (int j4 = 0; j4 < ND; j4 += 4) {
        frag_t vf[4];
        const uint32_t t0 = tile_lds + s * (32 * 2 * D);
        tr_frags4<T, 4 * 2 * D>(vf, t0 + tr_off[j4], t0 + tr_off[j4 + 1], t0 + tr_off[j4 + 2], t0 + tr_off[j4 + 3]);
#pragma unroll
        for (int j = 0; j < 4; j++) o[j4 + j] = M::run(vf[j], pf[s], o[j4 + j]);
      }
    if (a.p_out == nullptr) continue;   // ds is not asked for
        if constexpr (SUBS == 1) {
      store_block_rows<T>(stage_p, pz + (int64_t)tile_id * 4096 + wave * 1024, __builtin_bit_cast(u32x4, pf[0]), __builtin_bit_cast(u32x4, pf[1]), lane);
    } else {
#pragma unroll
      for (int s = 0; s < 2; s++) {
        const int id = chunk_block_id<SUBS>(ids, s, q);
        if (id >= 0)
          __builtin_nontemporal_store(__builtin_bit_cast(u32x4, pf[s]), reinterpret_cast<u32x4 *>(pz + (int64_t)id * ((64 / SUBS) * (64 / SUBS)) + chunk_in_block<SUBS>(wave, qrow, s, q)));
      }
    }
  }
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  store_rows<T, D>(cs, po, a.o_ld, o, lane);
}

template <typename T, int D, int SUBS, bool EXTRA>
__global__ void __launch_bounds__(256, 3) k_attn64_fwd_long(AttnArgs a) {
  typedef Mma16<T> M;
  typedef typename M::frag_t frag_t;
  typedef Pack<T, 8> P8;
  constexpr int NK = D / 32, ND = D / 16, LDK = D + 8;
  constexpr int TB = 64 * D * 2, LW = TB / 1024 / 4, CPR = D / 8;
  constexpr int kStages = ring_stages<D>();
  // dynamic LDS: the tile ring (at the end it stages o), a staging slice of p per wavefront, the raw key-padding values
  // of the k tile of each stage (128 bytes each)
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  unsigned char *ring = smem;
  unsigned char *kraw = smem + kStages * TB + 4 * 16 * 72 * 2;
  static_assert(4 * 16 * LDK * 2 <= kStages * TB, "the staged result fits into the ring");
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t n_wg = (int64_t)a.Z * a.H * a.R;
  const int64_t wg = xcd_remap(blockIdx.x, n_wg);
  const int br = a.R - 1 - (int)(wg % a.R);
  const int zh = (int)(wg / a.R);
  const int h = zh % a.H, z = zh / a.H;
  const table_ptr lut = as_table(a.lut);
  const int size = lut[2 * (h * a.R + br) + 0];
  const int offset = lut[2 * (h * a.R + br) + 1];
  const int qrow = lane & 15, q = lane >> 4;
  const int64_t row = (int64_t)br * 64 + wave * 16 + qrow;
  T *cs = reinterpret_cast<T *>(smem) + wave * 16 * LDK;
  T *stage_p = reinterpret_cast<T *>(smem + kStages * TB) + wave * (16 * 72);
  T *po = reinterpret_cast<T *>(a.o) + z * a.o_sz + h * a.o_sh + ((int64_t)br * 64 + wave * 16) * a.o_ld;
  f32x4 o[ND];
#pragma unroll
  for (int j = 0; j < ND; j++) o[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  if (size <= 0) {
    store_rows<T, D>(cs, po, a.o_ld, o, lane);
    return;
  }
  const table_ptr core = lut + offset;
  const T *px = reinterpret_cast<const T *>(a.x) + z * a.x_sz + h * a.x_sh + row * a.x_ld + 8 * q;
  frag_t xq[NK];
#pragma unroll
  for (int s2 = 0; s2 < NK; s2++) xq[s2] = *reinterpret_cast<const frag_t *>(px + 32 * s2);
  const T *py1 = reinterpret_cast<const T *>(a.y1) + z * a.y1_sz + h * a.y1_sh;
  const T *py2 = reinterpret_cast<const T *>(a.y2) + z * a.y2_sz + h * a.y2_sh;
  const bool has_kpm = a.kpm != nullptr;
  const T *pkpm = reinterpret_cast<const T *>(a.kpm) + z * a.kpm_sz;
  int64_t off1[LW], off2[LW];
#pragma unroll
  for (int i = 0; i < LW; i++) {
    const int r = (wave * LW + i) * (64 / CPR) + lane / CPR, slot = lane % CPR;
    off1[i] = (int64_t)r * a.y1_ld + ((slot ^ swz_first<D>(r)) << 3);
    off2[i] = (int64_t)r * a.y2_ld + (((((slot >> 1) ^ swz_second<D>(r)) << 1) | (slot & 1)) << 3);
  }
  const int rs = (16 * wave) / (64 / SUBS);
  constexpr int ES = entry_ints<SUBS>();
  // tile n < size: the k tile of block n (first sweep); then per block its k tile again and its v tile
  const int total = 3 * size;
  auto is_v = [&](int n) { return n >= size && ((n - size) & 1); };
  auto block_of = [&](int n) { return n < size ? n : (n - size) >> 1; };
  auto loads_of = [&](int n) { return n >= total ? 0 : is_v(n) ? LW : LW + (has_kpm ? 1 : 0); };
  // (small blocks: the block-column of the group of rows that this wavefront loads)
  auto tile_col = [&](int n) {
    const int m = block_of(n < total ? n : total - 1);
    return entry_group<SUBS>(core + ES * m, rs) - rs;
  };
  int next_col;
  auto issue = [&](int n, int col) {
    unsigned char *st = ring + (n % kStages) * TB;
    if (is_v(n)) {
      const T *base = py2 + (int64_t)col * (64 / SUBS) * a.y2_ld;
#pragma unroll
      for (int i = 0; i < LW; i++)
        __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(base + off2[i]), BSP_LDS_PTR(st + (wave * LW + i) * 1024), 16, 0, 0);
    } else {
      const T *base = py1 + (int64_t)col * (64 / SUBS) * a.y1_ld;
#pragma unroll
      for (int i = 0; i < LW; i++)
        __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(base + off1[i]), BSP_LDS_PTR(st + (wave * LW + i) * 1024), 16, 0, 0);
      // the 64 key-padding values of the tile's columns: one more load of every wavefront (eight lanes of it; all four
      // write the same 128 bytes, so that all count the same number of loads)
      if (has_kpm) {
        const i32x4 groups = entry_groups<SUBS>(core + ES * block_of(n));
        if (lane < 8)
          __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(pkpm + element_position<SUBS>(groups, lane * 8)), BSP_LDS_PTR(kraw + (n % kStages) * 128), 16, 0, 0);
      }
    }
  };
  // With per-element masks (EXTRA) the step of a k tile fetches the block's mask values into registers between the
  // barrier and the next tile load: four loads per lane (two masks, two chunks of eight columns; a mask that is not
  // given is replaced by the other, so that the count is fixed).  They share the counter of the tile loads and complete
  // in order with them: the wait for tile n also counts the mask loads of the k-tile steps n - kStages + 2 .. n - 1,
  // and using the values makes the tiles issued before them land one or two steps early.
  constexpr int MASK_LOADS = 4;
  auto is_k_step = [&](int m) { return m >= 0 && m < total && !is_v(m); };
  auto arrive = [&](int n) {   // stores of p issued in between are not counted: see k_attn64_bwd_long
    if constexpr (EXTRA) {
      wait_vm_exact(loads_of(n + 1) + (kStages > 3 ? loads_of(n + 2) : 0) +
                    MASK_LOADS * ((is_k_step(n - 1) ? 1 : 0) + (kStages > 3 && is_k_step(n - 2) ? 1 : 0)));
    } else {
      wait_vm(loads_of(n + 1) + (kStages > 3 ? loads_of(n + 2) : 0));
    }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  auto advance = [&](int n) {
    if (n + kStages - 1 < total) issue(n + kStages - 1, next_col);
    next_col = tile_col(n + kStages);
  };
  auto step = [&](int n) {
    arrive(n);
    advance(n);
  };
  // the mask values of the lane's two chunks of the block in block-column col (address: softmax.py:50-55, 67-70)
  auto load_masks = [&](const i32x4 &groups, P8 (&pr)[2], P8 (&pa)[2]) {
#pragma unroll
    for (int s = 0; s < 2; s++) {
      const int64_t gcol = chunk_position<SUBS>(groups, s, q);
      const T *attn = reinterpret_cast<const T *>(a.attn) + row * a.attn_sr + gcol;
      const T *rpe = reinterpret_cast<const T *>(a.rpe) + z * a.rpe_sz + h * a.rpe_sh + row * a.rpe_sr + gcol;
      pr[s].load(a.rpe ? rpe : attn);
      pa[s].load(a.attn ? attn : rpe);
    }
  };
#pragma unroll
  for (int n = 0; n < kStages - 1; n++) issue(n, tile_col(n));   // (three tiles at least)
  next_col = tile_col(kStages - 1);

  const int krow0 = 8 * (qrow >> 2) + (qrow & 3);
  const float unit = logit_unit<T>(), sc = a.scale * unit;
  // the logits of the lane's 16 values of the tile in stage n % kStages: fx[2s + t][e], columns 32s + 8q + 4t + e
  auto logits = [&](int n, const i32x4 &ids, f32x4 (&fx)[4], const P8 (&pr)[2], const P8 (&pa)[2]) {
    const unsigned char *tile = ring + (n % kStages) * TB;
    frag_t kf[4][NK];
#pragma unroll
    for (int jt = 0; jt < 4; jt++)
#pragma unroll
      for (int s2 = 0; s2 < NK; s2++)
        kf[jt][s2] = *reinterpret_cast<const frag_t *>(tile + first_offset<D>(32 * (jt >> 1) + 4 * (jt & 1) + krow0, 4 * s2 + q));
#pragma unroll
    for (int jt = 0; jt < 4; jt++) {
      fx[jt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s2 = 0; s2 < NK; s2++) fx[jt] = M::run(kf[jt][s2], xq[s2], fx[jt]);
    }
#pragma unroll
    for (int s = 0; s < 2; s++) {
      float add[8];
      if (has_kpm) {                                     // softmax.py:104-106, 122-124
        P8 kp;
        kp.raw = *reinterpret_cast<const u32x4 *>(kraw + (n % kStages) * 128 + (32 * s + 8 * q) * 2);
#pragma unroll
        for (int i = 0; i < 8; i++) {
          const float m = to_float(kp.e[i]);
          add[i] = a.kpm_mul ? (m == 0.f ? -INFINITY : 0.f) : m * unit;
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; i++) add[i] = 0.f;
      }
      if constexpr (SUBS > 1) {
        if (chunk_block_id<SUBS>(ids, s, q) < 0) {
#pragma unroll
          for (int i = 0; i < 8; i++) add[i] = -INFINITY;
        }
      }
#pragma unroll
      for (int i = 0; i < 8; i++) {                      // :112-116
        float f = fmaf(to_float(from_float<T>(fx[2 * s + (i >> 2)][i & 3])), sc, add[i]);
        if constexpr (EXTRA) {
          if (a.rpe) f = fmaf(to_float(pr[s].e[i]), unit, f);                                       // :118-120
          if (a.attn) {                                                                            // :126-128, 'mul' mode :108-110
            const float m = to_float(pa[s].e[i]);
            f += a.attn_mul ? (m == 0.f ? -INFINITY : 0.f) : m * unit;
          }
        }
        fx[2 * s + (i >> 2)][i & 3] = f;
      }
    }
  };

  // ---- first sweep: running maximum and running sum of exponentials of the lane's part of its row
  float m_run = -INFINITY, l_run = 0.f;
  int any_block = SUBS == 1;
  for (int b = 0; b < size; b++) {
    const i32x4 ids = entry_ids<SUBS>(core + ES * b, rs);
    if constexpr (SUBS > 1) any_block |= int(chunk_block_id<SUBS>(ids, 0, q) >= 0 || chunk_block_id<SUBS>(ids, 1, q) >= 0);
    P8 pr[2], pa[2];
    if constexpr (EXTRA) {
      arrive(b);
      load_masks(entry_groups<SUBS>(core + ES * b), pr, pa);
      advance(b);
    } else {
      step(b);
    }
    f32x4 fx[4];
    logits(b, ids, fx, pr, pa);
    float mb = m_run;
#pragma unroll
    for (int jt = 0; jt < 4; jt++)
#pragma unroll
      for (int e = 0; e < 4; e++) mb = fmaxf(mb, fx[jt][e]);
    const float ms = mb == -INFINITY ? 0.f : mb;         // (nothing but -inf so far: exp(-inf - 0) = 0, not exp(-inf + inf))
    float l = l_run * exp_sub<T>(m_run, ms);
#pragma unroll
    for (int jt = 0; jt < 4; jt++)
#pragma unroll
      for (int e = 0; e < 4; e++) l += exp_sub<T>(fx[jt][e], ms);
    l_run = l;
    m_run = mb;
  }
  // the four lanes of a row: one maximum, the sums brought to it
  float mx = fmaxf(m_run, __shfl_xor(m_run, 16));
  mx = fmaxf(mx, __shfl_xor(mx, 32));
  const float mxs = mx == -INFINITY ? 0.f : mx;
  float sum = l_run * exp_sub<T>(m_run, mxs);
  sum += __shfl_xor(sum, 16);
  sum += __shfl_xor(sum, 32);
  const float inv = 1.f / sum;                           // a row that is masked everywhere: 0 * inf = NaN, as the softmax operator gives
  if constexpr (SUBS > 1) {
    any_block |= __shfl_xor(any_block, 16);
    any_block |= __shfl_xor(any_block, 32);
  }

  // ---- second sweep: the scores again, p, p . v
  const int tr_row = q * 8 + (qrow >> 2), tr_col = (qrow & 3) * 4;
  const uint32_t ring_lds = (uint32_t)(uintptr_t)BSP_LDS_PTR(ring);
  uint32_t tr_off[ND];
#pragma unroll
  for (int j = 0; j < ND; j++) tr_off[j] = second_offset<D>(tr_row, 16 * j + tr_col);
  T *pz = reinterpret_cast<T *>(a.p_out) + z * a.pout_sz;
  for (int b = 0; b < size; b++) {
    const int tile_id = core[ES * b];
    const i32x4 ids = entry_ids<SUBS>(core + ES * b, rs);
    const int n = size + 2 * b;
    P8 pr[2], pa[2];
    if constexpr (EXTRA) {
      arrive(n);
      load_masks(entry_groups<SUBS>(core + ES * b), pr, pa);
      advance(n);
    } else {
      step(n);
    }
    f32x4 fx[4];
    logits(n, ids, fx, pr, pa);
    frag_t pf[2];
#pragma unroll
    for (int s = 0; s < 2; s++) {
      P8 y;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const float v = exp_sub<T>(fx[2 * s + (i >> 2)][i & 3], mxs) * inv;          // softmax.py:131-137
        y.e[i] = from_float<T>(SUBS > 1 && !any_block ? 0.f : v);
      }
      pf[s] = __builtin_bit_cast(frag_t, y.raw);
    }
    step(n + 1);
    const uint32_t tile_lds = ring_lds + ((n + 1) % kStages) * TB;
#pragma unroll
    for (int s = 0; s < 2; s++)
#pragma unroll
      for (int j4 = 0; j4 < ND; j4 += 4) {
        frag_t vf[4];
        const uint32_t t0 = tile_lds + s * (32 * 2 * D);
        tr_frags4<T, 4 * 2 * D>(vf, t0 + tr_off[j4], t0 + tr_off[j4 + 1], t0 + tr_off[j4 + 2], t0 + tr_off[j4 + 3]);
#pragma unroll
        for (int j = 0; j < 4; j++) o[j4 + j] = M::run(vf[j], pf[s], o[j4 + j]);
      }
    if (a.p_out == nullptr) continue;   // p is not asked for
    if constexpr (SUBS == 1) {
      store_block_rows<T>(stage_p, pz + (int64_t)tile_id * 4096 + wave * 1024, __builtin_bit_cast(u32x4, pf[0]), __builtin_bit_cast(u32x4, pf[1]), lane);
    } else {
#pragma unroll
      for (int s = 0; s < 2; s++) {
        const int id = chunk_block_id<SUBS>(ids, s, q);
        if (id >= 0)
          __builtin_nontemporal_store(__builtin_bit_cast(u32x4, pf[s]), reinterpret_cast<u32x4 *>(pz + (int64_t)id * ((64 / SUBS) * (64 / SUBS)) + chunk_in_block<SUBS>(wave, qrow, s, q)));
      }
    }
  }
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  store_rows<T, D>(cs, po, a.o_ld, o, lane);
}

template <typename T, int D, int SUBS> void launch_long(const AttnArgs &a, bool bwd, hipStream_t st) {
  const dim3 grid((unsigned)((int64_t)a.Z * a.H * a.R)), wg(256);
  constexpr int LDS = ring_stages<D>() * 64 * D * 2 + 4 * 16 * 72 * 2 + ring_stages<D>() * 128;
  static_assert(LDS <= 64 * 1024, "within what a launch may ask for without raising the kernel's limit");
  if (bwd) hipLaunchKernelGGL((k_attn64_bwd_long<T, D, SUBS>), grid, wg, LDS, st, a);
  else if (a.rpe || a.attn) hipLaunchKernelGGL((k_attn64_fwd_long<T, D, SUBS, true>), grid, wg, LDS, st, a);
  else hipLaunchKernelGGL((k_attn64_fwd_long<T, D, SUBS, false>), grid, wg, LDS, st, a);
}

template <typename T, int SUBS> int launch_long_d(const AttnArgs &a, int D, bool bwd, hipStream_t st) {
  if (D == 64) launch_long<T, 64, SUBS>(a, bwd, st);
  else if (D == 128) launch_long<T, 128, SUBS>(a, bwd, st);
  else return BSP_ERR_UNSUPPORTED;
  return BSP_OK;
}

template <typename T> int launch_long_t(const AttnArgs &a, int D, int block, bool bwd, hipStream_t st) {
  if (block == 64) return launch_long_d<T, 1>(a, D, bwd, st);
  if (block == 32) return launch_long_d<T, 2>(a, D, bwd, st);
  if (block == 16) return launch_long_d<T, 4>(a, D, bwd, st);
  return BSP_ERR_UNSUPPORTED;
}

}  // namespace

int attention_long(int dtype, const AttnArgs &a, int D, int block, bool bwd, hipStream_t st) {
  if (dtype == BSP_F16) return launch_long_t<f16>(a, D, block, bwd, st);
  if (dtype == BSP_BF16) return launch_long_t<bf16>(a, D, block, bwd, st);
  return BSP_ERR_UNSUPPORTED;
}

}  // namespace bsp
