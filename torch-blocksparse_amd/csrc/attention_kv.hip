// The key / value half of the fused attention backward pass: dk = ds^T . q and dv = p^T . do in one launch, one
// workgroup per column of 64 x 64 tiles of one (batch, head), with ds recomputed from p instead of read:
//     ds[row][key] = p[row][key] * (round(do[row] . v[key]) - delta[row]) * scale,
// delta[row] = sum_d do[row][d] o[row][d] written by the row kernel (which computes dq from the same formula and then
// has no reason to store ds).  The sparse gradient is neither written nor read: the backward pass moves p twice
// instead of p twice and ds twice.
//
// Columns differ in length far more than rows do (a global column of a causal layout holds a block of every later
// row): the table's work items are columns or, for long columns, parts of them, whose sums go to fp32 slots that a
// second small kernel adds in order (no atomics: the same bits every time).
//
// Blocks of 16 / 32 (SUBS = 4 / 2): a column of tiles is SUBS block-columns that need not be neighbours (the work item
// names them), and a tile's 64 rows are SUBS groups of consecutive rows gathered from anywhere (the tile's table entry
// names the block-row of each group and the ids of its blocks); the tile of p is gathered from the small blocks.
//
// A wavefront owns 16 of the column's 64 keys for all rows.  Per block of the column, three tiles through the ring:
//   p    [row][key]  read transposed (a lane: its key, 8 consecutive rows)              -> operand of dv, factor of ds
//   do   [row][d]    read along d for dp = do . v^T (the lane's v fragment stays in registers) and transposed for
//                    dv^T[d][key] += do^T[d][row] . p[row][key]; with it the 64 delta of the rows
//   q    [row][d]    read transposed for dk^T[d][key] += q^T[d][row] . ds[row][key]
// Rows are permuted inside the first product as in the other kernels, so that the lane that holds dp of rows
// 8g .. 8g + 7 of a 32-row half is the lane that holds p of these rows.
#include "attention_common.h"

namespace bsp {
namespace {

template <typename T, int D, int SUBS>
__global__ void __launch_bounds__(256, 2) k_attn64_bwd_kv(AttnArgs a) {
  typedef Mma16<T> M;
  typedef typename M::frag_t frag_t;
  typedef Pack<T, 8> P8;
  constexpr int NK = D / 32, ND = D / 16, LDK = D + 8;
  constexpr int TB = 64 * D * 2, LW = TB / 1024 / 4, LWP = 2, CPR = D / 8;
  constexpr int kStages = ring_stages<D>();
  // dynamic LDS: the tile ring (at the end it stages dk, then dv), the rows' delta of each stage (256 bytes)
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  unsigned char *ring = smem;
  unsigned char *dring = smem + kStages * TB;
  static_assert(4 * 16 * LDK * 2 <= kStages * TB, "the staged result fits into the ring");
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t n_wg = (int64_t)a.Z * a.R;             // R: work items (columns of tiles, the long ones in parts)
  const int64_t wg = xcd_remap(blockIdx.x, n_wg);
  const int item = (int)(wg % a.R), z = (int)(wg / a.R);
  const table_ptr lut = as_table(a.lut);                // per item twelve ints (entries, offset, head, column, slot of partial results or -1, ., ., ., its S block-columns)
  const int size = lut[12 * item + 0];
  const int offset = lut[12 * item + 1];
  const int h = lut[12 * item + 2], slot = lut[12 * item + 4];
  const int qrow = lane & 15, q = lane >> 4;
  // the column's 64 keys: S groups of 64 / S consecutive ones (S = SUBS block-columns, anywhere in the matrix); the first
  // key of the wavefront's 16
  const int64_t key0 = (int64_t)lut[12 * item + 8 + (16 * wave) / (64 / SUBS)] * (64 / SUBS) + (16 * wave) % (64 / SUBS);
  const int64_t key = key0 + qrow;
  T *cs = reinterpret_cast<T *>(smem) + wave * 16 * LDK;
  T *pdk = reinterpret_cast<T *>(a.o) + z * a.o_sz + h * a.o_sh + key0 * a.o_ld;
  T *pdv = reinterpret_cast<T *>(a.o2) + z * a.o2_sz + h * a.o2_sh + key0 * a.o2_ld;
  f32x4 dk[ND], dv[ND];
#pragma unroll
  for (int j = 0; j < ND; j++) dk[j] = dv[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  if (size <= 0) {   // a column without blocks: zero rows of dk and dv
    store_rows<T, D>(cs, pdk, a.o_ld, dk, lane);
    store_rows<T, D>(cs, pdv, a.o2_ld, dv, lane);
    return;
  }
  const table_ptr core = lut + offset;
  const T *px = reinterpret_cast<const T *>(a.x) + z * a.x_sz + h * a.x_sh + key * a.x_ld + 8 * q;
  frag_t vq[NK];
#pragma unroll
  for (int s2 = 0; s2 < NK; s2++) vq[s2] = *reinterpret_cast<const frag_t *>(px + 32 * s2);
  const T *py1 = reinterpret_cast<const T *>(a.y1) + z * a.y1_sz + h * a.y1_sh;   // do
  const T *py2 = reinterpret_cast<const T *>(a.y2) + z * a.y2_sz + h * a.y2_sh;   // q
  const T *pin = reinterpret_cast<const T *>(a.p_in) + z * a.pin_sz;
  const float *pdelta = a.delta + ((int64_t)z * a.H + h) * a.delta_sh;
  constexpr int ES = entry_ints<SUBS>();
  int64_t off1[LW], off2[LW];
  int offp[LWP], colp[LWP];
#pragma unroll
  for (int i = 0; i < LW; i++) {
    const int r = (wave * LW + i) * (64 / CPR) + lane / CPR, slot = lane % CPR;
    // the chunk of the row that belongs at this slot: the two swizzles are their own inverses
    off1[i] = (int64_t)r * a.y1_ld + (dual_slot<D>(r, slot) << 3);
    off2[i] = (int64_t)r * a.y2_ld + (((((slot >> 1) ^ swz_second<D>(r)) << 1) | (slot & 1)) << 3);
  }
#pragma unroll
  for (int i = 0; i < LWP; i++) {   // a tile of p: 64 rows of 128 bytes, laid out for the transposing reads
    const int r = (wave * LWP + i) * 8 + (lane >> 3), slot = lane & 7;
    const int chunk = (((slot >> 1) ^ swz_second<64>(r)) << 1) | (slot & 1);
    if constexpr (SUBS == 1) {
      offp[i] = r * 64 + (chunk << 3);
      colp[i] = 0;
    } else {
      constexpr int B = 64 / SUBS;
      offp[i] = (r % B) * B + (chunk * 8) % B;
      colp[i] = (chunk * 8) / B;
    }
  }
  const int rs = (16 * wave) / (64 / SUBS);       // the wavefront's row of small blocks when it loads, its column when it computes
  // tile n: block n / 3; its tile of p, its do tile (with delta), its q tile
  const int total = 3 * size;
  auto loads_of = [&](int n) { return n >= total ? 0 : (n % 3 == 0) ? LWP : (n % 3 == 1) ? LW + 1 : LW; };
  // tile id (p) or block-row (do, q; small blocks: of the group of rows that this wavefront loads), from the table;
  // clamped past the end
  auto tile_key = [&](int n) {
    const int m = n / 3;
    const table_ptr e = core + ES * (m < size ? m : size - 1);
    return n % 3 == 0 ? e[0] : entry_group<SUBS>(e, rs) - rs;
  };
  // small blocks, with the tile's key: the ids of the blocks in the wavefront's group of rows (tile of p: what it
  // gathers) or the block-rows of all groups (do tile: where the rows' delta lie)
  auto tile_vec = [&](int n) {
    i32x4 t = i32x4{0, 0, 0, 0};
    if constexpr (SUBS > 1) {
      const int m = n / 3;
      const table_ptr e = core + ES * (m < size ? m : size - 1) + (n % 3 == 0 ? 8 + rs * SUBS : 4);
#pragma unroll
      for (int c = 0; c < SUBS; c++) t[c] = e[c];
    }
    return t;
  };
  int next_key;
  i32x4 next_vec;
  auto issue = [&](int n, int key_, const i32x4 &vec) {
    unsigned char *st = ring + (n % kStages) * TB;
    const int kind = n % 3;
    if (kind == 0) {
      if constexpr (SUBS == 1) {
        const T *base = pin + (int64_t)key_ * 4096;
#pragma unroll
        for (int i = 0; i < LWP; i++)
          __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(base + offp[i]), BSP_LDS_PTR(st + (wave * LWP + i) * 1024), 16, 0, BSP_LOAD_ONCE);
      } else {
        // gathered from the small blocks; chunks of absent blocks fetch the start of the tensor (every load is issued:
        // the waits count them) and are replaced by zeros when they are read
#pragma unroll
        for (int i = 0; i < LWP; i++) {
          int id = vec[0];
#pragma unroll
          for (int c = 1; c < SUBS; c++) id = (colp[i] == c) ? vec[c] : id;
          const T *src = id >= 0 ? pin + (int64_t)id * ((64 / SUBS) * (64 / SUBS)) + offp[i] : pin;
          __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(src), BSP_LDS_PTR(st + (wave * LWP + i) * 1024), 16, 0, BSP_LOAD_ONCE);
        }
      }
    } else if (kind == 1) {
      const T *base = py1 + (int64_t)key_ * (64 / SUBS) * a.y1_ld;
#pragma unroll
      for (int i = 0; i < LW; i++)
        __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(base + off1[i]), BSP_LDS_PTR(st + (wave * LW + i) * 1024), 16, 0, 0);
      // the 64 delta of the tile's rows: every wavefront loads the same 256 bytes, so that all count the same loads
      const int64_t drow = SUBS == 1 ? (int64_t)key_ * 64 + lane : element_position<SUBS>(vec, lane);
      __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(pdelta + drow), BSP_LDS_PTR(dring + (n % kStages) * 256), 4, 0, 0);
    } else {
      const T *base = py2 + (int64_t)key_ * (64 / SUBS) * a.y2_ld;
#pragma unroll
      for (int i = 0; i < LW; i++)
        __builtin_amdgcn_global_load_lds(BSP_GLOBAL_PTR(base + off2[i]), BSP_LDS_PTR(st + (wave * LW + i) * 1024), 16, 0, 0);
    }
  };
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
  for (int n = 0; n < kStages - 1; n++) issue(n, tile_key(n), tile_vec(n));   // (a column has at least one block: three tiles)
  next_key = tile_key(kStages - 1);
  next_vec = tile_vec(kStages - 1);
  // small blocks: the ids of the wavefront's column of small blocks in a tile, by group of rows; fetched a block ahead
  auto column_ids = [&](int b) {
    i32x4 t = i32x4{0, 0, 0, 0};
    if constexpr (SUBS > 1) {
      const table_ptr e = core + ES * (b < size ? b : size - 1) + 8 + rs;
#pragma unroll
      for (int r2 = 0; r2 < SUBS; r2++) t[r2] = e[r2 * SUBS];
    }
    return t;
  };
  i32x4 present_next = column_ids(0);

  const int krow0 = 8 * (qrow >> 2) + (qrow & 3);
  const int tr_row = q * 8 + (qrow >> 2), tr_col = (qrow & 3) * 4;
  const uint32_t ring_lds = (uint32_t)(uintptr_t)BSP_LDS_PTR(ring);
  uint32_t tr_do[ND], tr_q[ND];
#pragma unroll
  for (int j = 0; j < ND; j++) {
    tr_do[j] = dual_offset<D>(tr_row, 16 * j + tr_col);
    tr_q[j] = second_offset<D>(tr_row, 16 * j + tr_col);
  }
  const uint32_t tr_p = second_offset<64>(tr_row, 16 * wave + tr_col);
  for (int b = 0; b < size; b++) {
    const i32x4 present = present_next;
    present_next = column_ids(b + 1);
    step(3 * b);
    frag_t pf[2];
    {
      const uint32_t t0 = ring_lds + ((3 * b) % kStages) * TB + tr_p;
      tr_frags2<T, 4 * 128>(pf, t0, t0 + 32 * 128);
    }
    step(3 * b + 1);
    const unsigned char *tile = ring + ((3 * b + 1) % kStages) * TB;
    f32x4 acc[4];
    {
      frag_t kf[4][NK];
#pragma unroll
      for (int jt = 0; jt < 4; jt++)
#pragma unroll
        for (int s2 = 0; s2 < NK; s2++) {
          const int r = 32 * (jt >> 1) + 4 * (jt & 1) + krow0;
          kf[jt][s2] = *reinterpret_cast<const frag_t *>(tile + r * (2 * D) + (dual_slot<D>(r, 4 * s2 + q) << 4));
        }
#pragma unroll
      for (int jt = 0; jt < 4; jt++) {
        acc[jt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s2 = 0; s2 < NK; s2++) acc[jt] = M::run(kf[jt][s2], vq[s2], acc[jt]);
      }
    }
    const float *dl = reinterpret_cast<const float *>(dring + ((3 * b + 1) % kStages) * 256) + 8 * q;
    frag_t df[2];
#pragma unroll
    for (int s = 0; s < 2; s++) {
      const f32x4 d0 = *reinterpret_cast<const f32x4 *>(dl + 32 * s), d1 = *reinterpret_cast<const f32x4 *>(dl + 32 * s + 4);
      P8 y, d;
      y.raw = __builtin_bit_cast(u32x4, pf[s]);
      bool here = true;
      if constexpr (SUBS == 2) here = present[s] >= 0;
      if constexpr (SUBS == 4) here = ((q >> 1) ? (s ? present[3] : present[1]) : (s ? present[2] : present[0])) >= 0;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const float dp = to_float(from_float<T>(acc[2 * s + (i >> 2)][i & 3]));   // dp as the sdd operator would have stored it
        const float dlt = i < 4 ? d0[i & 3] : d1[i & 3];
        const float v = to_float(y.e[i]) * (dp - dlt) * a.scale;                   // softmax.py:189
        d.e[i] = from_float<T>(here ? v : 0.f);
        if constexpr (SUBS > 1) y.e[i] = here ? y.e[i] : from_float<T>(0.f);
      }
      df[s] = __builtin_bit_cast(frag_t, d.raw);
      if constexpr (SUBS > 1) pf[s] = __builtin_bit_cast(frag_t, y.raw);
    }
    {
      const uint32_t tile_lds = ring_lds + ((3 * b + 1) % kStages) * TB;
#pragma unroll
      for (int s = 0; s < 2; s++)
#pragma unroll
        for (int j4 = 0; j4 < ND; j4 += 4) {
          frag_t tf[4];
          const uint32_t t0 = tile_lds + s * (32 * 2 * D);
          tr_frags4<T, 4 * 2 * D>(tf, t0 + tr_do[j4], t0 + tr_do[j4 + 1], t0 + tr_do[j4 + 2], t0 + tr_do[j4 + 3]);
#pragma unroll
          for (int j = 0; j < 4; j++) dv[j4 + j] = M::run(tf[j], pf[s], dv[j4 + j]);
        }
    }
    step(3 * b + 2);
    {
      const uint32_t tile_lds = ring_lds + ((3 * b + 2) % kStages) * TB;
#pragma unroll
      for (int s = 0; s < 2; s++)
#pragma unroll
        for (int j4 = 0; j4 < ND; j4 += 4) {
          frag_t tf[4];
          const uint32_t t0 = tile_lds + s * (32 * 2 * D);
          tr_frags4<T, 4 * 2 * D>(tf, t0 + tr_q[j4], t0 + tr_q[j4 + 1], t0 + tr_q[j4 + 2], t0 + tr_q[j4 + 3]);
#pragma unroll
          for (int j = 0; j < 4; j++) dk[j4 + j] = M::run(tf[j], df[s], dk[j4 + j]);
        }
    }
  }
  if (slot >= 0) {
    // one part of a long column: its sums in fp32 into the part's slot [dk, dv][64 keys][D]; k_attn64_kv_sum adds the
    // parts of the column in their order
    float *ws = a.partial + ((int64_t)z * a.n_slots + slot) * (2 * 64 * D) + (wave * 16 + qrow) * D + 4 * q;
#pragma unroll
    for (int j = 0; j < ND; j++) {
      *reinterpret_cast<f32x4 *>(ws + 16 * j) = dk[j];
      *reinterpret_cast<f32x4 *>(ws + 64 * D + 16 * j) = dv[j];
    }
    return;
  }
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  store_rows<T, D>(cs, pdk, a.o_ld, dk, lane);
  store_rows<T, D>(cs, pdv, a.o2_ld, dv, lane);
}

// dk and dv of the columns that were computed in parts: per (batch, such column) the sum of its parts' slots, in order.
// a.lut here: per column eight ints (head, column, first slot, parts, then its S block-columns).
template <typename T, int D, int SUBS>
__global__ void __launch_bounds__(256) k_attn64_kv_sum(AttnArgs a) {
  // four workgroups per (batch, column), a quarter of the 2 x 64 x D sums each
  const int quarter = blockIdx.x & 3, col = (blockIdx.x >> 2) % a.R, z = (blockIdx.x >> 2) / a.R;
  const table_ptr lut = as_table(a.lut);
  const int h = lut[8 * col + 0], first = lut[8 * col + 2], parts = lut[8 * col + 3];
  const i32x4 groups = i32x4{lut[8 * col + 4], lut[8 * col + 5], lut[8 * col + 6], lut[8 * col + 7]};
  const float *ws = a.partial + ((int64_t)z * a.n_slots + first) * (2 * 64 * D);
  constexpr int PER = 64 * D / 4;                        // groups of four values per result
#pragma unroll
  for (int t = 0; t < 2 * PER / 1024; t++) {
    const int g = (quarter * (2 * PER / 1024) + t) * 256 + threadIdx.x, which = g / PER, rem = g % PER, key = rem / (D / 4), d4 = rem % (D / 4);
    f32x4 sum = *reinterpret_cast<const f32x4 *>(ws + 4 * g);
    for (int part = 1; part < parts; part++) {
      const f32x4 v = *reinterpret_cast<const f32x4 *>(ws + (int64_t)part * (2 * 64 * D) + 4 * g);
#pragma unroll
      for (int e = 0; e < 4; e++) sum[e] += v[e];
    }
    union { u32x2 raw; T e[4]; } pk;
#pragma unroll
    for (int e = 0; e < 4; e++) pk.e[e] = from_float<T>(sum[e]);
    const int64_t pos = element_position<SUBS>(groups, key);
    T *dst = which ? reinterpret_cast<T *>(a.o2) + z * a.o2_sz + h * a.o2_sh + pos * a.o2_ld
                   : reinterpret_cast<T *>(a.o) + z * a.o_sz + h * a.o_sh + pos * a.o_ld;
    *reinterpret_cast<u32x2 *>(dst + 4 * d4) = pk.raw;
  }
}

template <typename T, int D, int SUBS> void launch_kv(const AttnArgs &a, hipStream_t st) {
  const dim3 grid((unsigned)((int64_t)a.Z * a.R)), wg(256);
  constexpr int LDS = ring_stages<D>() * 64 * D * 2 + ring_stages<D>() * 256;
  static_assert(LDS <= 64 * 1024, "within what a launch may ask for without raising the kernel's limit");
  hipLaunchKernelGGL((k_attn64_bwd_kv<T, D, SUBS>), grid, wg, LDS, st, a);
  if (a.n_split > 0) {
    AttnArgs b = a;
    b.lut = a.split_lut;
    b.R = a.n_split;
    hipLaunchKernelGGL((k_attn64_kv_sum<T, D, SUBS>), dim3((unsigned)((int64_t)a.Z * a.n_split * 4)), wg, 0, st, b);
  }
}

template <typename T, int SUBS> int launch_kv_d(const AttnArgs &a, int D, hipStream_t st) {
  if (D == 64) launch_kv<T, 64, SUBS>(a, st);
  else if (D == 128) launch_kv<T, 128, SUBS>(a, st);
  else return BSP_ERR_UNSUPPORTED;
  return BSP_OK;
}

template <typename T> int launch_kv_t(const AttnArgs &a, int D, int block, hipStream_t st) {
  if (block == 64) return launch_kv_d<T, 1>(a, D, st);
  if (block == 32) return launch_kv_d<T, 2>(a, D, st);
  if (block == 16) return launch_kv_d<T, 4>(a, D, st);
  return BSP_ERR_UNSUPPORTED;
}

}  // namespace

int attention_kv(int dtype, const AttnArgs &a, int D, int block, hipStream_t st) {
  if (dtype == BSP_F16) return launch_kv_t<f16>(a, D, block, st);
  if (dtype == BSP_BF16) return launch_kv_t<bf16>(a, D, block, st);
  return BSP_ERR_UNSUPPORTED;
}

}  // namespace bsp
