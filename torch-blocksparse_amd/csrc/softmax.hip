// Block-sparse softmax, forward and backward, for gfx950.
//
// Replaces the reference's softmax_fwd / softmax_bwd (softmax.py:7-138, 144-194).  The reference runs one
// program per matrix row; here a few lanes share a row, each owning one 16-byte chunk of every nonzero block of
// the row (block 64, fp16: 8 lanes per row, a 64-lane wavefront covers 8 consecutive rows, so every load or
// store instruction of a wavefront touches 1 KiB of consecutive addresses).  The row's values stay in registers
// between the passes; the row maximum / sum are a few xor-shuffles.  Each block is read and written exactly once,
// so the kernel moves the algorithmic 2 (forward) or 3 (backward) passes over x and nothing more.  Many small
// wavefronts rather than few large ones: that is what keeps enough loads in flight to fill the HBM pipe.
// Rows with more blocks than fit in registers take a streaming variant that re-reads x.
#include "softmax_common.h"
#include <type_traits>

namespace bsp {
namespace {

// Wavefronts per workgroup by bucket (NB as in the kernels below).  A workgroup starts only when every one of its
// wavefronts has a slot, and a wavefront of the 32-block bucket takes a third of a SIMD's registers: with 4 per
// workgroup the CUs ran 1.7 wavefronts per SIMD on average where 3 fit.  Measured (forward / backward, us):
// 32-block bucket (block 16, rows of 28 blocks) 117 / 137 with 4, 97 / 122 with 2, 89 / 119 with 1; 16-block bucket
// (block 32, 14 blocks) 88 / 121 with 4, 85 / 118 with 2, 86 / 120 with 1; 7 blocks at block 64: 80 / 116 with 4,
// 80.5 / 115 with 2, 82 / 116 with 1, 86 / 126 with 8.
template <int NB> constexpr int waves_per_group_fwd() { return NB >= 32 ? 1 : NB >= 16 ? 2 : 4; }
template <int NB> constexpr int waves_per_group_bwd() { return NB >= 32 ? 1 : NB > 0 ? 2 : 4; }
// Blocks per step of the streaming variants (rows longer than the register variants hold): all loads of a step are in
// flight together.  Such rows come with few wavefronts per byte (a 8192-column row of blocks of 64 is 128 blocks for one
// wavefront), so the bytes in flight per wavefront decide the rate: 16 blocks per step where the registers allow it
// (no relative position embedding / attention mask beside x), 8 otherwise.
constexpr int kChunk = 8;
constexpr int kChunkPlain = 16;

// Geometry: LPR lanes share a row and each owns one chunk of EV consecutive columns of every block (16 bytes,
// 8 bytes for blocks 16 and 32 in 16-bit types); a wavefront covers RPW = 64 / LPR consecutive rows of one block-row, so a
// load instruction of the wavefront reads RPW whole rows of a block: consecutive addresses.
template <typename T, int BLOCK> struct Geo {
  static constexpr int LPR_ = BLOCK * (int)sizeof(T) / 16;
  // 16-bit block 32: 8 lanes of 8 bytes rather than 4 of 16 (half the registers per lane, more wavefronts per SIMD:
  // measured 14 % faster on rows of 14 blocks); 4-byte pieces (8 lanes at block 16) were measured 60 % slower
  static constexpr int LPR_MIN = (sizeof(T) == 2 && BLOCK == 32) ? 8 : 64 / BLOCK;
  static constexpr int LPR = LPR_ > LPR_MIN ? LPR_ : LPR_MIN;
  static constexpr int EV = BLOCK / LPR;
  static constexpr int RPW = 64 / LPR;
  static constexpr int G = BLOCK / RPW;   // wavefronts per block-row
};

// where does this wavefront work?  unit = ((z * H*R) + block-row) * G + row group
template <typename T, int BLOCK> struct Unit {
  int z, hr, rxm, col;   // batch, head*R + block-row, row inside the block, lane's first column inside a block
  bool ok;
  // shared_masks: the launch reads a relative position embedding or an attention mask.  Their rows are the same for
  // every head (and batch), so the units are then ordered block-row first, heads and batches inside: the wavefronts
  // that need the same mask rows run at the same time on the same XCD and all but the first find them in its L2.
  __device__ __forceinline__ Unit(int64_t n_units, int HR, int wpg, bool shared_masks = false, int H = 1, int Z = 1) {
    typedef Geo<T, BLOCK> GE;
    const int64_t n_wg = (n_units + wpg - 1) / wpg;
    const int64_t wg = xcd_remap(blockIdx.x, n_wg);
    // the wavefront index is uniform: as a scalar it keeps row sizes, block ids and base addresses out of the VALU
    const int64_t u = wg * wpg + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    ok = u < n_units;
    const int lane = threadIdx.x & 63;
    int g = (int)(u % GE::G);
    const int64_t t = u / GE::G;
    // Block-rows are taken from the last one down.  The matmul kernels on either side of this one walk a causal
    // layout from its longest rows (the last ones) to its shortest, so this order reads first what the producer wrote
    // last; measured in the attention chain it makes this kernel and its consumer 3-5 % faster than the ascending order.
    if (shared_masks) {
      // (batch, head) fastest: the wavefronts of a workgroup then read the same mask rows at the same time, and all but
      // the first find them in the vector cache of their CU instead of fetching them from L2 again
      const int R = HR / H, ZH = Z * H;
      const int zh = (int)(u % ZH);
      const int64_t t2 = u / ZH;
      z = zh % Z;
      g = (int)(t2 % GE::G);
      // An XCD works on a contiguous eighth of the units.  Block-rows are dealt to the eighths in turn, so that each XCD
      // gets short and long rows of a causal layout alike (an XCD draws about its share of the memory bandwidth: the one
      // with the longest rows would finish last).
      int br = (int)((t2 / GE::G) % R);
      if (R % 8 == 0) br = (br % (R / 8)) * 8 + br / (R / 8);
      hr = (zh / Z) * R + (R - 1 - br);
    } else {
      hr = HR - 1 - (int)(t % HR);
      z = (int)(t / HR);
    }
    rxm = g * GE::RPW + lane / GE::LPR;
    col = (lane % GE::LPR) * GE::EV;
  }
};

template <typename T, int BLOCK, bool DROP>
__device__ __forceinline__ void fwd_store(const FwdArgs &a, const Unit<T, BLOCK> &u, int64_t blockid, const float (&y)[Geo<T, BLOCK>::EV]) {
  constexpr int EV = Geo<T, BLOCK>::EV;
  const int64_t in_z = blockid * (BLOCK * BLOCK) + u.rxm * BLOCK + u.col;
  T *x = reinterpret_cast<T *>(a.x) + (int64_t)u.z * a.x_sz + in_z;
  Pack<T, EV> p;
#pragma unroll
  for (int e = 0; e < EV; e++) p.e[e] = from_float<T>(y[e]);
  p.store(x);
  if constexpr (DROP) {   // the dropped copy goes to its own tensor: the backward pass needs the softmax itself
    float m[EV];
    keep_scale<EV>(a.drop, (int64_t)u.z * a.x_sz + in_z, m);
    Pack<T, EV> q;
#pragma unroll
    for (int e = 0; e < EV; e++) q.e[e] = from_float<T>(y[e] * m[e]);
    q.store(reinterpret_cast<T *>(a.drop.yd) + (int64_t)u.z * a.drop.yd_sz + in_z);
  }
}

// NB = number of blocks of a row kept in registers; NB == 0 selects the streaming variant.  EXTRA = a relative
// position embedding or an attention mask is present (their values are kept beside x until the logits are built; the
// plain variant does not pay registers for them).
template <typename T, int BLOCK, int NB, bool EXTRA, bool DROP>
__global__ void __launch_bounds__(64 * waves_per_group_fwd<NB>()) k_softmax_fwd(FwdArgs a) {
  typedef Geo<T, BLOCK> GE;
  constexpr int WPG = waves_per_group_fwd<NB>();
  const int HR = a.H * a.R;
  Unit<T, BLOCK> u(a.n_units, HR, WPG, EXTRA, a.H, a.Z);
  if (!u.ok) return;
  const table_ptr lut = as_table(a.lut);
  const int size = lut[2 * u.hr + 0];                   // header (size, offset), softmax.py:30-32
  const int offset = lut[2 * u.hr + 1];
  const int head = u.hr / a.R, brow = u.hr % a.R;       // = the table's (row, head) fields of every block of this row
  if (size <= 0) return;
  const table_ptr core = lut + offset;
  if constexpr (NB > 0) {
    if constexpr (NB >= 32) {
      typedef Pack<T, GE::EV> P;
      constexpr int NX = EXTRA ? NB : 1;
      // Long rows are guarded GS blocks at a time: a guard per block costs a scalar compare, a mask and a branch in
      // each of the five loops below (and the masks no longer fit the scalar registers at 32 blocks).  Inside a live
      // group the blocks past the end of the row repeat the row's last block, so every access is valid, and get
      // -inf added to their logits, so they contribute exp(-inf) = 0; they are not stored.
      constexpr int GS = 4;
      float fx[NB][GE::EV];
      P px[NB], pr[NX], pa[NX];
      int32_t bid[NB], bcol[NX];
      float mx = -INFINITY;
      const int last = size - 1;
#pragma unroll
      for (int b = 0; b < NB; b++) {
        const int bb = b < last ? b : last;               // blocks past the end repeat the last one
        bid[b] = core[4 * bb + 0];
        if constexpr (EXTRA) bcol[b] = core[4 * bb + 1];
      }
      // keeps the table reads here, all in flight together: left alone, each one sinks to just before its block's load
#pragma unroll
      for (int b = 0; b < NB; b++) asm volatile("" : "+s"(bid[b]));
      // Every load of the row is issued before anything waits for one: the wavefront pays the memory latency once,
      // not once per block.  (Loads and the arithmetic on them in one per-block branch end up serialised.)
      const T *xb = reinterpret_cast<const T *>(a.x) + (int64_t)u.z * a.x_sz + u.rxm * BLOCK + u.col;
      const int64_t grow = (int64_t)brow * BLOCK + u.rxm;  // row in the dense matrix
#pragma unroll
      for (int g = 0; g < NB; g += GS)
        if (g < size) {
#pragma unroll
          for (int b = g; b < g + GS; b++) {
            px[b].load(xb + (int64_t)bid[b] * (BLOCK * BLOCK));
            if constexpr (EXTRA) {
              const int64_t gcol = (int64_t)bcol[b] * BLOCK + u.col;   // lane's first column in the dense matrix
              if (a.rpe)                                               // address: softmax.py:50-55
                pr[b].load(reinterpret_cast<const T *>(a.rpe) + u.z * a.rpe_sz + head * a.rpe_sh + grow * a.rpe_sr + gcol);
              if (a.attn) pa[b].load(reinterpret_cast<const T *>(a.attn) + grow * a.attn_sr + gcol);   // :67-70
            }
          }
        }
      // All rows of a wavefront need the same BLOCK key-padding values per block.  The wavefront fetches them once
      // (one chunk per lane), turns them into the term that is added to the logits (softmax.py:104-106, 122-124) and
      // keeps that in its own piece of LDS: 1/RPW of the load instructions, of the bytes moved between the caches and
      // the CU, and of the conversions, compared with every row reading the mask itself.
      __shared__ __attribute__((aligned(16))) float kpm_lds[WPG * NB * BLOCK];
      float *kpm_s = kpm_lds + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) * (NB * BLOCK);
      const float unit = logit_unit<T>();
      const bool has_kpm = a.kpm != nullptr;
      if (has_kpm) {
        const int lane = threadIdx.x & 63;
        const T *kz = reinterpret_cast<const T *>(a.kpm) + u.z * a.kpm_sz;
        constexpr int CH = NB * GE::LPR;                  // chunks of EV values
#pragma unroll
        for (int c0 = 0; c0 < CH; c0 += 64) {
          const int c = c0 + lane, b = c / GE::LPR;
          if ((CH % 64 == 0 || c < CH) && c0 / GE::LPR / GS * GS < size) {
            const int col = a.lut[offset + 4 * (b < last ? b : last) + 1];   // the lane's block: a vector load of the table
            P p;
            p.load(kz + (int64_t)col * BLOCK + (c % GE::LPR) * GE::EV);
#pragma unroll
            for (int e4 = 0; e4 < GE::EV; e4 += 4) {       // EV is 4 or 8: whole 16-byte LDS accesses
              f32x4 add;
#pragma unroll
              for (int e = 0; e < 4; e++) {
                const float m = to_float(p.e[e4 + e]);
                add[e] = a.kpm_mul ? (m == 0.f ? -INFINITY : 0.f) : m * unit;
                if (b >= size) add[e] = -INFINITY;
              }
              *reinterpret_cast<f32x4 *>(&kpm_s[c * GE::EV + e4]) = add;
            }
          }
        }
        __builtin_amdgcn_wave_barrier();                  // LDS operations of one wavefront complete in order
      }
      const float sc = a.scale * unit;
      auto extra_terms = [&](int b) {                     // all terms of a block in one place: its raw registers die here
        if constexpr (EXTRA) {
          if (a.rpe) {                                    // :118-120
#pragma unroll
            for (int e = 0; e < GE::EV; e++) fx[b][e] = fmaf(to_float(pr[b].e[e]), unit, fx[b][e]);
          }
          if (a.attn) {                                   // :126-128, 'mul' mode :108-110
#pragma unroll
            for (int e = 0; e < GE::EV; e++) {
              const float m = to_float(pa[b].e[e]);
              fx[b][e] += a.attn_mul ? (m == 0.f ? -INFINITY : 0.f) : m * unit;
            }
          }
        }
        // In the large buckets the scheduler is kept from interleaving blocks: the raw registers of a block then die as
        // its logits are born (a quarter fewer registers, one more wavefront per SIMD where there were two).
        if constexpr (NB >= 16 || (EXTRA && NB >= 8)) __builtin_amdgcn_sched_barrier(0);
      };
#pragma unroll
      for (int g = 0; g < NB; g += GS)
        if (g < size) {                                   // softmax.py:112-116, 122-124
          float add[GS][GE::EV];
          if (has_kpm) {
#pragma unroll
            for (int b = g; b < g + GS; b++) {
#pragma unroll
              for (int e4 = 0; e4 < GE::EV; e4 += 4)
                *reinterpret_cast<f32x4 *>(&add[b - g][e4]) = *reinterpret_cast<const f32x4 *>(&kpm_s[b * BLOCK + u.col + e4]);
            }
          } else {
#pragma unroll
            for (int b = g; b < g + GS; b++) {
#pragma unroll
              for (int e = 0; e < GE::EV; e++) add[b - g][e] = b >= size ? -INFINITY : 0.f;
            }
          }
#pragma unroll
          for (int b = g; b < g + GS; b++) {
#pragma unroll
            for (int e = 0; e < GE::EV; e++) fx[b][e] = fmaf(to_float(px[b].e[e]), sc, add[b - g][e]);
            extra_terms(b);
          }
        }
#pragma unroll
      for (int g = 0; g < NB; g += GS)
        if (g < size) {
#pragma unroll
          for (int b = g; b < g + GS; b++) {
#pragma unroll
            for (int e = 0; e < GE::EV; e++) mx = fmaxf(mx, fx[b][e]);
          }
        }
      mx = row_max<GE::LPR>(mx);                          // :130
      float sum = 0.f;
#pragma unroll
      for (int g = 0; g < NB; g += GS)
        if (g < size) {
#pragma unroll
          for (int b = g; b < g + GS; b++) {
#pragma unroll
            for (int e = 0; e < GE::EV; e++) { fx[b][e] = exp_sub<T>(fx[b][e], mx); sum += fx[b][e]; }   // :131-132
          }
        }
      sum = row_sum<GE::LPR>(sum);
      const float inv = 1.f / sum;
#pragma unroll
      for (int b = 0; b < NB; b++)
        if (b < size) {
#pragma unroll
          for (int e = 0; e < GE::EV; e++) fx[b][e] *= inv;                                            // :137
          fwd_store<T, BLOCK, DROP>(a, u, bid[b], fx[b]);
        }
    } else {
      typedef Pack<T, GE::EV> P;
      constexpr int NX = EXTRA ? NB : 1;
      float fx[NB][GE::EV];
      P px[NB], pr[NX], pa[NX];
      int32_t bid[NB], bcol[NB];
      float mx = -INFINITY;
#pragma unroll
      for (int b = 0; b < NB; b++) {
        const int bb = b < size ? b : 0;                  // blocks past the end repeat the first one (never used, valid to read)
        bid[b] = core[4 * bb + 0];
        bcol[b] = core[4 * bb + 1];
      }
      // Every load of the row is issued before anything waits for one: the wavefront pays the memory latency once,
      // not once per block.  (Loads and the arithmetic on them in one per-block branch end up serialised.)
      const T *xb = reinterpret_cast<const T *>(a.x) + (int64_t)u.z * a.x_sz + u.rxm * BLOCK + u.col;
      const int64_t grow = (int64_t)brow * BLOCK + u.rxm;  // row in the dense matrix
#pragma unroll
      for (int b = 0; b < NB; b++)
        if (b < size) {
          px[b].load(xb + (int64_t)bid[b] * (BLOCK * BLOCK));
          if constexpr (EXTRA) {
            const int64_t gcol = (int64_t)bcol[b] * BLOCK + u.col;   // lane's first column in the dense matrix
            if (a.rpe)                                               // address: softmax.py:50-55
              pr[b].load(reinterpret_cast<const T *>(a.rpe) + u.z * a.rpe_sz + head * a.rpe_sh + grow * a.rpe_sr + gcol);
            if (a.attn) pa[b].load(reinterpret_cast<const T *>(a.attn) + grow * a.attn_sr + gcol);   // :67-70
          }
        }
      // All rows of a wavefront need the same BLOCK key-padding values per block.  The wavefront fetches them once
      // (one chunk per lane), turns them into the term that is added to the logits (softmax.py:104-106, 122-124) and
      // keeps that in its own piece of LDS: 1/RPW of the load instructions, of the bytes moved between the caches and
      // the CU, and of the conversions, compared with every row reading the mask itself.
      __shared__ __attribute__((aligned(16))) float kpm_lds[WPG * NB * BLOCK];
      float *kpm_s = kpm_lds + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) * (NB * BLOCK);
      const float unit = logit_unit<T>();
      if (a.kpm) {
        const int lane = threadIdx.x & 63;
        const T *kz = reinterpret_cast<const T *>(a.kpm) + u.z * a.kpm_sz;
        constexpr int CH = NB * GE::LPR;                  // chunks of EV values
#pragma unroll
        for (int c0 = 0; c0 < CH; c0 += 64) {
          const int c = c0 + lane, b = c / GE::LPR;
          int col = bcol[0];
#pragma unroll
          for (int i = 1; i < NB; i++) col = (b == i) ? bcol[i] : col;
          if (CH % 64 == 0 || c < CH) {
            P p;
            p.load(kz + (int64_t)col * BLOCK + (c % GE::LPR) * GE::EV);
#pragma unroll
            for (int e4 = 0; e4 < GE::EV; e4 += 4) {       // EV is 4 or 8: whole 16-byte LDS accesses
              f32x4 add;
#pragma unroll
              for (int e = 0; e < 4; e++) {
                const float m = to_float(p.e[e4 + e]);
                add[e] = a.kpm_mul ? (m == 0.f ? -INFINITY : 0.f) : m * unit;
              }
              *reinterpret_cast<f32x4 *>(&kpm_s[c * GE::EV + e4]) = add;
            }
          }
        }
        __builtin_amdgcn_wave_barrier();                  // LDS operations of one wavefront complete in order
      }
      const float sc = a.scale * unit;
      const bool has_kpm = a.kpm != nullptr;
#pragma unroll
      for (int b = 0; b < NB; b++)
        if (b < size) {                                   // softmax.py:112-116, 122-124
#pragma unroll
          for (int e4 = 0; e4 < GE::EV; e4 += 4) {
            const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
            const f32x4 add = has_kpm ? *reinterpret_cast<const f32x4 *>(&kpm_s[b * BLOCK + u.col + e4]) : zero4;
#pragma unroll
            for (int e = 0; e < 4; e++) fx[b][e4 + e] = fmaf(to_float(px[b].e[e4 + e]), sc, add[e]);
          }
          if constexpr (EXTRA) {                          // all terms of a block in one place: its raw registers die here
            if (a.rpe) {                                    // :118-120
#pragma unroll
              for (int e = 0; e < GE::EV; e++) fx[b][e] = fmaf(to_float(pr[b].e[e]), unit, fx[b][e]);
            }
            if (a.attn) {                                   // :126-128, 'mul' mode :108-110
#pragma unroll
              for (int e = 0; e < GE::EV; e++) {
                const float m = to_float(pa[b].e[e]);
                fx[b][e] += a.attn_mul ? (m == 0.f ? -INFINITY : 0.f) : m * unit;
              }
            }
          }
          // In the large buckets the scheduler is kept from interleaving blocks: the raw registers of a block then die as
          // its logits are born (a quarter fewer registers, one more wavefront per SIMD where there were two).
          if constexpr (NB >= 16 || (EXTRA && NB >= 8)) __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
      for (int b = 0; b < NB; b++)
        if (b < size) {
#pragma unroll
          for (int e = 0; e < GE::EV; e++) mx = fmaxf(mx, fx[b][e]);
        }
      mx = row_max<GE::LPR>(mx);                          // :130
      float sum = 0.f;
#pragma unroll
      for (int b = 0; b < NB; b++)
        if (b < size) {
#pragma unroll
          for (int e = 0; e < GE::EV; e++) { fx[b][e] = exp_sub<T>(fx[b][e], mx); sum += fx[b][e]; }   // :131-132
        }
      sum = row_sum<GE::LPR>(sum);
      const float inv = 1.f / sum;
#pragma unroll
      for (int b = 0; b < NB; b++)
        if (b < size) {
#pragma unroll
          for (int e = 0; e < GE::EV; e++) fx[b][e] *= inv;                                            // :137
          fwd_store<T, BLOCK, DROP>(a, u, bid[b], fx[b]);
        }
    }
  } else {
    // Rows with more blocks than the register variant holds: two passes over x, kChunk blocks at a time with all loads
    // of a chunk in flight together.  Pass 1 keeps a running maximum and a running sum per lane (the sum is rescaled
    // when the maximum grows), pass 2 reads x again and writes the result: 2 reads + 1 write of x.
    typedef Pack<T, GE::EV> P;
    constexpr int CH = EXTRA ? kChunk : kChunkPlain, NX = EXTRA ? CH : 1;
    const float unit = logit_unit<T>();
    const float sc = a.scale * unit;
    const T *xb = reinterpret_cast<const T *>(a.x) + (int64_t)u.z * a.x_sz + u.rxm * BLOCK + u.col;
    const int64_t grow = (int64_t)brow * BLOCK + u.rxm;
    const T *kz = reinterpret_cast<const T *>(a.kpm) + u.z * a.kpm_sz + u.col;
    const T *rz = reinterpret_cast<const T *>(a.rpe) + u.z * a.rpe_sz + head * a.rpe_sh + grow * a.rpe_sr + u.col;
    const T *az = reinterpret_cast<const T *>(a.attn) + grow * a.attn_sr + u.col;
    P px[CH], pk[CH], pr[NX], pa[NX];
    int32_t bid[CH], bcol[CH];
    auto load_chunk = [&](int b0) {
#pragma unroll
      for (int j = 0; j < CH; j++) {                    // table reads first, unconditional: one wait for all of them
        const int bb = b0 + j < size ? b0 + j : b0;
        bid[j] = core[4 * bb + 0];
        bcol[j] = core[4 * bb + 1];
      }
#pragma unroll
      for (int j = 0; j < CH; j++)
        if (b0 + j < size) {
          const int64_t c0 = (int64_t)bcol[j] * BLOCK;  // first column of the block in the dense matrix
          px[j].load(xb + (int64_t)bid[j] * (BLOCK * BLOCK));
          if (a.kpm) pk[j].load(kz + c0);
          if constexpr (EXTRA) {
            if (a.rpe) pr[j].load(rz + c0);
            if (a.attn) pa[j].load(az + c0);
          }
        }
    };
    auto logits = [&](int j, float (&l)[GE::EV]) {      // softmax.py:104-128
#pragma unroll
      for (int e = 0; e < GE::EV; e++) l[e] = to_float(px[j].e[e]) * sc;
      if (a.kpm) {
#pragma unroll
        for (int e = 0; e < GE::EV; e++) {
          const float m = to_float(pk[j].e[e]);
          l[e] += a.kpm_mul ? (m == 0.f ? -INFINITY : 0.f) : m * unit;
        }
      }
      if constexpr (EXTRA) {
        if (a.rpe) {
#pragma unroll
          for (int e = 0; e < GE::EV; e++) l[e] = fmaf(to_float(pr[j].e[e]), unit, l[e]);
        }
        if (a.attn) {
#pragma unroll
          for (int e = 0; e < GE::EV; e++) {
            const float m = to_float(pa[j].e[e]);
            l[e] += a.attn_mul ? (m == 0.f ? -INFINITY : 0.f) : m * unit;
          }
        }
      }
    };
    float mx = -INFINITY, sum = 0.f;
    for (int b0 = 0; b0 < size; b0 += CH) {
      load_chunk(b0);
#pragma unroll
      for (int j = 0; j < CH; j++)
        if (b0 + j < size) {
          float l[GE::EV];
          logits(j, l);
          float m = mx;
#pragma unroll
          for (int e = 0; e < GE::EV; e++) m = fmaxf(m, l[e]);
          const float ms = m == -INFINITY ? 0.f : m;    // everything masked so far: any finite shift does
          float part = 0.f;
#pragma unroll
          for (int e = 0; e < GE::EV; e++) part += exp_sub<T>(l[e], ms);
          sum = sum * exp_sub<T>(mx, ms) + part;
          mx = m;
        }
    }
    const float rmx = row_max<GE::LPR>(mx);             // :130
    const float shift = rmx == -INFINITY ? 0.f : rmx;   // a fully masked row ends as 0 * inf = NaN, like the register variant
    sum = row_sum<GE::LPR>(sum * exp_sub<T>(mx, shift));
    const float inv = 1.f / sum;
    for (int b0 = 0; b0 < size; b0 += CH) {
      load_chunk(b0);
#pragma unroll
      for (int j = 0; j < CH; j++)
        if (b0 + j < size) {
          float l[GE::EV];
          logits(j, l);
          float yv[GE::EV];
#pragma unroll
          for (int e = 0; e < GE::EV; e++) yv[e] = exp_sub<T>(l[e], shift) * inv;                     // :131-137
          fwd_store<T, BLOCK, DROP>(a, u, bid[j], yv);
        }
    }
  }
}

// dy <- dy * mask / (1 - p) for the chunk of block `blockid` this lane holds: the gradient of the dropped result turned
// into the gradient of the softmax itself (the mask is re-created from the counter, see DropArgs)
template <typename T, int BLOCK>
__device__ __forceinline__ void drop_grad(const BwdArgs &a, const Unit<T, BLOCK> &u, int64_t blockid, Pack<T, Geo<T, BLOCK>::EV> &pd) {
  constexpr int EV = Geo<T, BLOCK>::EV;
  float m[EV];
  keep_scale<EV>(a.drop, (int64_t)u.z * a.y_sz + blockid * (BLOCK * BLOCK) + u.rxm * BLOCK + u.col, m);
#pragma unroll
  for (int e = 0; e < EV; e++) pd.e[e] = from_float<T>(to_float(pd.e[e]) * m[e]);
}

template <typename T, int BLOCK, int NB, bool DROP>
__global__ void __launch_bounds__(64 * waves_per_group_bwd<NB>()) k_softmax_bwd(BwdArgs a) {
  typedef Geo<T, BLOCK> GE;
  typedef Pack<T, GE::EV> P;
  const int HR = a.H * a.R;
  Unit<T, BLOCK> u(a.n_units, HR, waves_per_group_bwd<NB>());
  if (!u.ok) return;
  const table_ptr lut = as_table(a.lut);
  const int size = lut[2 * u.hr + 0];
  const int offset = lut[2 * u.hr + 1];
  if (size <= 0) return;
  const table_ptr core = lut + offset;
  const T *yb = reinterpret_cast<const T *>(a.y) + (int64_t)u.z * a.y_sz + u.rxm * BLOCK + u.col;
  T *db = reinterpret_cast<T *>(a.dy) + (int64_t)u.z * a.dy_sz + u.rxm * BLOCK + u.col;
  if constexpr (NB > 0) {
    if constexpr (NB >= 32) {
      P py[NB], pd[NB];
      int32_t bid[NB];
      float dot = 0.f;
      // the long-row bucket is guarded four blocks at a time, like the forward kernel's: blocks past the end of the row
      // repeat its last block (valid to read), stay out of the dot product and are not stored
      const int last = size - 1;
#pragma unroll
      for (int b = 0; b < NB; b++) bid[b] = core[4 * (b < last ? b : last)];
#pragma unroll
      for (int b = 0; b < NB; b++) asm volatile("" : "+s"(bid[b]));   // all table reads in flight together, here
#pragma unroll
      for (int g = 0; g < NB; g += 4)
        if (g < size) {
#pragma unroll
          for (int b = g; b < g + 4; b++) {
            const int64_t o = (int64_t)bid[b] * (BLOCK * BLOCK);
            py[b].load_stream(yb + o);   // y is not read again after the backward pass
            pd[b].load(db + o);
          }
        }
      if constexpr (DROP) {
#pragma unroll
        for (int g = 0; g < NB; g += 4)
          if (g < size) {
#pragma unroll
            for (int b = g; b < g + 4; b++) drop_grad<T, BLOCK>(a, u, bid[b], pd[b]);
          }
      }
#pragma unroll
      for (int g = 0; g < NB; g += 4)
        if (g < size) {
#pragma unroll
          for (int b = g; b < g + 4; b++) {
            float part = 0.f;
#pragma unroll
            for (int e = 0; e < GE::EV; e++) part += to_float(py[b].e[e]) * to_float(pd[b].e[e]);   // softmax.py:187-188
            dot += b < size ? part : 0.f;
          }
        }
      dot = row_sum<GE::LPR>(dot);
#pragma unroll
      for (int b = 0; b < NB; b++)
        if (b < size) {
          P out;
#pragma unroll
          for (int e = 0; e < GE::EV; e++)
            out.e[e] = from_float<T>(to_float(py[b].e[e]) * (to_float(pd[b].e[e]) - dot) * a.scale);   // :189
          out.store(db + (int64_t)bid[b] * (BLOCK * BLOCK));
        }
    } else {
      P py[NB], pd[NB];
      int32_t bid[NB];
      float dot = 0.f;
      // the table reads come first and unconditionally (one wait for all of them, not one round trip per block)
#pragma unroll
      for (int b = 0; b < NB; b++) bid[b] = core[4 * (b < size ? b : 0)];
#pragma unroll
      for (int b = 0; b < NB; b++)
        if (b < size) {
          const int64_t o = (int64_t)bid[b] * (BLOCK * BLOCK);
          py[b].load_stream(yb + o);   // y is not read again after the backward pass
          pd[b].load(db + o);
        }
#pragma unroll
      for (int b = 0; b < NB; b++)
        if (b < size) {
          if constexpr (DROP) drop_grad<T, BLOCK>(a, u, bid[b], pd[b]);
#pragma unroll
          for (int e = 0; e < GE::EV; e++) dot += to_float(py[b].e[e]) * to_float(pd[b].e[e]);   // softmax.py:187-188
        }
      dot = row_sum<GE::LPR>(dot);
#pragma unroll
      for (int b = 0; b < NB; b++)
        if (b < size) {
          P out;
#pragma unroll
          for (int e = 0; e < GE::EV; e++)
            out.e[e] = from_float<T>(to_float(py[b].e[e]) * (to_float(pd[b].e[e]) - dot) * a.scale);   // :189
          out.store(db + (int64_t)bid[b] * (BLOCK * BLOCK));
        }
    }
  } else {
    // longer rows: two passes, kChunkPlain blocks at a time with all loads of a chunk in flight together
    constexpr int CH = kChunkPlain;
    P py[CH], pd[CH];
    int64_t off[CH];
    auto load_chunk = [&](int b0) {
#pragma unroll
      for (int j = 0; j < CH; j++) off[j] = (int64_t)core[4 * (b0 + j < size ? b0 + j : b0)] * (BLOCK * BLOCK);
#pragma unroll
      for (int j = 0; j < CH; j++)
        if (b0 + j < size) {
          py[j].load_stream(yb + off[j]);
          pd[j].load(db + off[j]);
        }
      if constexpr (DROP) {
#pragma unroll
        for (int j = 0; j < CH; j++)
          if (b0 + j < size) drop_grad<T, BLOCK>(a, u, off[j] / (BLOCK * BLOCK), pd[j]);
      }
    };
    float dot = 0.f;
    for (int b0 = 0; b0 < size; b0 += CH) {
      load_chunk(b0);
#pragma unroll
      for (int j = 0; j < CH; j++)
        if (b0 + j < size) {
#pragma unroll
          for (int e = 0; e < GE::EV; e++) dot += to_float(py[j].e[e]) * to_float(pd[j].e[e]);
        }
    }
    dot = row_sum<GE::LPR>(dot);
    for (int b0 = 0; b0 < size; b0 += CH) {
      load_chunk(b0);
#pragma unroll
      for (int j = 0; j < CH; j++)
        if (b0 + j < size) {
          P out;
#pragma unroll
          for (int e = 0; e < GE::EV; e++)
            out.e[e] = from_float<T>(to_float(py[j].e[e]) * (to_float(pd[j].e[e]) - dot) * a.scale);
          out.store(db + off[j]);
        }
    }
  }
}

// Register budget: a lane keeps NB * EV fp32 values (forward) or 2 * NB raw chunks (backward).
template <typename T, int BLOCK> constexpr int max_nb_fwd() { return 128 / Geo<T, BLOCK>::EV > 32 ? 32 : 128 / Geo<T, BLOCK>::EV; }
// backward: 2 raw chunks per block; 8-byte chunks (block 16, 16-bit types) leave room for 32 blocks
template <typename T, int BLOCK> constexpr int max_nb_bwd() { return Geo<T, BLOCK>::EV * (int)sizeof(T) <= 8 ? 32 : 16; }

template <typename T, int BLOCK, int NB> void launch_fwd_nb(const FwdArgs &a, hipStream_t st) {
  constexpr int WPG = waves_per_group_fwd<NB>();
  const int64_t n_wg = (a.n_units + WPG - 1) / WPG;
  const bool extra = a.rpe || a.attn, drop = a.drop.yd != nullptr;
  if (extra && drop) hipLaunchKernelGGL((k_softmax_fwd<T, BLOCK, NB, true, true>), dim3((unsigned)n_wg), dim3(64 * WPG), 0, st, a);
  else if (extra) hipLaunchKernelGGL((k_softmax_fwd<T, BLOCK, NB, true, false>), dim3((unsigned)n_wg), dim3(64 * WPG), 0, st, a);
  else if (drop) hipLaunchKernelGGL((k_softmax_fwd<T, BLOCK, NB, false, true>), dim3((unsigned)n_wg), dim3(64 * WPG), 0, st, a);
  else hipLaunchKernelGGL((k_softmax_fwd<T, BLOCK, NB, false, false>), dim3((unsigned)n_wg), dim3(64 * WPG), 0, st, a);
}
template <typename T, int BLOCK, int NB> void launch_bwd_nb(const BwdArgs &a, hipStream_t st) {
  constexpr int WPG = waves_per_group_bwd<NB>();
  const int64_t n_wg = (a.n_units + WPG - 1) / WPG;
  if (a.drop.p > 0.f) hipLaunchKernelGGL((k_softmax_bwd<T, BLOCK, NB, true>), dim3((unsigned)n_wg), dim3(64 * WPG), 0, st, a);
  else hipLaunchKernelGGL((k_softmax_bwd<T, BLOCK, NB, false>), dim3((unsigned)n_wg), dim3(64 * WPG), 0, st, a);
}

template <typename T> constexpr int dtype_of() { return sizeof(T) == 4 ? BSP_F32 : std::is_same<T, f16>::value ? BSP_F16 : BSP_BF16; }

template <typename T, int BLOCK> void launch_fwd(const FwdArgs &a, int maxlut, hipStream_t st) {
  constexpr int MX = max_nb_fwd<T, BLOCK>();
  if (maxlut <= 1) launch_fwd_nb<T, BLOCK, 1>(a, st);
  else if (maxlut <= 2) launch_fwd_nb<T, BLOCK, 2>(a, st);
  else if (maxlut <= 4) launch_fwd_nb<T, BLOCK, 4>(a, st);
  else if (maxlut <= 6) launch_fwd_nb<T, BLOCK, 6>(a, st);
  else if (maxlut <= 7) launch_fwd_nb<T, BLOCK, 7>(a, st);
  else if (maxlut <= 8) launch_fwd_nb<T, BLOCK, 8>(a, st);
  else if (maxlut <= 16 && 16 <= MX) launch_fwd_nb<T, BLOCK, (16 <= MX ? 16 : 0)>(a, st);
  else if (maxlut <= 32 && 32 <= MX) launch_fwd_nb<T, BLOCK, (32 <= MX ? 32 : 0)>(a, st);
  // longer rows: one wavefront per row while the row fits its registers, else the variant that re-reads x.  (For rows
  // that the register variants above hold, one wavefront per row is 2-3 x slower: measured on rows of 7, 14 and 28 blocks
  // of 64, 32 and 16, forward 0.22 against 0.08-0.09 ms: a kilobyte of work per wavefront does not pay for its set-up.)
  else if (!softmax_row_fwd(dtype_of<T>(), a, BLOCK, maxlut, st)) launch_fwd_nb<T, BLOCK, 0>(a, st);
}
template <typename T, int BLOCK> void launch_bwd(const BwdArgs &a, int maxlut, hipStream_t st) {
  if (maxlut <= 1) launch_bwd_nb<T, BLOCK, 1>(a, st);
  else if (maxlut <= 2) launch_bwd_nb<T, BLOCK, 2>(a, st);
  else if (maxlut <= 4) launch_bwd_nb<T, BLOCK, 4>(a, st);
  else if (maxlut <= 6) launch_bwd_nb<T, BLOCK, 6>(a, st);
  else if (maxlut <= 7) launch_bwd_nb<T, BLOCK, 7>(a, st);
  else if (maxlut <= 8) launch_bwd_nb<T, BLOCK, 8>(a, st);
  else if (maxlut <= 16) launch_bwd_nb<T, BLOCK, 16>(a, st);
  else if (maxlut <= 32 && max_nb_bwd<T, BLOCK>() >= 32) launch_bwd_nb<T, BLOCK, (max_nb_bwd<T, BLOCK>() >= 32 ? 32 : 0)>(a, st);
  else if (!softmax_row_bwd(dtype_of<T>(), a, BLOCK, maxlut, st)) launch_bwd_nb<T, BLOCK, 0>(a, st);
}

template <typename T> int dispatch_fwd(const FwdArgs &a, int block, int maxlut, hipStream_t st) {
  switch (block) {
    case 16: launch_fwd<T, 16>(a, maxlut, st); break;
    case 32: launch_fwd<T, 32>(a, maxlut, st); break;
    case 64: launch_fwd<T, 64>(a, maxlut, st); break;
    case 128: launch_fwd<T, 128>(a, maxlut, st); break;
    default: return BSP_ERR_UNSUPPORTED;
  }
  return BSP_OK;
}
template <typename T> int dispatch_bwd(const BwdArgs &a, int block, int maxlut, hipStream_t st) {
  switch (block) {
    case 16: launch_bwd<T, 16>(a, maxlut, st); break;
    case 32: launch_bwd<T, 32>(a, maxlut, st); break;
    case 64: launch_bwd<T, 64>(a, maxlut, st); break;
    case 128: launch_bwd<T, 128>(a, maxlut, st); break;
    default: return BSP_ERR_UNSUPPORTED;
  }
  return BSP_OK;
}

template <typename T> int64_t units_for(int block, int64_t rows_of_blocks) {
  switch (block) {
    case 16: return rows_of_blocks * Geo<T, 16>::G;
    case 32: return rows_of_blocks * Geo<T, 32>::G;
    case 64: return rows_of_blocks * Geo<T, 64>::G;
    case 128: return rows_of_blocks * Geo<T, 128>::G;
    default: return 0;
  }
}
int64_t n_units(int dtype, int block, int64_t rows_of_blocks) {
  return dtype == BSP_F32 ? units_for<float>(block, rows_of_blocks) : units_for<f16>(block, rows_of_blocks);
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace
}  // namespace bsp

using namespace bsp;

namespace {
bool drop_args(DropArgs &d, float p, uint64_t seed, uint64_t offset) {
  if (!(p >= 0.f) || !(p < 1.f)) return false;
  d.p = p; d.inv_keep = 1.f / (1.f - p);
  d.seed_lo = (uint32_t)seed; d.seed_hi = (uint32_t)(seed >> 32);
  d.off_lo = (uint32_t)offset; d.off_hi = (uint32_t)(offset >> 32);
  return true;
}

int softmax_fwd_impl(int dtype, void *x, float scale, const int32_t *d_lut, int maxlut, const void *rpe, int64_t rpe_stride_z,
                     int64_t rpe_stride_h, int64_t rpe_stride_r, const void *kpm, int64_t kpm_stride_z, int kpm_mul,
                     const void *attn, int64_t attn_stride_r, int attn_mul, int Z, int H, int R, int block, int64_t x_stride_z,
                     const DropArgs &drop, void *stream) {
  if (!x || !d_lut || Z <= 0 || H <= 0 || R <= 0 || maxlut < 0) return BSP_ERR_ARG;
  if ((int64_t)maxlut * block >= 32768) return BSP_ERR_ROW_TOO_LONG;   // softmax.py:225-227
  const int64_t es = dtype == BSP_F32 ? 4 : 2;
  // vector accesses: every row segment a lane touches must start on a 16-byte boundary
  const int64_t unit = 16 / es;
  if (!aligned16(x) || !aligned16(rpe) || !aligned16(kpm) || !aligned16(attn) || !aligned16(drop.yd)) return BSP_ERR_ARG;
  if (x_stride_z % unit || rpe_stride_z % unit || rpe_stride_h % unit || rpe_stride_r % unit || kpm_stride_z % unit ||
      attn_stride_r % unit || drop.yd_sz % unit)
    return BSP_ERR_ARG;
  FwdArgs a;
  a.x = x; a.scale = scale; a.lut = d_lut;
  a.rpe = rpe; a.rpe_sz = rpe_stride_z; a.rpe_sh = rpe_stride_h; a.rpe_sr = rpe_stride_r;
  a.kpm = kpm; a.kpm_sz = kpm_stride_z; a.kpm_mul = kpm_mul;
  a.attn = attn; a.attn_sr = attn_stride_r; a.attn_mul = attn_mul;
  a.Z = Z; a.H = H; a.R = R; a.x_sz = x_stride_z;
  a.drop = drop;
  a.n_units = n_units(dtype, block, (int64_t)Z * H * R);
  if (a.n_units <= 0 || a.n_units >= ((int64_t)1 << 26)) return BSP_ERR_UNSUPPORTED;   // one wavefront per unit: 2^32 threads per launch at most
  int rc;
  switch (dtype) {
    case BSP_F16: rc = dispatch_fwd<f16>(a, block, maxlut, as_stream(stream)); break;
    case BSP_BF16: rc = dispatch_fwd<bf16>(a, block, maxlut, as_stream(stream)); break;
    case BSP_F32: rc = dispatch_fwd<float>(a, block, maxlut, as_stream(stream)); break;
    default: return BSP_ERR_UNSUPPORTED;
  }
  if (rc != BSP_OK) return rc;
  BSP_LAUNCH_CHECK();
  return BSP_OK;
}

int softmax_bwd_impl(int dtype, const void *y, void *dy, float scale, const int32_t *d_lut, int maxlut, int Z, int H, int R,
                     int block, int64_t y_stride_z, int64_t dy_stride_z, const DropArgs &drop, void *stream) {
  if (!y || !dy || !d_lut || Z <= 0 || H <= 0 || R <= 0 || maxlut < 0) return BSP_ERR_ARG;
  if ((int64_t)maxlut * block >= 32768) return BSP_ERR_ROW_TOO_LONG;
  const int64_t unit = dtype == BSP_F32 ? 4 : 8;
  if (!aligned16(y) || !aligned16(dy) || y_stride_z % unit || dy_stride_z % unit) return BSP_ERR_ARG;
  BwdArgs a;
  a.y = y; a.dy = dy; a.scale = scale; a.lut = d_lut;
  a.Z = Z; a.H = H; a.R = R; a.y_sz = y_stride_z; a.dy_sz = dy_stride_z;
  a.drop = drop;
  a.n_units = n_units(dtype, block, (int64_t)Z * H * R);
  if (a.n_units <= 0 || a.n_units >= ((int64_t)1 << 26)) return BSP_ERR_UNSUPPORTED;   // one wavefront per unit: 2^32 threads per launch at most
  int rc;
  switch (dtype) {
    case BSP_F16: rc = dispatch_bwd<f16>(a, block, maxlut, as_stream(stream)); break;
    case BSP_BF16: rc = dispatch_bwd<bf16>(a, block, maxlut, as_stream(stream)); break;
    case BSP_F32: rc = dispatch_bwd<float>(a, block, maxlut, as_stream(stream)); break;
    default: return BSP_ERR_UNSUPPORTED;
  }
  if (rc != BSP_OK) return rc;
  BSP_LAUNCH_CHECK();
  return BSP_OK;
}
}  // namespace

extern "C" int bsp_softmax_fwd(int dtype, void *x, float scale, const int32_t *d_lut, int maxlut, const void *rpe,
                               int64_t rpe_stride_z, int64_t rpe_stride_h, int64_t rpe_stride_r, const void *kpm,
                               int64_t kpm_stride_z, int kpm_mul, const void *attn, int64_t attn_stride_r, int attn_mul, int Z,
                               int H, int R, int block, int64_t x_stride_z, void *stream) {
  return softmax_fwd_impl(dtype, x, scale, d_lut, maxlut, rpe, rpe_stride_z, rpe_stride_h, rpe_stride_r, kpm, kpm_stride_z, kpm_mul,
                          attn, attn_stride_r, attn_mul, Z, H, R, block, x_stride_z, DropArgs(), stream);
}

extern "C" int bsp_softmax_bwd(int dtype, const void *y, void *dy, float scale, const int32_t *d_lut, int maxlut, int Z, int H,
                               int R, int block, int64_t y_stride_z, int64_t dy_stride_z, void *stream) {
  return softmax_bwd_impl(dtype, y, dy, scale, d_lut, maxlut, Z, H, R, block, y_stride_z, dy_stride_z, DropArgs(), stream);
}

extern "C" int bsp_softmax_dropout_fwd(int dtype, void *x, void *y_drop, float scale, const int32_t *d_lut, int maxlut,
                                       const void *rpe, int64_t rpe_stride_z, int64_t rpe_stride_h, int64_t rpe_stride_r,
                                       const void *kpm, int64_t kpm_stride_z, int kpm_mul, const void *attn, int64_t attn_stride_r,
                                       int attn_mul, int Z, int H, int R, int block, int64_t x_stride_z, int64_t y_drop_stride_z,
                                       float drop_p, uint64_t seed, uint64_t offset, void *stream) {
  DropArgs d;
  if (!y_drop || !drop_args(d, drop_p, seed, offset)) return BSP_ERR_ARG;
  d.yd = y_drop; d.yd_sz = y_drop_stride_z;
  return softmax_fwd_impl(dtype, x, scale, d_lut, maxlut, rpe, rpe_stride_z, rpe_stride_h, rpe_stride_r, kpm, kpm_stride_z, kpm_mul,
                          attn, attn_stride_r, attn_mul, Z, H, R, block, x_stride_z, d, stream);
}

extern "C" int bsp_softmax_dropout_bwd(int dtype, const void *y, void *dy, float scale, const int32_t *d_lut, int maxlut, int Z,
                                       int H, int R, int block, int64_t y_stride_z, int64_t dy_stride_z, float drop_p, uint64_t seed,
                                       uint64_t offset, void *stream) {
  DropArgs d;
  if (!drop_args(d, drop_p, seed, offset)) return BSP_ERR_ARG;
  return softmax_bwd_impl(dtype, y, dy, scale, d_lut, maxlut, Z, H, R, block, y_stride_z, dy_stride_z, d, stream);
}
