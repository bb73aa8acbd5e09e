/*
 * bsp.h -- C ABI of the MI355X (gfx950) block-sparse matmul / softmax library.
 *
 * Everything here takes plain device pointers, sizes and element strides; no framework types cross the
 * boundary.  All launches are asynchronous on the given HIP stream (a hipStream_t passed as void*; NULL is
 * the default stream).  The look-up-table builders additionally copy a few scalars back to the host and
 * therefore synchronise that stream once before they return.  No function allocates or frees device
 * memory: outputs, tables and workspaces are provided by the caller.
 *
 * Each entry point names the interface of ptillet/torch-blocksparse that it replaces (file:line of the
 * reference checkout).  Sparse tensors use the reference's storage: [Z, nnz, block, block], block p being
 * the p-th nonzero of the [H, R, C] layout in row-major (head, block-row, block-col) order.
 *
 * Return value: 0 on success, a negative bsp_status otherwise (bsp_strerror gives the text).
 */
#ifndef BSP_H
#define BSP_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef enum { BSP_F16 = 0, BSP_BF16 = 1, BSP_F32 = 2 } bsp_dtype;

typedef enum {
  BSP_OK = 0,
  BSP_OK_WHOLE_LAYOUT = 1,   /* bsp_sdd_matmul only: the group plan was used, every block of the layout is written */
  BSP_NEEDS_TABLE = 2,       /* bsp_sdd_matmul called with the plan alone: nothing launched, call again with the sdd table */
  BSP_ERR_ARG = -1,          /* null pointer, bad size, misaligned operand */
  BSP_ERR_UNSUPPORTED = -2,  /* block size / dtype / mode not built */
  BSP_ERR_CAPACITY = -3,     /* caller-provided table or workspace too small */
  BSP_ERR_EMPTY_HEAD = -4,   /* a head of the layout has no nonzero block (the reference raises here) */
  BSP_ERR_HIP = -5,          /* a HIP runtime call failed */
  BSP_ERR_ROW_TOO_LONG = -6, /* softmax row of >= 32768 elements (reference softmax.py:225-227) */
  BSP_ERR_K_MULTIPLE = -7,   /* sdd reduction size not a multiple of 16 (reference matmul.py:318-319) */
  BSP_ERR_SCRATCH_LIMIT = -8 /* bsp_dsd_matmul_noalloc: the launch needs more scratch than the library's static buffer holds */
} bsp_status;

int bsp_version(void);
const char *bsp_strerror(int status);

/* ---------------------------------------------------------------------------------------------------
 * Layout generators on the device: d_layout receives a [H, NB, NB] int32 layout of 0/1 values, ready for the
 * table builders below; nothing crosses to the host.
 * bsp_layout_fixed: the Sparse-Transformer "fixed" pattern (dense != 0: all ones).  whole_stripes = 0 replaces
 *   torch_blocksparse_cpp_utils.make_layout (csrc/utils.cpp:123-148), which marks only the first column of a vertical
 *   stripe; whole_stripes = 1 replaces DeepSpeedSparseSelfAttention._make_layout
 *   (deepspeedsparseselfattention.py:31-65), which marks all `vertsize` of them.  NB must be a multiple of block_stride.
 * bsp_layout_sparse_transformer: local windows of local_blocks blocks + the last column of every global_stride blocks
 *   as a global column (the benchmark's attention layout; no counterpart in the reference).
 * bsp_layout_bigbird: sliding window + num_global leading global columns (and rows unless causal) + the random columns
 *   d_random_cols [H, NB, num_random] (int32, drawn by the caller); no counterpart in the reference.
 * ------------------------------------------------------------------------------------------------- */
int bsp_layout_fixed(int32_t *d_layout, int H, int NB, int dense, int block_stride, int unidirectional, int numverts,
                     int vertsize, int whole_stripes, void *stream);
int bsp_layout_sparse_transformer(int32_t *d_layout, int H, int NB, int local_blocks, int global_stride, int causal, void *stream);
int bsp_layout_bigbird(int32_t *d_layout, int H, int NB, int window, int num_global, int causal, const int32_t *d_random_cols,
                       int num_random, void *stream);

/* ---------------------------------------------------------------------------------------------------
 * Look-up-table builders.  d_layout is the layout as int32 [H, R, C] in device memory (0/1 values).
 * d_ws is scratch of at least bsp_lut_workspace_bytes(H, R, C) bytes.
 * ------------------------------------------------------------------------------------------------- */
int64_t bsp_lut_workspace_bytes(int H, int R, int C);

/* Number of nonzero blocks of a layout (host result).  Replaces layout.sum() / layout.nonzero().size(0). */
int bsp_layout_nnz(const int32_t *d_layout, int H, int R, int C, void *d_ws, int64_t ws_bytes, int64_t *nnz, void *stream);

/* softmax table: replaces _sparse_softmax.make_lut (softmax.py:201-221).
 * d_lut receives 2*H*R + 4*nnz int32: per block-row (size, offset), then per block (blockid, col, row, head).
 * *maxlut = largest number of blocks in a block-row. */
int bsp_softmax_lut_build(const int32_t *d_layout, int H, int R, int C, int32_t *d_lut, int64_t lut_cap,
                          void *d_ws, int64_t ws_bytes, int64_t *lut_len, int *maxlut, void *stream);

/* dsd/dds table: replaces _sparse_matmul.make_dxx_lut + load_balance (matmul.py:221-267, 372-458).
 * d_lut receives 6*width header ints (offset, segment length, column, depth, lockid, maxid), then the
 * 2*nnz*(block/step) interleaved pointer increments and two trailing zeros -- bit-identical to the reference.
 * d_plan (int32, at least bsp_dxx_plan_cap(...) ints; no counterpart in the reference) receives first the order
 * in which the launchers dispatch the segments (width ints: head by head, inside a head the longest first), then,
 * from int bsp_dxx_plan_pairs_offset(width) on, per block in table order (offset of the block in the dense
 * operand's reduction dimension, storage index of the block): the absolute positions the increments are
 * differences of; the matmul launchers below read them instead of re-summing the increments.
 * lut_cap >= bsp_dxx_lut_cap(...). */
int64_t bsp_dxx_lut_cap(int H, int R, int C, int64_t nnz, int block, int step, int trans);
int64_t bsp_dxx_plan_cap(int H, int R, int C, int64_t nnz, int trans);
int64_t bsp_dxx_plan_pairs_offset(int width);
int bsp_dxx_lut_build(const int32_t *d_layout, int H, int R, int C, int block, int step, int trans,
                      int32_t *d_lut, int64_t lut_cap, int32_t *d_plan, void *d_ws, int64_t ws_bytes,
                      int64_t *lut_len, int *width, int *num_locks, void *stream);

/* sdd table: replaces _sparse_matmul.make_sdd_lut + torch_blocksparse_cpp_utils.sdd_segment
 * (matmul.py:281-297, csrc/utils.cpp:11-120).  start_width is 64/block in the reference (matmul.py:283).
 * d_lut receives rows (head, block-row, block-col, blockid), all pack levels back to back in the order the
 * reference returns them; level k has pack packs[k] and rows[k] rows (host arrays of >= 8 entries).
 * d_valid (one byte per row) is 0 for the rows the reference emits for positions that are empty or were
 * already taken (it does so for some dense layouts at pack 4); the sdd launcher skips them.
 * cap_rows: capacity of d_lut / d_valid in rows; BSP_ERR_CAPACITY if exceeded (*total_rows = rows needed). */
int bsp_sdd_lut_build(const int32_t *d_layout, int H, int R, int C, int start_width, int32_t *d_lut,
                      uint8_t *d_valid, int64_t cap_rows, void *d_ws, int64_t ws_bytes, int *n_levels,
                      int *packs, int64_t *rows, int64_t *total_rows, int *all_valid, void *stream);

/* Group plan (no counterpart in the reference; an optional accelerator for the launchers below).
 * BSP_GROUP consecutive block-rows (by_rows != 0) or block-columns of one head form a group that one workgroup
 * processes together, sharing the dense tiles its members have in common.  d_plan receives 4 ints per group
 * (first entry, entries, head, group index; sorted by decreasing entries) followed by BSP_GROUP+1 ints per entry
 * (position along the other dimension, block id of each member or -1), positions ascending for row groups and
 * descending for column groups.  thin_min > 0: a line with at least thin_min blocks leaves its group and becomes a
 * chain of its own (group index field = -(line + 1), member 0 = the line), whose entries bsp_dsd_matmul /
 * bsp_dds_matmul spread over the wavefronts of a workgroup; bits 24..27 of a group's index field mark the members
 * that left it (needs fewer than 2^24 groups per head), bit 28 is the builder's hint that few groups want each
 * dense tile (the kernels then fetch those tiles with streaming loads).  Pass 0 for a plan given to bsp_sdd_matmul.
 * Plans over tiles (blocks of 16, for all three launchers): the plan of the layout coarsened to 64 x 64
 * tiles (a tile is present if any of its 4 x 4 blocks is), whose entries carry, after the BSP_GROUP+1 ints above (the
 * ids there number the tiles), the ids of the 16 blocks of each member's tile, row by row, -1 where absent:
 * 1 + BSP_GROUP + 16*BSP_GROUP ints per entry.  The caller assembles it from the coarse layout's plan and passes it
 * with a NEGATIVE plan_lines (minus the tile lines per head); the launchers then run the block-64 row-group kernels
 * and gather each tile from its blocks (bsp_sdd_matmul: scatter each result tile to the blocks present).
 * order_buckets > 0 sorts the header by entries in units of 1/order_buckets of the largest group instead of exactly
 * (equal keys head by head: better L2 reuse of the dense rows when one head's share of them is small); 0 = exact.
 * split_len > 0: a chain with more than split_len entries is cut into up to BSP_CHAIN_PARTS parts of equal length, one
 * header row each (next to each other, in part order): the count field holds the part's entries in bits 0..19, the
 * part's index in bits 20..25 and the number of parts minus one in bits 26..30; bits 16..30 of the head field number
 * the split chains of the plan (fewer than 2^15, and fewer than 2^16 heads).  bsp_dsd_matmul / bsp_dds_matmul give
 * every part a workgroup of its own; the parts leave fp32 partial results in the launcher's workspace and a second
 * pass adds them in part order (no atomics, no locks: the result does not depend on the order in which the parts
 * ran).  This is the role of the lock epilogue in the reference's kernel (matmul.py:191-203, 246-262).
 * Pass 0 for plans given to bsp_sdd_matmul and for blocks of 32.
 * *n_groups counts header rows (groups, chains and parts of chains), *n_split the chains that were split.
 * plan_cap >= bsp_group_plan_cap(...). */
#define BSP_GROUP 4
#define BSP_CHAIN_PARTS 8
int64_t bsp_group_plan_cap(int H, int R, int C, int64_t nnz, int by_rows);
int bsp_group_plan_build(const int32_t *d_layout, int H, int R, int C, int by_rows, int thin_min, int split_len,
                         int order_buckets, int32_t *d_plan, int64_t plan_cap, void *d_ws, int64_t ws_bytes, int *n_groups,
                         int *n_split, int64_t *plan_len, void *stream);

/* ---------------------------------------------------------------------------------------------------
 * Matmul launchers.  Strides are in elements; the innermost stride of every operand is 1 and rows start on
 * 16-byte boundaries.  trans_x means the stored matrix is read transposed, as in the reference.
 * flags: 0, or a combination of the bsp_launch_flags below.  Kernel selection is a pure function of the arguments:
 * the library reads no environment variable and keeps no state between calls.
 * ------------------------------------------------------------------------------------------------- */
typedef enum {
  BSP_FLAG_GENERAL_ONLY = 1,  /* take the general kernels even where a specialised one would serve (for cross-checks) */
  BSP_FLAG_NO_GROUPS = 2,     /* ignore the group plan (the per-block / per-segment kernels run instead) */
  BSP_FLAG_NO_WIDE = 4,       /* skip the kernels specialised for a wide free dimension (dsd / dds, blocks 64 and 128) */
  BSP_FLAG_PLAN_ROWPAIR = 8   /* bsp_sdd_matmul, block 16: d_gplan is a plan over PAIRS of block-rows (built by bsp_group_plan_build on
                                 the layout with every two block-rows merged, entries widened to 13 ints: position, 4 member ids,
                                 then the ids of the two blocks of each member, -1 where absent); plan_lines counts the pairs.  Such a
                                 plan serves the long-reduction kernel (K >= 256, K % 32 == 0, 16-bit types) and nothing else */
} bsp_launch_flags;

/* sparse = dense x dense: replaces _sparse_matmul._sdd_matmul + the SDD branch of the kernel
 * (matmul.py:299-364, 30-54).  One call per pack level of the sdd table.  For every valid table row
 * (h, i, j, p):  C[z, p] = op(A)[z, h, i*block:(i+1)*block, 0:K] . op(B)[z, h, 0:K, j*block:(j+1)*block].
 * lda / ldb: row stride of the stored 2-D matrices.  n_groups = rows / (pack*pack).
 * d_gplan / n_plan_groups / plan_lines: optional group plan of the layout built with by_rows = 1, its number of
 * groups and the number of block-rows per head (NULL / 0 / 0 if none); when given, a kernel that shares operand
 * tiles inside each group may take the launch.  The plan describes the whole layout, not one pack level: if that
 * kernel ran, the return value is BSP_OK_WHOLE_LAYOUT and the caller skips the remaining pack levels (pass the plan
 * with the first level only).  A caller that has the plan but has not built the table yet (its greedy packing is the
 * one sequential step of the builders) may call with d_lut = NULL, pack = 0 and n_groups = an upper bound on the number of
 * entries of any group of the plan: the number of block-columns of the layout always is one, the largest entry count
 * among the plan's header rows is the tightest (it sizes the grid of the kernels for long reductions at blocks of 16
 * and 32; 0 if unknown: those kernels then do not apply): the result is
 * BSP_OK_WHOLE_LAYOUT if a kernel that works from the plan alone took the product, else BSP_NEEDS_TABLE and nothing was
 * launched. */
int bsp_sdd_matmul(int dtype, const void *a, const void *b, void *c, int trans_a, int trans_b, int Z, int K,
                   int64_t a_stride_z, int64_t a_stride_h, int64_t lda, int64_t b_stride_z, int64_t b_stride_h,
                   int64_t ldb, int64_t c_stride_z, int block, int pack, const int32_t *d_lut,
                   const uint8_t *d_valid, int64_t n_groups, const int32_t *d_gplan, int n_plan_groups, int plan_lines, int flags,
                   void *stream);

/* sparse = dense x dense over a long reduction into few blocks of 128, the reduction cut into `parts` parts that run side by
 * side: replaces _sparse_matmul._sdd_matmul (matmul.py:299-364) where the reference would have used the split-K lock path of
 * its kernel (matmul.py:186-203; dead there, no locks or atomics here).  Blocks of 128 and 16-bit types only, K a multiple
 * of 32; d_lut / d_valid / n_groups: the pack-1 level of bsp_sdd_lut_build.  Each part leaves an fp32 partial block in d_ws
 * (bsp_sdd_splitk_workspace_bytes(Z, n_groups, parts) bytes, 16-byte aligned, no initialisation needed; unused when parts == 1)
 * and a second small kernel adds the parts of a block in part order: repeated launches agree bit for bit.
 * BSP_ERR_UNSUPPORTED for any other block size or dtype (the caller takes bsp_sdd_matmul). */
int64_t bsp_sdd_splitk_workspace_bytes(int Z, int64_t n_groups, int parts);
int bsp_sdd_matmul_splitk(int dtype, const void *a, const void *b, void *c, int trans_a, int trans_b, int Z, int K,
                          int64_t a_stride_z, int64_t a_stride_h, int64_t lda, int64_t b_stride_z, int64_t b_stride_h,
                          int64_t ldb, int64_t c_stride_z, int block, const int32_t *d_lut, const uint8_t *d_valid,
                          int64_t n_groups, int parts, void *d_ws, int64_t ws_bytes, int flags, void *stream);

/* dense = sparse x dense: replaces _sparse_matmul._dsd_matmul + the DSD branch (matmul.py:507-552, 56-82).
 * C[z, h] = op(A_sparse)[h] . op(B)[z, h], written transposed when trans_c.  N = free dimension of op(B).
 * a_stride_z = 0 shares one sparse operand over the batch.  d_lut / d_plan / width from bsp_dxx_lut_build
 * with trans = !trans_a; d_gplan (optional) from bsp_group_plan_build with by_rows = !trans_a; plan_lines < 0: a
 * plan over tiles (see bsp_group_plan_build).
 * n_split / d_ws / ws_bytes: a plan with split chains (n_split of them, as bsp_group_plan_build reported) needs
 * scratch memory of at least bsp_xsd_workspace_bytes(n_split, N, Z) bytes, 256-byte aligned: BSP_CHAIN_PARTS fp32
 * tiles of 64 x 64 per (split chain, 64-wide tile of the free dimension, batch).  Its contents need no
 * initialisation and mean nothing after the call; a second small kernel launched behind the product adds the parts
 * up.  Launches that share a buffer must not overlap (one stream, or one buffer per stream).
 * 0 / NULL / 0 for plans without split chains. */
int64_t bsp_xsd_workspace_bytes(int n_split, int free_dim, int Z);
int bsp_dsd_matmul(int dtype, const void *a, const void *b, void *c, int trans_a, int trans_b, int trans_c, int Z,
                   int N, int64_t a_stride_z, int64_t b_stride_z, int64_t b_stride_h, int64_t ldb,
                   int64_t c_stride_z, int64_t c_stride_h, int64_t ldc, int block, const int32_t *d_lut,
                   const int32_t *d_plan, int width, const int32_t *d_gplan, int n_plan_groups, int plan_lines,
                   int n_split, void *d_ws, int64_t ws_bytes, int flags, void *stream);

/* bsp_dsd_matmul for callers that cannot allocate.  No counterpart in the reference: it is for code under HIP graph
 * capture, tight serving loops and harnesses that forbid hipMalloc, which have nowhere to take the workspace of a plan
 * with split chains from.  Same arguments and results as bsp_dsd_matmul without d_ws / ws_bytes: the fp32 partial
 * tiles live in a buffer inside the library (static device memory, BSP_NOALLOC_SCRATCH_BYTES per GPU the library
 * runs on, held until the process ends).  It serves launches with at most BSP_NOALLOC_MAX_SLOTS =
 * n_split * ceil(N / 64) * Z (split chain, tile, batch) combinations and returns BSP_ERR_SCRATCH_LIMIT beyond that,
 * before anything is launched.  The call allocates and frees nothing (the first call on a device looks the buffer's address up
 * once; make that call outside a capture).  Every call on a GPU uses that GPU's one buffer: calls that overlap on one
 * GPU (two streams, two threads) race; calls ordered on one stream do not.  Nothing in the buffer has to start at
 * zero: every tile a call reads it has written before. */
#define BSP_NOALLOC_MAX_SLOTS 64
#define BSP_NOALLOC_SCRATCH_BYTES (BSP_NOALLOC_MAX_SLOTS * BSP_CHAIN_PARTS * 64 * 64 * 4)
int bsp_dsd_matmul_noalloc(int dtype, const void *a, const void *b, void *c, int trans_a, int trans_b, int trans_c, int Z,
                           int N, int64_t a_stride_z, int64_t b_stride_z, int64_t b_stride_h, int64_t ldb,
                           int64_t c_stride_z, int64_t c_stride_h, int64_t ldc, int block, const int32_t *d_lut,
                           const int32_t *d_plan, int width, const int32_t *d_gplan, int n_plan_groups, int plan_lines,
                           int n_split, int flags, void *stream);

/* dense = dense x sparse: replaces _sparse_matmul._dds_matmul + the DDS branch (matmul.py:460-505, 83-99).
 * C[z, h] = op(A)[z, h] . op(B_sparse)[h], written transposed when trans_c.  M = free dimension of op(A).
 * Tables from bsp_dxx_lut_build with trans = trans_b; d_gplan (optional) with by_rows = trans_b; workspace as for
 * bsp_dsd_matmul, with M as the free dimension. */
int bsp_dds_matmul(int dtype, const void *a, const void *b, void *c, int trans_a, int trans_b, int trans_c, int Z,
                   int M, int64_t a_stride_z, int64_t a_stride_h, int64_t lda, int64_t b_stride_z,
                   int64_t c_stride_z, int64_t c_stride_h, int64_t ldc, int block, const int32_t *d_lut,
                   const int32_t *d_plan, int width, const int32_t *d_gplan, int n_plan_groups, int plan_lines,
                   int n_split, void *d_ws, int64_t ws_bytes, int flags, void *stream);

/* ---------------------------------------------------------------------------------------------------
 * Softmax launchers: replace softmax_fwd / softmax_bwd and their dispatch (softmax.py:7-138, 144-194,
 * 253-326).  x is [Z, nnz, block, block], updated in place.  Optional operands are NULL when absent.
 *   rpe  : element (z, h, r, c) at rpe[z*rpe_stride_z + h*rpe_stride_h + r*rpe_stride_r + c]
 *   kpm  : key padding mask, element (z, c) at kpm[z*kpm_stride_z + c]
 *   attn : attention mask, element (r, c) at attn[r*attn_stride_r + c]
 * *_mul != 0 selects the reference's 'mul' mode (mask value 0 -> -inf, anything else -> 0).
 * y = softmax(x*scale + rpe + kpm + attn) over each row's nonzero blocks, computed in fp32. */
int bsp_softmax_fwd(int dtype, void *x, float scale, const int32_t *d_lut, int maxlut, const void *rpe,
                    int64_t rpe_stride_z, int64_t rpe_stride_h, int64_t rpe_stride_r, const void *kpm,
                    int64_t kpm_stride_z, int kpm_mul, const void *attn, int64_t attn_stride_r, int attn_mul,
                    int Z, int H, int R, int block, int64_t x_stride_z, void *stream);

/* dx = y * (dy - sum(y*dy)) * scale per row, written over dy (softmax.py:183-193). */
int bsp_softmax_bwd(int dtype, const void *y, void *dy, float scale, const int32_t *d_lut, int maxlut, int Z, int H,
                    int R, int block, int64_t y_stride_z, int64_t dy_stride_z, void *stream);

/* Softmax with dropout on its result.  No counterpart in the reference, whose attention module refuses dropout
 * (attention.py:223-224); this is what nn.MultiheadAttention's dropout on the attention weights needs.
 * Forward: x receives softmax(...) as bsp_softmax_fwd would leave it (the backward pass needs it), y_drop (same shape,
 * own batch stride) receives softmax(...) * mask / (1 - p).  The mask is not stored: element i (its linear offset in
 * x: z * x_stride_z + blockid * block^2 + row * block + col) is kept iff (w >> 8) * 2^-24 >= p, where w is word
 * i % 4 of Philox4x32-10 with counter (i / 4 as two 32-bit words, offset as two 32-bit words) and key seed.
 * Backward: dy holds the gradient of y_drop and is overwritten with the gradient of the softmax input,
 * y * (dy * mask / (1 - p) - sum(...)) * scale, the mask re-created from the same (seed, offset); y is x as the forward
 * call left it and y_stride_z the x_stride_z of that call.  0 <= p < 1. */
int bsp_softmax_dropout_fwd(int dtype, void *x, void *y_drop, float scale, const int32_t *d_lut, int maxlut, const void *rpe,
                            int64_t rpe_stride_z, int64_t rpe_stride_h, int64_t rpe_stride_r, const void *kpm,
                            int64_t kpm_stride_z, int kpm_mul, const void *attn, int64_t attn_stride_r, int attn_mul, int Z,
                            int H, int R, int block, int64_t x_stride_z, int64_t y_drop_stride_z, float drop_p, uint64_t seed,
                            uint64_t offset, void *stream);
int bsp_softmax_dropout_bwd(int dtype, const void *y, void *dy, float scale, const int32_t *d_lut, int maxlut, int Z, int H,
                            int R, int block, int64_t y_stride_z, int64_t dy_stride_z, float drop_p, uint64_t seed,
                            uint64_t offset, void *stream);

/* ---------------------------------------------------------------------------------------------------
 * The attention chain of the reference's modules in one launch per direction: replaces the sequence
 * sparse_dot_sdd_nt -> sparse_softmax -> sparse_dot_dsd_nn of DeepSpeedSparseSelfAttention.forward
 * (deepspeedsparseselfattention.py:152-157) and of multi_head_attention_forward (attention.py:190-202), and the
 * matching part of their autograd graph (matmul.py:587-606, softmax.py:315-326).  fp16 / bf16, head dimension
 * D = 64 or 128, blocks of 64, 32 or 16; BSP_ERR_UNSUPPORTED / BSP_ERR_ROW_TOO_LONG otherwise, and the caller runs
 * the three operators.  Rows of at most BSP_ATTENTION_MAX_ROW_BLOCKS tiles of 64 x 64 are held in registers; longer
 * rows (up to the softmax operator's 32768 elements) are streamed: forward in two sweeps over the row (running maximum
 * and sum first, then p and p . v), backward with dq accumulated block by block.
 *   block 64: d_lut / maxlut from bsp_softmax_lut_build on the layout, R = its block-rows.
 *   blocks 16 and 32 (S = 64 / block, layout sides divisible by S): the kernels work on 64 x 64 tiles that the caller
 *             forms: a line of tiles is S consecutive block-rows, and a tile takes S block-columns gathered from
 *             anywhere in the line (in practice: the columns in which any of the line's block-rows holds a block,
 *             ascending, S per tile, so that single block-columns do not cost whole tiles).  R = lines.  d_lut: per
 *             (head, line) two ints (tiles, offset of the first entry in ints from the start), then per tile
 *             8 + S * S ints (., ., ., ., its S block-columns, the last repeated up to four; then the ids of its blocks
 *             in the [Z, nnz, block, block] tensor, [block-row of the line][gathered block-column], -1 where the layout
 *             has none; unused column slots repeat a valid column and hold no block).  maxlut = the most tiles of a
 *             line.
 *   forward : p = softmax(round(q . k^T) * scale + rpe + kpm + attn) over each row's nonzero blocks, o = p . v.
 *             q, o: [Z, H, rows, D]; k, v: [Z, H, columns, D], unit stride along D; p: [Z, nnz, block, block] (every
 *             block is written), or NULL when no backward pass will follow: p is then not stored (most of the
 *             kernel's traffic); rows of o without any block are set to zero.  Masks as for bsp_softmax_fwd.
 *   backward: ds = p * (round(do . v^T) - delta) * scale, dq = ds . k, with delta = sum_d do[row][d] * o[row][d], o
 *             the result of the forward call: in exact arithmetic this is the sum over the row of p * (do . v^T) that
 *             the softmax gradient subtracts (softmax.py:187-189), and it is known before the row's blocks are, so
 *             each block is finished as soon as its product is.  ds: [Z, nnz, block, block], a tensor of its own, or
 *             NULL (not stored); delta: NULL, or [Z][H][delta_stride_h >= 64 R] fp32 that receives delta of every row
 *             that has a block.
 *             The two remaining gradients are ordinary products of the caller: dk = ds^T . q and dv = p^T . do
 *             (bsp_dsd_matmul with trans_a).
 * round() is the rounding to the storage type that the scores undergo when the sdd operator stores them, kept so
 * that the result matches the three-operator chain.  Every pointer 16-byte aligned, every stride a multiple of 8
 * elements. */
#define BSP_ATTENTION_MAX_ROW_BLOCKS 8
int bsp_attention_fwd(int dtype, const void *q, const void *k, const void *v, void *p, void *o, int Z, int H, int R,
                      int D, int64_t q_stride_z, int64_t q_stride_h, int64_t ldq, int64_t k_stride_z, int64_t k_stride_h,
                      int64_t ldk, int64_t v_stride_z, int64_t v_stride_h, int64_t ldv, int64_t o_stride_z,
                      int64_t o_stride_h, int64_t ldo, int64_t p_stride_z, int block, float scale, const int32_t *d_lut,
                      int maxlut, const void *rpe, int64_t rpe_stride_z, int64_t rpe_stride_h,
                      int64_t rpe_stride_r, const void *kpm, int64_t kpm_stride_z, int kpm_mul, const void *attn,
                      int64_t attn_stride_r, int attn_mul, void *stream);
int bsp_attention_bwd(int dtype, const void *d_o, const void *v, const void *k, const void *p, const void *o, void *ds,
                      void *dq, int Z, int H, int R, int D, int64_t do_stride_z, int64_t do_stride_h, int64_t lddo,
                      int64_t v_stride_z, int64_t v_stride_h, int64_t ldv, int64_t k_stride_z, int64_t k_stride_h,
                      int64_t ldk, int64_t o_stride_z, int64_t o_stride_h, int64_t ldo, int64_t dq_stride_z,
                      int64_t dq_stride_h, int64_t lddq, int64_t p_stride_z, int64_t ds_stride_z, int block, float scale,
                      const int32_t *d_lut, int maxlut, float *delta, int64_t delta_stride_h,
                      void *stream);
/* dk and dv of the same chain in one launch, one workgroup per column of 64 x 64 tiles: dv = p^T . do and
 * dk = ds^T . q with ds computed again from p (the formula above), delta = the row sums that bsp_attention_bwd wrote
 * ([Z][H][delta_stride_h], fp32).  Call bsp_attention_bwd with ds = NULL and delta given first: the sparse gradient
 * is then neither written nor read.  Replaces the two transposed dsd products of the operators' backward pass
 * (matmul.py:598-601).  d_col_lut: the layout read along columns: n_items work items of twelve ints (number of entries,
 * offset of the first entry in ints from the start, head, column, slot, 0, 0, 0, then the column's S block-columns,
 * the last repeated up to four), then the entries, a column's by row.  Block 64: a column is a block-column, an entry
 * four ints (id, row, column, head).  Blocks 16 / 32: a column is any S block-columns of a head (every block-column
 * in exactly one; the kernel takes the wavefronts' keys from them), an entry a tile of 8 + S * S ints (., ., ., ., the S
 * block-rows gathered into it, then the ids of its blocks, [gathered block-row][block-column of the column], -1 where
 * the layout has none).  A work item is a
 * whole column (slot -1; also every column without blocks, whose rows of dk and dv are set to zero) or one part of a
 * long column: columns differ in length far more than rows do, so the caller cuts the long ones into parts, whose
 * partial sums go to fp32 slots (partial: [Z][n_slots][2][64][D] floats, slot = the item's) and are added in order by a
 * second kernel of the same call, per d_split_lut: n_split entries of eight ints (head, column, first slot, parts, then
 * the column's block-columns as in the work items; a column's slots are consecutive).  No atomics.  C = columns of
 * tiles; dk, dv: [Z, H, keys, D]. */
int bsp_attention_bwd_kv(int dtype, const void *d_o, const void *q, const void *v, const void *p, const float *delta, void *dk,
                         void *dv, int Z, int H, int C, int D, int64_t do_stride_z, int64_t do_stride_h, int64_t lddo,
                         int64_t q_stride_z, int64_t q_stride_h, int64_t ldq, int64_t v_stride_z, int64_t v_stride_h,
                         int64_t ldv, int64_t dk_stride_z, int64_t dk_stride_h, int64_t lddk, int64_t dv_stride_z,
                         int64_t dv_stride_h, int64_t lddv, int64_t p_stride_z, int64_t delta_stride_h, int block,
                         float scale, const int32_t *d_col_lut, int n_items, float *partial, int n_slots,
                         const int32_t *d_split_lut, int n_split, void *stream);

/* ---------------------------------------------------------------------------------------------------
 * Dense utility ops of the reference package.
 * ReLU: replaces the relu_y / relu_dxdsdbdres kernels and their launches (relu.py:8-91).  All tensors hold n
 * elements in the same memory order; scale and bias are one-element device tensors of the data type (the
 * reference reads them on the host with .item(); here nothing synchronises).
 *   forward : y = max(x*scale + bias + res, 0)
 *   backward: du = (y > 0) ? dy : 0; dx = du*scale; dres = du; *d_dbias = sum(du); *d_dscale = sum(du*x), both in
 *             fp32, added in a fixed order (the reference uses floating-point atomics); d_ws is scratch of at
 *             least bsp_relu_workspace_bytes() bytes. */
int64_t bsp_relu_workspace_bytes(void);
int bsp_relu_fwd(int dtype, const void *x, const void *res, void *y, const void *d_scale, const void *d_bias, int64_t n,
                 void *stream);
int bsp_relu_bwd(int dtype, const void *x, const void *y, const void *dy, void *dx, void *dres, const void *d_scale,
                 float *d_dscale, float *d_dbias, void *d_ws, int64_t ws_bytes, int64_t n, void *stream);

/* Permutation: replaces the permute kernel of permute.py:5-30, 45-93.  NCHW -> CHWN is the transposition of an
 * [N, C*H*W] matrix, CHWN -> NCHW that of a [C*H*W, N] matrix: y[c*rows + r] = x[r*cols + c]. */
int bsp_transpose(int dtype, const void *x, void *y, int64_t rows, int64_t cols, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* BSP_H */
