// Device-side construction of the block-sparsity layouts ([heads, blocks, blocks] int32, 0/1): the layout never has to
// exist on the host, and the table builders of lut.hip read it where it is written.
//
// Replaces the reference's host generators: the C++ helper make_layout (csrc/utils.cpp:123-148) and the Python
// DeepSpeedSparseSelfAttention._make_layout (deepspeedsparseselfattention.py:31-65), which differ only in how much of
// a vertical stripe wider than one block they mark.  One thread per (head, row, column) evaluates the definition in
// closed form instead of replaying the generators' loops.
#include "bsp_common.h"

namespace bsp {
namespace {

// "fixed" (Sparse-Transformer) pattern: dense local windows of `stride` blocks on the diagonal, plus vertical stripes
// of `vertsize` blocks; head h places its stripes `(1 + h % numverts) * vertsize` blocks before the end of every
// window.  whole_stripes != 0: every column of a stripe is marked (the Python generator); 0: only the first column
// (the C++ helper steps through a stripe by num_blocks, utils.cpp:143).  Unidirectional: a window keeps its lower
// triangle, a stripe starting at column j is seen by the rows after j (utils.cpp:141-142; _set_s2_layout).
__global__ void k_layout_fixed(int32_t *lay, int H, int NB, int stride, int uni, int numverts, int vertsize, int whole_stripes) {
  const int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (idx >= (int64_t)H * NB * NB) return;
  const int j = (int)(idx % NB), i = (int)(idx / NB % NB), h = (int)(idx / ((int64_t)NB * NB));
  bool on = (i / stride == j / stride) && (!uni || j <= i);
  const int start = stride - (1 + h % numverts) * vertsize;
  // the stripe that column j belongs to starts at the largest s = start + t * stride <= j (t >= 0)
  if (j >= start) {
    const int s = start + (j - start) / stride * stride;
    const bool in_stripe = whole_stripes ? (j - s < vertsize) : (j == s);
    if (in_stripe && s >= 0 && (!uni || i > s)) on = true;
  }
  lay[idx] = on ? 1 : 0;
}

// dense local windows of `local` blocks + the last column of every `global_stride` blocks as a global column (seen by
// the rows below it when causal, by every row otherwise)
__global__ void k_layout_sparse_transformer(int32_t *lay, int H, int NB, int local, int global_stride, int causal) {
  const int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (idx >= (int64_t)H * NB * NB) return;
  const int j = (int)(idx % NB), i = (int)(idx / NB % NB);
  bool on = (i / local == j / local) && (!causal || j <= i);
  if (j % global_stride == global_stride - 1 && (!causal || i > j)) on = true;
  lay[idx] = on ? 1 : 0;
}

// sliding window + global columns (and rows, unless causal) at the start + the random columns picked for every row
// (d_random: [H, NB, num_random] column indices, drawn by the caller), intersected with the causal mask if asked
__global__ void k_layout_bigbird(int32_t *lay, int H, int NB, int window, int num_global, int causal, const int32_t *random_cols,
                                 int num_random) {
  const int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (idx >= (int64_t)H * NB * NB) return;
  const int j = (int)(idx % NB), i = (int)(idx / NB % NB), h = (int)(idx / ((int64_t)NB * NB));
  const int d = i - j;
  bool on = causal ? (d >= 0 && d < window) : ((d < 0 ? -d : d) <= window / 2);
  if (j < num_global || (!causal && i < num_global)) on = true;
  const int32_t *pick = random_cols + ((int64_t)h * NB + i) * num_random;
  for (int r = 0; r < num_random; r++)
    if (pick[r] == j) on = true;
  if (causal && j > i) on = false;
  lay[idx] = on ? 1 : 0;
}

__global__ void k_layout_ones(int32_t *lay, int64_t n) {
  const int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (idx < n) lay[idx] = 1;
}

int grid_for(int64_t n, dim3 *grid) {
  if (n <= 0 || n >= ((int64_t)1 << 31)) return BSP_ERR_UNSUPPORTED;
  *grid = dim3((unsigned)((n + 255) / 256));
  return BSP_OK;
}

}  // namespace
}  // namespace bsp

using namespace bsp;

extern "C" int bsp_layout_fixed(int32_t *d_layout, int H, int NB, int dense, int block_stride, int unidirectional, int numverts,
                                int vertsize, int whole_stripes, void *stream) {
  if (!d_layout || H <= 0 || NB <= 0) return BSP_ERR_ARG;
  dim3 grid;
  if (int rc = grid_for((int64_t)H * NB * NB, &grid)) return rc;
  if (dense) {
    hipLaunchKernelGGL(k_layout_ones, grid, dim3(256), 0, as_stream(stream), d_layout, (int64_t)H * NB * NB);
  } else {
    if (block_stride <= 0 || NB % block_stride || numverts <= 0 || vertsize <= 0) return BSP_ERR_ARG;
    hipLaunchKernelGGL(k_layout_fixed, grid, dim3(256), 0, as_stream(stream), d_layout, H, NB, block_stride, unidirectional, numverts,
                       vertsize, whole_stripes);
  }
  BSP_LAUNCH_CHECK();
  return BSP_OK;
}

extern "C" int bsp_layout_sparse_transformer(int32_t *d_layout, int H, int NB, int local_blocks, int global_stride, int causal,
                                             void *stream) {
  if (!d_layout || H <= 0 || NB <= 0 || local_blocks <= 0 || global_stride <= 0) return BSP_ERR_ARG;
  dim3 grid;
  if (int rc = grid_for((int64_t)H * NB * NB, &grid)) return rc;
  hipLaunchKernelGGL(k_layout_sparse_transformer, grid, dim3(256), 0, as_stream(stream), d_layout, H, NB, local_blocks, global_stride, causal);
  BSP_LAUNCH_CHECK();
  return BSP_OK;
}

extern "C" int bsp_layout_bigbird(int32_t *d_layout, int H, int NB, int window, int num_global, int causal,
                                  const int32_t *d_random_cols, int num_random, void *stream) {
  if (!d_layout || H <= 0 || NB <= 0 || window < 0 || num_global < 0 || num_random < 0 || (num_random > 0 && !d_random_cols)) return BSP_ERR_ARG;
  dim3 grid;
  if (int rc = grid_for((int64_t)H * NB * NB, &grid)) return rc;
  hipLaunchKernelGGL(k_layout_bigbird, grid, dim3(256), 0, as_stream(stream), d_layout, H, NB, window, num_global, causal, d_random_cols,
                     num_random);
  BSP_LAUNCH_CHECK();
  return BSP_OK;
}
