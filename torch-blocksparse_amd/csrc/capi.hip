// C-ABI entry points of the matmul launchers: argument validation and dispatch.  (The table builders and
// the softmax entry points live next to their kernels in lut.hip / softmax.hip.)
#include "matmul_generic.h"
#include <mutex>

using namespace bsp;

namespace {
bool no_groups(int flags) { return (flags & BSP_FLAG_NO_GROUPS) != 0; }
bool general_only(int flags) { return (flags & BSP_FLAG_GENERAL_ONLY) != 0; }
bool no_wide(int flags) { return (flags & (BSP_FLAG_NO_WIDE | BSP_FLAG_GENERAL_ONLY)) != 0; }
bool rowpair(int flags) { return (flags & BSP_FLAG_PLAN_ROWPAIR) != 0; }
bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
bool block_ok(int block) { return block == 16 || block == 32 || block == 64 || block == 128; }
int elems16(int dtype) { return dtype == BSP_F32 ? 4 : 8; }   // elements per 16 bytes
}  // namespace

extern "C" int bsp_version(void) { return 1; }

extern "C" const char *bsp_strerror(int status) {
  switch (status) {
    case BSP_OK: return "ok";
    case BSP_OK_WHOLE_LAYOUT: return "ok, every block of the layout written (skip the remaining pack levels)";
    case BSP_NEEDS_TABLE: return "nothing launched: this product needs the sdd table (call again with it)";
    case BSP_ERR_ARG: return "invalid argument (null pointer, bad size or operand not 16-byte aligned)";
    case BSP_ERR_UNSUPPORTED: return "unsupported block size, dtype or problem size";
    case BSP_ERR_CAPACITY: return "caller-provided table or workspace too small";
    case BSP_ERR_EMPTY_HEAD: return "a head of the layout has no nonzero block";
    case BSP_ERR_HIP: return "HIP runtime error";
    case BSP_ERR_ROW_TOO_LONG: return "Reductions larger than 32768 elements are not yet implemented";
    case BSP_ERR_K_MULTIPLE: return "Reduction size for SDD must be a multiple of 16";
    case BSP_ERR_SCRATCH_LIMIT: return "the launch needs more (split chain, tile, batch) slots than the library's static scratch buffer holds; use bsp_dsd_matmul with a workspace";
    default: return "unknown status";
  }
}

extern "C" int bsp_sdd_matmul(int dtype, const void *a, const void *b, void *c, int trans_a, int trans_b, int Z, int K,
                              int64_t a_stride_z, int64_t a_stride_h, int64_t lda, int64_t b_stride_z, int64_t b_stride_h,
                              int64_t ldb, int64_t c_stride_z, int block, int pack, const int32_t *d_lut,
                              const uint8_t *d_valid, int64_t n_groups, const int32_t *d_gplan, int n_plan_groups,
                              int plan_lines, int flags, void *stream) {
  if (!a || !b || !c || Z <= 0 || K <= 0 || n_groups < 0) return BSP_ERR_ARG;
  if (!d_lut && (!d_gplan || no_groups(flags) || general_only(flags))) return d_gplan ? BSP_NEEDS_TABLE : BSP_ERR_ARG;
  if (!block_ok(block)) return BSP_ERR_UNSUPPORTED;
  if (K % 16) return BSP_ERR_K_MULTIPLE;   // reference matmul.py:318-319
  const int u = elems16(dtype);
  if (!aligned16(a) || !aligned16(b) || !aligned16(c)) return BSP_ERR_ARG;
  if (a_stride_z % u || a_stride_h % u || lda % u || b_stride_z % u || b_stride_h % u || ldb % u || c_stride_z % u) return BSP_ERR_ARG;
  SddArgs g;
  g.a = a; g.b = b; g.c = c; g.Z = Z; g.K = K;
  g.a_sz = a_stride_z; g.a_sh = a_stride_h; g.lda = lda;
  g.b_sz = b_stride_z; g.b_sh = b_stride_h; g.ldb = ldb; g.c_sz = c_stride_z;
  g.lut = d_lut; g.valid = d_valid; g.n_groups = n_groups;
  g.gplan = no_groups(flags) ? nullptr : d_gplan; g.n_pgroups = n_plan_groups; g.lines = plan_lines;
  if (g.gplan && (n_plan_groups <= 0 || plan_lines == 0)) return BSP_ERR_ARG;
  // op(A)[m][k]: reduction contiguous unless A is read transposed; op(B)[k][n]: contiguous when B is read transposed
  const bool a_kc = !trans_a, b_kc = trans_b != 0;
  hipStream_t st = as_stream(stream);
  int rc = 0;
  if (!d_lut) {   // the plan alone: n_groups then carries an upper bound on the entries of a group (at most the block-columns of the layout)
    g.cols = (int)n_groups; g.n_groups = 0;
    rc = no_wide(flags) ? 0 : sdd_dl(dtype, g, block, rowpair(flags), a_kc, b_kc, st);
    if (rc < 0) return rc;
    if (rc == 2) { BSP_LAUNCH_CHECK(); return BSP_OK_WHOLE_LAYOUT; }
  }
  if (rowpair(flags)) {   // a plan over pairs of block-rows serves the long-reduction kernel only
    if (!d_lut) return BSP_NEEDS_TABLE;
    g.gplan = nullptr;
  }
  rc = general_only(flags) ? 0 : sdd_fast64(dtype, g, block, pack, a_kc, b_kc, st);
  if (rc < 0) return rc;
  if (rc >= 1) { BSP_LAUNCH_CHECK(); return rc == 2 ? BSP_OK_WHOLE_LAYOUT : BSP_OK; }
  if (!d_lut) return BSP_NEEDS_TABLE;      // a call with the plan alone, and no kernel that works from the plan applies
  switch (dtype) {
    case BSP_F16: rc = sdd_generic_f16(g, block, pack, a_kc, b_kc, st); break;
    case BSP_BF16: rc = sdd_generic_bf16(g, block, pack, a_kc, b_kc, st); break;
    case BSP_F32: rc = sdd_generic_f32(g, block, pack, a_kc, b_kc, st); break;
    default: return BSP_ERR_UNSUPPORTED;
  }
  if (rc != BSP_OK) return rc;
  BSP_LAUNCH_CHECK();
  return BSP_OK;
}

extern "C" int64_t bsp_sdd_splitk_workspace_bytes(int Z, int64_t n_groups, int parts) {
  if (Z <= 0 || n_groups <= 0 || parts <= 1) return 0;
  return (int64_t)Z * n_groups * parts * (int64_t)(128 * 128 * sizeof(float));
}

extern "C" int bsp_sdd_matmul_splitk(int dtype, const void *a, const void *b, void *c, int trans_a, int trans_b, int Z, int K,
                                     int64_t a_stride_z, int64_t a_stride_h, int64_t lda, int64_t b_stride_z, int64_t b_stride_h,
                                     int64_t ldb, int64_t c_stride_z, int block, const int32_t *d_lut, const uint8_t *d_valid,
                                     int64_t n_groups, int parts, void *d_ws, int64_t ws_bytes, int flags, void *stream) {
  if (!a || !b || !c || !d_lut || Z <= 0 || K <= 0 || n_groups < 0 || parts < 1 || parts > 64) return BSP_ERR_ARG;
  if (block != 128 || (dtype != BSP_F16 && dtype != BSP_BF16) || general_only(flags) || no_wide(flags)) return BSP_ERR_UNSUPPORTED;
  if (K % 16) return BSP_ERR_K_MULTIPLE;
  if (K % 32) return BSP_ERR_UNSUPPORTED;
  if (!aligned16(a) || !aligned16(b) || !aligned16(c)) return BSP_ERR_ARG;
  if (a_stride_z % 8 || a_stride_h % 8 || lda % 8 || b_stride_z % 8 || b_stride_h % 8 || ldb % 8 || c_stride_z % 8) return BSP_ERR_ARG;
  if (parts > 1) {
    if (!d_ws || !aligned16(d_ws)) return BSP_ERR_ARG;
    if (ws_bytes < bsp_sdd_splitk_workspace_bytes(Z, n_groups, parts)) return BSP_ERR_CAPACITY;
  }
  SddArgs g;
  g.a = a; g.b = b; g.c = c; g.Z = Z; g.K = K;
  g.a_sz = a_stride_z; g.a_sh = a_stride_h; g.lda = lda;
  g.b_sz = b_stride_z; g.b_sh = b_stride_h; g.ldb = ldb; g.c_sz = c_stride_z;
  g.lut = d_lut; g.valid = d_valid; g.n_groups = n_groups;
  g.gplan = nullptr; g.n_pgroups = 0; g.lines = 0;
  const int rc = sdd128_splitk(dtype, g, parts, reinterpret_cast<float *>(d_ws), !trans_a, trans_b != 0, as_stream(stream));
  if (rc != BSP_OK) return rc;
  BSP_LAUNCH_CHECK();
  return BSP_OK;
}

// Workspace of a plan with split chains: BSP_CHAIN_PARTS fp32 tiles of 64 x 64 per (split chain, free tile, batch).
static int64_t xsd_ws_slots(int n_split, int free_dim, int Z) { return (int64_t)n_split * ((free_dim + 63) / 64) * Z; }

extern "C" int64_t bsp_xsd_workspace_bytes(int n_split, int free_dim, int Z) {
  if (n_split <= 0 || free_dim <= 0 || Z <= 0) return 0;
  return xsd_ws_slots(n_split, free_dim, Z) * BSP_CHAIN_PARTS * (int64_t)(64 * 64 * sizeof(float));
}

// Fills in the workspace fields of the arguments.
static int xsd_workspace(XsdArgs &g, int n_split, int free_dim, void *d_ws, int64_t ws_bytes) {
  g.n_split = 0; g.partials = nullptr;
  if (n_split < 0) return BSP_ERR_ARG;
  if (!g.gplan || n_split == 0) return BSP_OK;
  if (!d_ws || (reinterpret_cast<uintptr_t>(d_ws) & 255)) return BSP_ERR_ARG;
  if (ws_bytes < bsp_xsd_workspace_bytes(n_split, free_dim, g.Z)) return BSP_ERR_CAPACITY;
  g.n_split = n_split;
  g.partials = reinterpret_cast<float *>(d_ws);
  return BSP_OK;
}

static int xsd_dispatch(int dtype, const XsdArgs &g, int block, bool sp_trans, bool dn_kc, bool out_nc, int flags, void *stream) {
  hipStream_t st = as_stream(stream);
  // a wide free dimension at blocks 64 / 128: the kernels bound by the matrix cores and the feed from L2
  int rc = no_wide(flags) ? 0 : xsd_dl(dtype, g, block, sp_trans, dn_kc, out_nc, st);
  if (rc < 0) return rc;
  if (rc == 1) { BSP_LAUNCH_CHECK(); return BSP_OK; }
  rc = general_only(flags) ? 0 : xsd_fast64(dtype, g, block, sp_trans, dn_kc, out_nc, st);
  if (rc < 0) return rc;
  if (rc == 1) { BSP_LAUNCH_CHECK(); return BSP_OK; }
  switch (dtype) {
    case BSP_F16: rc = xsd_generic_f16(g, block, sp_trans, dn_kc, out_nc, st); break;
    case BSP_BF16: rc = xsd_generic_bf16(g, block, sp_trans, dn_kc, out_nc, st); break;
    case BSP_F32: rc = xsd_generic_f32(g, block, sp_trans, dn_kc, out_nc, st); break;
    default: return BSP_ERR_UNSUPPORTED;
  }
  if (rc != BSP_OK) return rc;
  BSP_LAUNCH_CHECK();
  return BSP_OK;
}

extern "C" int bsp_dsd_matmul(int dtype, const void *a, const void *b, void *c, int trans_a, int trans_b, int trans_c, int Z,
                              int N, int64_t a_stride_z, int64_t b_stride_z, int64_t b_stride_h, int64_t ldb,
                              int64_t c_stride_z, int64_t c_stride_h, int64_t ldc, int block, const int32_t *d_lut,
                              const int32_t *d_plan, int width, const int32_t *d_gplan, int n_plan_groups, int plan_lines,
                              int n_split, void *d_ws, int64_t ws_bytes, int flags, void *stream) {
  if (!a || !b || !c || !d_lut || !d_plan || Z <= 0 || N <= 0 || width < 0) return BSP_ERR_ARG;
  if (d_gplan && (n_plan_groups <= 0 || plan_lines == 0)) return BSP_ERR_ARG;
  if (!block_ok(block)) return BSP_ERR_UNSUPPORTED;
  const int u = elems16(dtype);
  if (!aligned16(a) || !aligned16(b) || !aligned16(c)) return BSP_ERR_ARG;
  if (N % u || a_stride_z % u || b_stride_z % u || b_stride_h % u || ldb % u || c_stride_z % u || c_stride_h % u || ldc % u) return BSP_ERR_ARG;
  XsdArgs g;
  g.sp = a; g.dn = b; g.out = c; g.Z = Z; g.NF = N;
  g.sp_sz = a_stride_z; g.dn_sz = b_stride_z; g.dn_sh = b_stride_h; g.ldd = ldb;
  g.out_sz = c_stride_z; g.out_sh = c_stride_h; g.ldo = ldc;
  g.lut = d_lut; g.order = d_plan; g.plan = d_plan + bsp_dxx_plan_pairs_offset(width); g.width = width;
  g.div2 = 2 * (block / (dtype == BSP_F32 ? 8 : 16));   // step of the table: 8 for fp32, 16 otherwise (matmul.py:617)
  g.n_tiles = (N + 63) / 64;
  g.gplan = (no_groups(flags) || general_only(flags)) ? nullptr : d_gplan; g.n_pgroups = n_plan_groups; g.lines = plan_lines;
  if (int rc = xsd_workspace(g, n_split, N, d_ws, ws_bytes)) return rc;
  // rows of the kernel = rows of op(A); op(A)(m,k) is stored [k][m] when trans_a.  Dense (n,k) = op(B)[k][n]:
  // reduction contiguous when B is read transposed.  C[m][n] has n contiguous unless written transposed.
  return xsd_dispatch(dtype, g, block, trans_a != 0, trans_b != 0, !trans_c, flags, stream);
}

// Whether a dsd launch with these properties is taken by a kernel that runs split chains and so uses the workspace:
// the row-group kernels on 64 x 64 tiles (block 64, or block 16 with a plan over tiles: negative line count), 16-bit
// types, dense operand not reduction-contiguous, output rows contiguous, whole 64-wide tiles of the free dimension,
// and at block 64 a free dimension the wide kernel (xsd_dl, which comes first in xsd_dispatch) leaves alone.
static bool split_chains_run(int dtype, int block, int N, bool dn_kc, bool out_nc, int plan_lines, int flags) {
  if (dtype == BSP_F32 || dn_kc || !out_nc || N % 64) return false;
  if (no_groups(flags) || general_only(flags)) return false;
  if (block == 16) return plan_lines < 0;
  if (block == 64) return plan_lines > 0 && (N < 256 || no_wide(flags));
  return false;
}

// ---------------------------------------------------------------------------------------------------------
// The allocation-free variant of bsp_dsd_matmul: the workspace of the split chains is a static device array.
// In host code the array's name only stands for the symbol; its device address differs from GPU to GPU and is looked
// up once per device with hipGetSymbolAddress, with that device current, and kept.  Everything below uses that
// address, never the name.
// ---------------------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[BSP_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};   // per device: the address of its copy of `scratch`

// the device address of `scratch` on the current device (nullptr on failure)
void *scratch_address() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
    g_scratch_ptr[dev] = p;
  }
  return g_scratch_ptr[dev];
}

}  // namespace

extern "C" int bsp_dsd_matmul_noalloc(int dtype, const void *a, const void *b, void *c, int trans_a, int trans_b, int trans_c, int Z,
                                      int N, int64_t a_stride_z, int64_t b_stride_z, int64_t b_stride_h, int64_t ldb,
                                      int64_t c_stride_z, int64_t c_stride_h, int64_t ldc, int block, const int32_t *d_lut,
                                      const int32_t *d_plan, int width, const int32_t *d_gplan, int n_plan_groups,
                                      int plan_lines, int n_split, int flags, void *stream) {
  if (n_split < 0 || Z <= 0 || N <= 0) return BSP_ERR_ARG;
  void *ws = nullptr;
  int64_t ws_bytes = 0;
  if (d_gplan && n_split > 0 && !split_chains_run(dtype, block, N, trans_b != 0, !trans_c, plan_lines, flags)) {
    // A kernel that does not know split chains takes this launch (the wide kernel, the general one, fp32, ...): it
    // needs no scratch memory whatever the sizes, and must not see a plan whose chains are cut into parts.
    d_gplan = nullptr; n_plan_groups = 0; plan_lines = 0; n_split = 0;
  }
  if (d_gplan && n_split > 0) {
    if (xsd_ws_slots(n_split, N, Z) > BSP_NOALLOC_MAX_SLOTS) return BSP_ERR_SCRATCH_LIMIT;
    ws = scratch_address();
    if (!ws) return BSP_ERR_HIP;
    ws_bytes = BSP_NOALLOC_SCRATCH_BYTES;
    // (the buffer keeps what the last call left, which is harmless: every tile that is read was written by this call)
  }
  return bsp_dsd_matmul(dtype, a, b, c, trans_a, trans_b, trans_c, Z, N, a_stride_z, b_stride_z, b_stride_h, ldb, c_stride_z,
                        c_stride_h, ldc, block, d_lut, d_plan, width, d_gplan, n_plan_groups, plan_lines, n_split, ws, ws_bytes,
                        flags, stream);
}

extern "C" int bsp_dds_matmul(int dtype, const void *a, const void *b, void *c, int trans_a, int trans_b, int trans_c, int Z,
                              int M, int64_t a_stride_z, int64_t a_stride_h, int64_t lda, int64_t b_stride_z,
                              int64_t c_stride_z, int64_t c_stride_h, int64_t ldc, int block, const int32_t *d_lut,
                              const int32_t *d_plan, int width, const int32_t *d_gplan, int n_plan_groups, int plan_lines,
                              int n_split, void *d_ws, int64_t ws_bytes, int flags, void *stream) {
  if (!a || !b || !c || !d_lut || !d_plan || Z <= 0 || M <= 0 || width < 0) return BSP_ERR_ARG;
  if (d_gplan && (n_plan_groups <= 0 || plan_lines == 0)) return BSP_ERR_ARG;
  if (!block_ok(block)) return BSP_ERR_UNSUPPORTED;
  const int u = elems16(dtype);
  if (!aligned16(a) || !aligned16(b) || !aligned16(c)) return BSP_ERR_ARG;
  if (M % u || a_stride_z % u || a_stride_h % u || lda % u || b_stride_z % u || c_stride_z % u || c_stride_h % u || ldc % u) return BSP_ERR_ARG;
  XsdArgs g;
  g.sp = b; g.dn = a; g.out = c; g.Z = Z; g.NF = M;
  g.sp_sz = b_stride_z; g.dn_sz = a_stride_z; g.dn_sh = a_stride_h; g.ldd = lda;
  g.out_sz = c_stride_z; g.out_sh = c_stride_h; g.ldo = ldc;
  g.lut = d_lut; g.order = d_plan; g.plan = d_plan + bsp_dxx_plan_pairs_offset(width); g.width = width;
  g.div2 = 2 * (block / (dtype == BSP_F32 ? 8 : 16));
  g.n_tiles = (M + 63) / 64;
  g.gplan = (no_groups(flags) || general_only(flags)) ? nullptr : d_gplan; g.n_pgroups = n_plan_groups; g.lines = plan_lines;
  if (int rc = xsd_workspace(g, n_split, M, d_ws, ws_bytes)) return rc;
  // dds is dsd on the transposed problem: kernel rows = columns of op(B) (stored [k][col] unless trans_b), dense
  // rows = rows of op(A) (reduction contiguous unless trans_a), and C[row][col] has the kernel's m index contiguous
  // unless written transposed.
  return xsd_dispatch(dtype, g, block, !trans_b, !trans_a, trans_c != 0, flags, stream);
}
