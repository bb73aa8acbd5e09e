// Instantiates the general matmul kernels for one element type (one translation unit per type keeps the
// three compiles parallel).
#include "matmul_generic.h"
namespace bsp {
int sdd_generic_f16(const SddArgs &g, int block, int pack, bool a_kc, bool b_kc, hipStream_t st) {
  return launch_sdd<f16>(g, block, pack, a_kc, b_kc, st);
}
int xsd_generic_f16(const XsdArgs &g, int block, bool sp_trans, bool dn_kc, bool out_nc, hipStream_t st) {
  return launch_xsd<f16>(g, block, sp_trans, dn_kc, out_nc, st);
}
}  // namespace bsp
