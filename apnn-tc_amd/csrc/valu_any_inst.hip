// Any-precision instantiation of the VALU kernel (1..8 planes per operand chosen at launch): serves the
// (w, a) combinations that have no kernel of their own (w1a1, w1a5, w1a8, w2a6, w2a8, w4a4, ...).
#include "valu_kernel.h"

namespace apnn {

hipError_t valu_gemm_any_x(int vw, int tile, const KParams &p, hipStream_t s) {
  (void)vw;
  (void)tile;
  return launch_valu_any<4, false>(p, s);
}

hipError_t valu_conv_any_x(int vw, int tile, const KParams &p, hipStream_t s) {
  (void)tile;
  switch (vw) {
    case 4: return launch_valu_any<4, true>(p, s);
    case 2: return launch_valu_any<2, true>(p, s);
    default: return launch_valu_any<1, true>(p, s);
  }
}

}  // namespace apnn
