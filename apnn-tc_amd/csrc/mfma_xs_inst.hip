// One translation unit per (INST_PA, INST_PB, INST_CONV): tile-shape instantiations of the matrix-core
// kernel whose operands are expanded while staging (mfma_xs_kernel.h).
#include "mfma_xs_kernel.h"

#ifndef INST_PA
#error "compile with -DINST_PA=.. -DINST_PB=.. -DINST_CONV=0|1"
#endif
#define APNN_CAT2(a, b, c, d) a##b##_##c##_##d
#define APNN_CAT(a, b, c, d) APNN_CAT2(a, b, c, d)

namespace apnn {

#if INST_CONV
hipError_t APNN_CAT(mfmaxs_conv_, INST_PA, INST_PB, x)(int vw, int tile, const KParams &p, hipStream_t s) {
  if (vw != 4) return hipErrorNotSupported;  // 128-bit loads: at least 128 stored channels
  return launch_mfma_xs_tile<INST_PA, INST_PB, 4, true>(tile, p, s);
}
#else
hipError_t APNN_CAT(mfmaxs_gemm_, INST_PA, INST_PB, x)(int vw, int tile, const KParams &p, hipStream_t s) {
  (void)vw;
  return launch_mfma_xs_tile<INST_PA, INST_PB, 4, false>(tile, p, s);
}
#endif

}  // namespace apnn
