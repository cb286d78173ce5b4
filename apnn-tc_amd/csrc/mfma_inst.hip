// One translation unit per (INST_PA, INST_PB, INST_CONV): tile-shape instantiations of the MFMA kernel.
#include "mfma_kernel.h"

#ifndef INST_PA
#error "compile with -DINST_PA=.. -DINST_PB=.. -DINST_CONV=0|1"
#endif

#define APNN_CAT2(a, b, c, d) a##b##_##c##_##d
#define APNN_CAT(a, b, c, d) APNN_CAT2(a, b, c, d)

namespace apnn {

#if INST_CONV
hipError_t APNN_CAT(mfma_conv_, INST_PA, INST_PB, x)(int vw, int tile, const KParams &p, hipStream_t s) {
  switch (vw) {
    case 4: return launch_mfma_tile<INST_PA, INST_PB, 4, true>(tile, p, s);
    case 2: return launch_mfma_tile<INST_PA, INST_PB, 2, true>(tile, p, s);
    default: return launch_mfma_tile<INST_PA, INST_PB, 1, true>(tile, p, s);
  }
}
#else
hipError_t APNN_CAT(mfma_gemm_, INST_PA, INST_PB, x)(int vw, int tile, const KParams &p, hipStream_t s) {
  (void)vw;
  return launch_mfma_tile<INST_PA, INST_PB, 4, false>(tile, p, s);
}
#endif

}  // namespace apnn
