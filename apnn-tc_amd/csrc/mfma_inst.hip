// One translation unit per (INST_CORE, INST_PA, INST_PB, INST_CONV): tile-shape instantiations of
// the MFMA kernel.  INST_CORE 0 = int8 operands, 1 = FP4 operands.
#include "mfma_kernel.h"

#ifndef INST_PA
#error "compile with -DINST_PA=.. -DINST_PB=.. -DINST_CONV=0|1"
#endif

#if INST_CORE == 1
#define APNN_PFX(n) mfma4_##n
#else
#define APNN_PFX(n) mfma_##n
#endif
#define APNN_CAT2(a, b, c, d) a##b##_##c##_##d
#define APNN_CAT(a, b, c, d) APNN_CAT2(a, b, c, d)

namespace apnn {

#if INST_CONV
hipError_t APNN_CAT(APNN_PFX(conv_), INST_PA, INST_PB, x)(int vw, int tile, const KParams &p, hipStream_t s) {
  switch (vw) {
    case 4: return launch_mfma_tile<INST_CORE, INST_PA, INST_PB, 4, true>(tile, p, s);
    case 2: return launch_mfma_tile<INST_CORE, INST_PA, INST_PB, 2, true>(tile, p, s);
    default: return launch_mfma_tile<INST_CORE, INST_PA, INST_PB, 1, true>(tile, p, s);
  }
}
#else
hipError_t APNN_CAT(APNN_PFX(gemm_), INST_PA, INST_PB, x)(int vw, int tile, const KParams &p, hipStream_t s) {
  (void)vw;
  return launch_mfma_tile<INST_CORE, INST_PA, INST_PB, 4, false>(tile, p, s);
}
#endif

}  // namespace apnn
