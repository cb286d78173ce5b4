// One translation unit per (INST_PA, INST_PB): tile-shape instantiations of the patch-resident
// convolution kernel.
#include "patch_conv_kernel.h"

#ifndef INST_PA
#error "compile with -DINST_PA=.. -DINST_PB=.."
#endif
#define APNN_CAT2(a, b, c, d) a##b##_##c##_##d
#define APNN_CAT(a, b, c, d) APNN_CAT2(a, b, c, d)

namespace apnn {

hipError_t APNN_CAT(patch_conv_, INST_PA, INST_PB, x)(int tile, const KParams &p, hipStream_t s) {
  return launch_patch_tile<INST_PA, INST_PB>(tile, p, s);
}

}  // namespace apnn
