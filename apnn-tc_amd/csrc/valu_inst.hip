// One translation unit per (INST_PA, INST_PB, INST_CONV), selected on the compiler command line,
// so that the tile-shape instantiations of the VALU kernel build in parallel.
#include "valu_direct_kernel.h"
#include "valu_kernel.h"

#ifndef INST_PA
#error "compile with -DINST_PA=.. -DINST_PB=.. -DINST_CONV=0|1"
#endif

#define APNN_CAT2(a, b, c, d) a##b##_##c##_##d
#define APNN_CAT(a, b, c, d) APNN_CAT2(a, b, c, d)

namespace apnn {

#if INST_CONV
hipError_t APNN_CAT(valu_conv_, INST_PA, INST_PB, x)(int vw, int tile, const KParams &p, hipStream_t s) {
  // fully connected layer (filter spans the input map): rows of A are whole images, a plain GEMM
  if (tile == TILE_DIRECT) return launch_valu_direct<INST_PA, INST_PB, true>(p, s);
  switch (vw) {
    case 4: return launch_valu_tile<INST_PA, INST_PB, 4, true>(tile, p, s);
    case 2: return launch_valu_tile<INST_PA, INST_PB, 2, true>(tile, p, s);
    default: return launch_valu_tile<INST_PA, INST_PB, 1, true>(tile, p, s);
  }
}
#else
hipError_t APNN_CAT(valu_gemm_, INST_PA, INST_PB, x)(int vw, int tile, const KParams &p, hipStream_t s) {
  (void)vw;  // GEMM rows are whole int4 words (K % 128 == 0)
  if (tile == TILE_DIRECT) return launch_valu_direct<INST_PA, INST_PB, false>(p, s);
  return launch_valu_tile<INST_PA, INST_PB, 4, false>(tile, p, s);
}
#endif

}  // namespace apnn
