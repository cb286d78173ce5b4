// Host-side declarations of the per-(PA,PB) kernel launchers built from valu_inst.hip.
#pragma once
#include <hip/hip_runtime.h>

#include "kparams.h"

namespace apnn {

#define APNN_DECL_VALU(kind, pa, pb) \
  hipError_t valu_##kind##_##pa##_##pb##_x(int vw, int tile, const KParams &p, hipStream_t s);
APNN_DECL_VALU(gemm, 1, 2)
APNN_DECL_VALU(gemm, 1, 3)
APNN_DECL_VALU(gemm, 1, 4)
APNN_DECL_VALU(gemm, 2, 2)
APNN_DECL_VALU(conv, 2, 1)
APNN_DECL_VALU(conv, 3, 1)
APNN_DECL_VALU(conv, 4, 1)
APNN_DECL_VALU(conv, 2, 2)
#undef APNN_DECL_VALU
hipError_t valu_gemm_any_x(int vw, int tile, const KParams &p, hipStream_t s);
hipError_t valu_conv_any_x(int vw, int tile, const KParams &p, hipStream_t s);

#define APNN_DECL_MFMA(kind, pa, pb) \
  hipError_t mfma_##kind##_##pa##_##pb##_x(int vw, int tile, const KParams &p, hipStream_t s);
#define APNN_DECL_MFMA4(kind, pa, pb) \
  hipError_t mfma4_##kind##_##pa##_##pb##_x(int vw, int tile, const KParams &p, hipStream_t s);
APNN_DECL_MFMA(gemm, 1, 2)
APNN_DECL_MFMA(gemm, 1, 3)
APNN_DECL_MFMA(gemm, 1, 4)
APNN_DECL_MFMA(gemm, 2, 2)
APNN_DECL_MFMA4(gemm, 1, 2)
APNN_DECL_MFMA4(gemm, 1, 3)
APNN_DECL_MFMA4(gemm, 1, 4)
APNN_DECL_MFMA4(gemm, 2, 2)
APNN_DECL_MFMA4(conv, 2, 1)
APNN_DECL_MFMA4(conv, 3, 1)
APNN_DECL_MFMA4(conv, 4, 1)
APNN_DECL_MFMA4(conv, 2, 2)
#undef APNN_DECL_MFMA
#define APNN_DECL_PATCH(pa, pb) hipError_t patch_conv_##pa##_##pb##_x(int tile, const KParams &p, hipStream_t s);
APNN_DECL_PATCH(2, 1)
APNN_DECL_PATCH(3, 1)
APNN_DECL_PATCH(4, 1)
APNN_DECL_PATCH(2, 2)
#undef APNN_DECL_PATCH
#undef APNN_DECL_MFMA4

// tile shapes of the MFMA kernels, index = enum MfmaTile in mfma_kernel.h
constexpr int kMfmaTileCount = 8;
constexpr int kMfmaTileA[kMfmaTileCount] = {256, 128, 64, 128, 32, 32, 256, 128};
constexpr int kMfmaTileB[kMfmaTileCount] = {256, 128, 64, 64, 32, 64, 128, 256};

// tile shapes of the patch-resident convolution kernel, index = enum PatchTile in patch_conv_kernel.h
constexpr int kPatchTileCount = 5;
constexpr int kPatchTileRows[kPatchTileCount] = {128, 256, 64, 128, 64};
constexpr int kPatchTileCols[kPatchTileCount] = {128, 64, 128, 64, 64};

// aux_kernels.hip
hipError_t launch_pack_bits(const uint32_t *values, uint32_t *planes, int rows, int C, int cpad, int bits,
                            hipStream_t s);

hipError_t launch_quantize_pack(const float *values, uint32_t *planes, int rows, int C, int cpad, int bits, float min_v,
                                float max_v, hipStream_t s);

// nn_kernels.hip
hipError_t launch_conv_i8_bn(const int8_t *X, const int8_t *Wt, const int32_t *thr, uint8_t *codes, int32_t *acc_out,
                             uint32_t *planes, int B, int H, int W, int C, int COUT, int R, int S, int stride, int pad,
                             int bits, int zero_point, hipStream_t s);
hipError_t launch_pool_planes(const uint32_t *in, uint32_t *out, int B, int H, int W, int cw, int bits, int win,
                              int stride, int pad, hipStream_t s);
hipError_t launch_pool_pack(const uint8_t *codes, uint32_t *planes, int B, int H, int W, int C, int cpad, int bits,
                            int win, int stride, int pad, hipStream_t s);
hipError_t launch_unpack_sum(const uint32_t *planes, int8_t *out, long long rows_out, int group, int C, int cpad,
                             int bits, int shift, hipStream_t s);
hipError_t launch_fc_i8(const int8_t *X, const int8_t *Wt, const float *scale, const float *bias, float *out,
                        int32_t *acc_out, int Bn, int N, int K, hipStream_t s);

}  // namespace apnn
