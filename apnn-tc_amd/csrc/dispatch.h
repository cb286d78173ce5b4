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
APNN_DECL_MFMA(conv, 2, 1)
APNN_DECL_MFMA(conv, 3, 1)
APNN_DECL_MFMA(conv, 4, 1)
APNN_DECL_MFMA(conv, 2, 2)
APNN_DECL_MFMA4(gemm, 1, 1)
APNN_DECL_MFMA4(conv, 5, 1)
APNN_DECL_MFMA4(conv, 6, 2)
APNN_DECL_MFMA4(gemm, 4, 4)
APNN_DECL_MFMA4(gemm, 1, 8)
APNN_DECL_MFMA4(gemm, 2, 8)
APNN_DECL_MFMA4(conv, 8, 1)
APNN_DECL_MFMA4(conv, 8, 2)
APNN_DECL_MFMA4(conv, 4, 4)
APNN_DECL_MFMA4(gemm, 1, 2)
APNN_DECL_MFMA4(gemm, 1, 3)
APNN_DECL_MFMA4(gemm, 1, 4)
APNN_DECL_MFMA4(gemm, 2, 2)
APNN_DECL_MFMA4(conv, 2, 1)
APNN_DECL_MFMA4(conv, 3, 1)
APNN_DECL_MFMA4(conv, 4, 1)
APNN_DECL_MFMA4(conv, 2, 2)
#undef APNN_DECL_MFMA
#define APNN_DECL_MFMAXS(kind, pa, pb) \
  hipError_t mfmaxs_##kind##_##pa##_##pb##_x(int vw, int tile, const KParams &p, hipStream_t s);
APNN_DECL_MFMAXS(gemm, 1, 2)
APNN_DECL_MFMAXS(gemm, 1, 3)
APNN_DECL_MFMAXS(gemm, 1, 4)
APNN_DECL_MFMAXS(gemm, 2, 2)
APNN_DECL_MFMAXS(conv, 2, 1)
APNN_DECL_MFMAXS(conv, 3, 1)
APNN_DECL_MFMAXS(conv, 4, 1)
APNN_DECL_MFMAXS(conv, 2, 2)
#undef APNN_DECL_MFMAXS
#define APNN_DECL_PATCH(pa, pb) hipError_t patch_conv_##pa##_##pb##_x(int tile, const KParams &p, hipStream_t s);
APNN_DECL_PATCH(2, 1)
APNN_DECL_PATCH(3, 1)
APNN_DECL_PATCH(4, 1)
APNN_DECL_PATCH(2, 2)
#undef APNN_DECL_PATCH
#undef APNN_DECL_MFMA4

// operand encodings of the matrix-core kernels (mfma_kernel.h)
enum { CORE_I8 = 0, CORE_F4 = 1 };

// tile shapes of the MFMA kernels, index = enum MfmaTile in mfma_kernel.h
constexpr int kMfmaTileCount = 10;
constexpr int kMfmaTileA[kMfmaTileCount] = {256, 128, 64, 128, 32, 32, 256, 128, 32, 128};
constexpr int kMfmaTileB[kMfmaTileCount] = {256, 128, 64, 64, 32, 64, 128, 256, 128, 128};

// MT_128x128_G2: the 128x128 tile computed by two groups of four waves that share its k-steps (work-groups
// of 512 threads)
enum MfmaTile { MT_256x256 = 0, MT_128x128 = 1, MT_64x64 = 2, MT_128x64 = 3, MT_32x32_K4 = 4, MT_32x64_K4 = 5,
                MT_256x128 = 6, MT_128x256 = 7, MT_32x128_K4 = 8, MT_128x128_G2 = 9, MT_COUNT = 10 };

// Which (core, family, load width, tile, plane counts) combinations are built.  Every kernel
// instantiation costs seconds of compile time, so only the shapes the dispatcher can choose are kept:
//   int8 core : GEMM entry points 256x128, 128x128, 64x64; convolution with 128-bit loads 128x256,
//               128x128, 128x64, 64x64 and the 32x32 split-K tile, with narrower loads 64x64 only
//   FP4 core  : GEMM: all but 256x256 / 128x256;  convolution: all but 256x256 / 256x128, and only
//               the two small tiles when the stored channel count allows 32-bit loads only;
//               plus, for convolution with 128-bit loads, the 32x128 split-K tile;
//               more than five planes in all (w4a4, w1a8, w2a8): 128x128, 64x64, 32x32 split-K
//               (convolution with narrower loads: 64x64 only); the int8 core is not built for those.
constexpr bool mfma_tile_enabled(int core, bool conv, int vw, int tile, int pa, int pb) {
  // two wave groups: FP4 core, 128-bit loads, the four benchmark precisions
  if (tile == MT_128x128_G2) return core == CORE_F4 && pa + pb <= 5 && pa + pb > 2 && (!conv || vw == 4);
  if (pa + pb > 5 || pa + pb == 2) {
    if (core == CORE_I8) return false;
    if (conv && vw != 4) return tile == MT_64x64;
    return tile == MT_128x128 || tile == MT_64x64 || tile == MT_32x32_K4;
  }
  if (core == CORE_I8) {
    if (!conv) return tile == MT_128x128 || tile == MT_64x64 || tile == MT_256x128;
    if (vw != 4) return tile == MT_64x64;
    return tile == MT_128x256 || tile == MT_128x128 || tile == MT_128x64 || tile == MT_64x64 || tile == MT_32x32_K4;
  }
  // 32x128 split-K: FP4 convolution with 128-bit loads (operands go straight to registers)
  if (tile == MT_32x128_K4) return conv && vw == 4;
  if (!conv) return tile != MT_256x256 && tile != MT_128x256;
  if (vw == 1) return tile == MT_64x64 || tile == MT_32x32_K4;
  return tile != MT_256x256 && tile != MT_256x128;
}

// tiles of the kernel that expands operands while staging (mfma_xs_kernel.h), by their MfmaTile index:
// the shapes whose four waves tile the output; convolution with 128-bit loads only
constexpr bool mfma_xs_tile_enabled(bool conv, int vw, int tile) {
  if (conv) return vw == 4 && (tile == MT_128x128 || tile == MT_64x64 || tile == MT_128x64 || tile == MT_128x256);
  return tile == MT_128x128 || tile == MT_64x64 || tile == MT_128x64 || tile == MT_256x128;
}

// tile shapes of the patch-resident convolution kernel, index = enum PatchTile in patch_conv_kernel.h
constexpr int kPatchTileCount = 5;
constexpr int kPatchTileRows[kPatchTileCount] = {128, 256, 64, 128, 64};
constexpr int kPatchTileCols[kPatchTileCount] = {128, 64, 128, 64, 64};

// aux_kernels.hip
hipError_t launch_pack_bits(const uint32_t *values, uint32_t *planes, int rows, int C, int cpad, int bits,
                            hipStream_t s);
hipError_t launch_pack_top_plane(const uint32_t *values, uint32_t *plane, int rows, int C, int cpad, int bits,
                                 hipStream_t s);

hipError_t launch_quantize_pack(const float *values, uint32_t *planes, int rows, int C, int cpad, int bits, float min_v,
                                float max_v, hipStream_t s);

hipError_t launch_quantize_pack_u8(const uint8_t *values, uint32_t *planes, int rows, int C, int cpad, int bits,
                                   hipStream_t s);
hipError_t launch_binarize_pack(const float *values, uint32_t *planes, int rows, int C, int cpad, hipStream_t s);
hipError_t launch_residual_prepare(const int32_t *in, int32_t *out, int B, int Ho, int Wo, int in_pitch, int channels,
                                   int out_channels, int pool, hipStream_t s);

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
