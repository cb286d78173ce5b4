/*
 * apnn_tc.h -- C ABI of the MI355X (gfx950) arbitrary-precision GEMM / convolution library.
 *
 * Every entry point is host-callable, takes caller-owned DEVICE buffers (16-byte aligned, as the
 * reference's int4 loads require), enqueues work on the given HIP stream (NULL = default stream)
 * and returns without synchronizing.  Return value: 0 on success, a negative APNN_E* code for a
 * rejected argument (nothing is launched), or a positive hipError_t from the launch.  Nothing here
 * aborts, allocates device memory or keeps state between calls.
 *
 * Reference paths below are relative to the reference checkout:
 *   LIB = APNN-TC-lib/bmmaTensorCoreGemm/src,  NN = APNN-TC-nn/src
 *
 * Data layout (identical to the reference):
 *   bit-planes are plane-major, LSB plane first, uint32 words; element k of a row is bit k%32 of
 *   word k/32 (LIB/71_bmmaTensorCoreGemm.cu:362-369);
 *   GEMM  W:[wb][M][K/32]  X:[xb][N][K/32]  D:[M][N] int32            (LIB/71:362-373)
 *   conv  X:[xb][H+2][W+2][CIN/32] (halo stored)  W:[wb][COUT][3][3][CIN/32]  O:[H][W][COUT] int32
 *                                                                    (LIB/51_bmmaTensorCoreGemm.cu:395-411)
 *   packed outputs: [out_bits][rows][cols/32], column c at bit 31-c%32 (LIB/66_bmmaTensorCoreGemm.cuh:399-404,
 *   LIB/67_bmmaTensorCoreGemm.cuh:466-477).
 */
#ifndef APNN_TC_H
#define APNN_TC_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define APNN_OK            0
#define APNN_EINVAL      (-1)  /* dimension / bit-width / mode outside the supported set */
#define APNN_ENULL       (-2)  /* required pointer is NULL */
#define APNN_EALIGN      (-3)  /* operand not 16-byte aligned */
#define APNN_EUNSUPPORTED (-4) /* valid request that no kernel in this build serves */

typedef void *apnn_stream_t; /* a hipStream_t */

/* ---- reference kernel entry points --------------------------------------------------------- */

/* D[m][n] = sum_{i<xb} sum_{j<wb} 2^(i+j) popc(W_j[m] & X_i[n]), int32.
 * Replace the __global__ kernels  apmm_w1a2 (LIB/71:80), apmm_w1a4 (LIB/78_bmmaTensorCoreGemm.cu:80),
 * apmm_w2a2 (LIB/72_bmmaTensorCoreGemm.cu:80); w1a3 has no GEMM kernel in the reference tree (only
 * the mirrored apmm_w3a1, LIB/79_bmmaTensorCoreGemm.cu:80) and follows the same definition.
 * wb / xb must equal the bit widths in the function name.  Requires K % 128 == 0 (int4 rows). */
int apmm_w1a2(const void *W, const void *X, int *D, int M, int N, int K, int wb, int xb, apnn_stream_t s);
int apmm_w1a3(const void *W, const void *X, int *D, int M, int N, int K, int wb, int xb, apnn_stream_t s);
int apmm_w1a4(const void *W, const void *X, int *D, int M, int N, int K, int wb, int xb, apnn_stream_t s);
int apmm_w2a2(const void *W, const void *X, int *D, int M, int N, int K, int wb, int xb, apnn_stream_t s);

/* Further precisions of the reference tree, same definition and constraints: apmm_w1a8
 * (LIB/77_bmmaTensorCoreGemm.cu:80), apmm_w2a8 (LIB/76_bmmaTensorCoreGemm.cuh:80-82), apmm_w4a4
 * (LIB/83_bmmaTensorCoreGemm.cu:80), apmm_w1a1 (LIB/84_bmmaTensorCoreGemm.cu:80).  Any other (w, a) up to
 * 8 bits each is served by apnn_gemm / apnn_conv.  w4a4, w1a8 and w2a8 have FP4 matrix-core kernels
 * (digit pairs weighted through the block scale) besides the any-precision VALU kernel. */
int apmm_w1a8(const void *W, const void *X, int *D, int M, int N, int K, int wb, int xb, apnn_stream_t s);
int apmm_w2a8(const void *W, const void *X, int *D, int M, int N, int K, int wb, int xb, apnn_stream_t s);
int apmm_w4a4(const void *W, const void *X, int *D, int M, int N, int K, int wb, int xb, apnn_stream_t s);
int apmm_w1a1(const void *W, const void *X, int *D, int M, int N, int K, int wb, int xb, apnn_stream_t s);

/* Same accumulate, then the low xb bits of each result packed MSB-first along N:
 * D:[xb][M][N/32] uint32.  Replace apmm_w1a2_decompose (LIB/66h:82-280) and apmm_w2a2_decompose
 * (LIB/73_bmmaTensorCoreGemm.cuh:82).  Requires N % 32 == 0. */
int apmm_w1a2_decompose(const void *W, const void *X, int *D, int M, int N, int K, int wb, int xb, apnn_stream_t s);
int apmm_w1a3_decompose(const void *W, const void *X, int *D, int M, int N, int K, int wb, int xb, apnn_stream_t s);
int apmm_w1a4_decompose(const void *W, const void *X, int *D, int M, int N, int K, int wb, int xb, apnn_stream_t s);
int apmm_w2a2_decompose(const void *W, const void *X, int *D, int M, int N, int K, int wb, int xb, apnn_stream_t s);

/* 3x3 / stride 1 / pad 1 convolution on a halo-stored input, int32 NHWC output.
 * Replace compute_conv_imma: w1a2 LIB/51:58, w1a4 LIB/53_bmmaTensorCoreGemm.cu:58,
 * w1a3 LIB/59_bmmaTensorCoreGemm.cu:58, w2a2 LIB/48_bmmaTensorCoreGemm.cu:58.
 * Requires CIN % 128 == 0; any Height / Width / COUT. */
int apconv_w1a2(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);
int apconv_w1a3(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);
int apconv_w1a4(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);
int apconv_w2a2(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);

/* compute_conv_imma at w1a5 (LIB/61_bmmaTensorCoreGemm.cu:58, LIB/62) and w2a6 (LIB/63_bmmaTensorCoreGemm.cu:58). */
int apconv_w1a5(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);
int apconv_w2a6(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);
/* compute_conv_imma at w1a8 (LIB/55_bmmaTensorCoreGemm.cu:58, LIB/56) and w2a8 (LIB/57_bmmaTensorCoreGemm.cu:58, LIB/58). */
int apconv_w1a8(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);
int apconv_w2a8(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);

/* Convolution, then low-bit planes of the result: Output:[a][H][W][COUT/32].
 * Replace APConv_w1a2_pack (LIB/67h:60-325) and APConv_w2a2_pack (LIB/70_bmmaTensorCoreGemm.cu:58).
 * Requires COUT % 32 == 0. */
int APConv_w1a2_pack(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);
int APConv_w1a3_pack(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);
int APConv_w1a4_pack(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);
int APConv_w2a2_pack(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);

/* APConv_w2a8_pack (LIB/74_bmmaTensorCoreGemm.cuh:58-61): Output:[8][H][W][COUT/32]. */
int APConv_w2a8_pack(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);

/* Convolution, 2x2 average pool with C integer division, then low-bit planes:
 * Output:[a][H/2][W/2][COUT/32].  Replace APConv_w1a2_pack_pool (LIB/68_bmmaTensorCoreGemm.cu:58)
 * and APConv_w2a2_pack_pool (LIB/69_bmmaTensorCoreGemm.cuh:60).  Requires even Height and Width. */
int APConv_w1a2_pack_pool(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);
int APConv_w2a2_pack_pool(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);
/* APConv_w2a8_pack_pool (LIB/75_bmmaTensorCoreGemm.cu:58): Output:[8][H/2][W/2][COUT/32]. */
int APConv_w2a8_pack_pool(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT, apnn_stream_t s);

/* ---- general descriptor entry points ------------------------------------------------------- */

enum { APNN_EPI_INT32 = 0,    /* int32 result                                                     */
       APNN_EPI_LOWBITS = 1,  /* low out_bits bits of the result, packed (LIB/66h:255-276)         */
       APNN_EPI_BN = 2 };     /* per-channel thresholds -> out_bits code, packed                   */
enum { APNN_POOL_NONE = 0,
       APNN_POOL_AVG2X2 = 1,  /* (v0+v1+v2+v3)/4 on the int32 result before quantizing (LIB/68:280-292) */
       APNN_POOL_MAX2X2 = 2 };/* max over the 2x2 window of the quantized codes                     */
enum { APNN_PATH_AUTO = 0,
       APNN_PATH_VALU = 1,     /* v_and + v_bcnt popcount on packed words                           */
       APNN_PATH_MFMA = 2,     /* planes expanded to FP4 operands of v_mfma_f32_32x32x64_f8f6f4; fp32
                                  accumulation, exact while K*(2^wb-1)*(2^xb-1) < 2^24: beyond that a
                                  pinned FP4 path returns APNN_EUNSUPPORTED and AUTO uses the int8 core   */
       APNN_PATH_MFMA_I8 = 3,  /* planes expanded to int8 operands of v_mfma_i32_32x32x32_i8         */
       APNN_PATH_MFMA_PATCH = 4,/* convolution only: FP4 matrix-core path with the tile's input patch
                                  expanded once into LDS and read in place by every filter tap;
                                  APNN_EUNSUPPORTED when the patch or filter block does not fit   */
       APNN_PATH_MFMA_XS = 5 };/* FP4 matrix-core path whose staging threads expand the planes, so that
                                  LDS holds ready operands (tiles 128x128, 64x64, 128x64 and 256x128 /
                                  128x256; w1a2, w1a3, w1a4, w2a2; convolution needs cin_pad % 128 == 0) */
/* `path` fields: low byte = APNN_PATH_*; bits 8..15 = 0 (library picks the tile shape) or
 * 1 + tile index to pin it (tuning / test coverage of every tile shape; APNN_EINVAL if the
 * chosen kernel family has no such tile or the epilogue cannot use it). */
#define APNN_PATH_TILE(path, tile) ((path) | (((tile) + 1) << 8))
enum { APNN_WEIGHT_UNSIGNED = 0,   /* planes are an unsigned integer u (the reference's arithmetic)    */
       APNN_WEIGHT_SYMMETRIC = 1 };/* weight value is 2u - (2^wb - 1); wb = 1 gives {-1,+1}            */

/* Output stage shared by GEMM and convolution.  "channel" is the fast output index
 * (N for GEMM, COUT for convolution).
 *   v = acc (after AVG pooling if requested) + (residual ? residual[row][channel] : 0)
 *         + (residual_planes ? residual_scale * code(residual_planes)[row][channel] : 0)
 *   save_acc (optional) receives v as int32 [rows][channels]   (cf. save_residual, NN/kernel.cuh:779-831)
 *   LOWBITS: code = v & (2^out_bits - 1)
 *   BN     : code = #{ k < 2^out_bits-1 : (flip[channel] ? -v : v) >= thresholds[channel][k] }
 *            (out_bits = 1 is the reference's  !(v < bn[channel]), NN/kernel.cuh:833-834)
 *   planes of code are written MSB-first: [out_bits][rows][channels/32].
 * residual / save_acc cannot be combined with pooling. */
typedef struct apnn_epilogue {
  int mode;                  /* APNN_EPI_* */
  int out_bits;              /* 1..8, LOWBITS / BN */
  int pool;                  /* APNN_POOL_*, convolution only */
  const int32_t *thresholds; /* device, [channels][2^out_bits - 1], non-decreasing per channel (BN) */
  const uint8_t *flip;       /* device, [channels] or NULL (BN) */
  const int32_t *residual;   /* device, [rows][channels] int32 or NULL */
  int32_t *save_acc;         /* device, [rows][channels] int32 or NULL */
  const uint32_t *residual_planes; /* device, packed codes [residual_bits][rows][channels/32] of a
                                      shortcut branch (identity: the block input), or NULL */
  int residual_bits;         /* 1..8 */
  int residual_scale;        /* integer factor that brings the shortcut codes to accumulator scale */
} apnn_epilogue;

/* out[m][n] over W:[wb][M][K/32] (slow index) and X:[xb][N][K/32] (fast index). */
typedef struct apnn_gemm_desc {
  const void *W, *X;
  void *D;
  int M, N, K;               /* K % 128 == 0 */
  int wb, xb;                /* 1..4 each */
  int weight_mode;           /* APNN_WEIGHT_*; SYMMETRIC makes W the signed operand */
  apnn_epilogue epi;
  int path;                  /* APNN_PATH_* */
} apnn_gemm_desc;
int apnn_gemm(const apnn_gemm_desc *d, apnn_stream_t s);

/* Convolution / fully-connected (R=S=1, H=W=1, batch = rows) over NHWC bit-planes.
 * X:[xb][batch][Hs][Ws][cin_pad/32] with Hs = H + (halo ? 2*pad : 0); W:[wb][COUT][R][S][cin_pad/32];
 * output rows are (batch, oy, ox) in raster order, channels COUT. */
typedef struct apnn_conv_desc {
  const void *W, *X;
  void *O;
  int batch, H, Wd;          /* logical input size */
  int cin_pad;               /* stored channels per pixel, multiple of 32 (reference: multiple of 128) */
  int COUT;
  int R, S, stride, pad;
  int halo;                  /* 1: input stored with its halo, whose contents take part (LIB/51:395);
                                0: unpadded input, out-of-image taps are zero */
  int wb, xb;
  int weight_mode;           /* SYMMETRIC makes W the signed operand */
  apnn_epilogue epi;
  int path;
} apnn_conv_desc;
int apnn_conv(const apnn_conv_desc *d, apnn_stream_t s);

/* What apnn_gemm / apnn_conv would launch for a descriptor: same validation and kernel choice, nothing
 * is enqueued and no buffer is touched (no counterpart in the reference, whose kernels are picked at
 * compile time).  For tuning, and for checking the dispatcher without a device. */
enum { APNN_KERNEL_VALU_TILE = 0,   /* LDS-tiled popcount kernel                                     */
       APNN_KERNEL_VALU_DIRECT = 1, /* register-only popcount kernel (small GEMMs, FC layers)         */
       APNN_KERNEL_MFMA_FP4 = 2,
       APNN_KERNEL_MFMA_I8 = 3,
       APNN_KERNEL_PATCH_FP4 = 4,
       APNN_KERNEL_MFMA_FP4_XS = 5 };
typedef struct apnn_plan {
  int path;              /* APNN_PATH_* taken (never AUTO) */
  int kernel;            /* APNN_KERNEL_* */
  int tile;              /* tile index within the kernel family (the value APNN_PATH_TILE pins) */
  int tile_rows, tile_cols; /* outputs per work-group: slow x fast output index */
  int split_k;           /* waves of a work-group that share one output block */
  long long workgroups;
  int patch_pixels;      /* APNN_KERNEL_PATCH_FP4: padded-frame pixels a work-group stages, else 0 */
  int fp4_exact;         /* 1: fp32 accumulation of FP4 operands is exact for this reduction length */
} apnn_plan;
int apnn_gemm_plan(const apnn_gemm_desc *d, apnn_plan *plan);
int apnn_conv_plan(const apnn_conv_desc *d, apnn_plan *plan);

/* Bit-plane packer with the layout of Bit_compression (NN/kernel.cuh:46-77):
 * values:[rows][C] uint32 codes -> planes:[bits][rows][cpad/32], channel c at bit 31-c%32,
 * pad channels zero.  cpad % 32 == 0, cpad >= C. */
int apnn_pack_bits(const uint32_t *values, uint32_t *planes, int rows, int C, int cpad, int bits, apnn_stream_t s);

/* Bit_compression_fc_hidden (APNN-TC-nn/src/kernel.cuh:78-126, used by weight_quantization_fc_hidden, :272):
 * the same packer, except that the reference stores every bit-plane at the same words (the plane offset is
 * commented out, kernel.cuh:118-123), so what its buffer holds afterwards is the plane written last, bit
 * bits-1 of every value.  values:[rows][C] uint32 codes -> plane:[rows][cpad/32], channel c at bit 31-c%32,
 * pad channels zero; with bits == 1 identical to apnn_pack_bits. */
int apnn_pack_bits_fc_hidden(const uint32_t *values, uint32_t *plane, int rows, int C, int cpad, int bits,
                             apnn_stream_t s);

/* ---- layers on either side of the low-bit path ------------------------------------------------ */

/* Two convolutions of the same input onto the same output grid in one launch: the entry of a residual
 * block, where the 3x3 convolution of the main branch and the 1x1 downsample convolution of the
 * shortcut both read the block input (no counterpart in the reference, whose ResNet18 has no downsample
 * convolution, APNN-TC-nn/src/resnet18.cu:40-142).  a and b must agree in X, batch, H, Wd, cin_pad, COUT,
 * stride, halo, wb, xb, weight_mode and output size, and both use APNN_EPI_BN with the same out_bits and no
 * pooling / residual inputs; filter, filter size, padding, thresholds, flip and output differ.  When the
 * pair cannot share a matrix-core kernel the two are launched one after the other: the result is the
 * same either way. */
int apnn_conv_pair(const apnn_conv_desc *a, const apnn_conv_desc *b, apnn_stream_t s);

/* Float tensor -> bit-planes in one pass: the affine quantizer of Quantize_val
 * (APNN-TC-nn/src/kernel.cuh:29-44; the reference computes the code but its store is commented out)
 *     code = min(2^bits - 1, rint(((clip(x, min_v, max_v) - min_v) * 2^bits * 1.0f) / (max_v - min_v)))
 * in fp32 with exactly that operation order (rint = round half to even, __float2uint_rn), followed by
 * the Bit_compression layout of apnn_pack_bits.  values:[rows][C] float; planes:[bits][rows][cpad/32].
 * The reference fixes min_v = -10, max_v = 10 (kernel.cuh:17-18). */
int apnn_quantize_pack(const float *values, uint32_t *planes, int rows, int C, int cpad, int bits, float min_v,
                       float max_v, apnn_stream_t s);

/* uint8 samples (raw image bytes) -> bit-planes: code = value >> (8 - bits), a uniform 2^bits-level
 * quantizer of [0, 256), then the Bit_compression layout.  What images_quantization
 * (APNN-TC-nn/src/kernel.cuh:129-161) does for a float image, for the uint8 images the networks here take. */
int apnn_quantize_pack_u8(const uint8_t *values, uint32_t *planes, int rows, int C, int cpad, int bits,
                          apnn_stream_t s);

/* Float rows -> one bit-plane, bit = value >= 0, MSB-first: the input layer of the reference's fully
 * connected networks (In128Layer, APNN-TC-nn/src/kernel.cuh:321-340).  planes:[rows][cpad/32]. */
int apnn_binarize_pack(const float *values, uint32_t *planes, int rows, int C, int cpad, apnn_stream_t s);

/* int32 shortcut map saved by an earlier layer (apnn_epilogue.save_acc) -> the `residual` operand of a
 * later layer: the residual is added to channels below `channels` only and, with pool = 1, is the 2x2
 * maximum of a source map of twice the height and width (inject_residual / residual_channels /
 * residual_pool of Conv128Layer, APNN-TC-nn/src/kernel.cuh:779-831).
 * in:[B][Ho*(1+pool)][Wo*(1+pool)][in_pitch] -> out:[B][Ho][Wo][out_channels], zero at channels >= `channels`. */
int apnn_residual_prepare(const int32_t *in, int32_t *out, int B, int Ho, int Wo, int in_pitch, int channels,
                          int out_channels, int pool, apnn_stream_t s);

/* Host-side preparation (no device work): fold a batch-norm + uniform activation quantizer into the
 * integer thresholds of APNN_EPI_BN.  With y(v) = gamma[c] * (v * in_scale - mean[c]) / sqrt(var[c] + eps)
 * + beta[c] evaluated in double precision, code = clamp(floor(y / step), 0, 2^bits - 1) equals
 * #{k : s_c * v >= thresholds[c][k]} for every int32 v, where flip[c] = 1 (s_c = -1) when y decreases in
 * v.  thresholds:[C][2^bits-1] int32 (host), flip:[C] bytes (host).  The reference folds only a 1-bit
 * threshold offline (its layers read one float per channel, APNN-TC-nn/src/kernel.cuh:833-834). */
int apnn_fold_bn(const float *gamma, const float *beta, const float *mean, const float *var, float eps,
                 float in_scale, float step, int C, int bits, int32_t *thresholds, uint8_t *flip);

/* int8 NHWC convolution with zero padding (the first layer of a network, cf. the int8 convention of
 * cutlass_nn/src/config.h:215-255: int8 operands, int32 accumulate), followed by per-channel
 * thresholds: code = #{k : acc >= thresholds[c][k]}.
 * X:[B][H][W][C] int8, Wt:[COUT][R][S][C] int8; codes:[B][Ho][Wo][COUT] uint8 (NULL to skip),
 * acc_out:[B][Ho][Wo][COUT] int32 (NULL to skip); thresholds may be NULL when codes is NULL.
 * x_zero_point != 0: X holds uint8 pixels and x - x_zero_point is convolved (128 for raw images). */
int apnn_conv_i8_bn(const int8_t *X, const int8_t *Wt, const int32_t *thresholds, uint8_t *codes, int32_t *acc_out,
                    int B, int H, int W, int C, int COUT, int R, int S, int stride, int pad, int bits,
                    int x_zero_point, apnn_stream_t s);

/* Same convolution for image-like inputs (C <= 4), thresholds applied, result written directly as
 * MSB-first bit-planes [bits][B*Ho*Wo][COUT/32] (COUT % 32 == 0): the first layer's activations never
 * exist unpacked in memory. */
int apnn_conv_i8_bn_pack(const int8_t *X, const int8_t *Wt, const int32_t *thresholds, uint32_t *planes, int B, int H,
                         int W, int C, int COUT, int R, int S, int stride, int pad, int bits, int x_zero_point,
                         apnn_stream_t s);

/* win x win max-pool of multi-bit codes directly on their bit-planes (32 channels per bitwise
 * compare): in:[bits][B*H*W][cpad/32] -> out:[bits][B*Ho*Wo][cpad/32]; out-of-image taps are ignored. */
int apnn_pool_planes(const uint32_t *in, uint32_t *out, int B, int H, int W, int cpad, int bits, int win, int stride,
                     int pad, apnn_stream_t s);

/* win x win max-pool (stride, zero-free padding: out-of-image taps are ignored) over uint8 codes
 * [B][H][W][C], then bit-plane packing with the Bit_compression layout (NN/kernel.cuh:46-77):
 * planes:[bits][B*Ho*Wo][cpad/32].  win = stride = 1, pad = 0 packs without pooling. */
int apnn_pool_pack(const uint8_t *codes, uint32_t *planes, int B, int H, int W, int C, int cpad, int bits, int win,
                   int stride, int pad, apnn_stream_t s);

/* Packed codes -> int8: out[r][c] = min(127, (sum_{j<group} code[r*group+j][c]) >> shift).
 * group = 1, shift = 0 unpacks (inverse of the packer, cf. UnpackConvOutput32, NN/param.h:634-658);
 * group = H*W pools a feature map globally.  planes:[bits][rows_out*group][cpad/32]. */
int apnn_unpack_sum(const uint32_t *planes, int8_t *out, long long rows_out, int group, int C, int cpad, int bits,
                    int shift, apnn_stream_t s);

/* int8 classifier with a float affine output, out[b][n] = scale[n]*sum_k X[b][k]*Wt[n][k] + bias[n]
 * (the output layer's  val*bn_scale + bn_bias, NN/kernel.cuh:437-441).  acc_out (optional) receives
 * the int32 sums. */
int apnn_fc_i8(const int8_t *X, const int8_t *Wt, const float *scale, const float *bias, float *out,
               int32_t *acc_out, int B, int N, int K, apnn_stream_t s);

/* Device-side error report.  The reference's kernels have no error path at all (checkKernelErrors aborts
 * on a failed launch only, APNN-TC-lib/bmmaTensorCoreGemm/src/71_bmmaTensorCoreGemm.cu:65-75); here a
 * kernel that finds a launch it cannot serve (today: a tile of the patch-resident convolution whose input
 * patch exceeds the capacity the host computed) leaves that tile unwritten and ORs a code into one error
 * word per device.  This call waits for `stream`, copies the current device's word to *code (0 = no
 * kernel reported anything since the last call) and clears it.  It synchronizes: call it where a
 * host-side check of finished work belongs, not between launches of a latency-critical sequence. */
#define APNN_DEVERR_PATCH_CAPACITY 1
int apnn_device_error(int *code, apnn_stream_t stream);

/* Library / device information: number of compute units of the current device (0 if none). */
int apnn_device_cus(void);
const char *apnn_version(void);

#ifdef __cplusplus
}
#endif
#endif
