// Kernel-side problem description shared by the VALU and MFMA kernels and the host dispatcher.
//
// Every kernel computes  out[a][b] = sum_{i<PA} sum_{j<PB} 2^(i+j) popc(A_i[a] & B_j[b])  over KW
// 32-bit words, where A is the slow output index and B the fast (contiguous) one:
//   GEMM entry points : A = W rows (M),      B = X rows (N)
//   convolution / FC  : A = output pixels,   B = output channels (implicit im2col on A)
#pragma once
#include <stdint.h>

namespace apnn {

// TILE_DIRECT: the register-only kernel of valu_direct_kernel.h (GEMM entry points, int32 output)
enum TileSel { TILE_64x64 = 0, TILE_32x32 = 1, TILE_16x32 = 2, TILE_16x16 = 3, TILE_COUNT = 4, TILE_DIRECT = 4 };

struct KParams {
  const uint32_t *A;
  const uint32_t *B;
  int rowsA, rowsB;          // logical output size out[rowsA][rowsB]
  int KW;                    // reduction length in 32-bit words (GEMM: K/32, conv: R*S*C32)
  int planesA, planesB;      // bit-planes of A / B (read by the any-precision kernel instantiation only)
  long long planeA, planeB;  // plane strides in words

  // implicit im2col (convolution kernels only); halo-stored inputs are expressed as pad = 0 on the
  // stored frame
  int Hs, Ws;                // stored input height / width
  int C32;                   // words per pixel per plane
  int Ho, Wo;                // output height / width
  int S;                     // filter width (filter height = KW / (S*C32))
  int stride, pad;
  uint32_t magicC32, magicS; // ceil(2^32/d) for d >= 2 (unused when d == 1)
  int pool_order;            // 1: row index enumerates 2x2 output windows (4 consecutive rows each)

  // patch-resident convolution kernel only: padded frame (stored frame + pad on every side) and
  // the capacity of the LDS patch in pixels
  int batch, PHs, PWs, patch_cap;
  // ceil(2^32/d) for the row grid (Wo, Ho; in pool order Wo/2, Ho/2) and the padded frame (PWs, PHs):
  // exact quotients for dividends below d + 1024
  uint32_t magicGW, magicGH, magicPW, magicPH;
  // 1: every output row index times the larger of the row grid's sides stays below 2^32, so the
  // matrix-core kernels may decode a row index into (image, y, x) with magicGW / magicGH
  int geo_fast;
  // 1: the matrix-core kernels of mfma_kernel.h may run: every operand plane spans less than 2^32 bytes
  // (rows are addressed with 32-bit word offsets through buffer descriptors) and, for a convolution, the
  // filter is small enough for 24-bit index arithmetic: taps * S < 65536, so that (tap * magicS16) >> 16 ==
  // tap / S with magicS16 = ceil(65536 / S); stored width, C32 and KW below 2^24.
  // c32_shift: log2(C32) when C32 is a power of two, else -1.
  int addr32, c32_shift;
  // Matrix-core kernels, set by the launcher: 0, or the height (in tile rows) of the bands in which the
  // work-groups of one XCD walk the tile grid (see apnn_mfma_kernel's tile decode).
  int xcd_rows;
  uint32_t magicS16;

  // Paired launch (matrix-core convolution kernels only): work-groups pair_tiles .. 2*pair_tiles-1
  // compute a second convolution on the same input and output grid (same A, rows, columns, stride,
  // precisions, epilogue mode) that differs in filter, filter size, padding, thresholds and output:
  // the two branches of a residual block's entry (3x3 convolution and 1x1 downsample) in one launch.
  int pair_tiles;            // 0: single problem
  const uint32_t *B2;
  int KW2, S2, pad2;
  uint32_t magicS2, magicS16_2;
  long long planeB2;
  const int32_t *thr2;
  const uint8_t *flip2;
  void *out2;

  int sym;                   // symmetric weights: result = 2*raw - wmax * (activation row sum)
  int wmax;                  // 2^wb - 1

  int epi;                   // APNN_EPI_*
  int out_bits;
  int pool;                  // APNN_POOL_*
  const int32_t *thr;
  const uint8_t *flip;
  const int32_t *resid;
  int32_t *save_acc;
  const uint32_t *resid_planes;  // packed shortcut codes [resid_bits][rows][rowsB/32]
  int resid_bits, resid_scale;
  // 1: every value the quantizing epilogue compares (accumulator, correction, scaled shortcut code) is an
  // integer below 2^24 in magnitude, so the FP4 kernels may do the threshold compare in fp32
  int epi_float;
  // Shortcut add on the matrix cores (FP4 kernels, see fold_shortcut in mfma_kernel.h): resid_scale as the
  // sum of two terms +-{1, 3} * 2^j, each an FP4 value (sign and code in a nibble: bits 0-3 first term,
  // bits 4-7 second term, 0 = no term) times an E8M0 block scale (bits 8-15 and 16-23).  0: the shortcut is
  // added per value in the vector ALUs (scale not representable, fp32 would round, other core).
  uint32_t fold;
  void *out;
  long long out_plane;       // packed output: plane stride in words
  // Device error word of the current device (see apnn_device_error in apnn_tc.h): a kernel that meets a
  // launch it cannot serve ORs a KERR_* code into it before it leaves its tile unwritten.
  int *err;
};

enum KernelError { KERR_PATCH_CAPACITY = 1 };

}  // namespace apnn
