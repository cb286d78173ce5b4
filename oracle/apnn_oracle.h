/*
 * CPU oracle for the arbitrary-precision (wXaY) bit-plane GEMM / convolution path.
 *
 * THIS IS TEST INFRASTRUCTURE.  Nothing in the shipped library links, loads or calls it;
 * only the test-suite, the smoke check and the benchmark's cpu_baseline leg do, and there
 * only as the checker.
 *
 * It restates, in plain scalar C, the CPU reference functions that live next to the CUDA
 * kernels of the reference (paths relative to the reference checkout):
 *   LIB = APNN-TC-lib/bmmaTensorCoreGemm/src,  NN = APNN-TC-nn/src
 *
 * Conventions shared by every function (LIB/71_bmmaTensorCoreGemm.cu:350-376):
 *   - operands are bit-planes stored plane-major, LSB plane first, as uint32 words;
 *     element k of a row lives in word k/32 and bit k of the W row pairs with bit k of the X row;
 *   - result = sum_i sum_j 2^(i+j) * popcount(X_i & W_j);
 *   - produced (packed) outputs are MSB-first: column c sits at bit 31 - c%32
 *     (LIB/66_bmmaTensorCoreGemm.cuh:390-407).
 *
 * Pinning status (which independent evidence each function is checked against in tests/):
 *   gemm_literal / gemm            reference-derived known answers (glibc rand() inputs, checksums
 *                                  recorded from the reference's compute_ref), closed forms,
 *                                  numpy int64 matmul of the unpacked operands            : pinned
 *   conv3x3_literal / conv         same known answers for conv, scipy/numpy cross-correlation,
 *                                  1x1 filter == GEMM                                      : pinned
 *   lowbits_pack                   known answers (pack[0], fnv of packed planes)           : pinned
 *   avgpool2x2                     brute force on the unpacked tensor; no stored reference answer
 *                                  exists for the pooled variant                           : pinned by arithmetic only
 *   signed (+-1 / symmetric) mode  integer matmul/conv with the signed weight values       : pinned
 *   bn_quantize                    a=1 special case == (acc >= t) of NN/kernel.cuh:833-834;
 *                                  multi-bit form is defined by this build                 : parity unpinned beyond a=1
 *   pack_bits                      round trip + hand-written words (NN/kernel.cuh:58-76)   : pinned
 *   quantize_val                   end points, exact levels, ties-to-even, monotonicity and an
 *                                  independent numpy float32 evaluation (NN/kernel.cuh:29-44; the
 *                                  reference never stores its result, so no reference output exists) : pinned by arithmetic only
 */
#ifndef APNN_ORACLE_H
#define APNN_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- GEMM -------------------------------------------------------------------------------- */

/* Literal per-bit loops, same loop nest and indexing as compute_ref, LIB/71:350-376.
 * W: [wb][M][K/32], X: [xb][N][K/32], D: [M][N] int32. */
void oracle_gemm_literal(const uint32_t *W, const uint32_t *X, int32_t *D,
                         int M, int N, int K, int wb, int xb);

/* Same result by word-wise AND + popcount.  nthreads<=1: single thread.
 * sym_w != 0: weights are symmetric integers wt = 2u - (2^wb - 1), u the unsigned plane value
 * (for wb=1: wt = 2b-1); evaluated as 2*raw - (2^wb-1)*sum_k x_k and cross-checked in the tests
 * against an integer matmul of the signed weight values. */
void oracle_gemm(const uint32_t *W, const uint32_t *X, int32_t *D,
                 int M, int N, int K, int wb, int xb, int sym_w, int nthreads);

/* Rows [m0, m1) only (used to sample big shapes). D still indexed [m][N] from row 0. */
void oracle_gemm_rows(const uint32_t *W, const uint32_t *X, int32_t *D,
                      int M, int N, int K, int wb, int xb, int sym_w, int m0, int m1, int nthreads);

/* ---- convolution ------------------------------------------------------------------------- */

/* Literal 3x3 / stride 1 / halo-stored convolution, loop nest of compute_ref, LIB/51:380-415
 * (same text at LIB/67_bmmaTensorCoreGemm.cuh:378-413).
 * X: [xb][H+2][W+2][CIN/32], Wt: [wb][COUT][3][3][CIN/32], O: [H][W][COUT]. */
void oracle_conv3x3_literal(const uint32_t *Wt, const uint32_t *X, int32_t *O,
                            int H, int Wd, int CIN, int COUT, int wb, int xb);

typedef struct {
  int batch;       /* images */
  int H, W;        /* logical input height / width (without halo) */
  int cwords;      /* uint32 words per pixel per plane (channels padded / 32) */
  int cout;
  int R, S;        /* filter height / width */
  int stride;
  int pad;         /* logical zero padding on each side */
  int halo;        /* 1: X is stored with a halo of `pad` pixels per image whose contents take part
                         in the sum (the reference's layout, LIB/51:395); 0: X stored unpadded and
                         out-of-image taps contribute zero */
  int wb, xb;
  int sym_w;       /* symmetric weights, as oracle_gemm */
} oracle_conv_geom;

int oracle_conv_out_h(const oracle_conv_geom *g);
int oracle_conv_out_w(const oracle_conv_geom *g);

/* General convolution by word popcount.
 * X: [xb][batch][Hs][Ws][cwords] with Hs = H + (halo ? 2*pad : 0); Wt: [wb][cout][R][S][cwords];
 * O: [batch][Hout][Wout][cout] int32. */
void oracle_conv(const uint32_t *Wt, const uint32_t *X, int32_t *O,
                 const oracle_conv_geom *g, int nthreads);

/* ---- epilogues --------------------------------------------------------------------------- */

/* Low-bit extraction + MSB-first pack along the fast (column) index,
 * LIB/66h:390-407 (GEMM) and LIB/67h:459-480 (conv): out[b][r][cols/32], bit b of acc. */
void oracle_lowbits_pack(const int32_t *acc, uint32_t *out, int rows, int cols, int out_bit);

/* 2x2 average pooling of an NHWC int32 tensor with C integer division,
 * LIB/68_bmmaTensorCoreGemm.cu:524-539.  in: [B][H][W][C] -> out: [B][H/2][W/2][C]. */
void oracle_avgpool2x2(const int32_t *in, int32_t *out, int B, int H, int Wd, int C);

/* 2x2 max pooling of an NHWC int32 tensor (used on quantized codes). */
void oracle_maxpool2x2(const int32_t *in, int32_t *out, int B, int H, int Wd, int C);

/* Per-channel threshold quantizer.  v = acc[r][c] + (resid ? resid[r][c] : 0);
 * q[r][c] = #{ k < 2^abits-1 : (flip[c] ? -v : v) >= thr[c][k] }, thr rows non-decreasing.
 * abits = 1 reduces to the reference's  bit = !(res < bn[c])  (NN/kernel.cuh:833-834). */
void oracle_bn_quantize(const int32_t *acc, const int32_t *resid, const int32_t *thr,
                        const uint8_t *flip, int32_t *q, int rows, int C, int abits);

/* Bit-plane packer of NN/kernel.cuh:58-76 (Bit_compression): values [rows][C] (one unsigned code
 * per element) -> planes [bits][rows][cpad/32], channel c at bit 31 - c%32, pad channels zero. */
void oracle_pack_bits(const uint32_t *values, uint32_t *planes, int rows, int C, int cpad, int bits);

/* Affine quantizer of NN/kernel.cuh:29-44 (Quantize_val), fp32, same operation order, round half to
 * even, clamped to the top code: q = min(2^bits-1, rint(((clip(x)-min_v) * 2^bits * 1.0f) / (max_v-min_v))).
 * Pinned by closed forms (end points, exact mid-levels, monotonicity) and by an independent numpy
 * float32 evaluation in tests/test_oracle.py; the reference never stores this value (kernel.cuh:42). */
void oracle_quantize_val(const float *x, uint32_t *q, long long n, int bits, float min_v, float max_v);

/* Inverse of oracle_pack_bits (NN/param.h:634-658 shows the (r>>(31-lane))&1 indexing). */
void oracle_unpack_bits(const uint32_t *planes, uint32_t *values, int rows, int C, int cpad, int bits);

/* ---- int8 edge layers -------------------------------------------------------------------- */

/* int8 NHWC convolution with zero padding, int32 accumulate.
 * X: [B][H][W][C] int8, Wt: [cout][R][S][C] int8, O: [B][Hout][Wout][cout] int32. */
void oracle_conv_i8(const int8_t *Wt, const int8_t *X, int32_t *O,
                    int B, int H, int Wd, int C, int cout, int R, int S, int stride, int pad);

/* FNV-1a 64-bit over raw bytes (fixture checksums). */
uint64_t oracle_fnv1a64(const void *data, uint64_t nbytes);

#ifdef __cplusplus
}
#endif
#endif
