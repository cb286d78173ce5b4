/* Sanitizer driver for the CPU oracle (test infrastructure, like the oracle itself).
 *
 * Built by `make -C oracle asan` with -fsanitize=address,undefined and run by the CPU test suite: every
 * oracle function is called on ragged / edge-case shapes with heap buffers of exactly the documented
 * size, so an out-of-bounds index, a shift past the word width or a signed overflow in the checker
 * itself aborts the run.  The two tiers of the GEMM / convolution oracle (literal per-bit loops following
 * APNN-TC-lib/bmmaTensorCoreGemm/src/71_bmmaTensorCoreGemm.cu:350-376 and 51_bmmaTensorCoreGemm.cu:380-415,
 * and the word-popcount tier) are also compared with each other here.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "apnn_oracle.h"

static uint64_t rng_state = 0x5EED5EEDull;
static uint32_t rnd(void) { /* splitmix64 */
  uint64_t z = (rng_state += 0x9e3779b97f4a7c15ull);
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return (uint32_t)((z ^ (z >> 31)) >> 16);
}

static uint32_t *rand_words(size_t n) {
  uint32_t *p = malloc(n * sizeof *p + (n == 0));
  for (size_t i = 0; i < n; i++) p[i] = rnd() ^ (rnd() << 16);
  return p;
}

static int fails = 0;
#define CHECK(cond, what)                                   \
  do {                                                      \
    if (!(cond)) {                                          \
      fprintf(stderr, "asan_driver: %s failed\n", what);    \
      fails++;                                              \
    }                                                       \
  } while (0)

static void gemm_cases(void) {
  const int shapes[][3] = {{1, 1, 128}, {3, 5, 256}, {17, 33, 128}, {64, 32, 384}};
  const int bits[][2] = {{1, 2}, {1, 3}, {1, 4}, {2, 2}, {8, 8}, {3, 5}};
  for (unsigned s = 0; s < sizeof shapes / sizeof shapes[0]; s++)
    for (unsigned b = 0; b < sizeof bits / sizeof bits[0]; b++) {
      const int M = shapes[s][0], N = shapes[s][1], K = shapes[s][2], wb = bits[b][0], xb = bits[b][1];
      uint32_t *W = rand_words((size_t)wb * M * K / 32), *X = rand_words((size_t)xb * N * K / 32);
      int32_t *D0 = malloc(sizeof(int32_t) * M * N), *D1 = malloc(sizeof(int32_t) * M * N);
      int32_t *D2 = calloc((size_t)M * N, sizeof(int32_t));
      oracle_gemm_literal(W, X, D0, M, N, K, wb, xb);
      oracle_gemm(W, X, D1, M, N, K, wb, xb, 0, 1);
      CHECK(memcmp(D0, D1, sizeof(int32_t) * M * N) == 0, "gemm literal == word tier");
      oracle_gemm(W, X, D1, M, N, K, wb, xb, 0, 3);
      CHECK(memcmp(D0, D1, sizeof(int32_t) * M * N) == 0, "gemm threaded == literal");
      oracle_gemm_rows(W, X, D2, M, N, K, wb, xb, 0, M - 1, M, 2);
      CHECK(memcmp(D0 + (size_t)(M - 1) * N, D2 + (size_t)(M - 1) * N, sizeof(int32_t) * N) == 0, "gemm_rows last row");
      oracle_gemm(W, X, D1, M, N, K, wb, xb, 1, 2); /* symmetric weights: exercised for UB only */
      free(W), free(X), free(D0), free(D1), free(D2);
    }
}

static void conv_cases(void) {
  /* literal 3x3 (halo stored) against the general routine */
  const int H = 5, Wd = 7, CIN = 128, COUT = 33;
  for (int wb = 1; wb <= 2; wb++)
    for (int xb = 2; xb <= 4; xb += 2) {
      uint32_t *X = rand_words((size_t)xb * (H + 2) * (Wd + 2) * CIN / 32);
      uint32_t *Wt = rand_words((size_t)wb * COUT * 9 * CIN / 32);
      int32_t *O0 = malloc(sizeof(int32_t) * H * Wd * COUT), *O1 = malloc(sizeof(int32_t) * H * Wd * COUT);
      oracle_conv3x3_literal(Wt, X, O0, H, Wd, CIN, COUT, wb, xb);
      oracle_conv_geom g = {1, H, Wd, CIN / 32, COUT, 3, 3, 1, 1, 1, wb, xb, 0};
      CHECK(oracle_conv_out_h(&g) == H && oracle_conv_out_w(&g) == Wd, "conv output size");
      oracle_conv(Wt, X, O1, &g, 2);
      CHECK(memcmp(O0, O1, sizeof(int32_t) * H * Wd * COUT) == 0, "conv literal == general");
      free(X), free(Wt), free(O0), free(O1);
    }
  /* general geometries: stride, zero padding, 1x1, 5x5, odd sizes, one stored word per pixel */
  const oracle_conv_geom gs[] = {
      {2, 7, 9, 1, 5, 3, 3, 2, 1, 0, 1, 2, 1}, {3, 4, 4, 2, 8, 1, 1, 2, 0, 0, 2, 2, 0},
      {1, 6, 5, 1, 3, 5, 5, 1, 2, 0, 1, 3, 1}, {2, 3, 3, 4, 7, 3, 3, 1, 1, 1, 1, 4, 0},
      {4, 2, 2, 3, 9, 2, 2, 1, 0, 0, 3, 5, 1},
  };
  for (unsigned i = 0; i < sizeof gs / sizeof gs[0]; i++) {
    const oracle_conv_geom *g = &gs[i];
    const int Hs = g->H + (g->halo ? 2 * g->pad : 0), Ws = g->W + (g->halo ? 2 * g->pad : 0);
    const int Ho = oracle_conv_out_h(g), Wo = oracle_conv_out_w(g);
    uint32_t *X = rand_words((size_t)g->xb * g->batch * Hs * Ws * g->cwords);
    uint32_t *Wt = rand_words((size_t)g->wb * g->cout * g->R * g->S * g->cwords);
    int32_t *O = malloc(sizeof(int32_t) * g->batch * Ho * Wo * g->cout);
    oracle_conv(Wt, X, O, g, 1);
    free(X), free(Wt), free(O);
  }
}

static void epilogue_cases(void) {
  const int rows = 6, cols = 96;
  int32_t *acc = malloc(sizeof(int32_t) * rows * cols);
  for (int i = 0; i < rows * cols; i++) acc[i] = (int32_t)(rnd() % 4001) - 2000;
  for (int ob = 1; ob <= 8; ob++) {
    uint32_t *out = malloc(sizeof(uint32_t) * ob * rows * cols / 32);
    oracle_lowbits_pack(acc, out, rows, cols, ob);
    free(out);
    const int nt = (1 << ob) - 1;
    int32_t *thr = malloc(sizeof(int32_t) * cols * nt), *q = malloc(sizeof(int32_t) * rows * cols);
    uint8_t *flip = malloc(cols);
    for (int c = 0; c < cols; c++) {
      flip[c] = (uint8_t)(rnd() & 1);
      int32_t t = -2000;
      for (int k = 0; k < nt; k++) thr[c * nt + k] = (t += (int32_t)(rnd() % 40));
    }
    thr[0] = INT32_MIN, thr[nt - 1] = nt > 1 ? INT32_MAX : thr[0]; /* extreme thresholds: -v must not overflow */
    oracle_bn_quantize(acc, NULL, thr, flip, q, rows, cols, ob);
    for (int i = 0; i < rows * cols; i++) CHECK(q[i] >= 0 && q[i] <= nt, "bn_quantize range");
    oracle_bn_quantize(acc, acc, thr, NULL, q, rows, cols, ob);
    free(thr), free(q), free(flip);
  }
  /* pooling on a 2 x 4 x 6 x 5 tensor */
  int32_t *in = malloc(sizeof(int32_t) * 2 * 4 * 6 * 5), *po = malloc(sizeof(int32_t) * 2 * 2 * 3 * 5);
  for (int i = 0; i < 2 * 4 * 6 * 5; i++) in[i] = (int32_t)(rnd() % 1000);
  oracle_avgpool2x2(in, po, 2, 4, 6, 5);
  oracle_maxpool2x2(in, po, 2, 4, 6, 5);
  free(in), free(po), free(acc);
}

static void packer_cases(void) {
  const int cs[][4] = {{5, 3, 32, 2}, {7, 70, 128, 3}, {2, 64, 64, 8}, {3, 100, 128, 1}, {1, 33, 64, 16}};
  for (unsigned i = 0; i < sizeof cs / sizeof cs[0]; i++) {
    const int rows = cs[i][0], C = cs[i][1], cpad = cs[i][2], bits = cs[i][3];
    uint32_t *v = malloc(sizeof(uint32_t) * rows * C), *back = malloc(sizeof(uint32_t) * rows * C);
    for (int k = 0; k < rows * C; k++) v[k] = rnd() & ((1u << bits) - 1);
    uint32_t *planes = malloc(sizeof(uint32_t) * bits * rows * cpad / 32);
    oracle_pack_bits(v, planes, rows, C, cpad, bits);
    oracle_unpack_bits(planes, back, rows, C, cpad, bits);
    CHECK(memcmp(v, back, sizeof(uint32_t) * rows * C) == 0, "pack / unpack round trip");
    free(v), free(back), free(planes);
  }
  float x[9] = {-1e30f, -10.f, -9.99f, 0.f, 3.3f, 9.99f, 10.f, 1e30f, -0.f};
  uint32_t q[9];
  for (int bits = 1; bits <= 16; bits++) {
    oracle_quantize_val(x, q, 9, bits, -10.f, 10.f);
    for (int k = 0; k < 9; k++) CHECK(q[k] < (1u << bits), "quantize_val range");
  }
}

static void int8_cases(void) {
  const int B = 2, H = 9, Wd = 7, C = 3, cout = 5;
  const int geo[][4] = {{7, 7, 2, 3}, {3, 3, 1, 1}, {5, 5, 4, 0}, {1, 1, 1, 0}};
  int8_t *X = malloc((size_t)B * H * Wd * C);
  for (int i = 0; i < B * H * Wd * C; i++) X[i] = (int8_t)(rnd() & 0xff);
  for (unsigned i = 0; i < sizeof geo / sizeof geo[0]; i++) {
    const int R = geo[i][0], S = geo[i][1], st = geo[i][2], pad = geo[i][3];
    const int Ho = (H + 2 * pad - R) / st + 1, Wo = (Wd + 2 * pad - S) / st + 1;
    int8_t *Wt = malloc((size_t)cout * R * S * C);
    for (int k = 0; k < cout * R * S * C; k++) Wt[k] = (int8_t)(rnd() & 0xff);
    int32_t *O = malloc(sizeof(int32_t) * B * Ho * Wo * cout);
    oracle_conv_i8(Wt, X, O, B, H, Wd, C, cout, R, S, st, pad);
    free(Wt), free(O);
  }
  free(X);
  CHECK(oracle_fnv1a64("a", 1) == 0xaf63dc4c8601ec8cull, "fnv1a64 test vector");
}

int main(void) {
  gemm_cases();
  conv_cases();
  epilogue_cases();
  packer_cases();
  int8_cases();
  if (fails) return 1;
  puts("asan_driver: ok");
  return 0;
}
