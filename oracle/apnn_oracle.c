/*
 * CPU oracle (test infrastructure, never part of the shipped library) -- see apnn_oracle.h.
 * Plain scalar C; the only "intrinsic" is __builtin_popcountll.  OpenMP is used solely to spread
 * independent output rows over host threads when a caller asks for more than one thread.
 */
#include "apnn_oracle.h"

#include <stdlib.h>
#include <math.h>
#include <string.h>

/* ---------------------------------------------------------------------------------------- */
/* literal tier: the reference's own loop nests                                              */
/* ---------------------------------------------------------------------------------------- */

/* LIB/71:337-348 */
static int int_pow2(int exp) {
  int result = 1, base = 2;
  while (exp) {
    if (exp % 2) result *= base;
    exp /= 2;
    base *= base;
  }
  return result;
}

/* LIB/71:350-376 */
void oracle_gemm_literal(const uint32_t *W, const uint32_t *X, int32_t *D,
                         int M, int N, int K, int wb, int xb) {
  const int K32 = K / 32;
  for (int m = 0; m < M; m++) {
    for (int n = 0; n < N; n++) {
      int tmp = 0;
      for (int ib = 0; ib < xb; ib++) {
        const int xmul = int_pow2(ib);
        for (int jb = 0; jb < wb; jb++) {
          const int wmul = int_pow2(jb);
          for (int kt = 0; kt < K32; kt++) {
            const uint32_t w = W[(size_t)jb * M * K32 + (size_t)m * K32 + kt];
            const uint32_t x = X[(size_t)ib * N * K32 + (size_t)n * K32 + kt];
            for (int k = 0; k < 32; k++) {
              const int xv = (int)((x >> k) & 1u);
              const int wv = (int)((w >> k) & 1u);
              tmp += xmul * wmul * xv * wv;
            }
          }
        }
      }
      D[(size_t)m * N + n] = tmp;
    }
  }
}

/* LIB/51:380-415 == LIB/67h:378-413 */
void oracle_conv3x3_literal(const uint32_t *Wt, const uint32_t *X, int32_t *O,
                            int H, int Wd, int CIN, int COUT, int wb, int xb) {
  const int C32 = CIN / 32;
  for (int co = 0; co < COUT; co++) {
    for (int m = 0; m < H; m++) {
      for (int n = 0; n < Wd; n++) {
        int tmp = 0;
        for (int ib = 0; ib < xb; ib++) {
          const int xmul = int_pow2(ib);
          for (int jb = 0; jb < wb; jb++) {
            const int wmul = int_pow2(jb);
            for (int i = 0; i < 3; i++) {
              for (int j = 0; j < 3; j++) {
                for (int kt = 0; kt < C32; kt++) {
                  const uint32_t x = X[(size_t)ib * (H + 2) * (Wd + 2) * C32 +
                                       (size_t)(m + i) * (Wd + 2) * C32 + (size_t)(n + j) * C32 + kt];
                  const uint32_t w = Wt[(size_t)jb * COUT * 9 * C32 + (size_t)co * 9 * C32 +
                                        (size_t)i * 3 * C32 + (size_t)j * C32 + kt];
                  for (int k = 0; k < 32; k++) {
                    const int xv = (int)((x >> k) & 1u);
                    const int wv = (int)((w >> k) & 1u);
                    tmp += xmul * wmul * xv * wv;
                  }
                }
              }
            }
          }
        }
        O[(size_t)m * Wd * COUT + (size_t)n * COUT + co] = tmp;
      }
    }
  }
}

/* ---------------------------------------------------------------------------------------- */
/* word tier                                                                                 */
/* ---------------------------------------------------------------------------------------- */

static inline int popc32(uint32_t v) { return __builtin_popcountll((unsigned long long)v); }

/* dot of one X row (xb planes) with one W row (wb planes) over nwords words.
 * xs / ws: word stride between planes. */
static inline int64_t plane_dot(const uint32_t *x, size_t xs, int xb,
                                const uint32_t *w, size_t ws, int wb, int nwords) {
  int64_t acc = 0;
  for (int ib = 0; ib < xb; ib++) {
    for (int jb = 0; jb < wb; jb++) {
      const uint32_t *xp = x + (size_t)ib * xs;
      const uint32_t *wp = w + (size_t)jb * ws;
      int cnt = 0;
      for (int t = 0; t < nwords; t++) cnt += popc32(xp[t] & wp[t]);
      acc += (int64_t)cnt << (ib + jb);
    }
  }
  return acc;
}

/* sum_k x_k  (value of the activation row) over nwords words */
static inline int64_t plane_sum(const uint32_t *x, size_t xs, int xb, int nwords) {
  int64_t acc = 0;
  for (int ib = 0; ib < xb; ib++) {
    const uint32_t *xp = x + (size_t)ib * xs;
    int cnt = 0;
    for (int t = 0; t < nwords; t++) cnt += popc32(xp[t]);
    acc += (int64_t)cnt << ib;
  }
  return acc;
}

void oracle_gemm_rows(const uint32_t *W, const uint32_t *X, int32_t *D,
                      int M, int N, int K, int wb, int xb, int sym_w, int m0, int m1, int nthreads) {
  const int K32 = K / 32;
  const size_t ws = (size_t)M * K32, xs = (size_t)N * K32;
  const int wmax = (1 << wb) - 1;
  if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
  for (int m = m0; m < m1; m++) {
    for (int n = 0; n < N; n++) {
      const uint32_t *xr = X + (size_t)n * K32;
      const uint32_t *wr = W + (size_t)m * K32;
      int64_t v = plane_dot(xr, xs, xb, wr, ws, wb, K32);
      /* sum x*(2u - wmax) = 2*sum x*u - wmax*sum x */
      if (sym_w) v = 2 * v - (int64_t)wmax * plane_sum(xr, xs, xb, K32);
      D[(size_t)m * N + n] = (int32_t)v;
    }
  }
}

void oracle_gemm(const uint32_t *W, const uint32_t *X, int32_t *D,
                 int M, int N, int K, int wb, int xb, int sym_w, int nthreads) {
  oracle_gemm_rows(W, X, D, M, N, K, wb, xb, sym_w, 0, M, nthreads);
}

int oracle_conv_out_h(const oracle_conv_geom *g) { return (g->H + 2 * g->pad - g->R) / g->stride + 1; }
int oracle_conv_out_w(const oracle_conv_geom *g) { return (g->W + 2 * g->pad - g->S) / g->stride + 1; }

void oracle_conv(const uint32_t *Wt, const uint32_t *X, int32_t *O,
                 const oracle_conv_geom *g, int nthreads) {
  const int Ho = oracle_conv_out_h(g), Wo = oracle_conv_out_w(g);
  const int cw = g->cwords;
  const int Hs = g->H + (g->halo ? 2 * g->pad : 0);
  const int Ws = g->W + (g->halo ? 2 * g->pad : 0);
  const size_t xs = (size_t)g->batch * Hs * Ws * cw;        /* X plane stride */
  const size_t ws = (size_t)g->cout * g->R * g->S * cw;     /* W plane stride */
  const int wmax = (1 << g->wb) - 1;
  if (nthreads < 1) nthreads = 1;
  const long npix = (long)g->batch * Ho * Wo;
#pragma omp parallel for num_threads(nthreads) schedule(static)
  for (long p = 0; p < npix; p++) {
    const int b = (int)(p / ((long)Ho * Wo));
    const int oy = (int)((p / Wo) % Ho);
    const int ox = (int)(p % Wo);
    for (int co = 0; co < g->cout; co++) {
      int64_t v = 0, sx = 0;
      for (int r = 0; r < g->R; r++) {
        for (int s = 0; s < g->S; s++) {
          int iy = oy * g->stride + r, ix = ox * g->stride + s; /* coordinates in the padded frame */
          if (!g->halo) {
            iy -= g->pad;
            ix -= g->pad;
            if (iy < 0 || iy >= g->H || ix < 0 || ix >= g->W) continue; /* zero tap */
          }
          const uint32_t *xr = X + (((size_t)b * Hs + iy) * Ws + ix) * cw;
          const uint32_t *wr = Wt + (((size_t)co * g->R + r) * g->S + s) * cw;
          v += plane_dot(xr, xs, g->xb, wr, ws, g->wb, cw);
          if (g->sym_w) sx += plane_sum(xr, xs, g->xb, cw);
        }
      }
      if (g->sym_w) v = 2 * v - (int64_t)wmax * sx;
      O[(size_t)p * g->cout + co] = (int32_t)v;
    }
  }
}

/* ---------------------------------------------------------------------------------------- */
/* epilogues                                                                                 */
/* ---------------------------------------------------------------------------------------- */

/* LIB/66h:390-407: val = (val << 1) | bit b of acc, 32 columns per word, plane stride rows*cols/32 */
void oracle_lowbits_pack(const int32_t *acc, uint32_t *out, int rows, int cols, int out_bit) {
  const int cw = cols / 32;
  for (int r = 0; r < rows; r++) {
    for (int t = 0; t < cw; t++) {
      for (int b = 0; b < out_bit; b++) {
        uint32_t val = 0;
        for (int c = 0; c < 32; c++) {
          const uint32_t a = (uint32_t)acc[(size_t)r * cols + t * 32 + c];
          val = (val << 1) | ((a >> b) & 1u);
        }
        out[(size_t)b * rows * cw + (size_t)r * cw + t] = val;
      }
    }
  }
}

/* LIB/68:524-539 */
void oracle_avgpool2x2(const int32_t *in, int32_t *out, int B, int H, int Wd, int C) {
  const int hh = H / 2, hw = Wd / 2;
  for (int b = 0; b < B; b++)
    for (int m = 0; m < hh; m++)
      for (int n = 0; n < hw; n++)
        for (int c = 0; c < C; c++) {
          const int32_t *base = in + (size_t)b * H * Wd * C;
          const int v1 = base[((size_t)(2 * m) * Wd + 2 * n) * C + c];
          const int v2 = base[((size_t)(2 * m) * Wd + 2 * n + 1) * C + c];
          const int v3 = base[((size_t)(2 * m + 1) * Wd + 2 * n) * C + c];
          const int v4 = base[((size_t)(2 * m + 1) * Wd + 2 * n + 1) * C + c];
          out[(((size_t)b * hh + m) * hw + n) * C + c] = (v1 + v2 + v3 + v4) / 4;
        }
}

void oracle_maxpool2x2(const int32_t *in, int32_t *out, int B, int H, int Wd, int C) {
  const int hh = H / 2, hw = Wd / 2;
  for (int b = 0; b < B; b++)
    for (int m = 0; m < hh; m++)
      for (int n = 0; n < hw; n++)
        for (int c = 0; c < C; c++) {
          const int32_t *base = in + (size_t)b * H * Wd * C;
          int v = base[((size_t)(2 * m) * Wd + 2 * n) * C + c];
          const int v2 = base[((size_t)(2 * m) * Wd + 2 * n + 1) * C + c];
          const int v3 = base[((size_t)(2 * m + 1) * Wd + 2 * n) * C + c];
          const int v4 = base[((size_t)(2 * m + 1) * Wd + 2 * n + 1) * C + c];
          if (v2 > v) v = v2;
          if (v3 > v) v = v3;
          if (v4 > v) v = v4;
          out[(((size_t)b * hh + m) * hw + n) * C + c] = v;
        }
}

void oracle_bn_quantize(const int32_t *acc, const int32_t *resid, const int32_t *thr,
                        const uint8_t *flip, int32_t *q, int rows, int C, int abits) {
  const int nt = (1 << abits) - 1;
  for (int r = 0; r < rows; r++)
    for (int c = 0; c < C; c++) {
      int64_t v = acc[(size_t)r * C + c];
      if (resid) v += resid[(size_t)r * C + c];
      if (flip && flip[c]) v = -v;
      int code = 0;
      for (int k = 0; k < nt; k++) code += (v >= (int64_t)thr[(size_t)c * nt + k]) ? 1 : 0;
      q[(size_t)r * C + c] = code;
    }
}

/* NN/kernel.cuh:58-76: lane l of a 32-wide group supplies bit 31-l (brev of the ballot),
 * row stride PAD(C)/32 words, plane stride rows*PAD(C)/32 words. */
void oracle_pack_bits(const uint32_t *values, uint32_t *planes, int rows, int C, int cpad, int bits) {
  const int cw = cpad / 32;
  memset(planes, 0, (size_t)bits * rows * cw * sizeof(uint32_t));
  for (int b = 0; b < bits; b++)
    for (int r = 0; r < rows; r++)
      for (int c = 0; c < C; c++) {
        const uint32_t bit = (values[(size_t)r * C + c] >> b) & 1u;
        planes[(size_t)b * rows * cw + (size_t)r * cw + c / 32] |= bit << (31 - (c % 32));
      }
}

void oracle_quantize_val(const float *x, uint32_t *q, long long n, int bits, float min_v, float max_v) {
  const uint32_t top = (1u << bits) - 1u;
  const float levels = (float)(1 << bits), range = max_v - min_v;
  for (long long i = 0; i < n; i++) {
    float v = x[i];
    v = v < min_v ? min_v : (v > max_v ? max_v : v);
    volatile float a = v - min_v;   /* volatile: one rounding per operation, as on the device */
    volatile float b = a * levels;
    volatile float c = b * 1.0f;
    volatile float d = c / range;
    const float r = rintf(d);       /* default rounding mode: to nearest, ties to even */
    const uint32_t code = (uint32_t)r;
    q[i] = code > top ? top : code;
  }
}

void oracle_unpack_bits(const uint32_t *planes, uint32_t *values, int rows, int C, int cpad, int bits) {
  const int cw = cpad / 32;
  for (int r = 0; r < rows; r++)
    for (int c = 0; c < C; c++) {
      uint32_t v = 0;
      for (int b = 0; b < bits; b++) {
        const uint32_t word = planes[(size_t)b * rows * cw + (size_t)r * cw + c / 32];
        v |= ((word >> (31 - (c % 32))) & 1u) << b;
      }
      values[(size_t)r * C + c] = v;
    }
}

/* ---------------------------------------------------------------------------------------- */
/* int8 edge layers                                                                          */
/* ---------------------------------------------------------------------------------------- */

void oracle_conv_i8(const int8_t *Wt, const int8_t *X, int32_t *O,
                    int B, int H, int Wd, int C, int cout, int R, int S, int stride, int pad) {
  const int Ho = (H + 2 * pad - R) / stride + 1, Wo = (Wd + 2 * pad - S) / stride + 1;
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < B; b++)
    for (int oy = 0; oy < Ho; oy++)
      for (int ox = 0; ox < Wo; ox++)
        for (int co = 0; co < cout; co++) {
          int32_t acc = 0;
          for (int r = 0; r < R; r++) {
            const int iy = oy * stride + r - pad;
            if (iy < 0 || iy >= H) continue;
            for (int s = 0; s < S; s++) {
              const int ix = ox * stride + s - pad;
              if (ix < 0 || ix >= Wd) continue;
              const int8_t *xp = X + (((size_t)b * H + iy) * Wd + ix) * C;
              const int8_t *wp = Wt + (((size_t)co * R + r) * S + s) * C;
              for (int c = 0; c < C; c++) acc += (int32_t)xp[c] * (int32_t)wp[c];
            }
          }
          O[(((size_t)b * Ho + oy) * Wo + ox) * cout + co] = acc;
        }
}

uint64_t oracle_fnv1a64(const void *data, uint64_t nbytes) {
  const uint8_t *p = (const uint8_t *)data;
  uint64_t h = 0xcbf29ce484222325ull;
  for (uint64_t i = 0; i < nbytes; i++) {
    h ^= p[i];
    h *= 0x100000001b3ull;
  }
  return h;
}
