// Output stage shared by the VALU and MFMA kernels.
//
// Quantizing epilogues work from an int32 tile staged in LDS so that 64 consecutive output
// channels sit in the 64 lanes of a wave: one ballot per output bit-plane then yields two
// MSB-first 32-bit words (the wave64 counterpart of the reference's __brev(__ballot_sync()),
// APNN-TC-lib/bmmaTensorCoreGemm/src/66_bmmaTensorCoreGemm.cuh:255-276).
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>

#include "../../include/apnn_tc.h"
#include "kparams.h"

namespace apnn {

__device__ __forceinline__ int quantize_code(const KParams &p, int v, int gcol) {
  if (p.epi == APNN_EPI_LOWBITS) return v & ((1 << p.out_bits) - 1);
  const int nt = (1 << p.out_bits) - 1;
  if (p.flip != nullptr && p.flip[gcol]) v = -v;
  const int32_t *t = p.thr + (long long)gcol * nt;
  // the code is the number of thresholds <= v; the thresholds of a channel are sorted, so a binary
  // search over the 2^bits - 1 of them finds it with one load per output bit
  int code = 0;
  for (int h = (nt + 1) >> 1; h > 0; h >>= 1)
    if (v >= t[code + h - 1]) code += h;
  return code;
}

// shortcut contribution of a packed residual branch for output element (grow, gcol)
__device__ __forceinline__ int packed_residual(const KParams &p, int grow, int gcol) {
  const int w32 = p.rowsB >> 5;
  const long long plane = (long long)p.rowsA * w32;
  const long long wi = (long long)grow * w32 + (gcol >> 5);
  const int sh = 31 - (gcol & 31);
  int code = 0;
  for (int b = 0; b < p.resid_bits; ++b) code |= (int)((p.resid_planes[b * plane + wi] >> sh) & 1u) << b;
  return code * p.resid_scale;
}

// Per-lane view of the quantizer of one output channel: thresholds (and flip) are fetched once,
// not once per output row.
struct ChannelQuant {
  int t0, t1, t2;   // thresholds when there are at most three (out_bits <= 2)
  bool flip;
  bool in_regs;
};

__device__ __forceinline__ ChannelQuant load_channel_quant(const KParams &p, int gcol, bool col_ok) {
  ChannelQuant q{0, 0, 0, false, false};
  if (p.epi != APNN_EPI_BN || !col_ok) return q;
  q.flip = p.flip != nullptr && p.flip[gcol] != 0;
  const int nt = (1 << p.out_bits) - 1;
  if (nt <= 3) {
    const int32_t *t = p.thr + (long long)gcol * nt;
    q.t0 = t[0];
    q.t1 = nt > 1 ? t[1] : 0x7fffffff;
    q.t2 = nt > 2 ? t[2] : 0x7fffffff;
    q.in_regs = true;
  }
  return q;
}

__device__ __forceinline__ int quantize_with(const KParams &p, const ChannelQuant &q, int v, int gcol) {
  if (p.epi == APNN_EPI_LOWBITS) return v & ((1 << p.out_bits) - 1);
  if (!q.in_regs) return quantize_code(p, v, gcol);
  if (q.flip) v = -v;
  return (v >= q.t0 ? 1 : 0) + (v >= q.t1 ? 1 : 0) + (v >= q.t2 ? 1 : 0);
}

// Quantize-and-pack stage shared by all kernels.  `value(row, col)` returns the finished int32 sum
// of tile row `row`, tile column `col` (from LDS).  The tile has `n_rows` rows x NCOLS columns; with
// pooling, rows 4i..4i+3 are one 2x2 window.  Work is cut into units of 64 consecutive
// (row, column) elements -- one ballot per output bit gives two MSB-first words -- and this wave
// takes units part, part + nparts, ...  Units are processed four at a time: all global loads of a
// group (shortcut words, int32 residuals) are issued before any of them is consumed, so the loop
// pays one memory round trip per four units instead of one per unit.
//
// q0 / q1: quantizers of the (at most two) columns this lane meets, from load_tile_quant().
// res_lds: when not null, the shortcut words of the tile, [resid_bits][n_rows][NCOLS/32], already in
// LDS (fetched by the kernel before its K loop, so their latency is hidden); otherwise shortcut words
// are read from global memory inside the loop.
template <int NCOLS>
__device__ __forceinline__ void load_tile_quant(const KParams &p, int cbase, ChannelQuant &q0, ChannelQuant &q1) {
  const int col0 = (threadIdx.x & 63) % NCOLS;
  q0 = load_channel_quant(p, cbase + col0, cbase + col0 < p.rowsB);
  q1 = q0;
  if (NCOLS == 128) q1 = load_channel_quant(p, cbase + col0 + 64, cbase + col0 + 64 < p.rowsB);
}

// Shortcut words of a tile of n_rows x NCOLS outputs, two planes at most: word i of the tile is
// (plane b, row r, column word c) with i = (b * n_rows + r) * (NCOLS/32) + c, or, with ROWFAST,
// i = (b * (NCOLS/32) + c) * n_rows + r (four consecutive rows are then one 16-byte LDS read).
// prefetch: thread `t` of `nthreads` keeps words t, t + nthreads, ... in registers; publish: writes
// them to LDS.
template <int NCOLS, int NREGS, bool ROWFAST = false>
__device__ __forceinline__ void shortcut_prefetch(const KParams &p, int n_rows, int rbase, int cbase, int t,
                                                  int nthreads, uint32_t (&regs)[NREGS]) {
  constexpr int CW = NCOLS / 32;
  const int w32 = p.rowsB >> 5;
  const long long rplane = (long long)p.rowsA * w32;
  const int total = p.resid_bits * n_rows * CW;
#pragma unroll
  for (int j = 0; j < NREGS; ++j) {
    const int i = t + j * nthreads;
    uint32_t w = 0;
    if (i < total) {
      const int c = ROWFAST ? (i / n_rows) % CW : i % CW;
      const int r = ROWFAST ? i % n_rows : (i / CW) % n_rows;
      const int b = i / (CW * n_rows);
      const int grow = rbase + r, gw = (cbase >> 5) + c;
      if (grow < p.rowsA && gw < w32) w = p.resid_planes[b * rplane + (long long)grow * w32 + gw];
    }
    regs[j] = w;
  }
}

template <int NREGS>
__device__ __forceinline__ void shortcut_publish(uint32_t *res_lds, int t, int nthreads, const uint32_t (&regs)[NREGS]) {
#pragma unroll
  for (int j = 0; j < NREGS; ++j) res_lds[t + j * nthreads] = regs[j];
}

template <int NCOLS, class ValueFn>
__device__ __forceinline__ void pack_rows(const KParams &p, ValueFn value, int n_rows, int rbase, int cbase,
                                          int part, int nparts, const ChannelQuant &q0, const ChannelQuant &q1,
                                          const uint32_t *res_lds) {
  static_assert(NCOLS == 32 || NCOLS == 64 || NCOLS == 128, "tile width");
  constexpr int UB = 4;
  const int lane = threadIdx.x & 63;
  const bool pooled = p.pool != APNN_POOL_NONE;
  const int n_out = pooled ? n_rows / 4 : n_rows;
  const int out_rows_total = pooled ? p.rowsA / 4 : p.rowsA;
  const int row_base = pooled ? rbase / 4 : rbase;
  const int w32 = p.rowsB >> 5;
  const long long rplane = (long long)p.rowsA * w32;
  uint32_t *out = reinterpret_cast<uint32_t *>(p.out);
  const int nunits = n_out * NCOLS / 64;

  const bool res_global = p.resid_planes != nullptr && res_lds == nullptr;
  const bool res_local = p.resid_planes != nullptr && res_lds != nullptr;

  // Codes of three or four bits: a lane meets one channel (two when the tile is 128 wide), so its 7 or
  // 15 thresholds are fetched once into registers; the code is the number of thresholds <= v.
  constexpr int NCH = NCOLS == 128 ? 2 : 1;
  const bool wide = p.epi == APNN_EPI_BN && p.out_bits > 2 && p.out_bits <= 4;
  const int nt = (1 << p.out_bits) - 1;
  int tq[NCH][15];
  int tflip[NCH] = {};  // 0 or -1
  if (wide) {
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int gc = cbase + lane % NCOLS + 64 * c;
      const int32_t *t = p.thr + (long long)(gc < p.rowsB ? gc : 0) * nt;
#pragma unroll
      for (int k = 0; k < 15; ++k) tq[c][k] = t[k < nt ? k : nt - 1];
      tflip[c] = (p.flip != nullptr && gc < p.rowsB && p.flip[gc] != 0) ? -1 : 0;
    }
  }
  auto quant = [&](const ChannelQuant &q, int c, int v, int gc) {
    if (!wide) return quantize_with(p, q, v, gc);
    const int fm = (NCH == 2 && c) ? tflip[NCH - 1] : tflip[0];
    v = (v ^ fm) - fm;
    int code = 0;
#pragma unroll
    for (int k = 0; k < 7; ++k) code += (v >= (NCH == 2 && c ? tq[NCH - 1][k] : tq[0][k])) ? 1 : 0;
    if (nt > 7) {
#pragma unroll
      for (int k = 7; k < 15; ++k) code += (v >= (NCH == 2 && c ? tq[NCH - 1][k] : tq[0][k])) ? 1 : 0;
    }
    return code;
  };

  for (int u0 = part; u0 < nunits; u0 += nparts * UB) {
    int v[UB], grow[UB], gcol[UB];
    bool ok[UB];
    int ri[UB];
#pragma unroll
    for (int j = 0; j < UB; ++j) {
      const int e = (u0 + j * nparts) * 64 + lane;
      const int orow = e / NCOLS, col = e % NCOLS;
      grow[j] = row_base + orow;
      gcol[j] = cbase + col;
      ok[j] = (u0 + j * nparts) < nunits && grow[j] < out_rows_total && gcol[j] < p.rowsB;
      v[j] = 0;
      ri[j] = 0;
      if (ok[j] && !pooled) {
        const long long o = (long long)grow[j] * p.rowsB + gcol[j];
        if (p.resid != nullptr) ri[j] = p.resid[o];
      }
    }
#pragma unroll
    for (int j = 0; j < UB; ++j) {
      const int e = (u0 + j * nparts) * 64 + lane;
      const int orow = e / NCOLS, col = e % NCOLS;
      const ChannelQuant &q = (NCOLS == 128 && col >= 64) ? q1 : q0;
      const int ch = (NCOLS == 128 && col >= 64) ? 1 : 0;
      int code = 0;
      if (ok[j]) {
        if (!pooled) {
          int t = value(orow, col) + ri[j];
          if (res_global || res_local) {
            const int sh = 31 - (gcol[j] & 31);
            int rc = 0;
            // Shortcut words that were not brought to LDS before the K loop (codes wider than two bits)
            // are read here, one plane at a time.  They are not buffered in a per-lane array: indexed by
            // a run-time plane count it would live in scratch memory, and held in registers it would
            // spill at these kernels' register caps; this way most instantiations use no scratch at all.
            const long long wi = (long long)grow[j] * w32 + (gcol[j] >> 5);
            for (int b = 0; b < p.resid_bits; ++b) {
              uint32_t w = 0;
              if (res_local) w = res_lds[(b * n_rows + orow) * (NCOLS / 32) + (col >> 5)];
              if (res_global) w = p.resid_planes[b * rplane + wi];
              rc |= (int)((w >> sh) & 1u) << b;
            }
            t += rc * p.resid_scale;
          }
          if (p.save_acc != nullptr) p.save_acc[(long long)grow[j] * p.rowsB + gcol[j]] = t;
          code = quant(q, ch, t, gcol[j]);
        } else {
          const int t0 = value(4 * orow, col), t1 = value(4 * orow + 1, col);
          const int t2 = value(4 * orow + 2, col), t3 = value(4 * orow + 3, col);
          if (p.pool == APNN_POOL_AVG2X2) {
            code = quant(q, ch, (t0 + t1 + t2 + t3) / 4, gcol[j]);
          } else {
            code = max(max(quant(q, ch, t0, gcol[j]), quant(q, ch, t1, gcol[j])),
                       max(quant(q, ch, t2, gcol[j]), quant(q, ch, t3, gcol[j])));
          }
        }
      }
      for (int b = 0; b < p.out_bits; ++b) {
        const unsigned long long mask = __ballot(ok[j] && ((code >> b) & 1));
        const uint32_t word = (lane < 32) ? __brev((uint32_t)mask) : __brev((uint32_t)(mask >> 32));
        if (ok[j] && (lane & 31) == 0) out[b * p.out_plane + (long long)grow[j] * w32 + (gcol[j] >> 5)] = word;
      }
    }
  }
}

template <int I, int N, class F>
__device__ __forceinline__ void static_for_e(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for_e<I + 1, N>(f);
  }
}

// Burst version of pack_rows for the common case (at most two output bits, no int32 residual, no
// saved accumulator, shortcut words -- if any -- already in LDS).  Units are handled eight at a time
// with compile-time indices inside a group: the eight LDS gathers are issued back to back, the codes
// are computed in registers, and each packed word is parked in the lane whose index equals its
// output row; after the last group every lane stores its own row's words, one plane at a time.
// NR = tile rows, NPARTS waves share the tile (unit = u * NPARTS + part).
template <int NR, int NCOLS, int NPARTS, class ValueFn>
__device__ __forceinline__ void pack_rows_burst(const KParams &p, ValueFn value, int rbase, int cbase, int part,
                                                const ChannelQuant &q0, const ChannelQuant &q1,
                                                const uint32_t *res_lds) {
  static_assert(NCOLS == 32 || NCOLS == 64 || NCOLS == 128, "tile width");
  constexpr int CW = NCOLS / 32;
  constexpr int G = 8;
  const int lane = threadIdx.x & 63;
  const bool pooled = p.pool != APNN_POOL_NONE;
  const int n_out = pooled ? NR / 4 : NR;
  const int total = n_out * NCOLS / 64;  // units in the tile
  const int out_rows_total = pooled ? p.rowsA / 4 : p.rowsA;
  const int row_base = pooled ? rbase / 4 : rbase;
  const int w32 = p.rowsB >> 5;
  const bool shortcut = p.resid_planes != nullptr;
  uint32_t mine[2][CW];
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int c = 0; c < CW; ++c) mine[b][c] = 0;

#pragma unroll 1
  for (int u0 = 0; u0 * NPARTS < total; u0 += G) {
    int code[G];
    static_for_e<0, G>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      const int unit = (u0 + j) * NPARTS + part;
      const int e = unit * 64 + lane;
      const int orow = e / NCOLS, col = e % NCOLS;
      const int gcol = cbase + col;
      const ChannelQuant &q = (NCOLS == 128 && col >= 64) ? q1 : q0;
      int c = 0;
      if (unit < total) {
        if (!pooled) {
          int t = value(orow, col);
          if (shortcut) {
            const int sh = 31 - (gcol & 31);
            int rc = 0;
            for (int b = 0; b < p.resid_bits; ++b)
              rc |= (int)((res_lds[(b * NR + orow) * CW + (col >> 5)] >> sh) & 1u) << b;
            t += rc * p.resid_scale;
          }
          c = quantize_with(p, q, t, gcol);
        } else {
          const int t0 = value(4 * orow, col), t1 = value(4 * orow + 1, col);
          const int t2 = value(4 * orow + 2, col), t3 = value(4 * orow + 3, col);
          if (p.pool == APNN_POOL_AVG2X2) {
            c = quantize_with(p, q, (t0 + t1 + t2 + t3) / 4, gcol);
          } else {
            c = max(max(quantize_with(p, q, t0, gcol), quantize_with(p, q, t1, gcol)),
                    max(quantize_with(p, q, t2, gcol), quantize_with(p, q, t3, gcol)));
          }
        }
      }
      code[j] = c;
    });
    static_for_e<0, G>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      const int unit = (u0 + j) * NPARTS + part;  // out-of-range units have code 0 and match no lane below
      static_for_e<0, 2>([&](auto bc) {
        constexpr int b = decltype(bc)::value;
        const unsigned long long mask = __ballot((code[j] >> b) & 1);
        const uint32_t lo = __brev((uint32_t)mask), hi = __brev((uint32_t)(mask >> 32));
        // tile word index 2*unit + h  ->  row (2*unit + h) / CW, column word (2*unit + h) % CW
        if constexpr (CW == 1) {
          if (lane == 2 * unit) mine[b][0] = lo;
          if (lane == 2 * unit + 1) mine[b][0] = hi;
        } else if constexpr (CW == 2) {
          if (lane == unit) {
            mine[b][0] = lo;
            mine[b][1] = hi;
          }
        } else {
          if (lane == (unit >> 1)) {
            if (unit & 1) {
              mine[b][2] = lo;
              mine[b][3] = hi;
            } else {
              mine[b][0] = lo;
              mine[b][1] = hi;
            }
          }
        }
      });
    });
  }
  // lane r owns output row r of the tile, if that row belongs to one of this wave's units
  const int owner_unit = CW == 1 ? (lane >> 1) : CW == 2 ? lane : 2 * lane;
  const int grow = row_base + lane;
  if (lane < n_out && grow < out_rows_total && (owner_unit % NPARTS) == (NPARTS == 1 ? 0 : part)) {
    uint32_t *out = reinterpret_cast<uint32_t *>(p.out);
    for (int b = 0; b < p.out_bits; ++b) {
      uint32_t *dst = out + b * p.out_plane + (long long)grow * w32 + (cbase >> 5);
#pragma unroll
      for (int c = 0; c < CW; ++c)
        if ((cbase >> 5) + c < w32) dst[c] = b == 0 ? mine[0][c] : mine[1][c];
    }
  }
}

// tile: LDS, [TA][TB + 1] int32, row r of the tile is output row a0 + r (or, in pool order, rows
// 4i..4i+3 are the 2x2 window a0/4 + i).  Must be called by every thread of the block after a
// __syncthreads() that made the tile (and res_lds, if used) visible.
template <int TA, int TB>
__device__ __forceinline__ void epilogue_packed(const KParams &p, const int *tile, int a0, int b0,
                                                const ChannelQuant &q0, const ChannelQuant &q1,
                                                const uint32_t *res_lds) {
  static_assert(TB % 32 == 0, "packed epilogue needs whole 32-channel words per tile row");
  constexpr int LDT = TB + 1;
  auto value = [&](int row, int col) { return tile[row * LDT + col]; };
  if (p.out_bits <= 2 && p.resid == nullptr && p.save_acc == nullptr &&
      (p.resid_planes == nullptr || res_lds != nullptr)) {
    pack_rows_burst<TA, TB, 4>(p, value, a0, b0, threadIdx.x >> 6, q0, q1, res_lds);
  } else {
    pack_rows<TB>(p, value, TA, a0, b0, threadIdx.x >> 6, blockDim.x >> 6, q0, q1, res_lds);
  }
}

}  // namespace apnn
