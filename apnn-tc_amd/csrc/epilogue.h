// Output stage shared by the VALU and MFMA kernels.
//
// Quantizing epilogues work from an int32 tile staged in LDS so that 64 consecutive output
// channels sit in the 64 lanes of a wave: one ballot per output bit-plane then yields two
// MSB-first 32-bit words (the wave64 counterpart of the reference's __brev(__ballot_sync()),
// APNN-TC-lib/bmmaTensorCoreGemm/src/66_bmmaTensorCoreGemm.cuh:255-276).
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/apnn_tc.h"
#include "kparams.h"

namespace apnn {

__device__ __forceinline__ int quantize_code(const KParams &p, int v, int gcol) {
  if (p.epi == APNN_EPI_LOWBITS) return v & ((1 << p.out_bits) - 1);
  const int nt = (1 << p.out_bits) - 1;
  if (p.flip != nullptr && p.flip[gcol]) v = -v;
  const int32_t *t = p.thr + (long long)gcol * nt;
  int code = 0;
  for (int k = 0; k < nt; ++k) code += (v >= t[k]) ? 1 : 0;
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

// tile: LDS, [TA][TB + 1] int32, row r of the tile is output row a0 + r (or, in pool order, rows
// 4i..4i+3 are the 2x2 window a0/4 + i).  Must be called by every thread of the block after a
// __syncthreads() that made the tile visible.
template <int TA, int TB>
__device__ __forceinline__ void epilogue_packed(const KParams &p, const int *tile, int a0, int b0) {
  static_assert(TB % 32 == 0, "packed epilogue needs whole 32-channel words per tile row");
  constexpr int LDT = TB + 1;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nwaves = blockDim.x >> 6;
  const bool pooled = p.pool != APNN_POOL_NONE;
  const int n_out = pooled ? TA / 4 : TA;
  const int out_rows_total = pooled ? p.rowsA / 4 : p.rowsA;
  const int row_base = pooled ? a0 / 4 : a0;
  const int w32 = p.rowsB >> 5;
  uint32_t *out = reinterpret_cast<uint32_t *>(p.out);

  for (int unit = wave; unit < n_out * TB / 64; unit += nwaves) {
    const int e = unit * 64 + lane;
    const int orow = e / TB;
    const int col = e % TB;
    const int grow = row_base + orow;
    const int gcol = b0 + col;
    const bool valid = grow < out_rows_total && gcol < p.rowsB;
    int code = 0;
    if (valid) {
      if (!pooled) {
        int v = tile[orow * LDT + col];
        const long long o = (long long)grow * p.rowsB + gcol;
        if (p.resid != nullptr) v += p.resid[o];
        if (p.resid_planes != nullptr) v += packed_residual(p, grow, gcol);
        if (p.save_acc != nullptr) p.save_acc[o] = v;
        code = quantize_code(p, v, gcol);
      } else {
        const int t0 = tile[(4 * orow + 0) * LDT + col];
        const int t1 = tile[(4 * orow + 1) * LDT + col];
        const int t2 = tile[(4 * orow + 2) * LDT + col];
        const int t3 = tile[(4 * orow + 3) * LDT + col];
        if (p.pool == APNN_POOL_AVG2X2) {
          code = quantize_code(p, (t0 + t1 + t2 + t3) / 4, gcol);
        } else {
          const int c0 = quantize_code(p, t0, gcol), c1 = quantize_code(p, t1, gcol);
          const int c2 = quantize_code(p, t2, gcol), c3 = quantize_code(p, t3, gcol);
          code = max(max(c0, c1), max(c2, c3));
        }
      }
    }
    for (int b = 0; b < p.out_bits; ++b) {
      const unsigned long long mask = __ballot(valid && ((code >> b) & 1));
      const uint32_t word = (lane < 32) ? __brev((uint32_t)mask) : __brev((uint32_t)(mask >> 32));
      if (valid && (lane & 31) == 0) out[b * p.out_plane + (long long)grow * w32 + (gcol >> 5)] = word;
    }
  }
}

}  // namespace apnn
