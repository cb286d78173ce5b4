// Latency-oriented VALU GEMM for problems with few outputs (the M=64 sweep, fully connected layers
// at small batch): no LDS, no barrier, operands straight from global memory / L1.
//
// Eight consecutive lanes share four consecutive outputs out[a][b..b+3] and split K between them:
// lane l of the group owns the 128-bit word groups l, l+8, ... of every operand row, so the eight
// lanes of a group read 128 contiguous bytes of a row per load instruction.  Each lane ANDs /
// popcounts its slice for the four outputs (and the activation sums for symmetric weights), the
// partial results meet in three butterfly steps, and lanes 0..3 of a group hold the four outputs:
// a wave owns 32 consecutive columns of one output row -- 128 contiguous bytes of int32, or exactly
// one packed word per output bit-plane.  A work-group covers four rows x 32 columns (one row per
// wave), so its waves re-read the same 32 rows of B from the compute unit's L1.  All loads of a K
// step are independent; with eight lanes per four outputs the launch has twice as many waves as one
// thread per output would give, which matters because a lone wave on a SIMD issues VALU operations
// at half rate.
//
// Operands are plain row-major matrices (rows of KW words): the GEMM entry points (A = W rows,
// B = X rows, activation sums over B) and convolutions whose filter spans the whole input map, i.e.
// fully connected layers (A = one image per row, B = filters, activation sums over A: ACT_A).
// Output: int32, or codes (low bits / per-column thresholds) packed MSB-first; no pooling, residual
// or shortcut.  Requires rowsB % 4 == 0 (% 32 for packed output) and KW % 4 == 0.
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/apnn_tc.h"
#include "kparams.h"

namespace apnn {

template <int PA, int PB, bool ACT_A>
__global__ __launch_bounds__(256) void apnn_valu_direct_kernel(const KParams p) {
  constexpr int QC = 2;  // 128-bit word groups per lane, row and K step
  const int tid = threadIdx.x, lane = tid & 63;
  const int l = tid & 7;  // K slice
  const int chunks_b = (p.rowsB + 31) >> 5;
  const int ab = blockIdx.x / chunks_b, bc = blockIdx.x - ab * chunks_b;
  const int a = ab * 4 + (tid >> 6);
  const int b = bc * 32 + ((tid & 63) >> 3) * 4;
  const bool live = a < p.rowsA && b < p.rowsB;
  const int nq = p.KW >> 2;  // 128-bit groups per row
  const uint32_t *arow = p.A + (long long)a * p.KW;
  const uint32_t *brow = p.B + (long long)b * p.KW;

  int acc[4] = {0, 0, 0, 0}, sx[4] = {0, 0, 0, 0};
  for (int q0 = 0; q0 < nq; q0 += 8 * QC) {
    uint4 wa[PA][QC], xb[4][PB][QC];
#pragma unroll
    for (int q = 0; q < QC; ++q) {
      const int qi = q0 + l + 8 * q;
      const bool ok = live && qi < nq;
#pragma unroll
      for (int i = 0; i < PA; ++i) {
        wa[i][q] = make_uint4(0, 0, 0, 0);
        if (ok) wa[i][q] = *reinterpret_cast<const uint4 *>(arow + i * p.planeA + 4 * qi);
      }
#pragma unroll
      for (int o = 0; o < 4; ++o)
#pragma unroll
        for (int j = 0; j < PB; ++j) {
          xb[o][j][q] = make_uint4(0, 0, 0, 0);
          if (ok) xb[o][j][q] = *reinterpret_cast<const uint4 *>(brow + j * p.planeB + (long long)o * p.KW + 4 * qi);
        }
    }
#pragma unroll
    for (int q = 0; q < QC; ++q) {
      if (ACT_A) {
        int s = 0;
#pragma unroll
        for (int i = 0; i < PA; ++i) {
          const uint4 w = wa[i][q];
          s += (__popc(w.x) + __popc(w.y) + __popc(w.z) + __popc(w.w)) << i;
        }
        sx[0] += s;
      }
#pragma unroll
      for (int o = 0; o < 4; ++o) {
#pragma unroll
        for (int j = 0; j < PB; ++j) {
          const uint4 x = xb[o][j][q];
#pragma unroll
          for (int i = 0; i < PA; ++i) {
            const uint4 w = wa[i][q];
            acc[o] += (__popc(w.x & x.x) + __popc(w.y & x.y) + __popc(w.z & x.z) + __popc(w.w & x.w)) << (i + j);
          }
          if (!ACT_A) sx[o] += (__popc(x.x) + __popc(x.y) + __popc(x.z) + __popc(x.w)) << j;
        }
      }
    }
  }
  int v[4];
#pragma unroll
  for (int o = 0; o < 4; ++o) v[o] = p.sym ? 2 * acc[o] - p.wmax * sx[ACT_A ? 0 : o] : acc[o];
#pragma unroll
  for (int off = 1; off < 8; off <<= 1)
#pragma unroll
    for (int o = 0; o < 4; ++o) v[o] += __shfl_xor(v[o], off, 64);
  const int mine = l == 0 ? v[0] : l == 1 ? v[1] : l == 2 ? v[2] : v[3];  // output column b + l for l < 4

  if (p.epi == APNN_EPI_INT32) {
    if (live && l < 4) reinterpret_cast<int *>(p.out)[(long long)a * p.rowsB + b + l] = mine;
    return;
  }
  // packed output: bring the 32 outputs of the wave to lanes 0..31 in column order, quantize each in
  // its lane, one ballot per output bit-plane
  const int src = ((lane & 31) >> 2) * 8 + (lane & 3);
  int val = __shfl(mine, src, 64);
  const int col = bc * 32 + (lane & 31);
  const bool col_ok = lane < 32 && col < p.rowsB;
  int code = 0;
  if (p.epi == APNN_EPI_LOWBITS) {
    code = val & ((1 << p.out_bits) - 1);
  } else if (col_ok) {
    const int nt = (1 << p.out_bits) - 1;
    if (p.flip != nullptr && p.flip[col]) val = -val;
    const int32_t *t = p.thr + (long long)col * nt;
    for (int k = 0; k < nt; ++k) code += (val >= t[k]) ? 1 : 0;
  }
  const int w32 = p.rowsB >> 5;
  for (int bit = 0; bit < p.out_bits; ++bit) {
    const unsigned long long mask = __ballot(col_ok && ((code >> bit) & 1));
    if (lane == 0 && a < p.rowsA && bc < w32)
      reinterpret_cast<uint32_t *>(p.out)[bit * p.out_plane + (long long)a * w32 + bc] = __brev((uint32_t)mask);
  }
}

// hipErrorNotSupported when the shape or epilogue is outside what the kernel handles
template <int PA, int PB, bool ACT_A>
inline hipError_t launch_valu_direct(const KParams &p, hipStream_t stream) {
  if ((p.rowsB & 3) != 0 || (p.KW & 3) != 0) return hipErrorNotSupported;
  if (p.epi != APNN_EPI_INT32 &&
      ((p.rowsB & 31) != 0 || p.pool != APNN_POOL_NONE || p.resid != nullptr || p.save_acc != nullptr ||
       p.resid_planes != nullptr))
    return hipErrorNotSupported;
  const unsigned blocks = (unsigned)(((p.rowsA + 3) / 4) * ((p.rowsB + 31) / 32));
  hipLaunchKernelGGL((apnn_valu_direct_kernel<PA, PB, ACT_A>), dim3(blocks), dim3(256), 0, stream, p);
  return hipGetLastError();
}

}  // namespace apnn
