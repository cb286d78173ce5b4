// Latency-oriented VALU GEMM for small problems with a short reduction (the M=64 sweep): no LDS, no
// barrier, one round of global loads.
//
// Eight consecutive lanes share four consecutive outputs out[a][b..b+3] and split K between them:
// lane l of the group owns the 128-bit word groups l, l+8, ... of every operand row, so the eight
// lanes of a group read 128 contiguous bytes of a row per load instruction.  Each lane ANDs /
// popcounts its slice for the four outputs (and the activation sums for symmetric weights), the
// partial results meet in three butterfly steps, and lanes 0..3 of a group store the four outputs:
// a wave writes 32 consecutive int32 of one output row.  All loads of a lane are independent, so the
// kernel is one global-memory round trip plus a few dozen VALU operations; with eight lanes per four
// outputs the launch has twice as many waves as one-thread-per-output would give, which matters
// because a lone wave on a SIMD issues VALU operations at half rate.
//
// GEMM entry points only (A = W rows, B = X rows), int32 output, rowsB % 4 == 0, KW % 4 == 0 and
// KW <= 8 * 4 * DIRECT_MAXQ words.
#pragma once
#include <hip/hip_runtime.h>

#include "kparams.h"

namespace apnn {

constexpr int DIRECT_MAXQ = 2;  // 128-bit word groups per lane and row: K <= 8 * 2 * 128 = 2048 bits

template <int PA, int PB, int NQ>
__global__ __launch_bounds__(256) void apnn_valu_direct_kernel(const KParams p) {
  const int tid = threadIdx.x;
  const int l = tid & 7;                               // K slice
  // a work-group covers four output rows x 32 columns (one row per wave): its waves read the same 32
  // rows of B, so three of the four reads hit the compute unit's L1
  const int chunks_b = (p.rowsB + 31) >> 5;
  const int ab = blockIdx.x / chunks_b, bc = blockIdx.x - ab * chunks_b;
  const int a = ab * 4 + (tid >> 6);
  const int b = bc * 32 + ((tid & 63) >> 3) * 4;
  const bool live = a < p.rowsA && b < p.rowsB;
  const int nq = p.KW >> 2;                            // 128-bit groups per row

  uint4 wa[PA][NQ], xb[4][PB][NQ];
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int qi = l + 8 * q;
    const bool ok = live && qi < nq;
#pragma unroll
    for (int i = 0; i < PA; ++i) {
      wa[i][q] = make_uint4(0, 0, 0, 0);
      if (ok) wa[i][q] = *reinterpret_cast<const uint4 *>(p.A + i * p.planeA + (long long)a * p.KW + 4 * qi);
    }
#pragma unroll
    for (int o = 0; o < 4; ++o)
#pragma unroll
      for (int j = 0; j < PB; ++j) {
        xb[o][j][q] = make_uint4(0, 0, 0, 0);
        if (ok) xb[o][j][q] = *reinterpret_cast<const uint4 *>(p.B + j * p.planeB + (long long)(b + o) * p.KW + 4 * qi);
      }
  }

  int v[4];
#pragma unroll
  for (int o = 0; o < 4; ++o) {
    int t = 0, sx = 0;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
#pragma unroll
      for (int j = 0; j < PB; ++j) {
        const uint4 x = xb[o][j][q];
#pragma unroll
        for (int i = 0; i < PA; ++i) {
          const uint4 w = wa[i][q];
          t += (__popc(w.x & x.x) + __popc(w.y & x.y) + __popc(w.z & x.z) + __popc(w.w & x.w)) << (i + j);
        }
        sx += (__popc(x.x) + __popc(x.y) + __popc(x.z) + __popc(x.w)) << j;
      }
    }
    v[o] = p.sym ? 2 * t - p.wmax * sx : t;
  }
#pragma unroll
  for (int off = 1; off < 8; off <<= 1)
#pragma unroll
    for (int o = 0; o < 4; ++o) v[o] += __shfl_xor(v[o], off, 64);
  if (live && l < 4) {
    const int mine = l == 0 ? v[0] : l == 1 ? v[1] : l == 2 ? v[2] : v[3];
    reinterpret_cast<int *>(p.out)[(long long)a * p.rowsB + b + l] = mine;
  }
}

// hipErrorNotSupported when the shape is outside what the kernel handles
template <int PA, int PB>
inline hipError_t launch_valu_direct(const KParams &p, hipStream_t stream) {
  if ((p.rowsB & 3) != 0 || (p.KW & 3) != 0 || p.KW > 32 * DIRECT_MAXQ) return hipErrorNotSupported;
  const unsigned blocks = (unsigned)(((p.rowsA + 3) / 4) * ((p.rowsB + 31) / 32));
  if (p.KW <= 32)
    hipLaunchKernelGGL((apnn_valu_direct_kernel<PA, PB, 1>), dim3(blocks), dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((apnn_valu_direct_kernel<PA, PB, 2>), dim3(blocks), dim3(256), 0, stream, p);
  return hipGetLastError();
}

}  // namespace apnn
