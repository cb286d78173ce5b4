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

// popc(x) + acc in one instruction (the compiler otherwise counts into fresh registers and adds the
// counts in a tree, one more instruction per three words)
__device__ __forceinline__ int popc_acc(uint32_t x, int acc) {
  int r;
  asm("v_bcnt_u32_b32 %0, %1, %2" : "=v"(r) : "v"(x), "v"(acc));
  return r;
}
__device__ __forceinline__ int popc4_acc(const uint4 &x, int acc) {
  return popc_acc(x.w, popc_acc(x.z, popc_acc(x.y, popc_acc(x.x, acc))));
}
// QC: 128-bit word groups per lane, row and K step.  A lone wave on a SIMD issues one instruction every
// four clocks, so the popcount work of a wave is on the launch's critical path: rows of at most 32 words
// (eight groups, one per lane) run the QC = 1 instantiation, which does not carry a second, empty group.
// LPG: lanes that share four outputs and split K (8, or 4: a wave then owns 64 columns and the launch has
// half as many waves, each with the same fixed cost and twice the popcount work -- taken when eight
// lanes per group would put more than one wave on a SIMD).
template <int PA, int PB, bool ACT_A, int QC, int LPG>
__global__ __launch_bounds__(256) void apnn_valu_direct_kernel(const KParams p) {
  static_assert(LPG == 8 || LPG == 4, "lanes per output group");
  constexpr int CPW = 64 / LPG * 4;  // columns per wave
  const int tid = threadIdx.x, lane = tid & 63;
  const int l = tid & (LPG - 1);  // K slice
  const int ab = blockIdx.y, bc = blockIdx.x;  // four output rows x CPW columns per work-group
  const int a = ab * 4 + (tid >> 6);
  const int b = bc * CPW + ((tid & 63) / LPG) * 4;
  const bool live = a < p.rowsA && b < p.rowsB;
  const int nq = p.KW >> 2;  // 128-bit groups per row
  // Loads are never predicated: a lane outside the problem (row, column or K slice past the end) reads
  // the last valid row / group instead and its partial sums are dropped.  Addresses are a uniform
  // plane base plus a 32-bit byte offset (the launcher checks that every row offset fits).
  const uint32_t ac = (uint32_t)min(a, p.rowsA - 1), bcl = (uint32_t)(b < p.rowsB ? b : 0);
  const uint32_t row_bytes = (uint32_t)p.KW * 4u;
  const uint32_t offA = ac * row_bytes, offB = bcl * row_bytes;

  const char *baseA[PA], *baseB[PB];
#pragma unroll
  for (int i = 0; i < PA; ++i) baseA[i] = reinterpret_cast<const char *>(p.A + i * p.planeA);
#pragma unroll
  for (int j = 0; j < PB; ++j) baseB[j] = reinterpret_cast<const char *>(p.B + j * p.planeB);
  // Everything the kernel reads from its argument block is requested here, in one round of scalar
  // loads, instead of a second round before the operand loads and a third after the K loop.
  const int sym_sh = p.sym ? 1 : 0, sym_w = p.sym ? p.wmax : 0;
  const int epi = p.epi;
  int *out_i32 = reinterpret_cast<int *>(p.out);
  asm volatile("" ::"s"(baseA[0]), "s"(baseB[0]), "s"(baseA[PA - 1]), "s"(baseB[PB - 1]), "s"(out_i32), "s"(sym_sh), "s"(sym_w),
               "s"(epi));

  int acc[4] = {0, 0, 0, 0}, sx[4] = {0, 0, 0, 0};
  for (int q0 = 0; q0 < nq; q0 += LPG * QC) {
    uint4 wa[PA][QC], xb[4][PB][QC];
    bool ok[QC];
#pragma unroll
    for (int q = 0; q < QC; ++q) {
      const int qi = q0 + l + LPG * q;
      ok[q] = live && qi < nq;
      const uint32_t koff = (uint32_t)min(qi, nq - 1) * 16u;
#pragma unroll
      for (int i = 0; i < PA; ++i)
        wa[i][q] = *reinterpret_cast<const uint4 *>(baseA[i] + (offA + koff));
#pragma unroll
      for (int o = 0; o < 4; ++o)
#pragma unroll
        for (int j = 0; j < PB; ++j)
          xb[o][j][q] = *reinterpret_cast<const uint4 *>(baseB[j] + (offB + (uint32_t)o * row_bytes + koff));
    }
#pragma unroll
    for (int q = 0; q < QC; ++q) {
      int tacc[4] = {0, 0, 0, 0}, tsx[4] = {0, 0, 0, 0};
      if (ACT_A) {
#pragma unroll
        for (int i = 0; i < PA; ++i) {
          tsx[0] += popc4_acc(wa[i][q], 0) << i;
        }
      }
#pragma unroll
      for (int o = 0; o < 4; ++o) {
#pragma unroll
        for (int j = 0; j < PB; ++j) {
          const uint4 x = xb[o][j][q];
#pragma unroll
          for (int i = 0; i < PA; ++i) {
            const uint4 w = wa[i][q];
            const uint4 m = make_uint4(w.x & x.x, w.y & x.y, w.z & x.z, w.w & x.w);
            if (i + j == 0) tacc[o] = popc4_acc(m, tacc[o]); else tacc[o] += popc4_acc(m, 0) << (i + j);
          }
          if (!ACT_A) {
            if (j == 0) tsx[o] = popc4_acc(x, tsx[o]); else tsx[o] += popc4_acc(x, 0) << j;
          }
        }
      }
#pragma unroll
      for (int o = 0; o < 4; ++o) {
        acc[o] += ok[q] ? tacc[o] : 0;
        sx[o] += ok[q] ? tsx[o] : 0;
      }
    }
  }
  int v[4];
  // symmetric weights: 2 * raw - wmax * (activation sum), written without a branch (shift 0 and weight
  // range 0 for the plain result)
#pragma unroll
  for (int o = 0; o < 4; ++o) v[o] = (acc[o] << sym_sh) - sym_w * sx[ACT_A ? 0 : o];
  // butterfly over the eight lanes of a group with data-parallel-primitive adds: lane ^ 1 and lane ^ 2
  // inside a quad, then the mirror image within eight lanes (every lane of a quad already holds the
  // quad's sum, so lane 7 - i delivers the other quad's)
#pragma unroll
  for (int o = 0; o < 4; ++o) {
    v[o] += __builtin_amdgcn_update_dpp(0, v[o], 0xB1, 0xf, 0xf, true);   // quad_perm [1,0,3,2]
    v[o] += __builtin_amdgcn_update_dpp(0, v[o], 0x4E, 0xf, 0xf, true);   // quad_perm [2,3,0,1]
    if (LPG == 8) v[o] += __builtin_amdgcn_update_dpp(0, v[o], 0x141, 0xf, 0xf, true);  // row_half_mirror
  }
  const int l4 = l & 3;
  // output column b + l for l < 4 (two levels of selects, no branches)
  const int m01 = (l4 & 1) ? v[1] : v[0], m23 = (l4 & 1) ? v[3] : v[2];
  const int mine = (l4 & 2) ? m23 : m01;

  if (epi == APNN_EPI_INT32) {
    if (live && l < 4) out_i32[(long long)a * p.rowsB + b + l] = mine;
    return;
  }
  if constexpr (LPG == 4) {
    // packed output, four lanes per group: lane L holds column bc*64 + L, so one ballot per output
    // bit-plane is two finished words
    int val = mine;
    const int col = bc * 64 + lane;
    const bool col_ok = col < p.rowsB;
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
      const int wi = 2 * bc + (lane >> 5);
      if ((lane & 31) == 0 && a < p.rowsA && wi < w32)
        reinterpret_cast<uint32_t *>(p.out)[bit * p.out_plane + (long long)a * w32 + wi] =
            __brev((uint32_t)(lane == 0 ? mask : mask >> 32));
    }
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
  if ((p.rowsA + 3) / 4 > 65535) return hipErrorNotSupported;  // grid.y
  // 32-bit byte offsets inside a plane
  if ((unsigned long long)p.rowsA * p.KW * 4ull >= (1ull << 32) || (unsigned long long)p.rowsB * p.KW * 4ull >= (1ull << 32))
    return hipErrorNotSupported;
  static int cus = 0;  // compute units of the device (one device per process here)
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cus = n;
  }
  const unsigned rows4 = (unsigned)((p.rowsA + 3) / 4);
  const dim3 grid8((unsigned)((p.rowsB + 31) / 32), rows4), grid4((unsigned)((p.rowsB + 63) / 64), rows4);
  if (grid8.x * rows4 > (unsigned)cus && p.KW <= 16) {
    // rows of at most four word groups, more work-groups than compute units with eight lanes per group:
    // four lanes per group, one word group each (with two word groups per lane, K = 1024, the longer
    // popcount chain of a wave measured slower than two waves per SIMD: 2.55 vs 2.36 us)
    hipLaunchKernelGGL((apnn_valu_direct_kernel<PA, PB, ACT_A, 1, 4>), grid4, dim3(256), 0, stream, p);
  } else if (p.KW <= 32) {
    hipLaunchKernelGGL((apnn_valu_direct_kernel<PA, PB, ACT_A, 1, 8>), grid8, dim3(256), 0, stream, p);
  } else {
    hipLaunchKernelGGL((apnn_valu_direct_kernel<PA, PB, ACT_A, 2, 8>), grid8, dim3(256), 0, stream, p);
  }
  return hipGetLastError();
}

}  // namespace apnn
