// VALU path: bit-plane contraction by v_and + v_bcnt (popcount-accumulate) on packed 32-bit words.
//
// A 256-thread work-group owns a (16*RA) x (16*RB) output tile; thread (ta, tb) owns an RA x RB
// micro-tile.  Operand words are staged through LDS transposed (k-major), so a thread fetches its
// RA (or RB) consecutive rows of one k-word with a single 128/64/32-bit LDS read, and the next
// K-chunk's global loads are issued before the current chunk is consumed.
// Per k-word a thread spends PA+PB LDS reads on 2*RA*RB*PA*PB VALU operations.
//
// Accumulators are kept per plane-weight s = i + j (the reference combines the plane results
// v0 + 2*v1 (+ 4*v2 ...) after the K loop the same way,
// APNN-TC-lib/bmmaTensorCoreGemm/src/71_bmmaTensorCoreGemm.cu:259-283).
#pragma once
#include <hip/hip_runtime.h>

#include "epilogue.h"
#include "kparams.h"

namespace apnn {

template <int VW> struct WordVec;
template <> struct WordVec<4> { using type = uint4; };
template <> struct WordVec<2> { using type = uint2; };
template <> struct WordVec<1> { using type = uint32_t; };

template <int VW>
__device__ __forceinline__ void load_words(const uint32_t *ptr, bool valid, uint32_t (&dst)[VW]) {
  if (valid) {
    const typename WordVec<VW>::type v = *reinterpret_cast<const typename WordVec<VW>::type *>(ptr);
    const uint32_t *w = reinterpret_cast<const uint32_t *>(&v);
#pragma unroll
    for (int i = 0; i < VW; ++i) dst[i] = w[i];
  } else {
#pragma unroll
    for (int i = 0; i < VW; ++i) dst[i] = 0u;
  }
}

template <int R>
__device__ __forceinline__ void lds_read_rows(const uint32_t *ptr, uint32_t (&dst)[R]) {
  const typename WordVec<R>::type v = *reinterpret_cast<const typename WordVec<R>::type *>(ptr);
  const uint32_t *w = reinterpret_cast<const uint32_t *>(&v);
#pragma unroll
  for (int i = 0; i < R; ++i) dst[i] = w[i];
}

// n / d for n*d < 2^32 with m = ceil(2^32 / d), d >= 2; d == 1 handled by the caller's select
__device__ __forceinline__ uint32_t fast_div(uint32_t n, uint32_t d, uint32_t m) {
  return d == 1 ? n : __umulhi(n, m);
}

template <int PA, int PB, int RA, int RB, int VW, bool CONV>
__global__ __launch_bounds__(256) void apnn_valu_kernel(const KParams p) {
  // PA == PB == 8 is the any-precision instantiation: the plane counts of the launch (1..8 each) come
  // from KParams and the plane loops skip what is not there.
  constexpr bool ANY = PA == 8 && PB == 8;
  const int na = ANY ? p.planesA : PA, nb = ANY ? p.planesB : PB;
  constexpr int NT = 256;
  constexpr int TA = 16 * RA, TB = 16 * RB;
  constexpr int KC = 16;            // k-words per staged chunk
  constexpr int KQ = KC / VW;       // load units per row per chunk
  constexpr int LDA = TA + 4, LDB = TB + 4;
  constexpr int UA = TA * KQ, UB = TB * KQ;         // load units per plane
  constexpr int NIA = (UA + NT - 1) / NT, NIB = (UB + NT - 1) / NT;
  constexpr int NS = PA + PB - 1;
  constexpr int STAGE_WORDS = (PA * LDA + PB * LDB) * KC;
  constexpr int RES_WORDS = (TB % 32 == 0) ? 2 * TA * (TB / 32) : 0;   // two shortcut planes of the tile
  constexpr int RES_REGS = (RES_WORDS + NT - 1) / NT > 0 ? (RES_WORDS + NT - 1) / NT : 1;
  constexpr int TILE_WORDS = TA * (TB + 1) + RES_WORDS;
  constexpr int SMEM_WORDS = STAGE_WORDS > TILE_WORDS ? STAGE_WORDS : TILE_WORDS;

  __shared__ __attribute__((aligned(16))) uint32_t smem[SMEM_WORDS];
  uint32_t *As = smem;                       // [PA][KC][LDA]
  uint32_t *Bs = smem + PA * LDA * KC;       // [PB][KC][LDB]

  const int tid = threadIdx.x;
  const int ta = tid >> 4, tb = tid & 15;

  // fast (B) tile index varies fastest so that neighbouring work-groups share the same A rows
  const int tilesB = (p.rowsB + TB - 1) / TB;
  const int a0 = (blockIdx.x / tilesB) * TA;
  const int b0 = (blockIdx.x % tilesB) * TB;

  // ---- per-thread load bookkeeping (row / k-offset of each load unit never changes) ----------
  int a_row[NIA], a_kq[NIA];
  int a_b[NIA], a_y0[NIA], a_x0[NIA];  // conv: image, top-left input coordinate of the window
  bool a_ok[NIA];
#pragma unroll
  for (int it = 0; it < NIA; ++it) {
    const int u = tid + it * NT;
    a_kq[it] = u % KQ;
    a_row[it] = u / KQ;
    const int grow = a0 + a_row[it];
    a_ok[it] = (u < UA) && (grow < p.rowsA);
    if (CONV) {
      int pix = grow, oy, ox, b;
      if (p.pool_order) {
        const int win = pix >> 2, sub = pix & 3;
        const int hw = p.Wo >> 1, hh = p.Ho >> 1;
        const int px = win % hw, t = win / hw;
        const int py = t % hh;
        b = t / hh;
        oy = 2 * py + (sub >> 1);
        ox = 2 * px + (sub & 1);
      } else {
        ox = pix % p.Wo;
        const int t = pix / p.Wo;
        oy = t % p.Ho;
        b = t / p.Ho;
      }
      a_b[it] = b;
      a_y0[it] = oy * p.stride - p.pad;
      a_x0[it] = ox * p.stride - p.pad;
    }
  }
  int b_row[NIB], b_kq[NIB];
  bool b_ok[NIB];
#pragma unroll
  for (int it = 0; it < NIB; ++it) {
    const int u = tid + it * NT;
    b_kq[it] = u % KQ;
    b_row[it] = u / KQ;
    b_ok[it] = (u < UB) && (b0 + b_row[it] < p.rowsB);
  }

  uint32_t ra_[NIA][PA][VW], rb_[NIB][PB][VW];

  // quantizer and shortcut words of this tile: requested now, consumed after the K loop
  ChannelQuant q0{}, q1{};
  uint32_t res_regs[RES_REGS];
  bool res_prefetched = false;
  if constexpr (TB % 32 == 0) {
    if (p.epi != APNN_EPI_INT32) {
      load_tile_quant<TB>(p, b0, q0, q1);
      if (p.resid_planes != nullptr && p.resid_bits <= 2 && p.pool == APNN_POOL_NONE) {
        shortcut_prefetch<TB, RES_REGS>(p, TA, a0, b0, tid, NT, res_regs);
        res_prefetched = true;
      }
    }
  }

  auto fetch = [&](int k0) {
#pragma unroll
    for (int it = 0; it < NIA; ++it) {
      const int kw0 = k0 + a_kq[it] * VW;
      bool ok = a_ok[it] && kw0 < p.KW;
      long long off;
      if (CONV) {
        const uint32_t tap = fast_div((uint32_t)kw0, (uint32_t)p.C32, p.magicC32);
        const int cw = kw0 - (int)tap * p.C32;
        const uint32_t r = fast_div(tap, (uint32_t)p.S, p.magicS);
        const int s = (int)tap - (int)r * p.S;
        const int iy = a_y0[it] + (int)r, ix = a_x0[it] + s;
        ok = ok && iy >= 0 && iy < p.Hs && ix >= 0 && ix < p.Ws;
        off = (((long long)a_b[it] * p.Hs + iy) * p.Ws + ix) * p.C32 + cw;
      } else {
        off = (long long)(a0 + a_row[it]) * p.KW + kw0;
      }
#pragma unroll
      for (int pl = 0; pl < PA; ++pl)
        if (!ANY || pl < na) load_words<VW>(p.A + off + pl * p.planeA, ok, ra_[it][pl]);
    }
#pragma unroll
    for (int it = 0; it < NIB; ++it) {
      const int kw0 = k0 + b_kq[it] * VW;
      const bool ok = b_ok[it] && kw0 < p.KW;
      const long long off = (long long)(b0 + b_row[it]) * p.KW + kw0;
#pragma unroll
      for (int pl = 0; pl < PB; ++pl)
        if (!ANY || pl < nb) load_words<VW>(p.B + off + pl * p.planeB, ok, rb_[it][pl]);
    }
  };

  auto stage = [&]() {
#pragma unroll
    for (int it = 0; it < NIA; ++it) {
      if (UA % NT == 0 || tid + it * NT < UA) {
#pragma unroll
        for (int pl = 0; pl < PA; ++pl)
          if (!ANY || pl < na) {
#pragma unroll
            for (int i = 0; i < VW; ++i) As[(pl * KC + a_kq[it] * VW + i) * LDA + a_row[it]] = ra_[it][pl][i];
          }
      }
    }
#pragma unroll
    for (int it = 0; it < NIB; ++it) {
      if (UB % NT == 0 || tid + it * NT < UB) {
#pragma unroll
        for (int pl = 0; pl < PB; ++pl)
          if (!ANY || pl < nb) {
#pragma unroll
            for (int i = 0; i < VW; ++i) Bs[(pl * KC + b_kq[it] * VW + i) * LDB + b_row[it]] = rb_[it][pl][i];
          }
      }
    }
  };

  int acc[NS][RA][RB];
#pragma unroll
  for (int s = 0; s < NS; ++s)
#pragma unroll
    for (int i = 0; i < RA; ++i)
#pragma unroll
      for (int j = 0; j < RB; ++j) acc[s][i][j] = 0;
  // activation row sums per plane (symmetric-weight correction): activations are the A operand of
  // the convolution kernels and the B operand of the GEMM entry points
  constexpr int RS = CONV ? RA : RB, PS = CONV ? PA : PB;
  int ssum[PS][RS];
#pragma unroll
  for (int i = 0; i < PS; ++i)
#pragma unroll
    for (int j = 0; j < RS; ++j) ssum[i][j] = 0;

  const int nchunks = (p.KW + KC - 1) / KC;
  fetch(0);
  for (int ch = 0; ch < nchunks; ++ch) {
    stage();
    __syncthreads();
    if (ch + 1 < nchunks) fetch((ch + 1) * KC);
#pragma unroll
    for (int kw = 0; kw < KC; ++kw) {
      uint32_t a[PA][RA], b[PB][RB];
#pragma unroll
      for (int pl = 0; pl < PA; ++pl) {
        if (!ANY || pl < na) {
          lds_read_rows<RA>(&As[(pl * KC + kw) * LDA + ta * RA], a[pl]);
        } else {
#pragma unroll
          for (int x = 0; x < RA; ++x) a[pl][x] = 0;
        }
      }
#pragma unroll
      for (int pl = 0; pl < PB; ++pl) {
        if (!ANY || pl < nb) {
          lds_read_rows<RB>(&Bs[(pl * KC + kw) * LDB + tb * RB], b[pl]);
        } else {
#pragma unroll
          for (int y = 0; y < RB; ++y) b[pl][y] = 0;
        }
      }
#pragma unroll
      for (int i = 0; i < PA; ++i)
#pragma unroll
        for (int j = 0; j < PB; ++j)
          if (!ANY || (i < na && j < nb)) {
#pragma unroll
            for (int x = 0; x < RA; ++x)
#pragma unroll
              for (int y = 0; y < RB; ++y) acc[i + j][x][y] += __popc(a[i][x] & b[j][y]);
          }
      if (p.sym) {
#pragma unroll
        for (int i = 0; i < PS; ++i)
#pragma unroll
          for (int x = 0; x < RS; ++x) ssum[i][x] += __popc(CONV ? a[i][x] : b[i][x]);
      }
    }
    __syncthreads();
  }

  // ---- combine plane weights, symmetric correction -------------------------------------------
  int v[RA][RB];
#pragma unroll
  for (int x = 0; x < RA; ++x)
#pragma unroll
    for (int y = 0; y < RB; ++y) {
      int t = 0;
#pragma unroll
      for (int s = 0; s < NS; ++s) t += acc[s][x][y] << s;
      v[x][y] = t;
    }
  if (p.sym) {
#pragma unroll
    for (int x = 0; x < RA; ++x)
#pragma unroll
      for (int y = 0; y < RB; ++y) {
        int sx = 0;
#pragma unroll
        for (int i = 0; i < PS; ++i) sx += ssum[i][CONV ? x : y] << i;
        v[x][y] = 2 * v[x][y] - p.wmax * sx;
      }
  }

  // ---- output --------------------------------------------------------------------------------
  if (p.epi == APNN_EPI_INT32) {
    int *out = reinterpret_cast<int *>(p.out);
    const int gc = b0 + tb * RB;
#pragma unroll
    for (int x = 0; x < RA; ++x) {
      const int gr = a0 + ta * RA + x;
      if (gr >= p.rowsA) continue;
      int *dst = out + (long long)gr * p.rowsB + gc;
      if ((p.rowsB % RB) == 0) {
        if (gc < p.rowsB) {
          typename WordVec<RB>::type w;
          uint32_t *ww = reinterpret_cast<uint32_t *>(&w);
#pragma unroll
          for (int y = 0; y < RB; ++y) ww[y] = (uint32_t)v[x][y];
          *reinterpret_cast<typename WordVec<RB>::type *>(dst) = w;
        }
      } else {
#pragma unroll
        for (int y = 0; y < RB; ++y)
          if (gc + y < p.rowsB) dst[y] = v[x][y];
      }
    }
  } else if constexpr (TB % 32 == 0) {
    int *tile = reinterpret_cast<int *>(smem);  // staging buffers are dead after the last barrier
#pragma unroll
    for (int x = 0; x < RA; ++x)
#pragma unroll
      for (int y = 0; y < RB; ++y) tile[(ta * RA + x) * (TB + 1) + tb * RB + y] = v[x][y];
    uint32_t *res_lds = smem + TA * (TB + 1);
    if (res_prefetched) shortcut_publish<RES_REGS>(res_lds, tid, NT, res_regs);
    __syncthreads();
    epilogue_packed<TA, TB>(p, tile, a0, b0, q0, q1, res_prefetched ? res_lds : nullptr);
  }
}

template <int PA, int PB, int RA, int RB, int VW, bool CONV>
inline hipError_t launch_valu(const KParams &p, hipStream_t stream) {
  constexpr int TA = 16 * RA, TB = 16 * RB;
  const long long tiles = (long long)((p.rowsA + TA - 1) / TA) * ((p.rowsB + TB - 1) / TB);
  hipLaunchKernelGGL((apnn_valu_kernel<PA, PB, RA, RB, VW, CONV>), dim3((unsigned)tiles), dim3(256), 0, stream, p);
  return hipGetLastError();
}

// one instantiation set per (PA, PB): all tile shapes
template <int PA, int PB, int VW, bool CONV>
inline hipError_t launch_valu_tile(int tile, const KParams &p, hipStream_t stream) {
  switch (tile) {
    case TILE_64x64: return launch_valu<PA, PB, 4, 4, VW, CONV>(p, stream);
    case TILE_32x32: return launch_valu<PA, PB, 2, 2, VW, CONV>(p, stream);
    case TILE_16x32: return launch_valu<PA, PB, 1, 2, VW, CONV>(p, stream);
    default: return launch_valu<PA, PB, 1, 1, VW, CONV>(p, stream);
  }
}

// any-precision instantiation: 32x32 tile only
template <int VW, bool CONV>
inline hipError_t launch_valu_any(const KParams &p, hipStream_t stream) {
  return launch_valu<8, 8, 2, 2, VW, CONV>(p, stream);
}

}  // namespace apnn
