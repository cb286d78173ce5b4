// Matrix-core path with operands expanded while staging (FP4 operands, see mfma_kernel.h for the
// encoding and the output stage).
//
// apnn_mfma_kernel stages the *packed* planes in LDS and lets every wave expand the rows it consumes in
// registers, once per consuming wave and k-step; its large tiles are bound by that vector work, which
// shares the issue port with the matrix instructions.  Here the threads that stage a chunk expand it:
// each packed word (32 elements of a row, all planes) becomes, per 2-bit digit, the 16 bytes that ARE
// the matrix-core operand of one lane -- nibble c of dword t holds element 4c + t, the same element order
// for both operands, which only permutes the terms of each dot product -- and is written to LDS with one
// 128-bit store.  The K loop is then one 128-bit LDS read per operand block and k-step plus the matrix
// instructions: a word is expanded once per work-group instead of once per wave that uses it, and no
// expansion sits between an LDS read and the instruction that consumes it.
//
//   LDS, per buffer (two buffers):  A[DA][KC][TA] and B[DB][KC][TB] of 16-byte operands, (digit, k-word,
//   row); a wave's read of 64 consecutive rows' operands is contiguous and conflict-free.
//   Activation sums for the symmetric-weight correction are population counts taken by the staging
//   threads, combined per row at the end.
//
// Tiles: four waves as WA x WB, each FA x FB blocks of 32x32 (no split-K variant: few-output problems
// stay on apnn_mfma_kernel's split-K tiles).  Work-group index -> tile: consecutive indices land on
// different XCDs (round-robin), so the index is first regrouped into per-XCD contiguous ranges and each
// range walks the tile grid in bands of 8 tile rows, column-major inside a band: the work-groups resident
// on one XCD at a time share a few operand row blocks in that XCD's L2.
#pragma once
#include "mfma_kernel.h"

namespace apnn {

constexpr int kXcds = 8;

// Global loads run two chunks ahead of the matrix work.  (Three chunks in flight, with the chunk loop
// unrolled over three register sets, measured no faster at 4096^3 / 8192^3 -- the kernel is bound by LDS
// bandwidth, not by load latency -- and pushed the 256x128 tile into register spills.)
template <int PA, int PB, int FA, int FB, int WA, int WB, int VW, bool CONV, int OCC>
__global__ __launch_bounds__(256, OCC) void apnn_mfma_xs_kernel(const KParams pk) {
  static_assert(WA * WB == 4, "four waves tile the output");
  KParams p = pk;
  constexpr int DA = (PA + 1) / 2, DB = (PB + 1) / 2;
  constexpr int NT = 256;
  constexpr int TA = WA * FA * 32, TB = WB * FB * 32;
  constexpr int ROWS = DA * TA + DB * TB;  // 16-byte operands per k-word
  constexpr int KC = ROWS <= 256 ? 8 : 4;  // k-words per staged chunk: two buffers stay within 64 KiB
  constexpr int KQ = KC / VW;
  static_assert(KC % VW == 0 && KC % 2 == 0, "whole loads and whole k-steps per chunk");
  constexpr int UA = TA * KQ, UB = TB * KQ;
  constexpr int NIA = (UA + NT - 1) / NT, NIB = (UB + NT - 1) / NT;
  constexpr int BUF_U4 = ROWS * KC;
  constexpr int DIRECT_BITS = (CONV ? PA : PB) >= 3 ? 4 : 2;
  constexpr bool EPI_LAZY = FA * FB >= 8;

  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  __shared__ int sumbuf[CONV ? TA : TB];
  uint4 *lds4 = reinterpret_cast<uint4 *>(smem);

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int li = lane & 31, g = lane >> 5;
  const int wa = wave / WB, wb = wave % WB;

  // ---- work-group index -> tile ---------------------------------------------------------------
  const int tilesA = (p.rowsA + TA - 1) / TA, tilesB = (p.rowsB + TB - 1) / TB;
  int bid = blockIdx.x;
  if (CONV && pk.pair_tiles > 0 && bid >= pk.pair_tiles) {
    bid -= pk.pair_tiles;
    p.B = pk.B2;
    p.KW = pk.KW2;
    p.S = pk.S2;
    p.pad = pk.pad2;
    p.magicS = pk.magicS2;
    p.planeB = pk.planeB2;
    p.thr = pk.thr2;
    p.flip = pk.flip2;
    p.out = pk.out2;
  }
  int ta, tb;
  {
    const int ntiles = tilesA * tilesB;
    // per-XCD contiguous ranges (the tail that does not fill all XCDs keeps its index)
    const int per = ntiles / kXcds;
    int t = bid;
    if (bid < per * kXcds) t = (bid % kXcds) * per + bid / kXcds;
    // bands of 8 tile rows, column-major inside a band
    constexpr int BAND = 8;
    const int band = t / (BAND * tilesB);
    const int in_band = t - band * BAND * tilesB;
    const int band_rows = min(BAND, tilesA - band * BAND);
    tb = in_band / band_rows;
    ta = band * BAND + in_band - tb * band_rows;
  }
  const int a0 = ta * TA, b0 = tb * TB;

  auto pixel_origin = [&](int pix, int &b, int &y0, int &x0) {
    int oy, ox;
    if (p.geo_fast) {
      const int gw = p.pool_order ? p.Wo >> 1 : p.Wo, gh = p.pool_order ? p.Ho >> 1 : p.Ho;
      const int cell = p.pool_order ? pix >> 2 : pix, sub = pix & 3;
      const int t = (int)fast_div((uint32_t)cell, (uint32_t)gw, p.magicGW);
      const int px = cell - t * gw;
      b = (int)fast_div((uint32_t)t, (uint32_t)gh, p.magicGH);
      const int py = t - b * gh;
      oy = p.pool_order ? 2 * py + (sub >> 1) : py;
      ox = p.pool_order ? 2 * px + (sub & 1) : px;
    } else if (p.pool_order) {
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
    y0 = oy * p.stride - p.pad;
    x0 = ox * p.stride - p.pad;
  };

  // ---- staging bookkeeping: unit u = (row, group of VW k-words) ----------------------------------
  int a_row[NIA], a_kq[NIA], a_b[NIA], a_y0[NIA], a_x0[NIA];
  bool a_ok[NIA];
  int b_row[NIB], b_kq[NIB];
  bool b_ok[NIB];
#pragma unroll
  for (int it = 0; it < NIA; ++it) {
    const int u = tid + it * NT;
    a_kq[it] = u % KQ;
    a_row[it] = u / KQ;
    const int grow = a0 + a_row[it];
    a_ok[it] = (u < UA) && (grow < p.rowsA);
    a_b[it] = a_y0[it] = a_x0[it] = 0;
    if (CONV) pixel_origin(grow, a_b[it], a_y0[it], a_x0[it]);
  }
#pragma unroll
  for (int it = 0; it < NIB; ++it) {
    const int u = tid + it * NT;
    b_kq[it] = u % KQ;
    b_row[it] = u / KQ;
    b_ok[it] = (u < UB) && (b0 + b_row[it] < p.rowsB);
  }

  uint32_t ra_[NIA][PA][VW], rb_[NIB][PB][VW];
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
      for (int pl = 0; pl < PA; ++pl) load_words<VW>(p.A + off + pl * p.planeA, ok, ra_[it][pl]);
    }
#pragma unroll
    for (int it = 0; it < NIB; ++it) {
      const int kw0 = k0 + b_kq[it] * VW;
      const bool ok = b_ok[it] && kw0 < p.KW;
      const long long off = (long long)(b0 + b_row[it]) * p.KW + kw0;
#pragma unroll
      for (int pl = 0; pl < PB; ++pl) load_words<VW>(p.B + off + pl * p.planeB, ok, rb_[it][pl]);
    }
  };

  // activation sums (A rows for convolution, B rows for the GEMM entry points), per staged unit
  constexpr int NIS = CONV ? NIA : NIB;
  int psum[NIS];
#pragma unroll
  for (int it = 0; it < NIS; ++it) psum[it] = 0;

  // expand the fetched words and publish them: one 128-bit store per (row, k-word, digit)
  auto stage = [&](uint4 *buf) {
    uint4 *As = buf;                    // [DA][KC][TA]
    uint4 *Bs = buf + DA * KC * TA;     // [DB][KC][TB]
#pragma unroll
    for (int it = 0; it < NIA; ++it) {
      if (UA % NT == 0 || tid + it * NT < UA) {
#pragma unroll
        for (int i = 0; i < VW; ++i) {
          uint32_t w[PA];
#pragma unroll
          for (int pl = 0; pl < PA; ++pl) {
            w[pl] = ra_[it][pl][i];
            if (CONV) psum[CONV ? it : 0] += __popc(w[pl]) << pl;
          }
          static_for<0, DA>([&](auto dc) {
            constexpr int d = decltype(dc)::value;
            const v8i e = expand_fp4<PA, d>(w);
            As[(d * KC + a_kq[it] * VW + i) * TA + a_row[it]] =
                make_uint4((uint32_t)e[0], (uint32_t)e[1], (uint32_t)e[2], (uint32_t)e[3]);
          });
        }
      }
    }
#pragma unroll
    for (int it = 0; it < NIB; ++it) {
      if (UB % NT == 0 || tid + it * NT < UB) {
#pragma unroll
        for (int i = 0; i < VW; ++i) {
          uint32_t w[PB];
#pragma unroll
          for (int pl = 0; pl < PB; ++pl) {
            w[pl] = rb_[it][pl][i];
            if (!CONV) psum[CONV ? 0 : it] += __popc(w[pl]) << pl;
          }
          static_for<0, DB>([&](auto dc) {
            constexpr int d = decltype(dc)::value;
            const v8i e = expand_fp4<PB, d>(w);
            Bs[(d * KC + b_kq[it] * VW + i) * TB + b_row[it]] =
                make_uint4((uint32_t)e[0], (uint32_t)e[1], (uint32_t)e[2], (uint32_t)e[3]);
          });
        }
      }
    }
  };

  v16f acc[FA][FB];
#pragma unroll
  for (int x = 0; x < FA; ++x)
#pragma unroll
    for (int y = 0; y < FB; ++y)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[x][y][r] = 0;

  EpiOperands<FA, FB> eo;
  epi_prefetch<1, DIRECT_BITS, EPI_LAZY>(p, a0 + wa * FA * 32, b0 + wb * FB * 32, lane, eo);

  // operands of one k-step (two k-words: lane half g takes word 2*ks + g)
  uint4 fa[FA][DA], fb[FB][DB];
  auto read_frags = [&](const uint4 *buf, int ks, uint4 (&a)[FA][DA], uint4 (&b)[FB][DB]) {
    const uint4 *As = buf + (2 * ks + g) * TA + wa * FA * 32 + li;
    const uint4 *Bs = buf + DA * KC * TA + (2 * ks + g) * TB + wb * FB * 32 + li;
#pragma unroll
    for (int x = 0; x < FA; ++x)
#pragma unroll
      for (int d = 0; d < DA; ++d) a[x][d] = As[d * KC * TA + x * 32];
#pragma unroll
    for (int y = 0; y < FB; ++y)
#pragma unroll
      for (int d = 0; d < DB; ++d) b[y][d] = Bs[d * KC * TB + y * 32];
  };
  auto as_v8 = [](const uint4 &u) {
    v8i v = {(int)u.x, (int)u.y, (int)u.z, (int)u.w, 0, 0, 0, 0};
    return v;
  };
  auto mfma_all = [&](const uint4 (&a)[FA][DA], const uint4 (&b)[FB][DB]) {
#pragma unroll
    for (int x = 0; x < FA; ++x)
#pragma unroll
      for (int y = 0; y < FB; ++y) {
        static_for<0, DA>([&](auto dac) {
          static_for<0, DB>([&](auto dbc) {
            constexpr int da = decltype(dac)::value, db = decltype(dbc)::value;
            if constexpr (da + db == 0) {
              acc[x][y] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(as_v8(a[x][da]), as_v8(b[y][db]), acc[x][y], 4,
                                                                          4, 0, 0, 0, 0);
            } else {
              // E8M0 block scales: 127 = 2^0 on A, 127 + 2*(da+db) = 4^(da+db) on B
              acc[x][y] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                  as_v8(a[x][da]), as_v8(b[y][db]), acc[x][y], 4, 4, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F + 0x02020202 * (da + db));
            }
          });
        });
      }
  };

  // ---- K loop: global loads run two chunks ahead, LDS holds two chunks --------------------------
  constexpr int NKS = KC / 2;
  const int nchunks = (p.KW + KC - 1) / KC;
  fetch(0);
  stage(lds4);
  if (nchunks > 1) fetch(KC);
  __syncthreads();
  read_frags(lds4, 0, fa, fb);
  for (int ch = 0; ch < nchunks; ++ch) {
    const uint4 *cur = lds4 + (ch & 1) * BUF_U4;
    uint4 *nxt = lds4 + ((ch + 1) & 1) * BUF_U4;
    const bool more = ch + 1 < nchunks;
    const int nks = min(NKS, (p.KW - ch * KC + 1) / 2);  // k-steps of this chunk that hold data
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      if (ks < nks) {
        uint4 na[FA][DA], nb[FB][DB];
        if (ks + 1 < nks) read_frags(cur, ks + 1, na, nb);
        mfma_all(fa, fb);
        if (ks == 0 && more) {
          // every wave left `nxt` before the barrier that ended the previous chunk
          stage(nxt);
          if (ch + 2 < nchunks) fetch((ch + 2) * KC);
        }
        if (ks + 1 < nks) {
#pragma unroll
          for (int x = 0; x < FA; ++x)
#pragma unroll
            for (int d = 0; d < DA; ++d) fa[x][d] = na[x][d];
#pragma unroll
          for (int y = 0; y < FB; ++y)
#pragma unroll
            for (int d = 0; d < DB; ++d) fb[y][d] = nb[y][d];
        }
      }
    }
    __syncthreads();
    if (more) read_frags(nxt, 0, fa, fb);
  }

  // ---- activation sums: the KQ staging threads of a row are adjacent lanes -----------------------
  constexpr int TS = CONV ? TA : TB;
#pragma unroll
  for (int it = 0; it < NIS; ++it) {
    int t = psum[it];
#pragma unroll
    for (int m = 1; m < KQ; m <<= 1) t += __shfl_xor(t, m, 64);
    const int u = tid + it * NT;
    if (u % KQ == 0 && u / KQ < TS) sumbuf[u / KQ] = t;
  }
  __syncthreads();
  constexpr int FS = CONV ? FA : FB;
  int ssum[FS];
#pragma unroll
  for (int x = 0; x < FS; ++x) ssum[x] = sumbuf[((CONV ? wa * FA : wb * FB) + x) * 32 + li];

  epi_finish<true, 1, CONV, DIRECT_BITS, EPI_LAZY>(p, acc, ssum, smem, wave, lane, a0, b0, wa, wb, eo);
}

constexpr size_t mfma_xs_smem_bytes(int PA, int PB, int FA, int FB, int WA, int WB) {
  const size_t rows = (size_t)((PA + 1) / 2) * WA * FA * 32 + (size_t)((PB + 1) / 2) * WB * FB * 32;
  const size_t kc = rows <= 256 ? 8 : 4;
  const size_t stage = 2 * rows * kc * 16;
  const size_t slab = 4ull * (32 * (FB * 32 + 1) + 32 + FB * 32 + 2 * 32 * FB) * sizeof(int);
  return stage > slab ? stage : slab;
}

template <int PA, int PB, int FA, int FB, int WA, int WB, int VW, bool CONV, int OCC_WANTED>
inline hipError_t launch_mfma_xs(const KParams &p, hipStream_t stream) {
  constexpr int TA = WA * FA * 32, TB = WB * FB * 32;
  constexpr size_t smem_bytes = mfma_xs_smem_bytes(PA, PB, FA, FB, WA, WB);
  constexpr int OCC_FIT = (int)((160 * 1024 - 2048) / smem_bytes);
  constexpr int OCC = OCC_FIT < 1 ? 1 : (OCC_FIT < OCC_WANTED ? OCC_FIT : OCC_WANTED);
  static_assert(smem_bytes + 2048 <= 160 * 1024, "LDS budget of a gfx950 compute unit");
  auto kern = apnn_mfma_xs_kernel<PA, PB, FA, FB, WA, WB, VW, CONV, OCC>;
  if (smem_bytes > 64 * 1024) {
    static bool raised = false;
    if (!raised) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_bytes);
      if (e != hipSuccess) return e;
      raised = true;
    }
  }
  const long long tiles = (long long)((p.rowsA + TA - 1) / TA) * ((p.rowsB + TB - 1) / TB);
  KParams q = p;
  if (p.pair_tiles != 0) q.pair_tiles = (int)tiles;
  hipLaunchKernelGGL(kern, dim3((unsigned)(q.pair_tiles != 0 ? 2 * tiles : tiles)), dim3(256), smem_bytes, stream, q);
  return hipGetLastError();
}

template <int PA, int PB, int VW, bool CONV>
inline hipError_t launch_mfma_xs_tile(int tile, const KParams &p, hipStream_t stream) {
  if (!mfma_xs_tile_enabled(CONV, VW, tile)) return hipErrorNotSupported;
  switch (tile) {
    case MT_128x128: return launch_mfma_xs<PA, PB, 2, 2, 2, 2, VW, CONV, 2>(p, stream);
    case MT_64x64: return launch_mfma_xs<PA, PB, 1, 1, 2, 2, VW, CONV, 4>(p, stream);
    case MT_128x64: return launch_mfma_xs<PA, PB, 1, 2, 4, 1, VW, CONV, 4>(p, stream);
    case MT_256x128:
      if constexpr (!CONV) return launch_mfma_xs<PA, PB, 4, 2, 2, 2, VW, CONV, 2>(p, stream);
      return hipErrorNotSupported;
    case MT_128x256:
      if constexpr (CONV) return launch_mfma_xs<PA, PB, 2, 4, 2, 2, VW, CONV, 2>(p, stream);
      return hipErrorNotSupported;
    default: return hipErrorNotSupported;
  }
}

}  // namespace apnn
