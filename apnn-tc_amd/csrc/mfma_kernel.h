// MFMA path: bit-planes are expanded to int8 in registers and contracted with
// v_mfma_i32_32x32x32_i8, so a k-step of 32 elements costs one matrix instruction per 32x32 output
// block whatever the bit widths are:  sum_ij 2^(i+j) popc(x_i & w_j) == sum_k xval[k] * wval[k]
// with xval = sum_i 2^i x_i[k] (0..15) and wval likewise -- exact in int8 x int8 -> int32.
//
// Work-group = 4 waves arranged WA x WB, each wave owning an (FA*32) x (FB*32) output tile
// (FA*FB accumulator blocks of 16 registers).  The *packed* planes are staged through LDS
// (row-major, double-buffered, one barrier per chunk of KC words); every wave reads the one packed
// word per row and k-step that it needs and expands it in registers:
//   lane (i, g) of a wave supplies row i and the 16 k-positions { 8c + 4g + t : c,t < 4 } of the
//   word -- the same positions for both operands, so the contraction pairs bit k with bit k as the
//   reference does (APNN-TC-lib/bmmaTensorCoreGemm/src/71_bmmaTensorCoreGemm.cu:364-369).
//   ys_p = rotr(word_p, 4g - p);  byte-word t = OR_p ((ys_p >> t) & (0x01010101 << p))
// i.e. 8 VALU operations per plane for 16 int8 operands.
//
// Symmetric (+-) weights use the closed form  2*raw - wmax * (activation row sum); the row sums
// come from popcounts of the packed words the wave already holds.
//
// The epilogue works from the accumulator registers: a 32-lane half holds 32 consecutive channels
// of one output row, so one ballot per output bit yields the two MSB-first words of two rows, and
// the four rows of a 2x2 pooling window (pool order) are four consecutive accumulator registers.
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>

#include "epilogue.h"
#include "kparams.h"
#include "valu_kernel.h"  // load_words, fast_div

namespace apnn {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

template <int P>
__device__ __forceinline__ v4i expand_planes(const uint32_t (&w)[P], const uint32_t (&rot)[P]) {
  uint32_t ys[P];
#pragma unroll
  for (int p = 0; p < P; ++p) ys[p] = __builtin_amdgcn_alignbit(w[p], w[p], rot[p]);
  v4i out;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    uint32_t word = 0;
#pragma unroll
    for (int p = 0; p < P; ++p) word |= (ys[p] >> t) & (0x01010101u << p);
    out[t] = (int)word;
  }
  return out;
}

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

// Output stage for one 32x32 accumulator block.  Register r of the block holds
// row 8*(r/4) + 4*g + (r%4), column li (g = lane / 32, li = lane % 32).
// ssum: activation sum of row li of this block (CONV) or of column li (GEMM entry points).
template <bool CONV>
__device__ __forceinline__ void mfma_epilogue_block(const KParams &p, const v16i &blk, int ssum, int rbase,
                                                    int gcol, int g, int li) {
  const bool col_ok = gcol < p.rowsB;
  const int w32 = p.rowsB >> 5;
  int v[16];
  static_for<0, 16>([&](auto rc) {
    constexpr int r = decltype(rc)::value;
    int t = blk[r];
    if (p.sym) {
      const int rin = 8 * (r >> 2) + 4 * g + (r & 3);
      const int s = CONV ? __shfl(ssum, rin, 64) : ssum;
      t = 2 * t - p.wmax * s;
    }
    v[r] = t;
  });
  if (p.epi == APNN_EPI_INT32) {
    int *out = reinterpret_cast<int *>(p.out);
    static_for<0, 16>([&](auto rc) {
      constexpr int r = decltype(rc)::value;
      const int grow = rbase + 8 * (r >> 2) + 4 * g + (r & 3);
      if (col_ok && grow < p.rowsA) out[(long long)grow * p.rowsB + gcol] = v[r];
    });
  } else if (p.pool == APNN_POOL_NONE) {
    uint32_t *out = reinterpret_cast<uint32_t *>(p.out);
    static_for<0, 16>([&](auto rc) {
      constexpr int r = decltype(rc)::value;
      const int grow = rbase + 8 * (r >> 2) + 4 * g + (r & 3);
      const bool ok = col_ok && grow < p.rowsA;
      int code = 0;
      if (ok) {
        int t = v[r];
        const long long o = (long long)grow * p.rowsB + gcol;
        if (p.resid != nullptr) t += p.resid[o];
        if (p.save_acc != nullptr) p.save_acc[o] = t;
        code = quantize_code(p, t, gcol);
      }
      for (int b = 0; b < p.out_bits; ++b) {
        const unsigned long long mask = __ballot(ok && ((code >> b) & 1));
        const uint32_t word = g ? __brev((uint32_t)(mask >> 32)) : __brev((uint32_t)mask);
        if (ok && li == 0) out[b * p.out_plane + (long long)grow * w32 + (gcol >> 5)] = word;
      }
    });
  } else {
    uint32_t *out = reinterpret_cast<uint32_t *>(p.out);
    const int out_rows_total = p.rowsA / 4;
    static_for<0, 4>([&](auto qc) {
      constexpr int q = decltype(qc)::value;
      const int grow = (rbase + 8 * q + 4 * g) >> 2;  // 2x2 window index
      const bool ok = col_ok && grow < out_rows_total;
      int code = 0;
      if (ok) {
        if (p.pool == APNN_POOL_AVG2X2) {
          code = quantize_code(p, (v[4 * q] + v[4 * q + 1] + v[4 * q + 2] + v[4 * q + 3]) / 4, gcol);
        } else {
          const int c0 = quantize_code(p, v[4 * q], gcol), c1 = quantize_code(p, v[4 * q + 1], gcol);
          const int c2 = quantize_code(p, v[4 * q + 2], gcol), c3 = quantize_code(p, v[4 * q + 3], gcol);
          code = max(max(c0, c1), max(c2, c3));
        }
      }
      for (int b = 0; b < p.out_bits; ++b) {
        const unsigned long long mask = __ballot(ok && ((code >> b) & 1));
        const uint32_t word = g ? __brev((uint32_t)(mask >> 32)) : __brev((uint32_t)mask);
        if (ok && li == 0) out[b * p.out_plane + (long long)grow * w32 + (gcol >> 5)] = word;
      }
    });
  }
}

template <int PA, int PB, int FA, int FB, int WA, int WB, int VW, bool CONV>
__global__ __launch_bounds__(256) void apnn_mfma_kernel(const KParams p) {
  static_assert(WA * WB == 4, "four waves per work-group");
  constexpr int NT = 256;
  constexpr int TA = WA * FA * 32, TB = WB * FB * 32;
  constexpr int KC = 8;              // k-words (32 elements each) per staged chunk
  constexpr int LD = KC + 1;         // odd row pitch: 32 rows hit 32 different banks
  constexpr int KQ = KC / VW;
  constexpr int UA = TA * KQ, UB = TB * KQ;
  constexpr int NIA = (UA + NT - 1) / NT, NIB = (UB + NT - 1) / NT;
  constexpr int BUF_WORDS = (PA * TA + PB * TB) * LD;

  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];  // [2][BUF_WORDS]

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int li = lane & 31, g = lane >> 5;
  const int wa = wave / WB, wb = wave % WB;

  const int tilesB = (p.rowsB + TB - 1) / TB;
  const int a0 = (blockIdx.x / tilesB) * TA;
  const int b0 = (blockIdx.x % tilesB) * TB;

  // ---- staging bookkeeping (same scheme as the VALU kernel) ----------------------------------
  int a_row[NIA], a_kq[NIA];
  int a_b[NIA], a_y0[NIA], a_x0[NIA];
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

  auto stage = [&](uint32_t *buf) {
    uint32_t *As = buf;                   // [PA][TA][LD]
    uint32_t *Bs = buf + PA * TA * LD;    // [PB][TB][LD]
#pragma unroll
    for (int it = 0; it < NIA; ++it) {
      if (UA % NT == 0 || tid + it * NT < UA) {
#pragma unroll
        for (int pl = 0; pl < PA; ++pl)
#pragma unroll
          for (int i = 0; i < VW; ++i) As[(pl * TA + a_row[it]) * LD + a_kq[it] * VW + i] = ra_[it][pl][i];
      }
    }
#pragma unroll
    for (int it = 0; it < NIB; ++it) {
      if (UB % NT == 0 || tid + it * NT < UB) {
#pragma unroll
        for (int pl = 0; pl < PB; ++pl)
#pragma unroll
          for (int i = 0; i < VW; ++i) Bs[(pl * TB + b_row[it]) * LD + b_kq[it] * VW + i] = rb_[it][pl][i];
      }
    }
  };

  v16i acc[FA][FB];
#pragma unroll
  for (int x = 0; x < FA; ++x)
#pragma unroll
    for (int y = 0; y < FB; ++y)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[x][y][r] = 0;

  // activation row sums per plane for the symmetric-weight correction (activations: A for conv,
  // B for the GEMM entry points); always accumulated -- one popcount-accumulate per plane and
  // fragment is cheaper than a branch that would split the k-step into basic blocks
  constexpr int FS = CONV ? FA : FB, PS = CONV ? PA : PB;
  int psum[FS][PS];
#pragma unroll
  for (int x = 0; x < FS; ++x)
#pragma unroll
    for (int pl = 0; pl < PS; ++pl) psum[x][pl] = 0;

  uint32_t rotA[PA], rotB[PB];
#pragma unroll
  for (int pl = 0; pl < PA; ++pl) rotA[pl] = (uint32_t)(4 * g - pl) & 31u;
#pragma unroll
  for (int pl = 0; pl < PB; ++pl) rotB[pl] = (uint32_t)(4 * g - pl) & 31u;

  // packed words of this lane's rows for one k-step
  uint32_t wA[FA][PA], wB[FB][PB];
  auto read_words = [&](const uint32_t *buf, int ks) {
    const uint32_t *As = buf + (wa * FA * 32 + li) * LD + ks;
    const uint32_t *Bs = buf + PA * TA * LD + (wb * FB * 32 + li) * LD + ks;
#pragma unroll
    for (int x = 0; x < FA; ++x)
#pragma unroll
      for (int pl = 0; pl < PA; ++pl) wA[x][pl] = As[(pl * TA + x * 32) * LD];
#pragma unroll
    for (int y = 0; y < FB; ++y)
#pragma unroll
      for (int pl = 0; pl < PB; ++pl) wB[y][pl] = Bs[(pl * TB + y * 32) * LD];
  };
  v4i af[FA], bf[FB];
  auto expand_all = [&](v4i (&a)[FA], v4i (&b)[FB]) {
#pragma unroll
    for (int x = 0; x < FA; ++x) {
      if (CONV) {
#pragma unroll
        for (int pl = 0; pl < PA; ++pl) psum[x][pl] += __popc(wA[x][pl]);
      }
      a[x] = expand_planes<PA>(wA[x], rotA);
    }
#pragma unroll
    for (int y = 0; y < FB; ++y) {
      if (!CONV) {
#pragma unroll
        for (int pl = 0; pl < PB; ++pl) psum[y][pl] += __popc(wB[y][pl]);
      }
      b[y] = expand_planes<PB>(wB[y], rotB);
    }
  };

  // Software pipeline: while the matrix cores work on k-step s, the VALU expands the operands of
  // k-step s+1 (also across the chunk boundary: the barrier that publishes chunk ch+1 sits before
  // the last k-step of chunk ch).  Global loads run two chunks ahead, LDS holds two chunks.
  constexpr int N_MFMA = FA * FB;
  constexpr int N_VALU = FA * 8 * PA + FB * 8 * PB + FS * PS;
  constexpr int VALU_PER_MFMA = (N_VALU + N_MFMA - 1) / N_MFMA;

  const int nchunks = (p.KW + KC - 1) / KC;
  fetch(0);
  stage(smem);
  if (nchunks > 1) fetch(KC);
  __syncthreads();
  read_words(smem, 0);
  expand_all(af, bf);
  for (int ch = 0; ch < nchunks; ++ch) {
    const uint32_t *cur = smem + (ch & 1) * BUF_WORDS;
    uint32_t *nxt = smem + ((ch + 1) & 1) * BUF_WORDS;
    const bool more = ch + 1 < nchunks;
    if (more) {
      stage(nxt);  // every wave left this buffer before the barrier of the previous chunk
      if (ch + 2 < nchunks) fetch((ch + 2) * KC);
    }
#pragma unroll
    for (int ks = 0; ks < KC; ++ks) {
      const bool last = ks == KC - 1;
      if (last) __syncthreads();
      v4i an[FA], bn[FB];
      if (!last) {
        read_words(cur, ks + 1);
      } else if (more) {
        read_words(nxt, 0);
      }
#pragma unroll
      for (int x = 0; x < FA; ++x)
#pragma unroll
        for (int y = 0; y < FB; ++y)
          acc[x][y] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[x], bf[y], acc[x][y], 0, 0, 0);
      if (!last || more) {
        expand_all(an, bn);
#pragma unroll
        for (int x = 0; x < FA; ++x) af[x] = an[x];
#pragma unroll
        for (int y = 0; y < FB; ++y) bf[y] = bn[y];
#pragma unroll
        for (int i = 0; i < N_MFMA; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);              // one MFMA
          __builtin_amdgcn_sched_group_barrier(0x002, VALU_PER_MFMA, 0);  // then its share of VALU work
        }
      }
    }
  }
  int ssum[FS];
#pragma unroll
  for (int x = 0; x < FS; ++x) {
    int t = 0;
#pragma unroll
    for (int pl = 0; pl < PS; ++pl) t += psum[x][pl] << pl;
    ssum[x] = t;
  }

  // ---- epilogue from registers ---------------------------------------------------------------
  // Every accumulator index below is a compile-time constant (static_for), so the accumulators
  // stay in registers for the whole kernel.
  static_for<0, FA>([&](auto xc) {
    static_for<0, FB>([&](auto yc) {
      constexpr int x = decltype(xc)::value, y = decltype(yc)::value;
      const int gcol = b0 + (wb * FB + y) * 32 + li;
      const int rbase = a0 + (wa * FA + x) * 32;
      mfma_epilogue_block<CONV>(p, acc[x][y], ssum[CONV ? x : y], rbase, gcol, g, li);
    });
  });
}

template <int PA, int PB, int FA, int FB, int WA, int WB, int VW, bool CONV>
inline hipError_t launch_mfma(const KParams &p, hipStream_t stream) {
  constexpr int TA = WA * FA * 32, TB = WB * FB * 32;
  constexpr int LD = 9;
  constexpr size_t smem_bytes = 2ull * (PA * TA + PB * TB) * LD * sizeof(uint32_t);
  static_assert(smem_bytes <= 160 * 1024, "LDS budget of a gfx950 work-group");
  auto kern = apnn_mfma_kernel<PA, PB, FA, FB, WA, WB, VW, CONV>;
  if (smem_bytes > 64 * 1024) {
    static bool raised = false;  // per instantiation; a repeated call is harmless
    if (!raised) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_bytes);
      if (e != hipSuccess) return e;
      raised = true;
    }
  }
  const long long tiles = (long long)((p.rowsA + TA - 1) / TA) * ((p.rowsB + TB - 1) / TB);
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(256), smem_bytes, stream, p);
  return hipGetLastError();
}

enum MfmaTile { MT_256x256 = 0, MT_128x128 = 1, MT_64x64 = 2, MT_128x64 = 3, MT_COUNT = 4 };

template <int PA, int PB, int VW, bool CONV>
inline hipError_t launch_mfma_tile(int tile, const KParams &p, hipStream_t stream) {
  switch (tile) {
    case MT_256x256: return launch_mfma<PA, PB, 4, 4, 2, 2, VW, CONV>(p, stream);
    case MT_128x128: return launch_mfma<PA, PB, 2, 2, 2, 2, VW, CONV>(p, stream);
    case MT_128x64: return launch_mfma<PA, PB, 1, 2, 4, 1, VW, CONV>(p, stream);
    default: return launch_mfma<PA, PB, 1, 1, 2, 2, VW, CONV>(p, stream);
  }
}

}  // namespace apnn
