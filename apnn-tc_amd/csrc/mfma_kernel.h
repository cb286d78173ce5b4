// MFMA path: bit-planes are expanded in registers to small matrix-core operands and contracted on
// the matrix cores:  sum_ij 2^(i+j) popc(x_i & w_j) == sum_k xval[k] * wval[k]  with
// xval = sum_i 2^i x_i[k] and wval likewise.  Two operand encodings (template parameter CORE):
//
//  CORE_I8  v_mfma_i32_32x32x32_i8: operand bytes hold xval / wval (0..15); one instruction per 32x32
//           block and 32 k, exact in int8 x int8 -> int32.
//  CORE_F4  v_mfma_f32_32x32x64_f8f6f4 with FP4 (e2m1) operands: the codes 0..3 of e2m1 are the values
//           0, 0.5, 1, 1.5, i.e. a 2-bit digit v is the code v and means v/2.  Operands are split into
//           2-bit digits (plane pairs); digit pair (da, db) is one instruction per 32x32 block and
//           64 k -- at the same issue cost as the int8 instruction, so twice its rate -- with the
//           weight 4^(da+db) applied by the instruction's E8M0 block scale.  Products are multiples
//           of 1/4 and the host only launches this core while K * (2^w - 1) * (2^a - 1) < 2^24, so the
//           fp32 accumulators are exact and the result is acc * 4.
//
// Work-group = 4 waves arranged WA x WB, each wave owning an (FA*32) x (FB*32) output tile
// (FA*FB accumulator blocks of 16 registers).  The *packed* planes are staged through LDS
// (row-major, double-buffered, one barrier per chunk of KC words); every wave reads the one packed
// word per row and k-step that it needs and expands it in registers:
//   lane (i, g) of a wave supplies row i and the 16 k-positions { 8c + 4g + t : c,t < 4 } of the
//   word -- the same positions for both operands, so the contraction pairs bit k with bit k as the
//   reference does (APNN-TC-lib/bmmaTensorCoreGemm/src/71_bmmaTensorCoreGemm.cu:364-369).
//   CORE_I8: ys_p = rotr(word_p, 4g - p);  byte-word t = OR_p ((ys_p >> t) & (0x01010101 << p)),
//   i.e. 8 VALU operations per plane for 16 int8 operands; CORE_F4: see expand_fp4.
//
// Symmetric (+-) weights use the closed form  2*raw - wmax * (activation row sum); the row sums
// come from popcounts of the packed words the wave already holds.
//
// Output: int32 results and codes of up to two bits (four where the waves tile the output) leave
// straight from the accumulator registers (store_int32_direct, direct_epilogue); int32 residuals, saved
// accumulators and wider codes pass each wave's tile through an LDS slab, 32 rows at a time, which turns
// the matrix-core register layout into row-major order.
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>

#include "dispatch.h"
#include "epilogue.h"
#include "kparams.h"
#include "valu_kernel.h"  // load_words, fast_div

namespace apnn {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

// FP4 operand for digit D (planes 2D and, if present, 2D+1) of a P-plane row word: nibble c of
// result word t is the digit of element 4c + t.
// One plane: shift and mask per result word, 7 operations.  Two planes: the planes are first merged
// into two words of sixteen 2-bit digits (even elements, odd elements; one bit-field insert each), and
// every result word is a shift and a mask of one of those, 10 operations instead of 14 for separate
// shifts and masks of both planes.
template <int P, int D>
__device__ __forceinline__ v8i expand_fp4(const uint32_t (&w)[P]) {
  v8i out = {0, 0, 0, 0, 0, 0, 0, 0};
  const uint32_t x0 = w[2 * D];
  if constexpr (2 * D + 1 < P) {
    const uint32_t x1 = w[2 * D + 1];
    constexpr uint32_t EVEN = 0x55555555u;
    // digit of element 2i at bits 2i, 2i+1
    uint32_t qe = (x0 & EVEN) | ((x1 << 1) & ~EVEN);
    uint32_t qo = ((x0 >> 1) & EVEN) | (x1 & ~EVEN);
    // keep the merged words: without this the optimizer distributes the masks below over the two
    // planes again and emits the 14-operation form
    asm("" : "+v"(qe));
    asm("" : "+v"(qo));
    out[0] = (int)(qe & 0x33333333u);
    out[1] = (int)(qo & 0x33333333u);
    out[2] = (int)((qe >> 2) & 0x33333333u);
    out[3] = (int)((qo >> 2) & 0x33333333u);
  } else {
#pragma unroll
    for (int t = 0; t < 4; ++t) out[t] = (int)((x0 >> t) & 0x11111111u);
  }
  return out;
}

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

// old with lanes LANE_LO / LANE_HI replaced by the wave-uniform values lo / hi (v_writelane_b32: one VALU
// operation each).  A vector instruction that reads a scalar register written by the vector instruction
// just before it (a compare mask) needs wait states that the compiler inserts only for instructions it
// can see -- not for this opaque assembly -- so the block waits by itself (s_nop 1) and is safe whatever
// produced its scalar sources.
template <int LANE_LO, int LANE_HI>
__device__ __forceinline__ int write_lane_pair(int lo, int hi, int old) {
  static_assert(LANE_LO >= 0 && LANE_LO < 64 && LANE_HI >= 0 && LANE_HI < 64, "lane index");
  asm("s_nop 1\n\t"
      "v_writelane_b32 %0, %1, %3\n\t"
      "v_writelane_b32 %0, %2, %4"
      : "+v"(old)
      : "s"(lo), "s"(hi), "n"(LANE_LO), "n"(LANE_HI));
  return old;
}

// Quantize-and-pack output stage that works straight from the accumulator registers (no transpose
// through LDS).  In the matrix-core layout lane (li, g) holds column li of a 32x32 block and, in
// register r, row 8*(r/4) + 4*g + r%4.  The channel (column) is therefore fixed per lane: its
// thresholds live in registers, and a compare over the wave IS the ballot -- the 64-bit compare mask
// of register r holds the 32 channel bits of two output rows (one per lane half).  For a 2-bit code
// with sorted thresholds t0 <= t1 <= t2:  bit1 = v >= t1,  bit0 = v >= (bit1 ? t2 : t0): two
// compares and one select per 64 outputs.  Codes of 3 or 4 bits binary-search a threshold table in
// LDS, one compare per output bit (TABLE).  The masks are bit-reversed (channel c -> bit 31 - c%32)
// and parked in the lane whose index is the output row; after a block is finished each lane stores
// its row's words.  The four rows of a 2x2 pooling window (pool order) are the four registers
// 4q..4q+3 of one lane, so pooling is register-local.
//
// Row-dependent terms come from LDS with 16-byte broadcast reads (four consecutive rows):
//   lds[0 .. FA*32)                          activation row sums times the weight range (convolution,
//                                            symmetric weights; zero otherwise)
//   lds[FA*32 .. FA*32 + FA*2*FB*32)         shortcut words, index ((x*2 + plane)*FB + y)*32 + row
//   lds[FA*32 + FA*64*FB ...)                threshold table [k][FB*32] (TABLE only), filled here
// Q0, Q1: the register quads (rows 8q .. 8q+7 of a block) this call finishes; the split-K tiles give
// each of their four waves one quad of the summed block.
template <bool F4, int FA, int FB, bool CONV, bool TABLE, int Q0 = 0, int Q1 = 4, class AccT>
__device__ __forceinline__ void direct_epilogue(const KParams &p, AccT (&acc)[FA][FB],
                                                const int (&ssum)[CONV ? FA : FB], uint32_t *lds, int rbase,
                                                int cbase, int lane, const int (&T)[FB][3], const int (&fm)[FB],
                                                bool shortcut, const int *shared_table = nullptr) {
  constexpr int NCOLS = FB * 32;
  constexpr int NPARK = TABLE ? 2 : 1;
  const int li = lane & 31, g = lane >> 5;
  const int nb = p.out_bits;
  const bool bn = p.epi == APNN_EPI_BN;
  const int sh = p.sym ? 1 : 0;
  const int wmax = p.sym ? p.wmax : 0;
  const bool pooled = p.pool != APNN_POOL_NONE;
  const int lowmask = (1 << nb) - 1;
  const int bitpos = 31 - li;
  const int w32 = p.rowsB >> 5;
  const int *rowsum = reinterpret_cast<const int *>(lds);
  const uint32_t *res = lds + FA * 32;
  // threshold table [k][NCOLS]: this wave's own copy, filled here, or one the caller filled for the tile
  int *own_table = reinterpret_cast<int *>(lds + FA * 32 + FA * 64 * FB);
  const int *tl = shared_table != nullptr ? shared_table : own_table;
  if (TABLE && bn && shared_table == nullptr) {
    const int nt = (1 << nb) - 1;
#pragma unroll
    for (int y = 0; y < FB; ++y) {
      const int gcol = cbase + y * 32 + li;
      if (gcol < p.rowsB)
        for (int k = g; k < nt; k += 2) own_table[k * NCOLS + y * 32 + li] = p.thr[(long long)gcol * nt + k];
    }
  }
  int cneg[FB];  // GEMM entry points: the correction depends on the column only
#pragma unroll
  for (int y = 0; y < FB; ++y) cneg[y] = CONV ? 0 : -wmax * ssum[CONV ? 0 : y];

  // Float form of the 2-bit threshold compare (FP4 core): the accumulator is acc = raw / 4 in fp32, and
  // with every operand an integer below 2^24 in magnitude (the host checked: KParams::epi_float)
  //   v = 2^sh * 4 * acc - correction (+ shortcut)  is one exact fused multiply-add on the accumulator,
  // compared with the thresholds converted to float (clamped to +-2^24, which no value reaches): four
  // vector operations per value instead of nine (multiply, convert, shift, subtract, sign flip x2,
  // compare, select, compare).  Taken when no channel of this wave's tile has the flip flag.
  float Tf[FB][3];
  float cnegf[FB];
  bool fast = false;
  if constexpr (F4 && !TABLE) {
    int anyflip = 0;
#pragma unroll
    for (int y = 0; y < FB; ++y) {
      anyflip |= fm[y];
      cnegf[y] = (float)cneg[y];
#pragma unroll
      for (int k = 0; k < 3; ++k) Tf[y][k] = (float)min(max(T[y][k], -(1 << 24)), 1 << 24);
    }
    fast = bn && p.epi_float != 0 && p.pool != APNN_POOL_AVG2X2 && __ballot(anyflip != 0) == 0ull;
  }
  const float vscale = p.sym ? 8.0f : 4.0f;

  // The epilogue mode (thresholds or low bits, pooled or not) is the same for the whole launch: the
  // value loop is instantiated once per mode and entered through one branch, so the per-value code
  // carries no mode tests.
  auto run = [&](auto bn_c, auto pooled_c, auto fast_c) {
    constexpr bool BN = decltype(bn_c)::value, POOLED = decltype(pooled_c)::value;
    constexpr bool FAST = decltype(fast_c)::value;
    static_for<0, FA>([&](auto xc) {
      constexpr int x = decltype(xc)::value;
      uint32_t park[FB][NPARK];
#pragma unroll
      for (int y = 0; y < FB; ++y)
#pragma unroll
        for (int k = 0; k < NPARK; ++k) park[y][k] = 0;

      static_for<Q0, Q1>([&](auto qc) {
        constexpr int q = decltype(qc)::value;
        int negc[4] = {0, 0, 0, 0};
        float negcf[4] = {0.f, 0.f, 0.f, 0.f};
        if (CONV) {
          // the row sums were multiplied by the weight range when they were written
          const int4 rs = *reinterpret_cast<const int4 *>(rowsum + x * 32 + 8 * q + 4 * g);
          negc[0] = -rs.x;
          negc[1] = -rs.y;
          negc[2] = -rs.z;
          negc[3] = -rs.w;
          if constexpr (FAST) {
#pragma unroll
            for (int j = 0; j < 4; ++j) negcf[j] = (float)negc[j];
          }
        }
        static_for<0, FB>([&](auto yc) {
          constexpr int y = decltype(yc)::value;
          int v[4];
          float u[4];
          static_for<0, 4>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            if constexpr (FAST) {
              u[j] = __builtin_fmaf((float)acc[x][y][4 * q + j], vscale, CONV ? negcf[j] : cnegf[y]);
              v[j] = 0;
            } else {
              if constexpr (F4) {
                // acc * vscale is an integer already (also with a folded shortcut, which adds multiples
                // of 1 / vscale): the conversion is exact
                v[j] = (int)(acc[x][y][4 * q + j] * vscale) + (CONV ? negc[j] : cneg[y]);
              } else {
                v[j] = (acc[x][y][4 * q + j] << sh) + (CONV ? negc[j] : cneg[y]);
              }
              u[j] = 0.f;
            }
          });
          if (!POOLED && shortcut) {
            uint32_t rw[2][4];
#pragma unroll
            for (int b = 0; b < 2; ++b) {
              const uint4 w4 = *reinterpret_cast<const uint4 *>(res + ((x * 2 + b) * FB + y) * 32 + 8 * q + 4 * g);
              rw[b][0] = w4.x;
              rw[b][1] = w4.y;
              rw[b][2] = w4.z;
              rw[b][3] = w4.w;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int code = (int)(((rw[0][j] >> bitpos) & 1u) | (((rw[1][j] >> bitpos) & 1u) << 1));
              if constexpr (FAST) {
                u[j] += (float)(code * p.resid_scale);
              } else {
                v[j] += code * p.resid_scale;
              }
            }
          }
          // one item: value (or code) -> one ballot per output bit, words parked at lanes rlo (lane
          // half 0's row) and rhi (lane half 1's row)
          auto emit = [&](auto val, auto rlo_c, auto rhi_c) {
            using ValT = decltype(val);
            constexpr int rlo = decltype(rlo_c)::value, rhi = decltype(rhi_c)::value;
            auto put = [&](auto slot_c, unsigned long long mask) {
              constexpr int slot = decltype(slot_c)::value;
              // bit reversal: channel c -> bit 31 - c%32 (scalar unit)
              const int lo = (int)__brev((uint32_t)mask), hi = (int)__brev((uint32_t)(mask >> 32));
              park[y][slot >> 1] = (uint32_t)write_lane_pair<rlo + 32 * (slot & 1), rhi + 32 * (slot & 1)>(
                  lo, hi, (int)park[y][slot >> 1]);
            };
            if constexpr (std::is_same<ValT, float>::value) {
              const bool hi1 = val >= Tf[y][1];
              put(std::integral_constant<int, 1>{}, __ballot(hi1));
              const float tsel = hi1 ? Tf[y][2] : Tf[y][0];
              put(std::integral_constant<int, 0>{}, __ballot(val >= tsel));
            } else if constexpr (!BN) {
              static_for<0, 2 * NPARK>([&](auto bc) {
                constexpr int b = decltype(bc)::value;
                if (b < nb) put(bc, __ballot((val >> b) & 1));
              });
            } else if constexpr (!TABLE) {
              const bool hi1 = val >= T[y][1];
              put(std::integral_constant<int, 1>{}, __ballot(hi1));
              const int tsel = hi1 ? T[y][2] : T[y][0];
              put(std::integral_constant<int, 0>{}, __ballot(val >= tsel));
            } else {
              int idx = (1 << (nb - 1)) - 1, h = 1 << (nb - 1);
              static_for<0, 4>([&](auto lc) {
                constexpr int lvl = decltype(lc)::value;
                if (lvl < nb) {
                  h >>= 1;
                  const bool d = val >= tl[idx * NCOLS + y * 32 + li];
                  put(lc, __ballot(d));
                  idx += d ? h : -h;
                }
              });
            }
          };
          auto flipped = [&](int t) { return (t ^ fm[y]) - fm[y]; };
          if constexpr (FAST) {
            if constexpr (!POOLED) {
              static_for<0, 4>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                emit(u[j], std::integral_constant<int, 8 * q + j>{}, std::integral_constant<int, 8 * q + 4 + j>{});
              });
            } else {  // max pooling of codes == code of the maximum (thresholds are monotone, no flip here)
              emit(fmaxf(fmaxf(u[0], u[1]), fmaxf(u[2], u[3])), std::integral_constant<int, 2 * q>{},
                   std::integral_constant<int, 2 * q + 1>{});
            }
          } else if constexpr (!POOLED) {
            static_for<0, 4>([&](auto jc) {
              constexpr int j = decltype(jc)::value;
              emit(BN ? flipped(v[j]) : (v[j] & lowmask), std::integral_constant<int, 8 * q + j>{},
                   std::integral_constant<int, 8 * q + 4 + j>{});
            });
          } else {
            int val;
            if (p.pool == APNN_POOL_AVG2X2) {
              const int a = (v[0] + v[1] + v[2] + v[3]) / 4;
              val = BN ? flipped(a) : (a & lowmask);
            } else if (BN) {
              val = max(max(flipped(v[0]), flipped(v[1])), max(flipped(v[2]), flipped(v[3])));
            } else {
              val = max(max(v[0] & lowmask, v[1] & lowmask), max(v[2] & lowmask, v[3] & lowmask));
            }
            emit(val, std::integral_constant<int, 2 * q>{}, std::integral_constant<int, 2 * q + 1>{});
          }
        });
      });

      // lane L holds, in park[y][k], the word of block row L%32 for slot 2k + L/32
      const int row = lane & 31;
      const int rows_blk = POOLED ? 8 : 32;
      const int grow = (POOLED ? (rbase >> 2) + x * 8 : rbase + x * 32) + row;
      const int grow_end = POOLED ? (p.rowsA >> 2) : p.rowsA;
      uint32_t *out = reinterpret_cast<uint32_t *>(p.out);
      const int gw0 = cbase >> 5;
#pragma unroll
      for (int k = 0; k < NPARK; ++k) {
        const int slot = 2 * k + (lane >> 5);
        const int plane = (TABLE && BN) ? nb - 1 - slot : slot;
        const bool row_mine =
            (Q0 == 0 && Q1 == 4) || (POOLED ? (row >= 2 * Q0 && row < 2 * Q1) : (row >= 8 * Q0 && row < 8 * Q1));
        if (plane >= 0 && plane < nb && row < rows_blk && row_mine && grow < grow_end && gw0 < w32) {
          uint32_t *dst = out + plane * p.out_plane + (long long)grow * w32 + gw0;
          if (FB == 4 && (w32 & 3) == 0) {
            *reinterpret_cast<uint4 *>(dst) = make_uint4(park[0][k], park[FB > 1 ? 1 : 0][k], park[FB > 2 ? 2 : 0][k],
                                                         park[FB > 3 ? 3 : 0][k]);
          } else if (FB == 2 && (w32 & 1) == 0) {
            *reinterpret_cast<uint2 *>(dst) = make_uint2(park[0][k], park[FB > 1 ? 1 : 0][k]);
          } else {
#pragma unroll
            for (int y = 0; y < FB; ++y)
              if (gw0 + y < w32) dst[y] = park[y][k];
          }
        }
      }
    });
  };
  using std::false_type;
  using std::true_type;
  if constexpr (F4 && !TABLE) {
    if (fast) {
      if (pooled) run(true_type{}, true_type{}, true_type{}); else run(true_type{}, false_type{}, true_type{});
      return;
    }
  }
  if (bn) {
    if (pooled) run(true_type{}, true_type{}, false_type{}); else run(true_type{}, false_type{}, false_type{});
  } else {
    if (pooled) run(false_type{}, true_type{}, false_type{}); else run(false_type{}, false_type{}, false_type{});
  }
}

// int32 output straight from the accumulators.  Register r of a 32x32 block is row 8*(r/4) + 4*g + r%4,
// column li, and the output is row-major with the column index fastest, so one store instruction of the
// wave writes two full 128-byte rows of the block (one per lane half): no LDS round trip, two vector
// operations per value (scale, convert) and one address update per output row.  lds[0 .. FA*32) holds
// the activation row sums times the weight range (convolution with symmetric weights; unused otherwise).
template <bool F4, int FA, int FB, bool CONV, class AccT>
__device__ __forceinline__ void store_int32_direct(const KParams &p, AccT (&acc)[FA][FB],
                                                   const int (&ssum)[CONV ? FA : FB], const uint32_t *lds,
                                                   int rbase, int cbase, int lane) {
  const int li = lane & 31, g = lane >> 5;
  const int sh = p.sym ? 1 : 0;
  const int wmax = p.sym ? p.wmax : 0;
  const int *rowsum = reinterpret_cast<const int *>(lds);
  int cneg[FB];
  float cnegf[FB];
#pragma unroll
  for (int y = 0; y < FB; ++y) {
    cneg[y] = CONV ? 0 : -wmax * ssum[CONV ? 0 : y];
    cnegf[y] = (float)cneg[y];
  }
  // FP4 core: value = acc * 4 * 2^sym - correction as one fused multiply-add in fp32 and one conversion
  // (the host launches this core only while every such value is an integer below 2^24, so both are exact)
  const float vscale = p.sym ? 8.0f : 4.0f;
  int *out = reinterpret_cast<int *>(p.out);
  const long long pitch = p.rowsB;
  const bool full = rbase + FA * 32 <= p.rowsA && cbase + FB * 32 <= p.rowsB;  // same for the whole wave
  auto run = [&](auto full_c) {
    constexpr bool FULL = decltype(full_c)::value;
    int *rowp = out + (long long)(rbase + 4 * g) * pitch + cbase + li;
    static_for<0, FA>([&](auto xc) {
      constexpr int x = decltype(xc)::value;
      static_for<0, 4>([&](auto qc) {
        constexpr int q = decltype(qc)::value;
        int negc[4] = {0, 0, 0, 0};
        float negcf[4] = {0.f, 0.f, 0.f, 0.f};
        if (CONV && p.sym) {
          const int4 rs = *reinterpret_cast<const int4 *>(rowsum + x * 32 + 8 * q + 4 * g);
          negc[0] = -rs.x;
          negc[1] = -rs.y;
          negc[2] = -rs.z;
          negc[3] = -rs.w;
#pragma unroll
          for (int j = 0; j < 4; ++j) negcf[j] = (float)negc[j];
        }
        static_for<0, 4>([&](auto jc) {
          constexpr int j = decltype(jc)::value;
          int *dst = rowp + (long long)(x * 32 + 8 * q + j) * pitch;
          const bool row_ok = FULL || rbase + x * 32 + 8 * q + 4 * g + j < p.rowsA;
          static_for<0, FB>([&](auto yc) {
            constexpr int y = decltype(yc)::value;
            int v;
            if constexpr (F4) {
              v = (int)__builtin_fmaf((float)acc[x][y][4 * q + j], vscale, CONV ? negcf[j] : cnegf[y]);
            } else {
              v = (acc[x][y][4 * q + j] << sh) + (CONV ? negc[j] : cneg[y]);
            }
            if (FULL || (row_ok && cbase + y * 32 + li < p.rowsB)) dst[y * 32] = v;
          });
        });
      });
    });
  };
  if (full) run(std::true_type{}); else run(std::false_type{});
}

// Output stage of one wave for a 32-row slab of its tile, staged in LDS as slab[32][NCOLS + 1]
// (row-major, so the 64 lanes walk 64 consecutive output channels).  rowsum / colsum hold the
// activation sums for the symmetric-weight correction (rows for convolution, columns for the GEMM
// entry points).  Called by all 64 lanes of the wave; no other wave touches this slab.
// With KS > 1 the KS waves of the work-group each hold a partial sum over their share of K in their
// own slab (slab_stride words apart, sums included); every wave then finishes 1/KS of the elements,
// adding the KS partial slabs.  `part` is this wave's index among them.
template <int NCOLS, bool CONV, int KS>
__device__ __forceinline__ void wave_epilogue(const KParams &p, const int *slab, const int *rowsum,
                                              const int *colsum, int slab_stride, int part, int rbase, int cbase,
                                              int lane, const ChannelQuant &q0, const ChannelQuant &q1,
                                              const uint32_t *res_lds) {
  constexpr int LDT = NCOLS + 1;
  auto value = [&](int row, int col) {
    int v = 0, sx = 0;
#pragma unroll
    for (int w = 0; w < KS; ++w) {
      v += slab[w * slab_stride + row * LDT + col];
      sx += CONV ? rowsum[w * slab_stride + row] : colsum[w * slab_stride + col];
    }
    if (p.sym) v = 2 * v - p.wmax * sx;
    return v;
  };
  if (p.epi == APNN_EPI_INT32) {
    int *out = reinterpret_cast<int *>(p.out);
    if ((p.rowsB & 3) == 0) {
      // 4 channels per lane: a wave writes 1 KiB of contiguous output per step
      for (int e = lane * 4 + part * 256; e < 32 * NCOLS; e += 256 * KS) {
        const int row = e / NCOLS, col = e % NCOLS;
        const int grow = rbase + row, gcol = cbase + col;
        if (grow < p.rowsA && gcol < p.rowsB) {
          int4 v4;
          v4.x = value(row, col);
          v4.y = value(row, col + 1);
          v4.z = value(row, col + 2);
          v4.w = value(row, col + 3);
          *reinterpret_cast<int4 *>(out + (long long)grow * p.rowsB + gcol) = v4;
        }
      }
    } else {
      for (int e = lane + part * 64; e < 32 * NCOLS; e += 64 * KS) {
        const int row = e / NCOLS, col = e % NCOLS;
        const int grow = rbase + row, gcol = cbase + col;
        if (grow < p.rowsA && gcol < p.rowsB) out[(long long)grow * p.rowsB + gcol] = value(row, col);
      }
    }
    return;
  }
  if (KS > 1 && p.out_bits <= 2 && p.resid == nullptr && p.save_acc == nullptr &&
      (p.resid_planes == nullptr || res_lds != nullptr)) {
    pack_rows_burst<32, NCOLS, KS>(p, value, rbase, cbase, part, q0, q1, res_lds);
  } else {
    pack_rows<NCOLS>(p, value, 32, rbase, cbase, part, KS, q0, q1, res_lds);
  }
}

// Shortcut add on the matrix cores (FP4 core, shortcut codes of one or two bits).  The term
// resid_scale * code[row][channel] of a 32x32 block is the product of the 32x32 matrix of codes (an FP4
// operand like any activation row: digit v means v/2) with a scaled identity, so one more matrix
// instruction per block adds it to the accumulator -- instead of two bit extracts, a merge, a multiply, a
// conversion and an add per output value in the vector ALUs.  The scale travels as FP4 value x E8M0 block
// scale; the two lane halves (k positions 0..31 and 32..63) both see the codes and carry one term each, so
// resid_scale = t0 + t1 with t = +-{1, 3} * 2^j (the host finds the terms: KParams::fold, 0 when there
// are none or fp32 would round).  res: the wave's published shortcut words, index
// ((x * 2 + plane) * FB + y) * 32 + row.
template <int FA, int FB>
__device__ __forceinline__ void fold_shortcut(const KParams &p, v16f (&acc)[FA][FB], const uint32_t *res, int lane) {
  const int li = lane & 31, g = lane >> 5;
  const uint32_t nib = (p.fold >> (4 * g)) & 0xfu;
  const uint32_t e8 = (p.fold >> (8 + 8 * g)) & 0xffu;
  const int scale_b = (int)(e8 * 0x01010101u);
  // identity column li: the shortcut planes hold channel c at bit 31 - c%32, and element e of a packed word
  // is nibble e / 4 of operand word e % 4 (expand_fp4), so channel li pairs with element e = 31 - li
  const int e = 31 - li;
  const uint32_t one = nib << (4 * (e >> 2));
  const v8i bop = {(e & 3) == 0 ? (int)one : 0, (e & 3) == 1 ? (int)one : 0, (e & 3) == 2 ? (int)one : 0,
                   (e & 3) == 3 ? (int)one : 0, 0, 0, 0, 0};
  static_for<0, FA>([&](auto xc) {
    constexpr int x = decltype(xc)::value;
    static_for<0, FB>([&](auto yc) {
      constexpr int y = decltype(yc)::value;
      uint32_t w[2];
      w[0] = res[((x * 2 + 0) * FB + y) * 32 + li];
      w[1] = p.resid_bits > 1 ? res[((x * 2 + 1) * FB + y) * 32 + li] : 0u;
      const v8i aop = expand_fp4<2, 0>(w);
      acc[x][y] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(aop, bop, acc[x][y], 4, 4, 0, 0x7F7F7F7F, 0, scale_b);
    });
  });
}

// Epilogue operands a wave requests before its K loop and consumes after it.
template <int FA, int FB>
struct EpiOperands {
  bool direct;            // quantize straight from the accumulators (see direct_epilogue)
  bool res_prefetched;    // shortcut words are in res_regs
  ChannelQuant q0, q1;    // slab path (split-K kernels)
  int thrT[FB][3], flipm[FB];
  uint32_t res_regs[FA][FB];
};

// rbase / cbase: first output row / column of this wave's tile.  Kernels quantize straight from the
// accumulators when the epilogue allows it (`direct`; codes of up to DIRECT_BITS bits where the waves
// tile the output, up to two bits in the split-K kernels); the remaining epilogues go through the slab.
template <int KS, int FA, int FB>
__device__ __forceinline__ void epi_load(const KParams &p, int rbase, int cbase, int lane, EpiOperands<FA, FB> &eo) {
  constexpr int NCOLS_E = FB * 32;
  constexpr int RES_REGS = FB;  // two planes x 32 rows x NCOLS/32 words over 64 lanes
  const int li = lane & 31;
  if (p.epi == APNN_EPI_INT32) return;
  if (eo.direct) {
#pragma unroll
    for (int y = 0; y < FB; ++y) {
      const int gcol = cbase + y * 32 + li;
      eo.thrT[y][0] = eo.thrT[y][1] = eo.thrT[y][2] = 0;
      eo.flipm[y] = 0;
      if (p.epi == APNN_EPI_BN && gcol < p.rowsB) {
        eo.flipm[y] = (p.flip != nullptr && p.flip[gcol] != 0) ? -1 : 0;
        if (p.out_bits <= 2) {
          const int nt = (1 << p.out_bits) - 1;
          const int32_t *t = p.thr + (long long)gcol * nt;
          eo.thrT[y][0] = t[0];
          eo.thrT[y][1] = nt > 1 ? t[1] : t[0];
          eo.thrT[y][2] = nt > 2 ? t[2] : t[0];
        }
      }
    }
  } else if (KS > 1) {
    load_tile_quant<NCOLS_E>(p, cbase, eo.q0, eo.q1);
  }
  if (p.resid_planes != nullptr && p.resid_bits <= 2 && p.pool == APNN_POOL_NONE && (eo.direct || KS > 1)) {
#pragma unroll
    for (int x = 0; x < FA; ++x) {
      if (eo.direct)
        shortcut_prefetch<NCOLS_E, RES_REGS, true>(p, 32, rbase + x * 32, cbase, lane, 64, eo.res_regs[x]);
      else
        shortcut_prefetch<NCOLS_E, RES_REGS, false>(p, 32, rbase + x * 32, cbase, lane, 64, eo.res_regs[x]);
    }
    eo.res_prefetched = true;
  }
}

// LAZY: only decide the output path now and fetch the operands in epi_finish (the largest tiles have no
// registers to spare for values that are idle during the K loop).
template <int KS, int DIRECT_BITS, bool LAZY, int FA, int FB>
__device__ __forceinline__ void epi_prefetch(const KParams &p, int rbase, int cbase, int lane, EpiOperands<FA, FB> &eo) {
  eo.direct = p.epi != APNN_EPI_INT32 && p.out_bits <= DIRECT_BITS && p.resid == nullptr &&
              p.save_acc == nullptr && (p.resid_planes == nullptr || p.resid_bits <= 2);
  eo.q0 = ChannelQuant{};
  eo.q1 = ChannelQuant{};
  eo.res_prefetched = false;
  if (!LAZY) epi_load<KS>(p, rbase, cbase, lane, eo);
}

// Output stage of a work-group of four waves (WA x WB of them tile the output, KS = 4 / (WA*WB) split
// K).  acc: this wave's FA x FB accumulator blocks; ssum: activation sums of the lane's row li of each
// row block (convolution) or column li of each column block (GEMM entry points), complete in every
// lane.  smem: the work-group's LDS, free for reuse after the barrier at the top.
template <bool F4, int KS, bool CONV, int DIRECT_BITS, bool LAZY, int FA, int FB, class AccT>
__device__ __forceinline__ void epi_finish(const KParams &p, AccT (&acc)[FA][FB], const int (&ssum)[CONV ? FA : FB],
                                           uint32_t *smem, int wave, int lane, int a0, int b0, int wa, int wb,
                                           EpiOperands<FA, FB> &eo) {
  const int li = lane & 31, g = lane >> 5;
  if (LAZY) epi_load<KS>(p, a0 + wa * FA * 32, b0 + wb * FB * 32, lane, eo);
  constexpr int RES_REGS = FB;
  const bool direct = eo.direct, res_prefetched = eo.res_prefetched;
  ChannelQuant &q0 = eo.q0, &q1 = eo.q1;
  auto &thrT = eo.thrT;
  auto &flipm = eo.flipm;
  auto &res_regs = eo.res_regs;
  // ---- epilogue: one 32-row slab of the wave tile at a time through LDS ----------------------
  // Accumulator indices are compile-time constants (static_for) so they stay in registers; the
  // slab turns the matrix-core layout (register r of a block = row 8*(r/4) + 4*g + r%4, column li)
  // into row-major order for coalesced stores and 64-channel ballots.
  constexpr int NCOLS = FB * 32, LDT = NCOLS + 1;
  constexpr int RES_WORDS = 2 * 32 * (NCOLS / 32);
  constexpr int SLAB_WORDS = 32 * LDT + 32 + NCOLS + RES_WORDS;
  constexpr int DIRECT_WORDS = FA * 32 + FA * 64 * FB + 15 * NCOLS;
  static_assert(DIRECT_WORDS <= SLAB_WORDS, "the register epilogue reuses the slab area");
  __syncthreads();  // every wave is done with the staging buffers
  if constexpr (KS > 1) {
    if (direct) {
      // Split-K: the KS partial blocks meet in LDS in the accumulator's own register layout (16 bytes
      // per lane and register quad), then wave q sums quad q of every column block -- rows 8q .. 8q+7 --
      // and finishes it like a wave of the other kernels finishes its own accumulators.
      using Acc4 = typename std::conditional<F4, float4, int4>::type;
      constexpr int PART_WORDS = KS * FB * 4 * 64 * 4;
      constexpr int SUM_WORDS = KS * FB * 32;
      constexpr int AREA_WORDS = 32 + 64 * FB;
      // codes of three or four bits: one threshold table [15][NCOLS] for the tile, behind the waves' areas
      // (the four waves finish different rows of the same columns)
      constexpr int TABLE_WORDS = DIRECT_BITS > 2 ? 15 * NCOLS : 0;
      static_assert(PART_WORDS + SUM_WORDS + KS * AREA_WORDS + TABLE_WORDS <= KS * SLAB_WORDS + TABLE_WORDS,
                    "fits the slab area");
      Acc4 *part = reinterpret_cast<Acc4 *>(smem);
      int *sums = reinterpret_cast<int *>(smem) + PART_WORDS;
      uint32_t *area = smem + PART_WORDS + SUM_WORDS + wave * AREA_WORDS;
      int *table = reinterpret_cast<int *>(smem) + KS * SLAB_WORDS;
      const bool use_table = DIRECT_BITS > 2 && p.out_bits > 2;
      if (DIRECT_BITS > 2 && use_table && p.epi == APNN_EPI_BN) {
        const int nt = (1 << p.out_bits) - 1;
        for (int i = threadIdx.x; i < nt * NCOLS; i += 256) {
          const int k = i / NCOLS, c = i - k * NCOLS;
          const int gcol = b0 + c;
          table[i] = gcol < p.rowsB ? p.thr[(long long)gcol * nt + k] : 0;
        }
      }
      bool shortcut_vec = res_prefetched;
      if constexpr (F4) {
        if (res_prefetched && p.fold != 0u) {
          // the shortcut term enters one of the partial sums (wave 0's) on the matrix cores
          if (wave == 0) {
            shortcut_publish<RES_REGS>(area + 32, lane, 64, res_regs[0]);
            fold_shortcut<1, FB>(p, acc, area + 32, lane);
          }
          shortcut_vec = false;
        }
      }
      static_for<0, FB>([&](auto yc) {
        constexpr int y = decltype(yc)::value;
        static_for<0, 4>([&](auto qc) {
          constexpr int q = decltype(qc)::value;
          Acc4 v;
          v.x = acc[0][y][4 * q];
          v.y = acc[0][y][4 * q + 1];
          v.z = acc[0][y][4 * q + 2];
          v.w = acc[0][y][4 * q + 3];
          part[((wave * FB + y) * 4 + q) * 64 + lane] = v;
        });
      });
      if (g == 0) {
#pragma unroll
        for (int s = 0; s < (CONV ? 1 : FB); ++s) sums[(wave * FB + s) * 32 + li] = ssum[s];
      }
      if (res_prefetched) shortcut_publish<RES_REGS>(area + 32, lane, 64, res_regs[0]);
      __syncthreads();
      int stot[CONV ? FA : FB];
#pragma unroll
      for (int s = 0; s < (CONV ? 1 : FB); ++s) {
        int t = 0;
#pragma unroll
        for (int w = 0; w < KS; ++w) t += sums[(w * FB + s) * 32 + li];
        stot[s] = t;
      }
      if (CONV && g == 0) area[li] = (uint32_t)((p.sym ? p.wmax : 0) * stot[0]);
      const int rb = a0, cb = b0;
      auto finish_quad = [&](auto qc) {
        constexpr int q = decltype(qc)::value;
        AccT accr[1][FB];
        static_for<0, FB>([&](auto yc) {
          constexpr int y = decltype(yc)::value;
          Acc4 t = part[(y * 4 + q) * 64 + lane];
#pragma unroll
          for (int w = 1; w < KS; ++w) {
            const Acc4 u = part[((w * FB + y) * 4 + q) * 64 + lane];
            t.x += u.x;
            t.y += u.y;
            t.z += u.z;
            t.w += u.w;
          }
          accr[0][y][4 * q] = t.x;
          accr[0][y][4 * q + 1] = t.y;
          accr[0][y][4 * q + 2] = t.z;
          accr[0][y][4 * q + 3] = t.w;
        });
        if constexpr (DIRECT_BITS > 2) {
          if (use_table) {
            direct_epilogue<F4, 1, FB, CONV, true, q, q + 1>(p, accr, stot, area, rb, cb, lane, thrT, flipm,
                                                             shortcut_vec, table);
            return;
          }
        }
        direct_epilogue<F4, 1, FB, CONV, false, q, q + 1>(p, accr, stot, area, rb, cb, lane, thrT, flipm, shortcut_vec);
      };
      static_assert(KS == 4, "one register quad per wave");
      switch (wave) {
        case 0: finish_quad(std::integral_constant<int, 0>{}); break;
        case 1: finish_quad(std::integral_constant<int, 1>{}); break;
        case 2: finish_quad(std::integral_constant<int, 2>{}); break;
        default: finish_quad(std::integral_constant<int, 3>{}); break;
      }
      return;
    }
  }
  if constexpr (KS == 1) {
    if (p.epi == APNN_EPI_INT32) {
      uint32_t *area = smem + wave * SLAB_WORDS;
      if (CONV && p.sym) {
        if (g == 0) {
#pragma unroll
          for (int x = 0; x < FA; ++x) area[x * 32 + li] = (uint32_t)(p.wmax * ssum[CONV ? x : 0]);
        }
      }
      store_int32_direct<F4, FA, FB, CONV>(p, acc, ssum, area, a0 + wa * FA * 32, b0 + wb * FB * 32, lane);
      return;
    }
    if (direct) {
      uint32_t *area = smem + wave * SLAB_WORDS;
      if (CONV && g == 0) {
#pragma unroll
        for (int x = 0; x < FA; ++x) area[x * 32 + li] = (uint32_t)((p.sym ? p.wmax : 0) * ssum[CONV ? x : 0]);
      }
      if (res_prefetched) {
#pragma unroll
        for (int x = 0; x < FA; ++x) shortcut_publish<RES_REGS>(area + FA * 32 + x * 64 * FB, lane, 64, res_regs[x]);
      }
      bool shortcut_vec = res_prefetched;  // shortcut still to be added per value by the vector ALUs
      // (tiles of eight blocks per wave have no registers to spare for the extra operands)
      if constexpr (F4 && FA * FB <= 4) {
        if (res_prefetched && p.fold != 0u) {
          // LDS operations of one wave complete in order: the words published above are visible here
          fold_shortcut<FA, FB>(p, acc, area + FA * 32, lane);
          shortcut_vec = false;
        }
      }
      const int rb = a0 + wa * FA * 32, cb = b0 + wb * FB * 32;
      if (DIRECT_BITS == 2 || p.out_bits <= 2) {
        direct_epilogue<F4, FA, FB, CONV, false>(p, acc, ssum, area, rb, cb, lane, thrT, flipm, shortcut_vec);
      } else if constexpr (DIRECT_BITS > 2) {
        direct_epilogue<F4, FA, FB, CONV, true>(p, acc, ssum, area, rb, cb, lane, thrT, flipm, shortcut_vec);
      }
      return;
    }
  }
  int *slab = reinterpret_cast<int *>(smem) + wave * SLAB_WORDS;
  int *rowsum = slab + 32 * LDT;
  int *colsum = rowsum + 32;
  uint32_t *res_lds = reinterpret_cast<uint32_t *>(colsum + NCOLS);

  if (!CONV && g == 0) {
#pragma unroll
    for (int y = 0; y < FB; ++y) colsum[y * 32 + li] = ssum[CONV ? 0 : y];
  }
  static_for<0, FA>([&](auto xc) {
    constexpr int x = decltype(xc)::value;
    if (CONV && g == 0) rowsum[li] = ssum[CONV ? x : 0];
    if (res_prefetched) shortcut_publish<RES_REGS>(res_lds, lane, 64, res_regs[x]);
    static_for<0, FB>([&](auto yc) {
      constexpr int y = decltype(yc)::value;
      static_for<0, 16>([&](auto rc) {
        constexpr int r = decltype(rc)::value;
        int v;
        if constexpr (F4) {
          v = __float2int_rn(acc[x][y][r] * 4.0f);
        } else {
          v = acc[x][y][r];
        }
        slab[(8 * (r >> 2) + 4 * g + (r & 3)) * LDT + y * 32 + li] = v;
      });
    });
    if constexpr (KS > 1) {
      // all KS partial slabs must be complete before any wave sums them
      __syncthreads();
      const int *base = reinterpret_cast<const int *>(smem);
      wave_epilogue<NCOLS, CONV, KS>(p, base, base + 32 * LDT, base + 32 * LDT + 32, SLAB_WORDS, wave, a0, b0, lane,
                                     q0, q1, res_prefetched ? res_lds : nullptr);
    } else {
      // LDS operations of one wave complete in order: the reads below see the writes above, and the
      // next slab's writes come after these reads
      wave_epilogue<NCOLS, CONV, 1>(p, slab, rowsum, colsum, 0, 0, a0 + (wa * FA + x) * 32, b0 + wb * FB * 32, lane,
                                    q0, q1, res_prefetched ? res_lds : nullptr);
    }
  });
}


// k-words (32 elements each) per staged chunk.  The convolution kernels whose waves tile the output
// (64x64 and 128x64 per work-group with 128-bit loads, i.e. at least 128 stored channels; larger tiles
// and the short reductions of narrow layers measure no gain) stage 16; so do the 256x128 GEMM tiles while
// two work-groups' buffers still fit a compute unit (three planes in all: w1a2, -4 % at 4096^3 / 8192^3;
// with four planes the larger buffers leave one work-group per unit and cost 28 %); the split-K tiles, used
// for few outputs over a long K where every chunk iteration is a latency chain, stage 32: their per-chunk
// work (im2col addressing, LDS staging, barrier) is a large share of a short K loop, and k-steps past the
// end of K are skipped, so a longer chunk wastes nothing.
constexpr int mfma_chunk_words(int PA, int PB, int FA, int FB, int WA, int WB, bool conv, int vw, int ksx = 1) {
  if (ksx > 1) return 16;  // two wave groups share the k-steps of a chunk: four each
  if (WA * WB == 1) return 32;
  if (conv && FA * FB <= 2 && vw == 4) return 16;
  if (!conv && FA * FB >= 8 && (PA * WA * FA + PB * WB * FB) * 32 <= 512) return 16;
  return 8;
}

// longest reduction (32-bit words) the one- and two-block convolution tiles load without staging
constexpr int kDirectMaxKW = 40;

// KSX > 1: KSX groups of four waves each (work-groups of 256 * KSX threads).  Every group tiles the whole
// output tile WA x WB like the four waves of the other kernels and takes every KSX-th k-step of each
// staged chunk; after the K loop the groups exchange partial accumulators through LDS so that each group
// finishes 1 / KSX of the tile's row blocks.  For layers with too few large tiles to give every compute
// unit two work-groups: the second wave per SIMD comes from the same tile instead.
template <int CORE, int PA, int PB, int FA, int FB, int WA, int WB, int VW, bool CONV, int OCC, int KSX = 1>
__global__ __launch_bounds__(256 * KSX, OCC) void apnn_mfma_kernel(const KParams pk) {
  // paired launch: the second half of the grid works on the second problem (see KParams)
  KParams p = pk;
  int bid = blockIdx.x;
  if (CONV && pk.pair_tiles > 0 && bid >= pk.pair_tiles) {
    bid -= pk.pair_tiles;
    p.B = pk.B2;
    p.KW = pk.KW2;
    p.S = pk.S2;
    p.pad = pk.pad2;
    p.magicS = pk.magicS2;
    p.magicS16 = pk.magicS16_2;
    p.planeB = pk.planeB2;
    p.thr = pk.thr2;
    p.flip = pk.flip2;
    p.out = pk.out2;
  }
  // four waves per work-group: WA x WB of them tile the output, the remaining factor KS splits K
  static_assert(WA * WB == 4 || WA * WB == 1, "waves tile the output or all split K");
  constexpr int KS = 4 / (WA * WB);
  static_assert(KS == 1 || FA == 1, "the split-K reduction handles one 32-row slab");
  constexpr bool F4 = CORE == CORE_F4;
  static_assert(KSX == 1 || (KSX == 2 && KS == 1 && F4 && FA % 2 == 0), "wave groups: FP4 core, even row blocks");
  constexpr int WPS = F4 ? 2 : 1;                 // packed words per row consumed by one k-step
  constexpr int DA = F4 ? (PA + 1) / 2 : 1;       // operand digits (FP4: plane pairs)
  constexpr int DB = F4 ? (PB + 1) / 2 : 1;
  using AccT = typename std::conditional<F4, v16f, v16i>::type;
  using FragT = typename std::conditional<F4, v8i, v4i>::type;
  constexpr int NT = 256 * KSX;
  constexpr int TA = WA * FA * 32, TB = WB * FB * 32;
  constexpr int KC = mfma_chunk_words(PA, PB, FA, FB, WA, WB, CONV, VW, KSX);
  constexpr int LD = KC + 1;         // odd row pitch: 32 rows hit 32 different banks
  constexpr int KQ = KC / VW;
  constexpr int UA = TA * KQ, UB = TB * KQ;
  constexpr int NIA = (UA + NT - 1) / NT, NIB = (UB + NT - 1) / NT;
  constexpr int BUF_WORDS = (PA * TA + PB * TB) * LD;

  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];  // [2][BUF_WORDS]

  const int tid = threadIdx.x;
  // the wave index is the same in all 64 lanes: as a scalar it keeps loop control and the address terms that
  // depend on it (k-steps of a split-K wave, wave group) on the scalar unit
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 31, g = lane >> 5;
  const int kq = KSX > 1 ? wave >> 2 : 0;   // wave group
  const int wv = KSX > 1 ? wave & 3 : wave; // wave within its group
  const int wa = KS > 1 ? 0 : wv / WB, wb = KS > 1 ? 0 : wv % WB;

  // Work-group index -> tile.  Consecutive indices land on different XCDs (round-robin over the eight), each
  // with an L2 of its own.  In row-major order the work-groups of one XCD would therefore take every eighth
  // tile of every row band and each L2 would fetch all of one operand.  With xcd_rows set (large grids) the
  // index is regrouped into one contiguous range of tiles per XCD, and a range walks the grid in bands of
  // xcd_rows tile rows, column by column: the work-groups resident on an XCD at one time share a few row
  // blocks and a few column blocks in that XCD's L2.
  const int tilesB = (p.rowsB + TB - 1) / TB;
  int trow = bid / tilesB, tcol = bid % tilesB;
  if (p.xcd_rows > 0) {
    const int tilesA = (p.rowsA + TA - 1) / TA;
    const int per_xcd = (tilesA * tilesB) >> 3;  // the launcher checked that the grid is a multiple of 8
    const int lin = (bid & 7) * per_xcd + (bid >> 3);
    const int per_band = p.xcd_rows * tilesB;
    const int band = lin / per_band, w = lin - band * per_band;
    const int rows_in_band = min(p.xcd_rows, tilesA - band * p.xcd_rows);
    tcol = w / rows_in_band;
    trow = band * p.xcd_rows + (w - tcol * rows_in_band);
  }
  const int a0 = trow * TA;
  const int b0 = tcol * TB;

  // output pixel (row of A) -> image index and the input coordinates of its filter tap (0, 0)
  auto pixel_origin = [&](int pix, int &b, int &y0, int &x0) {
    int oy, ox;
    if (p.geo_fast) {
      // multiply-high by ceil(2^32 / d) is the exact quotient here (the host checked the range)
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

  // how the operands reach the matrix core (see direct_loop below)
  constexpr bool DIRECT_K = F4 && KS > 1 && VW == 4;
  constexpr bool DIRECT_OPT = F4 && CONV && KS == 1 && KSX == 1 && FA == 1 && FB <= 2;
  const bool direct_k = DIRECT_OPT && p.KW <= kDirectMaxKW;

  // Operands from global memory straight into the registers the matrix core reads -- no LDS staging, no
  // barrier.  K is cut into groups of 2*VW words; the lower lane half takes the first VW words of a
  // group and the upper half the last VW, for both operands alike, which only permutes the terms of
  // every dot product.  A wave requests GD groups at once (one memory latency per batch) and then runs
  // VW k-steps per group.  Used by
  //   - the split-K tiles with 128-bit loads (always): no wave shares an operand with another there;
  //   - the convolution tiles of one or two blocks per wave when the reduction is short (direct_k,
  //     decided per launch): the waves of a work-group then load the rows they share once each, through
  //     the L1 cache, which costs less than the staging pipeline's bookkeeping for a handful of k-steps.
  // The first batch is requested here, before thresholds, shortcut words and accumulators are set up,
  // so that the rest of the prologue runs under its memory latency.
  // One buffer descriptor per operand plane (base, size in bytes).  A buffer load whose offset lies past
  // the descriptor's size returns zeros, so a disabled load (row or k past the end, padding pixel) is the
  // same instruction with the offset 0xffffffff: no branch around the load, which also lets the compiler
  // count outstanding loads exactly (a register set waits for its own loads only).
  __amdgpu_buffer_rsrc_t rsrcA[PA], rsrcB[PB];
#pragma unroll
  for (int pl = 0; pl < PA; ++pl)
    rsrcA[pl] = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t *>(p.A + pl * p.planeA), 0,
                                                  (int)(uint32_t)(p.planeA * 4), 0x00020000);
#pragma unroll
  for (int pl = 0; pl < PB; ++pl)
    rsrcB[pl] = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t *>(p.B + pl * p.planeB), 0,
                                                  (int)(uint32_t)(p.planeB * 4), 0x00020000);
  auto load_buf = [](__amdgpu_buffer_rsrc_t rsrc, uint32_t woff, bool ok, uint32_t (&dst)[VW]) {
    const int boff = ok ? (int)(woff << 2) : -1;
    if constexpr (VW == 4) {
      const auto v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, boff, 0, 0);
      dst[0] = v[0], dst[1] = v[1], dst[2] = v[2], dst[3] = v[3];
    } else if constexpr (VW == 2) {
      const auto v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, boff, 0, 0);
      dst[0] = v[0], dst[1] = v[1];
    } else {
      dst[0] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, boff, 0, 0);
    }
  };

  constexpr int GW = 2 * VW;
  constexpr int GD_BUDGET = KS > 1 ? (FB == 1 ? 60 : 48) : (FB == 1 ? 40 : 32);  // registers of operands in flight
  constexpr int GD_FIT = GD_BUDGET / (VW * (PA + FB * PB));
  constexpr int GD = GD_FIT < 1 ? 1 : (GD_FIT > 8 ? 8 : GD_FIT);
  constexpr int GSTEP = KS > 1 ? KS : 1;
  const int gfirst = KS > 1 ? wave : 0;
  const int ngroups = (p.KW + GW - 1) / GW;
  uint32_t ga[GD][PA][VW], gbw[GD][FB][PB][VW];
  bool okA = false;
  int ay0 = 0, ax0 = 0;
  uint32_t baseA = 0;  // word offset of this lane's row (convolution: of its pixel's tap (0, 0), mod 2^32)
  uint32_t baseB[FB];
  bool okB[FB];
  // Rows are addressed as in the staged path (32-bit word offsets, buffer loads that return zeros when
  // disabled): the batch is straight-line code, so the wave starts on the first group while the loads of
  // the later ones are still in flight.
  auto direct_issue = [&](int gb) {
#pragma unroll
    for (int d = 0; d < GD; ++d) {
      const int kw0 = (gb + d * GSTEP) * GW + VW * g;
      const bool in_k = kw0 < p.KW;
      bool ok = okA && in_k;
      uint32_t woff;
      if (CONV) {
        const uint32_t tap = p.c32_shift >= 0 ? (uint32_t)kw0 >> p.c32_shift
                                               : fast_div((uint32_t)kw0, (uint32_t)p.C32, p.magicC32);
        const uint32_t cw = (uint32_t)kw0 - __umul24(tap, (uint32_t)p.C32);
        const uint32_t r = __umul24(tap, p.magicS16) >> 16;
        const uint32_t sx = tap - __umul24(r, (uint32_t)p.S);
        const int iy = ay0 + (int)r, ix = ax0 + (int)sx;
        ok = ok && (uint32_t)iy < (uint32_t)p.Hs && (uint32_t)ix < (uint32_t)p.Ws;
        woff = baseA + __umul24(__umul24(r, (uint32_t)p.Ws) + sx, (uint32_t)p.C32) + cw;
      } else {
        woff = baseA + (uint32_t)kw0;
      }
#pragma unroll
      for (int pl = 0; pl < PA; ++pl) load_buf(rsrcA[pl], woff, ok, ga[d][pl]);
#pragma unroll
      for (int y = 0; y < FB; ++y)
#pragma unroll
        for (int pl = 0; pl < PB; ++pl) load_buf(rsrcB[pl], baseB[y] + (uint32_t)kw0, okB[y] && in_k, gbw[d][y][pl]);
    }
  };
  if (DIRECT_K || direct_k) {
    const int growA = a0 + wa * FA * 32 + li;
    okA = growA < p.rowsA;
    int ab = 0;
    if (CONV) pixel_origin(growA, ab, ay0, ax0);
    baseA = CONV ? (((uint32_t)ab * (uint32_t)p.Hs + (uint32_t)ay0) * (uint32_t)p.Ws + (uint32_t)ax0) * (uint32_t)p.C32
                 : (uint32_t)growA * (uint32_t)p.KW;
#pragma unroll
    for (int y = 0; y < FB; ++y) {
      const int grow = b0 + (wb * FB + y) * 32 + li;
      okB[y] = grow < p.rowsB;
      baseB[y] = (uint32_t)grow * (uint32_t)p.KW;
    }
    direct_issue(gfirst);
  }

  // ---- staging bookkeeping (same scheme as the VALU kernel) ----------------------------------
  // The host launches this kernel only when every operand plane spans less than 2^32 bytes and the
  // filter is small (KParams::addr32), so a row's chunk is addressed by a 32-bit word offset: the row's
  // own offset, computed once, plus for a convolution a few full-rate operations per chunk -- tap =
  // k / C32 (a shift when C32 is a power of two), (r, s) by multiply-shift, 24-bit multiplies -- instead of
  // multiply-high decodes and 64-bit multiply-adds (quarter-rate operations) per chunk and row.
  int a_row[NIA], a_kq[NIA];
  int a_y0[NIA], a_x0[NIA];
  uint32_t a_base[NIA], b_base[NIB];  // word offset of the row (convolution: of the pixel's tap (0, 0), mod 2^32)
  bool a_ok[NIA];
  int b_row[NIB], b_kq[NIB];
  bool b_ok[NIB];
  if (!DIRECT_K && !direct_k) {
#pragma unroll
  for (int it = 0; it < NIA; ++it) {
    const int u = tid + it * NT;
    a_kq[it] = u % KQ;
    a_row[it] = u / KQ;
    const int grow = a0 + a_row[it];
    a_ok[it] = (u < UA) && (grow < p.rowsA);
    int ab = 0;
    a_y0[it] = a_x0[it] = 0;
    if (CONV) pixel_origin(grow, ab, a_y0[it], a_x0[it]);
    a_base[it] = CONV ? (((uint32_t)ab * (uint32_t)p.Hs + (uint32_t)a_y0[it]) * (uint32_t)p.Ws + (uint32_t)a_x0[it]) *
                            (uint32_t)p.C32
                      : (uint32_t)grow * (uint32_t)p.KW;
  }
#pragma unroll
  for (int it = 0; it < NIB; ++it) {
    const int u = tid + it * NT;
    b_kq[it] = u % KQ;
    b_row[it] = u / KQ;
    b_ok[it] = (u < UB) && (b0 + b_row[it] < p.rowsB);
    b_base[it] = (uint32_t)(b0 + b_row[it]) * (uint32_t)p.KW;
  }
  }

  // Chunks in flight between global memory and LDS: the tiles of at most four blocks per wave keep two
  // register sets, so a chunk's loads are issued two chunk iterations before they are staged (one iteration
  // does not cover the memory latency when a wave runs only a few k-steps per chunk); the larger tiles have
  // no registers to spare for a second set.
  constexpr int PF = (FA * FB <= 4 && VW == 4) ? 2 : 1;
  uint32_t ra_[PF][NIA][PA][VW], rb_[PF][NIB][PB][VW];

  auto fetch = [&](int k0, auto set_c) {
    constexpr int set = decltype(set_c)::value;
#pragma unroll
    for (int it = 0; it < NIA; ++it) {
      const int kw0 = k0 + a_kq[it] * VW;
      bool ok = a_ok[it] && kw0 < p.KW;
      uint32_t woff;
      if (CONV) {
        const uint32_t tap = p.c32_shift >= 0 ? (uint32_t)kw0 >> p.c32_shift
                                               : fast_div((uint32_t)kw0, (uint32_t)p.C32, p.magicC32);
        const uint32_t cw = (uint32_t)kw0 - __umul24(tap, (uint32_t)p.C32);
        const uint32_t r = __umul24(tap, p.magicS16) >> 16;
        const uint32_t sx = tap - __umul24(r, (uint32_t)p.S);
        const int iy = a_y0[it] + (int)r, ix = a_x0[it] + (int)sx;
        ok = ok && (uint32_t)iy < (uint32_t)p.Hs && (uint32_t)ix < (uint32_t)p.Ws;
        woff = a_base[it] + __umul24(__umul24(r, (uint32_t)p.Ws) + sx, (uint32_t)p.C32) + cw;
      } else {
        woff = a_base[it] + (uint32_t)kw0;
      }
#pragma unroll
      for (int pl = 0; pl < PA; ++pl) load_buf(rsrcA[pl], woff, ok, ra_[set][it][pl]);
    }
#pragma unroll
    for (int it = 0; it < NIB; ++it) {
      const int kw0 = k0 + b_kq[it] * VW;
      const bool ok = b_ok[it] && kw0 < p.KW;
      const uint32_t woff = b_base[it] + (uint32_t)kw0;
#pragma unroll
      for (int pl = 0; pl < PB; ++pl) load_buf(rsrcB[pl], woff, ok, rb_[set][it][pl]);
    }
  };

  auto stage = [&](uint32_t *buf, auto set_c) {
    constexpr int set = decltype(set_c)::value;
    uint32_t *As = buf;                   // [PA][TA][LD]
    uint32_t *Bs = buf + PA * TA * LD;    // [PB][TB][LD]
#pragma unroll
    for (int it = 0; it < NIA; ++it) {
      if (UA % NT == 0 || tid + it * NT < UA) {
#pragma unroll
        for (int pl = 0; pl < PA; ++pl)
#pragma unroll
          for (int i = 0; i < VW; ++i) As[(pl * TA + a_row[it]) * LD + a_kq[it] * VW + i] = ra_[set][it][pl][i];
      }
    }
#pragma unroll
    for (int it = 0; it < NIB; ++it) {
      if (UB % NT == 0 || tid + it * NT < UB) {
#pragma unroll
        for (int pl = 0; pl < PB; ++pl)
#pragma unroll
          for (int i = 0; i < VW; ++i) Bs[(pl * TB + b_row[it]) * LD + b_kq[it] * VW + i] = rb_[set][it][pl][i];
      }
    }
  };

  AccT acc[FA][FB];
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

  // quantizer and shortcut words of this wave's tile: requested now, consumed after the K loop
  constexpr int HA = FA / KSX;  // row blocks of the wave tile this wave finishes
  const int own_rbase = a0 + (wa * FA + kq * HA) * 32;
  EpiOperands<HA, FB> eo;
  constexpr bool EPI_LAZY = HA * FB >= 8;
  epi_prefetch<KS, (CONV ? PA : PB) >= 3 ? 4 : 2, EPI_LAZY>(p, own_rbase, b0 + wb * FB * 32, lane, eo);

  // packed words of this lane's rows for one k-step
  uint32_t wA[FA][PA], wB[FB][PB];
  auto read_words = [&](const uint32_t *buf, int ks) {
    // CORE_F4: the two lane halves take the two words of the 64-element k-step
    const int kw = ks * WPS + (F4 ? g : 0);
    const uint32_t *As = buf + (wa * FA * 32 + li) * LD + kw;
    const uint32_t *Bs = buf + PA * TA * LD + (wb * FB * 32 + li) * LD + kw;
#pragma unroll
    for (int x = 0; x < FA; ++x)
#pragma unroll
      for (int pl = 0; pl < PA; ++pl) wA[x][pl] = As[(pl * TA + x * 32) * LD];
#pragma unroll
    for (int y = 0; y < FB; ++y)
#pragma unroll
      for (int pl = 0; pl < PB; ++pl) wB[y][pl] = Bs[(pl * TB + y * 32) * LD];
  };
  FragT af[FA][DA], bf[FB][DB];
  auto expand_all = [&](FragT (&a)[FA][DA], FragT (&b)[FB][DB]) {
#pragma unroll
    for (int x = 0; x < FA; ++x) {
      if (CONV) {
#pragma unroll
        for (int pl = 0; pl < PA; ++pl) psum[x][pl] += __popc(wA[x][pl]);
      }
      if constexpr (F4) {
        static_for<0, DA>([&](auto dc) { a[x][decltype(dc)::value] = expand_fp4<PA, decltype(dc)::value>(wA[x]); });
      } else {
        a[x][0] = expand_planes<PA>(wA[x], rotA);
      }
    }
#pragma unroll
    for (int y = 0; y < FB; ++y) {
      if (!CONV) {
#pragma unroll
        for (int pl = 0; pl < PB; ++pl) psum[y][pl] += __popc(wB[y][pl]);
      }
      if constexpr (F4) {
        static_for<0, DB>([&](auto dc) { b[y][decltype(dc)::value] = expand_fp4<PB, decltype(dc)::value>(wB[y]); });
      } else {
        b[y][0] = expand_planes<PB>(wB[y], rotB);
      }
    }
  };
  auto mfma_all = [&]() {
#pragma unroll
    for (int x = 0; x < FA; ++x)
#pragma unroll
      for (int y = 0; y < FB; ++y) {
        if constexpr (F4) {
          static_for<0, DA>([&](auto dac) {
            static_for<0, DB>([&](auto dbc) {
              constexpr int da = decltype(dac)::value, db = decltype(dbc)::value;
              if constexpr (da + db == 0) {
                acc[x][y] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[x][da], bf[y][db], acc[x][y], 4, 4,
                                                                            0, 0, 0, 0);
              } else {
                // E8M0 block scales: 127 = 2^0 on A, 127 + 2*(da+db) = 4^(da+db) on B
                acc[x][y] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                    af[x][da], bf[y][db], acc[x][y], 4, 4, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F + 0x02020202 * (da + db));
              }
            });
          });
        } else {
          acc[x][y] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[x][0], bf[y][0], acc[x][y], 0, 0, 0);
        }
      }
  };

  // Software pipeline: while the matrix cores work on k-step s, the VALU expands the operands of
  // k-step s+1 (also across the chunk boundary: the barrier that publishes chunk ch+1 sits before
  // the last k-step of chunk ch).  Global loads run two chunks ahead, LDS holds two chunks.
  constexpr int NKS = KC / WPS;  // k-steps per chunk
  constexpr int N_MFMA = FA * FB * DA * DB;
  // expansion cost per row word: FP4 10 operations per plane pair + 7 for an odd plane, int8 8 per plane
  constexpr int XA = F4 ? 10 * (PA / 2) + 7 * (PA % 2) : 8 * PA, XB = F4 ? 10 * (PB / 2) + 7 * (PB % 2) : 8 * PB;
  constexpr int N_VALU = FA * XA + FB * XB + FS * PS;
  constexpr int VALU_PER_MFMA = (N_VALU + N_MFMA - 1) / N_MFMA;

  auto direct_loop = [&]() {
    for (int gb = gfirst; gb < ngroups; gb += GSTEP * GD) {
      if (gb != gfirst) direct_issue(gb);  // the first batch is in flight since the prologue
#pragma unroll
      for (int d = 0; d < GD; ++d) {
        if (gb + d * GSTEP < ngroups) {  // same for the whole wave
#pragma unroll
          for (int i = 0; i < VW; ++i) {
#pragma unroll
            for (int pl = 0; pl < PA; ++pl) wA[0][pl] = ga[d][pl][i];
#pragma unroll
            for (int y = 0; y < FB; ++y)
#pragma unroll
              for (int pl = 0; pl < PB; ++pl) wB[y][pl] = gbw[d][y][pl][i];
            expand_all(af, bf);
            mfma_all();
          }
        }
      }
    }
  };
  if constexpr (DIRECT_K) {
    direct_loop();
  } else if (direct_k) {
    if constexpr (DIRECT_OPT) direct_loop();
  } else {
  const int nchunks = (p.KW + KC - 1) / KC;
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, PF - 1>;
  // chunk c >= 1 travels in register set (c - 1) % PF
  // (a fetch past the end of K is issued all the same, with every load disabled: the number of loads in
  // flight is then the same on every path, and the compiler's wait counts stay exact)
  fetch(0, Set0{});
  stage(smem, Set0{});
  if (PF == 2 || nchunks > 1) fetch(KC, Set0{});
  if (PF == 2) fetch(2 * KC, Set1{});
  __syncthreads();
  if constexpr (KS == 1) {
    read_words(smem, kq);
    expand_all(af, bf);
  }
  // one chunk; par = ch % 2 is a compile-time constant (LDS buffer and register set of the iteration)
  auto chunk_body = [&](int ch, auto par_c) {
    const int par = par_c;
    const uint32_t *cur = smem + par * BUF_WORDS;
    uint32_t *nxt = smem + (par ^ 1) * BUF_WORDS;
    const bool more = ch + 1 < nchunks;
    // chunk ch + 1 leaves its registers (every wave left this LDS buffer before the barrier of the
    // previous chunk), chunk ch + 1 + PF is requested into them
    if constexpr (PF == 2) {
      using Set = std::integral_constant<int, decltype(par_c)::value>;
      if (more) stage(nxt, Set{});
      fetch((ch + 3) * KC, Set{});
    } else if (more) {
      stage(nxt, Set0{});
      if (ch + 2 < nchunks) fetch((ch + 2) * KC, Set0{});
    }
    if constexpr (KS > 1) {
      // split-K: wave w owns k-steps w, w + KS, ... of every chunk
#pragma unroll
      for (int ks = 0; ks < NKS / KS; ++ks) {
        read_words(cur, wave + ks * KS);
        expand_all(af, bf);
        mfma_all();
      }
      __syncthreads();
      return;
    }
    auto advance = [&]() {
      FragT an[FA][DA], bn[FB][DB];
      expand_all(an, bn);
#pragma unroll
      for (int x = 0; x < FA; ++x)
#pragma unroll
        for (int d = 0; d < DA; ++d) af[x][d] = an[x][d];
#pragma unroll
      for (int y = 0; y < FB; ++y)
#pragma unroll
        for (int d = 0; d < DB; ++d) bf[y][d] = bn[y][d];
#pragma unroll
      for (int i = 0; i < N_MFMA; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);              // one MFMA
        __builtin_amdgcn_sched_group_barrier(0x002, VALU_PER_MFMA, 0);  // then its share of VALU work
      }
    };
    if constexpr (KSX > 1) {
      // wave group kq owns k-steps kq, kq + KSX, ... of every chunk (steps past the end of K read the
      // zeros the staging wrote there)
#pragma unroll 1
      for (int ks = kq; ks + KSX < NKS; ks += KSX) {
        read_words(cur, ks + KSX);
        mfma_all();
        advance();
      }
      __syncthreads();
      if (more) read_words(nxt, kq);
      mfma_all();
      if (more) advance();
      return;
    }
    // k-steps of this chunk that hold data (the last chunk may be short)
    const int nks = min(NKS, (p.KW - ch * KC + WPS - 1) / WPS);
    // k-steps 0 .. nks-2 (kept as a real loop: one scheduling region per k-step)
#pragma unroll 1
    for (int ks = 0; ks + 1 < nks; ++ks) {
      read_words(cur, ks + 1);
      mfma_all();
      advance();
    }
    // last k-step of the chunk: publish the next chunk first, then prefetch its first operands
    __syncthreads();
    if (more) read_words(nxt, 0);
    mfma_all();
    if (more) advance();
  };
  if constexpr (PF == 2) {
    // two chunks per trip: register set and LDS buffer of each half are compile-time constants (the only
    // way back to the top is through both halves, so that the order of the loads in flight is the same on
    // every path into the loop)
#pragma unroll 1
    for (int ch = 0;; ch += 2) {
      chunk_body(ch, std::integral_constant<int, 0>{});
      if (ch + 1 >= nchunks) break;
      chunk_body(ch + 1, std::integral_constant<int, 1>{});
      if (ch + 2 >= nchunks) break;
    }
  } else {
    for (int ch = 0; ch < nchunks; ++ch) chunk_body(ch, ch & 1);
  }
  }
  int ssum[FS];
#pragma unroll
  for (int x = 0; x < FS; ++x) {
    int t = 0;
#pragma unroll
    for (int pl = 0; pl < PS; ++pl) t += psum[x][pl] << pl;
    if (F4) t += __shfl_xor(t, 32, 64);  // the lane halves counted different words of the row
    ssum[x] = t;
  }

  if constexpr (KSX == 1) {
    epi_finish<F4, KS, CONV, (CONV ? PA : PB) >= 3 ? 4 : 2, EPI_LAZY>(p, acc, ssum, smem, wave, lane, a0, b0, wa, wb, eo);
  } else {
    // The two wave groups hold partial sums over their k-steps for the same outputs.  Group 0 finishes the
    // first HA row blocks of every wave tile, group 1 the last HA: each wave parks the blocks it gives away
    // in LDS in the accumulator's own register layout (16 bytes per lane and register quad), its partner
    // (same position in the other group) adds them to its own.  Activation sums travel the same way.
    static_assert(KSX == 2, "two wave groups");
    __syncthreads();  // every wave is done with the staging buffers
    float4 *xch = reinterpret_cast<float4 *>(smem);                  // [8 waves][HA][FB][4 quads][64 lanes]
    int *xsum = reinterpret_cast<int *>(smem) + 8 * HA * FB * 4 * 64 * 4;  // [8 waves][FS][64 lanes]
    auto give = [&](auto first_c) {
      constexpr int first = decltype(first_c)::value;
      static_for<0, HA>([&](auto xc) {
        constexpr int x = decltype(xc)::value;
        static_for<0, FB>([&](auto yc) {
          constexpr int y = decltype(yc)::value;
          static_for<0, 4>([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            float4 v;
            v.x = acc[first + x][y][4 * q];
            v.y = acc[first + x][y][4 * q + 1];
            v.z = acc[first + x][y][4 * q + 2];
            v.w = acc[first + x][y][4 * q + 3];
            xch[(((wave * HA + x) * FB + y) * 4 + q) * 64 + lane] = v;
          });
        });
      });
    };
    if (kq == 0) give(std::integral_constant<int, HA>{}); else give(std::integral_constant<int, 0>{});
#pragma unroll
    for (int x = 0; x < FS; ++x) xsum[(wave * FS + x) * 64 + lane] = ssum[x];
    __syncthreads();
    const int partner = wave ^ 4;
    AccT own[HA][FB];
    auto take = [&](auto first_c) {
      constexpr int first = decltype(first_c)::value;
      static_for<0, HA>([&](auto xc) {
        constexpr int x = decltype(xc)::value;
        static_for<0, FB>([&](auto yc) {
          constexpr int y = decltype(yc)::value;
          static_for<0, 4>([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            const float4 v = xch[(((partner * HA + x) * FB + y) * 4 + q) * 64 + lane];
            own[x][y][4 * q] = acc[first + x][y][4 * q] + v.x;
            own[x][y][4 * q + 1] = acc[first + x][y][4 * q + 1] + v.y;
            own[x][y][4 * q + 2] = acc[first + x][y][4 * q + 2] + v.z;
            own[x][y][4 * q + 3] = acc[first + x][y][4 * q + 3] + v.w;
          });
        });
      });
    };
    if (kq == 0) take(std::integral_constant<int, 0>{}); else take(std::integral_constant<int, HA>{});
    int own_sum[CONV ? HA : FB];
#pragma unroll
    for (int x = 0; x < (CONV ? HA : FB); ++x) {
      // convolution: sums of this group's row blocks; GEMM entry points: column sums, the same blocks in both groups
      const int idx = CONV ? kq * HA + x : x;
      own_sum[x] = xsum[(wave * FS + idx) * 64 + lane] + xsum[(partner * FS + idx) * 64 + lane];
    }
    // epi_finish opens with a barrier: nobody overwrites the exchange area before every wave has read it
    epi_finish<F4, 1, CONV, (CONV ? PA : PB) >= 3 ? 4 : 2, EPI_LAZY>(p, own, own_sum, smem, wave, lane, own_rbase, b0, 0,
                                                                       wb, eo);
  }
}

constexpr size_t mfma_smem_bytes(int core, int PA, int PB, int FA, int FB, int WA, int WB, bool conv, int vw,
                                 int ksx = 1) {
  const size_t ld = mfma_chunk_words(PA, PB, FA, FB, WA, WB, conv, vw, ksx) + 1;
  // FP4 split-K tiles with 128-bit loads stage nothing (operands go from global memory to registers)
  const size_t stage = core == CORE_F4 && WA * WB == 1 && vw == 4
                           ? 0
                           : 2ull * ((size_t)PA * WA * FA * 32 + (size_t)PB * WB * FB * 32) * ld * sizeof(uint32_t);
  // split-K tiles whose activations have three or more planes quantize codes of up to four bits from
  // registers and keep one threshold table [15][FB * 32] behind the output stage's area
  const size_t table = (WA * WB == 1 && (conv ? PA : PB) >= 3) ? 15ull * FB * 32 * sizeof(int) : 0;
  const size_t slab = 4ull * ksx * (32 * (FB * 32 + 1) + 32 + FB * 32 + 2 * 32 * FB) * sizeof(int) + table;
  // wave groups: exchange area of the partial accumulators and activation sums (see the kernel's tail)
  const size_t fs = conv ? FA : FB;
  const size_t xch = ksx > 1 ? 4ull * ksx * ((size_t)(FA / ksx) * FB * 16 + fs) * 64 * sizeof(int) : 0;
  const size_t m = stage > slab ? stage : slab;
  return m > xch ? m : xch;
}

// OCC_WANTED work-groups per compute unit, or as many as the LDS budget (160 KiB) allows
constexpr long long kXcdOrderMinTiles = 256;

template <int CORE, int PA, int PB, int FA, int FB, int WA, int WB, int VW, bool CONV, int OCC_WANTED, int KSX = 1>
inline hipError_t launch_mfma(const KParams &p, hipStream_t stream) {
  constexpr int TA = WA * FA * 32, TB = WB * FB * 32;
  constexpr size_t smem_bytes = mfma_smem_bytes(CORE, PA, PB, FA, FB, WA, WB, CONV, VW, KSX);
  constexpr int OCC_FIT = (int)((160 * 1024) / smem_bytes);
  constexpr int OCC = OCC_FIT < 1 ? 1 : (OCC_FIT < OCC_WANTED ? OCC_FIT : OCC_WANTED);
  static_assert(smem_bytes * OCC <= 160 * 1024, "LDS budget of a gfx950 compute unit");
  auto kern = apnn_mfma_kernel<CORE, PA, PB, FA, FB, WA, WB, VW, CONV, OCC, KSX>;
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
  KParams q = p;
  if (p.pair_tiles != 0) q.pair_tiles = (int)tiles;  // the host only flags a pair; the tile count is known here
  // XCD-aware tile order for grids of at least one work-group per compute unit (smaller grids are over
  // before the L2s matter, and the regrouping costs every work-group two scalar divisions)
  const long long tilesB = (p.rowsB + TB - 1) / TB;
  q.xcd_rows = (p.pair_tiles == 0 && tiles % 8 == 0 && tiles >= kXcdOrderMinTiles && tilesB >= 2) ? 8 : 0;
  hipLaunchKernelGGL(kern, dim3((unsigned)(q.pair_tiles != 0 ? 2 * tiles : tiles)), dim3(256 * KSX), smem_bytes, stream,
                     q);
  return hipGetLastError();
}

template <int CORE, int PA, int PB, int FA, int FB, int WA, int WB, int VW, bool CONV, int OCC, int TILE, int KSX = 1>
inline hipError_t launch_mfma_if_enabled(const KParams &p, hipStream_t stream) {
  if constexpr (mfma_tile_enabled(CORE, CONV, VW, TILE, PA, PB)) {
    return launch_mfma<CORE, PA, PB, FA, FB, WA, WB, VW, CONV, OCC, KSX>(p, stream);
  } else {
    return hipErrorNotSupported;
  }
}

template <int CORE, int PA, int PB, int VW, bool CONV>
inline hipError_t launch_mfma_tile(int tile, const KParams &p, hipStream_t stream) {
  switch (tile) {
    case MT_256x256: return launch_mfma_if_enabled<CORE, PA, PB, 4, 4, 2, 2, VW, CONV, 1, MT_256x256>(p, stream);
    case MT_128x128: return launch_mfma_if_enabled<CORE, PA, PB, 2, 2, 2, 2, VW, CONV, 2, MT_128x128>(p, stream);
    case MT_64x64: return launch_mfma_if_enabled<CORE, PA, PB, 1, 1, 2, 2, VW, CONV, 4, MT_64x64>(p, stream);
    case MT_128x64: return launch_mfma_if_enabled<CORE, PA, PB, 1, 2, 4, 1, VW, CONV, 4, MT_128x64>(p, stream);
    case MT_32x32_K4: return launch_mfma_if_enabled<CORE, PA, PB, 1, 1, 1, 1, VW, CONV, 4, MT_32x32_K4>(p, stream);
    case MT_32x64_K4: return launch_mfma_if_enabled<CORE, PA, PB, 1, 2, 1, 1, VW, CONV, 4, MT_32x64_K4>(p, stream);
    case MT_32x128_K4: return launch_mfma_if_enabled<CORE, PA, PB, 1, 4, 1, 1, VW, CONV, 2, MT_32x128_K4>(p, stream);
    case MT_256x128: return launch_mfma_if_enabled<CORE, PA, PB, 4, 2, 2, 2, VW, CONV, 2, MT_256x128>(p, stream);
    case MT_128x256: return launch_mfma_if_enabled<CORE, PA, PB, 2, 4, 2, 2, VW, CONV, 2, MT_128x256>(p, stream);
    case MT_128x128_G2: return launch_mfma_if_enabled<CORE, PA, PB, 2, 2, 2, 2, VW, CONV, 1, MT_128x128_G2, 2>(p, stream);
    default: return hipErrorNotSupported;
  }
}

}  // namespace apnn
