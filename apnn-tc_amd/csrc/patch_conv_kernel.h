// Patch-resident convolution on the matrix cores (FP4 operands, see mfma_kernel.h for the encoding).
//
// The implicit-GEMM kernel in mfma_kernel.h gathers, for every filter tap, the packed activation
// words of every output pixel of its tile and expands them to matrix-core operands in registers --
// R*S times per input pixel and once more per column tile.  Here the input pixels a tile needs are
// expanded ONCE into LDS and every tap reads them in place:
//
//   * In the zero-padded frame (stored frame plus `pad` pixels on every side, PHs x PWs per image) the
//     input pixel of output pixel (b, oy, ox) and tap (r, s) has the linear index
//         q = (b*PHs + oy*stride)*PWs + ox*stride  +  r*PWs + s,
//     i.e. a per-pixel base plus a per-tap constant.  A tile of consecutive output pixels therefore
//     needs one contiguous range [q_lo, q_hi] of padded-frame pixels: the patch.
//   * Per chunk of 64 channels the work-group stages the patch (bit-plane words -> FP4 digit
//     operands, 16 bytes per pixel, 32-channel word and digit; padding pixels are zeros) and the
//     filter block of its output channels for all taps (same encoding), then runs
//     taps k-steps of pure LDS reads + MFMA:  A operand = patch[base(row) + tap offset], B operand =
//     filter[tap][column].
//   * Per-pixel activation sums (for the symmetric-weight correction) are taken once per patch pixel
//     while staging; a row's window sum is the sum over taps of those.
//
// Output stage, tile-to-row mapping, epilogue operands and all quantizing modes are the ones of the
// implicit-GEMM kernel (epi_prefetch / epi_finish).
#pragma once
#include "mfma_kernel.h"

namespace apnn {

constexpr int PATCH_NPT = 4;  // patch pixels per thread (patch capacity = 4 * 256 pixels)

template <int PA, int PB, int FA, int FB, int WA, int WB, int OCC>
__global__ __launch_bounds__(256, OCC) void apnn_patch_conv_kernel(const KParams p) {
  static_assert(WA * WB == 4, "four waves tile the output");
  constexpr int DA = (PA + 1) / 2, DB = (PB + 1) / 2;
  constexpr int NT = 256;
  constexpr int TA = WA * FA * 32, TB = WB * FB * 32;
  constexpr int DIRECT_BITS = PA >= 3 ? 4 : 2;

  extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 31, g = lane >> 5;
  const int wa = wave / WB, wb = wave % WB;
  const int tilesB = (p.rowsB + TB - 1) / TB;
  const int a0 = (blockIdx.x / tilesB) * TA;
  const int b0 = (blockIdx.x % tilesB) * TB;
  const int taps = p.KW / p.C32;
  const int cap = p.patch_cap;

  uint32_t *patchA = smem;                                 // [DA][cap][2 words][4 dwords]
  uint32_t *filtB = patchA + DA * cap * 8;                 // [DB][taps][TB][2 words][4 dwords]
  int *pixsum = reinterpret_cast<int *>(filtB + DB * taps * TB * 8);  // [cap]

  // ---- tile geometry.  Only the tile's first row is decoded with full divisions (uniform); every
  // other row and patch pixel is a small offset from it, for which the multiply-high quotients are
  // exact. -----------------------------------------------------------------------------------------
  const int last_row = min(a0 + TA, p.rowsA) - 1;
  const int R = taps / p.S;
  const bool pooled = p.pool_order != 0;
  const int gw = pooled ? p.Wo >> 1 : p.Wo, gh = pooled ? p.Ho >> 1 : p.Ho;  // row grid (windows when pooling)
  const int gst = pooled ? 2 * p.stride : p.stride;                          // its step in the padded frame
  const uint32_t u0 = (uint32_t)(pooled ? a0 >> 2 : a0);
  const uint32_t t0 = u0 / (uint32_t)gw;
  const int gx0 = (int)(u0 - t0 * (uint32_t)gw);
  const int b0i = (int)(t0 / (uint32_t)gh);
  const int gy0 = (int)(t0 - (uint32_t)b0i * (uint32_t)gh);
  // padded-frame base index of tile row k (k >= 0, relative to a0), relative to the frame origin of image b0i
  auto row_base = [&](int k) {
    const int u = pooled ? k >> 2 : k, sub = pooled ? k & 3 : 0;
    int gx = gx0 + u;
    const int cy = (int)fast_div((uint32_t)gx, (uint32_t)gw, p.magicGW);
    gx -= cy * gw;
    int gy = gy0 + cy;
    const int cb = (int)fast_div((uint32_t)gy, (uint32_t)gh, p.magicGH);
    gy -= cb * gh;
    return (cb * p.PHs + gy * gst + (sub >> 1) * p.stride) * p.PWs + gx * gst + (sub & 1) * p.stride;
  };
  const int q_lo = row_base(0);  // == (gy0*gst)*PWs + gx0*gst
  const int q_hi = row_base(last_row - a0) + (R - 1) * p.PWs + (p.S - 1);
  const int npp = q_hi - q_lo + 1;
  if (npp > cap) {
    // The host sizes the patch for the worst tile, so this is never taken; if it ever were, the tile
    // stays unwritten and the device error word says so instead of the launch looking successful.
    if (tid == 0 && p.err != nullptr) atomicOr(p.err, (int)KERR_PATCH_CAPACITY);
    return;
  }

  // this lane's rows: patch-relative pixel index of row li of each of its FA row blocks
  int prow[FA];
#pragma unroll
  for (int x = 0; x < FA; ++x) prow[x] = row_base(min((wa * FA + x) * 32 + li, last_row - a0)) - q_lo;

  // Global loads go through one buffer descriptor per operand plane (base, size in bytes; the host launches
  // this kernel only for planes below 4 GiB): a load whose offset lies past the descriptor's size returns
  // zeros, so padding pixels, rows past the end and the unused tail of a task batch are the same instruction
  // with the offset 0xffffffff instead of a branch around the load.
  constexpr uint32_t kOff = 0xffffffffu;
  __amdgpu_buffer_rsrc_t rsrcA[PA], rsrcB[PB];
#pragma unroll
  for (int pl = 0; pl < PA; ++pl)
    rsrcA[pl] = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t *>(p.A + pl * p.planeA), 0,
                                                  (int)(uint32_t)(p.planeA * 4), 0x00020000);
#pragma unroll
  for (int pl = 0; pl < PB; ++pl)
    rsrcB[pl] = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t *>(p.B + pl * p.planeB), 0,
                                                  (int)(uint32_t)(p.planeB * 4), 0x00020000);
  // word pair at byte offset boff (kOff: zeros); without 64-bit loads (odd number of channel words) the
  // second word of the last pair does not exist
  auto load_pair = [&](__amdgpu_buffer_rsrc_t rsrc, uint32_t boff, auto pair_c, bool second, uint32_t &w0,
                       uint32_t &w1) {
    if constexpr (decltype(pair_c)::value) {
      const auto v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, (int)boff, 0, 0);
      w0 = v[0], w1 = v[1];
    } else {
      w0 = __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)boff, 0, 0);
      w1 = __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)(second && boff != kOff ? boff + 4 : kOff), 0, 0);
    }
  };

  // patch pixels this thread stages: byte offset of the pixel (channel word 0) in a plane, or kOff for
  // padding / beyond the range
  uint32_t poff[PATCH_NPT];
  const int pad_v = (p.PHs - p.Hs) >> 1;
  const int yp0 = gy0 * gst, xp0 = gx0 * gst;
#pragma unroll
  for (int j = 0; j < PATCH_NPT; ++j) {
    const int q = tid + j * NT;
    poff[j] = kOff;
    if (q < npp) {
      int xp = xp0 + q;
      const int cy = (int)fast_div((uint32_t)xp, (uint32_t)p.PWs, p.magicPW);
      xp -= cy * p.PWs;
      int yp = yp0 + cy;
      const int ci = (int)fast_div((uint32_t)yp, (uint32_t)p.PHs, p.magicPH);
      yp -= ci * p.PHs;
      const int img = b0i + ci;
      const int iy = yp - pad_v, ix = xp - pad_v;
      if (img < p.batch && iy >= 0 && iy < p.Hs && ix >= 0 && ix < p.Ws)
        poff[j] = ((((uint32_t)img * (uint32_t)p.Hs + (uint32_t)iy) * (uint32_t)p.Ws + (uint32_t)ix) * (uint32_t)p.C32) << 2;
    }
  }

  v16f acc[FA][FB];
#pragma unroll
  for (int x = 0; x < FA; ++x)
#pragma unroll
    for (int y = 0; y < FB; ++y)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[x][y][r] = 0;
  int ssum[FA];
#pragma unroll
  for (int x = 0; x < FA; ++x) ssum[x] = 0;

  EpiOperands<FA, FB> eo;
  epi_prefetch<1, DIRECT_BITS, false>(p, a0 + wa * FA * 32, b0 + wb * FB * 32, lane, eo);

  const bool pair_ok = (p.C32 & 1) == 0;  // 64-bit loads of a channel-word pair
  const int nchunks = (p.C32 + 1) >> 1;
  for (int cc = 0; cc < nchunks; ++cc) {
    const int cw = cc * 2;
    if (cc > 0) __syncthreads();  // every wave has finished reading the previous chunk
    // ---- global loads of the chunk: patch pixels, then the first batch of filter tasks; all are in
    // flight before the first one is consumed ----------------------------------------------------
    uint32_t pw0[PATCH_NPT][PA], pw1[PATCH_NPT][PA];
    const bool second = cw + 1 < p.C32;
    // (one branch on the load width around each batch of loads, not one per load)
    auto patch_load = [&](auto pair_c) {
#pragma unroll
      for (int j = 0; j < PATCH_NPT; ++j) {
        const uint32_t boff = poff[j] != kOff ? poff[j] + ((uint32_t)cw << 2) : kOff;
#pragma unroll
        for (int pl = 0; pl < PA; ++pl) load_pair(rsrcA[pl], boff, pair_c, second, pw0[j][pl], pw1[j][pl]);
      }
    };
    if (pair_ok) patch_load(std::true_type{}); else patch_load(std::false_type{});
    constexpr int FT = 4;  // filter tasks (tap, column) per thread and batch
    const int ntask = taps * TB;
    uint32_t fw0[FT][PB], fw1[FT][PB];
    auto filter_load_w = [&](int first, auto pair_c) {
#pragma unroll
      for (int j = 0; j < FT; ++j) {
        const int t = first + tid + j * NT;
        const int tap = t / TB, col = t % TB;
        const int gcol = b0 + col;
        const uint32_t boff = t < ntask && gcol < p.rowsB
                                  ? (((uint32_t)gcol * (uint32_t)taps + (uint32_t)tap) * (uint32_t)p.C32 + (uint32_t)cw) << 2
                                  : kOff;
#pragma unroll
        for (int pl = 0; pl < PB; ++pl) load_pair(rsrcB[pl], boff, pair_c, second, fw0[j][pl], fw1[j][pl]);
      }
    };
    auto filter_load = [&](int first) {
      if (pair_ok) filter_load_w(first, std::true_type{}); else filter_load_w(first, std::false_type{});
    };
    auto filter_store = [&](int first) {
#pragma unroll
      for (int j = 0; j < FT; ++j) {
        const int t = first + tid + j * NT;
        if (t < ntask) {
          const int tap = t / TB, col = t % TB;
          static_for<0, DB>([&](auto dc) {
            constexpr int d = decltype(dc)::value;
            const v8i e0 = expand_fp4<PB, d>(fw0[j]), e1 = expand_fp4<PB, d>(fw1[j]);
            uint4 *dst = reinterpret_cast<uint4 *>(filtB + (((d * taps + tap) * TB + col) * 2) * 4);
            dst[0] = make_uint4((uint32_t)e0[0], (uint32_t)e0[1], (uint32_t)e0[2], (uint32_t)e0[3]);
            dst[1] = make_uint4((uint32_t)e1[0], (uint32_t)e1[1], (uint32_t)e1[2], (uint32_t)e1[3]);
          });
        }
      }
    };
    filter_load(0);
    // ---- patch chunk: packed words -> FP4 digit operands --------------------------------------
#pragma unroll
    for (int j = 0; j < PATCH_NPT; ++j) {
      const int q = tid + j * NT;
      if (q < npp) {
        int ps = 0;
#pragma unroll
        for (int pl = 0; pl < PA; ++pl) ps += (__popc(pw0[j][pl]) + __popc(pw1[j][pl])) << pl;
        pixsum[q] = ps;
        static_for<0, DA>([&](auto dc) {
          constexpr int d = decltype(dc)::value;
          const v8i e0 = expand_fp4<PA, d>(pw0[j]), e1 = expand_fp4<PA, d>(pw1[j]);
          uint4 *dst = reinterpret_cast<uint4 *>(patchA + ((d * cap + q) * 2) * 4);
          dst[0] = make_uint4((uint32_t)e0[0], (uint32_t)e0[1], (uint32_t)e0[2], (uint32_t)e0[3]);
          dst[1] = make_uint4((uint32_t)e1[0], (uint32_t)e1[1], (uint32_t)e1[2], (uint32_t)e1[3]);
        });
      }
    }
    // ---- filter chunk ----------------------------------------------------------------------
    for (int first = 0; first < ntask; first += FT * NT) {
      filter_store(first);
      if (first + FT * NT < ntask) filter_load(first + FT * NT);
    }
    __syncthreads();

    // ---- taps k-steps: operands straight from LDS --------------------------------------------
    int r = 0, sx = 0;
    for (int tap = 0; tap < taps; ++tap) {
      const int toff = r * p.PWs + sx;
      v8i af[FA][DA], bf[FB][DB];
#pragma unroll
      for (int x = 0; x < FA; ++x) {
        const int pix = prow[x] + toff;
        ssum[x] += pixsum[pix];
#pragma unroll
        for (int d = 0; d < DA; ++d) {
          const uint4 v = *reinterpret_cast<const uint4 *>(patchA + ((d * cap + pix) * 2 + g) * 4);
          af[x][d] = v8i{(int)v.x, (int)v.y, (int)v.z, (int)v.w, 0, 0, 0, 0};
        }
      }
#pragma unroll
      for (int y = 0; y < FB; ++y) {
#pragma unroll
        for (int d = 0; d < DB; ++d) {
          const uint4 v = *reinterpret_cast<const uint4 *>(
              filtB + (((d * taps + tap) * TB + (wb * FB + y) * 32 + li) * 2 + g) * 4);
          bf[y][d] = v8i{(int)v.x, (int)v.y, (int)v.z, (int)v.w, 0, 0, 0, 0};
        }
      }
#pragma unroll
      for (int x = 0; x < FA; ++x)
#pragma unroll
        for (int y = 0; y < FB; ++y) {
          static_for<0, DA>([&](auto dac) {
            static_for<0, DB>([&](auto dbc) {
              constexpr int da = decltype(dac)::value, db = decltype(dbc)::value;
              if constexpr (da + db == 0) {
                acc[x][y] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[x][da], bf[y][db], acc[x][y], 4, 4, 0,
                                                                            0, 0, 0);
              } else {
                acc[x][y] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                    af[x][da], bf[y][db], acc[x][y], 4, 4, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F + 0x02020202 * (da + db));
              }
            });
          });
        }
      if (++sx == p.S) {
        sx = 0;
        ++r;
      }
    }
  }
  epi_finish<true, 1, true, DIRECT_BITS, false>(p, acc, ssum, smem, wave, lane, a0, b0, wa, wb, eo);
}

// LDS bytes of a launch: patch + filter block + pixel sums, at least the slab area of the output stage
constexpr size_t patch_smem_bytes(int PA, int PB, int FB, int TB, int taps, int cap) {
  const size_t da = (PA + 1) / 2, db = (PB + 1) / 2;
  const size_t stage = (da * cap * 8 + db * (size_t)taps * TB * 8 + cap) * sizeof(uint32_t);
  const size_t slab = 4ull * (32 * (FB * 32 + 1) + 32 + FB * 32 + 2 * 32 * FB) * sizeof(int);
  return stage > slab ? stage : slab;
}

enum PatchTile { PT_128x128 = 0, PT_256x64 = 1, PT_64x128 = 2, PT_128x64 = 3, PT_64x64 = 4, PT_COUNT = 5 };
constexpr int kPatchTileA[PT_COUNT] = {128, 256, 64, 128, 64};
constexpr int kPatchTileB[PT_COUNT] = {128, 64, 128, 64, 64};

template <int PA, int PB, int FA, int FB, int WA, int WB>
inline hipError_t launch_patch(const KParams &p, hipStream_t stream) {
  constexpr int TA = WA * FA * 32, TB = WB * FB * 32;
  const int taps = p.KW / p.C32;
  const size_t smem_bytes = patch_smem_bytes(PA, PB, FB, TB, taps, p.patch_cap);
  if (smem_bytes > 160 * 1024 || p.patch_cap > PATCH_NPT * 256) return hipErrorNotSupported;
  auto kern = apnn_patch_conv_kernel<PA, PB, FA, FB, WA, WB, 2>;
  if (smem_bytes > 64 * 1024) {
    static bool raised = false;
    if (!raised) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
      if (e != hipSuccess) return e;
      raised = true;
    }
  }
  const long long tiles = (long long)((p.rowsA + TA - 1) / TA) * ((p.rowsB + TB - 1) / TB);
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(256), smem_bytes, stream, p);
  return hipGetLastError();
}

template <int PA, int PB>
inline hipError_t launch_patch_tile(int tile, const KParams &p, hipStream_t stream) {
  switch (tile) {
    case PT_128x128: return launch_patch<PA, PB, 2, 2, 2, 2>(p, stream);
    case PT_256x64: return launch_patch<PA, PB, 2, 2, 4, 1>(p, stream);
    case PT_64x128: return launch_patch<PA, PB, 1, 2, 2, 2>(p, stream);
    case PT_128x64: return launch_patch<PA, PB, 1, 2, 4, 1>(p, stream);
    case PT_64x64: return launch_patch<PA, PB, 1, 1, 2, 2>(p, stream);
    default: return hipErrorNotSupported;
  }
}

}  // namespace apnn
