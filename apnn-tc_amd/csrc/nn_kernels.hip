// Kernels on either side of the low-bit path of a network: the int8 first convolution with its
// threshold quantizer, max-pool + bit-plane packing of the resulting codes, global average pooling
// of packed codes, code unpacking and the int8 classifier.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "../../include/apnn_tc.h"
#include "dispatch.h"

namespace apnn {

// ---- int8 first convolution + per-channel thresholds -> codes ------------------------------------
// X: [B][H][W][C] int8 (or uint8 minus zero_point when zero_point != 0), Wt: [COUT][R][S][C] int8
// (C tiny: 3), thr: [COUT][2^bits-1] int32.
// One work-group computes a strip of 64 output pixels x COUT_T=64 channels; the filter block is
// staged in LDS once, each thread owns one pixel and 16 channels.
template <int COUT_T>
__global__ __launch_bounds__(256) void conv_i8_bn_kernel(const int8_t *__restrict__ X, const int8_t *__restrict__ Wt,
                                                         const int32_t *__restrict__ thr,
                                                         uint8_t *__restrict__ codes, int32_t *__restrict__ acc_out,
                                                         int B, int H, int W, int C, int COUT, int R, int S,
                                                         int stride, int pad, int Ho, int Wo, int bits, int zero_point) {
  extern __shared__ int8_t wlds[];  // [COUT_T][R*S*C]
  const int K = R * S * C;
  const int co0 = blockIdx.y * COUT_T;
  for (int i = threadIdx.x; i < COUT_T * K; i += 256) {
    const int co = co0 + i / K;
    wlds[i] = co < COUT ? Wt[(long long)co * K + (i % K)] : (int8_t)0;
  }
  __syncthreads();
  const int pl = threadIdx.x & 63;          // pixel within the strip
  const int cg = threadIdx.x >> 6;          // channel group: 16 channels
  const long long pix = (long long)blockIdx.x * 64 + pl;
  const long long npix = (long long)B * Ho * Wo;
  if (pix >= npix) return;
  const int ox = (int)(pix % Wo);
  const int oy = (int)((pix / Wo) % Ho);
  const int b = (int)(pix / ((long long)Wo * Ho));
  int acc[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) acc[j] = 0;
  for (int r = 0; r < R; ++r) {
    const int iy = oy * stride + r - pad;
    if (iy < 0 || iy >= H) continue;
    for (int s = 0; s < S; ++s) {
      const int ix = ox * stride + s - pad;
      if (ix < 0 || ix >= W) continue;
      const int8_t *xp = X + (((long long)b * H + iy) * W + ix) * C;
      const int8_t *wp = wlds + (cg * 16) * K + (r * S + s) * C;
      for (int c = 0; c < C; ++c) {
        const int xv = zero_point ? (int)(uint8_t)xp[c] - zero_point : (int)xp[c];
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[j] += xv * (int)wp[j * K + c];
      }
    }
  }
  const int nt = (1 << bits) - 1;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int co = co0 + cg * 16 + j;
    if (co >= COUT) break;
    if (acc_out != nullptr) acc_out[pix * COUT + co] = acc[j];
    if (codes != nullptr) {
      int code = 0;
      for (int k = 0; k < nt; ++k) code += acc[j] >= thr[co * nt + k] ? 1 : 0;
      codes[pix * COUT + co] = (uint8_t)code;
    }
  }
}

// ---- int8 first convolution on the matrix cores ------------------------------------------------------
// Implicit GEMM: rows = 32 consecutive output pixels of one output row (one wave), columns = 64 output
// channels (two 32x32 blocks), K = R*S*C rounded up to k-steps of 32 with v_mfma_i32_32x32x32_i8.
// The filter block [64][T*32] (zero padded) and, per wave, the input patch that the 32 pixels touch
// (R rows x ((31*stride + S) * C) bytes, already minus the zero point, zero outside the image) sit in
// LDS; a small table maps k -> (patch row offset) so that any R, S, C works.
typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef int v16i_t __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void conv_i8_mfma_kernel(const int8_t *__restrict__ X, const int8_t *__restrict__ Wt,
                                                           const int32_t *__restrict__ thr,
                                                           uint8_t *__restrict__ codes, int32_t *__restrict__ acc_out,
                                                           int B, int H, int W, int C, int COUT, int R, int S,
                                                           int stride, int pad, int Ho, int Wo, int bits,
                                                           int zero_point, int T, int rowlen, int patch_bytes) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int K = R * S * C, KP = T * 32;
  int8_t *wl = reinterpret_cast<int8_t *>(lds);                          // [64][KP]
  uint16_t *tab = reinterpret_cast<uint16_t *>(lds + 64 * KP);           // [KP]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 31, g = lane >> 5;
  int8_t *patch = reinterpret_cast<int8_t *>(lds + 64 * KP + 2 * KP) + wave * patch_bytes;
  const int co0 = blockIdx.y * 64;

  for (int i = tid; i < 64 * KP; i += 256) {
    const int co = co0 + i / KP, k = i % KP;
    wl[i] = (co < COUT && k < K) ? Wt[(long long)co * K + k] : (int8_t)0;
  }
  for (int k = tid; k < KP; k += 256) tab[k] = k < K ? (uint16_t)((k / (S * C)) * rowlen + (k % (S * C))) : (uint16_t)0xFFFF;

  const int gpr = (Wo + 31) / 32;
  const long long group = (long long)blockIdx.x * 4 + wave;
  const bool active = group < (long long)B * Ho * gpr;
  const int gx = (int)(group % gpr);
  const int oy = (int)((group / gpr) % Ho);
  const int b = (int)(group / ((long long)gpr * Ho));
  const int ox0 = gx * 32;
  if (active) {
    for (int idx = lane; idx < R * rowlen; idx += 64) {
      const int r = idx / rowlen, j = idx % rowlen;
      const int iy = oy * stride + r - pad;
      const int ix = ox0 * stride - pad + j / C;
      int v = 0;
      if (iy >= 0 && iy < H && ix >= 0 && ix < W) {
        const int8_t raw = X[(((long long)b * H + iy) * W + ix) * C + (j % C)];
        v = zero_point ? (int)(uint8_t)raw - zero_point : (int)raw;
      }
      patch[idx] = (int8_t)v;
    }
  }
  __syncthreads();
  if (!active) return;

  v16i_t acc[2];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[nb][r] = 0;
  const int pix_off = li * stride * C;  // this lane's pixel inside the patch row
  for (int t = 0; t < T; ++t) {
    const int kb = t * 32 + g * 16;
    uint32_t a[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t word = 0;
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) {
        const uint32_t off = tab[kb + q * 4 + bb];
        const uint32_t byte = off == 0xFFFFu ? 0u : (uint32_t)(uint8_t)patch[off + pix_off];
        word |= byte << (8 * bb);
      }
      a[q] = word;
    }
    const v4i_t af = {(int)a[0], (int)a[1], (int)a[2], (int)a[3]};
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const v4i_t bf = *reinterpret_cast<const v4i_t *>(wl + (nb * 32 + li) * KP + kb);
      acc[nb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bf, acc[nb], 0, 0, 0);
    }
  }
  const int nt = (1 << bits) - 1;
  const long long row0 = ((long long)b * Ho + oy) * Wo;
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int co = co0 + nb * 32 + li;
    if (co >= COUT) continue;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int ox = ox0 + 8 * (r >> 2) + 4 * g + (r & 3);
      if (ox >= Wo) continue;
      const long long o = (row0 + ox) * COUT + co;
      const int v = acc[nb][r];
      if (acc_out != nullptr) acc_out[o] = v;
      if (codes != nullptr) {
        int code = 0;
        for (int k = 0; k < nt; ++k) code += v >= thr[co * nt + k] ? 1 : 0;
        codes[o] = (uint8_t)code;
      }
    }
  }
}

// ---- int8 first convolution for C <= 4 (images), dword-per-pixel patch ------------------------------
// Same implicit GEMM as above, but the LDS patch stores every input pixel as one dword
// (c0, c1, c2, c3-or-zero), and K is laid out per filter row as S pixels x 4 bytes rounded up to whole
// k-steps of 32.  A lane's 16 operand bytes of a k-step are then four consecutive, 4-byte aligned
// dwords of the patch -- four LDS dword reads instead of thirty-two byte reads through a k table.  The
// padding bytes of K carry zero weights, so whatever the patch holds there does not matter.
// Output: uint8 codes, int32 sums and / or MSB-first bit-planes [bits][B*Ho*Wo][COUT/32].
__global__ __launch_bounds__(256) void conv_i8_c4_kernel(const int8_t *__restrict__ X, const int8_t *__restrict__ Wt,
                                                         const int32_t *__restrict__ thr,
                                                         uint8_t *__restrict__ codes, int32_t *__restrict__ acc_out,
                                                         uint32_t *__restrict__ planes, int B, int H, int W, int C,
                                                         int COUT, int R, int S, int stride, int pad, int Ho, int Wo,
                                                         int bits, int zero_point, int KR, int PW, int patch_words) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int KP = R * KR * 32;
  const int KPL = KP + 16;  // row pitch in LDS: 16 B of padding spreads the 32 rows over the banks
  int8_t *wl = reinterpret_cast<int8_t *>(lds);  // [64][KPL]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 31, g = lane >> 5;
  uint32_t *patch = reinterpret_cast<uint32_t *>(lds + 64 * KPL) + wave * patch_words;  // [R][PW] pixels
  const int co0 = blockIdx.y * 64;

  for (int i = tid; i < 64 * KP; i += 256) {
    const int co = co0 + i / KP, k = i % KP;
    const int r = k / (KR * 32), rem = k % (KR * 32);
    const int sx = rem >> 2, c = rem & 3;
    wl[(i / KP) * KPL + k] =
        (co < COUT && sx < S && c < C) ? Wt[(((long long)co * R + r) * S + sx) * C + c] : (int8_t)0;
  }

  __syncthreads();  // filter block staged once per work-group

  // Each wave walks over pixel groups (32 consecutive output pixels of one output row) with a
  // grid-wide stride; its patch is private, so no work-group barrier is needed inside the loop
  // (LDS operations of one wave complete in order).
  const int gpr = (Wo + 31) / 32;
  const long long ngroups = (long long)B * Ho * gpr;
  const int nt = (1 << bits) - 1;
  const long long rows_total = (long long)B * Ho * Wo;
  const int cw32 = COUT >> 5;
  int t0[2], t1[2], t2[2];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int co = co0 + nb * 32 + li;
    t0[nb] = t1[nb] = t2[nb] = 0x7fffffff;
    if (co < COUT && thr != nullptr && nt <= 3) {
      t0[nb] = thr[co * nt];
      if (nt > 1) t1[nb] = thr[co * nt + 1];
      if (nt > 2) t2[nb] = thr[co * nt + 2];
    }
  }
  for (long long group = (long long)blockIdx.x * 4 + wave; group < ngroups; group += (long long)gridDim.x * 4) {
    const int gx = (int)(group % gpr);
    const int oy = (int)((group / gpr) % Ho);
    const int b = (int)(group / ((long long)gpr * Ho));
    const int ox0 = gx * 32;
    // patch staging, eight pixels per lane at a time: all global byte loads of a batch are issued
    // before the first one is consumed (one memory round trip per batch, not per pixel)
    for (int base = 0; base < patch_words; base += 64 * 8) {
      uint8_t raw[8][4];
      bool inside[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int idx = base + j * 64 + lane;
        const int r = idx / PW, px = idx % PW;
        const int iy = oy * stride + r - pad;
        const int ix = ox0 * stride - pad + px;
        inside[j] = idx < patch_words && r < R && iy >= 0 && iy < H && ix >= 0 && ix < W;
        const int8_t *src = X + (((long long)b * H + (inside[j] ? iy : 0)) * W + (inside[j] ? ix : 0)) * C;
#pragma unroll
        for (int c = 0; c < 4; ++c) raw[j][c] = (c < C && inside[j]) ? (uint8_t)src[c] : (uint8_t)0;
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int idx = base + j * 64 + lane;
        uint32_t word = 0;
        if (inside[j]) {
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            if (c < C) {
              const int v = zero_point ? (int)raw[j][c] - zero_point : (int)(int8_t)raw[j][c];
              word |= (uint32_t)(uint8_t)(int8_t)v << (8 * c);
            }
          }
        }
        if (idx < patch_words) patch[idx] = word;
      }
    }

    v16i_t acc[2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[nb][r] = 0;
    for (int r = 0; r < R; ++r) {
      for (int h = 0; h < KR; ++h) {
        const uint32_t *ap = patch + r * PW + li * stride + h * 8 + g * 4;
        const v4i_t af = {(int)ap[0], (int)ap[1], (int)ap[2], (int)ap[3]};
        const int kb = (r * KR + h) * 32 + g * 16;
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
          const v4i_t bf = *reinterpret_cast<const v4i_t *>(wl + (nb * 32 + li) * KPL + kb);
          acc[nb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bf, acc[nb], 0, 0, 0);
        }
      }
    }
    const long long row0 = ((long long)b * Ho + oy) * Wo;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const int co = co0 + nb * 32 + li;
      const bool co_ok = co < COUT;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int ox = ox0 + 8 * (r >> 2) + 4 * g + (r & 3);
        const bool ok = co_ok && ox < Wo;
        const long long o = (row0 + ox) * COUT + co;
        const int v = acc[nb][r];
        int code = 0;
        if (ok && thr != nullptr) {
          if (nt <= 3) {
            code = (v >= t0[nb] ? 1 : 0) + (v >= t1[nb] ? 1 : 0) + (v >= t2[nb] ? 1 : 0);
          } else {
            for (int k = 0; k < nt; ++k) code += v >= thr[co * nt + k] ? 1 : 0;
          }
        }
        if (ok && acc_out != nullptr) acc_out[o] = v;
        if (ok && codes != nullptr) codes[o] = (uint8_t)code;
        if (planes != nullptr) {
          for (int bit = 0; bit < bits; ++bit) {
            const unsigned long long mask = __ballot(ok && ((code >> bit) & 1));
            const uint32_t word = g ? __brev((uint32_t)(mask >> 32)) : __brev((uint32_t)mask);
            if (ok && li == 0) planes[bit * rows_total * cw32 + (row0 + ox) * cw32 + (co >> 5)] = word;
          }
        }
      }
    }
  }
}

template <int I, int N, class F>
__device__ __forceinline__ void static_for_n(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for_n<I + 1, N>(f);
  }
}

// old with lanes L0, L0 + 4 replaced by the halves of m0 and lanes L0 + 32, L0 + 36 by the halves of m1
// (wave-uniform compare masks).  A vector instruction that takes a scalar register written by the vector
// instruction just before it needs two wait states, which the compiler inserts only for instructions it
// can see -- not for this opaque assembly, hence the leading s_nop.
template <int L0>
__device__ __forceinline__ int write_mask_lanes(unsigned long long m0, unsigned long long m1, int old) {
  static_assert(L0 >= 0 && L0 + 36 < 64, "lane index");
  asm("s_nop 1\n\t"
      "v_writelane_b32 %0, %1, %5\n\t"
      "v_writelane_b32 %0, %2, %6\n\t"
      "v_writelane_b32 %0, %3, %7\n\t"
      "v_writelane_b32 %0, %4, %8"
      : "+v"(old)
      : "s"((int)(uint32_t)m0), "s"((int)(uint32_t)(m0 >> 32)), "s"((int)(uint32_t)m1), "s"((int)(uint32_t)(m1 >> 32)),
        "n"(L0), "n"(L0 + 4), "n"(L0 + 32), "n"(L0 + 36));
  return old;
}

// ---- int8 first convolution for images, filter rows taken straight from the image bytes ------------
// In NHWC memory the S pixels x C channels under one filter row are S*C consecutive bytes, so K is laid
// out per filter row as that byte run, padded with zero weights to whole 16-byte halves (HPR halves per
// row); the halves of all R rows are numbered consecutively and k-step ks consumes halves 2ks (lane
// half 0) and 2ks+1 (lane half 1).  The patch of a pixel group (32 consecutive output pixels of one
// output row) is R image-row segments copied to LDS as aligned dwords -- no per-pixel repacking -- with
// the zero point removed by an XOR (x - 128 == x ^ 0x80 as int8) and out-of-image dwords set to zero.
// A lane's 16 operand bytes start at byte lead + pixel*stride*C + 16*half of its row segment: five
// aligned dword reads and four v_alignbyte.  With NKS > 0 the wave keeps its 64 x (NKS*32) weight
// block in registers for the whole (persistent) kernel; with NKS == 0 weights are read from LDS.
// The epilogue is the compare-is-ballot scheme of the matrix-core kernels: per accumulator register
// two compares and a select give both bit-plane masks of two output pixels.  Lane li of a column block
// works on output channel 31 - li (its filter row and thresholds are read in that order), so a compare
// mask already is the packed word (channel c at bit 31 - c%32) and needs no bit reversal.
// Requires C <= 4, (W*C) % 4 == 0, X 4-byte aligned, bits <= 2, COUT % 32 == 0.
// NWAV waves per work-group share one filter block in LDS (each wave has its own patch and walks its
// own pixel groups): eight waves where the filter block is large, so that its LDS cost per wave halves
// and four waves per SIMD stay resident (two work-groups per compute unit: the register budget of that
// variant is held to 128 by its launch bounds).
template <int NKS, int NSLOT, int NWAV>
__global__ __launch_bounds__(64 * NWAV, NWAV == 8 ? 4 : 1) void conv_i8_rows_kernel(const uint8_t *__restrict__ X, const int8_t *__restrict__ Wt,
                                                           const int32_t *__restrict__ thr,
                                                           uint32_t *__restrict__ planes, int B, int H, int W, int C,
                                                           int COUT, int R, int S, int stride, int pad, int Ho, int Wo,
                                                           int bits, uint32_t xor_mask, int HPR, int NDW, int PWD,
                                                           uint32_t magic_gpr, uint32_t magic_ho, uint32_t magic_ndw,
                                                           uint32_t magic_nh2, uint32_t magic_hpr, int wt_dwords) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  // n / d by multiply-high with ceil(2^32 / d) where the launcher found it exact (magic != 0)
  auto quot = [](uint32_t n, uint32_t d, uint32_t magic) { return magic != 0 ? __umulhi(n, magic) : (d == 1 ? n : n / d); };
  const int NH = R * HPR;
  const int nks = (NH + 1) / 2;
  const int KB = nks * 32, KPL = KB + 16;
  int8_t *wl = reinterpret_cast<int8_t *>(lds);  // [64][KPL]
  // the wave index is the same in all 64 lanes: as a scalar it keeps the pixel-group arithmetic below
  // (group -> image, output row, image row addresses) on the scalar unit
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 31, g = lane >> 5;
  uint32_t *patch = reinterpret_cast<uint32_t *>(lds + 64 * KPL) + wave * (R * PWD);
  const int co0 = blockIdx.y * 64;
  const int SC = S * C;

  // filter block -> LDS, one 16-byte half per task.  Four tasks per thread are in flight at a time:
  // all their byte loads are issued before the first LDS store, so the block costs one or two memory
  // round trips instead of one per task.
  const int ntasks = 64 * nks * 2;
  for (int t0 = 0; t0 < ntasks; t0 += 4 * 64 * NWAV) {
    uint32_t w[4][4];
    int dst_off[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int task = t0 + u * 64 * NWAV + tid;
      const int col = (int)quot((uint32_t)task, (uint32_t)(nks * 2), magic_nh2), hh = task - col * (nks * 2);
      const int r = (int)quot((uint32_t)hh, (uint32_t)HPR, magic_hpr), hq = hh - r * HPR;
      dst_off[u] = col * KPL + hh * 16;
      const int co = co0 + col;
      const int nvalid = (task < ntasks && co < COUT && r < R) ? min(max(SC - hq * 16, 0), 16) : 0;
      const int8_t *src = Wt + ((long long)co * R + r) * SC + hq * 16;
#pragma unroll
      for (int q = 0; q < 4; ++q) w[u][q] = 0;
      if (wt_dwords) {
        // filter array readable as whole aligned dwords: five dword loads cover the 16 bytes at any
        // byte offset, v_alignbyte shifts them into place, bytes past the row's end are masked off
        const long long boff = src - Wt;
        const uint32_t *wp = reinterpret_cast<const uint32_t *>(Wt) + (boff >> 2);
        const uint32_t sh = (uint32_t)boff & 3u;
        uint32_t d[5];
#pragma unroll
        for (int k = 0; k < 5; ++k) d[k] = (nvalid > 0 && 4 * k < (int)sh + nvalid) ? wp[k] : 0u;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int nb = min(max(nvalid - 4 * q, 0), 4);
          const uint32_t mask = nb == 4 ? 0xffffffffu : ((1u << (8 * nb)) - 1u);
          w[u][q] = __builtin_amdgcn_alignbyte(d[q + 1], d[q], sh) & mask;
        }
      } else {
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (i < nvalid) w[u][i >> 2] |= (uint32_t)(uint8_t)src[i] << (8 * (i & 3));
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int task = t0 + u * 64 * NWAV + tid;
      if (task < ntasks) *reinterpret_cast<uint4 *>(wl + dst_off[u]) = make_uint4(w[u][0], w[u][1], w[u][2], w[u][3]);
    }
  }
  __syncthreads();

  constexpr int NW = NKS > 0 ? NKS : 1;
  v4i_t wreg[2][NW];
  int koff[NW];  // byte offset of this lane's half of k-step ks inside the patch
  if (NKS > 0) {
#pragma unroll
    for (int ks = 0; ks < NW; ++ks) {
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
        wreg[nb][ks] = *reinterpret_cast<const v4i_t *>(wl + (nb * 32 + 31 - li) * KPL + ks * 32 + g * 16);
      const int hh = 2 * ks + g;
      const int r = min(hh / HPR, R - 1);
      koff[ks] = r * PWD * 4 + (hh % HPR) * 16;
    }
  }

  const int nt = (1 << bits) - 1;
  int t0[2], t1[2], t2[2];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int co = co0 + nb * 32 + 31 - li;
    t0[nb] = t1[nb] = t2[nb] = 0x7fffffff;
    if (co < COUT) {
      t0[nb] = thr[co * nt];
      t1[nb] = nt > 1 ? thr[co * nt + 1] : t0[nb];
      t2[nb] = nt > 2 ? thr[co * nt + 2] : t0[nb];
    }
  }

  const int gpr = (Wo + 31) / 32;
  const long long ngroups = (long long)B * Ho * gpr;
  const long long rows_total = (long long)B * Ho * Wo;
  const int cw32 = COUT >> 5;
  const int rowbytes = W * C;
  const int npatch = R * NDW;
  const int lane_bytes = li * stride * C;

  // Patch element idx = slot * 64 + lane is dword d of row segment r, the same for every group:
  // (r, d) is decoded once.  The raw dwords of the next group are requested before the current
  // group is computed (patches of up to 64 * NSLOT dwords: NSLOT = 8 covers a 7x7 stride-2 filter on
  // three channels, 18 an 11x11 stride-4 one; larger patches are staged in place, chunk by chunk).
  const bool prefetch = npatch <= 64 * NSLOT;
  // rd[j]: row segment r in the upper half-word, byte offset 4*d in the lower one; r = NO_ROW marks a
  // slot past the end of the patch (it then fails the row test of every group)
  constexpr int NO_ROW = 0x7fff;
  auto slot_code = [&](int idx) {
    const int r = (int)quot((uint32_t)idx, (uint32_t)NDW, magic_ndw);
    return idx < npatch ? ((r << 16) | (4 * (idx - r * NDW))) : (NO_ROW << 16);
  };
  int rd[NSLOT];
#pragma unroll
  for (int j = 0; j < NSLOT; ++j) rd[j] = slot_code(j * 64 + lane);
  // Loads are unconditional (addresses clamped into the image) and leave the registers untouched until
  // publish(): a load whose value is used inside a branch on its predicate makes the compiler wait
  // for it there, one memory round trip per slot.  raw_ok[j]: slot j lies inside the image.  The address
  // is the image's base (uniform) plus a 32-bit byte offset, seven vector operations per slot: row and
  // byte position, two range tests, two clamps, one multiply-add (the launcher checks H * W * C < 2^31,
  // W * C < 2^24 and H + pad < NO_ROW).
  uint32_t raw[NSLOT];
  bool raw_ok[NSLOT];
  // one patch dword of pixel group grp: image dword and whether it lies inside the image
  auto load_slot = [&](const uint8_t *img, int ybase, int sbase, int code, uint32_t &word, bool &inside) {
    const int iy = ybase + (code >> 16);
    const int sb = sbase + (code & 0xffff);
    inside = (uint32_t)iy < (uint32_t)H && (uint32_t)sb < (uint32_t)rowbytes;
    const int iyc = min(max(iy, 0), H - 1), sbc = min(max(sb, 0), rowbytes - 4);
    const uint32_t off = __umul24((uint32_t)iyc, (uint32_t)rowbytes) + (uint32_t)sbc;
    word = *reinterpret_cast<const uint32_t *>(img + off);
  };
  auto group_origin = [&](uint32_t grp, const uint8_t *&img, int &ybase, int &sbase) {
    const uint32_t trow = quot(grp, (uint32_t)gpr, magic_gpr);
    const int gx = (int)(grp - trow * (uint32_t)gpr);
    const int b = (int)quot(trow, (uint32_t)Ho, magic_ho);
    const int oy = (int)(trow - (uint32_t)b * (uint32_t)Ho);
    sbase = ((gx * 32 * stride - pad) * C) & ~3;  // two's complement: rounds towards minus infinity
    ybase = oy * stride - pad;
    img = X + (long long)b * H * rowbytes;
  };
  auto request = [&](uint32_t grp) {
    const uint8_t *img;
    int ybase, sbase;
    group_origin(grp, img, ybase, sbase);
#pragma unroll
    for (int j = 0; j < NSLOT; ++j) load_slot(img, ybase, sbase, rd[j], raw[j], raw_ok[j]);
  };
  auto publish = [&]() {
#pragma unroll
    for (int j = 0; j < NSLOT; ++j) {
      const uint32_t val = raw_ok[j] ? raw[j] ^ xor_mask : 0u;
      if (rd[j] < (NO_ROW << 16)) patch[(rd[j] >> 16) * PWD + ((rd[j] & 0xffff) >> 2)] = val;
    }
  };
  // patches larger than the slots: staged in place, one dword per lane and round trip
  auto stage_in_place = [&](uint32_t grp) {
    const uint8_t *img;
    int ybase, sbase;
    group_origin(grp, img, ybase, sbase);
#pragma unroll 1
    for (int idx = lane; idx < npatch; idx += 64) {
      const int code = slot_code(idx);
      uint32_t word;
      bool inside;
      load_slot(img, ybase, sbase, code, word, inside);
      patch[(code >> 16) * PWD + ((code & 0xffff) >> 2)] = inside ? word ^ xor_mask : 0u;
    }
  };

  // (the launcher keeps the number of groups below 2^31: 32-bit index arithmetic)
  const uint32_t gstep = gridDim.x * (uint32_t)NWAV, ng = (uint32_t)ngroups;
  uint32_t group = blockIdx.x * (uint32_t)NWAV + (uint32_t)wave;
  if (prefetch && group < ng) request(group);
  for (; group < ng; group += gstep) {
    const uint32_t trow = quot(group, (uint32_t)gpr, magic_gpr);
    const int gx = (int)(group - trow * (uint32_t)gpr);
    const int b = (int)quot(trow, (uint32_t)Ho, magic_ho);
    const int oy = (int)(trow - (uint32_t)b * (uint32_t)Ho);
    const int ox0 = gx * 32;
    const int s0 = (ox0 * stride - pad) * C;
    const int lead = s0 - (s0 & ~3);
    if (prefetch) {
      publish();
      if (group + gstep < ng) request(group + gstep);
    } else {
      stage_in_place(group);
    }

    v16i_t acc[2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[nb][r] = 0;
    const int a0 = lead + lane_bytes;
    auto operand = [&](int byte_off) {
      const int a = a0 + byte_off;
      const uint32_t *wp = patch + (a >> 2);
      const uint32_t sh = (uint32_t)a & 3u;
      const uint32_t w0 = wp[0], w1 = wp[1], w2 = wp[2], w3 = wp[3], w4 = wp[4];
      v4i_t af;
      af[0] = (int)__builtin_amdgcn_alignbyte(w1, w0, sh);
      af[1] = (int)__builtin_amdgcn_alignbyte(w2, w1, sh);
      af[2] = (int)__builtin_amdgcn_alignbyte(w3, w2, sh);
      af[3] = (int)__builtin_amdgcn_alignbyte(w4, w3, sh);
      return af;
    };
    if (NKS > 0) {
#pragma unroll
      for (int ks = 0; ks < NW; ++ks) {
        const v4i_t af = operand(koff[ks]);
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) acc[nb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, wreg[nb][ks], acc[nb], 0, 0, 0);
      }
    } else {
      int r = 0, h = g;  // half index 2ks + g = r * HPR + h
      while (h >= HPR) {
        h -= HPR;
        ++r;
      }
      // k-step 0 is peeled: its matrix instructions take the constant zero as their addend, which saves
      // clearing 32 accumulator registers per pixel group (this loop's trip count is a run-time value)
      auto k_step = [&](int ks, const v16i_t &c0, const v16i_t &c1) {
        const v4i_t af = operand(min(r, R - 1) * PWD * 4 + h * 16);
        const v4i_t b0 = *reinterpret_cast<const v4i_t *>(wl + (31 - li) * KPL + ks * 32 + g * 16);
        const v4i_t b1 = *reinterpret_cast<const v4i_t *>(wl + (63 - li) * KPL + ks * 32 + g * 16);
        acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, b0, c0, 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, b1, c1, 0, 0, 0);
        h += 2;
        while (h >= HPR) {
          h -= HPR;
          ++r;
        }
      };
      const v16i_t zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      k_step(0, zero, zero);
      for (int ks = 1; ks < nks; ++ks) k_step(ks, acc[0], acc[1]);
    }

    // ---- thresholds -> bit-plane words, parked at lane = pixel (+32 for plane 1) -------------------
    int park[2] = {0, 0};
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      static_for_n<0, 16>([&](auto rc) {
        constexpr int r = decltype(rc)::value;
        constexpr int rlo = 8 * (r >> 2) + (r & 3);  // lane half 0's pixel; lane half 1's is rlo + 4
        const int v = acc[nb][r];
        const bool hi1 = v >= t1[nb];
        const unsigned long long m1 = __ballot(hi1);
        const int tsel = hi1 ? t2[nb] : t0[nb];
        const unsigned long long m0 = __ballot(v >= tsel);
        park[nb] = write_mask_lanes<rlo>(m0, m1, park[nb]);
      });
    }
    const int ox = ox0 + li, plane = g;
    if (ox < Wo && plane < bits) {
      uint32_t *dst = planes + plane * rows_total * cw32 + (((long long)b * Ho + oy) * Wo + ox) * cw32 + (co0 >> 5);
      if ((cw32 & 1) == 0) {
        *reinterpret_cast<uint2 *>(dst) = make_uint2((uint32_t)park[0], (uint32_t)park[1]);
      } else {
        dst[0] = (uint32_t)park[0];
        if (co0 + 32 < COUT) dst[1] = (uint32_t)park[1];
      }
    }
  }
}

// ---- max-pool directly on bit-planes ----------------------------------------------------------------
// in: [bits][B*H*W][cw] -> out: [bits][B*Ho*Wo][cw]; the maximum of two multi-bit codes is computed for
// 32 channels at once with bitwise logic (compare from the top plane down).
// NB: planes held in registers (2 for the usual one- and two-bit codes, else 8).  VEC: channel words per
// thread; 2 (64-bit loads and stores, an even number of channel words, 3x3 windows on at most two planes)
// halves the number of load instructions, which is what bounds this kernel.
template <int NB, int VEC = 1>
__global__ __launch_bounds__(256) void pool_planes_kernel(const uint32_t *__restrict__ in, uint32_t *__restrict__ out,
                                                          int B, int H, int W, int cw, int bits, int win, int stride,
                                                          int pad, int Ho, int Wo) {
  const long long rows_in = (long long)B * H * W, rows_out = (long long)B * Ho * Wo;
  const int cwv = cw / VEC;  // threads per output pixel
  const long long total = rows_out * cwv;
  const bool small = total < 0x7fffffffLL;  // 32-bit index arithmetic (64-bit divisions cost ~100 instructions)
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (long long)gridDim.x * blockDim.x) {
    int wi, ox, oy, b;
    long long row;
    if (small) {
      const uint32_t iu = (uint32_t)i, r32 = iu / (uint32_t)cwv;
      wi = (int)(iu - r32 * (uint32_t)cwv) * VEC;
      const uint32_t t = r32 / (uint32_t)Wo;
      ox = (int)(r32 - t * (uint32_t)Wo);
      b = (int)(t / (uint32_t)Ho);
      oy = (int)(t - (uint32_t)b * (uint32_t)Ho);
      row = r32;
    } else {
      wi = (int)(i % cwv) * VEC;
      row = i / cwv;
      ox = (int)(row % Wo);
      oy = (int)((row / Wo) % Ho);
      b = (int)(row / ((long long)Wo * Ho));
    }
    if constexpr (VEC == 2) {
      // two channel words per thread: the same window logic on both halves of 64-bit loads
      uint2 v[9][2];
#pragma unroll
      for (int t = 0; t < 9; ++t) {
        const int iy = oy * stride + t / 3 - pad, ix = ox * stride + t % 3 - pad;
        const bool ok = iy >= 0 && iy < H && ix >= 0 && ix < W;
        const long long rin = ((long long)b * H + iy) * W + ix;
#pragma unroll
        for (int p = 0; p < 2; ++p)
          v[t][p] = (ok && p < bits) ? *reinterpret_cast<const uint2 *>(in + p * rows_in * cw + rin * cw + wi)
                                     : make_uint2(0u, 0u);
      }
      uint32_t m0x = 0, m0y = 0, m1x = 0, m1y = 0;
#pragma unroll
      for (int t = 0; t < 9; ++t) {
        const uint32_t ltx = (v[t][1].x & ~m1x) | (~(v[t][1].x ^ m1x) & v[t][0].x & ~m0x);
        const uint32_t lty = (v[t][1].y & ~m1y) | (~(v[t][1].y ^ m1y) & v[t][0].y & ~m0y);
        m0x = (m0x & ~ltx) | (v[t][0].x & ltx);
        m1x = (m1x & ~ltx) | (v[t][1].x & ltx);
        m0y = (m0y & ~lty) | (v[t][0].y & lty);
        m1y = (m1y & ~lty) | (v[t][1].y & lty);
      }
      *reinterpret_cast<uint2 *>(out + row * cw + wi) = make_uint2(m0x, m0y);
      if (bits > 1) *reinterpret_cast<uint2 *>(out + rows_out * cw + row * cw + wi) = make_uint2(m1x, m1y);
      continue;
    }
    uint32_t m[NB];
#pragma unroll
    for (int p = 0; p < NB; ++p) m[p] = 0;
    if (NB == 2 && win == 3) {
      // the usual 3x3 window on one- or two-bit codes: all eighteen loads are requested before the
      // first compare (out-of-image taps read as code 0, the identity of the maximum)
      uint32_t v[9][2];
#pragma unroll
      for (int t = 0; t < 9; ++t) {
        const int iy = oy * stride + t / 3 - pad, ix = ox * stride + t % 3 - pad;
        const bool ok = iy >= 0 && iy < H && ix >= 0 && ix < W;
        const long long rin = ((long long)b * H + iy) * W + ix;
#pragma unroll
        for (int p = 0; p < 2; ++p) v[t][p] = (ok && p < bits) ? in[p * rows_in * cw + rin * cw + wi] : 0u;
      }
#pragma unroll
      for (int t = 0; t < 9; ++t) {
        // per channel: v > m  <=>  (v1 & ~m1) | (~(v1 ^ m1) & v0 & ~m0)
        const uint32_t lt = (v[t][1] & ~m[1]) | (~(v[t][1] ^ m[1]) & v[t][0] & ~m[0]);
        m[0] = (m[0] & ~lt) | (v[t][0] & lt);
        m[1] = (m[1] & ~lt) | (v[t][1] & lt);
      }
    } else
    for (int r = 0; r < win; ++r) {
      const int iy = oy * stride + r - pad;
      if (iy < 0 || iy >= H) continue;
      for (int sx = 0; sx < win; ++sx) {
        const int ix = ox * stride + sx - pad;
        if (ix < 0 || ix >= W) continue;
        const long long rin = ((long long)b * H + iy) * W + ix;
        uint32_t v[NB];
#pragma unroll
        for (int p = 0; p < NB; ++p) v[p] = p < bits ? in[p * rows_in * cw + rin * cw + wi] : 0u;
        uint32_t gt = 0, lt = 0;  // per channel: m > v decided / m < v decided
#pragma unroll
        for (int p = NB - 1; p >= 0; --p) {
          const uint32_t diff = m[p] ^ v[p], open = ~(gt | lt);
          gt |= open & diff & m[p];
          lt |= open & diff & v[p];
        }
#pragma unroll
        for (int p = 0; p < NB; ++p) m[p] = (m[p] & ~lt) | (v[p] & lt);
      }
    }
#pragma unroll
    for (int p = 0; p < NB; ++p)
      if (p < bits) out[p * rows_out * cw + row * cw + wi] = m[p];
  }
}

// ---- max-pool on codes + bit-plane packing ---------------------------------------------------------
// codes: [B][H][W][C] uint8 -> planes [bits][B*Ho*Wo][cpad/32], window win x win, stride, pad
// (out-of-image taps ignored).  One wave per (pixel, 64-channel group).
__global__ __launch_bounds__(256) void pool_pack_kernel(const uint8_t *__restrict__ codes, uint32_t *__restrict__ planes,
                                                        int B, int H, int W, int C, int cpad, int bits, int win,
                                                        int stride, int pad, int Ho, int Wo) {
  const int lane = threadIdx.x & 63;
  const int cw = cpad >> 5;
  const int groups = (cpad + 63) >> 6;
  const long long rows = (long long)B * Ho * Wo;
  const long long total = rows * groups;
  for (long long gidx = (long long)blockIdx.x * 4 + (threadIdx.x >> 6); gidx < total; gidx += (long long)gridDim.x * 4) {
    const long long row = gidx / groups;
    const int c = (int)(gidx % groups) * 64 + lane;
    const int ox = (int)(row % Wo), oy = (int)((row / Wo) % Ho), b = (int)(row / ((long long)Wo * Ho));
    int v = 0;
    if (c < C) {
      for (int r = 0; r < win; ++r) {
        const int iy = oy * stride + r - pad;
        if (iy < 0 || iy >= H) continue;
        for (int s = 0; s < win; ++s) {
          const int ix = ox * stride + s - pad;
          if (ix < 0 || ix >= W) continue;
          v = max(v, (int)codes[(((long long)b * H + iy) * W + ix) * C + c]);
        }
      }
    }
    for (int bit = 0; bit < bits; ++bit) {
      const unsigned long long mask = __ballot((v >> bit) & 1);
      const uint32_t word = (lane < 32) ? __brev((uint32_t)mask) : __brev((uint32_t)(mask >> 32));
      const int wi = c >> 5;
      if ((lane & 31) == 0 && wi < cw) planes[bit * rows * cw + row * cw + wi] = word;
    }
  }
}

// ---- packed codes -> int8 values (optionally summed over `group` consecutive rows) ---------------
// planes: [bits][rows][cpad/32];  out[r][c] = (sum_{j<group} code[r*group + j][c]) >> shift, int8.
// group = 1, shift = 0: plain unpacking.  group = H*W: global pooling of a feature map.
// JP (a power of two <= 64) consecutive lanes share one output element and split its `group` rows;
// their partial sums meet in a butterfly reduction.
__global__ __launch_bounds__(256) void unpack_sum_kernel(const uint32_t *__restrict__ planes, int8_t *__restrict__ out,
                                                         long long rows_out, int group, int C, int cpad, int bits,
                                                         int shift, int JP) {
  const int cw = cpad >> 5;
  const long long rows_in = rows_out * group;
  const long long total = rows_out * C;
  const int part = threadIdx.x & (JP - 1);
  const long long nthreads = (long long)gridDim.x * blockDim.x;
  // every lane of a JP-group runs the same number of iterations (the shuffles need all of them)
  for (long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x; t / JP < total; t += nthreads) {
    const long long i = t / JP;
    long long r;
    int c;
    if (total < 0x7fffffffLL) {
      const uint32_t r32 = (uint32_t)i / (uint32_t)C;
      c = (int)((uint32_t)i - r32 * (uint32_t)C);
      r = r32;
    } else {
      r = i / C;
      c = (int)(i % C);
    }
    const int sh = 31 - (c & 31);
    int sum = 0;
    for (int j = part; j < group; j += JP) {
      const long long rin = r * group + j;
      int code = 0;
      for (int b = 0; b < bits; ++b) code |= (int)((planes[b * rows_in * cw + rin * cw + (c >> 5)] >> sh) & 1u) << b;
      sum += code;
    }
    for (int off = JP >> 1; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (part == 0) out[i] = (int8_t)min(127, sum >> shift);
  }
}

// Pooled variant of the above for group >= 8 (global pooling of a feature map): one wave per (output
// row, 32-channel word).  Lane j holds pixel j of the group (64 pixels per pass): one load per plane
// and lane, all in flight together; the sum over the pixels of channel c's bit in plane b is the
// population count of a wave-wide compare, accumulated in scalar registers.  Lane c stores channel c.
__global__ __launch_bounds__(256) void pool_sum_kernel(const uint32_t *__restrict__ planes, int8_t *__restrict__ out,
                                                       long long rows_out, int group, int C, int cpad, int bits,
                                                       int shift) {
  const int lane = threadIdx.x & 63;
  const int cw = cpad >> 5;
  const long long task = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (task >= rows_out * cw) return;  // the whole wave
  const long long r = task / cw;
  const int w = (int)(task - r * cw);
  const long long rows_in = rows_out * group;
  int cnt[32];
#pragma unroll
  for (int c = 0; c < 32; ++c) cnt[c] = 0;
  for (int j0 = 0; j0 < group; j0 += 64) {
    const int j = j0 + lane;
    uint32_t wv[8];
#pragma unroll
    for (int b = 0; b < 8; ++b)
      wv[b] = (b < bits && j < group) ? planes[(long long)b * rows_in * cw + (r * group + j) * cw + w] : 0u;
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      if (b < bits) {  // same for the whole wave
        static_for_n<0, 32>([&](auto cc) {
          constexpr int c = decltype(cc)::value;
          cnt[c] += __popcll(__ballot((wv[b] >> (31 - c)) & 1u)) << b;
        });
      }
    }
  }
  int mine = 0;
  static_for_n<0, 32>([&](auto cc) {
    constexpr int c = decltype(cc)::value;
    if (lane == c) mine = cnt[c];
  });
  const int ch = w * 32 + lane;
  if (lane < 32 && ch < C) out[r * C + ch] = (int8_t)min(127, mine >> shift);
}

// ---- int8 classifier: out[b][n] = scale[n] * sum_k X[b][k] * Wt[n][k] + bias[n] -----------------
// One wave per (group of NN output features, group of four batch rows): lanes stride over K in dwords
// (v_dot4_i32_i8 on four int8 pairs), every operand dword is used NN or four times, then wave64
// butterfly reductions.  K % 4 != 0 (or unaligned rows) falls back to byte loads.
// NN output features x 4 batch rows per wave (NN = 4 when the batch is large enough to make operand
// re-reads the cost, else 1: more waves for small batches).
template <int NN>
__global__ __launch_bounds__(256) void fc_i8_kernel(const int8_t *__restrict__ X, const int8_t *__restrict__ Wt,
                                                    const float *__restrict__ scale, const float *__restrict__ bias,
                                                    float *__restrict__ out, int32_t *__restrict__ acc_out, int Bn,
                                                    int N, int K, int vec_ok) {
  const int lane = threadIdx.x & 63;
  const int bgroups = (Bn + 3) >> 2, ngroups = (N + NN - 1) / NN;
  const long long wid = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (wid >= (long long)ngroups * bgroups) return;
  const int n0 = (int)(wid % ngroups) * NN;
  const int b0 = (int)(wid / ngroups) * 4;
  int acc[NN][4];
#pragma unroll
  for (int i = 0; i < NN; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0;
  // the affine map of this wave's features, requested before the K loop (clamped index, no branch) so
  // that the epilogue does not pay a memory round trip per output
  float sc[NN], bi[NN];
#pragma unroll
  for (int i = 0; i < NN; ++i) {
    const int n = min(n0 + i, N - 1);
    sc[i] = scale[n];
    bi[i] = bias[n];
  }
  if (vec_ok) {
    // four independent iterations in flight: a long K would otherwise be one memory round trip per step
#pragma unroll 4
    for (int k4 = lane; k4 < (K >> 2); k4 += 64) {
      int wv[NN], xv[4];
#pragma unroll
      for (int i = 0; i < NN; ++i)
        wv[i] = n0 + i < N ? reinterpret_cast<const int *>(Wt + (long long)(n0 + i) * K)[k4] : 0;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        xv[j] = b0 + j < Bn ? reinterpret_cast<const int *>(X + (long long)(b0 + j) * K)[k4] : 0;
#pragma unroll
      for (int i = 0; i < NN; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_sdot4(xv[j], wv[i], acc[i][j], false);
    }
  } else {
    for (int k = lane; k < K; k += 64) {
#pragma unroll
      for (int i = 0; i < NN; ++i) {
        const int wv = n0 + i < N ? (int)Wt[(long long)(n0 + i) * K + k] : 0;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (b0 + j < Bn) acc[i][j] += (int)X[(long long)(b0 + j) * K + k] * wv;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < NN; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) acc[i][j] += __shfl_xor(acc[i][j], off, 64);
      if (lane == 0 && b0 + j < Bn && n0 + i < N) {
        const long long o = (long long)(b0 + j) * N + n0 + i;
        if (acc_out != nullptr) acc_out[o] = acc[i][j];
        out[o] = (float)acc[i][j] * sc[i] + bi[i];
      }
    }
}

hipError_t launch_conv_i8_bn(const int8_t *X, const int8_t *Wt, const int32_t *thr, uint8_t *codes, int32_t *acc_out,
                             uint32_t *planes, int B, int H, int W, int C, int COUT, int R, int S, int stride, int pad,
                             int bits, int zero_point, hipStream_t s) {
  const int Ho = (H + 2 * pad - R) / stride + 1, Wo = (W + 2 * pad - S) / stride + 1;
  const long long npix = (long long)B * Ho * Wo;
  const long long groups = (long long)B * Ho * ((Wo + 31) / 32);
  dim3 grid((unsigned)((groups + 3) / 4), (unsigned)((COUT + 63) / 64));
  if (C <= 4 && planes != nullptr && codes == nullptr && acc_out == nullptr && bits <= 2 && (COUT % 32) == 0 &&
      groups < 0x7fffffffLL && (long long)H * W * C < 0x7fffffffLL && (long long)W * C < (1 << 24) &&
      (long long)H + pad < 0x7fff && ((W * C) % 4) == 0 && (reinterpret_cast<uintptr_t>(X) & 3u) == 0 && (zero_point == 0 || zero_point == 128) &&
      thr != nullptr) {
    // image rows consumed as bytes (no repacking): see conv_i8_rows_kernel
    const int HPR = (S * C + 15) / 16;
    const int nks = (R * HPR + 1) / 2;
    const int NDW = (3 + (31 * stride + S) * C + 3) / 4;
    const int need = (3 + 31 * stride * C + 16 * (HPR - 1) + 20 + 3) / 4;
    const int PWD = (need > NDW ? need : NDW) | 1;  // odd pitch
    // slots of image dwords a lane keeps in flight: 8 where that covers the patch, else 18 together with
    // eight waves per work-group (large filters: 11x11)
    const bool wide_patch = R * NDW > 64 * 8;
    const int nwav = wide_patch ? 8 : 4;
    const size_t lds = (size_t)64 * (nks * 32 + 16) + (size_t)nwav * R * PWD * 4;
    if (lds <= (wide_patch ? 80 * 1024 : 64 * 1024)) {
      // persistent grid: exactly as many work-groups as the device holds at once
      // Filter block in registers (two work-groups per compute unit fit) while one or two rounds of
      // work-groups cover all pixel groups; beyond that the variant that re-reads the filter from LDS
      // wins through its higher occupancy (four per compute unit).
      const bool wreg = nks == 7 && grid.x <= 1024 && !wide_patch;
      auto kern = wreg ? conv_i8_rows_kernel<7, 8, 4>
                       : (wide_patch ? conv_i8_rows_kernel<0, 18, 8> : conv_i8_rows_kernel<0, 8, 4>);
      if (wide_patch) {
        grid.x = (unsigned)((groups + 7) / 8);
        if (lds > 64 * 1024) {
          static bool raised = false;
          if (!raised) {
            const hipError_t e0 = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                      hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024);
            if (e0 != hipSuccess) return e0;
            raised = true;
          }
        }
      }
      int per_cu = 0, cus = 0, dev = 0;
      hipError_t e = hipGetDevice(&dev);
      if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
      if (e == hipSuccess)
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void *>(kern), 64 * nwav, lds);
      if (e != hipSuccess) return e;
      unsigned resident = (unsigned)(per_cu > 0 ? per_cu : 1) * (unsigned)(cus > 0 ? cus : 256);
      const unsigned slices = grid.y > 0 ? grid.y : 1;
      resident = resident / slices > 0 ? resident / slices : 1;
      dim3 g2(grid.x > resident ? resident : grid.x, grid.y);
      const uint32_t xm = zero_point == 128 ? 0x80808080u : 0u;
      const uint8_t *Xu = reinterpret_cast<const uint8_t *>(X);
      // multiply-high quotients for the pixel-group decode, where they are exact (n * d < 2^32)
      const unsigned long long gpr = (unsigned long long)(Wo + 31) / 32, ngr = (unsigned long long)B * Ho * gpr;
      auto magic = [&](unsigned long long d) {
        return (d >= 2 && ngr * d < (1ull << 32)) ? (uint32_t)(((1ull << 32) + d - 1) / d) : 0u;
      };
      const uint32_t mg = magic(gpr), mh = magic((unsigned long long)Ho);
      // small dividends (patch slots below 1152, filter tasks below 2^16): always exact
      auto small_magic = [](int d) { return d >= 2 ? (uint32_t)(((1ull << 32) + (unsigned)d - 1) / (unsigned)d) : 0u; };
      const uint32_t mn = small_magic(NDW), mt = small_magic(nks * 2), mp = small_magic(HPR);
      // the filter array as aligned dwords: base 4-byte aligned and a whole number of dwords long
      const int wt_dwords = (reinterpret_cast<uintptr_t>(Wt) & 3u) == 0 && ((long long)COUT * R * S * C) % 4 == 0;
      hipLaunchKernelGGL(kern, g2, dim3(64 * nwav), lds, s, Xu, Wt, thr, planes, B, H, W, C, COUT, R, S, stride, pad, Ho,
                         Wo, bits, xm, HPR, NDW, PWD, mg, mh, mn, mt, mp, wt_dwords);
      return hipGetLastError();
    }
  }
  if (C <= 4) {
    // dword-per-pixel patch kernel, persistent over pixel groups: the filter block is staged once
    // per work-group
    if (grid.x > 1024) grid.x = 1024;
    const int KR = (S * 4 + 31) / 32;
    const int PW = 31 * stride + KR * 8;
    const int patch_words = (R * PW + 15) / 16 * 16;
    const size_t lds = (size_t)64 * (R * KR * 32 + 16) + 4 * (size_t)patch_words * 4;
    if (lds <= 160 * 1024) {
      if (lds > 64 * 1024) {
        static bool raised = false;
        if (!raised) {
          const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(conv_i8_c4_kernel),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
          if (e != hipSuccess) return e;
          raised = true;
        }
      }
      hipLaunchKernelGGL(conv_i8_c4_kernel, grid, dim3(256), lds, s, X, Wt, thr, codes, acc_out, planes, B, H, W, C,
                         COUT, R, S, stride, pad, Ho, Wo, bits, zero_point, KR, PW, patch_words);
      return hipGetLastError();
    }
  }
  if (planes != nullptr) return hipErrorNotSupported;  // plane output is produced by the C <= 4 kernel only
  // general C: byte-gather matrix-core kernel whenever its LDS footprint (filter block, k table, 4 patches) fits
  const int T = (R * S * C + 31) / 32;
  const int rowlen = (31 * stride + S) * C;
  const int patch_bytes = (R * rowlen + 15) / 16 * 16;
  const size_t mfma_lds = (size_t)64 * T * 32 + 2 * T * 32 + 4 * (size_t)patch_bytes;
  if (mfma_lds <= 64 * 1024 && R * rowlen < 0xFFFF) {
    hipLaunchKernelGGL(conv_i8_mfma_kernel, grid, dim3(256), mfma_lds, s, X, Wt, thr, codes, acc_out, B, H, W, C, COUT,
                       R, S, stride, pad, Ho, Wo, bits, zero_point, T, rowlen, patch_bytes);
    return hipGetLastError();
  }
  const size_t lds = (size_t)64 * R * S * C;
  dim3 grid2((unsigned)((npix + 63) / 64), (unsigned)((COUT + 63) / 64));
  hipLaunchKernelGGL(conv_i8_bn_kernel<64>, grid2, dim3(256), lds, s, X, Wt, thr, codes, acc_out, B, H, W, C, COUT, R,
                     S, stride, pad, Ho, Wo, bits, zero_point);
  return hipGetLastError();
}

hipError_t launch_pool_planes(const uint32_t *in, uint32_t *out, int B, int H, int W, int cw, int bits, int win,
                              int stride, int pad, hipStream_t s) {
  const int Ho = (H + 2 * pad - win) / stride + 1, Wo = (W + 2 * pad - win) / stride + 1;
  long long blocks = ((long long)B * Ho * Wo * cw + 255) / 256;
  if (blocks > 262144) blocks = 262144;
  // 64-bit accesses need 8-byte aligned rows: an even number of channel words and 8-byte aligned buffers
  const bool vec2 = bits <= 2 && win == 3 && (cw & 1) == 0 &&
                    ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 7) == 0;
  if (vec2)
    hipLaunchKernelGGL((pool_planes_kernel<2, 2>), dim3((unsigned)((blocks + 1) / 2)), dim3(256), 0, s, in, out, B, H, W, cw,
                       bits, win, stride, pad, Ho, Wo);
  else if (bits <= 2)
    hipLaunchKernelGGL(pool_planes_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, s, in, out, B, H, W, cw, bits, win,
                       stride, pad, Ho, Wo);
  else
    hipLaunchKernelGGL(pool_planes_kernel<8>, dim3((unsigned)blocks), dim3(256), 0, s, in, out, B, H, W, cw, bits, win,
                       stride, pad, Ho, Wo);
  return hipGetLastError();
}

hipError_t launch_pool_pack(const uint8_t *codes, uint32_t *planes, int B, int H, int W, int C, int cpad, int bits,
                            int win, int stride, int pad, hipStream_t s) {
  const int Ho = (H + 2 * pad - win) / stride + 1, Wo = (W + 2 * pad - win) / stride + 1;
  const long long total = (long long)B * Ho * Wo * ((cpad + 63) / 64);
  long long blocks = (total + 3) / 4;
  if (blocks > 262144) blocks = 262144;
  hipLaunchKernelGGL(pool_pack_kernel, dim3((unsigned)blocks), dim3(256), 0, s, codes, planes, B, H, W, C, cpad, bits,
                     win, stride, pad, Ho, Wo);
  return hipGetLastError();
}

hipError_t launch_unpack_sum(const uint32_t *planes, int8_t *out, long long rows_out, int group, int C, int cpad,
                             int bits, int shift, hipStream_t s) {
  if (group >= 8) {
    const long long waves = rows_out * (cpad >> 5);
    if ((waves + 3) / 4 <= 0x7fffffffLL) {
      hipLaunchKernelGGL(pool_sum_kernel, dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, s, planes, out, rows_out,
                         group, C, cpad, bits, shift);
      return hipGetLastError();
    }
  }
  int JP = 1;
  while (JP < 16 && JP * 2 <= group) JP *= 2;
  long long blocks = (rows_out * C * JP + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(unpack_sum_kernel, dim3((unsigned)blocks), dim3(256), 0, s, planes, out, rows_out, group, C, cpad,
                     bits, shift, JP);
  return hipGetLastError();
}

// Larger batches: one wave per 8 output features x 8 batch rows (every operand dword is used eight times, so
// the waves re-read half as many bytes from L2 as with 4 x 4).  The 64 per-lane partial sums are reduced
// by a transposing butterfly: at step s a lane keeps the accumulator whose index has bit s equal to its own
// lane bit s and hands the other one to its partner lane, so the number of live accumulators halves at every
// step (63 exchanges in all instead of 6 x 64) and lane l ends up with the complete sum of accumulator l.
// Requires K % 4 == 0 and 4-byte aligned rows.
__global__ __launch_bounds__(256) void fc_i8_tile_kernel(const int8_t *__restrict__ X, const int8_t *__restrict__ Wt,
                                                         const float *__restrict__ scale, const float *__restrict__ bias,
                                                         float *__restrict__ out, int32_t *__restrict__ acc_out, int Bn,
                                                         int N, int K) {
  const int lane = threadIdx.x & 63;
  const int bgroups = (Bn + 7) >> 3, ngroups = (N + 7) >> 3;
  const long long wid = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (wid >= (long long)ngroups * bgroups) return;
  const int n0 = (int)(wid % ngroups) * 8;
  const int b0 = (int)(wid / ngroups) * 8;
  int acc[64];
#pragma unroll
  for (int a = 0; a < 64; ++a) acc[a] = 0;
  // the affine map of this lane's output feature, requested before the K loop
  const int nf = min(n0 + (lane >> 3), N - 1);
  const float out_scale = scale[nf], out_bias = bias[nf];
  const int *wrow[8], *xrow[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    wrow[i] = reinterpret_cast<const int *>(Wt + (long long)min(n0 + i, N - 1) * K);
    xrow[i] = reinterpret_cast<const int *>(X + (long long)min(b0 + i, Bn - 1) * K);
  }
#pragma unroll 2
  for (int k4 = lane; k4 < (K >> 2); k4 += 64) {
    int wv[8], xv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      wv[i] = wrow[i][k4];
      xv[i] = xrow[i][k4];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i * 8 + j] = __builtin_amdgcn_sdot4(xv[j], wv[i], acc[i * 8 + j], false);
  }
  static_for_n<0, 6>([&](auto sc) {
    constexpr int st = decltype(sc)::value;
    constexpr int n = 64 >> st;  // live accumulators before this step
    const bool hi = (lane >> st) & 1;
#pragma unroll
    for (int t = 0; t < n / 2; ++t) {
      const int keep = hi ? acc[2 * t + 1] : acc[2 * t];
      const int send = hi ? acc[2 * t] : acc[2 * t + 1];
      acc[t] = keep + __shfl_xor(send, 1 << st, 64);
    }
  });
  // lane l = 8 * feature + batch row (rows / features past the end were clamped duplicates: dropped here)
  const int i = lane >> 3, j = lane & 7;
  if (n0 + i < N && b0 + j < Bn) {
    const long long o = (long long)(b0 + j) * N + n0 + i;
    if (acc_out != nullptr) acc_out[o] = acc[0];
    out[o] = (float)acc[0] * out_scale + out_bias;
  }
}

hipError_t launch_fc_i8(const int8_t *X, const int8_t *Wt, const float *scale, const float *bias, float *out,
                        int32_t *acc_out, int Bn, int N, int K, hipStream_t s) {
  const int vec_ok = (K % 4 == 0) && ((reinterpret_cast<uintptr_t>(X) | reinterpret_cast<uintptr_t>(Wt)) & 3u) == 0;
  if (vec_ok && Bn >= 32 && (long long)((N + 7) / 8) * ((Bn + 7) / 8) >= 512) {
    const long long waves = (long long)((N + 7) / 8) * ((Bn + 7) / 8);
    hipLaunchKernelGGL(fc_i8_tile_kernel, dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, s, X, Wt, scale, bias, out,
                       acc_out, Bn, N, K);
    return hipGetLastError();
  }
  if ((long long)N * ((Bn + 3) / 4) >= 8192) {  // plenty of waves: four features per wave cut the re-reads of X
    const long long waves = (long long)((N + 3) / 4) * ((Bn + 3) / 4);
    hipLaunchKernelGGL(fc_i8_kernel<4>, dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, s, X, Wt, scale, bias, out,
                       acc_out, Bn, N, K, vec_ok);
  } else {
    const long long waves = (long long)N * ((Bn + 3) / 4);
    hipLaunchKernelGGL(fc_i8_kernel<1>, dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, s, X, Wt, scale, bias, out,
                       acc_out, Bn, N, K, vec_ok);
  }
  return hipGetLastError();
}

}  // namespace apnn
