// C ABI: argument validation, kernel-path / tile selection and launch.  See include/apnn_tc.h.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>

#include <atomic>

#include "../../include/apnn_tc.h"
#include "dispatch.h"

// One error word per device (each device holds its own copy of a __device__ variable).
__device__ int g_kernel_error_word;

namespace {

using apnn::KParams;

constexpr int kMaxDevices = 64;
std::atomic<int *> g_err_ptr[kMaxDevices];

// Address of the current device's error word (nullptr if it cannot be obtained: kernels then skip the
// report).  hipGetSymbolAddress once per device; the name of a __device__ variable is not a device
// address in host code.
int *kernel_error_word() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return nullptr;
  }
  int *ptr = g_err_ptr[dev].load(std::memory_order_acquire);
  if (ptr != nullptr) return ptr;
  void *sym = nullptr;
  if (hipGetSymbolAddress(&sym, HIP_SYMBOL(g_kernel_error_word)) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  g_err_ptr[dev].store(static_cast<int *>(sym), std::memory_order_release);
  return static_cast<int *>(sym);
}

int check_dev_ptr(const void *p) {
  if (p == nullptr) return APNN_ENULL;
  if ((reinterpret_cast<uintptr_t>(p) & 15u) != 0) return APNN_EALIGN;
  return APNN_OK;
}

std::atomic<int> g_cus{-1};

int device_cus() {
  int c = g_cus.load(std::memory_order_relaxed);
  if (c >= 0) return c;
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
    (void)hipGetLastError();
    n = 0;
  }
  g_cus.store(n, std::memory_order_relaxed);
  return n;
}

uint32_t magic_of(int d) { return d >= 2 ? (uint32_t)(((1ull << 32) + (uint32_t)d - 1) / (uint32_t)d) : 0u; }

// largest tile that still gives every compute unit a work-group, else the smallest one
int choose_tile(int rowsA, int rowsB, bool packed) {
  static const int ta[apnn::TILE_COUNT] = {64, 32, 16, 16};
  static const int tb[apnn::TILE_COUNT] = {64, 32, 32, 16};
  const int last = packed ? apnn::TILE_16x32 : apnn::TILE_16x16;
  int cus = device_cus();
  if (cus <= 0) cus = 256;
  for (int t = 0; t <= last; ++t) {
    const long long n = (long long)((rowsA + ta[t] - 1) / ta[t]) * ((rowsB + tb[t] - 1) / tb[t]);
    if (n >= cus) return t;
  }
  return last;
}

int pick_valu_tile(int tile_pin, const KParams &p, bool packed, int *tile) {
  if (tile_pin == 0) {
    *tile = choose_tile(p.rowsA, p.rowsB, packed);
    return APNN_OK;
  }
  const int t = tile_pin - 1;
  if (t >= apnn::TILE_COUNT || (packed && t == apnn::TILE_16x16)) return APNN_EINVAL;
  *tile = t;
  return APNN_OK;
}

int check_epilogue(const apnn_epilogue &e, int rowsB, bool is_conv, int Ho, int Wo) {
  if (e.mode != APNN_EPI_INT32 && e.mode != APNN_EPI_LOWBITS && e.mode != APNN_EPI_BN) return APNN_EINVAL;
  if (e.pool != APNN_POOL_NONE && e.pool != APNN_POOL_AVG2X2 && e.pool != APNN_POOL_MAX2X2) return APNN_EINVAL;
  if (e.mode == APNN_EPI_INT32) {
    if (e.pool != APNN_POOL_NONE || e.residual != nullptr || e.save_acc != nullptr || e.residual_planes != nullptr)
      return APNN_EINVAL;
    return APNN_OK;
  }
  if (e.residual_planes != nullptr) {
    if (e.residual_bits < 1 || e.residual_bits > 8) return APNN_EINVAL;
    if ((reinterpret_cast<uintptr_t>(e.residual_planes) & 3u) != 0) return APNN_EALIGN;
  }
  if (e.out_bits < 1 || e.out_bits > 8) return APNN_EINVAL;
  if (rowsB % 32 != 0) return APNN_EINVAL;
  if (e.mode == APNN_EPI_BN && e.thresholds == nullptr) return APNN_ENULL;
  if (e.pool != APNN_POOL_NONE) {
    if (!is_conv || (Ho & 1) || (Wo & 1)) return APNN_EINVAL;
    if (e.residual != nullptr || e.save_acc != nullptr || e.residual_planes != nullptr) return APNN_EINVAL;
  }
  return APNN_OK;
}

void fill_epilogue(KParams &p, const apnn_epilogue &e, void *out, long long out_rows) {
  p.epi = e.mode;
  p.out_bits = e.out_bits;
  p.pool = e.pool;
  p.thr = e.thresholds;
  p.flip = e.flip;
  p.resid = e.residual;
  p.save_acc = e.save_acc;
  p.resid_planes = e.residual_planes;
  p.resid_bits = e.residual_bits;
  p.resid_scale = e.residual_scale;
  p.out = out;
  p.out_plane = out_rows * (p.rowsB / 32);
}

typedef hipError_t (*valu_fn)(int, int, const KParams &, hipStream_t);

// Matrix-core kernels: both operand encodings for the four benchmark precisions; FP4 only (a reduced
// tile set, see mfma_tile_enabled) for the wider precisions of the reference tree.
valu_fn mfma_gemm_fn(int wb, int xb, bool i8) {
  if (wb == 1 && xb == 2) return i8 ? apnn::mfma_gemm_1_2_x : apnn::mfma4_gemm_1_2_x;
  if (wb == 1 && xb == 3) return i8 ? apnn::mfma_gemm_1_3_x : apnn::mfma4_gemm_1_3_x;
  if (wb == 1 && xb == 4) return i8 ? apnn::mfma_gemm_1_4_x : apnn::mfma4_gemm_1_4_x;
  if (wb == 2 && xb == 2) return i8 ? apnn::mfma_gemm_2_2_x : apnn::mfma4_gemm_2_2_x;
  if (i8) return nullptr;
  if (wb == 1 && xb == 1) return apnn::mfma4_gemm_1_1_x;
  if (wb == 4 && xb == 4) return apnn::mfma4_gemm_4_4_x;
  if (wb == 1 && xb == 8) return apnn::mfma4_gemm_1_8_x;
  if (wb == 2 && xb == 8) return apnn::mfma4_gemm_2_8_x;
  return nullptr;
}

valu_fn mfma_conv_fn(int xb, int wb, bool i8) {
  if (xb == 2 && wb == 1) return i8 ? apnn::mfma_conv_2_1_x : apnn::mfma4_conv_2_1_x;
  if (xb == 3 && wb == 1) return i8 ? apnn::mfma_conv_3_1_x : apnn::mfma4_conv_3_1_x;
  if (xb == 4 && wb == 1) return i8 ? apnn::mfma_conv_4_1_x : apnn::mfma4_conv_4_1_x;
  if (xb == 2 && wb == 2) return i8 ? apnn::mfma_conv_2_2_x : apnn::mfma4_conv_2_2_x;
  if (i8) return nullptr;
  if (xb == 5 && wb == 1) return apnn::mfma4_conv_5_1_x;
  if (xb == 6 && wb == 2) return apnn::mfma4_conv_6_2_x;
  if (xb == 8 && wb == 1) return apnn::mfma4_conv_8_1_x;
  if (xb == 8 && wb == 2) return apnn::mfma4_conv_8_2_x;
  if (xb == 4 && wb == 4) return apnn::mfma4_conv_4_4_x;
  return nullptr;
}

valu_fn mfmaxs_gemm_fn(int wb, int xb) {
  if (wb == 1 && xb == 2) return apnn::mfmaxs_gemm_1_2_x;
  if (wb == 1 && xb == 3) return apnn::mfmaxs_gemm_1_3_x;
  if (wb == 1 && xb == 4) return apnn::mfmaxs_gemm_1_4_x;
  if (wb == 2 && xb == 2) return apnn::mfmaxs_gemm_2_2_x;
  return nullptr;
}

valu_fn mfmaxs_conv_fn(int xb, int wb) {
  if (xb == 2 && wb == 1) return apnn::mfmaxs_conv_2_1_x;
  if (xb == 3 && wb == 1) return apnn::mfmaxs_conv_3_1_x;
  if (xb == 4 && wb == 1) return apnn::mfmaxs_conv_4_1_x;
  if (xb == 2 && wb == 2) return apnn::mfmaxs_conv_2_2_x;
  return nullptr;
}

// Tile of the expand-while-staging kernel: the largest of its shapes that still gives every compute
// unit a work-group (1.5 per unit for 128x128, as for the other matrix-core kernel), else 64x64.
int choose_xs_tile(int rowsA, int rowsB, bool conv) {
  int cus = device_cus();
  if (cus <= 0) cus = 256;
  auto ntiles = [&](int t) {
    return (long long)((rowsA + apnn::kMfmaTileA[t] - 1) / apnn::kMfmaTileA[t]) *
           ((rowsB + apnn::kMfmaTileB[t] - 1) / apnn::kMfmaTileB[t]);
  };
  auto fill = [&](int t) {
    return (double)rowsA * rowsB / ((double)ntiles(t) * apnn::kMfmaTileA[t] * apnn::kMfmaTileB[t]);
  };
  const int big = conv ? 7 : 6;
  if (rowsB > 64 && ntiles(big) >= cus && fill(big) >= 0.8) return big;
  if (rowsB > 64 && 2 * ntiles(1) >= 3 * cus && fill(1) >= 0.8) return 1;
  if (ntiles(3) >= cus && fill(3) >= 0.8) return 3;
  return 2;
}

// The FP4 matrix-core kernels accumulate in fp32: every partial sum is a multiple of 1/4 and stays
// exact while the largest possible result, K * (2^w - 1) * (2^a - 1), is below 2^24.
bool fp4_exact(long long kwords, int wb, int xb) {
  return kwords * 32 * ((1LL << wb) - 1) * ((1LL << xb) - 1) < (1LL << 24);
}

// Whether the quantizing epilogue of the FP4 kernels may compare in fp32: accumulator range (K x weight
// range x activation range) plus the largest scaled shortcut code stay below 2^24.
int epilogue_float_ok(const KParams &p, int wb, int xb) {
  const long long acc = (long long)p.KW * 32 * ((1LL << wb) - 1) * ((1LL << xb) - 1);
  long long sc = 0;
  if (p.resid_planes != nullptr) {
    const long long scale = p.resid_scale < 0 ? -(long long)p.resid_scale : p.resid_scale;
    sc = scale * ((1LL << p.resid_bits) - 1);
  }
  return acc + sc < (1LL << 24) ? 1 : 0;
}

// Every kernel accumulates (or, on the FP4 core, converts) into int32.  The largest magnitude a result
// can take -- K x weight range x activation range, doubled by the symmetric-weight form 2*raw - wmax*sum,
// plus the largest scaled shortcut code -- has to stay below 2^31; requests beyond that would wrap
// silently and are refused.  (An int32 residual map adds a caller-supplied term that cannot be bounded
// here; it wraps as int32 addition does.)
bool int32_range_ok(long long kwords, int wb, int xb, bool sym, const apnn_epilogue &e) {
  const long long span = ((1LL << wb) - 1) * ((1LL << xb) - 1);  // at most 255 * 255
  long long top = kwords * 32 * span;                              // kwords <= 2^26 here: no overflow of int64
  if (sym) top *= 2;
  if (e.mode != APNN_EPI_INT32 && e.residual_planes != nullptr) {
    const long long scale = e.residual_scale < 0 ? -(long long)e.residual_scale : e.residual_scale;
    top += scale * ((1LL << e.residual_bits) - 1);
  }
  return top < (1LL << 31);
}

// resid_scale as terms the matrix cores can apply to FP4 shortcut digits (KParams::fold).  A digit v means
// v / 2 and the accumulator holds result / vscale (vscale = 4, or 8 with symmetric weights), so a term
// t = s * m * 2^j (m = 1 or 3) needs the FP4 value s * m / 2 (codes 1 and 3, sign in bit 3) and the block
// scale 2^(j - sym).  Two terms at most; 0 when the scale needs more, when there is no packed shortcut of
// one or two bits, or when fp32 could round (accumulator range plus both terms' largest magnitude must stay
// below 2^24, as for epilogue_float_ok).
uint32_t shortcut_fold(const KParams &p, int wb, int xb) {
  if (p.resid_planes == nullptr || p.resid_bits < 1 || p.resid_bits > 2 || p.resid_scale == 0) return 0u;
  if (p.epi == APNN_EPI_INT32 || p.pool != APNN_POOL_NONE) return 0u;
  const long long S = p.resid_scale;
  const int sym = p.sym ? 1 : 0;
  auto term = [&](long long t, uint32_t *nib, uint32_t *e8) {  // t == +-{1,3} * 2^j with j >= 0?
    if (t == 0) return false;
    const long long a = t < 0 ? -t : t;
    int j = 0;
    long long m = a;
    while ((m & 1) == 0) {
      m >>= 1;
      ++j;
    }
    if (m != 1 && m != 3) return false;
    *nib = (m == 1 ? 1u : 3u) | (t < 0 ? 8u : 0u);
    *e8 = (uint32_t)(127 + j - sym);
    return true;
  };
  const long long acc = (long long)p.KW * 32 * ((1LL << wb) - 1) * ((1LL << xb) - 1);
  const long long cmax = (1LL << p.resid_bits) - 1;
  auto fits = [&](long long t0, long long t1) {
    const long long a0 = t0 < 0 ? -t0 : t0, a1 = t1 < 0 ? -t1 : t1;
    return acc + (a0 + a1) * cmax < (1LL << 24);
  };
  uint32_t n0 = 0, e0 = 127, n1 = 0, e1 = 127;
  if (term(S, &n0, &e0)) return fits(S, 0) ? (n0 | (e0 << 8) | (127u << 16)) : 0u;
  for (int j = 0; j < 24; ++j)
    for (int m = 1; m <= 3; m += 2)
      for (int sg = -1; sg <= 1; sg += 2) {
        const long long t0 = (long long)sg * m * (1LL << j);
        if (term(t0, &n0, &e0) && term(S - t0, &n1, &e1) && fits(t0, S - t0))
          return n0 | (n1 << 4) | (e0 << 8) | (e1 << 16);
      }
  return 0u;
}

// Reports a kernel choice instead of launching it (apnn_gemm_plan / apnn_conv_plan).
int fill_plan(apnn_plan *plan, int path, int kernel, int tile, int tr, int tc, int split_k, const KParams &p,
              int patch_pixels_, bool f4ok) {
  plan->path = path;
  plan->kernel = kernel;
  plan->tile = tile;
  plan->tile_rows = tr;
  plan->tile_cols = tc;
  plan->split_k = split_k;
  plan->workgroups = tr > 0 && tc > 0 ? (long long)((p.rowsA + tr - 1) / tr) * ((p.rowsB + tc - 1) / tc) : 0;
  plan->patch_pixels = patch_pixels_;
  plan->fp4_exact = f4ok ? 1 : 0;
  return APNN_OK;
}

// what the register-only kernel (valu_direct_kernel.h) handles
bool direct_kernel_serves(const KParams &p) {
  if ((p.rowsB & 3) != 0 || (p.KW & 3) != 0 || (p.rowsA + 3) / 4 > 65535) return false;
  if ((unsigned long long)p.rowsA * p.KW * 4ull >= (1ull << 32) || (unsigned long long)p.rowsB * p.KW * 4ull >= (1ull << 32))
    return false;  // the kernel addresses rows with 32-bit byte offsets
  if (p.epi == APNN_EPI_INT32) return true;
  return (p.rowsB & 31) == 0 && p.pool == APNN_POOL_NONE && p.resid == nullptr && p.save_acc == nullptr &&
         p.resid_planes == nullptr;
}

typedef hipError_t (*patch_fn)(int, const KParams &, hipStream_t);
patch_fn patch_conv_fn(int xb, int wb) {
  if (xb == 2 && wb == 1) return apnn::patch_conv_2_1_x;
  if (xb == 3 && wb == 1) return apnn::patch_conv_3_1_x;
  if (xb == 4 && wb == 1) return apnn::patch_conv_4_1_x;
  if (xb == 2 && wb == 2) return apnn::patch_conv_2_2_x;
  return nullptr;
}

// Pixels of the padded frame that `rows` consecutive output rows of the implicit GEMM can span,
// maximised over where the run starts.  With gr = b*Ho + oy counting output rows over the batch, the
// padded-frame base of an output pixel is gr*stride*PWs + b*(PHs - Ho*stride)*PWs + ox*stride, and
// along a run d(gr)*Wo + d(ox) = rows - 1; the filter window adds (R-1)*PWs + S.  In pool order a
// row run is rows/4 consecutive 2x2 windows (window grid Ho/2 x Wo/2, step 2*stride) plus one
// window's extent.
int patch_pixels(const KParams &p, int R, int rows) {
  const int st = p.pool_order ? 2 * p.stride : p.stride;
  const int Wo = p.pool_order ? p.Wo / 2 : p.Wo, Ho = p.pool_order ? p.Ho / 2 : p.Ho;
  const int n = p.pool_order ? rows / 4 : rows;
  const int dgr = n > 1 ? (n - 2) / Wo + 1 : 0;            // output-row boundaries crossed, at most
  const int db = dgr > 0 ? (dgr - 1) / Ho + 1 : 0;         // image boundaries crossed, at most
  const int row_gap = st * (p.PWs - Wo) > 0 ? st * (p.PWs - Wo) : 0;
  const int img_gap = (p.PHs - Ho * st) > 0 ? (p.PHs - Ho * st) * p.PWs : 0;
  long long span = (long long)(n - 1) * st + (long long)dgr * row_gap + (long long)db * img_gap;
  if (p.pool_order) span += p.stride * p.PWs + p.stride;
  span += (long long)(R - 1) * p.PWs + p.S;
  return span > 0x7fffffff ? 0x7fffffff : (int)span;
}

// Tile of the patch-resident convolution kernel, or -1 when it does not apply: the patch (at most
// 1024 pixels) and the filter block of all taps must fit in LDS twice per compute unit.  When the
// library chooses (`automatic`) the kernel is taken only where it measures faster than the
// implicit-GEMM kernel: at most 64 output channels over at most 64 input channels (one channel
// chunk, e.g. the first stage of ResNet18) with enough 128x64 tiles to occupy the chip, and layers whose
// channel words are odd in number.
int choose_patch_tile(const KParams &p, int R, int tile_pin, bool automatic) {
  int cus = device_cus();
  if (cus <= 0) cus = 256;
  const int taps = p.KW / p.C32;
  auto fits = [&](int t) {
    const int cap = patch_pixels(p, R, apnn::kPatchTileRows[t]);
    if (cap > 1024) return false;
    // digits: one per plane pair; the byte counts of patch_smem_bytes() for the widest case
    const size_t bytes = ((size_t)2 * cap * 8 + (size_t)taps * apnn::kPatchTileCols[t] * 8 + cap) * 4;
    return bytes <= 80 * 1024;
  };
  auto ntiles = [&](int t) {
    return (long long)((p.rowsA + apnn::kPatchTileRows[t] - 1) / apnn::kPatchTileRows[t]) *
           ((p.rowsB + apnn::kPatchTileCols[t] - 1) / apnn::kPatchTileCols[t]);
  };
  if (automatic) {
    if (tile_pin != 0) return -1;  // a pinned tile names a tile of the implicit-GEMM families
    const int t = 3;               // 128 x 64
    if (p.rowsB <= 64 && p.C32 <= 2 && taps > 1 && fits(t) && ntiles(t) >= 2 * cus) return t;
    // An odd number of channel words (96 channels: the second layer of the VGG variant) leaves the
    // implicit-GEMM kernel with 32-bit loads and its two smallest tiles; this kernel reads pixels, not
    // k-chunks, and is 22-34 % ahead there (56x56x96 -> 256 at batch 8 / 64).
    // (256x64 tiles while 128x64 would give fewer than four work-groups per compute unit: 9 % ahead at batch 8)
    if ((p.C32 & 1) && p.C32 >= 3 && taps > 1 && fits(t) && ntiles(t) >= 2 * cus)
      return (ntiles(t) < 4 * cus && fits(1)) ? 1 : t;
    return -1;
  }
  if (tile_pin != 0) {
    const int t = tile_pin - 1;
    return (t < apnn::kPatchTileCount && fits(t)) ? t : -1;
  }
  const int narrow[3] = {3, 1, 4}, wide[3] = {2, 0, 4};  // 128x64, 256x64, 64x64 / 64x128, 128x128, 64x64
  const int *cand = p.rowsB <= 64 ? narrow : wide;
  for (int i = 0; i < 3; ++i)
    if (fits(cand[i]) && ntiles(cand[i]) >= cus) return cand[i];
  for (int i = 2; i >= 0; --i)
    if (fits(cand[i])) return cand[i];
  return -1;
}

int from_hip(hipError_t e) { return e == hipErrorNotSupported ? APNN_EUNSUPPORTED : (int)e; }

// MFMA tile.  Large problems take the 256x128 (GEMM entry points) / 128x256 (convolution) shape: the
// longer side is on the weight operand, which has fewer bit-planes, so the cheaper operand expansion
// is the one done four times per k-step; then 128x128, 64x64 (128x64 for <= 64 output channels) while every
// compute unit still gets a work-group; when even 64x64 tiles leave most of the chip idle and the
// reduction is long, the 32-row tiles whose four waves split K.
int choose_mfma_tile(int rowsA, int rowsB, int KW, bool conv, int vw, bool i8, int planes = 3, int planesW = 1) {
  const bool wide = planes > 5 || planes == 2;  // the reduced tile set (see mfma_tile_enabled)
  int cus = device_cus();
  if (cus <= 0) cus = 256;
  auto ntiles = [&](int t) {
    return (long long)((rowsA + apnn::kMfmaTileA[t] - 1) / apnn::kMfmaTileA[t]) *
           ((rowsB + apnn::kMfmaTileB[t] - 1) / apnn::kMfmaTileB[t]);
  };
  // fraction of the launched tile area that is real output
  auto fill = [&](int t) {
    return (double)rowsA * rowsB / ((double)ntiles(t) * apnn::kMfmaTileA[t] * apnn::kMfmaTileB[t]);
  };
  if (wide) {  // more than five planes in all, or w1a1: 128x128, 64x64 and the 32x32 split-K tile are built
    if (conv && vw != 4) return 2;
    if (KW >= 32 && ntiles(4) <= 256) return 4;
    return (ntiles(1) >= cus && fill(1) >= 0.8) ? 1 : 2;
  }
  if (i8 && conv) {  // int8 core, convolution: 128x256, 128x128, 128x64, 64x64, 32x32 split-K (128-bit loads)
    if (vw != 4) return 2;
    if (KW >= 32 && ntiles(4) <= 256) return 4;
    if (rowsB > 64 && ntiles(7) >= cus && fill(7) >= 0.8) return 7;
    if (rowsB > 64 && ntiles(1) >= cus && fill(1) >= 0.8) return 1;
    if (rowsB <= 64 && ntiles(3) >= cus) return 3;
    return 2;
  }
  if (i8) {  // int8 core, GEMM entry points: 256x128, 128x128 and 64x64 are built
    if (ntiles(6) >= cus && fill(6) >= 0.8) return 6;
    return (ntiles(1) >= cus && fill(1) >= 0.8) ? 1 : 2;
  }
  if (conv && vw == 1) return (ntiles(2) >= cus / 2 || KW < 16) ? 2 : 4;  // 32-bit loads: two tiles built
  // About one 128x128 tile per compute unit over a long reduction (16x16 maps at batch 16 with 1024 channels,
  // 14x14x256 at batch 64, 2048^2 outputs): plain 128x128 work-groups would leave one wave per SIMD, so two
  // wave groups share each tile's k-steps.  Measured 11-18 % ahead of the best other tile there; with fewer
  // tiles than that the idle compute units cost more than the split-K tiles' extra operand traffic.  How
  // many units may idle depends on what the 32x64 split-K tile costs instead: in convolutions with one
  // weight plane it stays ahead until 9/10 of the units have a tile (16x16 maps with 640..896 channels;
  // 14x14x256 at batch 64: 5 % ahead for w1a2 with quantized output, 17 % for w1a3 / w1a4); with two weight
  // planes, whose expansion the small tiles repeat per 64 channels, and for the GEMM entry points 3/4 suffice
  // (w2a2 on 16x16 maps: 17 % ahead at 768 channels, 34 % at 896).
  if ((!conv || vw == 4) && planes > 2 && KW >= 64 && fill(1) >= 0.8) {
    const long long nt1 = ntiles(1);
    const bool strict = conv && planesW == 1;
    if (2 * nt1 < 3 * cus && (strict ? 10 * nt1 >= 9 * cus : 4 * nt1 >= 3 * cus)) return apnn::MT_128x128_G2;
  }
  // Few outputs over a long reduction (batch-1 / batch-8 layers, 7x7 maps): the split-K tiles give
  // every 32x32 (32x64) block a work-group of its own and the four waves share K.  Measured
  // cross-overs on ResNet18 / 16x16 benchmark shapes.
  if (conv) {
    const long long nb32 = ntiles(4);
    // 32x128 split-K tile: one activation expansion feeds four channel blocks.  It pays with four
    // activation planes over a long reduction while all its work-groups are resident at once (1.5 to 2 per
    // compute unit: 7x7x512 maps at batch 64, 16x16x512 at batch 16; 4-5 % ahead of 32x64).  With fewer
    // activation planes 32x64 is level or ahead, and a grid of 2.5 to 3.5 work-groups per unit pays for the
    // larger tile's longer last round (16x16 maps with 640..896 channels: 32x64 5-20 % ahead).
    if (vw == 4 && planes >= 5 && planesW == 1 && KW >= 128 && rowsB >= 512 && 2 * ntiles(8) >= 3 * cus &&
        ntiles(8) <= 2 * cus)
      return 8;
    // 32x32 blocks, one work-group each: with three planes in all while every compute unit gets at most one
    // (from 296 blocks the 32x64 tile, whose wave expands an activation block once for two channel blocks,
    // is 5-9 % ahead with quantized output and level with int32 output); with four or more planes up to 2.5
    // per compute unit (the second operand's expansion dominates and is not shared: 32x32 stays 2-12 %
    // ahead up to 592 blocks, 32x64 takes over at 784).  Measured on 14x14x256 maps at batch 4..16.
    if (KW >= 32 && nb32 <= (planes <= 3 ? 256 : 640)) return 4;
    if (KW >= 32 && nb32 <= 640) return 5;
    if (KW >= 64 && nb32 <= 14 * cus) return 5;  // up to 3584 blocks: 16x16 maps at batch 16, 896 channels
  }
  if (rowsB <= 64 && ntiles(3) >= cus) return 3;
  if (rowsB > 64) {
    const int big = conv ? 7 : 6;
    if (ntiles(big) >= cus && fill(big) >= 0.8) return big;
    // 128x128 wants more than one work-group per compute unit (measured with three planes in all: with
    // exactly one, the 128x64 tile's two work-groups per compute unit are 3-9 % faster, GEMM 2048^3 and
    // convolution 4096 x 1024; with five planes the larger tile's lower expansion cost per matrix
    // instruction wins by 11 %, w1a4 2048^3)
    if ((planes > 3 ? ntiles(1) >= cus : 2 * ntiles(1) >= 3 * cus) && fill(1) >= 0.8) return 1;
    if (ntiles(3) >= cus && fill(3) >= 0.8) return 3;
    if (ntiles(1) >= cus && fill(1) >= 0.8) return 1;
  }
  if (!conv) {
    // GEMM entry points with few 64x64 tiles (measured at 512^2 and 1024^2 outputs over 1024 bits): the
    // split-K tiles, one 32x32 block per work-group while that fills the chip once, 32x64 up to twice
    if (KW >= 32 && ntiles(4) <= cus) return 4;
    if (KW >= 32 && ntiles(5) <= 2 * cus) return 5;
  }
  if (ntiles(2) >= cus / 2 || KW < 16) return 2;
  return ntiles(5) >= cus / 2 ? 5 : 4;
}

int pick_mfma_tile(int tile_pin, const KParams &p, bool conv, int vw, bool i8, int *tile) {
  if (tile_pin == 0) {
    *tile = choose_mfma_tile(p.rowsA, p.rowsB, p.KW, conv, vw, i8, p.planesA + p.planesB, conv ? p.planesB : p.planesA);
    return APNN_OK;
  }
  if (tile_pin - 1 >= apnn::kMfmaTileCount) return APNN_EINVAL;
  *tile = tile_pin - 1;
  return APNN_OK;
}

// AUTO: the matrix-core path pays off once there are enough 32x32 blocks to fill the chip (measured
// cross-over: about 256x256 outputs at any reduction length, 128x128 when K is at least 1024 bits and
// the split-K tile applies); smaller, latency-bound problems stay on the VALU path, whose 16x16 tiles
// spread them over more compute units.
bool auto_prefers_mfma(const KParams &p) {
  const long long outputs = (long long)p.rowsA * p.rowsB;
  return outputs >= 256LL * 256 || (outputs >= 128LL * 128 && p.KW >= 32);  // long K: split-K matrix-core tile
}
// GEMM at exactly the cross-over size with a short reduction (64 x 1024 outputs over 1024 bits): both
// paths sit on the launch floor and the VALU tile measures a few percent faster.
bool auto_prefers_mfma_gemm(const KParams &p) {
  const long long outputs = (long long)p.rowsA * p.rowsB;
  return outputs > 256LL * 256 || (outputs == 256LL * 256 && p.KW > 32);
}

valu_fn valu_gemm_fn(int wb, int xb) {
  if (wb == 1 && xb == 2) return apnn::valu_gemm_1_2_x;
  if (wb == 1 && xb == 3) return apnn::valu_gemm_1_3_x;
  if (wb == 1 && xb == 4) return apnn::valu_gemm_1_4_x;
  if (wb == 2 && xb == 2) return apnn::valu_gemm_2_2_x;
  return apnn::valu_gemm_any_x;  // 1..8 planes each, one 32x32-tile kernel
}

valu_fn valu_conv_fn(int xb, int wb) {
  if (xb == 2 && wb == 1) return apnn::valu_conv_2_1_x;
  if (xb == 3 && wb == 1) return apnn::valu_conv_3_1_x;
  if (xb == 4 && wb == 1) return apnn::valu_conv_4_1_x;
  if (xb == 2 && wb == 2) return apnn::valu_conv_2_2_x;
  return apnn::valu_conv_any_x;
}

constexpr int kValuTileA[apnn::TILE_COUNT] = {64, 32, 16, 16};
constexpr int kValuTileB[apnn::TILE_COUNT] = {64, 32, 32, 16};

// the any-precision VALU instantiation has one 32x32 tile
int plan_valu(apnn_plan *plan, int tile, bool any, const KParams &p, bool f4ok) {
  const int t = any ? apnn::TILE_32x32 : tile;
  return fill_plan(plan, APNN_PATH_VALU, APNN_KERNEL_VALU_TILE, t, kValuTileA[t], kValuTileB[t], 1, p, 0, f4ok);
}

int plan_direct(apnn_plan *plan, const KParams &p, bool f4ok) {
  // one wave per row and 32 columns, four waves per work-group
  return fill_plan(plan, APNN_PATH_VALU, APNN_KERNEL_VALU_DIRECT, apnn::TILE_DIRECT, 1, 128, 1, p, 0, f4ok);
}

int plan_mfma(apnn_plan *plan, bool i8, int tile, const KParams &p, bool f4ok) {
  const bool split = tile == apnn::MT_32x32_K4 || tile == apnn::MT_32x64_K4 || tile == apnn::MT_32x128_K4;
  const int ksplit = split ? 4 : (tile == apnn::MT_128x128_G2 ? 2 : 1);
  return fill_plan(plan, i8 ? APNN_PATH_MFMA_I8 : APNN_PATH_MFMA, i8 ? APNN_KERNEL_MFMA_I8 : APNN_KERNEL_MFMA_FP4, tile,
                   apnn::kMfmaTileA[tile], apnn::kMfmaTileB[tile], ksplit, p, 0, f4ok);
}

// plan != nullptr: report the choice, launch nothing
int run_gemm(const apnn_gemm_desc *d, hipStream_t stream, apnn_plan *plan = nullptr) {
  if (d == nullptr) return APNN_ENULL;
  int rc;
  if ((rc = check_dev_ptr(d->W)) || (rc = check_dev_ptr(d->X)) || (rc = check_dev_ptr(d->D))) return rc;
  if (d->M <= 0 || d->N <= 0 || d->K <= 0 || (d->K % 128) != 0) return APNN_EINVAL;
  if (d->wb < 1 || d->xb < 1 || d->wb > 8 || d->xb > 8) return APNN_EINVAL;
  if (d->weight_mode != APNN_WEIGHT_UNSIGNED && d->weight_mode != APNN_WEIGHT_SYMMETRIC) return APNN_EINVAL;
  const int path = d->path & 0xff, tile_pin = (d->path >> 8) & 0xff;
  if ((d->path >> 16) != 0 || (path < APNN_PATH_AUTO || path > APNN_PATH_MFMA_XS))
    return APNN_EINVAL;
  if ((rc = check_epilogue(d->epi, d->N, false, 0, 0))) return rc;
  if (!int32_range_ok(d->K / 32, d->wb, d->xb, d->weight_mode == APNN_WEIGHT_SYMMETRIC, d->epi)) return APNN_EINVAL;

  KParams p{};
  p.A = static_cast<const uint32_t *>(d->W);
  p.B = static_cast<const uint32_t *>(d->X);
  p.rowsA = d->M;
  p.rowsB = d->N;
  p.KW = d->K / 32;
  p.planeA = (long long)d->M * p.KW;
  p.planeB = (long long)d->N * p.KW;
  p.sym = d->weight_mode == APNN_WEIGHT_SYMMETRIC;
  p.wmax = (1 << d->wb) - 1;
  fill_epilogue(p, d->epi, d->D, d->M);

  int tile;
  p.planesA = d->wb;
  p.planesB = d->xb;
  const bool f4ok = fp4_exact(p.KW, d->wb, d->xb);
  p.epi_float = epilogue_float_ok(p, d->wb, d->xb);
  p.fold = shortcut_fold(p, d->wb, d->xb);
  p.addr32 = (unsigned long long)p.planeA * 4ull < (1ull << 32) && (unsigned long long)p.planeB * 4ull < (1ull << 32);
  if (path == APNN_PATH_MFMA_PATCH) return APNN_EUNSUPPORTED;  // convolution only
  if ((path == APNN_PATH_MFMA || path == APNN_PATH_MFMA_XS) && !f4ok) return APNN_EUNSUPPORTED;  // fp32 would round
  if (path == APNN_PATH_MFMA_XS) {
    valu_fn fn = mfmaxs_gemm_fn(d->wb, d->xb);
    if (fn == nullptr) return APNN_EUNSUPPORTED;
    tile = tile_pin == 0 ? choose_xs_tile(p.rowsA, p.rowsB, false) : tile_pin - 1;
    if (tile >= apnn::kMfmaTileCount) return APNN_EINVAL;
    if (!apnn::mfma_xs_tile_enabled(false, 4, tile)) return APNN_EUNSUPPORTED;
    if (plan != nullptr)
      return fill_plan(plan, APNN_PATH_MFMA_XS, APNN_KERNEL_MFMA_FP4_XS, tile, apnn::kMfmaTileA[tile],
                       apnn::kMfmaTileB[tile], 1, p, 0, f4ok);
    return from_hip(fn(4, tile, p, stream));
  }
  // operand planes of 4 GiB or more: the matrix-core kernels address rows with 32-bit offsets and refuse
  if ((path == APNN_PATH_MFMA || path == APNN_PATH_MFMA_I8) && !p.addr32) return APNN_EUNSUPPORTED;
  if (path == APNN_PATH_MFMA || path == APNN_PATH_MFMA_I8 ||
      (path == APNN_PATH_AUTO && p.addr32 && auto_prefers_mfma_gemm(p))) {
    // AUTO: FP4 operands while their fp32 accumulation is exact, the int8 core (int32 accumulate) beyond
    const bool i8 = path == APNN_PATH_MFMA_I8 || (path == APNN_PATH_AUTO && !f4ok);
    valu_fn fn = mfma_gemm_fn(d->wb, d->xb, i8);
    if (fn != nullptr) {
      if ((rc = pick_mfma_tile(tile_pin, p, false, 4, i8, &tile))) return rc;
      // (The kernel that expands operands while staging, APNN_PATH_MFMA_XS, is never AUTO's choice: bound by
      // LDS bandwidth, it measures 15-21 % behind this kernel on its best case, w1a4 at 4096^3..8192^3, and
      // further behind with fewer planes -- see mfma_xs_kernel.h.)
      if (plan != nullptr) {
        // a pinned tile that is not built is reported by the launcher; mirror that here
        return apnn::mfma_tile_enabled(i8 ? apnn::CORE_I8 : apnn::CORE_F4, false, 4, tile, d->wb, d->xb)
                   ? plan_mfma(plan, i8, tile, p, f4ok)
                   : APNN_EUNSUPPORTED;
      }
      return from_hip(fn(4, tile, p, stream));
    }
    if (path != APNN_PATH_AUTO) return APNN_EUNSUPPORTED;  // precisions without a matrix-core kernel
  }
  valu_fn fn = valu_gemm_fn(d->wb, d->xb);
  if (fn == nullptr) return APNN_EUNSUPPORTED;
  const bool any = fn == apnn::valu_gemm_any_x;
  const bool direct_ok = !any && direct_kernel_serves(p);
  if (tile_pin == apnn::TILE_DIRECT + 1) {  // register-only kernel
    if (!direct_ok) return APNN_EUNSUPPORTED;
    return plan != nullptr ? plan_direct(plan, p, f4ok) : from_hip(fn(4, apnn::TILE_DIRECT, p, stream));
  }
  // small, latency-bound problems (the M = 64 sweep): one round of loads, no LDS, no barrier
  if (tile_pin == 0 && direct_ok && p.KW <= 64 && (long long)p.rowsA * p.rowsB <= 2 * 256LL * 256)
    return plan != nullptr ? plan_direct(plan, p, f4ok) : from_hip(fn(4, apnn::TILE_DIRECT, p, stream));
  if ((rc = pick_valu_tile(tile_pin, p, d->epi.mode != APNN_EPI_INT32, &tile))) return rc;
  if (plan != nullptr) return plan_valu(plan, tile, any, p, f4ok);
  return (int)fn(4, tile, p, stream);
}

// validation + kernel-side description of a convolution
int build_conv_params(const apnn_conv_desc *d, KParams &p, int *vw_out) {
  if (d == nullptr) return APNN_ENULL;
  int rc;
  if ((rc = check_dev_ptr(d->W)) || (rc = check_dev_ptr(d->X)) || (rc = check_dev_ptr(d->O))) return rc;
  if (d->batch <= 0 || d->H <= 0 || d->Wd <= 0 || d->COUT <= 0) return APNN_EINVAL;
  if (d->cin_pad <= 0 || (d->cin_pad % 32) != 0) return APNN_EINVAL;
  if (d->R <= 0 || d->S <= 0 || d->stride <= 0 || d->pad < 0) return APNN_EINVAL;
  if (d->wb < 1 || d->xb < 1 || d->wb > 8 || d->xb > 8) return APNN_EINVAL;
  if (d->weight_mode != APNN_WEIGHT_UNSIGNED && d->weight_mode != APNN_WEIGHT_SYMMETRIC) return APNN_EINVAL;
  const int path = d->path & 0xff;
  if ((d->path >> 16) != 0 || (path < APNN_PATH_AUTO || path > APNN_PATH_MFMA_XS))
    return APNN_EINVAL;
  if (d->H + 2 * d->pad < d->R || d->Wd + 2 * d->pad < d->S) return APNN_EINVAL;
  const int Ho = (d->H + 2 * d->pad - d->R) / d->stride + 1;
  const int Wo = (d->Wd + 2 * d->pad - d->S) / d->stride + 1;
  if ((rc = check_epilogue(d->epi, d->COUT, true, Ho, Wo))) return rc;
  const long long pixels = (long long)d->batch * Ho * Wo;
  const int C32 = d->cin_pad / 32;
  const long long KW = (long long)d->R * d->S * C32;
  if (pixels > 0x7fffffffLL || KW > (1 << 20)) return APNN_EINVAL;
  if (!int32_range_ok(KW, d->wb, d->xb, d->weight_mode == APNN_WEIGHT_SYMMETRIC, d->epi)) return APNN_EINVAL;
  // a chunk of 4 words must not straddle two taps when 128-bit loads are used
  const int vw = (C32 % 4 == 0) ? 4 : (C32 % 2 == 0) ? 2 : 1;

  p = KParams{};
  p.A = static_cast<const uint32_t *>(d->X);
  p.B = static_cast<const uint32_t *>(d->W);
  p.rowsA = (int)pixels;
  p.rowsB = d->COUT;
  p.KW = (int)KW;
  p.Hs = d->H + (d->halo ? 2 * d->pad : 0);
  p.Ws = d->Wd + (d->halo ? 2 * d->pad : 0);
  p.planeA = (long long)d->batch * p.Hs * p.Ws * C32;
  p.planeB = (long long)d->COUT * KW;
  p.C32 = C32;
  p.Ho = Ho;
  p.Wo = Wo;
  p.S = d->S;
  p.stride = d->stride;
  p.pad = d->halo ? 0 : d->pad;
  p.magicC32 = magic_of(C32);
  p.magicS = magic_of(d->S);
  p.pool_order = d->epi.pool != APNN_POOL_NONE;
  p.sym = d->weight_mode == APNN_WEIGHT_SYMMETRIC;
  p.wmax = (1 << d->wb) - 1;
  fill_epilogue(p, d->epi, d->O, p.pool_order ? pixels / 4 : pixels);

  p.planesA = d->xb;
  p.planesB = d->wb;
  p.epi_float = epilogue_float_ok(p, d->wb, d->xb);
  p.fold = shortcut_fold(p, d->wb, d->xb);
  {
    const bool pow2 = (C32 & (C32 - 1)) == 0;
    int sh = 0;
    while ((1 << sh) < C32) ++sh;
    const long long taps = (long long)d->R * d->S;
    p.c32_shift = pow2 ? sh : -1;
    p.magicS16 = (uint32_t)((65536 + d->S - 1) / d->S);
    p.addr32 = taps * d->S < 65536 && (long long)p.Ws * d->R < (1 << 24) && C32 < (1 << 24) && KW < (1 << 24) &&
               (unsigned long long)p.planeA * 4ull < (1ull << 32) && (unsigned long long)p.planeB * 4ull < (1ull << 32);
  }
  p.batch = d->batch;
  p.PHs = d->H + 2 * d->pad;  // the padded frame: stored frame (incl. a stored halo) plus virtual padding
  p.PWs = d->Wd + 2 * d->pad;
  {
    const int gw = p.pool_order ? Wo / 2 : Wo, gh = p.pool_order ? Ho / 2 : Ho;
    p.magicGW = magic_of(gw);
    p.magicGH = magic_of(gh);
    p.geo_fast = ((unsigned long long)pixels + 1024) * (unsigned long long)(gw > gh ? gw : gh) < (1ull << 32);
  }
  *vw_out = vw;
  return APNN_OK;
}

int run_conv(const apnn_conv_desc *d, hipStream_t stream, apnn_plan *plan = nullptr) {
  KParams p{};
  int vw = 1, rc, tile;
  if ((rc = build_conv_params(d, p, &vw))) return rc;
  const int path = d->path & 0xff, tile_pin = (d->path >> 8) & 0xff;
  const int Ho = p.Ho, Wo = p.Wo;
  const bool f4ok = fp4_exact(p.KW, d->wb, d->xb);
  // A filter that spans the whole stored input map (fully connected layer): every output pixel is one
  // image, whose im2col row is the image itself -- a plain GEMM over rows of KW words.  With few
  // outputs (small batch) the layer streams its weights; the register-only kernel serves it.
  const bool fc_shape = Ho == 1 && Wo == 1 && p.pad == 0 && d->R == p.Hs && d->S == p.Ws;
  {
    valu_fn vf = valu_conv_fn(d->xb, d->wb);
    const bool fc_direct_ok = fc_shape && vf != nullptr && vf != apnn::valu_conv_any_x && direct_kernel_serves(p);
    if (path == APNN_PATH_VALU && tile_pin == apnn::TILE_DIRECT + 1) {
      if (!fc_direct_ok) return APNN_EUNSUPPORTED;
      return plan != nullptr ? plan_direct(plan, p, f4ok) : from_hip(vf(vw, apnn::TILE_DIRECT, p, stream));
    }
    if (path == APNN_PATH_AUTO && tile_pin == 0 && fc_direct_ok && (long long)p.rowsA * p.rowsB <= 2 * 256LL * 256)
      return plan != nullptr ? plan_direct(plan, p, f4ok) : from_hip(vf(vw, apnn::TILE_DIRECT, p, stream));
  }
  // fp32 accumulation of the FP4 kernels would round: pinned FP4 paths refuse, AUTO moves on
  if ((path == APNN_PATH_MFMA || path == APNN_PATH_MFMA_PATCH || path == APNN_PATH_MFMA_XS) && !f4ok)
    return APNN_EUNSUPPORTED;
  if (path == APNN_PATH_MFMA_XS) {
    valu_fn fn = mfmaxs_conv_fn(d->xb, d->wb);
    if (fn == nullptr) return APNN_EUNSUPPORTED;
    tile = tile_pin == 0 ? choose_xs_tile(p.rowsA, p.rowsB, true) : tile_pin - 1;
    if (tile >= apnn::kMfmaTileCount) return APNN_EINVAL;
    if (!apnn::mfma_xs_tile_enabled(true, vw, tile)) return APNN_EUNSUPPORTED;
    if (plan != nullptr)
      return fill_plan(plan, APNN_PATH_MFMA_XS, APNN_KERNEL_MFMA_FP4_XS, tile, apnn::kMfmaTileA[tile],
                       apnn::kMfmaTileB[tile], 1, p, 0, f4ok);
    return from_hip(fn(vw, tile, p, stream));
  }
  if (path == APNN_PATH_MFMA_PATCH || (path == APNN_PATH_AUTO && f4ok)) {
    patch_fn pf = patch_conv_fn(d->xb, d->wb);
    // the kernel addresses pixels and filter rows by 32-bit byte offsets into each operand plane
    const bool planes32 = (unsigned long long)p.planeA * 4ull < (1ull << 32) && (unsigned long long)p.planeB * 4ull < (1ull << 32);
    const int pt = pf == nullptr || !planes32 ? -1 : choose_patch_tile(p, d->R, tile_pin, path == APNN_PATH_AUTO);
    if (pt >= 0) {
      p.patch_cap = patch_pixels(p, d->R, apnn::kPatchTileRows[pt]);
      if (plan == nullptr) p.err = kernel_error_word();
      p.magicPW = magic_of(p.PWs);
      p.magicPH = magic_of(p.PHs);
      if (plan != nullptr)
        return fill_plan(plan, APNN_PATH_MFMA_PATCH, APNN_KERNEL_PATCH_FP4, pt, apnn::kPatchTileRows[pt],
                         apnn::kPatchTileCols[pt], 1, p, p.patch_cap, f4ok);
      return from_hip(pf(pt, p, stream));
    }
    if (path == APNN_PATH_MFMA_PATCH) return APNN_EUNSUPPORTED;
  }
  // operand planes of 4 GiB or more, or a filter beyond the kernels' 24-bit index arithmetic: refused
  if ((path == APNN_PATH_MFMA || path == APNN_PATH_MFMA_I8) && !p.addr32) return APNN_EUNSUPPORTED;
  if (path == APNN_PATH_MFMA || path == APNN_PATH_MFMA_I8 || (path == APNN_PATH_AUTO && p.addr32 && auto_prefers_mfma(p))) {
    const bool i8 = path == APNN_PATH_MFMA_I8 || (path == APNN_PATH_AUTO && !f4ok);
    valu_fn fn = mfma_conv_fn(d->xb, d->wb, i8);
    if (fn != nullptr) {
      if ((rc = pick_mfma_tile(tile_pin, p, true, vw, i8, &tile))) return rc;
      if (plan != nullptr) {
        return apnn::mfma_tile_enabled(i8 ? apnn::CORE_I8 : apnn::CORE_F4, true, vw, tile, d->xb, d->wb)
                   ? plan_mfma(plan, i8, tile, p, f4ok)
                   : APNN_EUNSUPPORTED;
      }
      return from_hip(fn(vw, tile, p, stream));
    }
    if (path != APNN_PATH_AUTO) return APNN_EUNSUPPORTED;
  }
  valu_fn fn = valu_conv_fn(d->xb, d->wb);
  if (fn == nullptr) return APNN_EUNSUPPORTED;
  if ((rc = pick_valu_tile(tile_pin, p, d->epi.mode != APNN_EPI_INT32, &tile))) return rc;
  if (plan != nullptr) return plan_valu(plan, tile, fn == apnn::valu_conv_any_x, p, f4ok);
  return (int)fn(vw, tile, p, stream);
}

// Same input, same output grid, same precision / epilogue mode; see apnn_conv_pair in apnn_tc.h.
int run_conv_pair(const apnn_conv_desc *a, const apnn_conv_desc *b, hipStream_t stream) {
  KParams pa{}, pb{};
  int vwa = 1, vwb = 1, rc;
  if ((rc = build_conv_params(a, pa, &vwa)) || (rc = build_conv_params(b, pb, &vwb))) return rc;
  const bool same = a->X == b->X && a->batch == b->batch && a->H == b->H && a->Wd == b->Wd &&
                    a->cin_pad == b->cin_pad && a->COUT == b->COUT && a->stride == b->stride && a->halo == b->halo &&
                    a->wb == b->wb && a->xb == b->xb && a->weight_mode == b->weight_mode && pa.Ho == pb.Ho &&
                    pa.Wo == pb.Wo && pa.Hs == pb.Hs && pa.Ws == pb.Ws;
  if (!same) return APNN_EINVAL;
  auto plain_bn = [](const apnn_epilogue &e) {
    return e.mode == APNN_EPI_BN && e.pool == APNN_POOL_NONE && e.residual == nullptr && e.save_acc == nullptr &&
           e.residual_planes == nullptr;
  };
  valu_fn fn = mfma_conv_fn(a->xb, a->wb, false);
  const bool fusable = fn != nullptr && plain_bn(a->epi) && plain_bn(b->epi) && a->epi.out_bits == b->epi.out_bits &&
                       (a->path & 0xffff) == APNN_PATH_AUTO && (b->path & 0xffff) == APNN_PATH_AUTO &&
                       auto_prefers_mfma(pa) && pa.addr32 && pb.addr32 && a->O != b->O && fp4_exact(pa.KW, a->wb, a->xb) &&
                       fp4_exact(pb.KW, b->wb, b->xb);
  if (!fusable) {
    if ((rc = run_conv(a, stream))) return rc;
    return run_conv(b, stream);
  }
  // tile for the larger of the two problems, evaluated for twice the number of work-groups
  int tile = choose_mfma_tile(2 * pa.rowsA, pa.rowsB, pa.KW, true, vwa, false, a->xb + a->wb, a->wb);
  pa.pair_tiles = 1;  // flag; the launcher fills in the tile count
  pa.B2 = pb.B;
  pa.KW2 = pb.KW;
  pa.S2 = pb.S;
  pa.pad2 = pb.pad;
  pa.magicS2 = pb.magicS;
  pa.magicS16_2 = pb.magicS16;
  pa.planeB2 = pb.planeB;
  pa.thr2 = pb.thr;
  pa.flip2 = pb.flip;
  pa.out2 = pb.out;
  return from_hip(fn(vwa, tile, pa, stream));
}

int named_gemm(int want_wb, int want_xb, int mode, const void *W, const void *X, int *D, int M, int N, int K,
               int wb, int xb, apnn_stream_t s) {
  if (wb != want_wb || xb != want_xb) return APNN_EINVAL;
  apnn_gemm_desc d{};
  d.W = W;
  d.X = X;
  d.D = D;
  d.M = M;
  d.N = N;
  d.K = K;
  d.wb = wb;
  d.xb = xb;
  d.weight_mode = APNN_WEIGHT_UNSIGNED;
  d.epi.mode = mode;
  d.epi.out_bits = xb;  // the reference decomposes into as many planes as the activations have
  d.path = APNN_PATH_AUTO;
  return run_gemm(&d, static_cast<hipStream_t>(s));
}

int named_conv(int wb, int xb, int mode, int pool, const void *W, const void *X, int *O, int H, int Wd, int CIN,
               int COUT, apnn_stream_t s) {
  if (CIN <= 0 || (CIN % 128) != 0) return APNN_EINVAL;
  apnn_conv_desc d{};
  d.W = W;
  d.X = X;
  d.O = O;
  d.batch = 1;
  d.H = H;
  d.Wd = Wd;
  d.cin_pad = CIN;
  d.COUT = COUT;
  d.R = 3;
  d.S = 3;
  d.stride = 1;
  d.pad = 1;
  d.halo = 1;
  d.wb = wb;
  d.xb = xb;
  d.weight_mode = APNN_WEIGHT_UNSIGNED;
  d.epi.mode = mode;
  d.epi.out_bits = xb;
  d.epi.pool = pool;
  d.path = APNN_PATH_AUTO;
  return run_conv(&d, static_cast<hipStream_t>(s));
}

}  // namespace

extern "C" {

#define APNN_DEF_GEMM(name, w, a, mode)                                                                       \
  int name(const void *W, const void *X, int *D, int M, int N, int K, int wb, int xb, apnn_stream_t s) {      \
    return named_gemm(w, a, mode, W, X, D, M, N, K, wb, xb, s);                                                \
  }
APNN_DEF_GEMM(apmm_w1a2, 1, 2, APNN_EPI_INT32)
APNN_DEF_GEMM(apmm_w1a3, 1, 3, APNN_EPI_INT32)
APNN_DEF_GEMM(apmm_w1a4, 1, 4, APNN_EPI_INT32)
APNN_DEF_GEMM(apmm_w2a2, 2, 2, APNN_EPI_INT32)
APNN_DEF_GEMM(apmm_w1a8, 1, 8, APNN_EPI_INT32)
APNN_DEF_GEMM(apmm_w2a8, 2, 8, APNN_EPI_INT32)
APNN_DEF_GEMM(apmm_w4a4, 4, 4, APNN_EPI_INT32)
APNN_DEF_GEMM(apmm_w1a1, 1, 1, APNN_EPI_INT32)
APNN_DEF_GEMM(apmm_w1a2_decompose, 1, 2, APNN_EPI_LOWBITS)
APNN_DEF_GEMM(apmm_w1a3_decompose, 1, 3, APNN_EPI_LOWBITS)
APNN_DEF_GEMM(apmm_w1a4_decompose, 1, 4, APNN_EPI_LOWBITS)
APNN_DEF_GEMM(apmm_w2a2_decompose, 2, 2, APNN_EPI_LOWBITS)
#undef APNN_DEF_GEMM

#define APNN_DEF_CONV(name, w, a, mode, pool)                                                                  \
  int name(const void *W, const void *X, int *Output, int Height, int Width, int CIN, int COUT,               \
           apnn_stream_t s) {                                                                                  \
    return named_conv(w, a, mode, pool, W, X, Output, Height, Width, CIN, COUT, s);                           \
  }
APNN_DEF_CONV(apconv_w1a2, 1, 2, APNN_EPI_INT32, APNN_POOL_NONE)
APNN_DEF_CONV(apconv_w1a3, 1, 3, APNN_EPI_INT32, APNN_POOL_NONE)
APNN_DEF_CONV(apconv_w1a4, 1, 4, APNN_EPI_INT32, APNN_POOL_NONE)
APNN_DEF_CONV(apconv_w2a2, 2, 2, APNN_EPI_INT32, APNN_POOL_NONE)
APNN_DEF_CONV(apconv_w1a5, 1, 5, APNN_EPI_INT32, APNN_POOL_NONE)
APNN_DEF_CONV(apconv_w2a6, 2, 6, APNN_EPI_INT32, APNN_POOL_NONE)
APNN_DEF_CONV(apconv_w1a8, 1, 8, APNN_EPI_INT32, APNN_POOL_NONE)
APNN_DEF_CONV(apconv_w2a8, 2, 8, APNN_EPI_INT32, APNN_POOL_NONE)
APNN_DEF_CONV(APConv_w2a8_pack, 2, 8, APNN_EPI_LOWBITS, APNN_POOL_NONE)
APNN_DEF_CONV(APConv_w2a8_pack_pool, 2, 8, APNN_EPI_LOWBITS, APNN_POOL_AVG2X2)
APNN_DEF_CONV(APConv_w1a2_pack, 1, 2, APNN_EPI_LOWBITS, APNN_POOL_NONE)
APNN_DEF_CONV(APConv_w1a3_pack, 1, 3, APNN_EPI_LOWBITS, APNN_POOL_NONE)
APNN_DEF_CONV(APConv_w1a4_pack, 1, 4, APNN_EPI_LOWBITS, APNN_POOL_NONE)
APNN_DEF_CONV(APConv_w2a2_pack, 2, 2, APNN_EPI_LOWBITS, APNN_POOL_NONE)
APNN_DEF_CONV(APConv_w1a2_pack_pool, 1, 2, APNN_EPI_LOWBITS, APNN_POOL_AVG2X2)
APNN_DEF_CONV(APConv_w2a2_pack_pool, 2, 2, APNN_EPI_LOWBITS, APNN_POOL_AVG2X2)
#undef APNN_DEF_CONV

int apnn_gemm(const apnn_gemm_desc *d, apnn_stream_t s) { return run_gemm(d, static_cast<hipStream_t>(s)); }
int apnn_conv(const apnn_conv_desc *d, apnn_stream_t s) { return run_conv(d, static_cast<hipStream_t>(s)); }
int apnn_gemm_plan(const apnn_gemm_desc *d, apnn_plan *plan) {
  return plan == nullptr ? APNN_ENULL : run_gemm(d, nullptr, plan);
}
int apnn_conv_plan(const apnn_conv_desc *d, apnn_plan *plan) {
  return plan == nullptr ? APNN_ENULL : run_conv(d, nullptr, plan);
}
int apnn_conv_pair(const apnn_conv_desc *a, const apnn_conv_desc *b, apnn_stream_t s) {
  return run_conv_pair(a, b, static_cast<hipStream_t>(s));
}

int apnn_pack_bits(const uint32_t *values, uint32_t *planes, int rows, int C, int cpad, int bits,
                   apnn_stream_t s) {
  if (values == nullptr || planes == nullptr) return APNN_ENULL;
  if (rows <= 0 || C <= 0 || cpad < C || (cpad % 32) != 0 || bits < 1 || bits > 32) return APNN_EINVAL;
  return (int)apnn::launch_pack_bits(values, planes, rows, C, cpad, bits, static_cast<hipStream_t>(s));
}

int apnn_pack_bits_fc_hidden(const uint32_t *values, uint32_t *plane, int rows, int C, int cpad, int bits,
                             apnn_stream_t s) {
  if (values == nullptr || plane == nullptr) return APNN_ENULL;
  if (rows <= 0 || C <= 0 || cpad < C || (cpad % 32) != 0 || bits < 1 || bits > 32) return APNN_EINVAL;
  return (int)apnn::launch_pack_top_plane(values, plane, rows, C, cpad, bits, static_cast<hipStream_t>(s));
}

int apnn_quantize_pack(const float *values, uint32_t *planes, int rows, int C, int cpad, int bits, float min_v,
                       float max_v, apnn_stream_t s) {
  if (values == nullptr || planes == nullptr) return APNN_ENULL;
  if (rows <= 0 || C <= 0 || cpad < C || (cpad % 32) != 0 || bits < 1 || bits > 16 || !(max_v > min_v))
    return APNN_EINVAL;
  return (int)apnn::launch_quantize_pack(values, planes, rows, C, cpad, bits, min_v, max_v,
                                         static_cast<hipStream_t>(s));
}

int apnn_quantize_pack_u8(const uint8_t *values, uint32_t *planes, int rows, int C, int cpad, int bits,
                          apnn_stream_t s) {
  if (values == nullptr || planes == nullptr) return APNN_ENULL;
  if (rows <= 0 || C <= 0 || cpad < C || (cpad % 32) != 0 || bits < 1 || bits > 8) return APNN_EINVAL;
  return (int)apnn::launch_quantize_pack_u8(values, planes, rows, C, cpad, bits, static_cast<hipStream_t>(s));
}

int apnn_binarize_pack(const float *values, uint32_t *planes, int rows, int C, int cpad, apnn_stream_t s) {
  if (values == nullptr || planes == nullptr) return APNN_ENULL;
  if (rows <= 0 || C <= 0 || cpad < C || (cpad % 32) != 0) return APNN_EINVAL;
  return (int)apnn::launch_binarize_pack(values, planes, rows, C, cpad, static_cast<hipStream_t>(s));
}

int apnn_residual_prepare(const int32_t *in, int32_t *out, int B, int Ho, int Wo, int in_pitch, int channels,
                          int out_channels, int pool, apnn_stream_t s) {
  if (in == nullptr || out == nullptr) return APNN_ENULL;
  if (B <= 0 || Ho <= 0 || Wo <= 0 || out_channels <= 0 || channels < 0 || channels > out_channels ||
      in_pitch < channels || (pool != 0 && pool != 1))
    return APNN_EINVAL;
  return (int)apnn::launch_residual_prepare(in, out, B, Ho, Wo, in_pitch, channels, out_channels, pool,
                                            static_cast<hipStream_t>(s));
}

int apnn_fold_bn(const float *gamma, const float *beta, const float *mean, const float *var, float eps,
                 float in_scale, float step, int C, int bits, int32_t *thresholds, uint8_t *flip) {
  if (gamma == nullptr || beta == nullptr || mean == nullptr || var == nullptr || thresholds == nullptr ||
      flip == nullptr)
    return APNN_ENULL;
  if (C <= 0 || bits < 1 || bits > 8 || !(step > 0.0f) || in_scale == 0.0f) return APNN_EINVAL;
  const int nt = (1 << bits) - 1;
  const double lo = -2147483648.0, hi = 2147483647.0;
  for (int c = 0; c < C; ++c) {
    const double denom = std::sqrt((double)var[c] + (double)eps);
    if (!(denom > 0.0)) return APNN_EINVAL;
    const double slope = (double)gamma[c] / denom;          // dy / d(v * in_scale)
    const double dir = slope * (double)in_scale;            // dy / dv
    auto y_of = [&](double v) { return slope * (v * (double)in_scale - (double)mean[c]) + (double)beta[c]; };
    int32_t *t = thresholds + (long long)c * nt;
    flip[c] = dir < 0.0 ? 1 : 0;
    for (int k = 1; k <= nt; ++k) {
      const double target = (double)k * (double)step;
      if (dir == 0.0) {  // constant output: the comparison is always / never true
        t[k - 1] = (double)beta[c] >= target ? INT32_MIN : INT32_MAX;
        continue;
      }
      // u = v (rising) or -v (falling): smallest integer u with y >= target
      const double sgn = dir < 0.0 ? -1.0 : 1.0;
      double u = std::ceil(sgn * ((target - (double)beta[c]) / slope + (double)mean[c]) / (double)in_scale);
      if (u < lo) u = lo;
      if (u > hi) u = hi;
      // make the closed form agree with y_of() itself at the boundary
      for (int it = 0; it < 4 && u > lo && y_of(sgn * (u - 1.0)) >= target; ++it) u -= 1.0;
      for (int it = 0; it < 4 && u < hi && !(y_of(sgn * u) >= target); ++it) u += 1.0;
      t[k - 1] = (int32_t)u;
    }
  }
  return APNN_OK;
}

int apnn_conv_i8_bn(const int8_t *X, const int8_t *Wt, const int32_t *thresholds, uint8_t *codes, int32_t *acc_out,
                    int B, int H, int W, int C, int COUT, int R, int S, int stride, int pad, int bits,
                    int x_zero_point, apnn_stream_t s) {
  if (X == nullptr || Wt == nullptr || (codes == nullptr && acc_out == nullptr)) return APNN_ENULL;
  if (codes != nullptr && thresholds == nullptr) return APNN_ENULL;
  if (B <= 0 || H <= 0 || W <= 0 || C <= 0 || COUT <= 0 || R <= 0 || S <= 0 || stride <= 0 || pad < 0)
    return APNN_EINVAL;
  if (H + 2 * pad < R || W + 2 * pad < S) return APNN_EINVAL;
  if (codes != nullptr && (bits < 1 || bits > 8)) return APNN_EINVAL;
  if (x_zero_point < 0 || x_zero_point > 255) return APNN_EINVAL;
  if ((long long)64 * R * S * C > 64 * 1024) return APNN_EUNSUPPORTED;  // filter block must fit in LDS
  return from_hip(apnn::launch_conv_i8_bn(X, Wt, thresholds, codes, acc_out, nullptr, B, H, W, C, COUT, R, S, stride,
                                          pad, bits, x_zero_point, static_cast<hipStream_t>(s)));
}

int apnn_conv_i8_bn_pack(const int8_t *X, const int8_t *Wt, const int32_t *thresholds, uint32_t *planes, int B, int H,
                         int W, int C, int COUT, int R, int S, int stride, int pad, int bits, int x_zero_point,
                         apnn_stream_t s) {
  if (X == nullptr || Wt == nullptr || thresholds == nullptr || planes == nullptr) return APNN_ENULL;
  if (B <= 0 || H <= 0 || W <= 0 || C <= 0 || COUT <= 0 || R <= 0 || S <= 0 || stride <= 0 || pad < 0)
    return APNN_EINVAL;
  if (H + 2 * pad < R || W + 2 * pad < S || (COUT % 32) != 0 || bits < 1 || bits > 8) return APNN_EINVAL;
  if (x_zero_point < 0 || x_zero_point > 255) return APNN_EINVAL;
  if (C > 4) return APNN_EUNSUPPORTED;
  return from_hip(apnn::launch_conv_i8_bn(X, Wt, thresholds, nullptr, nullptr, planes, B, H, W, C, COUT, R, S, stride,
                                          pad, bits, x_zero_point, static_cast<hipStream_t>(s)));
}

int apnn_pool_planes(const uint32_t *in, uint32_t *out, int B, int H, int W, int cpad, int bits, int win, int stride,
                     int pad, apnn_stream_t s) {
  if (in == nullptr || out == nullptr) return APNN_ENULL;
  if (B <= 0 || H <= 0 || W <= 0 || cpad <= 0 || (cpad % 32) != 0 || bits < 1 || bits > 8) return APNN_EINVAL;
  if (win <= 0 || stride <= 0 || pad < 0 || pad >= win || H + 2 * pad < win || W + 2 * pad < win) return APNN_EINVAL;
  return (int)apnn::launch_pool_planes(in, out, B, H, W, cpad / 32, bits, win, stride, pad,
                                       static_cast<hipStream_t>(s));
}

int apnn_pool_pack(const uint8_t *codes, uint32_t *planes, int B, int H, int W, int C, int cpad, int bits, int win,
                   int stride, int pad, apnn_stream_t s) {
  if (codes == nullptr || planes == nullptr) return APNN_ENULL;
  if (B <= 0 || H <= 0 || W <= 0 || C <= 0 || cpad < C || (cpad % 32) != 0 || bits < 1 || bits > 8) return APNN_EINVAL;
  if (win <= 0 || stride <= 0 || pad < 0 || pad >= win || H + 2 * pad < win || W + 2 * pad < win) return APNN_EINVAL;
  return (int)apnn::launch_pool_pack(codes, planes, B, H, W, C, cpad, bits, win, stride, pad,
                                     static_cast<hipStream_t>(s));
}

int apnn_unpack_sum(const uint32_t *planes, int8_t *out, long long rows_out, int group, int C, int cpad, int bits,
                    int shift, apnn_stream_t s) {
  if (planes == nullptr || out == nullptr) return APNN_ENULL;
  if (rows_out <= 0 || group <= 0 || C <= 0 || cpad < C || (cpad % 32) != 0 || bits < 1 || bits > 8 || shift < 0 ||
      shift > 16)
    return APNN_EINVAL;
  return (int)apnn::launch_unpack_sum(planes, out, rows_out, group, C, cpad, bits, shift, static_cast<hipStream_t>(s));
}

int apnn_fc_i8(const int8_t *X, const int8_t *Wt, const float *scale, const float *bias, float *out,
               int32_t *acc_out, int B, int N, int K, apnn_stream_t s) {
  if (X == nullptr || Wt == nullptr || scale == nullptr || bias == nullptr || out == nullptr) return APNN_ENULL;
  if (B <= 0 || N <= 0 || K <= 0) return APNN_EINVAL;
  return (int)apnn::launch_fc_i8(X, Wt, scale, bias, out, acc_out, B, N, K, static_cast<hipStream_t>(s));
}

int apnn_device_error(int *code, apnn_stream_t s) {
  if (code == nullptr) return APNN_ENULL;
  *code = 0;
  int *word = kernel_error_word();
  if (word == nullptr) return APNN_EUNSUPPORTED;
  hipStream_t stream = static_cast<hipStream_t>(s);
  hipError_t e = hipStreamSynchronize(stream);
  if (e == hipSuccess) e = hipMemcpy(code, word, sizeof(int), hipMemcpyDeviceToHost);
  if (e == hipSuccess && *code != 0) e = hipMemset(word, 0, sizeof(int));
  return (int)e;
}

int apnn_device_cus(void) { return device_cus(); }
const char *apnn_version(void) { return "apnn-tc-amd 0.1 (gfx950)"; }

}  // extern "C"
