// Small helper kernels around the hot path.
#include <hip/hip_runtime.h>

#include "dispatch.h"

namespace apnn {

// Bit-plane packer with the layout of Bit_compression (APNN-TC-nn/src/kernel.cuh:46-77):
// one wave handles 64 consecutive channels of one row, a ballot per bit yields two MSB-first words.
// Bits first_bit .. bits-1 of every value are written, bit b as plane b - first_bit.
__global__ __launch_bounds__(256) void pack_bits_kernel(const uint32_t *__restrict__ values,
                                                        uint32_t *__restrict__ planes, int rows, int C,
                                                        int cpad, int bits, int first_bit) {
  const int lane = threadIdx.x & 63;
  const int wave_in_block = threadIdx.x >> 6;
  const int cw = cpad >> 5;              // words per row
  const int groups = (cpad + 63) >> 6;   // 64-channel groups per row
  const long long total = (long long)rows * groups;
  const long long plane_stride = (long long)rows * cw;
  for (long long g = (long long)blockIdx.x * 4 + wave_in_block; g < total; g += (long long)gridDim.x * 4) {
    const int row = (int)(g / groups);
    const int c = (int)(g % groups) * 64 + lane;
    const uint32_t v = (c < C) ? values[(long long)row * C + c] : 0u;
    for (int b = first_bit; b < bits; ++b) {
      const unsigned long long mask = __ballot((v >> b) & 1u);
      const uint32_t word = (lane < 32) ? __brev((uint32_t)mask) : __brev((uint32_t)(mask >> 32));
      const int wi = c >> 5;
      if ((lane & 31) == 0 && wi < cw) planes[(b - first_bit) * plane_stride + (long long)row * cw + wi] = word;
    }
  }
}

// Quantize_val (APNN-TC-nn/src/kernel.cuh:29-44) fused with the packer above: float -> code -> planes.
__global__ __launch_bounds__(256) void quantize_pack_kernel(const float *__restrict__ values,
                                                            uint32_t *__restrict__ planes, int rows, int C,
                                                            int cpad, int bits, float min_v, float max_v) {
  const int lane = threadIdx.x & 63;
  const int wave_in_block = threadIdx.x >> 6;
  const int cw = cpad >> 5;
  const int groups = (cpad + 63) >> 6;
  const long long total = (long long)rows * groups;
  const long long plane_stride = (long long)rows * cw;
  const uint32_t top = (1u << bits) - 1u;
  const float levels = (float)(1 << bits), range = max_v - min_v;
  for (long long g = (long long)blockIdx.x * 4 + wave_in_block; g < total; g += (long long)gridDim.x * 4) {
    const int row = (int)(g / groups);
    const int c = (int)(g % groups) * 64 + lane;
    uint32_t v = 0u;
    if (c < C) {
      float x = values[(long long)row * C + c];
      x = x < min_v ? min_v : (x > max_v ? max_v : x);
      const float q = __fdiv_rn(__fmul_rn(__fmul_rn(__fsub_rn(x, min_v), levels), 1.0f), range);
      v = min(top, __float2uint_rn(q));
    }
    for (int b = 0; b < bits; ++b) {
      const unsigned long long mask = __ballot((v >> b) & 1u);
      const uint32_t word = (lane < 32) ? __brev((uint32_t)mask) : __brev((uint32_t)(mask >> 32));
      const int wi = c >> 5;
      if ((lane & 31) == 0 && wi < cw) planes[b * plane_stride + (long long)row * cw + wi] = word;
    }
  }
}

// uint8 samples -> top `bits` bits as the code (a uniform 2^bits-level quantizer of [0, 256)) -> planes.
// THRESH: float samples -> one plane, bit = x >= 0 (In128Layer, APNN-TC-nn/src/kernel.cuh:321-340).
template <bool THRESH, class T>
__global__ __launch_bounds__(256) void code_pack_kernel(const T *__restrict__ values, uint32_t *__restrict__ planes,
                                                        int rows, int C, int cpad, int bits) {
  const int lane = threadIdx.x & 63;
  const int wave_in_block = threadIdx.x >> 6;
  const int cw = cpad >> 5;
  const int groups = (cpad + 63) >> 6;
  const long long total = (long long)rows * groups;
  const long long plane_stride = (long long)rows * cw;
  for (long long g = (long long)blockIdx.x * 4 + wave_in_block; g < total; g += (long long)gridDim.x * 4) {
    const int row = (int)(g / groups);
    const int c = (int)(g % groups) * 64 + lane;
    uint32_t v = 0u;
    if (c < C) {
      const T x = values[(long long)row * C + c];
      if constexpr (THRESH) {
        v = x >= (T)0 ? 1u : 0u;
      } else {
        v = (uint32_t)x >> (8 - bits);
      }
    }
    for (int b = 0; b < bits; ++b) {
      const unsigned long long mask = __ballot((v >> b) & 1u);
      const uint32_t word = (lane < 32) ? __brev((uint32_t)mask) : __brev((uint32_t)(mask >> 32));
      const int wi = c >> 5;
      if ((lane & 31) == 0 && wi < cw) planes[b * plane_stride + (long long)row * cw + wi] = word;
    }
  }
}

static unsigned pack_blocks(int rows, int cpad) {
  const long long total = (long long)rows * ((cpad + 63) / 64);
  long long blocks = (total + 3) / 4;
  if (blocks > 65536) blocks = 65536;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

hipError_t launch_quantize_pack_u8(const uint8_t *values, uint32_t *planes, int rows, int C, int cpad, int bits,
                                   hipStream_t s) {
  hipLaunchKernelGGL((code_pack_kernel<false, uint8_t>), dim3(pack_blocks(rows, cpad)), dim3(256), 0, s, values, planes,
                     rows, C, cpad, bits);
  return hipGetLastError();
}

hipError_t launch_binarize_pack(const float *values, uint32_t *planes, int rows, int C, int cpad, hipStream_t s) {
  hipLaunchKernelGGL((code_pack_kernel<true, float>), dim3(pack_blocks(rows, cpad)), dim3(256), 0, s, values, planes, rows,
                     C, cpad, 1);
  return hipGetLastError();
}

// int32 shortcut map -> residual operand of the quantizing epilogue: optional 2x2 max-pool of the source
// map and channel truncation / zero fill (the reference adds the residual to channels below
// residual_channels only and max-pools it when the block halves the map,
// APNN-TC-nn/src/kernel.cuh:779-831).  One thread per four output channels.
__global__ __launch_bounds__(256) void residual_prepare_kernel(const int32_t *__restrict__ in, int32_t *__restrict__ out,
                                                               long long quads, int Ho, int Wo, int in_pitch,
                                                               int channels, int out_channels, int pool) {
  const int q4 = (out_channels + 3) >> 2;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < quads;
       i += (long long)gridDim.x * blockDim.x) {
    const int cq = (int)(i % q4);
    const long long pix = i / q4;
    const int ox = (int)(pix % Wo);
    const long long t = pix / Wo;
    const int oy = (int)(t % Ho);
    const long long b = t / Ho;
    for (int j = 0; j < 4; ++j) {
      const int c = cq * 4 + j;
      if (c >= out_channels) break;
      int v = 0;
      if (c < channels) {
        if (pool) {
          const long long base = ((b * (2 * Ho) + 2 * oy) * (2 * Wo) + 2 * ox) * in_pitch + c;
          const long long down = (long long)(2 * Wo) * in_pitch;
          v = max(max(in[base], in[base + in_pitch]), max(in[base + down], in[base + down + in_pitch]));
        } else {
          v = in[pix * in_pitch + c];
        }
      }
      out[pix * out_channels + c] = v;
    }
  }
}

hipError_t launch_residual_prepare(const int32_t *in, int32_t *out, int B, int Ho, int Wo, int in_pitch, int channels,
                                   int out_channels, int pool, hipStream_t s) {
  const long long quads = (long long)B * Ho * Wo * ((out_channels + 3) / 4);
  long long blocks = (quads + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(residual_prepare_kernel, dim3((unsigned)blocks), dim3(256), 0, s, in, out, quads, Ho, Wo, in_pitch,
                     channels, out_channels, pool);
  return hipGetLastError();
}

hipError_t launch_quantize_pack(const float *values, uint32_t *planes, int rows, int C, int cpad, int bits, float min_v,
                                float max_v, hipStream_t s) {
  const long long total = (long long)rows * ((cpad + 63) / 64);
  long long blocks = (total + 3) / 4;
  if (blocks > 65536) blocks = 65536;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(quantize_pack_kernel, dim3((unsigned)blocks), dim3(256), 0, s, values, planes, rows, C, cpad, bits,
                     min_v, max_v);
  return hipGetLastError();
}

hipError_t launch_pack_bits(const uint32_t *values, uint32_t *planes, int rows, int C, int cpad, int bits,
                            hipStream_t s) {
  const long long total = (long long)rows * ((cpad + 63) / 64);
  long long blocks = (total + 3) / 4;
  if (blocks > 65536) blocks = 65536;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(pack_bits_kernel, dim3((unsigned)blocks), dim3(256), 0, s, values, planes, rows, C, cpad, bits, 0);
  return hipGetLastError();
}

hipError_t launch_pack_top_plane(const uint32_t *values, uint32_t *plane, int rows, int C, int cpad, int bits,
                                 hipStream_t s) {
  hipLaunchKernelGGL(pack_bits_kernel, dim3(pack_blocks(rows, cpad)), dim3(256), 0, s, values, plane, rows, C, cpad, bits,
                     bits - 1);
  return hipGetLastError();
}

}  // namespace apnn
