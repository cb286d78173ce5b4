// Layer API of the low-bit network path: host-side C++ classes with the names, constructor
// arguments and life cycle (constructor -> initialize() -> forward -> download_output() -> release())
// of the reference's layer parameter classes in APNN-TC-nn/src/param.h, driven through the C ABI of
// libapnn_tc.so.  Differences that are deliberate:
//   * a layer object stays on the host (the reference copies it to the device and hands the device
//     pointer to a kernel, param.h:949-960); the *_new_global wrappers take the host object and a
//     stream and enqueue the kernels;
//   * batch-norm is folded into 2^a-1 per-channel integer thresholds (the reference's layers have a
//     single float threshold, usable for 1-bit outputs only, kernel.cuh:833-834);
//   * residual blocks: the reference's own mechanism is kept (save_residual stores the int32 sum a layer
//     thresholds, inject_residual adds such a map -- max-pooled 2x2 with residual_pool, to the first
//     residual_channels channels only -- before the thresholds, kernel.cuh:779-869); in addition a layer
//     can take the *packed* output of an earlier layer as its shortcut, added at an integer scale
//     (set_packed_shortcut), which is what the standard ResNet18 here uses: no int32 map in memory;
//   * "ahead_fc" asks for a batch-major output layout (kernel.cuh:837-852); outputs here are always
//     batch-major ([bits][batch*H*W][C/32]), so the flag is accepted and changes nothing;
//   * a constructor argument this build cannot honour (stride_width != stride_height, pool sizes other
//     than 1 or 2, pooling together with an int32 residual) makes initialize() return APNN_EUNSUPPORTED
//     instead of being dropped;
//   * weights and thresholds are random-initialised from a seeded generator (the reference reads a
//     CSV through launch_array, which is disabled: utility.h:174-182).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "../../include/apnn_nn.h"
#include "../../include/apnn_tc.h"

namespace apnn_nn {

inline int pad_to(int x, int m) { return (x + m - 1) / m * m; }

// splitmix64: seeded, platform independent
struct Rng {
  uint64_t s;
  explicit Rng(uint64_t seed) : s(seed) {}
  uint64_t next() {
    uint64_t z = (s += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
  }
  uint32_t below(uint32_t n) { return (uint32_t)((next() >> 32) * (uint64_t)n >> 32); }
  double uniform() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }
};

// device allocation owned by a layer
class DeviceBuffer {
 public:
  DeviceBuffer() = default;
  ~DeviceBuffer() { release(); }
  DeviceBuffer(const DeviceBuffer &) = delete;
  DeviceBuffer &operator=(const DeviceBuffer &) = delete;
  hipError_t allocate(size_t bytes);
  hipError_t upload(const void *host, size_t bytes);
  void release();
  void *get() const { return ptr_; }
  size_t bytes() const { return bytes_; }
  template <class T> T *as() const { return static_cast<T *>(ptr_); }

 private:
  void *ptr_ = nullptr;
  size_t bytes_ = 0;
};

class Layer {
 public:
  virtual ~Layer() = default;
  virtual int forward(hipStream_t stream) = 0;
  virtual void describe(apnn_layer_desc *d) const = 0;
  virtual const uint32_t *get_output_gpu() const { return nullptr; }
  // set on a Conv128LayerParam that reads the same input as the Conv128LayerParam listed before it
  // (the 1x1 downsample convolution of a residual block): the network launches the two as a pair
  bool pairs_with_previous = false;
};

// Input layer of the reference's fully connected networks (In128LayerParam, param.h:106-217): float rows
// -> one bit-plane, bit = value >= 0 (In128Layer, kernel.cuh:321-340).
class In128LayerParam : public Layer {
 public:
  In128LayerParam(const char *name, int input_height, int input_width);
  int initialize(const float *input_gpu);
  int forward(hipStream_t stream) override;
  void describe(apnn_layer_desc *d) const override;
  const uint32_t *get_output_gpu() const override { return output_gpu.as<uint32_t>(); }

  std::string name;
  int input_height, input_width, output_height, output_width, out_cpad;
  const float *input_gpu = nullptr;
  DeviceBuffer output_gpu;
};

// Image quantizer in front of a low-bit first convolution: images_quantization (kernel.cuh:129-161) for
// the uint8 images the networks here take: code = pixel >> (8 - bit), packed into `bit` planes.
class ImageQuantLayerParam : public Layer {
 public:
  ImageQuantLayerParam(const char *name, int batch, int image_height, int image_width, int image_channel, int bit = 2);
  int initialize(const uint8_t *images_gpu);
  void set_input_gpu(const uint8_t *images_gpu) { input_gpu = images_gpu; }
  int forward(hipStream_t stream) override;
  void describe(apnn_layer_desc *d) const override;
  const uint32_t *get_output_gpu() const override { return output_gpu.as<uint32_t>(); }

  std::string name;
  int batch, image_height, image_width, image_channel, bit, out_cpad;
  const uint8_t *input_gpu = nullptr;
  DeviceBuffer output_gpu;
};

// First layer: int8 convolution on uint8 pixels (zero point 128), thresholds -> a-bit codes,
// optional max-pool, bit-plane packing.  Counterpart of InConv128LayerParam (param.h:701-875), which
// binarises a float image convolution; the int8 arithmetic follows cutlass_nn/src/config.h:215-255.
// Arguments up to save_residual are the reference's (param.h:704-708); pool_stride / pool_pad / a_bit
// follow them.  save_residual keeps the int32 convolution sums (before pooling) for a later layer's
// inject_residual.
class InConv128LayerParam : public Layer {
 public:
  InConv128LayerParam(const char *name, int input_height, int input_width, int filter_height, int filter_width,
                      int input_channels, int output_channels, int batch, int stride_height = 1,
                      int stride_width = 1, bool padding = true, int pool_height = 1, int pool_width = 1,
                      bool save_residual = false, int pool_stride = 0, int pool_pad = 0, int a_bit = 2);
  int initialize(Rng &rng, const uint8_t *images_gpu);
  void set_input_gpu(const uint8_t *images_gpu) { input_gpu = images_gpu; }
  int forward(hipStream_t stream) override;
  void describe(apnn_layer_desc *d) const override;
  const uint32_t *get_output_gpu() const override { return output_gpu.as<uint32_t>(); }
  int32_t *get_output_residual_gpu() const { return output_residual_gpu.as<int32_t>(); }
  std::vector<uint32_t> download_output() const;

  std::string name;
  int input_height, input_width, filter_height, filter_width, input_channels, output_channels, batch;
  int stride, pad, pool, pool_stride, pool_pad, a_bit;
  bool save_residual;
  int status = 0;  // APNN_EUNSUPPORTED when a constructor argument cannot be honoured
  int conv_height, conv_width, output_height, output_width, out_cpad;
  const uint8_t *input_gpu = nullptr;
  DeviceBuffer filter_gpu, bn_gpu, codes_gpu, output_gpu, output_residual_gpu;
};

// Low-bit convolution layer (param.h:877-1083), constructor arguments as the reference's
// (param.h:880-894).  pool_height == 2 applies a 2x2 max-pool to the quantized codes inside the
// epilogue.  save_residual stores the int32 value the thresholds see (accumulator plus injected
// residual, kernel.cuh:862-868) as [batch*H*W][output_channels]; inject_residual adds the map given to
// initialize() -- an earlier layer's get_output_residual_gpu() -- to channels below residual_channels,
// max-pooled 2x2 from a map of twice the size with residual_pool.
class Conv128LayerParam : public Layer {
 public:
  Conv128LayerParam(const char *name, int input_height, int input_width, int filter_height, int filter_width,
                    int input_channels, int output_channels, int batch, int stride_height = 1, int stride_width = 1,
                    bool padding = true, int pool_height = 1, int pool_width = 1, bool ahead_fc = false,
                    bool save_residual = false, bool inject_residual = false, int residual_channels = 0,
                    bool residual_pool = false, int a_bit = 2, int w_bit = 1);
  // sizes in the reference's terms (param.h:927-945), for this layout (channels padded to in_cpad)
  long long input_bit_words() const { return (long long)a_bit * batch * input_height * input_width * (in_cpad / 32); }
  long long filter_bit_words() const {
    return (long long)w_bit * output_channels * filter_height * filter_width * (in_cpad / 32);
  }
  long long output_bit_words() const {
    return (long long)a_bit * batch * output_height * output_width * (out_cpad / 32);
  }
  long long residual_words() const { return (long long)batch * conv_height * conv_width * output_channels; }
  // Shortcut taken from the packed codes of an earlier layer, added at an integer scale before the
  // thresholds (this build's form of a residual connection).  Call before initialize().
  void set_packed_shortcut(const uint32_t *planes, int scale, int layer_index) {
    packed_shortcut_gpu = planes;
    residual_scale = scale;
    shortcut_layer = layer_index;
  }
  // input_residual_pitch: int32 values per pixel of the injected map = channels of the layer that saved
  // it (0: residual_channels, capped at output_channels); residual_layer: index of that layer (reported
  // by describe()).
  int initialize(Rng &rng, const uint32_t *prev_layer_gpu, const int32_t *input_residual_gpu = nullptr,
                 int path = APNN_PATH_AUTO, int input_residual_pitch = 0, int residual_layer = -1);
  void set_input_gpu(const uint32_t *p) { input_gpu = p; }
  void set_input_residual_gpu(const int32_t *p) { input_residual_gpu = p; }
  int forward(hipStream_t stream) override;
  void describe(apnn_layer_desc *d) const override;
  const uint32_t *get_output_gpu() const override { return output_gpu.as<uint32_t>(); }
  int32_t *get_output_residual_gpu() const { return output_residual_gpu.as<int32_t>(); }
  std::vector<uint32_t> download_output() const;

  std::string name;
  int input_height, input_width, filter_height, filter_width, input_channels, output_channels, batch;
  int stride, pad, pool, a_bit, w_bit;
  bool ahead_fc, save_residual, inject_residual, residual_pool;
  int residual_channels;
  int status = 0;  // APNN_EUNSUPPORTED when a constructor argument cannot be honoured
  int conv_height, conv_width, output_height, output_width, in_cpad, out_cpad;
  int residual_scale = 0, path = APNN_PATH_AUTO, shortcut_layer = -1, residual_layer = -1, residual_pitch = 0;
  int residual_used = 0;  // channels that receive the injected residual
  const uint32_t *input_gpu = nullptr, *packed_shortcut_gpu = nullptr;
  const int32_t *input_residual_gpu = nullptr;
  DeviceBuffer filter_gpu, bn_gpu, output_gpu, output_residual_gpu, residual_tmp_gpu;
};

// Low-bit fully connected layer (param.h:219-385), constructor arguments as the reference's
// (param.h:222-223): input_height = rows (the batch), input_width = stored features per row -- the
// previous layer's whole packed output per image (H*W*padded channels, a multiple of 32), so a
// batch-major feature map is consumed as it lies in memory.
class Fc128LayerParam : public Layer {
 public:
  Fc128LayerParam(const char *name, int input_height, int input_width, int weight_width, int a_bit = 2,
                  int w_bit = 1);
  int initialize(Rng &rng, const uint32_t *prev_layer_gpu, int path = APNN_PATH_AUTO);
  int forward(hipStream_t stream) override;
  void describe(apnn_layer_desc *d) const override;
  const uint32_t *get_output_gpu() const override { return output_gpu.as<uint32_t>(); }

  std::string name;
  int input_height, input_width, weight_width, a_bit, w_bit;
  int status = 0;
  int out_cpad, path = APNN_PATH_AUTO;
  const uint32_t *input_gpu = nullptr;
  DeviceBuffer weight_gpu, bn_gpu, output_gpu;
};

// Output layer (param.h:388-531), constructor arguments as the reference's (param.h:391-392) followed
// by this build's global-pooling extension: the packed codes of the previous layer are unpacked
// (input_positions > 1: summed over that many consecutive rows per image and shifted right by
// global_pool_shift -- global average pooling up to a power of two) to int8 and multiplied by an int8
// weight matrix; logits = acc * bn_scale + bn_bias in float (kernel.cuh:437-441).  The classifier's
// weights are int8 whatever w_bit says (the reference's are 1-bit): w_bit is kept for the signature only
// and reported as 8 by describe().
class Out128LayerParam : public Layer {
 public:
  Out128LayerParam(const char *name, int input_height, int input_width, int weight_width, int a_bit = 2,
                   int w_bit = 1, int input_positions = 1, int global_pool_shift = -1);
  int initialize(Rng &rng, const uint32_t *prev_layer_gpu, float *logits_gpu);
  void set_output_gpu(float *logits) { output_gpu = logits; }
  int forward(hipStream_t stream) override;
  void describe(apnn_layer_desc *d) const override;

  std::string name;
  int batch, input_positions, input_channels, weight_width, global_pool_shift, a_bit, in_cpad;
  const uint32_t *input_gpu = nullptr;
  float *output_gpu = nullptr;
  DeviceBuffer weight_gpu, scale_gpu, bias_gpu, pooled_gpu;
};

// Launch wrappers with the reference's names (kernel.cuh:285-318): unpack the layer object into the
// kernel call.  The reference launches a __global__ wrapper around a __device__ kernel; here the
// wrapper is a host function that enqueues on `stream`.
int Conv_new_global(Conv128LayerParam *p, hipStream_t stream);
// both branches of a residual block's entry (3x3 convolution, 1x1 downsample) in one launch
int Conv_pair_global(Conv128LayerParam *main_branch, Conv128LayerParam *shortcut_branch, hipStream_t stream);
int FC_new_global(Fc128LayerParam *p, hipStream_t stream);
int Output_new_global(Out128LayerParam *p, hipStream_t stream);

// Random codes -> bit-planes on the device with the layout of filter_quantization /
// weight_quantization (kernel.cuh:164-282): values [rows][C] uniform in [0, 2^bits), packed with
// apnn_pack_bits (Bit_compression layout), pad channels zero.
int random_planes_gpu(Rng &rng, DeviceBuffer &planes, int rows, int C, int cpad, int bits);
// Thresholds [C][2^bits-1] around `center` with spread sigma (quartile-like spacing + jitter).
std::vector<int32_t> random_thresholds(Rng &rng, int C, int bits, double center, double sigma);

class Network {
 public:
  ~Network();
  int forward(const uint8_t *images, float *logits, hipStream_t stream);
  int forward_graph(const uint8_t *images, float *logits, hipStream_t stream);
  std::vector<std::unique_ptr<Layer>> layers;
  InConv128LayerParam *first = nullptr;       // int8 stem taking the images, or
  ImageQuantLayerParam *first_quant = nullptr;  // the image quantizer of the reference-style network
  Out128LayerParam *last = nullptr;
  int batch = 0;

 private:
  hipGraphExec_t graph_exec_ = nullptr;
  hipStream_t capture_stream_ = nullptr;
  const uint8_t *graph_images_ = nullptr;
  float *graph_logits_ = nullptr;
};

std::unique_ptr<Network> build_alexnet(int batch, uint64_t seed, int path);
std::unique_ptr<Network> build_resnet18(int batch, uint64_t seed, int path);
std::unique_ptr<Network> build_vgg(int batch, uint64_t seed, int path);
std::unique_ptr<Network> build_resnet18_reference(int batch, uint64_t seed, int path);

}  // namespace apnn_nn
