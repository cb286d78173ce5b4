// Host side of the layer API: buffer ownership, random initialisation, and the forward calls that
// unpack a layer object into libapnn_tc.so entry points.  See layers.h.
#include "layers.h"

#include <algorithm>
#include <cmath>
#include <cstring>

namespace apnn_nn {

// ---- DeviceBuffer --------------------------------------------------------------------------------

hipError_t DeviceBuffer::allocate(size_t bytes) {
  release();
  if (bytes == 0) bytes = 16;
  const hipError_t e = hipMalloc(&ptr_, bytes);
  if (e != hipSuccess) {
    ptr_ = nullptr;
    return e;
  }
  bytes_ = bytes;
  return hipSuccess;
}

hipError_t DeviceBuffer::upload(const void *host, size_t bytes) {
  hipError_t e = allocate(bytes);
  if (e != hipSuccess) return e;
  return hipMemcpy(ptr_, host, bytes, hipMemcpyHostToDevice);
}

void DeviceBuffer::release() {
  if (ptr_ != nullptr) (void)hipFree(ptr_);
  ptr_ = nullptr;
  bytes_ = 0;
}

// ---- initialisation helpers ----------------------------------------------------------------------

int random_planes_gpu(Rng &rng, DeviceBuffer &planes, int rows, int C, int cpad, int bits) {
  std::vector<uint32_t> values((size_t)rows * C);
  for (auto &v : values) v = rng.below(1u << bits);
  DeviceBuffer tmp;
  if (tmp.upload(values.data(), values.size() * sizeof(uint32_t)) != hipSuccess) return 1;
  if (planes.allocate((size_t)bits * rows * (cpad / 32) * sizeof(uint32_t)) != hipSuccess) return 1;
  const int rc = apnn_pack_bits(tmp.as<uint32_t>(), planes.as<uint32_t>(), rows, C, cpad, bits, nullptr);
  if (rc != 0) return rc;
  return (int)hipDeviceSynchronize();
}

std::vector<int32_t> random_thresholds(Rng &rng, int C, int bits, double center, double sigma) {
  const int nt = (1 << bits) - 1;
  std::vector<int32_t> thr((size_t)C * nt);
  for (int c = 0; c < C; ++c) {
    std::vector<int32_t> t(nt);
    const double shift = (rng.uniform() - 0.5) * 0.4 * sigma;
    for (int k = 0; k < nt; ++k) {
      // evenly spread over about +-0.7 sigma: roughly equal code frequencies for a bell-shaped sum
      const double q = nt == 1 ? 0.0 : (2.0 * k / (nt - 1) - 1.0) * 0.7;
      t[k] = (int32_t)std::lround(center + shift + q * sigma + (rng.uniform() - 0.5) * 0.1 * sigma);
    }
    std::sort(t.begin(), t.end());
    for (int k = 0; k < nt; ++k) thr[(size_t)c * nt + k] = t[k];
  }
  return thr;
}

static void copy_name(char (&dst)[16], const std::string &src) {
  std::memset(dst, 0, sizeof(dst));
  std::strncpy(dst, src.c_str(), sizeof(dst) - 1);
}

template <class T>
static std::vector<T> download(const void *dev, size_t count) {
  std::vector<T> host(count);
  (void)hipMemcpy(host.data(), dev, count * sizeof(T), hipMemcpyDeviceToHost);
  return host;
}

// ---- In128LayerParam / ImageQuantLayerParam -----------------------------------------------------------

static void clear_desc(apnn_layer_desc *d, const std::string &name, int kind, int batch) {
  std::memset(d, 0, sizeof(*d));
  copy_name(d->name, name);
  d->kind = kind;
  d->batch = batch;
  d->shortcut_layer = -1;
  d->residual_layer = -1;
  d->global_pool_shift = -1;
}

In128LayerParam::In128LayerParam(const char *name_, int input_height_, int input_width_)
    : name(name_), input_height(input_height_), input_width(input_width_), output_height(input_height_),
      output_width(input_width_), out_cpad(pad_to(input_width_, 32)) {}

int In128LayerParam::initialize(const float *input_gpu_) {
  if (output_gpu.allocate((size_t)output_height * (out_cpad / 32) * 4) != hipSuccess) return 1;
  input_gpu = input_gpu_;
  return 0;
}

int In128LayerParam::forward(hipStream_t stream) {
  return apnn_binarize_pack(input_gpu, output_gpu.as<uint32_t>(), input_height, input_width, out_cpad, stream);
}

void In128LayerParam::describe(apnn_layer_desc *d) const {
  clear_desc(d, name, APNN_LAYER_IMAGE_QUANT, input_height);
  d->in_h = 1, d->in_w = 1, d->in_c = input_width, d->in_cpad = input_width;
  d->out_h = 1, d->out_w = 1, d->out_c = input_width, d->out_cpad = out_cpad;
  d->a_bits = 32, d->out_bits = 1;
  d->input = input_gpu, d->output = output_gpu.get();
}

ImageQuantLayerParam::ImageQuantLayerParam(const char *name_, int batch_, int image_height_, int image_width_,
                                           int image_channel_, int bit_)
    : name(name_), batch(batch_), image_height(image_height_), image_width(image_width_),
      image_channel(image_channel_), bit(bit_), out_cpad(pad_to(image_channel_, 32)) {}

int ImageQuantLayerParam::initialize(const uint8_t *images_gpu) {
  if (output_gpu.allocate((size_t)bit * batch * image_height * image_width * (out_cpad / 32) * 4) != hipSuccess) return 1;
  input_gpu = images_gpu;
  return 0;
}

int ImageQuantLayerParam::forward(hipStream_t stream) {
  return apnn_quantize_pack_u8(input_gpu, output_gpu.as<uint32_t>(), batch * image_height * image_width, image_channel,
                               out_cpad, bit, stream);
}

void ImageQuantLayerParam::describe(apnn_layer_desc *d) const {
  clear_desc(d, name, APNN_LAYER_IMAGE_QUANT, batch);
  d->in_h = image_height, d->in_w = image_width, d->in_c = image_channel, d->in_cpad = image_channel;
  d->out_h = image_height, d->out_w = image_width, d->out_c = image_channel, d->out_cpad = out_cpad;
  d->a_bits = 8, d->out_bits = bit;
  d->input = input_gpu, d->output = output_gpu.get();
}

// ---- InConv128LayerParam ---------------------------------------------------------------------------

InConv128LayerParam::InConv128LayerParam(const char *name_, int input_height_, int input_width_, int filter_height_,
                                         int filter_width_, int input_channels_, int output_channels_, int batch_,
                                         int stride_height, int stride_width, bool padding, int pool_height,
                                         int pool_width, bool save_residual_, int pool_stride_, int pool_pad_,
                                         int a_bit_)
    : name(name_), input_height(input_height_), input_width(input_width_), filter_height(filter_height_),
      filter_width(filter_width_), input_channels(input_channels_), output_channels(output_channels_), batch(batch_),
      stride(stride_height), pad(padding ? (filter_height_ - 1) / 2 : 0), pool(pool_height),
      pool_stride(pool_stride_ > 0 ? pool_stride_ : pool_height), pool_pad(pool_pad_), a_bit(a_bit_),
      save_residual(save_residual_) {
  if (stride_width != stride_height || pool_width != pool_height || pool_height < 1 ||
      (padding && ((filter_height_ | filter_width_) & 1) == 0))
    status = APNN_EUNSUPPORTED;
  conv_height = (input_height + 2 * pad - filter_height) / stride + 1;
  conv_width = (input_width + 2 * pad - filter_width) / stride + 1;
  output_height = (conv_height + 2 * pool_pad - pool) / pool_stride + 1;
  output_width = (conv_width + 2 * pool_pad - pool) / pool_stride + 1;
  out_cpad = pad_to(output_channels, 32);
}

int InConv128LayerParam::initialize(Rng &rng, const uint8_t *images_gpu) {
  if (status != 0) return status;
  const size_t nw = (size_t)output_channels * filter_height * filter_width * input_channels;
  std::vector<int8_t> w(nw);
  for (auto &v : w) v = (int8_t)((int)rng.below(255) - 127);
  if (filter_gpu.upload(w.data(), nw) != hipSuccess) return 1;
  // pixel - 128 is uniform in [-128, 127] (variance 5461), weights uniform in [-127, 127] (5376)
  const double sigma = std::sqrt((double)filter_height * filter_width * input_channels * 5461.0 * 5376.0);
  const std::vector<int32_t> thr = random_thresholds(rng, output_channels, a_bit, 0.0, sigma);
  if (bn_gpu.upload(thr.data(), thr.size() * sizeof(int32_t)) != hipSuccess) return 1;
  const size_t conv_px = (size_t)batch * conv_height * conv_width;
  if (save_residual) {
    // the kernel that also writes the int32 sums produces byte codes; they are pooled and packed after it
    if (codes_gpu.allocate(conv_px * output_channels) != hipSuccess) return 1;
    if (output_residual_gpu.allocate(conv_px * output_channels * sizeof(int32_t)) != hipSuccess) return 1;
  } else if (pool > 1 && codes_gpu.allocate((size_t)a_bit * conv_px * (out_cpad / 32) * 4) != hipSuccess) {
    return 1;  // un-pooled packed codes of the convolution (skipped when there is no pooling stage)
  }
  if (output_gpu.allocate((size_t)a_bit * batch * output_height * output_width * (out_cpad / 32) * 4) != hipSuccess)
    return 1;
  input_gpu = images_gpu;
  return 0;
}

int InConv128LayerParam::forward(hipStream_t stream) {
  if (save_residual) {
    int rc = apnn_conv_i8_bn(reinterpret_cast<const int8_t *>(input_gpu), filter_gpu.as<int8_t>(), bn_gpu.as<int32_t>(),
                             codes_gpu.as<uint8_t>(), output_residual_gpu.as<int32_t>(), batch, input_height,
                             input_width, input_channels, output_channels, filter_height, filter_width, stride, pad,
                             a_bit, 128, stream);
    if (rc != 0) return rc;
    return apnn_pool_pack(codes_gpu.as<uint8_t>(), output_gpu.as<uint32_t>(), batch, conv_height, conv_width,
                          output_channels, out_cpad, a_bit, pool, pool_stride, pool_pad, stream);
  }
  uint32_t *conv_out = pool > 1 ? codes_gpu.as<uint32_t>() : output_gpu.as<uint32_t>();
  int rc = apnn_conv_i8_bn_pack(reinterpret_cast<const int8_t *>(input_gpu), filter_gpu.as<int8_t>(),
                                bn_gpu.as<int32_t>(), conv_out, batch, input_height, input_width, input_channels,
                                output_channels, filter_height, filter_width, stride, pad, a_bit, 128, stream);
  if (rc != 0 || pool <= 1) return rc;
  return apnn_pool_planes(conv_out, output_gpu.as<uint32_t>(), batch, conv_height, conv_width, out_cpad, a_bit, pool,
                          pool_stride, pool_pad, stream);
}

void InConv128LayerParam::describe(apnn_layer_desc *d) const {
  clear_desc(d, name, APNN_LAYER_INCONV_I8, batch);
  d->in_h = input_height, d->in_w = input_width, d->in_c = input_channels, d->in_cpad = input_channels;
  d->out_h = output_height, d->out_w = output_width, d->out_c = output_channels, d->out_cpad = out_cpad;
  d->R = filter_height, d->S = filter_width, d->stride = stride, d->pad = pad;
  d->pool_win = pool > 1 ? pool : 0, d->pool_stride = pool_stride, d->pool_pad = pool_pad;
  d->a_bits = 8, d->w_bits = 8, d->out_bits = a_bit;
  d->save_residual = save_residual ? 1 : 0;
  d->residual_out = output_residual_gpu.get();
  d->input = input_gpu, d->weights = filter_gpu.get(), d->thresholds = bn_gpu.get(), d->output = output_gpu.get();
}

std::vector<uint32_t> InConv128LayerParam::download_output() const {
  return download<uint32_t>(output_gpu.get(), output_gpu.bytes() / 4);
}

// ---- Conv128LayerParam -----------------------------------------------------------------------------

Conv128LayerParam::Conv128LayerParam(const char *name_, int input_height_, int input_width_, int filter_height_,
                                     int filter_width_, int input_channels_, int output_channels_, int batch_,
                                     int stride_height, int stride_width, bool padding, int pool_height,
                                     int pool_width, bool ahead_fc_, bool save_residual_, bool inject_residual_,
                                     int residual_channels_, bool residual_pool_, int a_bit_, int w_bit_)
    : name(name_), input_height(input_height_), input_width(input_width_), filter_height(filter_height_),
      filter_width(filter_width_), input_channels(input_channels_), output_channels(output_channels_), batch(batch_),
      stride(stride_height), pad(padding ? (filter_height_ - 1) / 2 : 0), pool(pool_height), a_bit(a_bit_),
      w_bit(w_bit_), ahead_fc(ahead_fc_), save_residual(save_residual_), inject_residual(inject_residual_),
      residual_pool(residual_pool_), residual_channels(residual_channels_) {
  // what the kernels behind this class cannot do is refused by initialize(), not dropped: anisotropic
  // stride / pooling, pooling windows other than 2x2, "same" padding of an even filter, and the int32
  // residual path together with pooling (the epilogue pools before it could add or save)
  if (stride_width != stride_height || pool_width != pool_height || (pool_height != 1 && pool_height != 2) ||
      (padding && ((filter_height_ | filter_width_) & 1) == 0) || filter_height_ != filter_width_ ||
      ((save_residual_ || inject_residual_) && pool_height != 1) || (inject_residual_ && residual_channels_ <= 0))
    status = APNN_EUNSUPPORTED;
  // output-size rule of param.h:915-924 for symmetric padding: ceil(in/stride) when padded
  conv_height = (input_height + 2 * pad - filter_height) / stride + 1;
  conv_width = (input_width + 2 * pad - filter_width) / stride + 1;
  output_height = conv_height / pool;
  output_width = conv_width / pool;
  in_cpad = pad_to(input_channels, 32);
  out_cpad = pad_to(output_channels, 32);
}

int Conv128LayerParam::initialize(Rng &rng, const uint32_t *prev_layer_gpu, const int32_t *input_residual_gpu_,
                                  int path_, int input_residual_pitch, int residual_layer_) {
  if (status != 0) return status;
  if (inject_residual && packed_shortcut_gpu != nullptr) return APNN_EUNSUPPORTED;  // one shortcut form per layer
  int rc = random_planes_gpu(rng, filter_gpu, output_channels * filter_height * filter_width, input_channels, in_cpad,
                             w_bit);
  if (rc != 0) return rc;
  const double amax = (double)((1 << a_bit) - 1), wmax = (double)((1 << w_bit) - 1);
  // codes uniform in 0..amax: E[x^2] = amax(2 amax + 1)/6; symmetric weights uniform in {-wmax..wmax step 2}
  const double ex2 = amax * (2 * amax + 1) / 6.0, ew2 = (wmax * wmax + 2 * wmax) / 3.0;
  const double sigma = std::sqrt((double)filter_height * filter_width * input_channels * ex2 * ew2);
  const double center = packed_shortcut_gpu != nullptr ? residual_scale * amax / 2.0 : 0.0;
  const std::vector<int32_t> thr = random_thresholds(rng, output_channels, a_bit, center, sigma);
  if (bn_gpu.upload(thr.data(), thr.size() * sizeof(int32_t)) != hipSuccess) return 1;
  if (output_gpu.allocate((size_t)output_bit_words() * 4) != hipSuccess) return 1;
  if (save_residual && output_residual_gpu.allocate((size_t)residual_words() * sizeof(int32_t)) != hipSuccess) return 1;
  input_gpu = prev_layer_gpu;
  if (inject_residual) {
    if (input_residual_gpu_ == nullptr) return APNN_ENULL;
    input_residual_gpu = input_residual_gpu_;
    residual_layer = residual_layer_;
    // channels that receive the residual: below residual_channels, and no more than the map holds (the
    // reference reads zero padding beyond the source layer's channels, kernel.cuh:779-817)
    residual_pitch = input_residual_pitch > 0 ? input_residual_pitch : std::min(residual_channels, output_channels);
    residual_used = std::min(std::min(residual_channels, output_channels), residual_pitch);
    // a map that is not already [rows][output_channels] is brought to that shape before the convolution
    if ((residual_pool || residual_used != output_channels || residual_pitch != output_channels) &&
        residual_tmp_gpu.allocate((size_t)residual_words() * sizeof(int32_t)) != hipSuccess)
      return 1;
  }
  path = path_;
  return 0;
}

static apnn_conv_desc conv_desc_of(const Conv128LayerParam *p) {
  apnn_conv_desc d{};
  d.W = p->filter_gpu.get();
  d.X = p->input_gpu;
  d.O = p->output_gpu.get();
  d.batch = p->batch;
  d.H = p->input_height;
  d.Wd = p->input_width;
  d.cin_pad = p->in_cpad;
  d.COUT = p->output_channels;
  d.R = p->filter_height;
  d.S = p->filter_width;
  d.stride = p->stride;
  d.pad = p->pad;
  d.halo = 0;
  d.wb = p->w_bit;
  d.xb = p->a_bit;
  d.weight_mode = APNN_WEIGHT_SYMMETRIC;
  d.epi.mode = APNN_EPI_BN;
  d.epi.out_bits = p->a_bit;
  d.epi.pool = p->pool == 2 ? APNN_POOL_MAX2X2 : APNN_POOL_NONE;
  d.epi.thresholds = p->bn_gpu.as<int32_t>();
  d.epi.residual_planes = p->packed_shortcut_gpu;
  d.epi.residual_bits = p->a_bit;
  d.epi.residual_scale = p->residual_scale;
  if (p->inject_residual)
    d.epi.residual = p->residual_tmp_gpu.get() != nullptr ? p->residual_tmp_gpu.as<int32_t>() : p->input_residual_gpu;
  if (p->save_residual) d.epi.save_acc = p->output_residual_gpu.as<int32_t>();
  d.path = p->path;
  return d;
}

int Conv_new_global(Conv128LayerParam *p, hipStream_t stream) {
  if (p->inject_residual && p->residual_tmp_gpu.get() != nullptr) {
    const int rc = apnn_residual_prepare(p->input_residual_gpu, p->residual_tmp_gpu.as<int32_t>(), p->batch,
                                         p->conv_height, p->conv_width, p->residual_pitch, p->residual_used,
                                         p->output_channels,
                                         p->residual_pool ? 1 : 0, stream);
    if (rc != 0) return rc;
  }
  const apnn_conv_desc d = conv_desc_of(p);
  return apnn_conv(&d, stream);
}

int Conv_pair_global(Conv128LayerParam *main_branch, Conv128LayerParam *shortcut_branch, hipStream_t stream) {
  const apnn_conv_desc a = conv_desc_of(main_branch), b = conv_desc_of(shortcut_branch);
  return apnn_conv_pair(&a, &b, stream);
}

int Conv128LayerParam::forward(hipStream_t stream) { return Conv_new_global(this, stream); }

void Conv128LayerParam::describe(apnn_layer_desc *d) const {
  clear_desc(d, name, APNN_LAYER_CONV, batch);
  d->in_h = input_height, d->in_w = input_width, d->in_c = input_channels, d->in_cpad = in_cpad;
  d->out_h = output_height, d->out_w = output_width, d->out_c = output_channels, d->out_cpad = out_cpad;
  d->R = filter_height, d->S = filter_width, d->stride = stride, d->pad = pad;
  d->pool_win = pool == 2 ? 2 : 0, d->pool_stride = pool == 2 ? 2 : 0, d->pool_pad = 0;
  d->a_bits = a_bit, d->w_bits = w_bit, d->out_bits = a_bit;
  d->shortcut_layer = shortcut_layer;
  d->shortcut_scale = residual_scale;
  if (inject_residual) {
    d->residual_layer = residual_layer;
    d->residual_channels = residual_used;
    d->residual_pitch = residual_pitch;
    d->residual_pool = residual_pool ? 1 : 0;
  }
  d->save_residual = save_residual ? 1 : 0;
  d->residual_out = output_residual_gpu.get();
  d->input = input_gpu, d->weights = filter_gpu.get(), d->thresholds = bn_gpu.get(), d->output = output_gpu.get();
}

std::vector<uint32_t> Conv128LayerParam::download_output() const {
  return download<uint32_t>(output_gpu.get(), output_gpu.bytes() / 4);
}

// ---- Fc128LayerParam -------------------------------------------------------------------------------

Fc128LayerParam::Fc128LayerParam(const char *name_, int input_height_, int input_width_, int weight_width_, int a_bit_,
                                 int w_bit_)
    : name(name_), input_height(input_height_), input_width(input_width_), weight_width(weight_width_), a_bit(a_bit_),
      w_bit(w_bit_) {
  if (input_width % 32 != 0) status = APNN_EUNSUPPORTED;  // rows are whole packed words
  out_cpad = pad_to(weight_width, 32);
}

int Fc128LayerParam::initialize(Rng &rng, const uint32_t *prev_layer_gpu, int path_) {
  if (status != 0) return status;
  int rc = random_planes_gpu(rng, weight_gpu, weight_width, input_width, input_width, w_bit);
  if (rc != 0) return rc;
  const double amax = (double)((1 << a_bit) - 1), wmax = (double)((1 << w_bit) - 1);
  const double ex2 = amax * (2 * amax + 1) / 6.0, ew2 = (wmax * wmax + 2 * wmax) / 3.0;
  const double sigma = std::sqrt((double)input_width * ex2 * ew2);
  const std::vector<int32_t> thr = random_thresholds(rng, weight_width, a_bit, 0.0, sigma);
  if (bn_gpu.upload(thr.data(), thr.size() * sizeof(int32_t)) != hipSuccess) return 1;
  if (output_gpu.allocate((size_t)a_bit * input_height * (out_cpad / 32) * 4) != hipSuccess) return 1;
  input_gpu = prev_layer_gpu;
  path = path_;
  return 0;
}

int FC_new_global(Fc128LayerParam *p, hipStream_t stream) {
  apnn_conv_desc d{};
  d.W = p->weight_gpu.get();
  d.X = p->input_gpu;
  d.O = p->output_gpu.get();
  d.batch = p->input_height;
  d.H = 1;
  d.Wd = 1;
  d.cin_pad = p->input_width;
  d.COUT = p->weight_width;
  d.R = 1;
  d.S = 1;
  d.stride = 1;
  d.pad = 0;
  d.halo = 0;
  d.wb = p->w_bit;
  d.xb = p->a_bit;
  d.weight_mode = APNN_WEIGHT_SYMMETRIC;
  d.epi.mode = APNN_EPI_BN;
  d.epi.out_bits = p->a_bit;
  d.epi.thresholds = p->bn_gpu.as<int32_t>();
  d.path = p->path;
  return apnn_conv(&d, stream);
}

int Fc128LayerParam::forward(hipStream_t stream) { return FC_new_global(this, stream); }

void Fc128LayerParam::describe(apnn_layer_desc *d) const {
  clear_desc(d, name, APNN_LAYER_FC, input_height);
  d->in_h = 1, d->in_w = 1, d->in_c = input_width, d->in_cpad = input_width;
  d->out_h = 1, d->out_w = 1, d->out_c = weight_width, d->out_cpad = out_cpad;
  d->R = 1, d->S = 1, d->stride = 1, d->pad = 0;
  d->a_bits = a_bit, d->w_bits = w_bit, d->out_bits = a_bit;
  d->input = input_gpu, d->weights = weight_gpu.get(), d->thresholds = bn_gpu.get(), d->output = output_gpu.get();
}

// ---- Out128LayerParam ------------------------------------------------------------------------------

Out128LayerParam::Out128LayerParam(const char *name_, int input_height_, int input_width_, int weight_width_,
                                   int a_bit_, int /*w_bit: the classifier's weights are int8*/, int input_positions_,
                                   int global_pool_shift_)
    : name(name_), batch(input_height_), input_positions(input_positions_), input_channels(input_width_),
      weight_width(weight_width_), global_pool_shift(global_pool_shift_), a_bit(a_bit_) {
  in_cpad = pad_to(input_channels, 32);
}

int Out128LayerParam::initialize(Rng &rng, const uint32_t *prev_layer_gpu, float *logits_gpu) {
  const size_t nw = (size_t)weight_width * input_channels;
  std::vector<int8_t> w(nw);
  for (auto &v : w) v = (int8_t)((int)rng.below(255) - 127);
  if (weight_gpu.upload(w.data(), nw) != hipSuccess) return 1;
  std::vector<float> scale(weight_width), bias(weight_width);
  for (int n = 0; n < weight_width; ++n) {
    scale[n] = (float)(0.5 + rng.uniform()) * 1e-4f;
    bias[n] = (float)(rng.uniform() - 0.5);
  }
  if (scale_gpu.upload(scale.data(), scale.size() * sizeof(float)) != hipSuccess) return 1;
  if (bias_gpu.upload(bias.data(), bias.size() * sizeof(float)) != hipSuccess) return 1;
  if (pooled_gpu.allocate((size_t)batch * input_channels) != hipSuccess) return 1;
  input_gpu = prev_layer_gpu;
  output_gpu = logits_gpu;
  return 0;
}

int Output_new_global(Out128LayerParam *p, hipStream_t stream) {
  const bool pool = p->global_pool_shift >= 0;
  int rc = apnn_unpack_sum(p->input_gpu, p->pooled_gpu.as<int8_t>(), p->batch, pool ? p->input_positions : 1,
                           p->input_channels, p->in_cpad, p->a_bit, pool ? p->global_pool_shift : 0, stream);
  if (rc != 0) return rc;
  return apnn_fc_i8(p->pooled_gpu.as<int8_t>(), p->weight_gpu.as<int8_t>(), p->scale_gpu.as<float>(),
                    p->bias_gpu.as<float>(), p->output_gpu, nullptr, p->batch, p->weight_width, p->input_channels,
                    stream);
}

int Out128LayerParam::forward(hipStream_t stream) { return Output_new_global(this, stream); }

void Out128LayerParam::describe(apnn_layer_desc *d) const {
  clear_desc(d, name, APNN_LAYER_OUT_I8, batch);
  d->in_h = input_positions, d->in_w = 1, d->in_c = input_channels, d->in_cpad = in_cpad;
  d->out_h = 1, d->out_w = 1, d->out_c = weight_width, d->out_cpad = weight_width;
  d->R = 1, d->S = 1, d->stride = 1;
  d->a_bits = a_bit, d->w_bits = 8, d->out_bits = 32;
  d->global_pool_shift = global_pool_shift;
  d->input = input_gpu, d->weights = weight_gpu.get(), d->scale = scale_gpu.get(), d->bias = bias_gpu.get();
  d->output = output_gpu;
}

// ---- Network ---------------------------------------------------------------------------------------

Network::~Network() {
  if (graph_exec_ != nullptr) (void)hipGraphExecDestroy(graph_exec_);
  if (capture_stream_ != nullptr) (void)hipStreamDestroy(capture_stream_);
}

int Network::forward(const uint8_t *images, float *logits, hipStream_t stream) {
  if (images == nullptr || logits == nullptr) return APNN_ENULL;
  if (first != nullptr) first->set_input_gpu(images);
  if (first_quant != nullptr) first_quant->set_input_gpu(images);
  last->set_output_gpu(logits);
  for (size_t i = 0; i < layers.size(); ++i) {
    // a residual block's first convolution and the downsample convolution listed right after it read
    // the same input: one paired launch
    if (i + 1 < layers.size() && layers[i + 1]->pairs_with_previous) {
      auto *a = static_cast<Conv128LayerParam *>(layers[i].get());
      auto *b = static_cast<Conv128LayerParam *>(layers[i + 1].get());
      const int rc = Conv_pair_global(a, b, stream);
      if (rc != 0) return rc;
      ++i;
      continue;
    }
    const int rc = layers[i]->forward(stream);
    if (rc != 0) return rc;
  }
  return 0;
}

int Network::forward_graph(const uint8_t *images, float *logits, hipStream_t stream) {
  if (images == nullptr || logits == nullptr) return APNN_ENULL;
  if (graph_exec_ == nullptr || images != graph_images_ || logits != graph_logits_) {
    if (graph_exec_ != nullptr) {
      (void)hipGraphExecDestroy(graph_exec_);
      graph_exec_ = nullptr;
    }
    // one eager pass first: one-time kernel attribute changes must not happen inside a capture
    int rc = forward(images, logits, stream);
    if (rc != 0) return rc;
    hipError_t e = hipStreamSynchronize(stream);
    if (e != hipSuccess) return (int)e;
    if (capture_stream_ == nullptr && (e = hipStreamCreate(&capture_stream_)) != hipSuccess) return (int)e;
    if ((e = hipStreamBeginCapture(capture_stream_, hipStreamCaptureModeThreadLocal)) != hipSuccess) return (int)e;
    rc = forward(images, logits, capture_stream_);
    hipGraph_t graph = nullptr;
    e = hipStreamEndCapture(capture_stream_, &graph);
    if (rc != 0) return rc;
    if (e != hipSuccess) return (int)e;
    e = hipGraphInstantiate(&graph_exec_, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) {
      graph_exec_ = nullptr;
      return (int)e;
    }
    graph_images_ = images;
    graph_logits_ = logits;
  }
  return (int)hipGraphLaunch(graph_exec_, stream);
}

}  // namespace apnn_nn
