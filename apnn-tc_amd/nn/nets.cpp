// Network builders (the counterparts of the reference's demo drivers) and the C ABI of
// libapnn_nn.so.  See include/apnn_nn.h.
#include <chrono>
#include <cmath>
#include <new>

#include "layers.h"

namespace apnn_nn {

namespace {

// shortcut codes (0..amax) are brought to roughly half a standard deviation of the main branch
int shortcut_scale_for(int filter_h, int filter_w, int cin, int a_bit) {
  const double amax = (double)((1 << a_bit) - 1);
  const double sigma = std::sqrt((double)filter_h * filter_w * cin * amax * (2 * amax + 1) / 6.0);
  const int s = (int)std::lround(sigma / (2.0 * amax));
  return s < 1 ? 1 : s;
}

template <class L>
L *add(Network &net, L *layer) {
  net.layers.emplace_back(layer);
  return layer;
}

}  // namespace

// AlexNet-style network, layer list of APNN-TC-nn/src/alexnet.cu:42-81: conv 11x11/4 3->64 pool 2,
// conv 5x5 64->192 pool 2, conv 3x3 192->384, 384->256, 256->256 pool 2, FC 12544->4096->4096->1000.
// First conv and classifier in int8, hidden layers w1a2.
std::unique_ptr<Network> build_alexnet(int batch, uint64_t seed, int path) {
  auto net = std::make_unique<Network>();
  net->batch = batch;
  Rng rng(seed);
  auto *c1 = add(*net, new InConv128LayerParam("Conv1", 224, 224, 11, 11, 3, 64, batch, 4, 4, true, 2, 2));
  if (c1->initialize(rng, nullptr)) return nullptr;
  net->first = c1;
  auto *c2 = add(*net, new Conv128LayerParam("Conv2", c1->output_height, c1->output_width, 5, 5, 64, 192, batch, 1, 1,
                                             true, 2, 2));
  if (c2->initialize(rng, c1->get_output_gpu(), nullptr, path)) return nullptr;
  auto *c3 = add(*net, new Conv128LayerParam("Conv3", c2->output_height, c2->output_width, 3, 3, 192, 384, batch));
  if (c3->initialize(rng, c2->get_output_gpu(), nullptr, path)) return nullptr;
  auto *c4 = add(*net, new Conv128LayerParam("Conv4", c3->output_height, c3->output_width, 3, 3, 384, 256, batch));
  if (c4->initialize(rng, c3->get_output_gpu(), nullptr, path)) return nullptr;
  auto *c5 = add(*net, new Conv128LayerParam("Conv5", c4->output_height, c4->output_width, 3, 3, 256, 256, batch, 1, 1,
                                             true, 2, 2));
  if (c5->initialize(rng, c4->get_output_gpu(), nullptr, path)) return nullptr;
  // the FC layer consumes the batch-major feature map as it lies in memory: H*W*C features per image
  auto *f1 = add(*net, new Fc128LayerParam("Fc1", batch, c5->output_height * c5->output_width * c5->out_cpad, 4096));
  if (f1->initialize(rng, c5->get_output_gpu(), path)) return nullptr;
  auto *f2 = add(*net, new Fc128LayerParam("Fc2", batch, 4096, 4096));
  if (f2->initialize(rng, f1->get_output_gpu(), path)) return nullptr;
  auto *out = add(*net, new Out128LayerParam("Fout", batch, 4096, 1000));
  if (out->initialize(rng, f2->get_output_gpu(), nullptr)) return nullptr;
  net->last = out;
  return net;
}

// VGG-variant of APNN-TC-nn/src/vgg.cu:49-127: ten 3x3 convolutions (3->96 stride 2, 96->256, 256->256 x2,
// 256->512, 512->512 x5) with 2x2 pooling after the 1st, 4th, 7th and 10th, FC 4096 x2, 1000 outputs.
// The first convolution runs in int8 on the raw image (the reference quantizes the image to bit-planes
// instead, vgg.cu:46-52).
std::unique_ptr<Network> build_vgg(int batch, uint64_t seed, int path) {
  auto net = std::make_unique<Network>();
  net->batch = batch;
  Rng rng(seed);
  auto *c1 = add(*net, new InConv128LayerParam("Conv1", 224, 224, 3, 3, 3, 96, batch, 2, 2, true, 2, 2));
  if (c1->initialize(rng, nullptr)) return nullptr;
  net->first = c1;
  const int chans[9] = {256, 256, 256, 512, 512, 512, 512, 512, 512};
  const uint32_t *prev = c1->get_output_gpu();
  int h = c1->output_height, w = c1->output_width, cin = 96;
  for (int i = 0; i < 9; ++i) {
    char nm[16];
    snprintf(nm, sizeof nm, "Conv%d", i + 2);
    const int pool = (i == 2 || i == 5 || i == 8) ? 2 : 1;  // Conv4, Conv7, Conv10
    auto *c = add(*net, new Conv128LayerParam(nm, h, w, 3, 3, cin, chans[i], batch, 1, 1, true, pool, pool));
    if (c->initialize(rng, prev, nullptr, path)) return nullptr;
    prev = c->get_output_gpu();
    h = c->output_height;
    w = c->output_width;
    cin = chans[i];
  }
  auto *f1 = add(*net, new Fc128LayerParam("Fc1", batch, h * w * 512, 4096));
  if (f1->initialize(rng, prev, path)) return nullptr;
  auto *f2 = add(*net, new Fc128LayerParam("Fc2", batch, 4096, 4096));
  if (f2->initialize(rng, f1->get_output_gpu(), path)) return nullptr;
  auto *out = add(*net, new Out128LayerParam("Fout", batch, 4096, 1000));
  if (out->initialize(rng, f2->get_output_gpu(), nullptr)) return nullptr;
  net->last = out;
  return net;
}

// Standard ResNet18: 7x7/2 int8 stem + 3x3/2 max-pool, four stages of two basic blocks at
// 64/128/256/512 channels, a strided 1x1 convolution on the shortcut where the shape changes, global
// average pool and an int8 classifier.  (The reference's own demo, APNN-TC-nn/src/resnet18.cu:40-142,
// uses a stride-4 stem and pooled int32 residuals instead of 1x1 convolutions.)
std::unique_ptr<Network> build_resnet18(int batch, uint64_t seed, int path) {
  auto net = std::make_unique<Network>();
  net->batch = batch;
  Rng rng(seed);
  auto *stem = add(*net, new InConv128LayerParam("Conv1", 224, 224, 7, 7, 3, 64, batch, 2, 2, true, 3, 3, false, 2, 1));
  if (stem->initialize(rng, nullptr)) return nullptr;
  net->first = stem;
  const uint32_t *prev = stem->get_output_gpu();
  int prev_index = 0;
  int h = stem->output_height, w = stem->output_width, cin = 64;
  for (int stage = 0; stage < 4; ++stage) {
    const int ch = 64 << stage;
    for (int blk = 0; blk < 2; ++blk) {
      const int stride = (stage > 0 && blk == 0) ? 2 : 1;
      char nm[16];
      snprintf(nm, sizeof nm, "L%dB%dC1", stage + 1, blk + 1);
      auto *c1 = add(*net, new Conv128LayerParam(nm, h, w, 3, 3, cin, ch, batch, stride, stride));
      if (c1->initialize(rng, prev, nullptr, path)) return nullptr;
      const uint32_t *shortcut = prev;
      int shortcut_index = prev_index;
      if (stride != 1 || cin != ch) {
        snprintf(nm, sizeof nm, "L%dB%dDS", stage + 1, blk + 1);
        auto *ds = add(*net, new Conv128LayerParam(nm, h, w, 1, 1, cin, ch, batch, stride, stride, false));
        if (ds->initialize(rng, prev, nullptr, path)) return nullptr;
        ds->pairs_with_previous = true;  // same input as c1: launched together
        shortcut = ds->get_output_gpu();
        shortcut_index = (int)net->layers.size() - 1;
      }
      snprintf(nm, sizeof nm, "L%dB%dC2", stage + 1, blk + 1);
      auto *c2 = add(*net, new Conv128LayerParam(nm, c1->output_height, c1->output_width, 3, 3, ch, ch, batch));
      // the shortcut is the packed output of the block input (or of the downsample convolution)
      c2->set_packed_shortcut(shortcut, shortcut_scale_for(3, 3, ch, 2), shortcut_index);
      if (c2->initialize(rng, c1->get_output_gpu(), nullptr, path)) return nullptr;
      prev = c2->get_output_gpu();
      prev_index = (int)net->layers.size() - 1;
      h = c2->output_height;
      w = c2->output_width;
      cin = ch;
    }
  }
  auto *out = add(*net, new Out128LayerParam("Fc", batch, 512, 1000, 2, 1, h * w, 1));
  if (out->initialize(rng, prev, nullptr)) return nullptr;
  net->last = out;
  return net;
}

// The reference's ResNet18 demo with its own constructor argument lists
// (APNN-TC-nn/src/resnet18.cu:40-142): the image is quantized to bit-planes (images_quantization), the stem
// is a low-bit 7x7 stride-4 convolution that saves its int32 sums, every block's second convolution
// injects the saved sums of the layer two convolutions back (and saves its own), max-pooled 2x2 and
// limited to residual_channels where a stage halves the map; FC 7*7*512 -> 512 and 1000 outputs.
// Differences forced by this build: thresholds are 2-bit (a_bit = 2, the reference's layers compare
// against one float), and the output layer's weights are int8.
std::unique_ptr<Network> build_resnet18_reference(int batch, uint64_t seed, int path) {
  auto net = std::make_unique<Network>();
  net->batch = batch;
  Rng rng(seed);
  auto *img = add(*net, new ImageQuantLayerParam("Image", batch, 224, 224, 3, 2));
  if (img->initialize(nullptr)) return nullptr;
  net->first_quant = img;
  auto index_of_last = [&]() { return (int)net->layers.size() - 1; };

  auto *bconv1 = add(*net, new Conv128LayerParam("Conv1", 224, 224, 7, 7, 3, 64, batch, 4, 4, true, 1, 1, true));
  // resnet18.cu:40-41 passes `true` in the ahead_fc position with the comment "save residual", and
  // l1b1c2 reads bconv1->get_output_residual_gpu(): the stem has to save its sums
  bconv1->save_residual = true;
  if (bconv1->initialize(rng, img->get_output_gpu(), nullptr, path)) return nullptr;

  struct Saved {
    const int32_t *gpu;
    int channels, layer;
  };
  Saved saved{bconv1->get_output_residual_gpu(), 64, index_of_last()};
  Conv128LayerParam *prev = bconv1;
  // (input channels, output channels, stride of the first convolution, residual_channels / residual_pool of
  // the second one), resnet18.cu:44-131
  struct Block {
    int cin, cout, stride, res_channels;
    bool res_pool, ahead_fc, save;
  };
  const Block blocks[8] = {{64, 64, 1, 64, false, false, true},    {64, 64, 1, 128, false, false, true},
                           {64, 128, 2, 128, true, false, true},   {128, 128, 1, 128, false, false, true},
                           {128, 256, 2, 128, true, false, true},  {256, 256, 1, 256, false, false, true},
                           {256, 512, 2, 256, true, false, true},  {512, 512, 1, 512, false, true, false}};
  for (int i = 0; i < 8; ++i) {
    const Block &b = blocks[i];
    char nm[16];
    snprintf(nm, sizeof nm, "L%dB%dC1", i / 2 + 1, i % 2 + 1);
    auto *c1 = add(*net, new Conv128LayerParam(nm, prev->output_height, prev->output_width, 3, 3, b.cin, b.cout, batch,
                                               b.stride, b.stride));
    if (c1->initialize(rng, prev->get_output_gpu(), nullptr, path)) return nullptr;
    snprintf(nm, sizeof nm, "L%dB%dC2", i / 2 + 1, i % 2 + 1);
    auto *c2 = add(*net, new Conv128LayerParam(nm, c1->output_height, c1->output_width, 3, 3, b.cout, b.cout, batch, 1, 1,
                                               true, 1, 1, b.ahead_fc, b.save, true, b.res_channels, b.res_pool));
    if (c2->initialize(rng, c1->get_output_gpu(), saved.gpu, path, saved.channels, saved.layer)) return nullptr;
    saved = Saved{c2->get_output_residual_gpu(), b.cout, index_of_last()};
    prev = c2;
  }
  auto *fc = add(*net, new Fc128LayerParam("Fc1", batch, prev->output_height * prev->output_width * 512, 512));
  if (fc->initialize(rng, prev->get_output_gpu(), path)) return nullptr;
  auto *out = add(*net, new Out128LayerParam("Fout", batch, 512, 1000));
  if (out->initialize(rng, fc->get_output_gpu(), nullptr)) return nullptr;
  net->last = out;
  return net;
}

}  // namespace apnn_nn

struct apnn_net {
  std::unique_ptr<apnn_nn::Network> impl;
};

extern "C" {

apnn_net *apnn_net_create(int kind, int batch, unsigned long long seed, int path) {
  if (batch <= 0) return nullptr;
  std::unique_ptr<apnn_nn::Network> n;
  if (kind == APNN_NET_ALEXNET) {
    n = apnn_nn::build_alexnet(batch, seed, path);
  } else if (kind == APNN_NET_RESNET18) {
    n = apnn_nn::build_resnet18(batch, seed, path);
  } else if (kind == APNN_NET_VGG) {
    n = apnn_nn::build_vgg(batch, seed, path);
  } else if (kind == APNN_NET_RESNET18_REFERENCE) {
    n = apnn_nn::build_resnet18_reference(batch, seed, path);
  }
  if (!n) return nullptr;
  apnn_net *h = new (std::nothrow) apnn_net;
  if (h == nullptr) return nullptr;
  h->impl = std::move(n);
  return h;
}

void apnn_net_destroy(apnn_net *net) { delete net; }

int apnn_net_forward(apnn_net *net, const uint8_t *images, float *logits, apnn_stream_t s) {
  if (net == nullptr) return APNN_ENULL;
  return net->impl->forward(images, logits, static_cast<hipStream_t>(s));
}

int apnn_net_forward_graph(apnn_net *net, const uint8_t *images, float *logits, apnn_stream_t s) {
  if (net == nullptr) return APNN_ENULL;
  return net->impl->forward_graph(images, logits, static_cast<hipStream_t>(s));
}

int apnn_net_layer_count(const apnn_net *net) { return net == nullptr ? 0 : (int)net->impl->layers.size(); }

int apnn_net_layer(const apnn_net *net, int index, apnn_layer_desc *out) {
  if (net == nullptr || out == nullptr) return APNN_ENULL;
  if (index < 0 || index >= (int)net->impl->layers.size()) return APNN_EINVAL;
  net->impl->layers[index]->describe(out);
  return APNN_OK;
}

int apnn_net_bench(apnn_net *net, const uint8_t *images, float *logits, int warmup, int iters, int use_graph,
                   apnn_stream_t s, float *event_ms, double *wall_ms) {
  if (net == nullptr || event_ms == nullptr || wall_ms == nullptr) return APNN_ENULL;
  hipStream_t stream = static_cast<hipStream_t>(s);
  auto step = [&]() {
    return use_graph ? net->impl->forward_graph(images, logits, stream) : net->impl->forward(images, logits, stream);
  };
  int rc = 0;
  for (int i = 0; i < warmup && rc == 0; ++i) rc = step();
  if (rc != 0) return rc;
  hipError_t e = hipStreamSynchronize(stream);
  if (e != hipSuccess) return (int)e;
  hipEvent_t e0, e1;
  if ((e = hipEventCreate(&e0)) != hipSuccess) return (int)e;
  if ((e = hipEventCreate(&e1)) != hipSuccess) return (int)e;
  const auto t0 = std::chrono::steady_clock::now();
  (void)hipEventRecord(e0, stream);
  for (int i = 0; i < iters && rc == 0; ++i) rc = step();
  (void)hipEventRecord(e1, stream);
  e = hipStreamSynchronize(stream);
  const auto t1 = std::chrono::steady_clock::now();
  if (rc == 0 && e != hipSuccess) rc = (int)e;
  if (rc == 0) {
    (void)hipEventElapsedTime(event_ms, e0, e1);
    *wall_ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return rc;
}

int apnn_nn_download(void *host_dst, const void *dev_src, unsigned long long bytes) {
  if (host_dst == nullptr || dev_src == nullptr) return APNN_ENULL;
  hipError_t e = hipDeviceSynchronize();
  if (e != hipSuccess) return (int)e;
  return (int)hipMemcpy(host_dst, dev_src, bytes, hipMemcpyDeviceToHost);
}

}  // extern "C"
