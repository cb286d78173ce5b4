/*
 * apnn_nn.h -- C view of the network layer (libapnn_nn.so), the counterpart of the reference's
 * APNN-TC-nn demo drivers (APNN-TC-nn/src/alexnet.cu, resnet18.cu) and layer classes
 * (APNN-TC-nn/src/param.h).  The C++ classes themselves (Conv128LayerParam, Fc128LayerParam,
 * Out128LayerParam, InConv128LayerParam and the *_new_global wrappers) are declared in
 * apnn-tc_amd/nn/layers.h; this header is what a non-C++ host (tests, benchmark) binds.
 *
 * A network owns its device buffers (weights, thresholds, activations); forward() only enqueues
 * kernels on the given stream: no allocation, no host synchronisation between layers.
 */
#ifndef APNN_NN_H
#define APNN_NN_H

#include <stdint.h>

#include "apnn_tc.h"

#ifdef __cplusplus
extern "C" {
#endif

enum { APNN_NET_ALEXNET = 0,   /* topology of APNN-TC-nn/src/alexnet.cu:42-81, int8 first conv / classifier */
       APNN_NET_RESNET18 = 1,  /* standard ResNet18 (3x3 basic blocks, strided 1x1 downsample convs)        */
       APNN_NET_VGG = 2,       /* topology of APNN-TC-nn/src/vgg.cu:49-127 (ten 3x3 convs, 96..512 channels,
                                  first one stride 2; 2x2 pools after convs 1, 4, 7, 10; two 4096 FCs)       */
       APNN_NET_RESNET18_REFERENCE = 3 }; /* the reference's own ResNet18 demo, layer for layer with its
                                  constructor arguments (APNN-TC-nn/src/resnet18.cu:40-142): quantized image,
                                  7x7 stride-4 low-bit stem, basic blocks whose shortcut is the saved int32 sum
                                  of an earlier layer (max-pooled 2x2 and added to the first residual_channels
                                  channels where the shape changes; no 1x1 convolutions), FC 25088->512, 1000
                                  outputs */

enum { APNN_LAYER_INCONV_I8 = 0, /* int8 conv + thresholds (+ max-pool) + pack                               */
       APNN_LAYER_CONV = 1,      /* low-bit conv, fused threshold / pool / shortcut epilogue                  */
       APNN_LAYER_FC = 2,        /* low-bit fully connected (a conv whose filter covers its whole input)      */
       APNN_LAYER_OUT_I8 = 3,    /* (global pool +) int8 classifier, float logits                             */
       APNN_LAYER_IMAGE_QUANT = 4 }; /* uint8 image -> bit-planes (code = pixel >> (8 - out_bits))            */

typedef struct apnn_layer_desc {
  char name[16];
  int kind;
  int batch;
  int in_h, in_w, in_c, in_cpad;       /* input feature map (cpad = stored channels) */
  int out_h, out_w, out_c, out_cpad;   /* output after pooling */
  int R, S, stride, pad;
  int pool_win, pool_stride, pool_pad; /* max-pool applied to the quantized codes (0 = none) */
  int a_bits, w_bits, out_bits;
  int shortcut_layer;                  /* index of the layer whose packed output is the shortcut, -1 none */
  int shortcut_scale;
  int global_pool_shift;               /* OUT_I8: pooled = min(127, sum_of_codes >> shift); -1: no pooling */
  int residual_layer;                  /* index of the layer whose saved int32 sums are injected, -1 none   */
  int residual_channels;               /* the injected map is added to channels below this                  */
  int residual_pitch;                  /* int32 values per pixel of the injected map                        */
  int residual_pool;                   /* 1: the injected map is twice the size and max-pooled 2x2          */
  int save_residual;                   /* 1: residual_out receives the int32 value the thresholds see       */
  const void *input;                   /* device pointers, valid for the lifetime of the network */
  const void *weights;                 /* CONV/FC: packed planes [w][cout][R][S][in_cpad/32]; I8: [cout][R][S][in_c] */
  const void *thresholds;              /* [out_c][2^out_bits-1] int32 */
  const void *scale, *bias;            /* OUT_I8: float [out_c] */
  const void *output;                  /* packed planes [out_bits][batch*out_h*out_w][out_cpad/32]; OUT_I8: float */
  const void *residual_out;            /* save_residual: int32 [batch*conv_h*conv_w][out_c] (before pooling)  */
} apnn_layer_desc;

typedef struct apnn_net apnn_net;

/* Builds the network with random-init weights / thresholds from `seed`.  path: APNN_PATH_* for the
 * low-bit layers.  Returns NULL on failure. */
apnn_net *apnn_net_create(int kind, int batch, unsigned long long seed, int path);
void apnn_net_destroy(apnn_net *net);

/* images: device, [batch][224][224][3] uint8; logits: device, [batch][1000] float. */
int apnn_net_forward(apnn_net *net, const uint8_t *images, float *logits, apnn_stream_t s);

/* Records forward() into a HIP graph once (on an internal capture stream) and replays it with a
 * single launch per call: removes the per-kernel launch gaps of a 20-layer network. */
int apnn_net_forward_graph(apnn_net *net, const uint8_t *images, float *logits, apnn_stream_t s);

int apnn_net_layer_count(const apnn_net *net);
int apnn_net_layer(const apnn_net *net, int index, apnn_layer_desc *out);

/* Timing loop of the demo drivers (the reference wraps its layer launches in clock() calls,
 * APNN-TC-nn/src/resnet18.cu:270-323): `warmup` untimed forwards, then `iters` back-to-back forwards
 * with no host synchronisation in between; event_ms = HIP-event time, wall_ms = host wall clock, both
 * for all `iters` forwards.  use_graph != 0 replays the captured HIP graph. */
int apnn_net_bench(apnn_net *net, const uint8_t *images, float *logits, int warmup, int iters, int use_graph,
                   apnn_stream_t s, float *event_ms, double *wall_ms);

/* Blocking device-to-host copy for buffers owned by a network. */
int apnn_nn_download(void *host_dst, const void *dev_src, unsigned long long bytes);

#ifdef __cplusplus
}
#endif
#endif
