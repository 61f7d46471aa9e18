/* C entry points onto the C++ operator layer, for callers without a C++ compiler at hand (ctypes, other
 * FFIs) and for the stand-alone bench.  Not part of the reference interface: it stands where MATLAB's
 * mexFunction call mechanism stands in the reference. */
#ifndef MCN_AMD_HARNESS_CAPI_H
#define MCN_AMD_HARNESS_CAPI_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VLH_API __attribute__((visibility("default")))

/* one argument / one result of a front-end call */
typedef struct vlh_arg {
  int kind;        /* 0 = numeric array, 1 = string */
  void* data;      /* array memory (device or host) */
  int device;      /* 0 = host (VLDT_CPU), 1 = HIP device (VLDT_GPU) */
  int dtype;       /* 1 = float, 2 = double (vl::DataType) */
  int ndims;
  size_t dims[8];
  const char* text; /* kind == 1 */
} vlh_arg;

typedef void* (*vlh_alloc_fn)(void* user, int device, size_t bytes);

/* function: "vl_nnconv" | "vl_nnconvt" | "vl_nnbnorm" | "vl_nnpool".  `out` must have room for 4 entries.  Returns a
   vl::ErrorCode; vlh_last_message() has the text. */
VLH_API int vlh_call(const char* function, int nout, vlh_arg* out, int nin, const vlh_arg* in, vlh_alloc_fn alloc,
                     void* user, void* stream);
VLH_API const char* vlh_last_message(void);

/* direct calls of the operator classes (device fp32 tensors, MATLAB-shaped H x W x C x N) */
VLH_API int vlh_pooling_backward(void* stream, float* derInput, const float* input, const float* derOutput, int H,
                                 int W, int C, int N, int poolH, int poolW, int strideY, int strideX, int padTop,
                                 int padBottom, int padLeft, int padRight, int method, int overwrite);
VLH_API int vlh_cpu_tensor_is_refused(void);

/* ResNet bottleneck block */
VLH_API void* vlh_bottleneck_create(int H, int W, int C, int M, int N, double epsilon);
/* the general unit: Cout output channels, stride 1 or 2 on the 3x3 layer, adapter != 0: conv1x1 (same stride) +
   bnorm on the shortcut (buffers "fs", "gs", "bs", "dfs", "dgs", "dbs"); same handle functions as above */
VLH_API void* vlh_unit_create(int H, int W, int C, int M, int N, double epsilon, int Cout, int stride, int adapter);
VLH_API void vlh_bottleneck_destroy(void* block);
VLH_API float* vlh_bottleneck_buffer(void* block, const char* name, size_t* count);
VLH_API int vlh_bottleneck_set_stream(void* block, void* stream);
/* fused != 0: batch-norm forward also applies the ReLU / shortcut sum that follows it (same bits, fewer passes) */
VLH_API void vlh_bottleneck_set_fused(void* block, int fused);
/* overlap != 0: backward runs each convolution's filter gradient on a second stream beside its input gradient
   (same bits; the second stream is joined before vlh_bottleneck_backward's work is complete on the block's stream) */
VLH_API int vlh_bottleneck_set_overlap(void* block, int overlap);
/* packed != 0: the convolutions read filter banks packed ahead; vlh_bottleneck_pack refreshes them (one launch) and
   must follow every change of the filters */
/* deferred != 0: one launch sums the reduction splits of all the unit's filter gradients at the end of backward */
VLH_API int vlh_bottleneck_set_deferred(void* block, int deferred);
VLH_API int vlh_bottleneck_set_packed(void* block, int packed);
/* the forward convolutions also sum their output per channel; the batch normalisations take those sums (fused mode) */
VLH_API int vlh_bottleneck_set_epilogue_sums(void* block, int on);
VLH_API int vlh_bottleneck_set_mask_bits(void* block, int on);
VLH_API int vlh_bottleneck_mask_bits_on(void* block);  /* 1 when the shapes allowed it */
VLH_API int vlh_bottleneck_pack(void* block);
VLH_API int vlh_bottleneck_forward(void* block);
VLH_API int vlh_bottleneck_backward(void* block);
/* runs `steps` forward+backward passes; if stage != NULL the launches of that stage are bracketed by HIP
   events and *stage_ms receives their mean duration */
VLH_API int vlh_bottleneck_run(void* block, int steps, const char* stage, float* stage_ms);
VLH_API const char* vlh_bottleneck_message(void* block);

/* ResNet-50 (examples/imagenet/cnn_imagenet_init_resnet.m:52-134 without the loss layers): imageSize x imageSize x 3 x N
   input, `classes` outputs.  Buffers: "input", "prediction", "dprediction", "stem.f|g|b|df|dg|db", "fc.f|b|df|db",
   "unit<i>.<name>" for the i-th bottleneck unit (names as for vlh_bottleneck_buffer). */
VLH_API void* vlh_resnet50_create(int N, double epsilon, int imageSize, int classes);
VLH_API void vlh_resnet50_destroy(void* net);
VLH_API int vlh_resnet50_units(void* net);
VLH_API float* vlh_resnet50_buffer(void* net, const char* name, size_t* count);
VLH_API int vlh_resnet50_set_stream(void* net, void* stream);
VLH_API void vlh_resnet50_set_fused(void* net, int fused);
/* test != 0: batch normalisation uses the moving averages "running.*" (evaluation of a trained network); forward only */
VLH_API void vlh_resnet50_set_test_mode(void* net, int test);
/* He-normal filters, gains 1, biases 0 from a seeded host generator */
/* packed != 0: all convolutions read filter banks packed ahead, refreshed by ONE launch: by vlh_resnet50_pack, and at the
   end of vlh_resnet50_sgd_step and vlh_resnet50_init.  Call vlh_resnet50_pack after writing filters through
   vlh_resnet50_buffer.  Same bits as packing on every call (the default). */
/* deferred != 0: the sums over reduction splits that finish the filter gradients run in ONE launch at the end of
   vlh_resnet50_backward instead of one per layer (same bits) */
VLH_API int vlh_resnet50_set_deferred(void* net, int deferred);
/* on != 0: the units' filter gradients run on a second stream beside the kernels that follow them, joined once at the end
   of vlh_resnet50_backward (same bits) */
VLH_API int vlh_resnet50_set_overlap(void* net, int on);
VLH_API int vlh_resnet50_set_channel_sums(void* net, int on);
VLH_API int vlh_resnet50_set_packed(void* net, int packed);
VLH_API int vlh_resnet50_pack(void* net);
VLH_API int vlh_resnet50_init(void* net, unsigned long long seed);
VLH_API int vlh_resnet50_forward(void* net);
VLH_API int vlh_resnet50_backward(void* net);
/* SGD with momentum and weight decay on all parameters (one worker) and the moving average of the batch moments, as
   examples/cnn_train_dag.m:316-364 with the rates of cnn_imagenet_init_resnet.m:178-195; buffers "momentum.<parameter>"
   and "running.<moments>" hold the solver state */
VLH_API int vlh_resnet50_sgd_step(void* net, double learningRate, double momentum, double weightDecay);
/* the loss layers at the end of the network (cnn_imagenet_init_resnet.m:128-139) on buffers "prediction" and "labels"
   (N class numbers 1..classes as floats, 0 = skip): _loss_derivative writes "dprediction" for vlh_resnet50_backward
   (softmax log-loss normalised by N, times derOutput); _losses returns {that loss, top-1 error, top-5 error} */
VLH_API int vlh_resnet50_loss_derivative(void* net, double derOutput);
VLH_API int vlh_resnet50_losses(void* net, double values[3]);
VLH_API size_t vlh_resnet50_parameters(void* net);
/* records forward (training == 0) or a whole training step (forward, backward, SGD update with these rates) on the
   network's stream -- which must not be the default stream -- into a HIP graph; vlh_resnet50_replay launches it.  The
   recorded work must have run once eagerly before; capture again after changing rates, modes or the stream. */
VLH_API int vlh_resnet50_capture(void* net, int training, double learningRate, double momentum, double weightDecay);
VLH_API int vlh_resnet50_replay(void* net);
/* forward FLOPs of the convolutions for one image */
VLH_API double vlh_resnet50_forward_flops(void* net);
VLH_API const char* vlh_resnet50_message(void* net);

#ifdef __cplusplus
}
#endif
#endif
