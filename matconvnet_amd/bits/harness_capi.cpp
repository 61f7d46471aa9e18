#include "harness_capi.h"

#include <cstring>
#include <string>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "bottleneck.hpp"
#include "resnet.hpp"
#include "frontend.hpp"
#include "hiphelper.hpp"
#include "nnpooling.hpp"

using namespace vl;

namespace {

thread_local std::string g_message;

class CallbackAllocator : public frontend::Allocator {
 public:
  CallbackAllocator(vlh_alloc_fn fn, void* user) : fn(fn), user(user) {}
  void* allocate(DeviceType device, std::size_t bytes) { return fn ? fn(user, (int)device, bytes) : NULL; }

 private:
  vlh_alloc_fn fn;
  void* user;
};

Tensor toTensor(vlh_arg const& a) {
  std::size_t n = a.ndims > 0 ? 1 : 0;
  for (int i = 0; i < a.ndims; ++i) n *= a.dims[i];
  const DataType dt = a.dtype == 2 ? VLDT_Double : (a.dtype == 1 ? VLDT_Float : VLDT_Char);
  return Tensor(TensorShape(a.dims, (std::size_t)a.ndims), dt, a.device ? VLDT_GPU : VLDT_CPU, a.data,
                n * getDataTypeSizeInBytes(dt));
}

void fromTensor(Tensor const& t, vlh_arg* a) {
  a->kind = 0;
  a->data = const_cast<void*>(t.getMemory());
  a->device = t.getDeviceType() == VLDT_GPU ? 1 : 0;
  a->dtype = (int)t.getDataType();
  a->ndims = (int)t.getNumDimensions();
  for (int i = 0; i < 8; ++i) a->dims[i] = i < a->ndims ? t.getDimension(i) : 0;
  a->text = NULL;
}

// one context per front-end function, like the static vl::MexContext of each MEX file
Context& contextOf(int which) {
  static Context contexts[8];
  return contexts[which];
}

struct StageTimer {
  std::string stage;
  hipStream_t stream;
  std::vector<hipEvent_t> begin, end;
  std::size_t used;
};

void stageHook(void* user, char const* stage, int begin) {
  StageTimer* t = (StageTimer*)user;
  if (t->stage != stage) return;
  if (begin) {
    if (t->used == t->begin.size()) {
      hipEvent_t b, e;
      hipEventCreate(&b);
      hipEventCreate(&e);
      t->begin.push_back(b);
      t->end.push_back(e);
    }
    hipEventRecord(t->begin[t->used], t->stream);
  } else {
    hipEventRecord(t->end[t->used], t->stream);
    ++t->used;
  }
}

struct BlockHandle {
  harness::Bottleneck* block;
  void* stream;
};

}  // namespace

extern "C" {

const char* vlh_last_message(void) { return g_message.c_str(); }

int vlh_call(const char* function, int nout, vlh_arg* out, int nin, const vlh_arg* in, vlh_alloc_fn alloc, void* user,
             void* stream) {
  g_message.clear();
  if (!function || !out || (nin > 0 && !in)) {
    g_message = "vlh_call: null argument";
    return VLE_IllegalArgument;
  }
  int which = !std::strcmp(function, "vl_nnconv") ? 0 : !std::strcmp(function, "vl_nnbnorm") ? 1 : !std::strcmp(function, "vl_nnpool") ? 2 : !std::strcmp(function, "vl_nnconvt") ? 3 : !std::strcmp(function, "vl_taccum") ? 4 : !std::strcmp(function, "vl_nnloss") ? 5 : !std::strcmp(function, "vl_nnrelu") ? 6 : !std::strcmp(function, "vl_nnsoftmax") ? 7 : -1;
  if (which < 0) {
    g_message = std::string("vlh_call: unknown function '") + function + "'";
    return VLE_IllegalArgument;
  }
  std::vector<frontend::Arg> args;
  for (int i = 0; i < nin; ++i) {
    if (in[i].kind == 1) args.push_back(frontend::Arg::string(in[i].text ? in[i].text : ""));
    else args.push_back(frontend::Arg::array(toTensor(in[i])));
  }
  Context& context = contextOf(which);
  context.getHipHelper().setStream(stream);
  CallbackAllocator allocator(alloc, user);
  Tensor results[4];
  ErrorCode e;
  frontend::Arg const* a = args.empty() ? NULL : &args[0];
  if (which == 0) e = frontend::vl_nnconv(context, allocator, nout, results, nin, a, g_message);
  else if (which == 1) e = frontend::vl_nnbnorm(context, allocator, nout, results, nin, a, g_message);
  else if (which == 3) e = frontend::vl_nnconvt(context, allocator, nout, results, nin, a, g_message);
  else if (which == 4) e = frontend::vl_taccum(context, allocator, nout, results, nin, a, g_message);
  else if (which == 5) e = frontend::vl_nnloss(context, allocator, nout, results, nin, a, g_message);
  else if (which == 6) e = frontend::vl_nnrelu(context, allocator, nout, results, nin, a, g_message);
  else if (which == 7) e = frontend::vl_nnsoftmax(context, allocator, nout, results, nin, a, g_message);
  else e = frontend::vl_nnpool(context, allocator, nout, results, nin, a, g_message);
  for (int i = 0; i < 4; ++i) fromTensor(results[i], &out[i]);
  return (int)e;
}

int vlh_pooling_backward(void* stream, float* derInput, const float* input, const float* derOutput, int H, int W, int C,
                         int N, int poolH, int poolW, int strideY, int strideX, int padTop, int padBottom, int padLeft,
                         int padRight, int method, int overwrite) {
  Context& context = contextOf(2);
  context.getHipHelper().setStream(stream);
  nn::Pooling op(context, poolH, poolW, strideY, strideX, padTop, padBottom, padLeft, padRight,
                 method == 0 ? nn::Pooling::Max : nn::Pooling::Average);
  const int oh = (H + padTop + padBottom - poolH) / strideY + 1, ow = (W + padLeft + padRight - poolW) / strideX + 1;
  Tensor dx(TensorShape(H, W, C, N), VLDT_Float, VLDT_GPU, derInput, sizeof(float) * (size_t)H * W * C * N);
  Tensor x(TensorShape(H, W, C, N), VLDT_Float, VLDT_GPU, (void*)input, sizeof(float) * (size_t)H * W * C * N);
  Tensor dy(TensorShape(oh, ow, C, N), VLDT_Float, VLDT_GPU, (void*)derOutput, sizeof(float) * (size_t)oh * ow * C * N);
  ErrorCode e = overwrite ? op.backwardOverwrite(dx, x, dy) : op.backward(dx, x, dy);
  g_message = context.getLastErrorMessage();
  return (int)e;
}

// A CPU tensor must be refused loudly (no silent CPU path exists in this library): returns 1 when it is.
int vlh_cpu_tensor_is_refused(void) {
  Context context;
  float host[16] = {0};
  float pooled[4] = {0};
  Tensor x(TensorShape(4, 4, 1, 1), VLDT_Float, VLDT_CPU, host, sizeof(host));
  Tensor y(TensorShape(2, 2, 1, 1), VLDT_Float, VLDT_CPU, pooled, sizeof(pooled));
  nn::Pooling op(context, 2, 2, 2, 2, 0, 0, 0, 0, nn::Pooling::Max);
  ErrorCode e = op.forward(y, x);
  g_message = context.getLastErrorMessage();
  return e == VLE_Unsupported ? 1 : 0;
}

void* vlh_bottleneck_create(int H, int W, int C, int M, int N, double epsilon) {
  BlockHandle* h = new BlockHandle;
  h->block = new harness::Bottleneck(H, W, C, M, N, epsilon);
  h->stream = NULL;
  return h;
}

void* vlh_unit_create(int H, int W, int C, int M, int N, double epsilon, int Cout, int stride, int adapter) {
  BlockHandle* h = new BlockHandle;
  h->block = new harness::Bottleneck(H, W, C, M, N, epsilon, Cout, stride, adapter != 0);
  h->stream = NULL;
  return h;
}

void vlh_bottleneck_destroy(void* block) {
  BlockHandle* h = (BlockHandle*)block;
  if (!h) return;
  delete h->block;
  delete h;
}

float* vlh_bottleneck_buffer(void* block, const char* name, size_t* count) {
  return ((BlockHandle*)block)->block->buffer(name, count);
}

int vlh_bottleneck_set_stream(void* block, void* stream) {
  BlockHandle* h = (BlockHandle*)block;
  h->stream = stream;
  return (int)h->block->setStream(stream);
}

void vlh_bottleneck_set_fused(void* block, int fused) { ((BlockHandle*)block)->block->setFused(fused != 0); }

int vlh_bottleneck_set_overlap(void* block, int overlap) { return (int)((BlockHandle*)block)->block->setOverlap(overlap != 0); }

int vlh_bottleneck_set_deferred(void* block, int deferred) {
  return (int)((BlockHandle*)block)->block->setDeferred(deferred != 0);
}
int vlh_bottleneck_set_epilogue_sums(void* block, int on) { return (int)((BlockHandle*)block)->block->setEpilogueSums(on != 0); }
int vlh_bottleneck_set_mask_bits(void* block, int on) { return (int)((BlockHandle*)block)->block->setMaskBits(on != 0); }
int vlh_bottleneck_mask_bits_on(void* block) { return ((BlockHandle*)block)->block->maskBitsOn() ? 1 : 0; }
int vlh_bottleneck_set_packed(void* block, int packed) { return (int)((BlockHandle*)block)->block->setPacked(packed != 0); }
int vlh_bottleneck_pack(void* block) { return (int)((BlockHandle*)block)->block->pack(); }
int vlh_bottleneck_forward(void* block) { return (int)((BlockHandle*)block)->block->forward(); }
int vlh_bottleneck_backward(void* block) { return (int)((BlockHandle*)block)->block->backward(); }
const char* vlh_bottleneck_message(void* block) { return ((BlockHandle*)block)->block->lastMessage().c_str(); }

int vlh_bottleneck_run(void* block, int steps, const char* stage, float* stage_ms) {
  BlockHandle* h = (BlockHandle*)block;
  StageTimer timer;
  timer.used = 0;
  timer.stream = (hipStream_t)h->stream;
  if (stage) {
    timer.stage = stage;
    h->block->setStageHook(stageHook, &timer);
  }
  int rc = 0;
  for (int i = 0; i < steps && rc == 0; ++i) {
    rc = (int)h->block->pack();  // (packed mode: the filters may have changed since the last step; else nothing)
    if (rc == 0) rc = (int)h->block->forward();
    if (rc == 0) rc = (int)h->block->backward();
  }
  h->block->setStageHook(NULL, NULL);
  if (stage && stage_ms) {
    *stage_ms = 0.f;
    if (timer.used > 0) {
      hipEventSynchronize(timer.end[timer.used - 1]);
      double total = 0.0;
      for (std::size_t i = 0; i < timer.used; ++i) {
        float ms = 0.f;
        hipEventElapsedTime(&ms, timer.begin[i], timer.end[i]);
        total += ms;
      }
      *stage_ms = (float)(total / timer.used);
    }
  }
  for (std::size_t i = 0; i < timer.begin.size(); ++i) {
    hipEventDestroy(timer.begin[i]);
    hipEventDestroy(timer.end[i]);
  }
  return rc;
}

void* vlh_resnet50_create(int N, double epsilon, int imageSize, int classes) {
  return new harness::ResNet50(N, epsilon, imageSize, classes);
}
void vlh_resnet50_destroy(void* net) { delete (harness::ResNet50*)net; }
int vlh_resnet50_units(void* net) { return ((harness::ResNet50*)net)->numUnits(); }
float* vlh_resnet50_buffer(void* net, const char* name, size_t* count) {
  return ((harness::ResNet50*)net)->buffer(name, count);
}
int vlh_resnet50_set_stream(void* net, void* stream) { return (int)((harness::ResNet50*)net)->setStream(stream); }
void vlh_resnet50_set_fused(void* net, int fused) { ((harness::ResNet50*)net)->setFused(fused != 0); }
void vlh_resnet50_set_test_mode(void* net, int test) { ((harness::ResNet50*)net)->setTestMode(test != 0); }
int vlh_resnet50_set_deferred(void* net, int deferred) { return (int)((harness::ResNet50*)net)->setDeferred(deferred != 0); }
int vlh_resnet50_set_overlap(void* net, int on) { return (int)((harness::ResNet50*)net)->setOverlap(on != 0); }
int vlh_resnet50_set_channel_sums(void* net, int on) { return (int)((harness::ResNet50*)net)->setChannelSums(on != 0); }
int vlh_resnet50_set_packed(void* net, int packed) { return (int)((harness::ResNet50*)net)->setPacked(packed != 0); }
int vlh_resnet50_pack(void* net) { return (int)((harness::ResNet50*)net)->pack(); }
int vlh_resnet50_init(void* net, unsigned long long seed) { return (int)((harness::ResNet50*)net)->initParameters(seed); }
int vlh_resnet50_forward(void* net) { return (int)((harness::ResNet50*)net)->forward(); }
int vlh_resnet50_backward(void* net) { return (int)((harness::ResNet50*)net)->backward(); }
int vlh_resnet50_loss_derivative(void* net, double derOutput) { return (int)((harness::ResNet50*)net)->lossDerivative(derOutput); }
int vlh_resnet50_losses(void* net, double values[3]) {
  return (int)((harness::ResNet50*)net)->losses(values, values + 1, values + 2);
}
int vlh_resnet50_sgd_step(void* net, double learningRate, double momentum, double weightDecay) {
  return (int)((harness::ResNet50*)net)->sgdStep(learningRate, momentum, weightDecay);
}
int vlh_resnet50_capture(void* net, int training, double learningRate, double momentum, double weightDecay) {
  return (int)((harness::ResNet50*)net)->capture(training != 0, learningRate, momentum, weightDecay);
}
int vlh_resnet50_replay(void* net) { return (int)((harness::ResNet50*)net)->replay(); }
size_t vlh_resnet50_parameters(void* net) { return ((harness::ResNet50*)net)->numParameters(); }
double vlh_resnet50_forward_flops(void* net) { return ((harness::ResNet50*)net)->convForwardFlopsPerImage(); }
const char* vlh_resnet50_message(void* net) { return ((harness::ResNet50*)net)->lastMessage().c_str(); }

}  // extern "C"
