#include "resnet.hpp"

#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdlib>
#include <random>

#include "../../include/mcn_hip.h"
#include "hiphelper.hpp"
#include "nnbnorm.hpp"
#include "nnconv.hpp"
#include "nnpooling.hpp"

namespace vl { namespace harness {

namespace {
double conv_flops(int outH, int outW, int fh, int fw, int cin, int cout) {
  return 2.0 * outH * outW * fh * fw * cin * cout;
}
}  // namespace

#define STEP(stage, call)                                   \
  do {                                                      \
    ErrorCode e_ = (call);                                  \
    if (e_ != VLE_Success) return fail(e_, stage);          \
  } while (0)

#define ABI(stage, call)                                                                    \
  do {                                                                                      \
    int rc_ = (call);                                                                       \
    if (rc_ != 0) {                                                                         \
      context.setError((ErrorCode)rc_, mcn_last_error_message());                           \
      return fail((ErrorCode)rc_, stage);                                                   \
    }                                                                                       \
  } while (0)

ResNet50::ResNet50(int N, double epsilon, int imageSize, int classes)
    : N(N), S(imageSize), classes(classes), epsilon(epsilon), fused(true), testMode(false), error(VLE_Success), flops(0), values(NULL),
      ders(NULL), state(NULL), batchMoments(NULL), runningMoments(NULL), chunkParam(NULL), rates(NULL), chunks(0),
      momentsCount(0), parameterCount(0), deferred(false), partialArena(NULL), sumJobsDevice(NULL), stemPartialBytes(0),
      fcPartialBytes(0), sumJobCount(0), sumBlocks(0), packed(false), packedArena(NULL), packedJobs(NULL), stemBytes(0),
      fcForwardBytes(0), fcBackwardBytes(0), fcBackwardOffset(0), packedJobCount(0), packedBlocks(0), graph(NULL),
      graphExec(NULL), overlap(false), sideStream(NULL), sideDone(NULL) {
  if (S < 32 || S % 32 != 0) {
    error = VLE_IllegalArgument;
    message = "the image size must be a multiple of 32";
    return;
  }
  const int S2 = S / 2, S4 = S / 4;
  make("input", TensorShape(S, S, 3, N));
  make("stem.a", TensorShape(S2, S2, 64, N)); make("stem.n", TensorShape(S2, S2, 64, N)); make("stem.r", TensorShape(S2, S2, 64, N));
  make("stem.p", TensorShape(S4, S4, 64, N));
  make("stem.dp", TensorShape(S4, S4, 64, N)); make("stem.dr", TensorShape(S2, S2, 64, N)); make("stem.dn", TensorShape(S2, S2, 64, N));
  make("stem.da", TensorShape(S2, S2, 64, N));
  flops += conv_flops(S2, S2, 7, 7, 3, 64);

  // sections 2..5 (cnn_imagenet_init_resnet.m:73-118)
  static const int sectionLen[4] = {3, 4, 6, 3};
  int H = S4, C = 64;
  for (int s = 0; s < 4 && error == VLE_Success; ++s) {
    const int depth = 64 << s, out = 256 << s;
    for (int l = 0; l < sectionLen[s] && error == VLE_Success; ++l) {
      const bool first = l == 0;
      const int stride = (first && s >= 1) ? 2 : 1;
      Bottleneck* u = new Bottleneck(H, H, C, depth, N, epsilon, out, stride, first, &context);
      units.push_back(u);
      if (!u->ok()) {
        error = u->lastError();
        message = u->lastMessage();
        break;
      }
      const int Ho = u->outHeight();
      flops += conv_flops(H, H, 1, 1, C, depth) + conv_flops(Ho, Ho, 3, 3, depth, depth) + conv_flops(Ho, Ho, 1, 1, depth, out);
      if (first) flops += conv_flops(Ho, Ho, 1, 1, C, out);
      H = Ho;
      C = out;
    }
  }
  if (error != VLE_Success) return;
  // wiring: a unit's input is the previous unit's output; the derivative it receives is the next unit's dzdx
  units[0]->alias("x", (float*)slot("stem.p").getMemory());
  for (std::size_t i = 1; i < units.size(); ++i) units[i]->alias("x", units[i - 1]->buffer("y"));
  for (std::size_t i = 0; i + 1 < units.size(); ++i) units[i]->alias("dzdy", units[i + 1]->buffer("dzdx"));
  units[0]->alias("dzdx", (float*)slot("stem.dp").getMemory());

  make("avg", TensorShape(1, 1, C, N)); make("davg", TensorShape(1, 1, C, N));
  make("prediction", TensorShape(1, 1, classes, N)); make("dprediction", TensorShape(1, 1, classes, N));
  make("labels", TensorShape(1, 1, 1, N)); make("loss.terms", TensorShape(1, 1, 1, N)); make("loss.values", TensorShape(4, 1, 1, 1));
  flops += conv_flops(1, 1, 1, 1, C, classes);
  if (error == VLE_Success) buildArenas();
  setFused(true);
}

// Lays all parameters out in the arenas (each parameter whole chunks of MCN_SGD_CHUNK floats, zero padded) and points
// the layers' parameter, derivative and moments buffers into them.
ErrorCode ResNet50::buildArenas() {
  const int finalDepth = units.back()->outDepth();
  struct Shape { std::string name; TensorShape shape; double lr; };
  std::vector<Shape> own;
  // the first filter bank learns 100^2 times slower (cnn_imagenet_init_resnet.m:186-188)
  own.push_back({"stem.f", TensorShape(7, 7, 3, 64), 1.0 / (100.0 * 100.0)});
  own.push_back({"stem.g", TensorShape(64, 1, 1, 1), 1.0});
  own.push_back({"stem.b", TensorShape(64, 1, 1, 1), 1.0});
  auto add = [&](std::string const& name, std::string const& der, std::size_t count, double lr) {
    Param p;
    p.name = name; p.der = der; p.count = count; p.learningRate = lr; p.weightDecay = 1.0;
    p.offset = chunks * MCN_SGD_CHUNK;
    chunks += (count + MCN_SGD_CHUNK - 1) / MCN_SGD_CHUNK;
    parameterCount += count;
    params.push_back(p);
  };
  auto addMoments = [&](std::string const& name, std::size_t count) {
    Moments m;
    m.name = name; m.count = count; m.offset = momentsCount;
    momentsCount += count;
    moments.push_back(m);
  };
  for (std::size_t i = 0; i < own.size(); ++i)
    add(own[i].name, "stem.d" + own[i].name.substr(5), own[i].shape.getNumElements(), own[i].lr);
  addMoments("stem.m", 128);
  for (std::size_t u = 0; u < units.size(); ++u) {
    const std::string prefix = "unit" + std::to_string(u) + ".";
    for (char const* layer : {"1", "2", "3", "s"}) {
      std::size_t n = 0;
      if (!units[u]->buffer(std::string("f") + layer, &n)) continue;  // (no adapter)
      add(prefix + "f" + layer, prefix + "df" + layer, n, 1.0);
      units[u]->buffer(std::string("g") + layer, &n);
      add(prefix + "g" + layer, prefix + "dg" + layer, n, 1.0);
      add(prefix + "b" + layer, prefix + "db" + layer, n, 1.0);
      addMoments(prefix + "m" + layer, 2 * n);
    }
  }
  add("fc.f", "fc.df", (std::size_t)finalDepth * classes, 1.0);
  add("fc.b", "fc.db", (std::size_t)classes, 1.0);
  if (params.size() >= 65536) {
    message = "too many parameters";
    return error = VLE_Unsupported;
  }

  const std::size_t arenaBytes = chunks * MCN_SGD_CHUNK * sizeof(float), momentsBytes = momentsCount * sizeof(float);
  std::vector<unsigned short> hostChunks;
  std::vector<double> hostRates;
  for (std::size_t p = 0; p < params.size(); ++p) {
    hostChunks.insert(hostChunks.end(), (params[p].count + MCN_SGD_CHUNK - 1) / MCN_SGD_CHUNK, (unsigned short)p);
    hostRates.push_back(params[p].learningRate);
    hostRates.push_back(params[p].weightDecay);
  }
  bool good = hipMalloc((void**)&values, arenaBytes) == hipSuccess && hipMalloc((void**)&ders, arenaBytes) == hipSuccess &&
              hipMalloc((void**)&state, arenaBytes) == hipSuccess &&
              hipMalloc((void**)&batchMoments, momentsBytes) == hipSuccess &&
              hipMalloc((void**)&runningMoments, momentsBytes) == hipSuccess &&
              hipMalloc((void**)&chunkParam, hostChunks.size() * sizeof(unsigned short)) == hipSuccess &&
              hipMalloc((void**)&rates, hostRates.size() * sizeof(double)) == hipSuccess;
  good = good && hipMemset(values, 0, arenaBytes) == hipSuccess && hipMemset(ders, 0, arenaBytes) == hipSuccess &&
         hipMemset(state, 0, arenaBytes) == hipSuccess && hipMemset(batchMoments, 0, momentsBytes) == hipSuccess &&
         hipMemset(runningMoments, 0, momentsBytes) == hipSuccess &&
         hipMemcpy(chunkParam, hostChunks.data(), hostChunks.size() * sizeof(unsigned short), hipMemcpyHostToDevice) == hipSuccess &&
         hipMemcpy(rates, hostRates.data(), hostRates.size() * sizeof(double), hipMemcpyHostToDevice) == hipSuccess;
  if (!good) {
    (void)hipGetLastError();
    message = "cannot allocate the parameter arenas";
    return error = VLE_OutOfGPUMemeory;
  }

  // views
  for (std::size_t i = 0; i < own.size(); ++i) {
    view(own[i].name, own[i].shape, values + params[i].offset);
    view(params[i].der, own[i].shape, ders + params[i].offset);
  }
  view("stem.m", TensorShape(64, 2, 1, 1), batchMoments + moments[0].offset);
  for (std::size_t p = own.size(); p + 2 < params.size(); ++p) {
    const std::size_t dot = params[p].name.find('.');
    Bottleneck* u = units[std::atoi(params[p].name.substr(4, dot - 4).c_str())];
    if (u->alias(params[p].name.substr(dot + 1), values + params[p].offset) != VLE_Success ||
        u->alias(params[p].der.substr(dot + 1), ders + params[p].offset) != VLE_Success) {
      message = u->lastMessage();
      return error = u->lastError();
    }
  }
  for (std::size_t m = 1; m < moments.size(); ++m) {
    const std::size_t dot = moments[m].name.find('.');
    Bottleneck* u = units[std::atoi(moments[m].name.substr(4, dot - 4).c_str())];
    if (u->alias(moments[m].name.substr(dot + 1), batchMoments + moments[m].offset) != VLE_Success ||
        u->alias("r" + moments[m].name.substr(dot + 1), runningMoments + moments[m].offset) != VLE_Success) {
      message = u->lastMessage();
      return error = u->lastError();
    }
  }
  const Param& ff = params[params.size() - 2];
  const Param& fb = params[params.size() - 1];
  view("fc.f", TensorShape(1, 1, finalDepth, classes), values + ff.offset);
  view("fc.df", TensorShape(1, 1, finalDepth, classes), ders + ff.offset);
  view("fc.b", TensorShape(classes, 1, 1, 1), values + fb.offset);
  view("fc.db", TensorShape(classes, 1, 1, 1), ders + fb.offset);
  return VLE_Success;
}

void ResNet50::view(std::string const& name, TensorShape const& shape, float* memory) {
  Slot s;
  s.name = name;
  s.tensor = Tensor(shape, VLDT_Float, VLDT_GPU, memory, shape.getNumElements() * sizeof(float));
  s.owned = false;
  slots.push_back(s);
}

ErrorCode ResNet50::sgdStep(double learningRate, double momentum, double weightDecay) {
  if (error != VLE_Success) return error;
  void* st = context.getHipHelper().getStream();
  // gradient-trained parameters: the default solver of examples/cnn_train_dag.m:340-364, one worker
  ABI("sgd", mcn_sgd_momentum(st, values, state, ders, chunks, chunkParam, rates, learningRate, weightDecay, momentum, 1.0, 0));
  // moments: trainMethod 'average' (:331-335) with the rate cnn_imagenet_init_resnet.m:190-195 sets, fan-out 1
  const double rate = 0.3;
  ABI("moments", mcn_taccum(st, runningMoments, (float)(1.0 - rate), runningMoments, (float)rate, batchMoments, momentsCount));
  return pack();  // (the filters have changed)
}

namespace {
mcn_loss_geom lossGeometry(Tensor const& prediction, int kind, int topK) {
  mcn_loss_geom g;
  g.H = g.W = 1;
  g.C = (int)prediction.getDepth();
  g.N = (int)prediction.getSize();
  g.loss = kind;
  g.topK = topK;
  g.normalise = 1;
  g.threshold = 0;
  return g;
}
}  // namespace

ErrorCode ResNet50::lossDerivative(double derOutput) {
  if (error != VLE_Success) return error;
  void* st = context.getHipHelper().getStream();
  const mcn_loss_geom g = lossGeometry(slot("prediction"), MCN_LOSS_SOFTMAXLOG, 5);
  ABI("loss", mcn_loss_backward(st, &g, (float*)slot("dprediction").getMemory(), (float const*)slot("prediction").getMemory(),
                                (float const*)slot("labels").getMemory(), (size_t)g.N, NULL, 0, derOutput));
  return VLE_Success;
}

ErrorCode ResNet50::losses(double* objective, double* top1Error, double* top5Error) {
  if (error != VLE_Success) return error;
  void* st = context.getHipHelper().getStream();
  float* values = (float*)slot("loss.values").getMemory();
  void* terms = slot("loss.terms").getMemory();
  const size_t termBytes = slot("loss.terms").getNumElements() * sizeof(float);
  const int kinds[3] = {MCN_LOSS_SOFTMAXLOG, MCN_LOSS_CLASSERROR, MCN_LOSS_TOPKERROR};
  for (int k = 0; k < 3; ++k) {
    const mcn_loss_geom g = lossGeometry(slot("prediction"), kinds[k], 5);
    ABI("loss", mcn_loss_forward(st, &g, values + k, (float const*)slot("prediction").getMemory(),
                                 (float const*)slot("labels").getMemory(), (size_t)g.N, NULL, 0, terms, termBytes));
  }
  float host[3] = {0, 0, 0};
  if (hipMemcpyAsync(host, values, sizeof(host), hipMemcpyDeviceToHost, (hipStream_t)st) != hipSuccess ||
      hipStreamSynchronize((hipStream_t)st) != hipSuccess) {
    (void)hipGetLastError();
    message = "cannot read the loss values back";
    return VLE_Cuda;
  }
  if (objective) *objective = host[0];
  if (top1Error) *top1Error = host[1];
  if (top5Error) *top5Error = host[2];
  return VLE_Success;
}

void ResNet50::dropGraph() {
  if (graphExec) (void)hipGraphExecDestroy((hipGraphExec_t)graphExec);
  if (graph) (void)hipGraphDestroy((hipGraph_t)graph);
  graph = graphExec = NULL;
}

ErrorCode ResNet50::setPacked(bool on) {
  if (error != VLE_Success) return error;
  dropGraph();
  if (packedArena) (void)hipFree(packedArena);
  if (packedJobs) (void)hipFree(packedJobs);
  packedArena = packedJobs = NULL;
  packed = false;
  for (std::size_t i = 0; i < units.size(); ++i)
    if (units[i]->setPacked(on) != VLE_Success) {
      message = units[i]->lastMessage();
      return VLE_OutOfGPUMemeory;
    }
  if (!on) return VLE_Success;
  nn::Convolution stem(context, 2, 2, 3, 3, 3, 3, 1, 1), fc(context, 1, 1, 0, 0, 0, 0, 1, 1);
  const TensorShape inputShape = slot("input").getShape(), avgShape = slot("avg").getShape();
  stemBytes = stem.packedBytes(MCN_CONV_FORWARD, inputShape, slot("stem.f").getShape());
  fcForwardBytes = fc.packedBytes(MCN_CONV_FORWARD, avgShape, slot("fc.f").getShape());
  fcBackwardBytes = fc.packedBytes(MCN_CONV_BACKWARD_DATA, avgShape, slot("fc.f").getShape());
  fcBackwardOffset = stemBytes + fcForwardBytes;
  const std::size_t total = stemBytes + fcForwardBytes + fcBackwardBytes;
  if (hipMalloc(&packedArena, total ? total : 16) != hipSuccess) {
    (void)hipGetLastError();
    packedArena = NULL;
    message = "cannot allocate the packed filter banks";
    return VLE_OutOfGPUMemeory;
  }
  std::vector<mcn_conv_pack_job> jobs;
  char* arena = (char*)packedArena;
  if ((stemBytes && stem.planPack(MCN_CONV_FORWARD, inputShape, slot("stem.f"), arena, stemBytes, jobs) != VLE_Success) ||
      (fcForwardBytes && fc.planPack(MCN_CONV_FORWARD, avgShape, slot("fc.f"), arena + stemBytes, fcForwardBytes, jobs) != VLE_Success) ||
      (fcBackwardBytes && fc.planPack(MCN_CONV_BACKWARD_DATA, avgShape, slot("fc.f"), arena + fcBackwardOffset, fcBackwardBytes, jobs) != VLE_Success))
    return fail(context.getLastError(), "planPack");
  for (std::size_t i = 0; i < units.size(); ++i) jobs.insert(jobs.end(), units[i]->packJobs().begin(), units[i]->packJobs().end());
  packedJobCount = (int)jobs.size();
  packedBlocks = mcn_conv_pack_layout(jobs.data(), packedJobCount);
  const std::size_t bytes = jobs.size() * sizeof(mcn_conv_pack_job);
  if (hipMalloc(&packedJobs, bytes ? bytes : 16) != hipSuccess ||
      hipMemcpy(packedJobs, jobs.data(), bytes, hipMemcpyHostToDevice) != hipSuccess) {
    (void)hipGetLastError();
    message = "cannot upload the packing jobs";
    return VLE_Cuda;
  }
  packed = true;
  return pack();
}

ErrorCode ResNet50::setChannelSums(bool on) {
  if (error != VLE_Success) return error;
  dropGraph();
  for (std::size_t i = 0; i < units.size(); ++i) {
    if (units[i]->setEpilogueSums(on) != VLE_Success || units[i]->setMaskBits(on) != VLE_Success) {
      message = units[i]->lastMessage();
      return VLE_OutOfGPUMemeory;
    }
    // Only units that can also keep their mask as bits take the sums from their convolutions: elsewhere the summing
    // convolution (one 32-channel block per wavefront, whole banks only) costs the forward pass more than the saved
    // summing launches give back (forward 4.09 -> 4.28 ms at 32 images with all units, 7.53 -> 7.88 ms at 64).
    if (on && !units[i]->maskBitsOn() && units[i]->setEpilogueSums(false) != VLE_Success) {
      message = units[i]->lastMessage();
      return VLE_OutOfGPUMemeory;
    }
  }
  return VLE_Success;
}

ErrorCode ResNet50::setOverlap(bool on) {
  if (error != VLE_Success) return error;
  dropGraph();
  if (on && !sideStream) {
    hipStream_t st = NULL;
    hipEvent_t ev = NULL;
    if (hipStreamCreateWithFlags(&st, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      if (st) (void)hipStreamDestroy(st);
      message = "cannot create the second stream";
      return VLE_Cuda;
    }
    sideStream = st;
    sideDone = ev;
    (void)mcn_stream_beside(sideStream, 1);  // its launches run beside the main stream's: one workgroup slot per CU
  }
  for (std::size_t i = 0; i < units.size(); ++i)
    if (units[i]->setOverlap(on, sideStream) != VLE_Success) {
      message = units[i]->lastMessage();
      return VLE_Cuda;
    }
  overlap = on;
  return VLE_Success;
}

ErrorCode ResNet50::setDeferred(bool on) {
  if (error != VLE_Success) return error;
  dropGraph();
  if (partialArena) (void)hipFree(partialArena);
  if (sumJobsDevice) (void)hipFree(sumJobsDevice);
  partialArena = sumJobsDevice = NULL;
  deferred = false;
  for (std::size_t i = 0; i < units.size(); ++i)
    if (units[i]->setDeferred(on, true) != VLE_Success) {
      message = units[i]->lastMessage();
      return VLE_OutOfGPUMemeory;
    }
  if (!on) return VLE_Success;
  nn::Convolution stem(context, 2, 2, 3, 3, 3, 3, 1, 1), fc(context, 1, 1, 0, 0, 0, 0, 1, 1);
  const TensorShape inputShape = slot("input").getShape(), avgShape = slot("avg").getShape();
  stemPartialBytes = stem.filterPartialBytes(inputShape, slot("stem.df").getShape());
  fcPartialBytes = fc.filterPartialBytes(avgShape, slot("fc.df").getShape());
  const std::size_t total = stemPartialBytes + fcPartialBytes;
  if (hipMalloc(&partialArena, total ? total : 16) != hipSuccess) {
    (void)hipGetLastError();
    partialArena = NULL;
    message = "cannot allocate the partial filter gradients";
    return VLE_OutOfGPUMemeory;
  }
  std::vector<mcn_conv_reduce_job> jobs;
  char* arena = (char*)partialArena;
  if ((stemPartialBytes && stem.planFilterPartial(inputShape, slot("stem.df"), arena, stemPartialBytes, jobs) != VLE_Success) ||
      (fcPartialBytes && fc.planFilterPartial(avgShape, slot("fc.df"), arena + stemPartialBytes, fcPartialBytes, jobs) != VLE_Success))
    return fail(context.getLastError(), "planFilterPartial");
  for (std::size_t i = 0; i < units.size(); ++i)
    jobs.insert(jobs.end(), units[i]->reduceJobs().begin(), units[i]->reduceJobs().end());
  sumJobCount = (int)jobs.size();
  sumBlocks = mcn_conv_reduce_layout(jobs.data(), sumJobCount);
  const std::size_t bytes = jobs.size() * sizeof(mcn_conv_reduce_job);
  if (hipMalloc(&sumJobsDevice, bytes ? bytes : 16) != hipSuccess ||
      hipMemcpy(sumJobsDevice, jobs.data(), bytes, hipMemcpyHostToDevice) != hipSuccess) {
    (void)hipGetLastError();
    message = "cannot upload the summing jobs";
    return VLE_Cuda;
  }
  deferred = true;
  return VLE_Success;
}

ErrorCode ResNet50::pack() {
  if (error != VLE_Success) return error;
  if (!packed) return VLE_Success;
  ABI("pack", mcn_conv_pack_batch(context.getHipHelper().getStream(), (mcn_conv_pack_job const*)packedJobs, packedJobCount,
                                  packedBlocks));
  return VLE_Success;
}

ErrorCode ResNet50::capture(bool training, double learningRate, double momentum, double weightDecay) {
  if (error != VLE_Success) return error;
  hipStream_t st = (hipStream_t)context.getHipHelper().getStream();
  if (!st) {
    message = "capture needs a stream of its own (the default stream cannot be captured)";
    return VLE_IllegalArgument;
  }
  dropGraph();
  if (hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal) != hipSuccess) {
    (void)hipGetLastError();
    message = "cannot begin the stream capture";
    return VLE_Cuda;
  }
  ErrorCode e = forward();
  if (e == VLE_Success && training) e = backward();
  if (e == VLE_Success && training) e = sgdStep(learningRate, momentum, weightDecay);
  hipGraph_t g = NULL;
  const hipError_t ended = hipStreamEndCapture(st, &g);
  if (e != VLE_Success) {
    if (g) (void)hipGraphDestroy(g);
    (void)hipGetLastError();
    return e;
  }
  if (ended != hipSuccess || !g) {
    (void)hipGetLastError();
    message = std::string("the stream capture failed: ") + hipGetErrorString(ended) +
              " (run the step once eagerly first: capture cannot grow the workspace)";
    return VLE_Cuda;
  }
  hipGraphExec_t x = NULL;
  if (hipGraphInstantiate(&x, g, NULL, NULL, 0) != hipSuccess) {
    (void)hipGetLastError();
    (void)hipGraphDestroy(g);
    message = "cannot instantiate the graph";
    return VLE_Cuda;
  }
  graph = g;
  graphExec = x;
  return VLE_Success;
}

ErrorCode ResNet50::replay() {
  if (error != VLE_Success) return error;
  if (!graphExec) {
    message = "nothing has been captured";
    return VLE_IllegalArgument;
  }
  if (hipGraphLaunch((hipGraphExec_t)graphExec, (hipStream_t)context.getHipHelper().getStream()) != hipSuccess) {
    (void)hipGetLastError();
    message = "cannot launch the graph";
    return VLE_Cuda;
  }
  return VLE_Success;
}

ResNet50::~ResNet50() {
  dropGraph();
  if (sideStream) (void)hipStreamSynchronize((hipStream_t)sideStream);
  for (std::size_t i = 0; i < units.size(); ++i) delete units[i];
  if (sideDone) (void)hipEventDestroy((hipEvent_t)sideDone);
  if (sideStream) {
    (void)mcn_stream_beside(sideStream, 0);
    (void)hipStreamDestroy((hipStream_t)sideStream);
  }
  for (std::size_t i = 0; i < slots.size(); ++i)
    if (slots[i].owned && slots[i].tensor.getMemory()) (void)hipFree(slots[i].tensor.getMemory());
  void* arenas[] = {values, ders, state, batchMoments, runningMoments, chunkParam, rates, packedArena, packedJobs,
                    partialArena, sumJobsDevice};
  for (void* a : arenas)
    if (a) (void)hipFree(a);
}

Tensor ResNet50::make(std::string const& name, TensorShape const& shape) {
  void* memory = NULL;
  const std::size_t bytes = shape.getNumElements() * sizeof(float);
  if (error == VLE_Success && hipMalloc(&memory, bytes ? bytes : 4) != hipSuccess) {
    (void)hipGetLastError();
    error = VLE_OutOfGPUMemeory;
    message = "cannot allocate buffer '" + name + "'";
    memory = NULL;
  }
  Slot s;
  s.name = name;
  s.tensor = Tensor(shape, VLDT_Float, VLDT_GPU, memory, bytes);
  s.owned = true;
  slots.push_back(s);
  return s.tensor;
}

Tensor& ResNet50::slot(std::string const& name) {
  for (std::size_t i = 0; i < slots.size(); ++i)
    if (slots[i].name == name) return slots[i].tensor;
  static Tensor none;
  return none;
}

float* ResNet50::buffer(std::string const& name, std::size_t* count) {
  if (name.compare(0, 4, "unit") == 0) {
    const std::size_t dot = name.find('.');
    if (dot == std::string::npos) return NULL;
    const int i = std::atoi(name.substr(4, dot - 4).c_str());
    if (i < 0 || i >= (int)units.size()) return NULL;
    return units[i]->buffer(name.substr(dot + 1), count);
  }
  if (name.compare(0, 9, "momentum.") == 0) {
    for (std::size_t p = 0; p < params.size(); ++p)
      if (params[p].name == name.substr(9)) {
        if (count) *count = params[p].count;
        return state + params[p].offset;
      }
    return NULL;
  }
  if (name.compare(0, 8, "running.") == 0) {
    for (std::size_t m = 0; m < moments.size(); ++m)
      if (moments[m].name == name.substr(8)) {
        if (count) *count = moments[m].count;
        return runningMoments + moments[m].offset;
      }
    return NULL;
  }
  Tensor& t = slot(name);
  if (count) *count = t.getNumElements();
  return (float*)t.getMemory();
}

ErrorCode ResNet50::setStream(void* stream) { return context.getHipHelper().setStream(stream); }

void ResNet50::setFused(bool on) {
  fused = on;
  for (std::size_t i = 0; i < units.size(); ++i) units[i]->setFused(on);
}

void ResNet50::setTestMode(bool on) {
  testMode = on;
  for (std::size_t i = 0; i < units.size(); ++i) units[i]->setTestMode(on);
}

ErrorCode ResNet50::fail(ErrorCode e, char const* where) {
  if (e != VLE_Success) {
    error = e;
    message = std::string(where) + ": " + context.getLastErrorMessage();
  }
  return e;
}

ErrorCode ResNet50::initParameters(unsigned long long seed) {
  if (error != VLE_Success) return error;
  std::mt19937_64 gen(seed);
  std::normal_distribution<float> dist(0.f, 1.f);
  std::vector<float> host;
  auto upload = [&](float* dst, std::size_t n, float scale, float constant, bool random) -> bool {
    host.resize(n);
    for (std::size_t i = 0; i < n; ++i) host[i] = random ? scale * dist(gen) : constant;
    return hipMemcpy(dst, host.data(), n * sizeof(float), hipMemcpyHostToDevice) == hipSuccess;
  };
  auto filter = [&](std::string const& name) -> bool {
    std::size_t n = 0;
    float* p = buffer(name, &n);
    if (!p) return true;  // (a unit without adapter has no "fs")
    // fan-in = elements per filter: the last extent of the bank is the number of filters
    Tensor* t = NULL;
    if (name.compare(0, 4, "unit") != 0) t = &slot(name);
    std::size_t filters = t ? t->getSize() : 0;
    if (!t) {
      // bank shapes of a unit follow from its name
      const std::size_t dot = name.find('.');
      Bottleneck* u = units[std::atoi(name.substr(4, dot - 4).c_str())];
      const std::string leaf = name.substr(dot + 1);
      std::size_t m = 0, c3 = 0;
      u->buffer("g1", &m);
      u->buffer("g3", &c3);
      filters = (leaf == "f1" || leaf == "f2") ? m : c3;
    }
    const float scale = std::sqrt(2.f / (float)(n / filters));
    return upload(p, n, scale, 0.f, true);
  };
  auto constant = [&](std::string const& name, float value) -> bool {
    std::size_t n = 0;
    float* p = buffer(name, &n);
    return !p || upload(p, n, 0.f, value, false);
  };
  bool good = filter("stem.f") && constant("stem.g", 1.f) && constant("stem.b", 0.f);
  for (std::size_t i = 0; i < units.size() && good; ++i) {
    const std::string u = "unit" + std::to_string(i) + ".";
    good = filter(u + "f1") && filter(u + "f2") && filter(u + "f3") && filter(u + "fs");
    for (char const* g : {"g1", "g2", "g3", "gs"}) good = good && constant(u + g, 1.f);
    for (char const* b : {"b1", "b2", "b3", "bs"}) good = good && constant(u + b, 0.f);
  }
  good = good && filter("fc.f") && constant("fc.b", 0.f);
  if (!good) {
    (void)hipGetLastError();
    message = "cannot upload the parameters";
    return error = VLE_Cuda;
  }
  return pack();
}

ErrorCode ResNet50::forward() {
  if (error != VLE_Success) return error;
  void* st = context.getHipHelper().getStream();
  Tensor none;
  const int S2 = S / 2;
  nn::Convolution stem(context, 2, 2, 3, 3, 3, 3, 1, 1), fc(context, 1, 1, 0, 0, 0, 0, 1, 1);
  nn::BatchNorm bn(context, epsilon);
  nn::Pooling maxPool(context, 3, 3, 2, 2, 1, 1, 1, 1, nn::Pooling::Max);
  if (packed) {
    stem.usePacked(stemBytes ? packedArena : NULL, stemBytes, NULL, 0);
    fc.usePacked(fcForwardBytes ? (char*)packedArena + stemBytes : NULL, fcForwardBytes, NULL, 0);
  }
  STEP("stem conv", stem.forward(slot("stem.a"), 0, slot("input"), 1, slot("stem.f"), none));
  if (fused) {
    const size_t wsBytes = mcn_bnorm_workspace_bytes(S2, S2, 64, N);
    void* ws = context.getWorkspace(VLDT_GPU, wsBytes);
    if (!ws) return fail(context.getLastError(), "workspace");
    float* stemMoments = testMode ? runningMoments + moments[0].offset : (float*)slot("stem.m").getMemory();
    ABI("stem bnorm", mcn_bnorm_forward_fused(st, (float*)slot("stem.r").getMemory(), stemMoments,
                                              (float const*)slot("stem.a").getMemory(), (float const*)slot("stem.g").getMemory(),
                                              (float const*)slot("stem.b").getMemory(), NULL, 1, S2, S2, 64, N, epsilon,
                                              testMode ? 1 : 0, ws, wsBytes));
  } else {
    if (testMode) {
      Tensor running(TensorShape(64, 2, 1, 1), VLDT_Float, VLDT_GPU, runningMoments + moments[0].offset, 128 * sizeof(float));
      STEP("stem bnorm", bn.forwardWithMoment(slot("stem.n"), running, slot("stem.a"), slot("stem.g"), slot("stem.b")));
    } else {
      STEP("stem bnorm", bn.forward(slot("stem.n"), slot("stem.m"), slot("stem.a"), slot("stem.g"), slot("stem.b")));
    }
    ABI("stem relu", mcn_relu_forward(st, (float*)slot("stem.r").getMemory(), (float const*)slot("stem.n").getMemory(),
                                      slot("stem.n").getNumElements()));
  }
  STEP("stem pool", maxPool.forward(slot("stem.p"), slot("stem.r")));
  for (std::size_t i = 0; i < units.size(); ++i)
    if (units[i]->forward() != VLE_Success) {
      message = "unit " + std::to_string(i) + ": " + units[i]->lastMessage();
      return error = units[i]->lastError();
    }
  Bottleneck* last = units.back();
  const int Hf = last->outHeight(), Cf = last->outDepth();
  Tensor features(TensorShape(Hf, Hf, Cf, N), VLDT_Float, VLDT_GPU, last->buffer("y"), sizeof(float) * (size_t)Hf * Hf * Cf * N);
  nn::Pooling avgPool(context, Hf, Hf, 1, 1, 0, 0, 0, 0, nn::Pooling::Average);
  STEP("average pool", avgPool.forward(slot("avg"), features));
  STEP("classifier", fc.forward(slot("prediction"), 0, slot("avg"), 1, slot("fc.f"), slot("fc.b")));
  return VLE_Success;
}

ErrorCode ResNet50::backward() {
  if (error != VLE_Success) return error;
  if (testMode) {
    message = "backward needs the batch moments of a training-mode forward pass";
    return VLE_IllegalArgument;
  }
  void* st = context.getHipHelper().getStream();
  Tensor none;
  const int S2 = S / 2;
  nn::Convolution stem(context, 2, 2, 3, 3, 3, 3, 1, 1), fc(context, 1, 1, 0, 0, 0, 0, 1, 1);
  nn::BatchNorm bn(context, epsilon);
  nn::Pooling maxPool(context, 3, 3, 2, 2, 1, 1, 1, 1, nn::Pooling::Max);
  Bottleneck* last = units.back();
  const int Hf = last->outHeight(), Cf = last->outDepth();
  const size_t nFeatures = (size_t)Hf * Hf * Cf * N;
  Tensor features(TensorShape(Hf, Hf, Cf, N), VLDT_Float, VLDT_GPU, last->buffer("y"), sizeof(float) * nFeatures);
  Tensor derFeatures(TensorShape(Hf, Hf, Cf, N), VLDT_Float, VLDT_GPU, last->buffer("dzdy"), sizeof(float) * nFeatures);
  nn::Pooling avgPool(context, Hf, Hf, 1, 1, 0, 0, 0, 0, nn::Pooling::Average);
  if (packed) fc.usePacked(NULL, 0, fcBackwardBytes ? (char*)packedArena + fcBackwardOffset : NULL, fcBackwardBytes);
  if (deferred && fcPartialBytes) {
    STEP("classifier", fc.backward(slot("davg"), none, slot("fc.db"), slot("avg"), slot("fc.f"), slot("dprediction")));
    STEP("classifier", fc.backwardFilterPartial(slot("fc.df"), slot("avg"), slot("dprediction"),
                                                (char*)partialArena + stemPartialBytes, fcPartialBytes));
  } else {
    STEP("classifier", fc.backward(slot("davg"), slot("fc.df"), slot("fc.db"), slot("avg"), slot("fc.f"), slot("dprediction")));
  }
  STEP("average pool", avgPool.backwardOverwrite(derFeatures, features, slot("davg")));
  for (std::size_t i = units.size(); i-- > 0;)
    if (units[i]->backward() != VLE_Success) {
      message = "unit " + std::to_string(i) + ": " + units[i]->lastMessage();
      return error = units[i]->lastError();
    }
  STEP("stem pool", maxPool.backwardOverwrite(slot("stem.dr"), slot("stem.r"), slot("stem.dp")));
  if (fused) {
    const size_t wsBytes = mcn_bnorm_workspace_bytes(S2, S2, 64, N);
    void* ws = context.getWorkspace(VLDT_GPU, wsBytes);
    if (!ws) return fail(context.getLastError(), "workspace");
    ABI("stem bnorm", mcn_bnorm_backward_relu(st, (float*)slot("stem.da").getMemory(), (float*)slot("stem.dg").getMemory(),
                                              (float*)slot("stem.db").getMemory(), (float const*)slot("stem.m").getMemory(),
                                              (float const*)slot("stem.a").getMemory(), (float const*)slot("stem.g").getMemory(),
                                              (float const*)slot("stem.b").getMemory(), (float const*)slot("stem.dr").getMemory(),
                                              S2, S2, 64, N, epsilon, ws, wsBytes));
  } else {
    ABI("stem relu", mcn_relu_backward(st, (float*)slot("stem.dn").getMemory(), (float const*)slot("stem.n").getMemory(),
                                       (float const*)slot("stem.dr").getMemory(), slot("stem.dn").getNumElements()));
    STEP("stem bnorm", bn.backwardWithMoment(slot("stem.da"), slot("stem.dg"), slot("stem.db"), slot("stem.m"), slot("stem.a"),
                                             slot("stem.g"), slot("stem.b"), slot("stem.dn")));
  }
  // the network's input needs no derivative: filter gradient only
  if (deferred && stemPartialBytes) {
    STEP("stem conv", stem.backwardFilterPartial(slot("stem.df"), slot("input"), slot("stem.da"), partialArena, stemPartialBytes));
  } else {
    STEP("stem conv", stem.backward(none, slot("stem.df"), none, slot("input"), slot("stem.f"), slot("stem.da")));
  }
  if (overlap && (hipEventRecord((hipEvent_t)sideDone, (hipStream_t)sideStream) != hipSuccess ||
                  hipStreamWaitEvent((hipStream_t)st, (hipEvent_t)sideDone, 0) != hipSuccess)) {
    (void)hipGetLastError();
    message = "cannot join the second stream";
    return error = VLE_Cuda;
  }
  if (deferred)  // the sums over the reduction splits of every filter gradient of the network
    ABI("filter sums", mcn_conv_reduce_batch(st, (mcn_conv_reduce_job const*)sumJobsDevice, sumJobCount, sumBlocks));
  return VLE_Success;
}

} }  // namespace vl::harness
