#include "bottleneck.hpp"
#include <cstdlib>

#include <hip/hip_runtime_api.h>

#include "../../include/mcn_hip.h"
#include "hiphelper.hpp"
#include "nnbnorm.hpp"
#include "nnconv.hpp"

namespace vl { namespace harness {

Bottleneck::Bottleneck(int H, int W, int C, int M, int N, double epsilon, int CoutArg, int stride, bool adapter,
                       Context* shared)
    : H(H), W(W), C(C), M(M), N(N), Cout(CoutArg > 0 ? CoutArg : C), stride(stride), Ho((H - 1) / stride + 1),
      Wo((W - 1) / stride + 1), adapter(adapter), epsilon(epsilon), context(shared ? *shared : ownContext),
      error(VLE_Success), stageHook(NULL), hookUser(NULL), fused(false), overlap(false), testMode(false), packed(false), packedArena(NULL), packedJobs(NULL), packedBlocks(0), deferred(false), externalSums(false),
      partialArena(NULL), sumJobsDevice(NULL), sumBlocks(0), epilogueSums(false), sumsBuffer(NULL), maskBits(NULL), sumsBytes(0),
      sideStream(NULL), sideShared(false) {
  for (int i = 0; i < 4; ++i) sumGroupsOf[i] = 0;
  for (int i = 0; i < 5; ++i) events[i] = NULL;
  if (!adapter && (Cout != C || stride != 1)) {
    error = VLE_IllegalArgument;
    message = "a unit that changes the number of channels or the resolution needs the adapter on its shortcut";
    return;
  }
  const TensorShape in(H, W, C, N), mid(H, W, M, N), midOut(Ho, Wo, M, N), out(Ho, Wo, Cout, N);
  // inputs and parameters
  make("x", in); make("dzdy", out);
  make("f1", TensorShape(1, 1, C, M)); make("f2", TensorShape(3, 3, M, M)); make("f3", TensorShape(1, 1, M, Cout));
  make("g1", TensorShape(M, 1, 1, 1)); make("b1", TensorShape(M, 1, 1, 1));
  make("g2", TensorShape(M, 1, 1, 1)); make("b2", TensorShape(M, 1, 1, 1));
  make("g3", TensorShape(Cout, 1, 1, 1)); make("b3", TensorShape(Cout, 1, 1, 1));
  // forward activations
  make("a1", mid); make("n1", mid); make("r1", mid);
  make("a2", midOut); make("n2", midOut); make("r2", midOut);
  make("a3", out); make("n3", out); make("s", out); make("y", out);
  make("m1", TensorShape(M, 2, 1, 1)); make("m2", TensorShape(M, 2, 1, 1)); make("m3", TensorShape(Cout, 2, 1, 1));
  make("rm1", TensorShape(M, 2, 1, 1)); make("rm2", TensorShape(M, 2, 1, 1)); make("rm3", TensorShape(Cout, 2, 1, 1));
  // derivatives
  make("ds", out); make("da3", out); make("dr2", midOut); make("dn2", midOut); make("da2", midOut);
  make("dr1", mid); make("dn1", mid); make("da1", mid); make("dxm", in); make("dzdx", in);
  make("df1", TensorShape(1, 1, C, M)); make("df2", TensorShape(3, 3, M, M)); make("df3", TensorShape(1, 1, M, Cout));
  make("dg1", TensorShape(M, 1, 1, 1)); make("db1", TensorShape(M, 1, 1, 1));
  make("dg2", TensorShape(M, 1, 1, 1)); make("db2", TensorShape(M, 1, 1, 1));
  make("dg3", TensorShape(Cout, 1, 1, 1)); make("db3", TensorShape(Cout, 1, 1, 1));
  if (adapter) {
    make("fs", TensorShape(1, 1, C, Cout)); make("gs", TensorShape(Cout, 1, 1, 1)); make("bs", TensorShape(Cout, 1, 1, 1));
    make("as", out); make("ns", out); make("ms", TensorShape(Cout, 2, 1, 1));
    make("rms", TensorShape(Cout, 2, 1, 1));
    make("das", out); make("dfs", TensorShape(1, 1, C, Cout));
    make("dgs", TensorShape(Cout, 1, 1, 1)); make("dbs", TensorShape(Cout, 1, 1, 1));
  }
}

ErrorCode Bottleneck::setOverlap(bool on, void* stream) {
  if (on && sideStream && (stream ? sideStream != stream : sideShared)) {
    message = "the second stream cannot be changed once set";
    return VLE_IllegalArgument;
  }
  if (on && !sideStream) {
    hipStream_t st = (hipStream_t)stream;
    if (!st && hipStreamCreateWithFlags(&st, hipStreamNonBlocking) != hipSuccess) {
      (void)hipGetLastError();
      message = "cannot create the second stream";
      return error = VLE_Cuda;
    }
    sideStream = st;
    sideShared = stream != NULL;
    for (int i = 0; i < 5; ++i) {
      hipEvent_t e = NULL;
      if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) {
        (void)hipGetLastError();
        message = "cannot create an event";
        return error = VLE_Cuda;
      }
      events[i] = e;
    }
    sideContext.getHipHelper().setStream(sideStream);
    // (a stream of the unit's own: its launches run beside the caller's stream; a shared one is marked by its owner)
    if (!sideShared) (void)mcn_stream_beside(sideStream, 1);
  }
  overlap = on;
  return VLE_Success;
}

Bottleneck::~Bottleneck() {
  if (sideStream) {
    (void)hipStreamSynchronize((hipStream_t)sideStream);
    sideContext.clear();
    for (int i = 0; i < 5; ++i)
      if (events[i]) (void)hipEventDestroy((hipEvent_t)events[i]);
    if (!sideShared) {
      (void)mcn_stream_beside(sideStream, 0);
      (void)hipStreamDestroy((hipStream_t)sideStream);
    }
  }
  for (std::size_t i = 0; i < slots.size(); ++i)
    if (slots[i].owned && slots[i].tensor.getMemory()) (void)hipFree(slots[i].tensor.getMemory());
  if (packedArena) (void)hipFree(packedArena);
  if (packedJobs) (void)hipFree(packedJobs);
  if (partialArena) (void)hipFree(partialArena);
  if (sumJobsDevice) (void)hipFree(sumJobsDevice);
  if (sumsBuffer) (void)hipFree(sumsBuffer);
  if (maskBits) (void)hipFree(maskBits);
}

#define STEP(stage, call)                                   \
  do {                                                      \
    mark(stage, 1);                                         \
    ErrorCode e_ = (call);                                  \
    mark(stage, 0);                                         \
    if (e_ != VLE_Success) return fail(e_, stage);          \
  } while (0)

#define ABI(stage, call)                                                                    \
  do {                                                                                      \
    mark(stage, 1);                                                                         \
    int rc_ = (call);                                                                       \
    mark(stage, 0);                                                                         \
    if (rc_ != 0) {                                                                         \
      context.setError((ErrorCode)rc_, mcn_last_error_message());                           \
      return fail((ErrorCode)rc_, stage);                                                   \
    }                                                                                       \
  } while (0)

// The four convolutions in a fixed order: 1x1 in, 3x3, 1x1 out, adapter.
ErrorCode Bottleneck::setPacked(bool on) {
  if (packedArena) (void)hipFree(packedArena);
  if (packedJobs) (void)hipFree(packedJobs);
  packedArena = NULL;
  packedJobs = NULL;
  jobs.clear();
  packed = false;
  if (!on || error != VLE_Success) return error;
  nn::Convolution c1(context, 1, 1, 0, 0, 0, 0, 1, 1), c2(context, stride, stride, 1, 1, 1, 1, 1, 1),
      cs(context, stride, stride, 0, 0, 0, 0, 1, 1);
  struct Layer { nn::Convolution* op; char const* data; char const* filter; };
  const Layer layers[4] = {{&c1, "x", "f1"}, {&c2, "r1", "f2"}, {&c1, "r2", "f3"}, {&cs, "x", "fs"}};
  const int count = adapter ? 4 : 3;
  std::size_t total = 0;
  for (int l = 0; l < count; ++l)
    for (int product = 0; product < 2; ++product) {  // MCN_CONV_FORWARD, MCN_CONV_BACKWARD_DATA
      banks[l][product].offset = total;
      banks[l][product].bytes = layers[l].op->packedBytes(product, slot(layers[l].data).getShape(), slot(layers[l].filter).getShape());
      total += banks[l][product].bytes;
    }
  if (hipMalloc(&packedArena, total ? total : 16) != hipSuccess) {
    (void)hipGetLastError();
    packedArena = NULL;
    message = "cannot allocate the packed filter banks";
    return VLE_OutOfGPUMemeory;
  }
  for (int l = 0; l < count; ++l)
    for (int product = 0; product < 2; ++product) {
      if (banks[l][product].bytes == 0) continue;
      ErrorCode e = layers[l].op->planPack(product, slot(layers[l].data).getShape(), slot(layers[l].filter),
                                           (char*)packedArena + banks[l][product].offset, banks[l][product].bytes, jobs);
      if (e != VLE_Success) return fail(e, "planPack");
    }
  packed = true;
  return VLE_Success;
}

ErrorCode Bottleneck::setDeferred(bool on, bool external) {
  if (partialArena) (void)hipFree(partialArena);
  if (sumJobsDevice) (void)hipFree(sumJobsDevice);
  partialArena = sumJobsDevice = NULL;
  sumJobs.clear();
  deferred = false;
  if (!on || error != VLE_Success) return error;
  nn::Convolution c1(context, 1, 1, 0, 0, 0, 0, 1, 1), c2(context, stride, stride, 1, 1, 1, 1, 1, 1),
      cs(context, stride, stride, 0, 0, 0, 0, 1, 1);
  struct Layer { nn::Convolution* op; char const* data; char const* der; };
  const Layer layers[4] = {{&c1, "x", "df1"}, {&c2, "r1", "df2"}, {&c1, "r2", "df3"}, {&cs, "x", "dfs"}};
  const int count = adapter ? 4 : 3;
  std::size_t total = 0;
  for (int l = 0; l < 4; ++l) partialBank[l].offset = partialBank[l].bytes = 0;
  for (int l = 0; l < count; ++l) {
    partialBank[l].offset = total;
    partialBank[l].bytes = layers[l].op->filterPartialBytes(slot(layers[l].data).getShape(), slot(layers[l].der).getShape());
    total += partialBank[l].bytes;
  }
  if (hipMalloc(&partialArena, total ? total : 16) != hipSuccess) {
    (void)hipGetLastError();
    partialArena = NULL;
    message = "cannot allocate the partial filter gradients";
    return VLE_OutOfGPUMemeory;
  }
  for (int l = 0; l < count; ++l) {
    if (partialBank[l].bytes == 0) continue;
    ErrorCode e = layers[l].op->planFilterPartial(slot(layers[l].data).getShape(), slot(layers[l].der),
                                                  (char*)partialArena + partialBank[l].offset, partialBank[l].bytes, sumJobs);
    if (e != VLE_Success) return fail(e, "planFilterPartial");
  }
  if (!external && !sumJobs.empty()) {
    std::vector<mcn_conv_reduce_job> numbered(sumJobs);
    sumBlocks = mcn_conv_reduce_layout(numbered.data(), (int)numbered.size());
    const std::size_t bytes = numbered.size() * sizeof(mcn_conv_reduce_job);
    if (hipMalloc(&sumJobsDevice, bytes) != hipSuccess ||
        hipMemcpy(sumJobsDevice, numbered.data(), bytes, hipMemcpyHostToDevice) != hipSuccess) {
      (void)hipGetLastError();
      message = "cannot upload the summing jobs";
      return VLE_Cuda;
    }
  }
  deferred = true;
  externalSums = external;
  return VLE_Success;
}

ErrorCode Bottleneck::setEpilogueSums(bool on) {
  if (sumsBuffer) (void)hipFree(sumsBuffer);
  sumsBuffer = NULL;
  sumsBytes = 0;
  epilogueSums = false;
  if (maskBits) (void)hipFree(maskBits);  // (the mask bits are written by the pass that takes the channel sums)
  maskBits = NULL;
  for (int i = 0; i < 4; ++i) sumGroupsOf[i] = 0;
  if (!on || error != VLE_Success) return error;
  nn::Convolution c1(context, 1, 1, 0, 0, 0, 0, 1, 1), c2(context, stride, stride, 1, 1, 1, 1, 1, 1),
      cs(context, stride, stride, 0, 0, 0, 0, 1, 1);
  struct Layer { nn::Convolution* op; char const* data; char const* filter; };
  const Layer layers[4] = {{&c1, "x", "f1"}, {&c2, "r1", "f2"}, {&c1, "r2", "f3"}, {&cs, "x", "fs"}};
  for (int l = 0; l < (adapter ? 4 : 3); ++l) {
    sumGroupsOf[l] = layers[l].op->sumGroups(slot(layers[l].data).getShape(), slot(layers[l].filter).getShape());
    const std::size_t bytes = (std::size_t)slot(layers[l].filter).getSize() * sumGroupsOf[l] * 2 * sizeof(double);
    if (bytes > sumsBytes) sumsBytes = bytes;
  }
  if (sumsBytes && hipMalloc(&sumsBuffer, sumsBytes) != hipSuccess) {
    (void)hipGetLastError();
    sumsBuffer = NULL;
    message = "cannot allocate the partial channel sums";
    return VLE_OutOfGPUMemeory;
  }
  epilogueSums = true;
  return VLE_Success;
}

ErrorCode Bottleneck::setMaskBits(bool on) {
  if (maskBits) (void)hipFree(maskBits);
  maskBits = NULL;
  if (!on || error != VLE_Success) return error;
  // needs: the folded schedule with the third convolution's channel sums, an identity shortcut, planes of whole mask
  // words, and a first convolution whose input gradient can take the second term
  if (!fused || !epilogueSums || adapter || sumGroupsOf[2] <= 0 || !mcn_bnorm_mask_bits_supported(Ho, Wo, Cout, N)) return VLE_Success;
  nn::Convolution c1(context, 1, 1, 0, 0, 0, 0, 1, 1);
  if (!c1.maskedAddSupported(slot("x").getShape(), slot("f1").getShape())) return VLE_Success;
  const std::size_t words = (slot("y").getNumElements() + 31) / 32;
  if (hipMalloc((void**)&maskBits, words * sizeof(unsigned)) != hipSuccess) {
    (void)hipGetLastError();
    maskBits = NULL;
    message = "cannot allocate the ReLU mask";
    return VLE_OutOfGPUMemeory;
  }
  return VLE_Success;
}

void Bottleneck::attachPacked(nn::Convolution& c1, nn::Convolution& c2, nn::Convolution& c3, nn::Convolution& cs) {
  if (!packed) return;
  nn::Convolution* ops[4] = {&c1, &c2, &c3, &cs};
  for (int l = 0; l < (adapter ? 4 : 3); ++l)
    ops[l]->usePacked(banks[l][0].bytes ? (char*)packedArena + banks[l][0].offset : NULL, banks[l][0].bytes,
                      banks[l][1].bytes ? (char*)packedArena + banks[l][1].offset : NULL, banks[l][1].bytes);
}

ErrorCode Bottleneck::pack() {
  if (!packed) return VLE_Success;
  if (!packedJobs && !jobs.empty()) {
    std::vector<mcn_conv_pack_job> numbered(jobs);
    packedBlocks = mcn_conv_pack_layout(numbered.data(), (int)numbered.size());
    const std::size_t bytes = numbered.size() * sizeof(mcn_conv_pack_job);
    if (hipMalloc(&packedJobs, bytes) != hipSuccess ||
        hipMemcpy(packedJobs, numbered.data(), bytes, hipMemcpyHostToDevice) != hipSuccess) {
      (void)hipGetLastError();
      message = "cannot upload the packing jobs";
      return VLE_Cuda;
    }
  }
  ABI("pack", mcn_conv_pack_batch(context.getHipHelper().getStream(), (mcn_conv_pack_job const*)packedJobs, (int)jobs.size(),
                                  packedBlocks));
  return VLE_Success;
}

Tensor Bottleneck::make(std::string const& name, TensorShape const& shape) {
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

Tensor& Bottleneck::slot(std::string const& name) {
  for (std::size_t i = 0; i < slots.size(); ++i)
    if (slots[i].name == name) return slots[i].tensor;
  static Tensor none;
  return none;
}

float* Bottleneck::buffer(std::string const& name, std::size_t* count) {
  Tensor& t = slot(name);
  if (count) *count = t.getNumElements();
  return (float*)t.getMemory();
}

ErrorCode Bottleneck::alias(std::string const& name, float* memory) {
  if (packed) setPacked(false);  // (the packing jobs hold the old addresses)
  if (deferred) setDeferred(false);
  for (std::size_t i = 0; i < slots.size(); ++i) {
    if (slots[i].name != name) continue;
    if (slots[i].owned && slots[i].tensor.getMemory()) (void)hipFree(slots[i].tensor.getMemory());
    const TensorShape shape = slots[i].tensor.getShape();
    slots[i].tensor = Tensor(shape, VLDT_Float, VLDT_GPU, memory, shape.getNumElements() * sizeof(float));
    slots[i].owned = false;
    return VLE_Success;
  }
  message = "no buffer '" + name + "'";
  return error = VLE_IllegalArgument;
}

ErrorCode Bottleneck::setStream(void* stream) { return context.getHipHelper().setStream(stream); }

ErrorCode Bottleneck::fail(ErrorCode e, char const* where) {
  if (e != VLE_Success) {
    error = e;
    message = std::string(where) + ": " + context.getLastErrorMessage();
  }
  return e;
}

ErrorCode Bottleneck::forward() {
  if (error != VLE_Success) return error;
  void* st = context.getHipHelper().getStream();
  Tensor none;
  nn::Convolution c1(context, 1, 1, 0, 0, 0, 0, 1, 1), c2(context, stride, stride, 1, 1, 1, 1, 1, 1),
      c3(context, 1, 1, 0, 0, 0, 0, 1, 1), cs(context, stride, stride, 0, 0, 0, 0, 1, 1);
  attachPacked(c1, c2, c3, cs);
  nn::BatchNorm bn(context, epsilon);
  const std::size_t nMid = slot("a1").getNumElements(), nMidOut = slot("a2").getNumElements(),
                    nOut = slot("a3").getNumElements();
  // training: moments from the batch, kept for the backward pass; test mode: the stored moments "rm*"
  // (matlab/+dagnn/BatchNorm.m:12-24)
  const int given = testMode ? 1 : 0;
  char const* m1 = testMode ? "rm1" : "m1";
  char const* m2 = testMode ? "rm2" : "m2";
  char const* m3 = testMode ? "rm3" : "m3";
  char const* ms = testMode ? "rms" : "ms";
  auto bnForward = [&](char const* out, char const* moments, char const* in, char const* g, char const* b) -> ErrorCode {
    return testMode ? bn.forwardWithMoment(slot(out), slot(moments), slot(in), slot(g), slot(b))
                    : bn.forward(slot(out), slot(moments), slot(in), slot(g), slot(b));
  };
  // the shortcut: the input, or its adapted version (matlab: Conv([name '_adapt_conv'], 1, ..., 'relu', false))
  char const* shortcut = "x";
  if (adapter) {
    STEP("convs_fwd", cs.forward(slot("as"), 0, slot("x"), 1, slot("fs"), none));
    STEP("bns_fwd", bnForward("ns", ms, "as", "gs", "bs"));
    shortcut = "ns";
  }
  if (fused && epilogueSums && !testMode) {
    // convolution + the channel sums of its output in one launch, then only the output pass of the batch normalisation
    struct Stage {
      nn::Convolution* op; int layer; char const* convStage; char const* bnStage;
      char const* out; char const* in; char const* filter; char const* act; char const* moments; char const* g; char const* b;
      char const* residual; int relu; int h, w, c;
    };
    const Stage stages[3] = {
        {&c1, 0, "conv1_fwd", "bn1_fwd", "a1", "x", "f1", "r1", "m1", "g1", "b1", NULL, 1, H, W, M},
        {&c2, 1, "conv2_fwd", "bn2_fwd", "a2", "r1", "f2", "r2", "m2", "g2", "b2", NULL, 1, Ho, Wo, M},
        {&c3, 2, "conv3_fwd", "bn3_fwd", "a3", "r2", "f3", "y", "m3", "g3", "b3", shortcut, 1, Ho, Wo, Cout}};
    for (int i = 0; i < 3; ++i) {
      const Stage& sg = stages[i];
      const int groups = sumGroupsOf[sg.layer];
      float* residual = sg.residual ? buffer(sg.residual) : NULL;
      if (groups > 0) {
        STEP(sg.convStage, sg.op->forwardSums(slot(sg.out), slot(sg.in), slot(sg.filter), (double*)sumsBuffer, sumsBytes));
        if (i == 2 && maskBits)
          ABI(sg.bnStage, mcn_bnorm_forward_sums_mask(st, buffer(sg.act), maskBits, buffer(sg.moments), buffer(sg.out), buffer(sg.g),
                                                      buffer(sg.b), residual, sg.h, sg.w, sg.c, N, epsilon,
                                                      (double const*)sumsBuffer, groups));
        else
        ABI(sg.bnStage, mcn_bnorm_forward_sums(st, buffer(sg.act), buffer(sg.moments), buffer(sg.out), buffer(sg.g), buffer(sg.b),
                                               residual, sg.relu, sg.h, sg.w, sg.c, N, epsilon, (double const*)sumsBuffer, groups));
      } else {
        STEP(sg.convStage, sg.op->forward(slot(sg.out), 0, slot(sg.in), 1, slot(sg.filter), none));
        const size_t wsBytes = mcn_bnorm_workspace_bytes(sg.h, sg.w, sg.c, N);
        void* ws = context.getWorkspace(VLDT_GPU, wsBytes);
        if (!ws) return fail(context.getLastError(), "workspace");
        ABI(sg.bnStage, mcn_bnorm_forward_fused(st, buffer(sg.act), buffer(sg.moments), buffer(sg.out), buffer(sg.g), buffer(sg.b),
                                                residual, sg.relu, sg.h, sg.w, sg.c, N, epsilon, 0, ws, wsBytes));
      }
    }
    return VLE_Success;
  }
  if (fused) {
    const size_t wsMid = mcn_bnorm_workspace_bytes(H, W, M, N), wsOut = mcn_bnorm_workspace_bytes(Ho, Wo, Cout, N);
    STEP("conv1_fwd", c1.forward(slot("a1"), 0, slot("x"), 1, slot("f1"), none));
    void* ws = context.getWorkspace(VLDT_GPU, wsMid > wsOut ? wsMid : wsOut);
    if (!ws) return fail(context.getLastError(), "workspace");
    ABI("bn1_fwd", mcn_bnorm_forward_fused(st, buffer("r1"), buffer(m1), buffer("a1"), buffer("g1"), buffer("b1"), NULL, 1,
                                           H, W, M, N, epsilon, given, ws, wsMid));
    STEP("conv2_fwd", c2.forward(slot("a2"), 0, slot("r1"), 1, slot("f2"), none));
    ws = context.getWorkspace(VLDT_GPU, wsMid > wsOut ? wsMid : wsOut);  // (a convolution may have grown it)
    if (!ws) return fail(context.getLastError(), "workspace");
    ABI("bn2_fwd", mcn_bnorm_forward_fused(st, buffer("r2"), buffer(m2), buffer("a2"), buffer("g2"), buffer("b2"), NULL, 1,
                                           Ho, Wo, M, N, epsilon, given, ws, wsMid));
    STEP("conv3_fwd", c3.forward(slot("a3"), 0, slot("r2"), 1, slot("f3"), none));
    ws = context.getWorkspace(VLDT_GPU, wsMid > wsOut ? wsMid : wsOut);
    if (!ws) return fail(context.getLastError(), "workspace");
    ABI("bn3_fwd", mcn_bnorm_forward_fused(st, buffer("y"), buffer(m3), buffer("a3"), buffer("g3"), buffer("b3"),
                                           buffer(shortcut), 1, Ho, Wo, Cout, N, epsilon, given, ws, wsOut));
    return VLE_Success;
  }
  STEP("conv1_fwd", c1.forward(slot("a1"), 0, slot("x"), 1, slot("f1"), none));
  STEP("bn1_fwd", bnForward("n1", m1, "a1", "g1", "b1"));
  ABI("relu1_fwd", mcn_relu_forward(st, buffer("r1"), buffer("n1"), nMid));
  STEP("conv2_fwd", c2.forward(slot("a2"), 0, slot("r1"), 1, slot("f2"), none));
  STEP("bn2_fwd", bnForward("n2", m2, "a2", "g2", "b2"));
  ABI("relu2_fwd", mcn_relu_forward(st, buffer("r2"), buffer("n2"), nMidOut));
  STEP("conv3_fwd", c3.forward(slot("a3"), 0, slot("r2"), 1, slot("f3"), none));
  STEP("bn3_fwd", bnForward("n3", m3, "a3", "g3", "b3"));
  ABI("sum_fwd", mcn_add(st, buffer("s"), buffer("n3"), buffer(shortcut), nOut));
  ABI("relu3_fwd", mcn_relu_forward(st, buffer("y"), buffer("s"), nOut));
  return VLE_Success;
}

ErrorCode Bottleneck::backward() {
  if (error != VLE_Success) return error;
  if (testMode) {
    message = "backward needs the batch moments of a training-mode forward pass";
    return VLE_IllegalArgument;
  }
  void* st = context.getHipHelper().getStream();
  Tensor none;
  nn::Convolution c1(context, 1, 1, 0, 0, 0, 0, 1, 1), c2(context, stride, stride, 1, 1, 1, 1, 1, 1),
      c3(context, 1, 1, 0, 0, 0, 0, 1, 1), cs(context, stride, stride, 0, 0, 0, 0, 1, 1);
  attachPacked(c1, c2, c3, cs);
  nn::BatchNorm bn(context, epsilon);
  const std::size_t nMid = slot("a1").getNumElements(), nMidOut = slot("a2").getNumElements(),
                    nIn = slot("x").getNumElements(), nOut = slot("a3").getNumElements();
  // ReLU masks: the layer's input, or (fused mode) its output -- max(v, 0) > 0 exactly when v > 0
  char const* mask3 = fused ? "y" : "s";
  char const* mask2 = fused ? "r2" : "n2";
  char const* mask1 = fused ? "r1" : "n1";
  // The sum passes ds to both of its inputs: the branch (n3) and the shortcut.  With an identity shortcut the fused
  // mode keeps ds in the output buffer and lets the first convolution add its derivative to it.
  char const* dsName = (fused && !adapter) ? "dzdx" : "ds";

  // A convolution's backward: the input gradient on the caller's stream; the filter gradient beside it on the
  // second stream when overlapping (enqueued after it, so the persistent input-gradient kernel takes its CUs
  // first and the filter-gradient workgroups fill in beside and behind it).
  nn::Convolution c1s(sideContext, 1, 1, 0, 0, 0, 0, 1, 1), c2s(sideContext, stride, stride, 1, 1, 1, 1, 1, 1),
      css(sideContext, stride, stride, 0, 0, 0, 0, 1, 1);
  Tensor none2, none3;
  // (k: the event of the two-stream schedule; 3 - k = the layer's place in {conv1, conv2, conv3, adapter} for k < 3)
  // maskedAdd: the input gradient also takes the shortcut's share of the derivative, dzdy behind the unit's last ReLU
  // (mask bits), in its epilogue (derInMult is then 0: nothing is accumulated onto)
  auto convBackward = [&](nn::Convolution& onMain, nn::Convolution& onSide, int k, Tensor& derIn, double derInMult,
                          Tensor& derFilter, Tensor const& in, Tensor const& filter, Tensor const& derOut,
                          bool maskedAdd = false) -> ErrorCode {
    const int layer = k == 3 ? 3 : 2 - k;
    auto dataPart = [&]() -> ErrorCode {
      if (maskedAdd) return onMain.backwardDataMaskedAdd(derIn, filter, derOut, buffer("dzdy"), maskBits);
      return onMain.backwardAccumulate(derIn, derInMult, none2, none, in, filter, derOut);
    };
    if (!overlap && deferred && partialBank[layer].bytes) {
      ErrorCode ed = dataPart();
      if (ed != VLE_Success) return ed;
      return onMain.backwardFilterPartial(derFilter, in, derOut, (char*)partialArena + partialBank[layer].offset,
                                          partialBank[layer].bytes);
    }
    if (!overlap && !maskedAdd) return onMain.backwardAccumulate(derIn, derInMult, derFilter, none, in, filter, derOut);
    if (!overlap) {
      ErrorCode ed = dataPart();
      if (ed != VLE_Success) return ed;
      return onMain.backwardAccumulate(none3, 0, derFilter, none, in, filter, derOut);
    }
    if (hipEventRecord((hipEvent_t)events[k], (hipStream_t)st) != hipSuccess ||
        hipStreamWaitEvent((hipStream_t)sideStream, (hipEvent_t)events[k], 0) != hipSuccess)
      return context.setError(VLE_Cuda, "cannot order the second stream");
    ErrorCode e = dataPart();
    if (e != VLE_Success) return e;
    // (deferred: only the matrix kernel runs on the second stream, into the layer's partial banks; the sums over the
    // splits of all layers follow the join, in one launch on the caller's stream)
    if (deferred && partialBank[layer].bytes)
      e = onSide.backwardFilterPartial(derFilter, in, derOut, (char*)partialArena + partialBank[layer].offset,
                                       partialBank[layer].bytes);
    else
      e = onSide.backwardAccumulate(none3, 0, derFilter, none, in, filter, derOut);
    if (e != VLE_Success) context.setError(e, sideContext.getLastErrorMessage().c_str());
    return e;
  };
  auto joinSide = [&]() -> ErrorCode {
    // (a shared second stream is joined by its owner, unless this unit sums its own filter gradients right here)
    if (overlap && (!sideShared || (deferred && !externalSums)) &&
        (hipEventRecord((hipEvent_t)events[4], (hipStream_t)sideStream) != hipSuccess ||
         hipStreamWaitEvent((hipStream_t)st, (hipEvent_t)events[4], 0) != hipSuccess))
      return context.setError(VLE_Cuda, "cannot join the second stream");
    if (deferred && !externalSums && !sumJobs.empty()) {
      int rcSum = mcn_conv_reduce_batch(st, (mcn_conv_reduce_job const*)sumJobsDevice, (int)sumJobs.size(), sumBlocks);
      if (rcSum) return context.setError((ErrorCode)rcSum, mcn_last_error_message());
    }
    return VLE_Success;
  };

  const size_t wsMid = mcn_bnorm_workspace_bytes(H, W, M, N), wsOut = mcn_bnorm_workspace_bytes(Ho, Wo, Cout, N);
  const size_t wsBnBytes = wsMid > wsOut ? wsMid : wsOut;
  void* wsBn = NULL;
  if (fused) {
    // the unit's last ReLU sits behind the shortcut sum: its derivative is taken and written (for the shortcut
    // branch) in the summing pass of the batch-norm derivative
    wsBn = context.getWorkspace(VLDT_GPU, wsBnBytes);
    if (!wsBn) return fail(context.getLastError(), "workspace");
    if (maskBits)  // (the mask as bits; the shortcut's share of the derivative is added by the first convolution below)
      ABI("bn3_bwd", mcn_bnorm_backward_bits(st, buffer("da3"), buffer("dg3"), buffer("db3"), buffer("m3"), buffer("a3"),
                                             buffer("g3"), buffer("dzdy"), maskBits, Ho, Wo, Cout, N, epsilon, wsBn, wsOut));
    else
    ABI("bn3_bwd", mcn_bnorm_backward_masked(st, buffer("da3"), buffer("dg3"), buffer("db3"), buffer("m3"), buffer("a3"),
                                             buffer("g3"), buffer("dzdy"), buffer(mask3), buffer(dsName), Ho, Wo, Cout, N,
                                             epsilon, wsBn, wsOut));
  } else {
    ABI("relu3_bwd", mcn_relu_backward(st, buffer(dsName), buffer(mask3), buffer("dzdy"), nOut));
    STEP("bn3_bwd", bn.backwardWithMoment(slot("da3"), slot("dg3"), slot("db3"), slot("m3"), slot("a3"), slot("g3"), slot("b3"), slot(dsName)));
  }
  STEP("conv3_bwd", convBackward(c3, c1s, 0, slot("dr2"), 0, slot("df3"), slot("r2"), slot("f3"), slot("da3")));
  if (fused) {
    // ReLU's derivative folded into the batch-norm derivative that follows it: the mask is recomputed from the
    // layer's input and stored moments, the masked derivative is never written out
    wsBn = context.getWorkspace(VLDT_GPU, wsBnBytes);  // (the convolution in between may have grown the workspace)
    if (!wsBn) return fail(context.getLastError(), "workspace");
    ABI("bn2_bwd", mcn_bnorm_backward_relu(st, buffer("da2"), buffer("dg2"), buffer("db2"), buffer("m2"), buffer("a2"),
                                           buffer("g2"), buffer("b2"), buffer("dr2"), Ho, Wo, M, N, epsilon, wsBn, wsMid));
  } else {
    ABI("relu2_bwd", mcn_relu_backward(st, buffer("dn2"), buffer(mask2), buffer("dr2"), nMidOut));
    STEP("bn2_bwd", bn.backwardWithMoment(slot("da2"), slot("dg2"), slot("db2"), slot("m2"), slot("a2"), slot("g2"), slot("b2"), slot("dn2")));
  }
  STEP("conv2_bwd", convBackward(c2, c2s, 1, slot("dr1"), 0, slot("df2"), slot("r1"), slot("f2"), slot("da2")));
  if (fused) {
    wsBn = context.getWorkspace(VLDT_GPU, wsBnBytes);
    if (!wsBn) return fail(context.getLastError(), "workspace");
    ABI("bn1_bwd", mcn_bnorm_backward_relu(st, buffer("da1"), buffer("dg1"), buffer("db1"), buffer("m1"), buffer("a1"),
                                           buffer("g1"), buffer("b1"), buffer("dr1"), H, W, M, N, epsilon, wsBn, wsMid));
  } else {
    ABI("relu1_bwd", mcn_relu_backward(st, buffer("dn1"), buffer(mask1), buffer("dr1"), nMid));
    STEP("bn1_bwd", bn.backwardWithMoment(slot("da1"), slot("dg1"), slot("db1"), slot("m1"), slot("a1"), slot("g1"), slot("b1"), slot("dn1")));
  }
  if (adapter) {
    // the shortcut branch: bnorm (no ReLU) and the strided 1x1 convolution, whose input gradient opens dzdx
    STEP("bns_bwd", bn.backwardWithMoment(slot("das"), slot("dgs"), slot("dbs"), slot("ms"), slot("as"), slot("gs"), slot("bs"), slot("ds")));
    if (fused) {
      STEP("convs_bwd", convBackward(cs, css, 3, slot("dzdx"), 0, slot("dfs"), slot("x"), slot("fs"), slot("das")));
      STEP("conv1_bwd", convBackward(c1, c1s, 2, slot("dzdx"), 1, slot("df1"), slot("x"), slot("f1"), slot("da1")));
    } else {
      STEP("convs_bwd", convBackward(cs, css, 3, slot("dxm"), 0, slot("dfs"), slot("x"), slot("fs"), slot("das")));
      STEP("conv1_bwd", convBackward(c1, c1s, 2, slot("dzdx"), 0, slot("df1"), slot("x"), slot("f1"), slot("da1")));
      ABI("sum_bwd", mcn_add(st, buffer("dzdx"), buffer("dzdx"), buffer("dxm"), nIn));
    }
    STEP("join", joinSide());
    return VLE_Success;
  }
  if (fused) {
    if (maskBits) STEP("conv1_bwd", convBackward(c1, c1s, 2, slot("dzdx"), 0, slot("df1"), slot("x"), slot("f1"), slot("da1"), true));
    else STEP("conv1_bwd", convBackward(c1, c1s, 2, slot("dzdx"), 1, slot("df1"), slot("x"), slot("f1"), slot("da1")));
    STEP("join", joinSide());
    return VLE_Success;
  }
  STEP("conv1_bwd", convBackward(c1, c1s, 2, slot("dxm"), 0, slot("df1"), slot("x"), slot("f1"), slot("da1")));
  ABI("sum_bwd", mcn_add(st, buffer("dzdx"), buffer("dxm"), buffer("ds"), nIn));
  STEP("join", joinSide());
  return VLE_Success;
}

} }  // namespace vl::harness
