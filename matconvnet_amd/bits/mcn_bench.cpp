// Stand-alone bench of the operator layer: no MATLAB, no Python.  Drives vl::nn::Convolution / BatchNorm /
// Pooling (HIP device tensors) and the bottleneck block on the benchmark configurations with seeded
// synthetic inputs, times them with HIP events and prints TFLOP/s, GB/s and images/s beside the
// fraction of the MI355X rooflines (fp32 matrix 157.3 TFLOP/s, HBM 8 TB/s).
//
//   mcn_bench [--iters K] [--warmup W] [--rotate R] [--only conv5|conv1|bnorm|maxpool|avgpool|block|blocktimed|blockoverlap|copy|yardstick|resnet50] [--batch N] [--config C] [--set tunable=value]...
//
// The bandwidth-bound operators (bnorm, pooling, copy) are timed over R independent sets of tensors used in
// turn (default 4), so that no launch finds its inputs in the 256 MB memory-side cache because the previous
// launch left them there: with R sets, more than 256 MB of other traffic passes between two uses of a buffer.
// --rotate 1 gives the warm figure a loop over one set of buffers shows.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <random>
#include <string>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "bottleneck.hpp"
#include "hiphelper.hpp"
#include "nnbnorm.hpp"
#include "nnconv.hpp"
#include "nnpooling.hpp"
#include "resnet.hpp"
#include "../../include/mcn_hip.h"

using namespace vl;

static const double kPeakMfma = 157.3e12, kPeakHbm = 8.0e12;

#define HIP_OK(call)                                                                  \
  do {                                                                                \
    hipError_t e_ = (call);                                                           \
    if (e_ != hipSuccess) {                                                           \
      std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));          \
      std::exit(2);                                                                   \
    }                                                                                 \
  } while (0)

struct DeviceTensor {
  Tensor view;
  DeviceTensor(TensorShape const& shape) {
    void* p = NULL;
    HIP_OK(hipMalloc(&p, std::max<size_t>(shape.getNumElements(), 1) * sizeof(float)));
    view = Tensor(shape, VLDT_Float, VLDT_GPU, p, shape.getNumElements() * sizeof(float));
  }
  ~DeviceTensor() { (void)hipFree(view.getMemory()); }
  void randn(unsigned seed, float scale = 1.f, float shift = 0.f) {
    std::mt19937_64 gen(seed);
    std::normal_distribution<float> dist(0.f, 1.f);
    std::vector<float> host(view.getNumElements());
    for (size_t i = 0; i < host.size(); ++i) host[i] = shift + scale * dist(gen);
    HIP_OK(hipMemcpy(view.getMemory(), host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice));
  }
  void fill(float v) {
    std::vector<float> host(view.getNumElements(), v);
    HIP_OK(hipMemcpy(view.getMemory(), host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice));
  }
};

static int gRotate = 4;

// R device tensors of one shape holding the same values
struct TensorSet {
  std::vector<std::unique_ptr<DeviceTensor>> t;
  TensorSet(TensorShape const& shape, int count) {
    for (int i = 0; i < count; ++i) t.emplace_back(new DeviceTensor(shape));
  }
  void spread() {
    for (size_t i = 1; i < t.size(); ++i)
      HIP_OK(hipMemcpy(t[i]->view.getMemory(), t[0]->view.getMemory(), t[0]->view.getNumElements() * sizeof(float),
                       hipMemcpyDeviceToDevice));
  }
  DeviceTensor& first() { return *t[0]; }
  Tensor& operator[](int i) { return t[i % t.size()]->view; }
};

template <typename F>
static double medianMs(F&& body, int warmup, int iters, hipStream_t stream = 0) {
  hipEvent_t a, b;
  HIP_OK(hipEventCreate(&a));
  HIP_OK(hipEventCreate(&b));
  for (int i = 0; i < warmup; ++i) body();
  HIP_OK(hipDeviceSynchronize());
  std::vector<float> ms(iters);
  for (int i = 0; i < iters; ++i) {
    HIP_OK(hipEventRecord(a, stream));
    body();
    HIP_OK(hipEventRecord(b, stream));
    HIP_OK(hipEventSynchronize(b));
    HIP_OK(hipEventElapsedTime(&ms[i], a, b));
  }
  std::sort(ms.begin(), ms.end());
  hipEventDestroy(a);
  hipEventDestroy(b);
  return ms[iters / 2];
}

static void check(Context& ctx, ErrorCode e, char const* what) {
  if (e != VLE_Success) {
    std::fprintf(stderr, "%s: %s\n", what, ctx.getLastErrorMessage().c_str());
    std::exit(3);
  }
}

static void benchConv(char const* name, int H, int W, int C, int N, int F, int K, int pad, int warmup, int iters, int stride = 1) {
  Context ctx;
  const int OH = (H + 2 * pad - F) / stride + 1, OW = (W + 2 * pad - F) / stride + 1;
  DeviceTensor x(TensorShape(H, W, C, N)), f(TensorShape(F, F, C, K)), dy(TensorShape(OH, OW, K, N));
  DeviceTensor dx(TensorShape(H, W, C, N)), df(TensorShape(F, F, C, K)), db(TensorShape(K, 1, 1, 1));
  x.randn(1);
  f.randn(2, std::sqrt(2.f / (F * F * C)));
  dy.randn(3);
  nn::Convolution op(ctx, stride, stride, pad, pad, pad, pad, 1, 1);
  Tensor none;
  const double flops = 2.0 * OH * OW * (double)F * F * C * K * N;
  double tData = medianMs([&] { check(ctx, op.backward(dx.view, none, none, none, f.view, dy.view), name); }, warmup, iters);
  double tFilt = medianMs([&] { check(ctx, op.backward(none, df.view, none, x.view, none, dy.view), name); }, warmup, iters);
  double tBias = medianMs([&] { check(ctx, op.backward(none, none, db.view, none, none, dy.view), name); }, warmup, iters);
  double tAll = medianMs([&] { check(ctx, op.backward(dx.view, df.view, db.view, x.view, f.view, dy.view), name); }, warmup, iters);
  std::printf("%-28s bwd-data %8.3f ms %6.1f TFLOP/s (%4.1f%%) | bwd-filter %8.3f ms %6.1f TFLOP/s (%4.1f%%) | bias %6.1f us | all three %8.3f ms %6.1f TFLOP/s (%4.1f%% of fp32 MFMA peak)\n",
              name, tData, flops / tData / 1e9, 100 * flops / (tData * 1e-3) / kPeakMfma, tFilt, flops / tFilt / 1e9,
              100 * flops / (tFilt * 1e-3) / kPeakMfma, tBias * 1e3, tAll, 2 * flops / tAll / 1e9,
              100 * 2 * flops / (tAll * 1e-3) / kPeakMfma);
}

static void benchBnorm(int warmup, int iters) {
  const int H = 56, W = 56, C = 256, N = 32;
  Context ctx;
  TensorSet x(TensorShape(H, W, C, N), gRotate), dy(TensorShape(H, W, C, N), gRotate), dx(TensorShape(H, W, C, N), gRotate);
  DeviceTensor g(TensorShape(C, 1, 1, 1)), b(TensorShape(C, 1, 1, 1)), dg(TensorShape(C, 1, 1, 1)), db(TensorShape(C, 1, 1, 1)), m(TensorShape(C, 2, 1, 1));
  x.first().randn(4, 1.3f, 0.5f);
  dy.first().randn(5);
  x.spread();
  dy.spread();
  g.fill(1.f);
  b.fill(0.f);
  nn::BatchNorm op(ctx, 1e-4);
  const double bytes = 5.0 * H * W * C * N * 4;
  int turn = 0;
  double t = medianMs([&] {
    check(ctx, op.backward(dx[turn], dg.view, db.view, m.view, x[turn], g.view, b.view, dy[turn]), "bnorm");
    ++turn;
  }, warmup, iters);
  std::printf("%-28s %8.1f us %7.0f GB/s (%4.1f%% of HBM peak; 5 tensor sweeps = %.1f MB; %d buffer sets in turn)\n",
              "bnorm bwd 56x56x256x32", t * 1e3, bytes / t / 1e6, 100 * bytes / (t * 1e-3) / kPeakHbm, bytes / 1e6, gRotate);
}

static void benchPool(bool isMax, int warmup, int iters) {
  const int H = isMax ? 112 : 56, C = isMax ? 64 : 256, N = 32, P = isMax ? 3 : 2, pad = isMax ? 1 : 0;
  const int OH = (H + 2 * pad - P) / 2 + 1;
  Context ctx;
  TensorSet x(TensorShape(H, H, C, N), gRotate), dy(TensorShape(OH, OH, C, N), gRotate), dx(TensorShape(H, H, C, N), gRotate);
  x.first().randn(6);
  dy.first().randn(7);
  x.spread();
  dy.spread();
  nn::Pooling op(ctx, P, P, 2, 2, pad, pad, pad, pad, isMax ? nn::Pooling::Max : nn::Pooling::Average);
  const double e = (double)H * H * C * N * 4, o = (double)OH * OH * C * N * 4;
  const double bytes = isMax ? (2 * e + o) : (e + o);
  int turn = 0;
  double t = medianMs([&] {
    check(ctx, op.backwardOverwrite(dx[turn], x[turn], dy[turn]), "pool");
    ++turn;
  }, warmup, iters);
  std::printf("%-28s %8.1f us %7.0f GB/s (%4.1f%% of HBM peak; %.1f MB; %d buffer sets in turn)\n",
              isMax ? "max-pool bwd 112x112x64x32" : "avg-pool bwd 56x56x256x32", t * 1e3, bytes / t / 1e6,
              100 * bytes / (t * 1e-3) / kPeakHbm, bytes / 1e6, gRotate);
}

// A plain streaming copy of known size (ReLU of positive data): the yardstick the HBM byte counters of the
// other kernels are scaled by.
static void benchCopy(int warmup, int iters) {
  const size_t n = 64u << 20;  // 64 Mi floats: reads 256 MiB, writes 256 MiB
  TensorSet a(TensorShape(n, 1, 1, 1), gRotate), b(TensorShape(n, 1, 1, 1), gRotate);
  a.first().fill(1.f);
  a.spread();
  int turn = 0;
  double t = medianMs([&] {
    mcn_relu_forward(NULL, (float*)b[turn].getMemory(), (float const*)a[turn].getMemory(), n);
    ++turn;
  }, warmup, iters);
  std::printf("%-28s %8.1f us %7.0f GB/s (%4.1f%% of HBM peak; reads %zu B, writes %zu B per launch; %d buffer sets in turn)\n",
              "copy 256 MiB", t * 1e3, 2.0 * n * 4 / t / 1e6, 100 * 2.0 * n * 4 / (t * 1e-3) / kPeakHbm, n * 4, n * 4, gRotate);
}

// Sweep of the plain streaming kernels (read-only, write-only, copy) over launch shapes: workgroups per compute
// unit (0 = one step per workgroup, not persistent), 16-byte accesses in flight per lane, walk (slab by slab over the
// whole chip, or one contiguous run per workgroup), store hint, access width.  256 MiB per stream, buffer sets used in
// turn like the operators' measurements.  The best line of each mode is the measured ceiling of that traffic mix.
// `fixed` >= 0: run only that one configuration (for counter runs): mode*1000 + perCu*100 + inFlight*10 + flags.
static void benchYardstick(int warmup, int iters, int fixed) {
  const size_t bytes = 256u << 20;
  TensorSet a(TensorShape(bytes / 4, 1, 1, 1), gRotate), b(TensorShape(bytes / 4, 1, 1, 1), gRotate);
  a.first().fill(1.f);
  a.spread();
  const int cus = mcn_device_compute_units();
  char const* modeName[3] = {"read", "write", "copy"};
  struct Best { double gbs; char text[160]; } best[3] = {{0, ""}, {0, ""}, {0, ""}};
  const int perCuList[] = {0, 2, 4, 8, 16, 32};
  for (int mode = 0; mode < 3; ++mode)
    for (int width : {16, 4})
      for (int perCu : perCuList)
        for (int inFlight : {1, 2, 4, 8})
          for (int flags = 0; flags < 4; ++flags) {
            if (mode == MCN_YARDSTICK_READ && (flags & MCN_YARDSTICK_NONTEMPORAL)) continue;
            if (perCu == 0 && (flags & MCN_YARDSTICK_CHUNKED)) continue;
            if (width == 4 && (perCu == 2 || perCu == 32 || inFlight == 1)) continue;  // (a thinner sweep of the narrow accesses)
            if (fixed >= 0 && (fixed != mode * 1000 + perCu * 100 + inFlight * 10 + flags || width != 16)) continue;
            int turn = 0;
            double t = medianMs([&] {
              int rc = mcn_hbm_yardstick(NULL, b[turn].getMemory(), a[turn].getMemory(), bytes, mode, width, inFlight,
                                         perCu * cus, flags);
              if (rc) {
                std::fprintf(stderr, "yardstick: %s\n", mcn_last_error_message());
                std::exit(3);
              }
              ++turn;
            }, warmup, iters);
            const double moved = (mode == MCN_YARDSTICK_COPY ? 2.0 : 1.0) * bytes;
            const double gbs = moved / t / 1e6;
            char line[160];
            std::snprintf(line, sizeof line, "%-5s width %2d B  workgroups/CU %2d  in flight %d  %-10s %-12s %8.1f us %7.0f GB/s (%4.1f%% of 8 TB/s)",
                          modeName[mode], width, perCu, inFlight, (flags & MCN_YARDSTICK_CHUNKED) ? "chunked" : "slab-wise",
                          (flags & MCN_YARDSTICK_NONTEMPORAL) ? "non-temporal" : "", t * 1e3, gbs, 100 * gbs * 1e9 / kPeakHbm);
            std::printf("%s\n", line);
            if (gbs > best[mode].gbs) {
              best[mode].gbs = gbs;
              std::strcpy(best[mode].text, line);
            }
          }
  for (int mode = 0; mode < 3; ++mode)
    if (best[mode].gbs > 0) std::printf("best %s\n", best[mode].text);
}

// sums: (with packed) the forward convolutions sum their output per channel and the last ReLU's mask is kept as bits:
// the schedule bench.py times
static void benchBlock(int warmup, int iters, bool fused, bool overlap = false, bool packed = false, bool sums = false) {
  const int H = 56, W = 56, C = 256, M = 64, N = 32;
  harness::Bottleneck block(H, W, C, M, N, 1e-5);
  block.setFused(fused);
  if (overlap) block.setOverlap(true);
  if (!block.ok()) {
    std::fprintf(stderr, "bottleneck: %s\n", block.lastMessage().c_str());
    std::exit(3);
  }
  std::mt19937_64 gen(8);
  std::normal_distribution<float> dist(0.f, 1.f);
  auto upload = [&](char const* name, float scale, float constant, bool random) {
    size_t n = 0;
    float* p = block.buffer(name, &n);
    std::vector<float> host(n);
    for (size_t i = 0; i < n; ++i) host[i] = random ? scale * dist(gen) : constant;
    HIP_OK(hipMemcpy(p, host.data(), n * sizeof(float), hipMemcpyHostToDevice));
  };
  upload("x", 1, 0, true);
  upload("dzdy", 1, 0, true);
  upload("f1", std::sqrt(2.f / C), 0, true);
  upload("f2", std::sqrt(2.f / (9 * M)), 0, true);
  upload("f3", std::sqrt(2.f / M), 0, true);
  for (char const* g : {"g1", "g2", "g3"}) upload(g, 0, 1.f, false);
  for (char const* b : {"b1", "b2", "b3"}) upload(b, 0, 0.f, false);
  if (packed && (block.setPacked(true) != VLE_Success || block.setDeferred(true) != VLE_Success)) {
    std::fprintf(stderr, "bottleneck: %s\n", block.lastMessage().c_str());
    std::exit(3);
  }
  if (sums && (block.setEpilogueSums(true) != VLE_Success || block.setMaskBits(true) != VLE_Success)) {
    std::fprintf(stderr, "bottleneck: %s\n", block.lastMessage().c_str());
    std::exit(3);
  }
  double t = medianMs([&] {
    // (packed: the banks are re-packed every step, as they would be after an update of the filters: one launch)
    if (block.pack() != VLE_Success || block.forward() != VLE_Success || block.backward() != VLE_Success) {
      std::fprintf(stderr, "bottleneck: %s\n", block.lastMessage().c_str());
      std::exit(3);
    }
  }, warmup, iters);
  std::printf("%-28s %8.3f ms/step %9.0f images/s (fwd+bwd, N = %d, 41.93 GFLOP of convolution per step; %s)\n",
              "resnet-50 bottleneck 56x56", t, N / (t * 1e-3), N, sums && overlap ? "folded, banks packed by one launch, filter gradients on a second stream and summed by one launch, channel sums from the convolutions, last mask as bits"
                     : sums ? "folded, banks packed by one launch, filter gradients summed by one, channel sums from the convolutions, last mask as bits"
                     : packed ? "folded, filter banks packed by one launch per step, filter gradients summed by one"
                     : (overlap ? "folded, filter gradients on a second stream" : (fused ? "relu/sum folded into bnorm" : "layer by layer")));
}

// Whole ResNet-50 (224 x 224 images, 1000 classes): forward alone (training-mode batch normalisation: moments are
// computed, nothing is merged into the filters) and forward + backward.
static bool gTwoStreams = false;  // --two-streams: the network's filter gradients on a second stream

static void benchResNet(int warmup, int iters, int N, bool fused) {
  harness::ResNet50 net(N, 1e-5, 224, 1000);
  if (!net.ok() || net.initParameters(11) != VLE_Success) {
    std::fprintf(stderr, "resnet-50: %s\n", net.lastMessage().c_str());
    std::exit(3);
  }
  net.setFused(fused);
  // (the folded run also packs the filter banks ahead, once per update)
  if (fused && (net.setPacked(true) != VLE_Success || net.setChannelSums(true) != VLE_Success)) {
    std::fprintf(stderr, "resnet-50: %s\n", net.lastMessage().c_str());
    std::exit(3);
  }
  if (fused && gTwoStreams && net.setOverlap(true) != VLE_Success) {
    std::fprintf(stderr, "resnet-50: %s\n", net.lastMessage().c_str());
    std::exit(3);
  }
  {
    std::mt19937_64 gen(12);
    std::normal_distribution<float> dist(0.f, 1.f);
    for (char const* name : {"input", "dprediction"}) {
      size_t n = 0;
      float* p = net.buffer(name, &n);
      std::vector<float> host(n);
      for (size_t i = 0; i < n; ++i) host[i] = dist(gen);
      HIP_OK(hipMemcpy(p, host.data(), n * sizeof(float), hipMemcpyHostToDevice));
    }
  }
  {
    // one class number per image for the loss layers
    size_t n = 0;
    float* p = net.buffer("labels", &n);
    std::vector<float> host(n);
    for (size_t i = 0; i < n; ++i) host[i] = (float)(1 + (i * 37) % 1000);
    HIP_OK(hipMemcpy(p, host.data(), n * sizeof(float), hipMemcpyHostToDevice));
  }
  auto stop = [&] {
    std::fprintf(stderr, "resnet-50: %s\n", net.lastMessage().c_str());
    std::exit(3);
  };
  double tf = medianMs([&] { if (net.forward() != VLE_Success) stop(); }, warmup, iters);
  double t = medianMs([&] { if (net.forward() != VLE_Success || net.backward() != VLE_Success) stop(); }, warmup, iters);
  double ts = medianMs([&] {
    if (net.forward() != VLE_Success || net.lossDerivative() != VLE_Success || net.backward() != VLE_Success ||
        net.sgdStep(1e-3, 0.9, 1e-4) != VLE_Success) stop();
  }, warmup, iters);
  // the same training step and evaluation pass replayed from HIP graphs (recorded on a stream of the network's own)
  hipStream_t own = NULL;
  HIP_OK(hipStreamCreateWithFlags(&own, hipStreamNonBlocking));
  HIP_OK(hipDeviceSynchronize());
  net.setStream(own);
  double tsg = 0, teg = 0;
  if (net.forward() != VLE_Success || net.backward() != VLE_Success || net.sgdStep(1e-3, 0.9, 1e-4) != VLE_Success ||
      net.capture(true, 1e-3, 0.9, 1e-4) != VLE_Success) stop();
  tsg = medianMs([&] { if (net.replay() != VLE_Success) stop(); }, warmup, iters, own);
  // evaluation: batch normalisation with the moving averages the training steps above have produced
  net.setTestMode(true);
  double te = medianMs([&] { if (net.forward() != VLE_Success) stop(); }, warmup, iters, own);
  if (net.capture(false) != VLE_Success) stop();
  teg = medianMs([&] { if (net.replay() != VLE_Success) stop(); }, warmup, iters, own);
  net.setTestMode(false);
  HIP_OK(hipStreamSynchronize(own));
  net.setStream(NULL);
  const double gf = net.convForwardFlopsPerImage() * 1e-9;
  std::printf("%-28s %8.2f ms evaluation (stored moments) %8.0f images/s %6.1f TFLOP/s | replayed from a HIP graph: evaluation "
              "%8.2f ms %8.0f images/s, training step %8.2f ms %8.0f images/s\n", "resnet-50 224x224", te,
              N / (te * 1e-3), gf * N / te, teg, N / (teg * 1e-3), tsg, N / (tsg * 1e-3));
  std::printf("%-28s %8.2f ms forward  %8.0f images/s %6.1f TFLOP/s | %8.2f ms fwd+bwd %8.0f images/s %6.1f TFLOP/s | "
              "%8.2f ms training step (with the loss derivative and the SGD update of %.1f M parameters) %8.0f images/s "
              "(N = %d, %.2f GFLOP of convolution per image forward; %s)\n",
              "resnet-50 224x224", tf, N / (tf * 1e-3), gf * N / tf, t, N / (t * 1e-3), 3 * gf * N / t, ts,
              net.numParameters() * 1e-6, N / (ts * 1e-3), N, gf, fused ? (gTwoStreams ? "relu/sum folded into bnorm, filter banks packed once per update, channel sums from the convolutions and mask bits where the shapes allow, filter gradients on a second stream"
                                                   : "relu/sum folded into bnorm, filter banks packed once per update, channel sums from the convolutions and mask bits where the shapes allow") : "layer by layer");
}

int main(int argc, char** argv) {
  int iters = 20, warmup = 3, batch = 32, fixed = -1;
  std::string only;
  for (int i = 1; i < argc; ++i) {
    if (!std::strcmp(argv[i], "--iters") && i + 1 < argc) iters = std::atoi(argv[++i]);
    else if (!std::strcmp(argv[i], "--warmup") && i + 1 < argc) warmup = std::atoi(argv[++i]);
    else if (!std::strcmp(argv[i], "--only") && i + 1 < argc) only = argv[++i];
    else if (!std::strcmp(argv[i], "--batch") && i + 1 < argc) batch = std::max(1, std::atoi(argv[++i]));
    else if (!std::strcmp(argv[i], "--rotate") && i + 1 < argc) gRotate = std::max(1, std::atoi(argv[++i]));
    else if (!std::strcmp(argv[i], "--config") && i + 1 < argc) fixed = std::atoi(argv[++i]);
    else if (!std::strcmp(argv[i], "--two-streams")) gTwoStreams = true;
    else if (!std::strcmp(argv[i], "--set") && i + 1 < argc && std::strchr(argv[i + 1], '=')) {
      // a tunable of the back-end (mcn_set_tunable), as name=value
      std::string kv = argv[++i];
      const size_t eq = kv.find('=');
      if (mcn_set_tunable(kv.substr(0, eq).c_str(), std::atoi(kv.c_str() + eq + 1)) != 0) {
        std::fprintf(stderr, "mcn_bench: %s\n", mcn_last_error_message());
        return 1;
      }
    }
    else {
      std::fprintf(stderr, "usage: mcn_bench [--iters K] [--warmup W] [--rotate R] [--only conv5|conv1|bnorm|maxpool|avgpool|block|blocktimed|blockoverlap|copy|yardstick|resnet50] [--batch N] [--config C] [--two-streams] [--set tunable=value]...\n");
      return 1;
    }
  }
  hipDeviceProp_t prop;
  HIP_OK(hipGetDeviceProperties(&prop, 0));
  std::printf("device: %s, %d CUs, %.0f MHz\n", prop.name, prop.multiProcessorCount, prop.clockRate / 1000.0);
  auto want = [&](char const* k) { return only.empty() || only == k; };
  if (only == "copy") benchCopy(warmup, iters);
  if (only == "yardstick") benchYardstick(warmup, iters, fixed);
  if (only == "resnet50") {
    benchResNet(warmup, iters, batch, false);
    benchResNet(warmup, iters, batch, true);
  }
  if (want("conv1")) benchConv("conv 5x5x3x32 on 32x32x3x100", 32, 32, 3, 100, 5, 32, 2, warmup, iters);
  if (only == "stem") benchConv("conv 7x7x3x64 /2 on 224x224x3x32", 224, 224, 3, 32, 7, 64, 3, warmup, iters, 2);
  if (want("bnorm")) benchBnorm(warmup, iters);
  if (want("maxpool")) benchPool(true, warmup, iters);
  if (want("avgpool")) benchPool(false, warmup, iters);
  if (want("block")) {
    benchBlock(warmup, iters, false);
    benchBlock(warmup, iters, true);
    benchBlock(warmup, iters, true, true);
    benchBlock(warmup, iters, true, false, true);
    benchBlock(warmup, iters, true, false, true, true);
    benchBlock(warmup, iters, true, true, true, true);
  }
  if (only == "blocktimed") benchBlock(warmup, iters, true, false, true, true);
  if (only == "blockoverlap") benchBlock(warmup, iters, true, true, true, true);
  if (want("conv5")) benchConv("conv 3x3x256x256 56x56 N=64", 56, 56, 256, 64, 3, 256, 1, warmup, iters);
  return 0;
}
