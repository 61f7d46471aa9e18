// ResNet-50 forward + backward on the vl::nn operators: the network that
// examples/imagenet/cnn_imagenet_init_resnet.m:52-134 builds (without the loss layers: the derivative with respect
// to the prediction is an input).
//   conv 7x7/2 3->64, bnorm, relu, max-pool 3x3/2 pad 1
//   sections 2..5 of 3, 4, 6, 3 bottleneck segments, 64/128/256/512 channels inside and 4x that out; the first
//   segment of a section has the conv + bnorm adapter on its shortcut and, from section 3 on, stride 2
//   average pooling over the remaining extent (7x7 for 224x224 images), 1x1 convolution 2048 -> classes with bias
// Training follows examples/cnn_train_dag.m:316-364: SGD with momentum and weight decay on filters, gains and biases
// (rates of examples/imagenet/cnn_imagenet_init_resnet.m:178-192), a moving average of the batch moments.  All
// parameters live in one arena (values), their derivatives in a second, the momentum in a third, so that the update is
// one launch over everything instead of three per parameter.
// All buffers are allocated at construction; a step performs no allocation.
#ifndef MCN_AMD_BITS_RESNET_HPP
#define MCN_AMD_BITS_RESNET_HPP

#include <string>
#include <vector>

#include "bottleneck.hpp"
#include "data.hpp"

namespace vl { namespace harness {

class ResNet50 {
 public:
  // imageSize: input height = width (a multiple of 32); 224 gives the reference network
  ResNet50(int N, double epsilon, int imageSize = 224, int classes = 1000);
  ~ResNet50();
  bool ok() const { return error == VLE_Success; }
  std::string const& lastMessage() const { return message; }

  // "input" (S x S x 3 x N), "prediction" / "dprediction" (1 x 1 x classes x N), the stem's "stem.f", "stem.g",
  // "stem.b" and their derivatives "stem.df", ..., the classifier's "fc.f", "fc.b", "fc.df", "fc.db", and every
  // buffer of segment i (0-based, in network order) as "unit<i>.<name>" (see Bottleneck::buffer); the momentum of a
  // parameter as "momentum.<parameter>" ("momentum.unit3.f2") and the moving average of a batch normalisation's
  // moments as "running.<moments>" ("running.stem.m", "running.unit3.m1")
  float* buffer(std::string const& name, std::size_t* count = NULL);
  int numUnits() const { return (int)units.size(); }
  ErrorCode setStream(void* stream);
  void setFused(bool on);
  // test mode: every batch normalisation uses the moving averages "running.*" instead of the batch's moments
  // (matlab/+dagnn/BatchNorm.m:12-17), as evaluation of a trained network does; forward only
  void setTestMode(bool on);
  // He-normal filters (matlab/+dagnn/Conv.m:40 style), gains 1, biases 0, from a seeded generator on the host
  ErrorCode initParameters(unsigned long long seed);
  // packed = true: every convolution reads filter banks packed ahead; pack() refreshes them all in ONE launch.
  // sgdStep() and initParameters() end with pack(); a caller that writes filters itself (through buffer()) calls it.
  ErrorCode setPacked(bool on);
  ErrorCode pack();
  // deferred = true: backward() runs the matrix kernels of all filter gradients and sums their reduction splits in ONE
  // launch at its end instead of one per layer.  Same bits.
  ErrorCode setDeferred(bool on);
  // channel sums = true (folded mode, training): units with an identity shortcut whose planes are whole mask words
  // (the 56x56 section) keep their last ReLU's mask as one bit per element, and their forward convolutions sum their
  // own output per channel for the batch normalisation that follows (Bottleneck::setEpilogueSums, setMaskBits).  The
  // moments of those units then come from another summation order: same values to rounding, not the same bits.
  ErrorCode setChannelSums(bool on);
  // overlap = true: in backward() the filter gradients of every unit run on a second stream of the network's, beside
  // the kernels that follow them on the network's own stream (the batch-norm derivatives of the layer below, the next
  // unit's first kernels); the network's stream waits for the second one once, at the end of backward() (before the
  // sums over the reduction splits when those are deferred).  Same bits; only the schedule changes.
  ErrorCode setOverlap(bool on);
  ErrorCode forward();
  ErrorCode backward();
  // The network's last layers (cnn_imagenet_init_resnet.m:128-139): from "prediction" and "labels" (one class number
  // 1..classes per image, as floats; 0 = skip the image), lossDerivative() writes "dprediction" = the derivative of
  // derOutput * (softmax log-loss, normalised by the batch size) -- what backward() starts from in training -- and
  // losses() returns that loss and the top-1 / top-5 error rates of the batch (it waits for the stream).
  ErrorCode lossDerivative(double derOutput = 1.0);
  ErrorCode losses(double* objective, double* top1Error, double* top5Error);
  // one update of all parameters from the derivatives backward() left (numWorkers = 1), and of the moving averages of
  // the moments from those forward() left
  ErrorCode sgdStep(double learningRate, double momentum, double weightDecay);
  std::size_t numParameters() const { return parameterCount; }
  // Records forward() -- and, when `training`, backward() and sgdStep(...) behind it -- on the network's stream into a
  // HIP graph; replay() launches that graph, which saves the host's per-launch work (several hundred launches per
  // step, many of them a few microseconds long).  The network's stream must not be the default stream; the recorded
  // work must have run once eagerly beforehand (so that the workspace has its final size: capture cannot allocate);
  // rates, modes (fused, test) and buffers are those at capture time -- capture again after changing any.
  ErrorCode capture(bool training, double learningRate = 0, double momentum = 0, double weightDecay = 0);
  ErrorCode replay();
  // forward FLOPs of all convolutions per image (2 per multiply-add); backward is twice that, minus the stem's dzdx
  double convForwardFlopsPerImage() const { return flops; }

 private:
  struct Slot { std::string name; Tensor tensor; bool owned; };
  struct Param { std::string name, der; std::size_t count, offset; double learningRate, weightDecay; };
  struct Moments { std::string name; std::size_t count, offset; };
  void view(std::string const& name, TensorShape const& shape, float* memory);
  ErrorCode buildArenas();
  Tensor& slot(std::string const& name);
  Tensor make(std::string const& name, TensorShape const& shape);
  ErrorCode fail(ErrorCode e, char const* where);

  int N, S, classes;
  double epsilon;
  bool fused, testMode;
  Context context;
  std::vector<Slot> slots;
  std::vector<Bottleneck*> units;
  ErrorCode error;
  std::string message;
  double flops;
  std::vector<Param> params;
  std::vector<Moments> moments;
  float *values, *ders, *state, *batchMoments, *runningMoments;
  unsigned short* chunkParam;   // device
  double* rates;                // device
  std::size_t chunks, momentsCount, parameterCount;
  bool deferred;
  void *partialArena, *sumJobsDevice;   // partial banks of the stem and the classifier; device table of all summing jobs
  std::size_t stemPartialBytes, fcPartialBytes;
  int sumJobCount;
  unsigned sumBlocks;
  bool packed;
  void *packedArena, *packedJobs;   // banks of the stem and the classifier; device table of all the network's jobs
  std::size_t stemBytes, fcForwardBytes, fcBackwardBytes, fcBackwardOffset;
  int packedJobCount;
  unsigned packedBlocks;
  void *graph, *graphExec;      // hipGraph_t, hipGraphExec_t
  bool overlap;
  void *sideStream, *sideDone;  // hipStream_t, hipEvent_t: the second stream of setOverlap and "its work is done"
  void dropGraph();
};

} }  // namespace vl::harness
#endif
