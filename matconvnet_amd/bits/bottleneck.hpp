// ResNet-50 bottleneck block (forward + backward) wired directly onto the vl::nn operators, the way the
// reference's DagNN would drive them for the block built by examples/imagenet/cnn_imagenet_init_resnet.m:16-48:
//   conv1x1 C->M, bnorm, relu, conv3x3 M->M (pad 1), bnorm, relu, conv1x1 M->C, bnorm, + identity, relu
// Convolutions have no bias.  Batch-norm backward uses the moments cached by the forward pass
// (matlab/+dagnn/BatchNorm.m:27-34); the shortcut's derivative is added to the branch's as
// matlab/+dagnn/Layer.m:127-135 does for variables with fan-out > 1.
// All buffers are allocated once; a step performs no allocation.
#ifndef MCN_AMD_BITS_BOTTLENECK_HPP
#define MCN_AMD_BITS_BOTTLENECK_HPP

#include <string>
#include <vector>

#include "data.hpp"

namespace vl { namespace harness {

class Bottleneck {
 public:
  Bottleneck(int H, int W, int C, int M, int N, double epsilon);
  ~Bottleneck();
  bool ok() const { return error == VLE_Success; }
  ErrorCode lastError() const { return error; }
  std::string const& lastMessage() const { return message; }

  // named device buffers: inputs "x","dzdy","f1","f2","f3","g1","b1",...; outputs "y","dzdx","df1","dg1","db1",...
  float* buffer(std::string const& name, std::size_t* count = NULL);
  ErrorCode setStream(void* stream);

  // fused = true: batch-norm forward applies the ReLU (and, for the last one, the shortcut sum) in its output
  // pass (mcn_bnorm_forward_fused); the un-activated tensors n1, n2, n3, s are then never written and the
  // ReLU derivatives take their masks from r1, r2, y.  Results are bit-identical to the layer-by-layer mode.
  void setFused(bool on) { fused = on; }
  // overlap = true: in the backward pass each convolution's filter gradient runs on a second stream (with a
  // context and workspace of its own) beside the same layer's input gradient, which is all the following layers
  // wait for; the second stream is joined before backward() returns its work to the caller's stream.  Results are
  // the same bits; only the schedule changes.
  ErrorCode setOverlap(bool on);
  ErrorCode forward();
  ErrorCode backward();

  // optional hook called around the launch(es) of one stage ("conv2_bwd", "bn3_bwd", ...) for timing
  typedef void (*StageHook)(void* user, char const* stage, int begin);
  void setStageHook(StageHook hook, void* user) { stageHook = hook; hookUser = user; }

 private:
  struct Slot { std::string name; Tensor tensor; };
  Tensor& slot(std::string const& name);
  Tensor make(std::string const& name, TensorShape const& shape);
  ErrorCode fail(ErrorCode e, char const* where);
  void mark(char const* stage, int begin) { if (stageHook) stageHook(hookUser, stage, begin); }

  int H, W, C, M, N;
  double epsilon;
  Context context;
  std::vector<Slot> slots;
  ErrorCode error;
  std::string message;
  StageHook stageHook;
  void* hookUser;
  bool fused;
  bool overlap;
  Context sideContext;
  void* sideStream;     // hipStream_t
  void* events[4];      // hipEvent_t: "derivative ready" for the three convolutions, "second stream done"
};

} }  // namespace vl::harness
#endif
