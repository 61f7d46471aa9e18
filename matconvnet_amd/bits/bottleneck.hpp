// ResNet bottleneck unit (forward + backward) wired directly onto the vl::nn operators, the way the reference's
// DagNN would drive them for one segment of examples/imagenet/cnn_imagenet_init_resnet.m:86-118:
//   conv1x1 C->M, bnorm, relu, conv3x3 M->M (pad 1, stride s), bnorm, relu, conv1x1 M->Cout, bnorm,
//   + shortcut, relu
// where the shortcut is the input itself, or (first segment of a section: `adapter`) conv1x1 C->Cout with
// stride s followed by bnorm.  Convolutions have no bias.  Batch-norm backward uses the moments cached by the
// forward pass (matlab/+dagnn/BatchNorm.m:27-34); derivatives of a variable with two consumers are added as
// matlab/+dagnn/Layer.m:127-135 does.
// All buffers are allocated once; a step performs no allocation.
#ifndef MCN_AMD_BITS_BOTTLENECK_HPP
#define MCN_AMD_BITS_BOTTLENECK_HPP

#include <string>
#include <vector>

#include "../../include/mcn_hip.h"
#include "data.hpp"
#include "nnconv.hpp"

namespace vl { namespace harness {

class Bottleneck {
 public:
  // H x W x C x N input, M channels inside, Cout channels out (0: same as C), stride 1 or 2 on the 3x3 layer and
  // the adapter.  `shared`: use this context (stream, workspace) instead of one of the unit's own.
  Bottleneck(int H, int W, int C, int M, int N, double epsilon, int Cout = 0, int stride = 1, bool adapter = false,
             Context* shared = NULL);
  ~Bottleneck();
  bool ok() const { return error == VLE_Success; }
  ErrorCode lastError() const { return error; }
  std::string const& lastMessage() const { return message; }

  // named device buffers: inputs "x","dzdy","f1","f2","f3","g1","b1",... (adapter: "fs","gs","bs");
  // outputs "y","dzdx","df1","dg1","db1",...; batch moments "m1",..., stored moments "rm1",...
  float* buffer(std::string const& name, std::size_t* count = NULL);
  // makes a named buffer a view of memory owned by someone else (the previous unit's output, say); the unit's own
  // allocation for it is released
  ErrorCode alias(std::string const& name, float* memory);
  ErrorCode setStream(void* stream);
  int outHeight() const { return Ho; }
  int outWidth() const { return Wo; }
  int outDepth() const { return Cout; }

  // fused = true: batch-norm forward applies the ReLU (and, for the last one, the shortcut sum) in its output
  // pass (mcn_bnorm_forward_fused), so the un-activated tensors n1, n2, n3, s are never written; in the backward
  // pass ReLU's derivatives are taken inside the batch-norm derivatives and the shortcut's fan-out sum inside the
  // first convolution's.  Results are bit-identical to the layer-by-layer mode.
  void setFused(bool on) { fused = on; }
  // overlap = true: in the backward pass each convolution's filter gradient runs on a second stream (with a
  // context and workspace of its own) beside the same layer's input gradient, which is all the following layers
  // wait for; the second stream is joined before backward() returns its work to the caller's stream.  Results are
  // the same bits; only the schedule changes.  `stream`: a second stream of the caller's, shared by several units, in
  // place of one of the unit's own; with it backward() does NOT join: the caller makes its stream wait for that
  // second stream once, after the last unit (so a unit's last filter gradient also runs beside the next unit's
  // first kernels), and before anything reads the filter gradients or rewrites the unit's activations.
  ErrorCode setOverlap(bool on, void* stream = NULL);
  // test mode: batch normalisation uses the stored moments "rm1", "rm2", "rm3" ("rms") instead of the batch's
  // (matlab/+dagnn/BatchNorm.m:12-17); forward only
  void setTestMode(bool on) { testMode = on; }
  // packed = true: the convolutions read filter banks packed ahead (mcn_conv_pack_* of the C ABI) instead of
  // packing them on every call; pack() refreshes all of the unit's banks in one launch and must be called after
  // every change of the filters (setPacked does not pack).  packJobs(): the unit's jobs, for a caller that packs
  // several units in one launch of its own.  Same bits either way.
  ErrorCode setPacked(bool on);
  ErrorCode pack();
  std::vector<mcn_conv_pack_job> const& packJobs() const { return jobs; }
  // deferred = true: backward() runs only the matrix kernels of the filter gradients and keeps their partial banks;
  // the sums over reduction splits of all the unit's layers run in one launch at the end of backward() -- or, with
  // `external`, in a launch of the caller's that covers several units (reduceJobs()).  Same bits.  Not combined with
  // setOverlap.
  ErrorCode setDeferred(bool on, bool external = false);
  std::vector<mcn_conv_reduce_job> const& reduceJobs() const { return sumJobs; }
  // epilogue sums = true (fused mode, training): the forward convolutions also sum their output per channel
  // (mcn_conv_forward_sums) and the batch normalisations that follow take those sums instead of reading the tensor
  // in a summing pass of their own (mcn_bnorm_forward_sums).  The moments then come from a different summation order
  // than the two-launch form's: same values to rounding (1e-7 relative), not the same bits.
  ErrorCode setEpilogueSums(bool on);
  // mask bits = true (with epilogue sums, identity shortcut): the unit's last ReLU leaves its mask as one bit per
  // element (mcn_bnorm_forward_sums_mask); backward reads the bits instead of the unit's output
  // (mcn_bnorm_backward_bits) and the shortcut's share of the derivative is added, masked, in the epilogue of the
  // first convolution's input gradient (mcn_conv_backward_data_masked_add) instead of being written out and read
  // back.  Same bits as without.  Stays off (returns success) where the shapes have no such form.
  ErrorCode setMaskBits(bool on);
  bool maskBitsOn() const { return maskBits != NULL; }
  ErrorCode forward();
  ErrorCode backward();

  // optional hook called around the launch(es) of one stage ("conv2_bwd", "bn3_bwd", ...) for timing
  typedef void (*StageHook)(void* user, char const* stage, int begin);
  void setStageHook(StageHook hook, void* user) { stageHook = hook; hookUser = user; }

 private:
  struct Slot { std::string name; Tensor tensor; bool owned; };
  Tensor& slot(std::string const& name);
  Tensor make(std::string const& name, TensorShape const& shape);
  ErrorCode fail(ErrorCode e, char const* where);
  void mark(char const* stage, int begin) { if (stageHook) stageHook(hookUser, stage, begin); }

  int H, W, C, M, N, Cout, stride, Ho, Wo;
  bool adapter;
  double epsilon;
  Context ownContext;
  Context& context;
  std::vector<Slot> slots;
  ErrorCode error;
  std::string message;
  StageHook stageHook;
  void* hookUser;
  bool fused;
  bool overlap;
  bool testMode;
  void attachPacked(nn::Convolution& c1, nn::Convolution& c2, nn::Convolution& c3, nn::Convolution& cs);
  struct Bank { std::size_t offset, bytes; };
  bool packed;
  Bank banks[4][2];              // [convolution][forward, backward-data]
  void* packedArena;
  void* packedJobs;              // device copy of `jobs`, numbered for the unit's own launch
  unsigned packedBlocks;
  std::vector<mcn_conv_pack_job> jobs;
  bool deferred, externalSums;
  Bank partialBank[4];           // [convolution]: its partial banks inside partialArena (bytes 0: no deferred form)
  void* partialArena;
  void* sumJobsDevice;
  unsigned sumBlocks;
  std::vector<mcn_conv_reduce_job> sumJobs;
  bool epilogueSums;
  int sumGroupsOf[4];   // [convolution]: partial sums per channel its forward writes (0: it cannot)
  void* sumsBuffer;     // the partial sums of the convolution that ran last
  unsigned* maskBits;   // one bit per element of y: what the unit's last ReLU let through (setMaskBits)
  std::size_t sumsBytes;
  Context sideContext;
  void* sideStream;     // hipStream_t
  bool sideShared;      // the second stream is the caller's: not joined and not destroyed here
  void* events[5];      // hipEvent_t: "derivative ready" for the convolutions, "second stream done"
};

} }  // namespace vl::harness
#endif
