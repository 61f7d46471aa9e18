// vl::nn::BatchNorm on the HIP device (reference semantics: matlab/src/bits/nnbnorm.cu:46-365).
#include "nnbnorm.hpp"

#include "impl/dispatcher.hpp"

using namespace vl;
using namespace vl::nn;
using namespace vl::impl;

BatchNorm::BatchNorm(Context& context, double epsilon) : context(context), epsilon(epsilon) {}

namespace {

struct Extents { int H, W, C, N; };

Extents extentsOf(Tensor const& t) {
  Extents e = {asInt(t.getHeight()), asInt(t.getWidth()), asInt(t.getDepth()), asInt(t.getSize())};
  return e;
}

ErrorCode checkParameters(Context& context, char const* op, Extents const& e, Tensor const& multiplier,
                          Tensor const& bias, Tensor const& moment, bool momentRequired) {
  if (!multiplier || multiplier.getNumElements() != (size_t)e.C)
    return context.setError(VLE_IllegalArgument, (std::string(op) + ": the number of MULTIPLIERS is not the same as the number of channels").c_str());
  if (bias && bias.getNumElements() != (size_t)e.C)
    return context.setError(VLE_IllegalArgument, (std::string(op) + ": the number of BIASES is not the same as the number of channels").c_str());
  if (momentRequired && !moment)
    return context.setError(VLE_IllegalArgument, (std::string(op) + ": MOMENTS are required").c_str());
  if (moment && moment.getNumElements() != 2 * (size_t)e.C)
    return context.setError(VLE_IllegalArgument, (std::string(op) + ": MOMENTS does not have 2 x (number of channels) elements").c_str());
  return VLE_Success;
}

ErrorCode forwardAny(BatchNorm& op, char const* name, Tensor& output, Tensor const& moment, Tensor const& input,
                     Tensor const& multiplier, Tensor const& bias, bool given) {
  Context& context = op.context;
  tensor_type tt = findTensorType(output, moment, input, multiplier, bias);
  bool isDouble;
  ErrorCode e = requireHip(context, tt, name, &isDouble);
  if (e != VLE_Success) return e;
  if (!output || !input || !bias) return context.setError(VLE_IllegalArgument, (std::string(name) + ": OUTPUT, INPUT and BIASES are required").c_str());
  Extents x = extentsOf(input);
  if ((e = checkParameters(context, name, x, multiplier, bias, moment, given)) != VLE_Success) return e;
  if (isDouble) {
    const size_t need = moment ? 0 : 2 * (size_t)x.C * sizeof(double);
    void* scratch = need ? context.getWorkspace(VLDT_GPU, need) : NULL;
    if (need && !scratch) return context.getLastError();
    int rc64 = mcn_bnorm_forward_f64(context.getHipHelper().getStream(), (double*)output.getMemory(),
                                     (double*)const_cast<void*>(moment.getMemory()), (double const*)input.getMemory(),
                                     (double const*)multiplier.getMemory(), (double const*)bias.getMemory(), x.H, x.W, x.C,
                                     x.N, op.epsilon, given ? 1 : 0, scratch, need);
    return fromAbi(context, rc64, name);
  }
  const size_t bytes = mcn_bnorm_workspace_bytes(x.H, x.W, x.C, x.N);
  void* ws = bytes ? context.getWorkspace(VLDT_GPU, bytes) : NULL;
  if (bytes && !ws) return context.getLastError();
  int rc = mcn_bnorm_forward(context.getHipHelper().getStream(), (float*)output.getMemory(),
                             (float*)const_cast<void*>(moment.getMemory()), (float const*)input.getMemory(),
                             (float const*)multiplier.getMemory(), (float const*)bias.getMemory(), x.H, x.W, x.C, x.N,
                             op.epsilon, given ? 1 : 0, ws, bytes);
  return fromAbi(context, rc, name);
}

ErrorCode backwardAny(BatchNorm& op, char const* name, Tensor& derInput, Tensor& derMultiplier, Tensor& derBias,
                      Tensor const& moment, Tensor const& input, Tensor const& multiplier, Tensor const& bias,
                      Tensor const& derOutput, bool given) {
  Context& context = op.context;
  tensor_type tt = findTensorType(derInput, derMultiplier, derBias, moment, input, multiplier, bias, derOutput);
  bool isDouble;
  ErrorCode e = requireHip(context, tt, name, &isDouble);
  if (e != VLE_Success) return e;
  if (!derInput || !derMultiplier || !derBias || !input || !derOutput)
    return context.setError(VLE_IllegalArgument, (std::string(name) + ": DERINPUT, DERMULTIPLIERS, DERBIASES, INPUT and DEROUTPUT are required").c_str());
  Extents x = extentsOf(input);
  if ((e = checkParameters(context, name, x, multiplier, bias, moment, given)) != VLE_Success) return e;
  if (derOutput.getNumElements() != input.getNumElements() || derInput.getNumElements() != input.getNumElements())
    return context.setError(VLE_IllegalArgument, (std::string(name) + ": DEROUTPUT and DERINPUT must have the size of INPUT").c_str());
  if (isDouble) {
    const size_t need = moment ? 0 : 2 * (size_t)x.C * sizeof(double);
    void* scratch = need ? context.getWorkspace(VLDT_GPU, need) : NULL;
    if (need && !scratch) return context.getLastError();
    int rc64 = mcn_bnorm_backward_f64(context.getHipHelper().getStream(), (double*)derInput.getMemory(),
                                      (double*)derMultiplier.getMemory(), (double*)derBias.getMemory(),
                                      (double*)const_cast<void*>(moment.getMemory()), (double const*)input.getMemory(),
                                      (double const*)multiplier.getMemory(), (double const*)derOutput.getMemory(), x.H,
                                      x.W, x.C, x.N, op.epsilon, given ? 1 : 0, scratch, need);
    return fromAbi(context, rc64, name);
  }
  const size_t bytes = mcn_bnorm_workspace_bytes(x.H, x.W, x.C, x.N);
  void* ws = bytes ? context.getWorkspace(VLDT_GPU, bytes) : NULL;
  if (bytes && !ws) return context.getLastError();
  int rc = mcn_bnorm_backward(context.getHipHelper().getStream(), (float*)derInput.getMemory(),
                              (float*)derMultiplier.getMemory(), (float*)derBias.getMemory(),
                              (float*)const_cast<void*>(moment.getMemory()), (float const*)input.getMemory(),
                              (float const*)multiplier.getMemory(), (float const*)derOutput.getMemory(), x.H, x.W,
                              x.C, x.N, op.epsilon, given ? 1 : 0, ws, bytes);
  return fromAbi(context, rc, name);
}

}  // namespace

ErrorCode BatchNorm::forward(Tensor& output, Tensor& moment, Tensor const& input, Tensor const& multiplier,
                             Tensor const& bias) {
  return forwardAny(*this, "BatchNorm::forward", output, moment, input, multiplier, bias, false);
}

ErrorCode BatchNorm::forwardWithMoment(Tensor& output, Tensor const& moment, Tensor const& input,
                                       Tensor const& multiplier, Tensor const& bias) {
  return forwardAny(*this, "BatchNorm::forwardWithMoment", output, moment, input, multiplier, bias, true);
}

ErrorCode BatchNorm::backward(Tensor& derInput, Tensor& derMultiplier, Tensor& derBias, Tensor& moment,
                              Tensor const& input, Tensor const& multiplier, Tensor const& bias,
                              Tensor const& derOutput) {
  return backwardAny(*this, "BatchNorm::backward", derInput, derMultiplier, derBias, moment, input, multiplier, bias,
                     derOutput, false);
}

ErrorCode BatchNorm::backwardWithMoment(Tensor& derInput, Tensor& derMultiplier, Tensor& derBias, Tensor const& moment,
                                        Tensor const& input, Tensor const& multiplier, Tensor const& bias,
                                        Tensor const& derOutput) {
  return backwardAny(*this, "BatchNorm::backwardWithMoment", derInput, derMultiplier, derBias, moment, input,
                     multiplier, bias, derOutput, true);
}
