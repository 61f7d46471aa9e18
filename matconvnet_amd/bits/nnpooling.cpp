// vl::nn::Pooling on the HIP device (reference semantics: matlab/src/bits/nnpooling.cu:33-237).
#include "nnpooling.hpp"

#include "impl/dispatcher.hpp"

using namespace vl;
using namespace vl::nn;
using namespace vl::impl;

Pooling::Pooling(Context& context, int poolHeight, int poolWidth, int strideY, int strideX, int padTop, int padBottom,
                 int padLeft, int padRight, Method method)
    : context(context), poolHeight(poolHeight), poolWidth(poolWidth), strideY(strideY), strideX(strideX),
      padTop(padTop), padBottom(padBottom), padLeft(padLeft), padRight(padRight), method(method) {}

namespace {

mcn_pool_geom geometry(Pooling const& op, TensorShape const& data) {
  mcn_pool_geom g;
  g.H = asInt(data.getHeight()); g.W = asInt(data.getWidth()); g.C = asInt(data.getDepth()); g.N = asInt(data.getSize());
  g.poolH = op.poolHeight; g.poolW = op.poolWidth;
  g.strideY = op.strideY; g.strideX = op.strideX;
  g.padTop = op.padTop; g.padBottom = op.padBottom; g.padLeft = op.padLeft; g.padRight = op.padRight;
  g.method = op.method == Pooling::Max ? MCN_POOL_MAX : MCN_POOL_AVERAGE;
  return g;
}

ErrorCode checkOutput(Context& context, char const* name, mcn_pool_geom const& g, TensorShape const& pooled,
                      TensorShape const& data) {
  int oh = 0, ow = 0;
  int rc = mcn_pool_output_size(&g, &oh, &ow);
  if (rc) return fromAbi(context, rc, name);
  if ((int)pooled.getHeight() != oh || (int)pooled.getWidth() != ow || pooled.getDepth() != data.getDepth() ||
      pooled.getSize() != data.getSize())
    return context.setError(VLE_IllegalArgument, (std::string(name) + ": the pooled tensor's dimensions are incompatible with X and POOL").c_str());
  return VLE_Success;
}

ErrorCode backwardAny(Pooling& op, char const* name, Tensor& derInput, Tensor const& input, Tensor const& derOutput,
                      int accumulate) {
  Context& context = op.context;
  tensor_type tt = findTensorType(derInput, input, derOutput);
  bool isDouble;
  ErrorCode e = requireHip(context, tt, name, &isDouble);
  if (e != VLE_Success) return e;
  if (!derInput || !derOutput || (op.method == Pooling::Max && !input))
    return context.setError(VLE_IllegalArgument, (std::string(name) + ": DERINPUT, INPUT and DEROUTPUT are required").c_str());
  mcn_pool_geom g = geometry(op, derInput);
  if ((e = checkOutput(context, name, g, derOutput, derInput)) != VLE_Success) return e;
  int rc = isDouble ? mcn_pool_backward_f64(context.getHipHelper().getStream(), &g, (double*)derInput.getMemory(),
                                            (double const*)input.getMemory(), (double const*)derOutput.getMemory(),
                                            accumulate)
                    : mcn_pool_backward(context.getHipHelper().getStream(), &g, (float*)derInput.getMemory(),
                                        (float const*)input.getMemory(), (float const*)derOutput.getMemory(), accumulate);
  return fromAbi(context, rc, name);
}

}  // namespace

ErrorCode Pooling::forward(Tensor& output, Tensor const& input) {
  tensor_type tt = findTensorType(output, input);
  bool isDouble;
  ErrorCode e = requireHip(context, tt, "Pooling::forward", &isDouble);
  if (e != VLE_Success) return e;
  if (!output || !input) return context.setError(VLE_IllegalArgument, "Pooling::forward: OUTPUT and INPUT are required");
  mcn_pool_geom g = geometry(*this, input);
  if ((e = checkOutput(context, "Pooling::forward", g, output, input)) != VLE_Success) return e;
  int rc = isDouble ? mcn_pool_forward_f64(context.getHipHelper().getStream(), &g, (double*)output.getMemory(),
                                           (double const*)input.getMemory())
                    : mcn_pool_forward(context.getHipHelper().getStream(), &g, (float*)output.getMemory(),
                                       (float const*)input.getMemory());
  return fromAbi(context, rc, "Pooling::forward");
}

ErrorCode Pooling::backward(Tensor& derInput, Tensor const& input, Tensor const& derOutput) {
  return backwardAny(*this, "Pooling::backward", derInput, input, derOutput, 1);
}

ErrorCode Pooling::backwardOverwrite(Tensor& derInput, Tensor const& input, Tensor const& derOutput) {
  return backwardAny(*this, "Pooling::backwardOverwrite", derInput, input, derOutput, 0);
}
