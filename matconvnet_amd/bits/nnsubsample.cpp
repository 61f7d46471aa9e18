// vl::nn::Subsample on the HIP device (matlab/src/bits/nnsubsample.cu:31-216 restated as two calls into the C ABI:
// the per-image bias GEMM / GEMV with the all-ones vector become part of the subsampling kernel and the bias
// reduction kernel).
#include "nnsubsample.hpp"

#include "impl/dispatcher.hpp"

using namespace vl;
using namespace vl::nn;
using namespace vl::impl;

Subsample::Subsample(Context& context, int strideY, int strideX, int padTop, int padBottom, int padLeft, int padRight)
    : context(context), strideY(strideY), strideX(strideX), padTop(padTop), padBottom(padBottom), padLeft(padLeft),
      padRight(padRight) {}

namespace {

// the extents the reference asserts on (nnsubsample.cu:48-52,142-146)
bool extentsMatch(Subsample const& op, Tensor const& big, Tensor const& small) {
  int oh = 0, ow = 0;
  if (mcn_subsample_output_size(asInt(big.getHeight()), asInt(big.getWidth()), op.strideY, op.strideX, op.padTop, op.padBottom,
                                op.padLeft, op.padRight, &oh, &ow))
    return false;
  return (int)small.getHeight() == oh && (int)small.getWidth() == ow && small.getDepth() == big.getDepth() &&
         small.getSize() == big.getSize();
}

}  // namespace

ErrorCode Subsample::forwardWithBias(Tensor& output, Tensor const& input, Tensor const& biases) {
  tensor_type tt = findTensorType(output, input, biases);
  bool isDouble;
  ErrorCode e = requireHip(context, tt, "Subsample::forwardWithBias", &isDouble);
  if (e != VLE_Success) return e;
  if (!output || !input) return context.setError(VLE_IllegalArgument, "Subsample::forwardWithBias: OUTPUT and INPUT are required");
  if (!extentsMatch(*this, input, output))
    return context.setError(VLE_IllegalArgument, "Subsample::forwardWithBias: OUTPUT dimensions are incompatible with INPUT");
  if (biases && biases.getNumElements() != input.getDepth())
    return context.setError(VLE_IllegalArgument, "Subsample::forwardWithBias: the number of elements of BIASES is not the DATA depth");
  int rc = isDouble
               ? mcn_subsample_forward_f64(context.getHipHelper().getStream(), (double*)output.getMemory(),
                                           (double const*)input.getMemory(), (double const*)biases.getMemory(),
                                           asInt(input.getHeight()), asInt(input.getWidth()), asInt(input.getDepth()),
                                           asInt(input.getSize()), strideY, strideX, padTop, padBottom, padLeft, padRight)
               : mcn_subsample_forward(context.getHipHelper().getStream(), (float*)output.getMemory(),
                                       (float const*)input.getMemory(), (float const*)biases.getMemory(),
                                       asInt(input.getHeight()), asInt(input.getWidth()), asInt(input.getDepth()),
                                       asInt(input.getSize()), strideY, strideX, padTop, padBottom, padLeft, padRight);
  return fromAbi(context, rc, "Subsample::forwardWithBias");
}

ErrorCode Subsample::backwardWithBias(Tensor& derInput, Tensor& derBiases, Tensor const& derOutput) {
  tensor_type tt = findTensorType(derInput, derBiases, derOutput);
  bool isDouble;
  ErrorCode e = requireHip(context, tt, "Subsample::backwardWithBias", &isDouble);
  if (e != VLE_Success) return e;
  if (!derOutput) return context.setError(VLE_IllegalArgument, "Subsample::backwardWithBias: DEROUTPUT is required");
  void* stream = context.getHipHelper().getStream();
  int rc;
  if (derInput) {
    if (!extentsMatch(*this, derInput, derOutput))
      return context.setError(VLE_IllegalArgument, "Subsample::backwardWithBias: DEROUTPUT dimensions are incompatible with DERINPUT");
    rc = isDouble ? mcn_subsample_backward_f64(stream, (double*)derInput.getMemory(), (double const*)derOutput.getMemory(),
                                               asInt(derInput.getHeight()), asInt(derInput.getWidth()),
                                               asInt(derInput.getDepth()), asInt(derInput.getSize()), strideY, strideX,
                                               padTop, padBottom, padLeft, padRight)
                  : mcn_subsample_backward(stream, (float*)derInput.getMemory(), (float const*)derOutput.getMemory(),
                                           asInt(derInput.getHeight()), asInt(derInput.getWidth()),
                                           asInt(derInput.getDepth()), asInt(derInput.getSize()), strideY, strideX, padTop,
                                           padBottom, padLeft, padRight);
    if (rc) return fromAbi(context, rc, "Subsample::backwardWithBias");
  }
  if (derBiases) {
    if (derBiases.getNumElements() != derOutput.getDepth())
      return context.setError(VLE_IllegalArgument, "Subsample::backwardWithBias: DERBIASES has the wrong number of elements");
    // per-channel sum of DEROUTPUT: the bias product of a 1x1 convolution over DEROUTPUT itself
    mcn_conv_geom g;
    g.H = asInt(derOutput.getHeight()); g.W = asInt(derOutput.getWidth()); g.C = asInt(derOutput.getDepth()); g.N = asInt(derOutput.getSize());
    g.FH = g.FW = 1; g.FC = g.C; g.K = g.C;
    g.strideY = g.strideX = 1; g.padTop = g.padBottom = g.padLeft = g.padRight = 0; g.dilateY = g.dilateX = 1;
    if (isDouble) {
      rc = mcn_conv_backward_bias_f64(stream, &g, (double*)derBiases.getMemory(), (double const*)derOutput.getMemory());
      return fromAbi(context, rc, "Subsample::backwardWithBias");
    }
    size_t bytes = mcn_conv_workspace_bytes(&g, MCN_CONV_BACKWARD_BIAS);
    void* ws = bytes ? context.getWorkspace(VLDT_GPU, bytes) : NULL;
    if (bytes && !ws) return context.getLastError();
    rc = mcn_conv_backward_bias(stream, &g, (float*)derBiases.getMemory(), (float const*)derOutput.getMemory(), ws, bytes);
    if (rc) return fromAbi(context, rc, "Subsample::backwardWithBias");
  }
  return VLE_Success;
}
