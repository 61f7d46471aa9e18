// vl::nn::Convolution on the HIP device.  Where the reference loops over images calling im2row and a BLAS
// GEMM (matlab/src/bits/nnconv.cu:71-317), each product here is one call into the C ABI, which runs an
// implicit-GEMM kernel over the whole batch.
#include "nnconv.hpp"

#include <algorithm>

#include "impl/dispatcher.hpp"

using namespace vl;
using namespace vl::nn;
using namespace vl::impl;

Convolution::Convolution(Context& context, int strideY, int strideX, int padTop, int padBottom, int padLeft,
                         int padRight, int dilateY, int dilateX)
    : context(context), strideY(strideY), strideX(strideX), padTop(padTop), padBottom(padBottom), padLeft(padLeft),
      padRight(padRight), dilateY(dilateY), dilateX(dilateX), packedForward(NULL), packedForwardBytes(0),
      packedBackward(NULL), packedBackwardBytes(0) {}

namespace {

mcn_conv_geom geometry(Convolution const& op, TensorShape const& data, TensorShape const& filter) {
  mcn_conv_geom g;
  g.H = asInt(data.getHeight()); g.W = asInt(data.getWidth()); g.C = asInt(data.getDepth()); g.N = asInt(data.getSize());
  g.FH = asInt(filter.getHeight()); g.FW = asInt(filter.getWidth()); g.FC = asInt(filter.getDepth()); g.K = asInt(filter.getSize());
  g.strideY = op.strideY; g.strideX = op.strideX;
  g.padTop = op.padTop; g.padBottom = op.padBottom; g.padLeft = op.padLeft; g.padRight = op.padRight;
  g.dilateY = op.dilateY; g.dilateX = op.dilateX;
  return g;
}

// Scratch from the context, sized by the back-end; NULL with an error recorded when it cannot be had.
bool scratch(Context& context, mcn_conv_geom const& g, int product, void** ws, size_t* bytes, int alsoProduct = -1) {
  *bytes = mcn_conv_workspace_bytes(&g, product);
  if (alsoProduct >= 0) *bytes = std::max(*bytes, mcn_conv_workspace_bytes(&g, alsoProduct));
  *ws = NULL;
  if (*bytes == 0) return true;
  *ws = context.getWorkspace(VLDT_GPU, *bytes);
  return *ws != NULL;
}

}  // namespace

ErrorCode Convolution::forward(Tensor& output, double outputMult, Tensor const& input, double inputMult,
                               Tensor const& filter, Tensor const& bias) {
  tensor_type tt = findTensorType(output, input, filter, bias);
  bool isDouble;
  ErrorCode e = requireHip(context, tt, "Convolution::forward", &isDouble);
  if (e != VLE_Success) return e;
  if (!output || !input || !filter)
    return context.setError(VLE_IllegalArgument, "Convolution::forward: OUTPUT, INPUT and FILTER are required");
  mcn_conv_geom g = geometry(*this, input, filter);
  int oh = 0, ow = 0;
  int rc = mcn_conv_output_size(&g, &oh, &ow);
  if (rc) return fromAbi(context, rc, "Convolution::forward");
  if ((int)output.getHeight() != oh || (int)output.getWidth() != ow || output.getDepth() != filter.getSize() ||
      output.getSize() != input.getSize())
    return context.setError(VLE_IllegalArgument, "Convolution::forward: OUTPUT dimensions are incompatible with X and FILTERS");
  if (bias && bias.getNumElements() != filter.getSize())
    return context.setError(VLE_IllegalArgument, "Convolution::forward: the number of elements of BIASES is not the number of filters");
  if (isDouble) {
    rc = mcn_conv_forward_f64(context.getHipHelper().getStream(), &g, (double*)output.getMemory(), outputMult,
                              (double const*)input.getMemory(), inputMult, (double const*)filter.getMemory(),
                              (double const*)bias.getMemory());
    return fromAbi(context, rc, "Convolution::forward");
  }
  void* ws;
  size_t bytes;
  if (!scratch(context, g, MCN_CONV_FORWARD, &ws, &bytes)) return context.getLastError();
  rc = mcn_conv_forward_packed(context.getHipHelper().getStream(), &g, (float*)output.getMemory(), (float)outputMult,
                               (float const*)input.getMemory(), (float)inputMult, (float const*)filter.getMemory(),
                               packedForward, packedForwardBytes, (float const*)bias.getMemory(), ws, bytes);
  return fromAbi(context, rc, "Convolution::forward");
}

int Convolution::sumGroups(TensorShape const& data, TensorShape const& filter) const {
  mcn_conv_geom g = geometry(*this, data, filter);
  return mcn_conv_forward_sums_groups(&g);
}

ErrorCode Convolution::forwardSums(Tensor& output, Tensor const& input, Tensor const& filter, double* sums,
                                   std::size_t sumsBytes) {
  tensor_type tt = findTensorType(output, input, filter);
  ErrorCode e = requireHipFloat(context, tt, "Convolution::forwardSums");
  if (e != VLE_Success) return e;
  if (!output || !input || !filter)
    return context.setError(VLE_IllegalArgument, "Convolution::forwardSums: OUTPUT, INPUT and FILTER are required");
  mcn_conv_geom g = geometry(*this, input, filter);
  int oh = 0, ow = 0;
  int rc = mcn_conv_output_size(&g, &oh, &ow);
  if (rc) return fromAbi(context, rc, "Convolution::forwardSums");
  if ((int)output.getHeight() != oh || (int)output.getWidth() != ow || output.getDepth() != filter.getSize() ||
      output.getSize() != input.getSize())
    return context.setError(VLE_IllegalArgument, "Convolution::forwardSums: OUTPUT dimensions are incompatible with X and FILTERS");
  void* ws;
  size_t bytes;
  if (!scratch(context, g, MCN_CONV_FORWARD, &ws, &bytes)) return context.getLastError();
  rc = mcn_conv_forward_sums(context.getHipHelper().getStream(), &g, (float*)output.getMemory(), (float const*)input.getMemory(),
                             (float const*)filter.getMemory(), packedForward, packedForwardBytes, sums, sumsBytes, ws, bytes);
  return fromAbi(context, rc, "Convolution::forwardSums");
}

bool Convolution::maskedAddSupported(TensorShape const& data, TensorShape const& filter) const {
  mcn_conv_geom g = geometry(*this, data, filter);
  return mcn_conv_backward_data_masked_add_supported(&g) != 0;
}

ErrorCode Convolution::backwardDataMaskedAdd(Tensor& derInput, Tensor const& filter, Tensor const& derOutput,
                                             float const* addend, unsigned const* maskBits) {
  tensor_type tt = findTensorType(derInput, filter, derOutput);
  ErrorCode e = requireHipFloat(context, tt, "Convolution::backwardDataMaskedAdd");
  if (e != VLE_Success) return e;
  if (!derInput || !filter || !derOutput || !addend || !maskBits)
    return context.setError(VLE_IllegalArgument, "Convolution::backwardDataMaskedAdd: DERINPUT, FILTER, DEROUTPUT, the addend and its mask are required");
  mcn_conv_geom g = geometry(*this, derInput, filter);
  int oh = 0, ow = 0;
  int rc = mcn_conv_output_size(&g, &oh, &ow);
  if (rc) return fromAbi(context, rc, "Convolution::backwardDataMaskedAdd");
  if ((int)derOutput.getHeight() != oh || (int)derOutput.getWidth() != ow || derOutput.getDepth() != filter.getSize() ||
      derOutput.getSize() != derInput.getSize())
    return context.setError(VLE_IllegalArgument, "Convolution::backwardDataMaskedAdd: DEROUTPUT dimensions are incompatible with X and FILTERS");
  void* ws;
  size_t bytes;
  if (!scratch(context, g, MCN_CONV_BACKWARD_DATA, &ws, &bytes)) return context.getLastError();
  rc = mcn_conv_backward_data_masked_add(context.getHipHelper().getStream(), &g, (float*)derInput.getMemory(),
                                         (float const*)filter.getMemory(), packedBackward, packedBackwardBytes,
                                         (float const*)derOutput.getMemory(), addend, maskBits, ws, bytes);
  return fromAbi(context, rc, "Convolution::backwardDataMaskedAdd");
}

std::size_t Convolution::packedBytes(int product, TensorShape const& data, TensorShape const& filter) const {
  mcn_conv_geom g = geometry(*this, data, filter);
  return mcn_conv_packed_bytes(&g, product);
}

ErrorCode Convolution::planPack(int product, TensorShape const& data, Tensor const& filter, void* packed, std::size_t bytes,
                                std::vector<mcn_conv_pack_job>& jobs) {
  mcn_conv_geom g = geometry(*this, data, filter);
  mcn_conv_pack_job found[64];
  int n = 0;
  int rc = mcn_conv_pack_plan(&g, product, (float const*)filter.getMemory(), packed, bytes, found, 64, &n);
  if (rc) return fromAbi(context, rc, "Convolution::planPack");
  jobs.insert(jobs.end(), found, found + n);
  return VLE_Success;
}

std::size_t Convolution::filterPartialBytes(TensorShape const& data, TensorShape const& filter) const {
  mcn_conv_geom g = geometry(*this, data, filter);
  return mcn_conv_backward_filter_partial_bytes(&g);
}

ErrorCode Convolution::planFilterPartial(TensorShape const& data, Tensor& derFilter, void* partials, std::size_t bytes,
                                         std::vector<mcn_conv_reduce_job>& jobs) {
  mcn_conv_geom g = geometry(*this, data, derFilter);
  mcn_conv_reduce_job found[64];
  int n = 0;
  int rc = mcn_conv_backward_filter_plan(&g, (float*)derFilter.getMemory(), partials, bytes, found, 64, &n);
  if (rc) return fromAbi(context, rc, "Convolution::planFilterPartial");
  jobs.insert(jobs.end(), found, found + n);
  return VLE_Success;
}

ErrorCode Convolution::backwardFilterPartial(Tensor& derFilter, Tensor const& input, Tensor const& derOutput, void* partials,
                                             std::size_t bytes) {
  tensor_type tt = findTensorType(derFilter, input, derOutput);
  ErrorCode e = requireHipFloat(context, tt, "Convolution::backwardFilterPartial");
  if (e != VLE_Success) return e;
  if (!derFilter || !input || !derOutput)
    return context.setError(VLE_IllegalArgument, "Convolution::backwardFilterPartial: DERFILTER, INPUT and DEROUTPUT are required");
  mcn_conv_geom g = geometry(*this, input, derFilter);
  int oh = 0, ow = 0;
  int rc = mcn_conv_output_size(&g, &oh, &ow);
  if (rc) return fromAbi(context, rc, "Convolution::backwardFilterPartial");
  if ((int)derOutput.getHeight() != oh || (int)derOutput.getWidth() != ow || derOutput.getDepth() != derFilter.getSize() ||
      derOutput.getSize() != input.getSize())
    return context.setError(VLE_IllegalArgument, "Convolution::backwardFilterPartial: DEROUTPUT dimensions are incompatible with X and FILTERS");
  rc = mcn_conv_backward_filter_partial(context.getHipHelper().getStream(), &g, (float*)derFilter.getMemory(),
                                        (float const*)input.getMemory(), (float const*)derOutput.getMemory(), partials, bytes);
  return fromAbi(context, rc, "Convolution::backwardFilterPartial");
}

ErrorCode Convolution::backward(Tensor& derInput, Tensor& derFilter, Tensor& derBias, Tensor const& input,
                                Tensor const& filter, Tensor const& derOutput) {
  return backwardAccumulate(derInput, 0, derFilter, derBias, input, filter, derOutput);
}

ErrorCode Convolution::backwardAccumulate(Tensor& derInput, double derInputMult, Tensor& derFilter, Tensor& derBias,
                                          Tensor const& input, Tensor const& filter, Tensor const& derOutput) {
  tensor_type tt = findTensorType(derInput, derFilter, derBias, input, filter, derOutput);
  bool isDouble;
  ErrorCode e = requireHip(context, tt, "Convolution::backward", &isDouble);
  if (e != VLE_Success) return e;
  if (!derOutput) return context.setError(VLE_IllegalArgument, "Convolution::backward: DEROUTPUT is required");
  if (isDouble && derInputMult != 0)
    return context.setError(VLE_Unsupported, "Convolution::backwardAccumulate: accumulation is implemented in single precision only");
  void* stream = context.getHipHelper().getStream();
  void* ws;
  size_t bytes;
  int rc;

  // DERBIASES together with DERFILTER in single precision: one call below gives both (first layers take them from the
  // same pass over DEROUTPUT)
  const bool biasWithFilter = derBias && derFilter && !isDouble;
  if (derBias && derBias.getNumElements() != derOutput.getDepth())
    return context.setError(VLE_IllegalArgument, "Convolution::backward: DERBIASES has the wrong number of elements");
  if (derBias && !biasWithFilter) {
    // only the extent of DEROUTPUT matters: describe it as a 1x1 convolution over itself
    TensorShape unit(1, 1, derOutput.getDepth(), derOutput.getDepth());
    Convolution plain(context, 1, 1, 0, 0, 0, 0, 1, 1);
    mcn_conv_geom g = geometry(plain, derOutput, unit);
    if (isDouble) {
      rc = mcn_conv_backward_bias_f64(stream, &g, (double*)derBias.getMemory(), (double const*)derOutput.getMemory());
      if (rc) return fromAbi(context, rc, "Convolution::backward");
    } else {
    if (!scratch(context, g, MCN_CONV_BACKWARD_BIAS, &ws, &bytes)) return context.getLastError();
    rc = mcn_conv_backward_bias(stream, &g, (float*)derBias.getMemory(), (float const*)derOutput.getMemory(), ws, bytes);
    if (rc) return fromAbi(context, rc, "Convolution::backward");
    }
  }

  if (derInput) {
    if (!filter) return context.setError(VLE_IllegalArgument, "Convolution::backward: FILTER is required for DERINPUT");
    mcn_conv_geom g = geometry(*this, derInput, filter);
    int oh = 0, ow = 0;
    rc = mcn_conv_output_size(&g, &oh, &ow);
    if (rc) return fromAbi(context, rc, "Convolution::backward");
    if ((int)derOutput.getHeight() != oh || (int)derOutput.getWidth() != ow || derOutput.getDepth() != filter.getSize() ||
        derOutput.getSize() != derInput.getSize())
      return context.setError(VLE_IllegalArgument, "Convolution::backward: DEROUTPUT dimensions are incompatible with X and FILTERS");
    if (isDouble) {
      rc = mcn_conv_backward_data_f64(stream, &g, (double*)derInput.getMemory(), (double const*)filter.getMemory(),
                                      (double const*)derOutput.getMemory());
    } else {
      if (!scratch(context, g, MCN_CONV_BACKWARD_DATA, &ws, &bytes)) return context.getLastError();
      rc = mcn_conv_backward_data_packed(stream, &g, (float*)derInput.getMemory(), (float)derInputMult,
                                         (float const*)filter.getMemory(), packedBackward, packedBackwardBytes,
                                         (float const*)derOutput.getMemory(), ws, bytes);
    }
    if (rc) return fromAbi(context, rc, "Convolution::backward");
  }

  if (derFilter) {
    if (!input) return context.setError(VLE_IllegalArgument, "Convolution::backward: INPUT is required for DERFILTER");
    mcn_conv_geom g = geometry(*this, input, derFilter);
    int oh = 0, ow = 0;
    rc = mcn_conv_output_size(&g, &oh, &ow);
    if (rc) return fromAbi(context, rc, "Convolution::backward");
    if ((int)derOutput.getHeight() != oh || (int)derOutput.getWidth() != ow || derOutput.getDepth() != derFilter.getSize() ||
        derOutput.getSize() != input.getSize())
      return context.setError(VLE_IllegalArgument, "Convolution::backward: DEROUTPUT dimensions are incompatible with X and FILTERS");
    if (isDouble) {
      rc = mcn_conv_backward_filter_f64(stream, &g, (double*)derFilter.getMemory(), (double const*)input.getMemory(),
                                        (double const*)derOutput.getMemory());
    } else {
      if (!scratch(context, g, MCN_CONV_BACKWARD_FILTER, &ws, &bytes, biasWithFilter ? MCN_CONV_BACKWARD_BIAS : -1))
        return context.getLastError();
      if (biasWithFilter)
        rc = mcn_conv_backward_filter_bias(stream, &g, (float*)derFilter.getMemory(), (float*)derBias.getMemory(),
                                           (float const*)input.getMemory(), (float const*)derOutput.getMemory(), ws, bytes);
      else
        rc = mcn_conv_backward_filter(stream, &g, (float*)derFilter.getMemory(), (float const*)input.getMemory(),
                                      (float const*)derOutput.getMemory(), ws, bytes);
    }
    if (rc) return fromAbi(context, rc, "Convolution::backward");
  }
  return VLE_Success;
}

// ---------------------------------------------------------------------------------- ConvolutionTranspose
//
// The transpose of a convolution with stride = upsample and pad = crop (matlab/src/bits/nnconv.cu:323-421):
// forward is that convolution's backward-data product with the roles of input and output exchanged, backward is
// its forward and backward-filter products.  The reference loops over images in forward because its
// per-image GEMM would otherwise fold the batch; the batched kernels here take the whole batch in one call.

ConvolutionTranspose::ConvolutionTranspose(Context& context, int upsampleY, int upsampleX, int cropTop, int cropBottom,
                                           int cropLeft, int cropRight)
    : context(context), upsampleY(upsampleY), upsampleX(upsampleX), cropTop(cropTop), cropBottom(cropBottom),
      cropLeft(cropLeft), cropRight(cropRight) {}

ErrorCode ConvolutionTranspose::forward(Tensor& output, Tensor const& input, Tensor const& filter, Tensor const& bias) {
  tensor_type tt = findTensorType(output, input, filter, bias);
  bool isDouble;
  ErrorCode e = requireHip(context, tt, "ConvolutionTranspose::forward", &isDouble);
  if (e != VLE_Success) return e;
  if (!output || !input || !filter)
    return context.setError(VLE_IllegalArgument, "ConvolutionTranspose::forward: OUTPUT, INPUT and FILTER are required");
  if (bias && bias.getNumElements() != output.getDepth())
    return context.setError(VLE_IllegalArgument, "ConvolutionTranspose::forward: the number of elements of BIASES is not the output depth");
  Convolution opc(context, upsampleY, upsampleX, cropTop, cropBottom, cropLeft, cropRight, 1, 1);
  Tensor null;
  e = opc.backward(output, null, null, null, filter, input);
  if (e != VLE_Success) return context.passError(e, "ConvolutionTranspose::forward");
  if (bias) {
    int rc = isDouble ? mcn_bias_add_f64(context.getHipHelper().getStream(), (double*)output.getMemory(),
                                         (double const*)bias.getMemory(), asInt(output.getHeight()), asInt(output.getWidth()),
                                         asInt(output.getDepth()), asInt(output.getSize()))
                      : mcn_bias_add(context.getHipHelper().getStream(), (float*)output.getMemory(),
                                     (float const*)bias.getMemory(), asInt(output.getHeight()), asInt(output.getWidth()),
                                     asInt(output.getDepth()), asInt(output.getSize()));
    return fromAbi(context, rc, "ConvolutionTranspose::forward");
  }
  return VLE_Success;
}

ErrorCode ConvolutionTranspose::backward(Tensor& derData, Tensor& derFilter, Tensor& derBias, Tensor const& input,
                                         Tensor const& filter, Tensor const& derOutput) {
  tensor_type tt = findTensorType(derData, derFilter, derBias, input, filter, derOutput);
  bool isDouble;
  ErrorCode e = requireHip(context, tt, "ConvolutionTranspose::backward", &isDouble);
  if (e != VLE_Success) return e;
  if (!derOutput) return context.setError(VLE_IllegalArgument, "ConvolutionTranspose::backward: DEROUTPUT is required");
  Convolution opc(context, upsampleY, upsampleX, cropTop, cropBottom, cropLeft, cropRight, 1, 1);
  Tensor null;
  if (derData) {
    if (!filter) return context.setError(VLE_IllegalArgument, "ConvolutionTranspose::backward: FILTER is required for DERDATA");
    e = opc.forward(derData, 0, derOutput, 1, filter, null);
    if (e != VLE_Success) return context.passError(e, "ConvolutionTranspose::backward");
  }
  if (derFilter) {
    if (!input) return context.setError(VLE_IllegalArgument, "ConvolutionTranspose::backward: INPUT is required for DERFILTER");
    e = opc.backward(null, derFilter, null, derOutput, null, input);
    if (e != VLE_Success) return context.passError(e, "ConvolutionTranspose::backward");
  }
  if (derBias) {
    Tensor none1, none2;
    e = opc.backward(none1, none2, derBias, null, null, derOutput);
    if (e != VLE_Success) return context.passError(e, "ConvolutionTranspose::backward");
  }
  return VLE_Success;
}
