// vl::nn::Convolution -- same class interface as matlab/src/bits/nnconv.hpp:23-52.
#ifndef MCN_AMD_BITS_NNCONV_HPP
#define MCN_AMD_BITS_NNCONV_HPP

#include "data.hpp"

namespace vl { namespace nn {

class Convolution {
 public:
  Convolution(Context& context, int strideY, int strideX, int padTop, int padBottom, int padLeft, int padRight,
              int dilateY, int dilateX);

  // output = outputMult*output + inputMult*conv(input, filter) + bias.  `bias` may be a null tensor.
  vl::ErrorCode forward(vl::Tensor& output, double outputMult, vl::Tensor const& input, double inputMult,
                        vl::Tensor const& filter, vl::Tensor const& bias);

  // Any of derInput / derFilter / derBias may be a null tensor, meaning "do not compute".  The ones given
  // are fully overwritten.  `input` is needed for derFilter, `filter` for derInput.
  vl::ErrorCode backward(vl::Tensor& derInput, vl::Tensor& derFilter, vl::Tensor& derBias, vl::Tensor const& input,
                         vl::Tensor const& filter, vl::Tensor const& derOutput);

  // The same with derInput = derInputMult*derInput + dzdx: the sum a network wrapper makes where a variable
  // feeds several layers (matlab/+dagnn/Layer.m:130-132), folded into the convolution's output pass.  Not part
  // of the reference's class.
  vl::ErrorCode backwardAccumulate(vl::Tensor& derInput, double derInputMult, vl::Tensor& derFilter, vl::Tensor& derBias,
                                   vl::Tensor const& input, vl::Tensor const& filter, vl::Tensor const& derOutput);

  Context& context;
  int strideY;
  int strideX;
  int padTop;
  int padBottom;
  int padLeft;
  int padRight;
  int dilateY;
  int dilateX;
};

// Same class interface as matlab/src/bits/nnconv.hpp:54-81.  FILTER is FH x FW x (output depth / groups) x (input
// depth); output extent (H-1)*upsample - (cropA + cropB) + FH.
class ConvolutionTranspose {
 public:
  ConvolutionTranspose(Context& context, int upsampleY, int upsampleX, int cropTop, int cropBottom, int cropLeft,
                       int cropRight);

  // output (fully overwritten) = convt(input, filter) + bias.  `bias` may be a null tensor.
  vl::ErrorCode forward(vl::Tensor& output, vl::Tensor const& input, vl::Tensor const& filter, vl::Tensor const& bias);

  // Any of derData / derFilter / derBias may be a null tensor, meaning "do not compute".
  vl::ErrorCode backward(vl::Tensor& derData, vl::Tensor& derFilter, vl::Tensor& derBias, vl::Tensor const& input,
                         vl::Tensor const& filter, vl::Tensor const& derOutput);

  Context& context;
  int upsampleY;
  int upsampleX;
  int cropTop;
  int cropBottom;
  int cropLeft;
  int cropRight;
};

} }  // namespace vl::nn
#endif
