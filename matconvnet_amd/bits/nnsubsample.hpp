// vl::nn::Subsample -- same class interface as matlab/src/bits/nnsubsample.hpp:20-44: what vl_nnconv runs when
// FILTERS is empty (the identity filter bank: sample every stride-th pixel of the padded input, add the bias).
#ifndef MCN_AMD_BITS_NNSUBSAMPLE_HPP
#define MCN_AMD_BITS_NNSUBSAMPLE_HPP

#include "data.hpp"

namespace vl { namespace nn {

class Subsample {
 public:
  Subsample(vl::Context& context, int strideY, int strideX, int padTop, int padBottom, int padLeft, int padRight);

  // output = subsample(input) + biases; `biases` may be a null tensor
  vl::ErrorCode forwardWithBias(vl::Tensor& output, vl::Tensor const& input, vl::Tensor const& biases);

  // derInput (fully overwritten) and/or derBiases; either may be a null tensor
  vl::ErrorCode backwardWithBias(vl::Tensor& derInput, vl::Tensor& derBiases, vl::Tensor const& derOutput);

  vl::Context& context;
  int strideY;
  int strideX;
  int padTop;
  int padBottom;
  int padLeft;
  int padRight;
};

} }  // namespace vl::nn
#endif
