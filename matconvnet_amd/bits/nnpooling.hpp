// vl::nn::Pooling -- same class interface as matlab/src/bits/nnpooling.hpp:21-49, plus one method.
#ifndef MCN_AMD_BITS_NNPOOLING_HPP
#define MCN_AMD_BITS_NNPOOLING_HPP

#include "data.hpp"

namespace vl { namespace nn {

class Pooling {
 public:
  enum Method { Max, Average };

  Pooling(vl::Context& context, int poolHeight, int poolWidth, int strideY, int strideX, int padTop, int padBottom,
          int padLeft, int padRight, Method method);

  vl::ErrorCode forward(vl::Tensor& output, vl::Tensor const& input);

  // derInput += pooling'(derOutput): callers zero-fill derInput first, as vl_nnpool does
  // (matlab/src/vl_nnpool.cu:255-259).
  vl::ErrorCode backward(vl::Tensor& derInput, vl::Tensor const& input, vl::Tensor const& derOutput);

  // Addition to the reference interface: derInput is write-only and receives exactly what backward()
  // leaves in a zero-filled buffer, so the caller's fill pass over derInput can be dropped.
  vl::ErrorCode backwardOverwrite(vl::Tensor& derInput, vl::Tensor const& input, vl::Tensor const& derOutput);

  vl::Context& context;
  int poolHeight;
  int poolWidth;
  int strideY;
  int strideX;
  int padTop;
  int padBottom;
  int padLeft;
  int padRight;
  Method method;
};

} }  // namespace vl::nn
#endif
