// vl::nn::BatchNorm -- same class interface as matlab/src/bits/nnbnorm.hpp:22-59.
#ifndef MCN_AMD_BITS_NNBNORM_HPP
#define MCN_AMD_BITS_NNBNORM_HPP

#include "data.hpp"

namespace vl { namespace nn {

class BatchNorm {
 public:
  BatchNorm(vl::Context& context, double epsilon);

  // Moments are computed from the batch; `moment` (C x 2: means then sigmas) receives them unless null.
  vl::ErrorCode forward(vl::Tensor& output, vl::Tensor& moment, vl::Tensor const& input,
                        vl::Tensor const& multiplier, vl::Tensor const& bias);
  // Moments are taken from `moment`.
  vl::ErrorCode forwardWithMoment(vl::Tensor& output, vl::Tensor const& moment, vl::Tensor const& input,
                                  vl::Tensor const& multiplier, vl::Tensor const& bias);
  vl::ErrorCode backward(vl::Tensor& derInput, vl::Tensor& derMultiplier, vl::Tensor& derBias, vl::Tensor& moment,
                         vl::Tensor const& input, vl::Tensor const& multiplier, vl::Tensor const& bias,
                         vl::Tensor const& derOutput);
  vl::ErrorCode backwardWithMoment(vl::Tensor& derInput, vl::Tensor& derMultiplier, vl::Tensor& derBias,
                                   vl::Tensor const& moment, vl::Tensor const& input, vl::Tensor const& multiplier,
                                   vl::Tensor const& bias, vl::Tensor const& derOutput);

  vl::Context& context;
  double epsilon;
};

} }  // namespace vl::nn
#endif
