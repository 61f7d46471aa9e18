// vl::nn::Convolution -- same class interface as matlab/src/bits/nnconv.hpp:23-52.
#ifndef MCN_AMD_BITS_NNCONV_HPP
#define MCN_AMD_BITS_NNCONV_HPP

#include <vector>

#include "../../include/mcn_hip.h"
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

  // Filter banks packed ahead (mcn_conv_pack_filters and friends, include/mcn_hip.h), for callers whose filters stay
  // put between calls.  Not part of the reference's class.
  //   packedBytes   size of the packed bank of a product (MCN_CONV_FORWARD / MCN_CONV_BACKWARD_DATA) for data of
  //                 this shape (the layer's input) and this filter bank; 0: the product reads none
  //   planPack      appends the product's packing jobs (filter bank -> `packed`) to `jobs`, for one batched launch
  //   usePacked     the banks forward / backward[Accumulate] read from now on (null: pack on the fly, the default)
  std::size_t packedBytes(int product, vl::TensorShape const& data, vl::TensorShape const& filter) const;
  vl::ErrorCode planPack(int product, vl::TensorShape const& data, vl::Tensor const& filter, void* packed, std::size_t bytes,
                         std::vector<mcn_conv_pack_job>& jobs);
  void usePacked(void const* forwardBank, std::size_t forwardBytes, void const* backwardBank, std::size_t backwardBytes) {
    packedForward = forwardBank; packedForwardBytes = forwardBytes;
    packedBackward = backwardBank; packedBackwardBytes = backwardBytes;
  }

  // Filter gradient with its final sum deferred (mcn_conv_backward_filter_partial and friends): the matrix kernel
  // leaves the partial banks in `partials`; the jobs planned once sum them into derFilter in a launch the caller
  // makes for many layers at once.  filterPartialBytes == 0: this geometry has no deferred form (use backward).
  // Not part of the reference's class.
  std::size_t filterPartialBytes(vl::TensorShape const& data, vl::TensorShape const& filter) const;
  vl::ErrorCode planFilterPartial(vl::TensorShape const& data, vl::Tensor& derFilter, void* partials, std::size_t bytes,
                                  std::vector<mcn_conv_reduce_job>& jobs);
  vl::ErrorCode backwardFilterPartial(vl::Tensor& derFilter, vl::Tensor const& input, vl::Tensor const& derOutput,
                                      void* partials, std::size_t bytes);

  // Forward (no bias, output overwritten) that also sums the output and its square per channel in the same launch
  // (mcn_conv_forward_sums): the summing pass of a batch normalisation that follows.  sumGroups: partial sums per
  // channel for this geometry (0: no such form; use forward); sums: device buffer of K * sumGroups * 2 doubles.  Not
  // part of the reference's class.
  int sumGroups(vl::TensorShape const& data, vl::TensorShape const& filter) const;
  vl::ErrorCode forwardSums(vl::Tensor& output, vl::Tensor const& input, vl::Tensor const& filter, double* sums,
                            std::size_t sumsBytes);

  // DERINPUT = backward-data + a second term gated by one bit per element (mcn_conv_backward_data_masked_add): the
  // derivative an identity shortcut brings to the same tensor from behind a ReLU.  maskedAddSupported: whether this
  // geometry has that form.  Not part of the reference's class.
  bool maskedAddSupported(vl::TensorShape const& data, vl::TensorShape const& filter) const;
  vl::ErrorCode backwardDataMaskedAdd(vl::Tensor& derInput, vl::Tensor const& filter, vl::Tensor const& derOutput,
                                      float const* addend, unsigned const* maskBits);

  Context& context;
  int strideY;
  int strideX;
  int padTop;
  int padBottom;
  int padLeft;
  int padRight;
  int dilateY;
  int dilateX;
  void const* packedForward;
  std::size_t packedForwardBytes;
  void const* packedBackward;
  std::size_t packedBackwardBytes;
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
