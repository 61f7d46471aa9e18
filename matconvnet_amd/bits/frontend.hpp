// Argument conventions of the MATLAB-facing drivers vl_nnconv / vl_nnbnorm / vl_nnpool, restated as plain
// C++ entry points (no MATLAB needed).  Each function takes what the MEX driver's mexFunction takes --
// a list of inputs (arrays and strings) and a number of requested outputs -- and applies the same
// parsing, validation, output-allocation and error rules:
//   vl_nnconv (x, f, b [, dzdy], options...)   matlab/src/vl_nnconv.cu:87-502  (empty f: subsample + bias)
//   vl_nnconvt(x, f, b [, dzdy], options...)   matlab/src/vl_nnconvt.cu:81-417
//   vl_nnbnorm(x, g, b [, dzdy], options...)   matlab/src/vl_nnbnorm.cu:73-301
//   vl_nnpool (x, pool [, dzdy], options...)   matlab/src/vl_nnpool.cu:72-314
//   vl_taccum (alpha, a, beta, b [, 'InPlace']) matlab/src/vl_taccummex.cu:151-224
// Where the MEX drivers raise a MATLAB error these return a vl::ErrorCode and leave the reference's
// message text in `message`.
#ifndef MCN_AMD_BITS_FRONTEND_HPP
#define MCN_AMD_BITS_FRONTEND_HPP

#include <memory>
#include <string>
#include <vector>

#include "data.hpp"

namespace vl { namespace frontend {

// One element of the argument list: a numeric array (device or host tensor view) or a string.
struct Arg {
  enum Kind { Array, String };
  Kind kind;
  Tensor tensor;
  std::string text;
  std::shared_ptr<std::vector<double> > owned;  // backing store of host option values

  static Arg array(Tensor const& t);
  static Arg string(std::string const& s);
  // host double row vector, what MATLAB passes for 'stride', 'pad', 'epsilon', the pooling size...
  static Arg numeric(std::vector<double> const& values);
};

// Who provides memory for outputs (MATLAB's allocator in the MEX drivers).  Returning NULL = out of memory.
class Allocator {
 public:
  virtual ~Allocator() {}
  virtual void* allocate(DeviceType device, std::size_t bytes) = 0;
};

// out[0..nout-1] receive views of freshly allocated outputs.  A skipped output is an empty 0 x 0 null
// tensor, as the MEX drivers return empty matrices.  Outputs by position:
//   vl_nnconv : forward [y]             backward [dzdx, dzdf, dzdb]
//   vl_nnconvt: forward [y]             backward [dzdx, dzdf, dzdb]
//   vl_nnbnorm: forward [y, moments]    backward [dzdx, dzdg, dzdb, moments]
//   vl_nnpool : forward [y]             backward [dzdx]
//   vl_taccum : [alpha*a + beta*b]; nothing with 'InPlace' (a itself is updated)
//   vl_nnloss : forward [y] (1 x 1 on the device)   backward [dzdx]
//   vl_nnrelu : forward [y]             backward [dzdx]
//   vl_nnsoftmax: forward [y]           backward [dzdx]
ErrorCode vl_nnconv(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in,
                    std::string& message);
ErrorCode vl_nnconvt(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in,
                     std::string& message);
ErrorCode vl_nnbnorm(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in,
                     std::string& message);
ErrorCode vl_nnpool(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in,
                    std::string& message);
ErrorCode vl_taccum(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in,
                    std::string& message);
// vl_nnrelu(x [, dzdy], 'leak', value)  (matlab/vl_nnrelu.m:33-55; a MATLAB function in the reference)
ErrorCode vl_nnrelu(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in,
                    std::string& message);
// vl_nnsoftmax(x [, dzdy])  (matlab/vl_nnsoftmax.m:20-28; a MATLAB function in the reference)
ErrorCode vl_nnsoftmax(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in,
                       std::string& message);
// vl_nnloss(x, c [, dzdy], 'loss', name, 'instanceWeights', w, 'normalise', tf, 'threshold', t, 'topK', k)
// (matlab/vl_nnloss.m:129-142; a MATLAB function in the reference).  x: single, on the device.  c and the instance
// weights: on the device (single) or host arrays (copied over).  dzdy: a host scalar, or empty for the forward mode.
ErrorCode vl_nnloss(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in,
                    std::string& message);

} }  // namespace vl::frontend
#endif
