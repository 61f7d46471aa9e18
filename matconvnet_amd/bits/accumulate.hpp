// vl::accumulate: output = alpha*a + beta*b, the tensor update behind vl_taccum (matlab/src/vl_taccummex.cu:48-113,
// where it is defined beside the MEX driver).  Same signature; output may share a's memory ("in place").
#ifndef MCN_AMD_BITS_ACCUMULATE_HPP
#define MCN_AMD_BITS_ACCUMULATE_HPP

#include "data.hpp"

namespace vl {

vl::ErrorCode accumulate(vl::Context& context, vl::Tensor output, double alpha, vl::Tensor a, double beta, vl::Tensor b);

}  // namespace vl
#endif
