// output = alpha*a + beta*b on the HIP device: one pass (the reference copies a, scales the copy with BLAS scal and
// adds b with BLAS axpy, matlab/src/vl_taccummex.cu:57-74; the kernel keeps that pair's roundings).
#include "accumulate.hpp"

#include "impl/dispatcher.hpp"

namespace vl {

ErrorCode accumulate(Context& context, Tensor output, double alpha, Tensor a, double beta, Tensor b) {
  using namespace vl::impl;
  tensor_type tt = findTensorType(output, a, b);
  bool isDouble;
  ErrorCode e = requireHip(context, tt, "accumulate", &isDouble);
  if (e != VLE_Success) return e;
  const std::size_t n = a.getNumElements();
  if (b.getNumElements() != n || output.getNumElements() != n)
    return context.setError(VLE_IllegalArgument, "accumulate: OUTPUT, A and B do not have the same number of elements");
  int rc = isDouble ? mcn_taccum_f64(context.getHipHelper().getStream(), (double*)output.getMemory(), alpha,
                                     (double const*)a.getMemory(), beta, (double const*)b.getMemory(), n)
                    : mcn_taccum(context.getHipHelper().getStream(), (float*)output.getMemory(), (float)alpha,
                                 (float const*)a.getMemory(), (float)beta, (float const*)b.getMemory(), n);
  return fromAbi(context, rc, "accumulate");
}

}  // namespace vl
