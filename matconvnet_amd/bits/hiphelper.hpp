// Stream and error capture for the HIP device: what remains of the reference's CudaHelper
// (matlab/src/bits/datacu.hpp:36-158) once cuBLAS and cuDNN handles are gone.
#ifndef MCN_AMD_BITS_HIPHELPER_HPP
#define MCN_AMD_BITS_HIPHELPER_HPP

#include <string>

#include "data.hpp"

namespace vl {

class HipHelper {
 public:
  HipHelper();
  // The stream every operator of the owning context enqueues on (NULL = the default stream).
  void* getStream() const;
  ErrorCode setStream(void* stream);
  // Non-blocking look at the runtime's error state; records the text and returns VLE_Cuda on error.
  ErrorCode catchHipError(char const* description = NULL);
  std::string const& getLastHipErrorMessage() const;
  void clear();
  void invalidateGpu();

 private:
  void* stream;
  std::string lastMessage;
};

}  // namespace vl
#endif
