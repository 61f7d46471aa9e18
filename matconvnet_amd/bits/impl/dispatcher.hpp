// Picks the back-end of an operator call from its tensor arguments.  Same rule as the reference
// (matlab/src/bits/impl/dispatcher.hpp:30-53): the LAST non-null tensor argument decides device and
// element type.  This library holds one back-end only -- the HIP device, single and double precision for the
// operators the reference has (the calls it does not have -- fused, packed-ahead, accumulating -- are single
// precision only); any other combination is reported as VLE_Unsupported with a message instead of silently
// running elsewhere.
#ifndef MCN_AMD_BITS_IMPL_DISPATCHER_HPP
#define MCN_AMD_BITS_IMPL_DISPATCHER_HPP

#include <string>

#include "../../../include/mcn_hip.h"
#include "../data.hpp"
#include "../hiphelper.hpp"

namespace vl { namespace impl {

struct tensor_type {
  DeviceType deviceType = VLDT_CPU;
  DataType dataType = VLDT_Float;
  bool any = false;
};

inline void noteTensor(tensor_type& tt, Tensor const& t) {
  if (!t.isNull()) {
    tt.deviceType = t.getDeviceType();
    tt.dataType = t.getDataType();
    tt.any = true;
  }
}
template <typename T> inline void noteTensor(tensor_type&, T const&) {}

inline void scanTensors(tensor_type&) {}
template <typename First, typename... Rest>
inline void scanTensors(tensor_type& tt, First const& first, Rest const&... rest) {
  noteTensor(tt, first);
  scanTensors(tt, rest...);
}

template <typename... Types>
inline tensor_type findTensorType(Types const&... args) {
  tensor_type tt;
  scanTensors(tt, args...);
  return tt;
}

// VLE_Success when the call can run on the HIP back-end, else the error (recorded in the context).
inline ErrorCode requireHipFloat(Context& context, tensor_type const& tt, char const* op) {
  if (tt.deviceType != VLDT_GPU)
    return context.setError(VLE_Unsupported,
                            (std::string(op) + ": tensors are on the CPU; this library implements the GPU (HIP, gfx950) device only").c_str());
  if (tt.dataType != VLDT_Float)
    return context.setError(VLE_Unsupported, (std::string(op) + ": only single precision is implemented on the HIP device").c_str());
  return VLE_Success;
}

// The same for operators that also have double precision kernels; *isDouble tells which to call.
inline ErrorCode requireHip(Context& context, tensor_type const& tt, char const* op, bool* isDouble) {
  *isDouble = false;
  if (tt.deviceType != VLDT_GPU) return requireHipFloat(context, tt, op);
  if (tt.dataType == VLDT_Double) {
    *isDouble = true;
    return VLE_Success;
  }
  return requireHipFloat(context, tt, op);
}

// Turns a C-ABI return code into a vl::ErrorCode recorded in the context (codes are numerically equal).
inline ErrorCode fromAbi(Context& context, int rc, char const* op) {
  if (rc == MCN_SUCCESS) return VLE_Success;
  ErrorCode e = (rc > 0 && rc <= (int)VLE_Interrupted) ? (ErrorCode)rc : VLE_Unknown;
  if (e == VLE_Cuda) context.getHipHelper().catchHipError(op);
  context.setError(e, mcn_last_error_message());
  return context.passError(e, op);
}

inline int asInt(std::size_t v) { return (int)v; }

} }  // namespace vl::impl
#endif
