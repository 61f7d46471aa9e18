// placeholder: MFMA kernels not yet enabled
#include "conv_common.hpp"
namespace mcn {
bool conv_mfma_forward_supported(const ConvP&) { return false; }
bool conv_mfma_backward_data_supported(const ConvP&) { return false; }
bool conv_mfma_backward_filter_supported(const ConvP&) { return false; }
size_t conv_mfma_workspace_bytes(const ConvP&, int) { return 0; }
int conv_forward_mfma(hipStream_t, const ConvP&, float*, float, const float*, float, const float*, const float*, void*, size_t) { return fail(MCN_UNSUPPORTED, "n/a"); }
int conv_backward_data_mfma(hipStream_t, const ConvP&, float*, const float*, const float*, void*, size_t) { return fail(MCN_UNSUPPORTED, "n/a"); }
int conv_backward_filter_mfma(hipStream_t, const ConvP&, float*, const float*, const float*, void*, size_t) { return fail(MCN_UNSUPPORTED, "n/a"); }
}
