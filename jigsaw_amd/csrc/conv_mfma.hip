// placeholder while the direct kernels are validated
#include "conv_common.h"
namespace jg {
bool mfma_fwd_supported(const ConvGeom&, int) { return false; }
bool mfma_dgrad_supported(const ConvGeom&, int) { return false; }
bool mfma_wgrad_supported(const ConvGeom&, int) { return false; }
size_t mfma_fwd_workspace(const ConvGeom&) { return 0; }
size_t mfma_dgrad_workspace(const ConvGeom&) { return 0; }
size_t mfma_wgrad_workspace(const ConvGeom&) { return 0; }
int mfma_fwd(void*, const void*, const void*, const void*, const ConvGeom&, void*, size_t, hipStream_t) { return JG_ERR_UNSUPPORTED; }
int mfma_dgrad(void*, const void*, const void*, const ConvGeom&, void*, size_t, hipStream_t) { return JG_ERR_UNSUPPORTED; }
int mfma_wgrad(void*, const void*, const void*, const ConvGeom&, void*, size_t, hipStream_t) { return JG_ERR_UNSUPPORTED; }
}  // namespace jg
