// placeholder until the MFMA backward kernels land
#include "jg_common.h"
namespace jg {
bool attn_mfma_bwd_supported(long long, int, int, int, int, bool) { return false; }
size_t attn_mfma_bwd_workspace(long long, int, int) { return 0; }
int attn_mfma_bwd(void*, void*, void*, const void*, const void*, const void*, const void*,
                  const void*, const float*, long long, int, int, float, void*, hipStream_t) {
  return JG_ERR_UNSUPPORTED;
}
}  // namespace jg
