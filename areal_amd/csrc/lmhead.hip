// Fused lm_head path (placeholder entry points until the MFMA kernels land).
#include "device_utils.h"

extern "C" int64_t aa_lmhead_workspace_bytes(int64_t T, int64_t H, int64_t V) {
  (void)T; (void)H; (void)V;
  return 0;
}

extern "C" int aa_lmhead_fwd(const void*, const void*, int64_t, int64_t, int64_t, const int64_t*, float, float*,
                             float*, float*, float*, void*, int64_t, void*) {
  return AA_ERR_UNSUPPORTED;
}

extern "C" int aa_lmhead_bwd(const void*, const void*, int64_t, int64_t, int64_t, const int64_t*, float, const float*,
                             const float*, const float*, const float*, void*, float*, void*, int64_t, void*) {
  return AA_ERR_UNSUPPORTED;
}
