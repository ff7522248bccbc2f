// Internal entry of the fused logits kernel for callers inside the library.
#pragma once
#include <cstdint>

#include "../../include/areal_amd.h"

namespace aa {

// aa_logits_ppo_fused with a row map for the gradient: row t of d(loss)/d(logits) is written to row out_rows[t] of
// dlogits, or not at all where out_rows[t] < 0 (which the caller uses for tokens whose gradient is known to be
// zero).  out_rows == nullptr is aa_logits_ppo_fused itself.  With a row map, dlogits must not alias logits.
int logits_ppo_fused_rows(const void* logits, int dtype, int64_t T, int64_t V, int64_t row_stride,
                          const int64_t* labels, float inv_temperature, int64_t T_active, const float* prox_logp,
                          const float* adv, const uint8_t* mask_eff, const float* behave_w, const aa_ppo_params* params,
                          const int32_t* n_valid, const float* grad_scale, float* logp, float* entropy, float* vmax,
                          float* vmin, float* stat_loss, float* ratio, uint8_t* flags, void* dlogits,
                          const int32_t* out_rows, int32_t* work, void* stream);

// aa_logits_bwd with the same kind of row map.
int logits_bwd_rows(const void* logits, int dtype, int64_t T, int64_t V, int64_t row_stride, const int64_t* labels,
                    float inv_temperature, const float* row_lse, const float* row_ez, const float* g_logp,
                    const float* g_entropy, int64_t T_active, void* dlogits, const int32_t* out_rows, void* stream);

}  // namespace aa
