// Parallel (all tokens at once) forms of the linear attention: the f32 block-tiled
// normalised form of src/kernel/linear_attention.rs:11-115 and the bf16 MFMA chunked
// prefill.  Filled in below as the kernels land.
#include "bdh_internal.h"

extern "C" {

int bdh_fused_state_aligned(bdh_ctx *ctx, int, int, int, int, int, const float *, const float *, const float *,
                            const float *, int, const int32_t *, int, int, int, float *) {
  if (!ctx) return BDH_E_INVAL;
  return bdh_fail(ctx, BDH_E_UNSUPPORTED, "bdh_fused_state_aligned is not implemented yet");
}

int bdh_prefill_chunked(bdh_ctx *ctx, int, int, int, int, int, const uint16_t *, const uint16_t *, const float *,
                        int64_t, float *, float *) {
  if (!ctx) return BDH_E_INVAL;
  return bdh_fail(ctx, BDH_E_UNSUPPORTED, "bdh_prefill_chunked is not implemented yet");
}

}  // extern "C"
