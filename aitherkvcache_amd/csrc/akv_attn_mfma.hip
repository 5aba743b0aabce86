// MFMA paged decode attention for 4-bit, head_dim 128 (placeholder: not built yet, the
// general kernel in akv_attn.hip serves every case).
#include "akv_attn_common.h"

int akv_attn_mfma_try(const akv_attn_args& a, int d, int bits, int grid, hipStream_t stream) {
  (void)a; (void)d; (void)bits; (void)grid; (void)stream;
  return AKV_ERR_UNSUPPORTED;
}
