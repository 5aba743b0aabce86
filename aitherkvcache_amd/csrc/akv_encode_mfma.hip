// MFMA encode path for fp16 input, head_dim 128 (placeholder: not built yet, the general
// kernel in akv_codec.hip serves every case).
#include "akv_common.h"

int akv_prepare_rotation_mfma(const float* rotation, int d, void* prep, hipStream_t stream) {
  (void)rotation; (void)d; (void)prep; (void)stream;
  return AKV_OK;
}

int akv_encode_mfma_try(const akv_gen_args& a, bool paged, int x_dtype, int d, int bits,
                        const void* rot_prep, hipStream_t stream) {
  (void)a; (void)paged; (void)x_dtype; (void)d; (void)bits; (void)rot_prep; (void)stream;
  return AKV_ERR_UNSUPPORTED;
}
