// bfloat16 attention on the matrix cores (placeholder until the MFMA kernels
// land: it refuses every shape, so the float32-arithmetic kernels run instead).
#include "common.h"
#include "yalm_hip.h"

int yalm_attn_prefill_bf16_mfma(const void*, const void*, const void*, void*, const int*, const int*, const int*, int,
                                int, int, int, int, int, hipStream_t) {
  return YALM_ERR_ARG;
}
int yalm_attn_decode_bf16_mfma(const void*, const void*, const void*, const int*, int, int, const int*, const int*,
                               void*, float*, int, int, int, int, int, int, int, hipStream_t) {
  return YALM_ERR_ARG;
}
