// bfloat16 GEMMs on the matrix cores (placeholder until the MFMA kernels land:
// it refuses every shape, so the float32-arithmetic kernel runs instead).
#include "common.h"
#include "yalm_hip.h"

int yalm_gemm_bf16_mfma(const void*, const void*, void*, int, int, int, int, int, hipStream_t) { return YALM_ERR_ARG; }
