// Error strings and the ABI version of the kernel library.
#include "common.h"
#include "yalm_hip.h"

extern "C" const char* yalm_error_string(int code) {
  switch (code) {
    case YALM_OK: return "ok";
    case YALM_ERR_ARG: return "argument refused by the kernel (unsupported size or option)";
    case YALM_ERR_DTYPE: return "unknown dtype code";
    case YALM_ERR_SCRATCH: return "the sizes need more scratch than the fixed device array of this entry point holds";
    default: return hipGetErrorString((hipError_t)code);
  }
}

extern "C" int yalm_abi_version(void) { return 24; }
