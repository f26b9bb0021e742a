// Error strings and the ABI version of the kernel library.
#include "common.h"
#include "yalm_hip.h"

extern "C" const char* yalm_error_string(int code) {
  switch (code) {
    case YALM_OK: return "ok";
    case YALM_ERR_ARG: return "argument refused by the kernel (unsupported size or option)";
    case YALM_ERR_DTYPE: return "unknown dtype code";
    default: return hipGetErrorString((hipError_t)code);
  }
}

extern "C" int yalm_abi_version(void) { return 12; }
