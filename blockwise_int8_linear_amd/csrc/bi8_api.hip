// Version and error-string entry points of libbi8.
#include "bi8_common.h"

extern "C" int bi8_version(void) { return 5; }

extern "C" const char *bi8_strerror(int code) {
    switch (code) {
    case BI8_OK: return "success";
    case BI8_ERR_NULL_POINTER: return "null pointer argument";
    case BI8_ERR_BAD_DTYPE: return "unsupported element type (0 = fp32, 1 = bf16, 2 = fp16)";
    case BI8_ERR_BAD_BLOCK: return "unsupported block size";
    case BI8_ERR_BAD_SHAPE: return "negative size or leading dimension smaller than the row length";
    case BI8_ERR_TOO_LARGE: return "problem too large for one launch";
    case BI8_ERR_UNSUPPORTED: return "arguments outside what this entry point covers";
    case BI8_ERR_SCRATCH_TOO_SMALL: return "the problem wants more scratch memory than the library's static buffer holds";
    default: break;
    }
    if (code >= BI8_ERR_HIP_BASE) return hipGetErrorString((hipError_t)(code - BI8_ERR_HIP_BASE));
    return "unknown error";
}
