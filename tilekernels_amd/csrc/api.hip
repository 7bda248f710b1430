// Status strings and version of the C ABI.
#include "../../include/tk_quant.h"

extern "C" const char *tk_strerror(int status) {
    switch (status) {
        case TK_OK: return "ok";
        case TK_ERR_NULL_POINTER: return "null pointer";
        case TK_ERR_BAD_SHAPE: return "bad shape";
        case TK_ERR_BAD_DTYPE: return "unsupported input dtype";
        case TK_ERR_BAD_FORMAT: return "unsupported quantisation format";
        case TK_ERR_BAD_GROUP: return "unsupported group / block size";
        case TK_ERR_BAD_LAYOUT: return "scale-factor layout not usable with these options";
        case TK_ERR_BAD_MODE: return "mode not usable with these options";
        case TK_ERR_BAD_STRIDE: return "row stride or scale-factor leading dimension too small";
        case TK_ERR_MISALIGNED: return "pointer or stride not aligned for vector access";
        case TK_ERR_TOO_LARGE: return "problem too large for 32-bit tile indexing or for the library's static scratch";
        case TK_ERR_BAD_VALUE: return "clamp or floor value not usable";
        default: return status > 0 ? "hip error" : "unknown status";
    }
}

extern "C" int tk_version(void) { return TK_QUANT_VERSION; }
