// Library version and the text of the return codes of every entry point.

#include <hip/hip_runtime.h>
#include "proteus_hip.h"

extern "C" int proteus_version(void) { return PROTEUS_VERSION; }

extern "C" const char* proteus_strerror(int code) {
    switch (code) {
        case PROTEUS_OK:                return "ok";
        case PROTEUS_ERR_NULL_POINTER:  return "a required pointer is NULL";
        case PROTEUS_ERR_BAD_SHAPE:     return "a dimension is not positive or exceeds the supported maximum";
        case PROTEUS_ERR_BAD_HEAD_DIM:  return "d_head must be 32, 64 or 128";
        case PROTEUS_ERR_BAD_LAYOUT:    return "unknown coords_layout";
        case PROTEUS_ERR_BAD_ALIGNMENT: return "a pointer is not 16-byte aligned";
        case PROTEUS_ERR_BAD_TUNING:    return "unknown tuning selector";
        case PROTEUS_ERR_UNSUPPORTED:   return "option not implemented";
        case PROTEUS_ERR_TOO_LARGE:     return "size beyond the fixed capacity of this entry point";
        case PROTEUS_ERR_BAD_OPERAND_TYPE: return "operand_type must be PROTEUS_OPERAND_BF16, or PROTEUS_OPERAND_F16 with the beta-weighted logits";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error code";
}
