// Library-level entry points: ABI version and error text.
#include "common.h"

extern "C" int slayer_abi_version(void) { return SLAYER_ABI_VERSION; }

extern "C" const char* slayer_error_string(int code) {
    switch (code) {
        case 0: return "success";
        case SLAYER_EINVAL: return "slayer_hip: inconsistent sizes";
        case SLAYER_ENULL: return "slayer_hip: required pointer is NULL";
        case SLAYER_ERANGE: return "slayer_hip: size beyond what the kernels index";
        case SLAYER_ESCRATCH: return "slayer_hip: size beyond the library's built-in scratch buffer";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "slayer_hip: unknown error code";
}
