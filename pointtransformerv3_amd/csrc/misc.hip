// Version and error strings of libptv3_hip.so.
#include "common.h"

extern "C" int ptv3_version(void) { return 1; }

extern "C" const char* ptv3_strerror(int rc) {
    switch (rc) {
        case PTV3_OK: return "ok";
        case PTV3_EINVAL: return "invalid argument (null pointer, negative size or unknown enum)";
        case PTV3_EDEPTH: return "depth outside 1..16 or code wider than 63 bits";
        case PTV3_EWORKSPACE: return "workspace too small";
        case PTV3_ESHAPE: return "shape not covered by the kernels";
        case PTV3_ESTATIC: return "input larger than the fixed on-device buffer of this entry point";
        default: return rc > 0 ? hipGetErrorString((hipError_t)rc) : "unknown error";
    }
}
