// Library identity and error strings.
#include "amct_common.h"

extern "C" int amct_hip_version(void) { return 100; }

extern "C" const char* amct_hip_strerror(int code) {
    switch (code) {
        case AMCT_OK: return "ok";
        case AMCT_E_BADARG: return "bad argument (null pointer, negative size or unknown enum)";
        case AMCT_E_UNSUPPORTED: return "shape or combination not supported by the kernels";
        case AMCT_E_ALIGN: return "alignment or divisibility requirement violated";
        case AMCT_E_HIP: return "HIP runtime reported a launch error";
        default: return "unknown error code";
    }
}
