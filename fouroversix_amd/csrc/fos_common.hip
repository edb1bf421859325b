// Version and error strings of the C ABI.
#include "fouroversix_hip.h"

extern "C" int fos_version(void) { return 100; }

extern "C" const char *fos_error_string(int code) {
    switch (code) {
        case FOS_OK: return "success";
        case FOS_E_BAD_SHAPE: return "bad shape: a dimension is non-positive, too large or not a supported multiple";
        case FOS_E_BAD_ALIGNMENT: return "bad alignment: a pointer or leading dimension is not aligned as documented";
        case FOS_E_UNSUPPORTED: return "unsupported format / scale rule / rounding style / element type";
        case FOS_E_NULL_POINTER: return "null pointer argument";
        case FOS_E_WORKSPACE: return "workspace missing or smaller than the size query reports";
        case FOS_E_LAUNCH: return "kernel launch failed";
        default: return "unknown error code";
    }
}
