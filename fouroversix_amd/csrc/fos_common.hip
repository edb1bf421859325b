// Version and error strings of the C ABI, and the tuning overrides.
#include <cstdlib>
#include <mutex>

#include "fos_tuning.h"
#include "fouroversix_hip.h"

namespace fos {
namespace {
Tuning g_tuning;
std::once_flag g_tuning_once;
int env_int(const char *name) {
    const char *e = getenv(name);
    return e ? atoi(e) : 0;
}
void load_tuning() {
    g_tuning.gemm_tile = env_int("FOS_GEMM_TILE");
    g_tuning.gemm_splitk = env_int("FOS_GEMM_SPLITK");
    g_tuning.mx_tile = env_int("FOS_MX_TILE");
    g_tuning.mx_quant = env_int("FOS_MX_QUANT");
    g_tuning.quant_grid = env_int("FOS_QUANT_GRID");
    g_tuning.amax_grid = env_int("FOS_AMAX_GRID");
    g_tuning.quant_map = env_int("FOS_QUANT_MAP");
    g_tuning.quant_passes = env_int("FOS_QUANT_PASSES");
    g_tuning.amax_units = env_int("FOS_AMAX_UNITS");
}
}  // namespace
const Tuning &tuning() {
    std::call_once(g_tuning_once, load_tuning);
    return g_tuning;
}
}  // namespace fos

extern "C" void fos_tuning_reload(void) {
    (void)fos::tuning();
    fos::load_tuning();
}

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
