// Instantiations of the pass-2 kernel for NVFP4 with round-to-nearest (the fast
// formulation of fos_quantize_fast.h), kept in their own translation unit so that the
// library builds in parallel.
#include "fos_quantize_kernel.h"

namespace fos {

template <int RULE>
static void by_dim(QuantParams &p, bool two_d, bool aligned, hipStream_t s) {
    if (two_d) launch_quantize<true, FOS_DTYPE_NVFP4, RULE, FOS_ROUND_NEAREST, true>(p, aligned, s);
    else launch_quantize<true, FOS_DTYPE_NVFP4, RULE, FOS_ROUND_NEAREST, false>(p, aligned, s);
}

void launch_quantize_nvfp4_rtn(QuantParams &p, int rule, bool two_d, bool aligned, hipStream_t s) {
    switch (rule) {
        case FOS_RULE_STATIC_6:
        case FOS_RULE_STATIC_4:
            // the two static rules differ only in the host-computed constants
            by_dim<FOS_RULE_STATIC_6>(p, two_d, aligned, s);
            break;
        case FOS_RULE_MAE: by_dim<FOS_RULE_MAE>(p, two_d, aligned, s); break;
        case FOS_RULE_MSE: by_dim<FOS_RULE_MSE>(p, two_d, aligned, s); break;
        default: by_dim<FOS_RULE_ABS_MAX>(p, two_d, aligned, s); break;
    }
}

}  // namespace fos
