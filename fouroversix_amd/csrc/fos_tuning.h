// Kernel-choice overrides for tuning runs and tests.  The FOS_* environment variables are
// read once, when the first call needs them (and again on fos_tuning_reload()); the entry
// points themselves only read these integers.  0 = no override.
#pragma once

#include <atomic>

namespace fos {

struct Tuning {
    std::atomic<int> gemm_tile{0};    // FOS_GEMM_TILE
    std::atomic<int> gemm_splitk{0};  // FOS_GEMM_SPLITK
    std::atomic<int> mx_tile{0};      // FOS_MX_TILE
    std::atomic<int> mx_quant{0};     // FOS_MX_QUANT: 1 = the tile kernel of the MXFP4 quantizer also for aligned inputs
    std::atomic<int> quant_grid{0};   // FOS_QUANT_GRID
    std::atomic<int> amax_grid{0};    // FOS_AMAX_GRID
    std::atomic<int> amax_units{0};   // FOS_AMAX_UNITS: -1 = flat pass 1 also ahead of a streaming pass 2
    std::atomic<int> quant_map{0};    // FOS_QUANT_MAP: tile order of the streaming quantize kernels (1 + TileMap)
    std::atomic<int> quant_passes{0};  // FOS_QUANT_PASSES: 1 = fos_quantize stops after the tensor-maximum pass (timing runs: what pass 2 adds to a step)
};

const Tuning &tuning();

}  // namespace fos
