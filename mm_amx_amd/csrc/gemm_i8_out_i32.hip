// i8 inputs (v_mfma_i32_32x32x32_i8), i32 outputs: the MFMA tile GEMM instantiations of this pair of types
// (one translation unit per pair, so that they compile side by side).
#include "gemm_tile.hpp"

namespace mmx {

int launch_tiles_i8_out_i32(const GemmArgs& g, TileCfg t, int mode, int grid, hipStream_t st) {
    return launch_tiles<int8_t, int32_t>(g, t, mode, grid, st);
}

}  // namespace mmx
