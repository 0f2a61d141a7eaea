// bf16 activations on int8-compressed weights (converted to bf16 between LDS and v_mfma_f32_32x32x16_bf16), i8 outputs:
// the MFMA tile GEMM instantiations of this pair of types (one translation unit per pair, so that they compile side by side).
#include "gemm_tile.hpp"

namespace mmx {

int launch_tiles_w8_out_i8(const GemmArgs& g, TileCfg t, int mode, int grid, hipStream_t st) {
    return launch_tiles<w8_t, int8_t>(g, t, mode, grid, st);
}

}  // namespace mmx
