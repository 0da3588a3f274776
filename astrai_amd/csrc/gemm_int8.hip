// int8 x int8 -> int32 tiled MFMA GEMM (v_mfma_i32_16x16x64_i8), per-token x
// per-channel dequant epilogue.
#include "gemm_tile.cuh"

namespace w8a8 {

bool launch_gemm_int8_tiled(const GemmArgs& g, hipStream_t stream) {
    if (!tiled_shape_ok(g)) return false;
    launch_tiled_auto<OpI8, SCALE_ROWCOL>(g, stream);
    return true;
}

}  // namespace w8a8
