// int8 x int8 -> int32 MFMA GEMMs, per-token x per-channel dequant epilogue:
// the 256x256 ping-pong kernel (v_mfma_i32_32x32x32_i8) for large shapes, the
// generic tiled kernel otherwise.
#include "gemm_pingpong.cuh"
#include "gemm_tile.cuh"

namespace w8a8 {

bool launch_gemm_int8_tiled(const GemmArgs& g, hipStream_t stream) {
    if (!tiled_shape_ok(g)) return false;
    if (pingpong_shape_ok(g))
        launch_pingpong<Op32I8, SCALE_ROWCOL>(g, stream);
    else
        launch_tiled_auto<OpI8, SCALE_ROWCOL>(g, stream);
    return true;
}

}  // namespace w8a8
