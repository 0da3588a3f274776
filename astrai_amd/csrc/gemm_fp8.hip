// fp8 (OCP e4m3fn / e5m2) tiled MFMA GEMM (v_mfma_f32_16x16x128_f8f6f4),
// per-tensor scales, optional bias, bf16 / e4m3 / fp32 output.
#include "gemm_tile.cuh"

namespace w8a8 {

bool launch_gemm_fp8_tiled(const GemmArgs& g, int fmt, hipStream_t stream) {
    if (!tiled_shape_ok(g)) return false;
    if (fmt)
        launch_tiled_auto<OpF8<1>, SCALE_TENSOR>(g, stream);
    else
        launch_tiled_auto<OpF8<0>, SCALE_TENSOR>(g, stream);
    return true;
}

}  // namespace w8a8
