// fp8 (OCP e4m3fn / e5m2) MFMA GEMMs, per-tensor scales, optional bias, bf16 /
// e4m3 / fp32 output: the 256x256 ping-pong kernel (v_mfma_f32_32x32x64_f8f6f4)
// for large shapes, the generic tiled kernel otherwise.
#include "gemm_pingpong.cuh"
#include "gemm_tile.cuh"

namespace w8a8 {

bool launch_gemm_fp8_tiled(const GemmArgs& g, int fmt, hipStream_t stream) {
    if (!tiled_shape_ok(g)) return false;
    const bool big = pingpong_shape_ok(g);
    if (fmt) {
        if (big) launch_pingpong<Op32F8<1>, SCALE_TENSOR>(g, stream);
        else launch_tiled_auto<OpF8<1>, SCALE_TENSOR>(g, stream);
    } else {
        if (big) launch_pingpong<Op32F8<0>, SCALE_TENSOR>(g, stream);
        else launch_tiled_auto<OpF8<0>, SCALE_TENSOR>(g, stream);
    }
    return true;
}

}  // namespace w8a8
