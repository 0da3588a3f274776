// e4m3fn tiled MFMA GEMM with 128-block scales: one 16x16x128 MFMA spans
// exactly one scale block, so each K slab's partial product is promoted into
// the fp32 accumulator with sa[m,kb] * sb[n/128,kb].
#include "gemm_tile.cuh"

namespace w8a8 {

bool launch_gemm_fp8_block128_tiled(const GemmArgs& g, hipStream_t stream) {
    if (!tiled_shape_ok(g) || (g.k & 127) != 0) return false;
    launch_tiled_auto<OpF8<0>, SCALE_BLOCK128>(g, stream);
    return true;
}

}  // namespace w8a8
