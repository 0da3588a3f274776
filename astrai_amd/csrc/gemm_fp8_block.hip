// e4m3fn MFMA GEMM with 128-block scales (1x128 activation groups, 128x128
// weight blocks): the 256x256 ping-pong kernel for large shapes (a K slab is
// exactly one scale block; the promotion runs in place on the accumulators),
// 128x128 tiles of the same instruction for mid-size shapes (a slab's product scaled before it
// joins the accumulator), the generic tiled kernel otherwise (one 16x16x128 MFMA per scale
// block, partial product promoted with sa[m,kb] * sb[n/128,kb]).
#include "gemm_pingpong.cuh"
#include "gemm_mid128.cuh"
#include "gemm_small64.cuh"
#include "gemm_tile.cuh"

namespace w8a8 {

bool launch_gemm_fp8_block128_tiled(const GemmArgs& g, hipStream_t stream) {
    if (!tiled_shape_ok(g) || (g.k & 127) != 0) return false;
    if (pingpong_shape_ok(g) && (g.n & 7) == 0 && g.out_kind == OUT_BF16) {
        launch_pingpong<Op32F8<0>, SCALE_BLOCK128, PingPongCfgBlock>(g, stream);
        return true;
    }
    // the 256x256 configuration of the generic tiled kernel runs out of registers
    // with the per-block promotion; 128x128 and 64x64 do not
    const int64_t tiles128 = (int64_t)((g.m + 127) / 128) * ((g.n + 127) / 128);
    if (mid128_shape_ok(g))   // blocks of a few hundred to a few thousand tokens: 128 x 128 tiles of the 32x32x64 MFMA
        launch_mid128<Op32F8<0>, SCALE_BLOCK128>(g, stream);
    else if (small64_shape_ok(g))   // fewer tokens: 64 x 64 tiles behind a ring of stages
        launch_small64<Op32F8<0>, SCALE_BLOCK128>(g, stream);
    else if (tiles128 >= 192)
        launch_tiled<OpF8<0>, CfgMid, SCALE_BLOCK128>(g, stream);
    else
        launch_tiled<OpF8<0>, CfgSmall, SCALE_BLOCK128>(g, stream);
    return true;
}

}  // namespace w8a8
