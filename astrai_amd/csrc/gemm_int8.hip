// int8 x int8 -> int32 MFMA GEMMs, per-token x per-channel dequant epilogue.
// Large shapes run v_mfma_i32_32x32x32_i8 on 256x256 tiles: the four-wave
// 128x128-register-tile kernel for bf16 output, the eight-wave ping-pong kernel
// for int32 output; shapes with too few of those tiles for the chip run 128x128
// tiles of the same instruction; the generic tiled kernel takes everything else.
#include "gemm_wave128.cuh"
#include "gemm_mid128.cuh"
#include "gemm_small64.cuh"
#include "gemm_tile.cuh"

namespace w8a8 {

bool launch_gemm_int8_tiled(const GemmArgs& g, hipStream_t stream, bool tail_on_decode_kernel) {
    if (!tiled_shape_ok(g)) return false;
#ifndef W8A8_NO_WAVE128
    if (wave128_shape_ok(g)) {
        if (const int r = tail_on_decode_kernel ? ragged_tail_rows(g) : 0) {
            GemmArgs head, tail;
            split_rows(g, r, true, head, tail);
            if (wave128_shape_ok(head) && launch_gemv_int8(tail, stream)) {   // (disjoint rows: either order)
                launch_wave128<Op32I8, SCALE_ROWCOL>(head, stream);
                return true;
            }
        }
        launch_wave128<Op32I8, SCALE_ROWCOL>(g, stream);
    } else
#endif
    if (pingpong_shape_ok(g))
        launch_pingpong<Op32I8, SCALE_ROWCOL>(g, stream);
    else if (mid128_shape_ok(g))
        launch_mid128<Op32I8, SCALE_ROWCOL>(g, stream);
    else if (small64_shape_ok(g))
        launch_small64<Op32I8, SCALE_ROWCOL>(g, stream);
    else
        launch_tiled_auto<OpI8, SCALE_ROWCOL>(g, stream);
    return true;
}

bool launch_gemm_int8_swiglu(const GemmArgs& g, hipStream_t stream) {
    if (!tiled_shape_ok(g) || !wave128_shape_ok(g) || (g.n & 127) != 0 || g.bias != nullptr || !g.row_max)
        return false;
    launch_wave128<Op32I8, SCALE_ROWCOL, EPI_SWIGLU>(g, stream);
    return true;
}

bool launch_gemm_int8_resid(const GemmArgs& g, hipStream_t stream) {
    if (!g.resid || g.out_kind != OUT_BF16) return false;
    if (g.m <= 128 && launch_gemv_int8(g, stream)) return true;
    if (!tiled_shape_ok(g) || !wave128_shape_ok(g) || g.bias != nullptr) return false;
    if (const int r = ragged_tail_rows(g)) {
        GemmArgs head, tail;
        split_rows(g, r, true, head, tail);
        if (wave128_shape_ok(head) && launch_gemv_int8(tail, stream)) {
            launch_wave128<Op32I8, SCALE_ROWCOL, EPI_RESID>(head, stream);
            return true;
        }
    }
    launch_wave128<Op32I8, SCALE_ROWCOL, EPI_RESID>(g, stream);
    return true;
}

bool launch_gemm_int8_rope_cache_large(const GemmArgs& g, const RopeCacheArgs& rc, hipStream_t stream) {
    if (!tiled_shape_ok(g) || !wave128_shape_ok(g) || (g.n & 127) != 0 || g.bias != nullptr) return false;
    if (rc.head_dim != 128 || g.m >= (1 << 23) || g.m != rc.batch * rc.seq || g.n != (rc.n_heads + 2 * rc.n_kv_heads) * 128) return false;
    // destinations are addressed with 32-bit byte offsets below the out-of-range marker
    const int64_t lim = (int64_t)1 << 31;
    if ((int64_t)g.m * rc.n_heads * 256 >= lim || (int64_t)rc.batch * rc.n_kv_heads * rc.max_len * 256 >= lim)
        return false;
    launch_wave128<Op32I8, SCALE_ROWCOL, EPI_ROPE>(g, stream, rc);
    return true;
}

}  // namespace w8a8
