// fp8 (OCP e4m3fn / e5m2) MFMA GEMMs, per-tensor scales (optional bias, bf16 /
// e4m3 / fp32 output) or one scale per activation row and per weight row (bf16 output). Large shapes run v_mfma_f32_32x32x64_f8f6f4 on 256x256
// tiles: the four-wave 128x128-register-tile kernel for bf16 output, the
// eight-wave ping-pong kernel for the other outputs; bf16 shapes with too few of
// those tiles for the chip run 128x128 tiles of the same instruction; the generic
// tiled kernel takes everything else.
#include "gemm_wave128.cuh"
#include "gemm_mid128.cuh"
#include "gemm_tile.cuh"

namespace w8a8 {

namespace {
template <int Fmt, int ScaleKind>
void launch_for(const GemmArgs& g, hipStream_t stream) {
#ifndef W8A8_NO_WAVE128
    if (wave128_shape_ok(g)) {
        if (const int r = ragged_tail_rows(g)) {
            GemmArgs head, tail;
            split_rows(g, r, ScaleKind == SCALE_ROWCOL, head, tail);
            if (wave128_shape_ok(head) && launch_gemv_fp8(tail, Fmt, ScaleKind, stream))   // (disjoint rows: either order)
                return launch_wave128<Op32F8<Fmt>, ScaleKind>(head, stream);
        }
        return launch_wave128<Op32F8<Fmt>, ScaleKind>(g, stream);
    }
#endif
    if (pingpong_shape_ok(g)) return launch_pingpong<Op32F8<Fmt>, ScaleKind>(g, stream);
    if (mid128_shape_ok(g)) return launch_mid128<Op32F8<Fmt>, ScaleKind>(g, stream);
    launch_tiled_auto<OpF8<Fmt>, ScaleKind>(g, stream);
}
}  // namespace

bool launch_gemm_fp8_tiled(const GemmArgs& g, int fmt, hipStream_t stream) {
    if (!tiled_shape_ok(g)) return false;
    if (fmt) launch_for<1, SCALE_TENSOR>(g, stream);
    else launch_for<0, SCALE_TENSOR>(g, stream);
    return true;
}

bool launch_gemm_fp8_rowcol_tiled(const GemmArgs& g, int fmt, hipStream_t stream) {
    if (!tiled_shape_ok(g) || g.out_kind != OUT_BF16) return false;
    if (fmt) launch_for<1, SCALE_ROWCOL>(g, stream);
    else launch_for<0, SCALE_ROWCOL>(g, stream);
    return true;
}

}  // namespace w8a8
