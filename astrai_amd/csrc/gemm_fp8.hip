// fp8 (OCP e4m3fn / e5m2) MFMA GEMMs, per-tensor scales (optional bias, bf16 /
// e4m3 / fp32 output) or one scale per activation row and per weight row (bf16 output).
// Large shapes run 256x256 tiles: the four-wave 128x128-register-tile kernel for bf16
// output (v_mfma_f32_16x16x128_f8f6f4, or v_mfma_f32_32x32x64_f8f6f4 for an odd number of
// K slabs), the eight-wave ping-pong kernel (32x32x64) for the other outputs; bf16 shapes with too few of
// those tiles for the chip run 128x128 tiles of the same instruction; the generic
// tiled kernel takes everything else.
#include "gemm_wave128.cuh"
#include "gemm_wave128_q16.cuh"
#include "gemm_mid128.cuh"
#include "gemm_small64.cuh"
#include "gemm_tile.cuh"

namespace w8a8 {

namespace {
// The four-wave kernel has two instances: on the 16x16x128 MFMA (faster under the board's power
// cap: 49.6 against 52.3 us at 4096^3 on normally distributed operands) when the slab count is
// even -- its loop walks two slabs a turn --, else on the 32x32x64 MFMA.
template <int Fmt, int ScaleKind>
void launch_big(const GemmArgs& g, hipStream_t stream) {
    if ((g.k & 255) == 0) launch_wave128_q16<Fmt, ScaleKind>(g, stream);
    else launch_wave128<Op32F8<Fmt>, ScaleKind>(g, stream);
}
template <int Fmt, int ScaleKind>
void launch_for(const GemmArgs& g, hipStream_t stream) {
#ifndef W8A8_NO_WAVE128
    if (wave128_shape_ok(g)) {
        if (const int r = ragged_tail_rows(g)) {
            GemmArgs head, tail;
            split_rows(g, r, ScaleKind == SCALE_ROWCOL, head, tail);
            if (wave128_shape_ok(head) && launch_gemv_fp8(tail, Fmt, ScaleKind, stream))   // (disjoint rows: either order)
                return launch_big<Fmt, ScaleKind>(head, stream);
        }
        return launch_big<Fmt, ScaleKind>(g, stream);
    }
#endif
    if (pingpong_shape_ok(g)) return launch_pingpong<Op32F8<Fmt>, ScaleKind>(g, stream);
    if (mid128_shape_ok(g)) return launch_mid128<Op32F8<Fmt>, ScaleKind>(g, stream);
    if (small64_shape_ok(g)) return launch_small64<Op32F8<Fmt>, ScaleKind>(g, stream);
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
