// Skinny int8 W8A8 kernel for decode shapes (M <= 64): bandwidth-bound, the
// weight matrix is streamed from HBM exactly once.
//
// A workgroup of NW waves owns RG*16 weight rows; the waves split K into
// 256-byte chunks (wave w takes chunks w, w+NW, ...), so that at K = 4096 every
// wave issues all of its loads at once and the whole matrix is in flight
// together. Per chunk a lane loads 64 contiguous bytes of one weight row (four
// lanes cover the 256-byte chunk of that row) and the matching bytes of the
// activation rows; the products run on v_mfma_i32_16x16x64_i8 with the weight
// rows as the first operand, which leaves the MFMA pipe almost idle -- the
// kernel's speed is set by bytes in flight. The int32 partials of the waves are
// summed through LDS (integer addition is associative, so the split keeps the
// accumulator bit-exact) and the first waves run the dequant epilogue.
#include "gemm_tile.cuh"

namespace w8a8 {

namespace {

template <int RG, int MB, int NW>
__global__ __launch_bounds__(NW * 64) void gemv_int8_kernel(GemmArgs g) {
    __shared__ i32x4 red[NW][RG * MB][64];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int lrow = lane & 15, lgrp = lane >> 4;
    const int K = g.k;
    const int nchunks = K >> 8;
    const int n0 = blockIdx.x * (RG * 16);

    const __amdgpu_buffer_rsrc_t rw = make_rsrc(g.b, (uint32_t)g.n * (uint32_t)K);
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(g.a, (uint32_t)g.m * (uint32_t)K);

    uint32_t w_off[RG], x_off[MB];
#pragma unroll
    for (int r = 0; r < RG; ++r) {
        const int n = n0 + r * 16 + lrow;
        w_off[r] = (n < g.n) ? (uint32_t)n * (uint32_t)K + lgrp * 64 : kOutOfRange;
    }
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        const int m = b * 16 + lrow;
        x_off[b] = (m < g.m) ? (uint32_t)m * (uint32_t)K + lgrp * 64 : kOutOfRange;
    }

    i32x4 acc[RG][MB];
#pragma unroll
    for (int r = 0; r < RG; ++r)
#pragma unroll
        for (int b = 0; b < MB; ++b) acc[r][b] = i32x4{0, 0, 0, 0};

    for (int c = wave; c < nchunks; c += NW) {
        const uint32_t k0 = (uint32_t)c << 8;
        u32x4 wf[RG][4], xf[MB][4];
#pragma unroll
        for (int r = 0; r < RG; ++r)
#pragma unroll
            for (int j = 0; j < 4; ++j) wf[r][j] = buf_load16(rw, w_off[r] + j * 16, k0);
#pragma unroll
        for (int b = 0; b < MB; ++b)
#pragma unroll
            for (int j = 0; j < 4; ++j) xf[b][j] = buf_load16(rx, x_off[b] + j * 16, k0);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < RG; ++r)
#pragma unroll
                for (int b = 0; b < MB; ++b)
                    acc[r][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(
                        (i32x4)wf[r][j], (i32x4)xf[b][j], acc[r][b], 0, 0, 0);
    }

#pragma unroll
    for (int r = 0; r < RG; ++r)
#pragma unroll
        for (int b = 0; b < MB; ++b) red[wave][r * MB + b][lane] = acc[r][b];
    __syncthreads();

    const EpilogueScalars es = load_epilogue_scalars<SCALE_ROWCOL>(g);
    for (int t = wave; t < RG * MB; t += NW) {
        i32x4 sum = red[0][t][lane];
#pragma unroll
        for (int w = 1; w < NW; ++w) sum += red[w][t][lane];
        const int r = t / MB, b = t % MB;
        store_subtile<OpI8, SCALE_ROWCOL>(g, es, sum, b * 16 + lrow, n0 + r * 16 + lgrp * 4);
    }
}

template <int RG, int MB, int NW>
void launch(const GemmArgs& g, hipStream_t stream) {
    const int blocks = (g.n + RG * 16 - 1) / (RG * 16);
    gemv_int8_kernel<RG, MB, NW><<<dim3((unsigned)blocks), dim3(NW * 64), 0, stream>>>(g);
}

template <int RG, int MB>
void launch_nw(const GemmArgs& g, hipStream_t stream) {
    if ((g.k >> 8) >= 16)
        launch<RG, MB, 16>(g, stream);
    else
        launch<RG, MB, 4>(g, stream);
}

}  // namespace

bool launch_gemv_int8(const GemmArgs& g, hipStream_t stream) {
    if (g.m <= 0 || g.m > 64 || g.n <= 0 || g.k <= 0 || (g.k & 255) != 0) return false;
    const int64_t lim = (int64_t)1 << 31;
    if ((int64_t)g.n * g.k >= lim) return false;
    const int mb = (g.m + 15) / 16;
    switch (mb) {
        case 1: launch_nw<2, 1>(g, stream); break;
        case 2: launch_nw<1, 2>(g, stream); break;
        case 3: launch_nw<1, 3>(g, stream); break;
        default: launch_nw<1, 4>(g, stream); break;
    }
    return true;
}

}  // namespace w8a8
