// Any-shape fallback for the 8-bit NT GEMMs: one wave per 16(n) x 16(m) output
// tile, operands fetched with guarded byte loads straight into the MFMA
// registers. Used only where the tiled kernel's addressing assumptions fail
// (K not a multiple of 16, or tensors of 2 GiB and more); correctness over speed.
#include "gemm_tile.cuh"

namespace w8a8 {

namespace {

// 16 bytes of row `row` starting at byte k (zero outside the matrix)
__device__ __forceinline__ u32x4 guarded_chunk(const uint8_t* base, int64_t row, int64_t rows,
                                               int64_t k, int64_t K) {
    u32x4 v = {0, 0, 0, 0};
    if (row >= rows) return v;
    const uint8_t* p = base + row * K;
    uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int64_t kk = k + i;
        const uint32_t b = (kk < K) ? p[kk] : 0u;
        w[i >> 2] |= b << (8 * (i & 3));
    }
    v.x = w[0]; v.y = w[1]; v.z = w[2]; v.w = w[3];
    return v;
}

template <class Op, int ScaleKind>
__global__ __launch_bounds__(256) void gemm_generic_kernel(GemmArgs g) {
    using Acc = typename Op::Acc;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int lrow = lane & 15, lgrp = lane >> 4;
    const int tiles_n = (g.n + 15) / 16;
    const int tiles_m = (g.m + 15) / 16;
    const int64_t tile = (int64_t)blockIdx.x * 4 + wave;
    if (tile >= (int64_t)tiles_m * tiles_n) return;
    const int tm = (int)(tile / tiles_n), tn = (int)(tile % tiles_n);
    const int m = tm * 16 + lrow;           // this lane's activation row (second operand)
    const int nrow = tn * 16 + lrow;        // this lane's weight row (first operand)
    const auto* A = static_cast<const uint8_t*>(g.a);
    const auto* B = static_cast<const uint8_t*>(g.b);
    const int64_t K = g.k;
    const int kblocks = (int)(K >> 7);
    Acc acc = Acc{0, 0, 0, 0};
    for (int64_t k0 = 0; k0 < K; k0 += 128) {
        const int64_t kc = k0 + lgrp * 32;
        const u32x4 w0 = guarded_chunk(B, nrow, g.n, kc, K);
        const u32x4 w1 = guarded_chunk(B, nrow, g.n, kc + 16, K);
        const u32x4 x0 = guarded_chunk(A, m, g.m, kc, K);
        const u32x4 x1 = guarded_chunk(A, m, g.m, kc + 16, K);
        if constexpr (ScaleKind == SCALE_BLOCK128) {
            const int kb = (int)(k0 >> 7);
            const float sav = (m < g.m) ? g.sa[(size_t)m * kblocks + kb] : 0.0f;
            const float sbv = g.sb[(size_t)((tn * 16) >> 7) * kblocks + kb];
            const Acc part = Op::mma(w0, w1, x0, x1, Acc{0, 0, 0, 0});
            acc += part * (sav * sbv);
        } else {
            acc = Op::mma(w0, w1, x0, x1, acc);
        }
    }
    const EpilogueScalars es = load_epilogue_scalars<ScaleKind>(g);
    store_subtile<Op, ScaleKind>(g, es, acc, m, tn * 16 + lgrp * 4);
}

template <class Op, int ScaleKind>
void launch(const GemmArgs& g, hipStream_t stream) {
    const int64_t tiles = (int64_t)((g.m + 15) / 16) * ((g.n + 15) / 16);
    const int64_t blocks = (tiles + 3) / 4;
    note_kernel("generic");
    gemm_generic_kernel<Op, ScaleKind><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(g);
}

}  // namespace

void launch_gemm_generic(const GemmArgs& g, int op, int scale_kind, hipStream_t stream) {
    if (op == 0) {
        if (scale_kind == SCALE_ROWCOL) launch<OpI8, SCALE_ROWCOL>(g, stream);
        else launch<OpI8, SCALE_TENSOR>(g, stream);
    } else if (op == 1) {
        if (scale_kind == SCALE_BLOCK128) launch<OpF8<0>, SCALE_BLOCK128>(g, stream);
        else if (scale_kind == SCALE_ROWCOL) launch<OpF8<0>, SCALE_ROWCOL>(g, stream);
        else launch<OpF8<0>, SCALE_TENSOR>(g, stream);
    } else {
        if (scale_kind == SCALE_ROWCOL) launch<OpF8<1>, SCALE_ROWCOL>(g, stream);
        else launch<OpF8<1>, SCALE_TENSOR>(g, stream);
    }
}

}  // namespace w8a8
