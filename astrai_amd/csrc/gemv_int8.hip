// Skinny int8 W8A8 kernels for decode shapes (M <= 128): bandwidth-bound, the
// weight matrix is streamed from HBM exactly once (with the streaming cache hint:
// no line of it is used twice) and the MFMA pipe is almost idle -- speed is set by
// whole-line requests, by a steady, modest number of bytes in flight per wave and by
// how often the activation block is pulled out of L2 again. The int32 partials of
// the waves that split K are summed through LDS (integer addition is associative,
// so the split keeps the accumulator bit-exact) and the first waves run the dequant
// epilogue.
//
//  * M = 1: gemv_int8_dot_kernel, one wave per two weight rows, whole 1 KiB row
//    pieces straight into registers and v_dot4 on the vector ALU -- no LDS, no
//    barrier, every wave of the launch resident.
//  * 2 <= M <= 128: gemv_int8_rows_kernel (gemv_rows.cuh), about one workgroup per
//    compute unit with an equal share of the rows, a rolling ring of loads per wave,
//    one to eight groups of sixteen tokens per wave.
// Measured at N=11008, K=4096 (weights from HBM, graph replay): M=1 8.6 us, M=2..16
// 9.3-9.9, M=32 11.2, M=64 13.9, M=96 16.5, M=128 21.6 (the tiled GEMM kernel needs 29 us
// for any M <= 128; a kernel that staged the weights in LDS by direct-to-LDS loads and
// waited for each step took 19.9 us at M=64 and 30.6 us at M=128).
#include "gemm_tile.cuh"
#include "gemv_rows.cuh"

namespace w8a8 {

namespace {

// Single-token kernel (M = 1). A workgroup is one wave and owns R weight rows
// (two, or four for a short matrix); lane l holds bytes [16 l, 16 l + 16) of every 1 KiB K-step of its rows and
// of the token, so each load instruction moves one whole 1 KiB row piece (the
// request pattern HBM and the address coalescer like best) and the matching
// activation bytes sit in the same lane. The dot products run on the vector ALU
// (v_dot4_i32_i8, exact int32), which frees the kernel of LDS, barriers and
// operand shuffles: a wave needs few registers, so the ~5500 waves of an
// 11008-row matrix are all resident at once, each with four K-steps (8 KiB of
// weights) in flight. Two rows per wave measured faster than four or eight (8.6 us
// against 8.8 / 9.3 at 11008 x 4096, and the streaming hint is worth 1.2 us: 10.2 ->
// 8.8). Lane partials are summed across the wave at the end (integer addition: the
// split over lanes keeps the accumulator bit-exact). The vector ALU's dot4 rate
// carries one token comfortably, not several: from two tokens on the MFMA kernel
// is faster.
template <int R>
__global__ __launch_bounds__(64) void gemv_int8_dot_kernel(GemmArgs g) {
    const int lane = threadIdx.x;
    const int n0 = blockIdx.x * R;
    const int K = g.k;
    const __amdgpu_buffer_rsrc_t rw = make_rsrc(g.b, (uint32_t)g.n * (uint32_t)K);
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(g.a, (uint32_t)K);

    // rows past N start past the buffer's num_records: zeros
    uint32_t w_off[R];
#pragma unroll
    for (int r = 0; r < R; ++r) w_off[r] = (uint32_t)(n0 + r) * (uint32_t)K + lane * 16;

    // epilogue operands of the lane that will write row n0 + lane, requested
    // first so that their latency hides under the weight stream
    const int en = n0 + lane;
    const bool writer = lane < R && en < g.n;
    float e_sx = 0.0f, e_sw = 0.0f, e_b = 0.0f, e_r = 0.0f;
    if (writer && g.out_kind != OUT_ACC) {
        e_sx = g.sa[0];
        e_sw = g.sb[en];
        if (g.bias) e_b = bf16_to_f32(static_cast<const uint16_t*>(g.bias)[en]);
        if (g.resid) e_r = bf16_to_f32(static_cast<const uint16_t*>(g.resid)[en]);
    }

    int acc[R] = {};
    constexpr int kSteps = 8 / R;  // K-steps in flight: 8 KiB of weights per wave
#pragma unroll kSteps
    for (int k0 = 0; k0 < K; k0 += 1024) {
        const bool in = k0 + lane * 16 < K;
        u32x4 wv[R];
#pragma unroll
        for (int r = 0; r < R; ++r)
            wv[r] = buf_load16_aux<kAuxStream>(rw, in ? w_off[r] : kOutOfRange, (uint32_t)k0);
        const u32x4 xv = buf_load16(rx, in ? (uint32_t)(lane * 16) : kOutOfRange, (uint32_t)k0);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int a = acc[r];
            a = __builtin_amdgcn_sdot4((int)wv[r].x, (int)xv.x, a, false);
            a = __builtin_amdgcn_sdot4((int)wv[r].y, (int)xv.y, a, false);
            a = __builtin_amdgcn_sdot4((int)wv[r].z, (int)xv.z, a, false);
            a = __builtin_amdgcn_sdot4((int)wv[r].w, (int)xv.w, a, false);
            acc[r] = a;
        }
    }

    int mine = 0;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int v = acc[r];
#pragma unroll
        for (int off = 32; off; off >>= 1) v += __shfl_xor(v, off, kWave);
        if (lane == r) mine = v;
    }
    if (writer) {
        if (g.out_kind == OUT_ACC) {
            static_cast<int*>(g.out)[en] = mine;
        } else {
            // product and bias add rounded separately (no fused multiply-add): the
            // int8 epilogue is specified as elementwise fp32 on the exact integer
#pragma clang fp contract(off)
            const float scaled = (float)mine * e_sx * e_sw;
            uint16_t y = f32_to_bf16(scaled + e_b);
            if (g.resid) y = f32_to_bf16(bf16_to_f32(y) + e_r);   // bf16(y + residual) on the rounded y
            static_cast<uint16_t*>(g.out)[en] = y;
        }
    }
}

void launch_dot(const GemmArgs& g, hipStream_t stream) {
    note_kernel("gemv_dot");
    // a short matrix has too few rows to fill the chip with two-row waves' small windows
    if (g.n < 4096)
        gemv_int8_dot_kernel<4><<<dim3((unsigned)((g.n + 3) / 4)), dim3(64), 0, stream>>>(g);
    else
        gemv_int8_dot_kernel<2><<<dim3((unsigned)((g.n + 1) / 2)), dim3(64), 0, stream>>>(g);
}

// Rows kernel launch plan. The rows are dealt out over 256 x rounds workgroups, rounds
// being the smallest count that keeps a workgroup's range within 48 rows (three MFMA
// row groups); ranges are rounded up to four rows (one load instruction). Four waves
// split K; a short matrix (one row group) with K >= 2048 takes eight so that enough bytes
// are in flight (2048 x 5632: 5.7 us against 6.6 at M = 16; at K = 2048 the decoder's q|k|v
// and output projections gain 0.15 us each inside the decode step). Measured per
// shape against deeper rings (IB = 2..4), fewer / more waves and one workgroup per
// sixteen rows: this plan was the fastest or within 2% of it on every decoder shape.
struct RowsPlan { int rows_per_wg, rg, nw, blocks; };

RowsPlan plan_rows(const GemmArgs& g) {
    RowsPlan p;
    const int rounds = (g.n + 256 * 48 - 1) / (256 * 48);
    const int wgs = 256 * rounds;
    p.rows_per_wg = (((g.n + wgs - 1) / wgs) + 3) & ~3;
    p.rg = (p.rows_per_wg + 15) / 16;
    p.nw = (p.rg == 1 && g.k >= 2048) ? 8 : 4;
    p.blocks = (g.n + p.rows_per_wg - 1) / p.rows_per_wg;
    return p;
}

template <int RG, int MB, int NW, bool ROPE>
void launch_rows_inst(const GemmArgs& g, const RopeCacheArgs& rc, const RowsPlan& p, hipStream_t stream) {
    constexpr int lds_bytes = gemv_rows_lds_bytes<RG, MB, NW>();
    static_assert(lds_bytes <= 160 * 1024, "patches and partials of all waves must fit in LDS");
    auto kern = gemv_int8_rows_kernel<RG, MB, NW, 1, ROPE>;
    static std::atomic<uint64_t> lds_allowed{0};
    allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_allowed);
    note_kernel(ROPE ? "gemv_rows_rope" : "gemv_rows");
    kern<<<dim3((unsigned)p.blocks), dim3(NW * 64), lds_bytes, stream>>>(g, rc, p.rows_per_wg);
}

template <int RG, int NW, bool ROPE>
void launch_rows_mb(const GemmArgs& g, const RopeCacheArgs& rc, const RowsPlan& p, hipStream_t stream) {
    switch ((g.m + 15) / 16) {
        case 1: launch_rows_inst<RG, 1, NW, ROPE>(g, rc, p, stream); break;
        case 2: launch_rows_inst<RG, 2, NW, ROPE>(g, rc, p, stream); break;
        case 3: launch_rows_inst<RG, 3, NW, ROPE>(g, rc, p, stream); break;
        case 4: launch_rows_inst<RG, 4, NW, ROPE>(g, rc, p, stream); break;
        default:
            if constexpr (ROPE || NW == 8) launch_rows_inst<RG, 4, NW, ROPE>(g, rc, p, stream);  // at most 64 tokens there
            else if ((g.m + 15) / 16 <= 6) launch_rows_inst<RG, 6, NW, ROPE>(g, rc, p, stream);
            else launch_rows_inst<RG, 8, NW, ROPE>(g, rc, p, stream);
            break;
    }
}

// M <= 128 (ROPE: M <= 64)
template <bool ROPE>
void launch_rows(const GemmArgs& g, const RopeCacheArgs& rc, hipStream_t stream) {
    const RowsPlan p = plan_rows(g);
    if (p.rg == 3) launch_rows_mb<3, 4, ROPE>(g, rc, p, stream);
    else if (p.rg == 2) launch_rows_mb<2, 4, ROPE>(g, rc, p, stream);
    // (eight waves share a SIMD's registers two by two: enough for four token groups, not for eight)
    else if (p.nw == 8 && g.m <= 64) launch_rows_mb<1, 8, ROPE>(g, rc, p, stream);
    else launch_rows_mb<1, 4, ROPE>(g, rc, p, stream);
}

// fp8: the same plan and the same token-group instances; bf16 or fp32-accumulator output
template <int Fmt, int RG, int MB, int NW>
void launch_rows_fp8_inst(const GemmArgs& g, const RowsPlan& p, bool rowcol, hipStream_t stream) {
    constexpr int lds_bytes = gemv_rows_lds_bytes<RG, MB, NW>();
    auto kern = gemv_fp8_rows_kernel<Fmt, RG, MB, NW>;
    static std::atomic<uint64_t> lds_allowed{0};
    allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_allowed);
    note_kernel("gemv_rows_fp8");
    kern<<<dim3((unsigned)p.blocks), dim3(NW * 64), lds_bytes, stream>>>(g, p.rows_per_wg, rowcol ? 1 : 0);
}

template <int Fmt, int RG, int NW>
void launch_rows_fp8_mb(const GemmArgs& g, const RowsPlan& p, bool rowcol, hipStream_t stream) {
    switch ((g.m + 15) / 16) {
        case 1: launch_rows_fp8_inst<Fmt, RG, 1, NW>(g, p, rowcol, stream); break;
        case 2: launch_rows_fp8_inst<Fmt, RG, 2, NW>(g, p, rowcol, stream); break;
        case 3: launch_rows_fp8_inst<Fmt, RG, 3, NW>(g, p, rowcol, stream); break;
        case 4: launch_rows_fp8_inst<Fmt, RG, 4, NW>(g, p, rowcol, stream); break;
        default:
            if constexpr (NW == 8) launch_rows_fp8_inst<Fmt, RG, 4, NW>(g, p, rowcol, stream);  // at most 64 tokens there
            else if ((g.m + 15) / 16 <= 6) launch_rows_fp8_inst<Fmt, RG, 6, NW>(g, p, rowcol, stream);
            else launch_rows_fp8_inst<Fmt, RG, 8, NW>(g, p, rowcol, stream);
            break;
    }
}

template <int Fmt>
void launch_rows_fp8(const GemmArgs& g, bool rowcol, hipStream_t stream) {
    const RowsPlan p = plan_rows(g);
    if (p.rg == 3) launch_rows_fp8_mb<Fmt, 3, 4>(g, p, rowcol, stream);
    else if (p.rg == 2) launch_rows_fp8_mb<Fmt, 2, 4>(g, p, rowcol, stream);
    else if (p.nw == 8 && g.m <= 64) launch_rows_fp8_mb<Fmt, 1, 8>(g, p, rowcol, stream);
    else launch_rows_fp8_mb<Fmt, 1, 4>(g, p, rowcol, stream);
}

template <int RG, int MB, int NW>
void launch_rows_fp8_block_inst(const GemmArgs& g, const RowsPlan& p, hipStream_t stream) {
    constexpr int lds_bytes = gemv_rows_lds_bytes<RG, MB, NW>();
    auto kern = gemv_fp8_block128_rows_kernel<RG, MB, NW>;
    static std::atomic<uint64_t> lds_allowed{0};
    allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_allowed);
    note_kernel("gemv_rows_fp8_block128");
    kern<<<dim3((unsigned)p.blocks), dim3(NW * 64), lds_bytes, stream>>>(g, p.rows_per_wg);
}

template <int RG, int NW>
void launch_rows_fp8_block_mb(const GemmArgs& g, const RowsPlan& p, hipStream_t stream) {
    switch ((g.m + 15) / 16) {
        case 1: launch_rows_fp8_block_inst<RG, 1, NW>(g, p, stream); break;
        case 2: launch_rows_fp8_block_inst<RG, 2, NW>(g, p, stream); break;
        case 3: launch_rows_fp8_block_inst<RG, 3, NW>(g, p, stream); break;
        default: launch_rows_fp8_block_inst<RG, 4, NW>(g, p, stream); break;
    }
}

}  // namespace

bool launch_gemv_fp8_block128(const GemmArgs& g, hipStream_t stream) {
    if (g.m <= 0 || g.m > 64 || g.n <= 0 || g.k <= 0 || (g.k & 255) != 0) return false;
    if ((int64_t)g.n * g.k >= ((int64_t)1 << 31)) return false;
    if (g.out_kind != OUT_BF16 || g.resid || g.row_max) return false;
    const RowsPlan p = plan_rows(g);
    if (p.rg == 3) launch_rows_fp8_block_mb<3, 4>(g, p, stream);
    else if (p.rg == 2) launch_rows_fp8_block_mb<2, 4>(g, p, stream);
    else if (p.nw == 8) launch_rows_fp8_block_mb<1, 8>(g, p, stream);
    else launch_rows_fp8_block_mb<1, 4>(g, p, stream);
    return true;
}

bool launch_gemv_fp8(const GemmArgs& g, int fmt, int scale_kind, hipStream_t stream) {
    if (g.m <= 0 || g.m > 128 || g.n <= 0 || g.k <= 0 || (g.k & 255) != 0) return false;
    if ((int64_t)g.n * g.k >= ((int64_t)1 << 31)) return false;
    if (g.out_kind != OUT_BF16 && g.out_kind != OUT_ACC) return false;
    if (scale_kind != SCALE_TENSOR && scale_kind != SCALE_ROWCOL) return false;
    if (g.resid || g.row_max) return false;
    if (fmt) launch_rows_fp8<1>(g, scale_kind == SCALE_ROWCOL, stream);
    else launch_rows_fp8<0>(g, scale_kind == SCALE_ROWCOL, stream);
    return true;
}

bool launch_gemm_int8_rope_cache(const GemmArgs& g, const RopeCacheArgs& rc, hipStream_t stream) {
    if (g.m <= 0 || g.m > 64 || g.n <= 0 || g.k <= 0 || (g.k & 255) != 0 || (g.n & 3) != 0) return false;
    if (g.out_kind != OUT_BF16 || g.bias != nullptr || (rc.head_dim & 3) != 0) return false;
    if (g.m != rc.batch * rc.seq || g.n != (rc.n_heads + 2 * rc.n_kv_heads) * rc.head_dim) return false;
    if ((int64_t)g.n * g.k >= ((int64_t)1 << 31)) return false;
    launch_rows<true>(g, rc, stream);
    return true;
}

bool launch_gemv_int8(const GemmArgs& g, hipStream_t stream) {
    if (g.m <= 0 || g.m > 128 || g.n <= 0 || g.k <= 0 || (g.k & 255) != 0) return false;
    const int64_t lim = (int64_t)1 << 31;
    if ((int64_t)g.n * g.k >= lim) return false;
    // the row-range kernel's residual epilogue works on whole 8-byte pieces of bf16 rows
    if (g.resid && g.out_kind != OUT_BF16) return false;
    if (g.resid && g.m > 1 && (g.n & 3) != 0) return false;
    if (g.m == 1)
        launch_dot(g, stream);
    else
        launch_rows<false>(g, RopeCacheArgs{}, stream);
    return true;
}

}  // namespace w8a8
