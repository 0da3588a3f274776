// Batched-decode W8A8 kernel (int8: 2 <= M <= 128 tokens; fp8: 1 <= M <= 128): bandwidth-bound. The weight
// matrix is streamed from HBM exactly once with the streaming cache hint; what decides the
// time besides that stream is how often the activation block X[M,K] is pulled out of
// L2 again (every workgroup that owns weight rows over all of K needs all of it), how
// many bytes are in flight from the first microsecond, and how evenly the rows fall
// on the compute units.
//
//  * The weight rows are dealt out in equal contiguous ranges, one workgroup per range
//    (about one per compute unit; ranges are multiples of four rows, not of the MFMA's
//    sixteen: rows past a range read as zero without memory traffic). X is therefore
//    read about 256 times per launch instead of N / 16 times.
//  * The NW waves of a workgroup split K into contiguous slices of 256-byte items; a
//    wave keeps all M tokens and all RG row groups of its slice, so it loads its part of
//    X once.
//  * Every load instruction moves 4 rows x 256 contiguous bytes (whole 128-byte lines,
//    in order) into registers; the 16 x 256-byte item is then turned into MFMA operand
//    order (lane = row, 16 bytes of K) through a 4 KiB wave-private LDS patch with an
//    XOR chunk swizzle that keeps both the row-major writes and the operand reads
//    conflict-free. Weights and activations take the same route, so any K order inside
//    an item is the same for both operands.
//  * int32 partials of the waves are summed through LDS (integer addition: the split
//    keeps the accumulator bit-exact), then the dequant epilogue, optionally continued
//    by rotary embedding and the KV-cache write for a fused q|k|v projection.
//  * fp8 operands take the same route with v_mfma_f32_16x16x128_f8f6f4 on pairs of operand
//    registers (any K order inside an item is a valid contraction); the waves' fp32 partials
//    are added in wave order, so a result does not change from launch to launch.
#pragma once

#include "common.cuh"
#include "launchers.h"

namespace w8a8 {

template <int AUX>
__device__ __forceinline__ u32x4 buf_load16_aux(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, AUX);
}
constexpr int kAuxStream = 2;  // "nt": the line is not kept once it has been delivered

// 16 rows x 256 bytes held as four load results (lane l of instruction i: row 4i + l/16,
// chunk l%16) -> four MFMA operand registers (lane l: row l%16, chunk 4j + l/16)
__device__ __forceinline__ void to_operand_order(uint8_t* patch, int lane, const u32x4 (&in)[4], u32x4 (&out)[4]) {
    const int lrow = lane & 15, lgrp = lane >> 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = i * 4 + lgrp;
        *reinterpret_cast<u32x4*>(patch + row * 256 + ((lrow ^ row) << 4)) = in[i];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
        out[j] = *reinterpret_cast<const u32x4*>(patch + lrow * 256 + (((4 * j + lgrp) ^ lrow) << 4));
}

struct RowsOpI8 {
    using Acc = i32x4;
    using AccScalar = int;
    static constexpr bool kIsInt = true;
};
template <int Fmt>  // 0 = e4m3fn, 1 = e5m2
struct RowsOpF8 {
    using Acc = f32x4;
    using AccScalar = float;
    static constexpr bool kIsInt = false;
    static constexpr int kFmt = Fmt;
};

// e4m3fn with one step per 1 x 128 K-group of the activations and per 128 x 128 block of the weights
// (sa [M, K/128], sb [ceil(N/128), K/128]): each 128-byte half of an item is one K-block, its
// MFMA result is scaled by the two steps before it joins the accumulator
struct RowsOpF8Block {
    using Acc = f32x4;
    using AccScalar = float;
    static constexpr bool kIsInt = false;
    static constexpr int kFmt = 0;
    static constexpr bool kBlock = true;
};
template <class Op, class = void> struct rows_op_block { static constexpr bool value = false; };
template <class Op> struct rows_op_block<Op, decltype((void)Op::kBlock)> { static constexpr bool value = Op::kBlock; };

// `rowcol`: one step per token and per weight row (always so for int8); else one per tensor
template <class Op, int RG, int MB, int NW, int IB, bool ROPE>
__device__ __forceinline__ void gemv_rows_body(const GemmArgs& g, const RopeCacheArgs& rc, int rows_per_wg,
                                               bool rowcol) {
    using Acc = typename Op::Acc;
    constexpr int PATCH = 8192;                     // per wave: 4 KiB weights + 4 KiB activations
    constexpr int RED = RG * MB * 1024;             // per wave: its partial accumulators
    constexpr int WAVE_LDS = PATCH > RED ? PATCH : RED;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lrow = lane & 15, lgrp = lane >> 4;
    const int K = g.k;
    const int ni = K >> 8;
    const int i0 = (wave * ni) / NW, i1 = ((wave + 1) * ni) / NW;
    const int r0 = blockIdx.x * rows_per_wg;
    const int r1 = min(r0 + rows_per_wg, g.n);

    const __amdgpu_buffer_rsrc_t rw = make_rsrc(g.b, (uint32_t)g.n * (uint32_t)K);
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(g.a, (uint32_t)g.m * (uint32_t)K);

    // epilogue operands of the (row group, token group) tasks this wave will write,
    // requested now so that their latency hides under the weight stream
    constexpr int TASKS = (RG * MB + NW - 1) / NW;
    float e_sx[TASKS], e_sw[TASKS][4], e_b[TASKS][4];
    u32x2 e_res[TASKS];   // four bf16 of the residual row (g.resid given: N % 4 == 0, bf16 output)
#pragma unroll
    for (int ti = 0; ti < TASKS; ++ti) {
        const int t = wave + ti * NW;
        const int m = (t % MB) * 16 + lrow;
        const int en = r0 + (t / MB) * 16 + lgrp * 4;
        const bool live = t < RG * MB && g.out_kind != OUT_ACC;
        if constexpr (rows_op_block<Op>::value) e_sx[ti] = (live && m < g.m) ? 1.0f : 0.0f;   // steps applied per K-block
        else e_sx[ti] = (live && m < g.m) ? (rowcol ? g.sa[m] : g.sa[0] * g.sb[0]) : 0.0f;
        e_res[ti] = (g.resid && live && m < g.m && en < r1)
            ? *reinterpret_cast<const u32x2*>(static_cast<const uint16_t*>(g.resid) + (size_t)m * g.n + en)
            : u32x2{0u, 0u};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool in = live && en + j < r1;
            if constexpr (rows_op_block<Op>::value) e_sw[ti][j] = in ? 1.0f : 0.0f;
            else e_sw[ti][j] = in ? (rowcol ? g.sb[en + j] : 1.0f) : 0.0f;
            e_b[ti][j] = (in && g.bias) ? bf16_to_f32(static_cast<const uint16_t*>(g.bias)[en + j]) : 0.0f;
        }
    }
    // ROPE: (cos, sin) of the lane's two pairs and the token's cache slot, per task
    [[maybe_unused]] f32x4 e_cs[TASKS];
    [[maybe_unused]] int64_t e_pos[TASKS];
    if constexpr (ROPE) {
#pragma unroll
        for (int ti = 0; ti < TASKS; ++ti) {
            const int t = wave + ti * NW;
            const int m = (t % MB) * 16 + lrow;
            const int en = r0 + (t / MB) * 16 + lgrp * 4;
            e_cs[ti] = f32x4{1.0f, 0.0f, 1.0f, 0.0f};
            e_pos[ti] = -1;
            if (t < RG * MB && m < g.m && en < r1) {
                const int sq = m % rc.seq;
                const int d = en % rc.head_dim;
                e_pos[ti] = rc.positions[sq];
                if (en < (rc.n_heads + rc.n_kv_heads) * rc.head_dim)
                    e_cs[ti] = *reinterpret_cast<const f32x4*>(
                        rc.freqs + ((int64_t)sq * (rc.head_dim >> 1) + (d >> 1)) * 2);
            }
        }
    }

    Acc acc[RG][MB];
#pragma unroll
    for (int r = 0; r < RG; ++r)
#pragma unroll
        for (int b = 0; b < MB; ++b) acc[r][b] = Acc{0, 0, 0, 0};

    uint8_t* const wpatch = smem + wave * WAVE_LDS;
    uint8_t* const xpatch = wpatch + 4096;
    // load plan of both operands: instruction i of an item covers rows 4i .. 4i+3, lane l
    // row 4i + l/16, 16-byte chunk l%16
    const uint32_t lane_off = (uint32_t)lgrp * (uint32_t)K + (uint32_t)lrow * 16;

    // A unit is four load instructions = 16 rows x 256 bytes of one operand; an item is MB
    // activation units (token groups) followed by RG weight units (row groups). The wave
    // keeps a ring of IB items in flight: as soon as a unit has been consumed, the same unit
    // of the item IB further on is requested into its registers, so the number of bytes
    // in flight per wave stays constant from the first instruction to the last (a burst of
    // every load followed by one wait measured slower by more than a microsecond, and so did
    // fewer, deeper bursts: the memory system is fed best by many waves with a steady, modest
    // window each).
    constexpr int P = MB + RG;
    u32x4 ring[IB][P][4];
    // block steps of an item's two K-blocks, per unit: activations' for token s * 16 + lrow, weights'
    // for the 128-row block of rows r0 + (s - MB) * 16 + 4 * lgrp .. + 3 (requested with the unit)
    [[maybe_unused]] f32x2 steps[IB][P];
    [[maybe_unused]] const int kblocks = K >> 7;
    auto issue_steps = [&](f32x2& dst, int item, int s) {
        if constexpr (rows_op_block<Op>::value) {
            dst = f32x2{0.0f, 0.0f};
            if (item < i1) {
                if (s < MB) {
                    const int m = s * 16 + lrow;
                    if (m < g.m) dst = *reinterpret_cast<const f32x2*>(g.sa + (size_t)m * kblocks + 2 * item);
                } else {
                    const int row = r0 + (s - MB) * 16 + 4 * lgrp;
                    if (row < r1) dst = *reinterpret_cast<const f32x2*>(g.sb + (size_t)(row >> 7) * kblocks + 2 * item);
                }
            }
        }
    };
    auto issue = [&](u32x4 (&dst)[4], int item, int s) {
        const bool live = item < i1;
        const uint32_t k0 = (uint32_t)item << 8;
        if (s < MB) {
#pragma unroll
            for (int i = 0; i < 4; ++i)   // tokens past M start past num_records: zeros
                dst[i] = buf_load16(rx, live ? lane_off + (uint32_t)(s * 16 + i * 4) * (uint32_t)K : kOutOfRange, k0);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = r0 + (s - MB) * 16 + i * 4;   // + lgrp, inside lane_off
                dst[i] = buf_load16_aux<kAuxStream>(
                    rw, (live && row + lgrp < r1) ? lane_off + (uint32_t)row * (uint32_t)K : kOutOfRange, k0);
            }
        }
    };
#pragma unroll
    for (int t = 0; t < IB; ++t)
#pragma unroll
        for (int s = 0; s < P; ++s) {
            issue(ring[t][s], i0 + t, s);
            issue_steps(steps[t][s], i0 + t, s);
        }

    for (int ib = i0; ib < i1; ib += IB) {
#pragma unroll
        for (int t = 0; t < IB; ++t) {
            u32x4 xf[MB][4];
            [[maybe_unused]] f32x2 xs[MB];
#pragma unroll
            for (int s = 0; s < P; ++s) {
                if (s < MB) {
                    to_operand_order(xpatch, lane, ring[t][s], xf[s < MB ? s : 0]);
                    if constexpr (rows_op_block<Op>::value) xs[s < MB ? s : 0] = steps[t][s];
                } else {
                    u32x4 wf[4];
                    to_operand_order(wpatch, lane, ring[t][s], wf);
                    if constexpr (Op::kIsInt) {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
#pragma unroll
                            for (int b = 0; b < MB; ++b)
                                acc[s < MB ? 0 : s - MB][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(
                                    (i32x4)wf[j], (i32x4)xf[b][j], acc[s < MB ? 0 : s - MB][b], 0, 0, 0);
                    } else if constexpr (rows_op_block<Op>::value) {
                        const f32x2 ws = steps[t][s];
#pragma unroll
                        for (int j = 0; j < 4; j += 2)
#pragma unroll
                            for (int b = 0; b < MB; ++b) {
                                const f32x4 part = OpF8<0>::mma(wf[j], wf[j + 1], xf[b][j], xf[b][j + 1],
                                                                f32x4{0.0f, 0.0f, 0.0f, 0.0f});
                                const float sc = xs[b][j >> 1] * ws[j >> 1];
#pragma unroll
                                for (int e = 0; e < 4; ++e) acc[s < MB ? 0 : s - MB][b][e] += part[e] * sc;
                            }
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; j += 2)
#pragma unroll
                            for (int b = 0; b < MB; ++b)
                                acc[s < MB ? 0 : s - MB][b] = OpF8<Op::kFmt>::mma(
                                    wf[j], wf[j + 1], xf[b][j], xf[b][j + 1], acc[s < MB ? 0 : s - MB][b]);
                    }
                }
                issue(ring[t][s], ib + t + IB, s);
                issue_steps(steps[t][s], ib + t + IB, s);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    // sum the waves' partials through LDS (the patches are free now)
    __syncthreads();
    Acc* const red = reinterpret_cast<Acc*>(smem);  // [NW] x WAVE_LDS bytes
#pragma unroll
    for (int r = 0; r < RG; ++r)
#pragma unroll
        for (int b = 0; b < MB; ++b) red[wave * (WAVE_LDS / 16) + (r * MB + b) * 64 + lane] = acc[r][b];
    __syncthreads();
#pragma unroll
    for (int ti = 0; ti < TASKS; ++ti) {
        const int t = wave + ti * NW;
        if (t >= RG * MB) break;
        Acc sum = red[t * 64 + lane];
#pragma unroll
        for (int w = 1; w < NW; ++w) sum += red[w * (WAVE_LDS / 16) + t * 64 + lane];
        const int r = t / MB, b = t % MB;
        const int m = b * 16 + lrow;
        const int en = r0 + r * 16 + lgrp * 4;
        if (m >= g.m || en >= r1) continue;
        const size_t o = (size_t)m * g.n + en;
        if (g.out_kind == OUT_ACC) {
            typename Op::AccScalar* out = static_cast<typename Op::AccScalar*>(g.out);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (en + j < r1) out[o + j] = sum[j];
            continue;
        }
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // product and bias add rounded separately (no fused multiply-add): the
            // int8 epilogue is specified as elementwise fp32 on the exact integer
            // (per-tensor fp8: e_sx is the product of the two steps, e_sw is 1)
#pragma clang fp contract(off)
            const float f = (float)sum[j] * e_sx[ti] * e_sw[ti][j];
            v[j] = f + e_b[ti][j];
        }
        if constexpr (ROPE) {
            // what the plain epilogue would have stored, as the rotary kernel would read it
            u32x2 pk;
            pk.x = pack_bf16x2(v[0], v[1]);
            pk.y = pack_bf16x2(v[2], v[3]);
            const int hh = en / rc.head_dim, d = en - hh * rc.head_dim;
            const int bt = m / rc.seq, sq = m - bt * rc.seq;
            if (hh < rc.n_heads + rc.n_kv_heads) {
                const float x[4] = {__uint_as_float(pk.x << 16), __uint_as_float(pk.x & 0xffff0000u),
                                    __uint_as_float(pk.y << 16), __uint_as_float(pk.y & 0xffff0000u)};
                float y[4];
#pragma unroll
                for (int p = 0; p < 2; ++p) {
#pragma clang fp contract(off)
                    const float c = e_cs[ti][2 * p], sn = e_cs[ti][2 * p + 1];
                    const float xe = x[2 * p], xo = x[2 * p + 1];
                    const float a0 = xe * c, a1 = xo * sn, b0 = xe * sn, b1 = xo * c;
                    y[2 * p] = a0 - a1;
                    y[2 * p + 1] = b0 + b1;
                }
                pk.x = pack_bf16x2(y[0], y[1]);
                pk.y = pack_bf16x2(y[2], y[3]);
            }
            if (hh < rc.n_heads) {
                uint16_t* dst = static_cast<uint16_t*>(rc.q_out) +
                                (((int64_t)bt * rc.n_heads + hh) * rc.seq + sq) * rc.head_dim + d;
                *reinterpret_cast<u32x2*>(dst) = pk;
            } else if (e_pos[ti] >= 0 && e_pos[ti] < rc.max_len) {  // a slot outside the cache: nothing
                const bool is_k = hh < rc.n_heads + rc.n_kv_heads;
                const int hk = hh - rc.n_heads - (is_k ? 0 : rc.n_kv_heads);
                uint16_t* dst = static_cast<uint16_t*>(is_k ? rc.k_cache : rc.v_cache) +
                                (((int64_t)bt * rc.n_kv_heads + hk) * rc.max_len + e_pos[ti]) * rc.head_dim + d;
                *reinterpret_cast<u32x2*>(dst) = pk;
            }
            continue;
        }
        uint16_t* out = static_cast<uint16_t*>(g.out);
        if ((g.n & 3) == 0) {
            u32x2 pk;
            pk.x = pack_bf16x2(v[0], v[1]);
            pk.y = pack_bf16x2(v[2], v[3]);
            if (g.resid) {   // bf16(y + residual) on the rounded y
                const u32x2 r = e_res[ti];
                pk.x = pack_bf16x2(__uint_as_float(pk.x << 16) + __uint_as_float(r.x << 16),
                                   __uint_as_float(pk.x & 0xffff0000u) + __uint_as_float(r.x & 0xffff0000u));
                pk.y = pack_bf16x2(__uint_as_float(pk.y << 16) + __uint_as_float(r.y << 16),
                                   __uint_as_float(pk.y & 0xffff0000u) + __uint_as_float(r.y & 0xffff0000u));
            }
            *reinterpret_cast<u32x2*>(out + o) = pk;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (en + j < r1) out[o + j] = f32_to_bf16(v[j]);
        }
    }
}

template <int RG, int MB, int NW, int IB, bool ROPE>
__global__ __launch_bounds__(NW * 64) void gemv_int8_rows_kernel(GemmArgs g, RopeCacheArgs rc, int rows_per_wg) {
    gemv_rows_body<RowsOpI8, RG, MB, NW, IB, ROPE>(g, rc, rows_per_wg, true);
}

template <int Fmt, int RG, int MB, int NW>
__global__ __launch_bounds__(NW * 64) void gemv_fp8_rows_kernel(GemmArgs g, int rows_per_wg, int rowcol) {
    gemv_rows_body<RowsOpF8<Fmt>, RG, MB, NW, 1, false>(g, RopeCacheArgs{}, rows_per_wg, rowcol != 0);
}

template <int RG, int MB, int NW>
__global__ __launch_bounds__(NW * 64) void gemv_fp8_block128_rows_kernel(GemmArgs g, int rows_per_wg) {
    gemv_rows_body<RowsOpF8Block, RG, MB, NW, 1, false>(g, RopeCacheArgs{}, rows_per_wg, false);
}

template <int RG, int MB, int NW>
constexpr int gemv_rows_lds_bytes() {
    return NW * (RG * MB * 1024 > 8192 ? RG * MB * 1024 : 8192);
}

}  // namespace w8a8
