// 8-bit NT GEMM for shapes with too few 128 x 128 tiles to occupy the chip: a few hundred
// activation rows against a narrow weight matrix (a short prompt, a large decode batch), or few
// rows with a K the decode kernels do not take.
//
// 64 x 64 output tiles, four waves of 32 x 32 (one MFMA 32x32 sub-tile, 16 accumulator registers),
// K in 128-byte slabs. With one or two workgroups on a compute unit little else hides a slab's
// memory latency, so the slabs come through a ring of S LDS stages of 16 KiB filled by
// direct-to-LDS loads S - 1 slabs ahead, and a wave reads the fragments of slab k + 1 into a second
// register set before it issues the MFMAs of slab k (the generic tiled kernel, which stages a slab
// through registers and waits for it, needs 1.2 k cycles a slab on these shapes; this one ~500,
// which is the L2 bandwidth 256 workgroups pulling 16 KiB a slab get). One workgroup barrier per slab: it publishes
// slab k + 1 (every wave has waited for its own loads) and retires slab k - 1's stage, which the
// load of slab k + S - 1 then overwrites. Past the end of K the loads run on an empty descriptor
// (no traffic), so the wait counts are the same in every iteration.
//
// LDS layout of a slab, load plan per wave (rows 16 w .. 16 w + 15 of both operands), fragment
// reads, accumulator layout and epilogue are those of gemm_mid128_kernel.
#pragma once
#include "gemm_pingpong.cuh"

namespace w8a8 {

template <int S>
struct Small64Cfg {
    static constexpr int BM = 64, BN = 64, BK = 128;
    static constexpr int THREADS = 256;
    static constexpr int STAGES = S;
    static constexpr int OPERAND_BYTES = 64 * BK;        // one operand's slab: 8 KiB
    static constexpr int STAGE_BYTES = 2 * OPERAND_BYTES;
    static constexpr int LDS_BYTES = S * STAGE_BYTES;
    static_assert(S >= 3 && 4 * (S - 2) < 64, "ring depth");
};

template <class Op, int ScaleKind, int S>
__global__ __launch_bounds__(256) void gemm_small64_kernel(GemmArgs g) {
    using Cfg = Small64Cfg<S>;
    using Acc = typename Op::Acc;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wave_m = wave & 1, wave_n = wave >> 1;   // 2 x 2 waves
    const int lrow = lane & 31, lgrp = lane >> 5;

    const int tiles_m = (g.m + Cfg::BM - 1) / Cfg::BM;
    const int tiles_n = (g.n + Cfg::BN - 1) / Cfg::BN;
    const TileCoord tc = map_tile(tiles_m, tiles_n);
    const int m0 = tc.tm * Cfg::BM, n0 = tc.tn * Cfg::BN;
    const int K = g.k;
    const int ksteps = K >> 7;

    // epilogue operands, requested now
    const EpilogueScalars es = load_epilogue_scalars<ScaleKind>(g);
    [[maybe_unused]] const float s_tensor = es.sa * es.sb;
    const int mw = m0 + wave_m * 32, nw = n0 + wave_n * 32;
    float sx = 1.0f;
    if constexpr (ScaleKind == SCALE_ROWCOL) {
        const int m = mw + lrow;
        sx = (m < g.m) ? g.sa[m] : 0.0f;
    }
    f32x4 sw4[4], b4[4];
    const uint16_t* bias = static_cast<const uint16_t*>(g.bias);
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = nw + q * 8 + lgrp * 4 + j;
            sw4[q][j] = 1.0f;
            b4[q][j] = 0.0f;
            if (n < g.n) {
                if constexpr (ScaleKind == SCALE_ROWCOL) sw4[q][j] = g.sb[n];
                // (the block-scaled instance fetches the bias at the end: its loop counts its own loads)
                if constexpr (ScaleKind != SCALE_BLOCK128)
                    if (bias) b4[q][j] = bf16_to_f32(bias[n]);
            }
        }

    // ---- direct-to-LDS load plan: wave w fills rows 16w .. 16w+15 of both operands, 8 rows per
    // instruction (two instructions an operand and slab). Rows past M / N are past the buffer's
    // num_records and read as zero.
    const uint32_t x_bytes = (uint32_t)g.m * (uint32_t)K, w_bytes = (uint32_t)g.n * (uint32_t)K;
    uint32_t x_off[2], w_off[2];
    {
        const int c0 = (lane & 7) ^ (lane >> 3);
        const uint32_t xr = (uint32_t)(m0 + wave * 16 + (lane >> 3)) * (uint32_t)K;
        const uint32_t wr = (uint32_t)(n0 + wave * 16 + (lane >> 3)) * (uint32_t)K;
        x_off[0] = xr + (uint32_t)c0 * 16;
        x_off[1] = xr + (uint32_t)(c0 ^ 1) * 16;
        w_off[0] = wr + (uint32_t)c0 * 16;
        w_off[1] = wr + (uint32_t)(c0 ^ 1) * 16;
    }
    const uint32_t row8 = 8u * (uint32_t)K;
    uint8_t* const dma_base = lds + wave * (16 * 128);
    auto issue = [&](int stage, int slab) __attribute__((always_inline)) {
        const bool live = slab < ksteps;
        const __amdgpu_buffer_rsrc_t rx = make_rsrc(g.a, live ? x_bytes : 0u);
        const __amdgpu_buffer_rsrc_t rw = make_rsrc(g.b, live ? w_bytes : 0u);
        const uint32_t k0 = (uint32_t)slab << 7;
        uint8_t* const dst = dma_base + stage * Cfg::STAGE_BYTES;
#pragma unroll
        for (int r = 0; r < 2; ++r) lds_dma16(rx, dst + r * 1024, x_off[r & 1] + (uint32_t)r * row8, k0);
#pragma unroll
        for (int r = 0; r < 2; ++r)
            lds_dma16(rw, dst + Cfg::OPERAND_BYTES + r * 1024, w_off[r & 1] + (uint32_t)r * row8, k0);
    };

    // ---- fragment read plan: lane (row lrow of a 32-row sub-tile, K-group lgrp) owns chunks 4 lgrp .. 4 lgrp + 3
    int frag_off[4];
    {
        const int sw = (lrow & 7) ^ ((lrow >> 3) & 1);
#pragma unroll
        for (int j = 0; j < 4; ++j) frag_off[j] = lrow * 128 + (((4 * lgrp + j) ^ sw) << 4);
    }
    const int x_rd = (wave_m * 32) * 128;
    const int w_rd = Cfg::OPERAND_BYTES + (wave_n * 32) * 128;
    auto read = [&](int stage, u32x4 (&xf)[4], u32x4 (&wf)[4]) __attribute__((always_inline)) {
        const uint8_t* const base = lds + stage * Cfg::STAGE_BYTES;
#pragma unroll
        for (int j = 0; j < 4; ++j) wf[j] = *reinterpret_cast<const u32x4*>(base + w_rd + frag_off[j]);
#pragma unroll
        for (int j = 0; j < 4; ++j) xf[j] = *reinterpret_cast<const u32x4*>(base + x_rd + frag_off[j]);
    };

    Acc acc;
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[j] = 0;
    u32x4 xa[4], wa[4], xb[4], wb[4];

    // ---- 128-block scales: a slab is exactly one K-block and the tile's 64 columns lie in one
    // weight block. The slab's product is formed in a temporary and joins the accumulator scaled by
    // the row's and the block's steps, requested one slab ahead -- two loads an iteration, issued
    // BEFORE the iteration's four slab loads, so that "all but the four youngest" below still means
    // slab k + 1 has landed, and the steps with it.
    [[maybe_unused]] float blk_sa_next = 0.0f, blk_sb_next = 0.0f;
    [[maybe_unused]] const int kblocks = ksteps;
    auto request_steps = [&](int kb) __attribute__((always_inline)) {
        if constexpr (ScaleKind == SCALE_BLOCK128) {
            static_assert(S == 4, "the wait counts of the block-scaled loop are written for four stages");
            const int mrow = mw + lrow;
            const int kc = min(kb, kblocks - 1);   // past the end: a harmless re-read
            blk_sa_next = (mrow < g.m) ? g.sa[(size_t)mrow * kblocks + kc] : 0.0f;
            blk_sb_next = g.sb[(size_t)(n0 >> 7) * kblocks + kc];
        }
    };

    // ---- prologue: slabs 0 .. S-2 in flight; slab 0 visible and in the first register set
    request_steps(0);
#pragma unroll
    for (int s = 0; s < S - 1; ++s) issue(s, s);
    wait_vmcnt<4 * (S - 2)>();
    phase_barrier();
    read(0, xa, wa);

    int rd_stage = 1;        // stage of slab k + 1
    int wr_stage = S - 1;    // stage of slab k + S - 1
    // one slab: MFMAs on (xc, wc) = slab k; slab k + 1 published and read into (xn, wn); slab k + S - 1 requested
    auto step = [&](int k, const u32x4 (&xc)[4], const u32x4 (&wc)[4], u32x4 (&xn)[4], u32x4 (&wn)[4]) __attribute__((always_inline)) {
        wait_vmcnt<4 * (S - 3)>();   // own loads of slab k + 1 (younger: slabs k + 2 .. k + S - 2)
        wait_lgkmcnt0();             // own reads of slab k
        phase_barrier();
        [[maybe_unused]] const float sc = blk_sa_next * blk_sb_next;   // slab k's steps
        request_steps(k + 1);
        issue(wr_stage, k + S - 1);
        read(rd_stage, xn, wn);
        if constexpr (ScaleKind == SCALE_BLOCK128) {
            Acc part;
#pragma unroll
            for (int j = 0; j < 16; ++j) part[j] = 0;
#pragma unroll
            for (int q = 0; q < Op::STEPS; ++q) part = Op::mma_step(q, wc, xc, part);
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[j] += part[j] * sc;
        } else {
#pragma unroll
            for (int q = 0; q < Op::STEPS; ++q) acc = Op::mma_step(q, wc, xc, acc);
        }
        rd_stage = (rd_stage == S - 1) ? 0 : rd_stage + 1;
        wr_stage = (wr_stage == S - 1) ? 0 : wr_stage + 1;
    };
    for (int k = 0; k < ksteps; k += 2) {
        step(k, xa, wa, xb, wb);
        if (k + 1 < ksteps) step(k + 1, xb, wb, xa, wa);
    }
    // no load outlives the kernel's use of LDS: the remaining ones ran on empty descriptors or are waited for here
    wait_vmcnt<0>();

    // ---- epilogue: a lane holds four consecutive n of one m per quad: 8-byte stores
    uint16_t* const out = static_cast<uint16_t*>(g.out);
    const bool vec_ok = (g.n & 3) == 0;
    const int m = mw + lrow;
    if (m >= g.m) return;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int n = nw + q * 8 + lgrp * 4;
        if (n >= g.n) continue;
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float f = (float)acc[4 * q + j];
            if constexpr (ScaleKind == SCALE_BLOCK128) {
                v[j] = f + ((bias && n + j < g.n) ? bf16_to_f32(bias[n + j]) : 0.0f);
            } else if constexpr (ScaleKind == SCALE_TENSOR) {
                v[j] = f * s_tensor + b4[q][j];
            } else {
#pragma clang fp contract(off)
                const float scaled = f * sx * sw4[q][j];
                v[j] = scaled + b4[q][j];
            }
        }
        const size_t o = (size_t)m * g.n + n;
        if (vec_ok) {
            u32x2 pk;
            pk.x = pack_bf16x2(v[0], v[1]);
            pk.y = pack_bf16x2(v[2], v[3]);
            *reinterpret_cast<u32x2*>(out + o) = pk;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (n + j < g.n) out[o + j] = f32_to_bf16(v[j]);
        }
    }
}

// bf16 output, K in whole slabs; the caller decides by tile counts
inline bool small64_shape_ok(const GemmArgs& g) {
    return tiled_shape_ok(g) && (g.k & 127) == 0 && g.k >= 128 && g.out_kind == OUT_BF16;
}

// Four stages (three slabs ahead, 64 KiB: two workgroups share a compute unit). A ring of eight
// stages measured the same or slower (256 x 2048 x 2048: 8.3 against 7.6 us; 384 x 2048 x 5632: 14.4
// against 15.0 us): 128 KiB of LDS leaves one workgroup per compute unit, and what bounds the
// kernel is the 16 KiB a 64 x 64 tile pulls out of L2 per slab, not latency.
constexpr int kSmall64Stages = 4;

template <class Op, int ScaleKind>
inline void launch_small64(const GemmArgs& g, hipStream_t stream) {
    using Cfg = Small64Cfg<kSmall64Stages>;
    const int64_t tiles = (int64_t)((g.m + 63) / 64) * ((g.n + 63) / 64);
    auto kern = gemm_small64_kernel<Op, ScaleKind, kSmall64Stages>;
    static std::atomic<uint64_t> lds_allowed{0};
    allow_dynamic_lds(reinterpret_cast<const void*>(kern), Cfg::LDS_BYTES, lds_allowed);
    note_kernel("small64");
    kern<<<dim3((unsigned)tiles), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream>>>(g);
}

}  // namespace w8a8
