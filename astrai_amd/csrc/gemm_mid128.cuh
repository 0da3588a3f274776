// 8-bit NT GEMM for shapes between the decode kernels and the large-tile kernels: a few
// hundred to a few thousand activation rows, where 256 x 256 tiles leave most of the chip
// idle (2048 x 3072: 96 tiles for 256 compute units) and what counts is having every
// compute unit busy, not the last percent of operand reuse.
//
// 128 x 128 output tiles, eight waves of 64 x 32 (two MFMA 32x32 sub-tiles, 32 accumulator
// registers), K in 128-byte slabs through two LDS stages of 32 KiB filled by direct-to-LDS
// loads: 64 KiB per workgroup and ~95 registers per wave, so two workgroups -- four waves per
// SIMD -- share a compute unit and cover each other's barriers and memory waits; no hand-pinned
// schedule here (four waves of 64 x 64 measured 2-4% slower on the decoder's shapes). LDS
// layout of a slab, fragment reads and accumulator layout are those of the large-tile
// kernels (gemm_pingpong.cuh): 128 activation rows then 128 weight rows of 128 bytes, chunk
// c of row r at position c ^ (r & 7) ^ ((r >> 3) & 1); weight rows are the first MFMA operand.
#pragma once
#include "gemm_pingpong.cuh"

namespace w8a8 {

struct Mid128Cfg {
    static constexpr int BM = 128, BN = 128, BK = 128;
    static constexpr int THREADS = 512;
    static constexpr int MI = 2, NI = 1;                 // 32-row sub-tiles per wave: 64 m x 32 n
    static constexpr int OPERAND_BYTES = 128 * BK;       // one operand's slab: 16 KiB
    static constexpr int STAGE_BYTES = 2 * OPERAND_BYTES;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;    // 64 KiB
};

template <class Op, int ScaleKind>
__global__ __launch_bounds__(Mid128Cfg::THREADS, 4) void gemm_mid128_kernel(GemmArgs g) {
    using Cfg = Mid128Cfg;
    using Acc = typename Op::Acc;
    constexpr int MI = Cfg::MI, NI = Cfg::NI;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wave_m = wave & 1, wave_n = wave >> 1;   // 2 x 4 waves
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
    const int mw = m0 + wave_m * 64, nw = n0 + wave_n * 32;
    float sx[MI];
    f32x4 sw4[NI][4], b4[NI][4];
    const uint16_t* bias = static_cast<const uint16_t*>(g.bias);
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
        sx[mi] = 1.0f;
        if constexpr (ScaleKind == SCALE_ROWCOL) {
            const int m = mw + mi * 32 + lrow;
            sx[mi] = (m < g.m) ? g.sa[m] : 0.0f;
        }
    }
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = nw + ni * 32 + q * 8 + lgrp * 4 + j;
                sw4[ni][q][j] = 1.0f;
                b4[ni][q][j] = 0.0f;
                if (n < g.n) {
                    if constexpr (ScaleKind == SCALE_ROWCOL) sw4[ni][q][j] = g.sb[n];
                    // (the block-scaled instance needs its registers in the loop and fetches the bias at the end)
                    if constexpr (ScaleKind != SCALE_BLOCK128)
                        if (bias) b4[ni][q][j] = bf16_to_f32(bias[n]);
                }
            }

    // ---- direct-to-LDS load plan: wave w fills rows 16w .. 16w+15 of both operands, 8 rows per
    // instruction. Lane l lands at row l>>3, position l&7 of its 1 KiB block and fetches logical
    // chunk (l&7) ^ f(row): c0 for even instructions, c0 ^ 1 for odd ones. Rows past M / N are
    // past the buffer's num_records and read as zero.
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(g.a, (uint32_t)g.m * (uint32_t)K);
    const __amdgpu_buffer_rsrc_t rw = make_rsrc(g.b, (uint32_t)g.n * (uint32_t)K);
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
    auto issue = [&](int stage, uint32_t k0) {
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
    const int x_rd = (wave_m * 64) * 128;
    const int w_rd = Cfg::OPERAND_BYTES + (wave_n * 32) * 128;

    Acc acc[NI][MI];
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[ni][mi][j] = 0;

    // ---- 128-block scales: a slab is exactly one K-block. The slab's product is formed in a
    // temporary and joins the accumulator scaled by the activation rows' and the weight block's
    // steps (the tile's 128 columns lie in one weight block); the steps of slab k + 1 are requested
    // while slab k is computed.
    [[maybe_unused]] float blk_sa[MI], blk_sa_next[MI];
    [[maybe_unused]] float blk_sb = 0.0f, blk_sb_next = 0.0f;
    [[maybe_unused]] const int kblocks = K >> 7;
    auto request_steps = [&](int kb) {
        if constexpr (ScaleKind == SCALE_BLOCK128) {
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
                const int m = mw + mi * 32 + lrow;
                blk_sa_next[mi] = (m < g.m && kb < kblocks) ? g.sa[(size_t)m * kblocks + kb] : 0.0f;
            }
            blk_sb_next = kb < kblocks ? g.sb[(size_t)(n0 >> 7) * kblocks + kb] : 0.0f;
        }
    };

    auto compute = [&](int stage) {
        const uint8_t* const base = lds + stage * Cfg::STAGE_BYTES;
        u32x4 xf[MI][4], wf[NI][4];
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                wf[ni][j] = *reinterpret_cast<const u32x4*>(base + w_rd + ni * 4096 + frag_off[j]);
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                xf[mi][j] = *reinterpret_cast<const u32x4*>(base + x_rd + mi * 4096 + frag_off[j]);
        if constexpr (ScaleKind == SCALE_BLOCK128) {
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) {
                    Acc part;
#pragma unroll
                    for (int j = 0; j < 16; ++j) part[j] = 0;
#pragma unroll
                    for (int q = 0; q < Op::STEPS; ++q) part = Op::mma_step(q, wf[ni], xf[mi], part);
                    const float sc = blk_sa[mi] * blk_sb;
#pragma unroll
                    for (int j = 0; j < 16; ++j) acc[ni][mi][j] += part[j] * sc;
                }
        } else {
#pragma unroll
            for (int q = 0; q < Op::STEPS; ++q)
#pragma unroll
                for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni) acc[ni][mi] = Op::mma_step(q, wf[ni], xf[mi], acc[ni][mi]);
        }
    };

    // ---- main loop: slab k+1 in flight while slab k is read; a barrier before a stage is
    // read (every wave's part has landed) and one before it is filled again
    request_steps(0);
    issue(0, 0u);
    for (int k = 0; k < ksteps; ++k) {
        if constexpr (ScaleKind == SCALE_BLOCK128) {
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) blk_sa[mi] = blk_sa_next[mi];
            blk_sb = blk_sb_next;
        }
        if (k + 1 < ksteps) {
            issue((k + 1) & 1, (uint32_t)(k + 1) << 7);
            wait_vmcnt<4>();   // the four loads of slab k are older than those just issued
        } else {
            wait_vmcnt<0>();
        }
        phase_barrier();
        // (after the wait: the next slab's steps are then older than the slab loads of the following
        // iteration, whose wait they pass without holding it up -- a compute phase has gone by)
        request_steps(k + 1);
        compute(k & 1);
        wait_lgkmcnt0();
        phase_barrier();
    }

    // ---- epilogue: a lane holds four consecutive n of one m per (sub-tile, quad): 8-byte stores
    if (g.out_kind != OUT_BF16) return;   // (the launcher sends other outputs elsewhere)
    uint16_t* const out = static_cast<uint16_t*>(g.out);
    const bool vec_ok = (g.n & 3) == 0;
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
        const int m = mw + mi * 32 + lrow;
        if (m >= g.m) continue;
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = nw + ni * 32 + q * 8 + lgrp * 4;
                if (n >= g.n) continue;
                float v[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float f = (float)acc[ni][mi][4 * q + j];
                    if constexpr (ScaleKind == SCALE_BLOCK128) {
                        v[j] = f + ((bias && n + j < g.n) ? bf16_to_f32(bias[n + j]) : 0.0f);
                    } else if constexpr (ScaleKind == SCALE_TENSOR) {
                        v[j] = f * s_tensor + b4[ni][q][j];
                    } else {
#pragma clang fp contract(off)
                        const float scaled = f * sx[mi] * sw4[ni][q][j];
                        v[j] = scaled + b4[ni][q][j];
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
}

// bf16 output, K in whole slabs, and a shape this tile size suits: at least 140 tiles of 128 x 128
// (below that the 64 x 64 tiles of the generic kernel spread the work further and win or draw: 512 x
// 3072 x 2048 13.2 against 15.1 us, 1024 x 2048 x 2048 13.3 against 14.9 us, 512 x 4096 x 4096 (128
// tiles) 22.5 against 22.3 us; from there on this kernel wins: 768 x 3072 x 2048 (144 tiles) 14.2
// against 16.4 us, 256 x 11008 x 4096 (172) 23.7 against 28.6 us, 1024 x 3072 x 2048 16.0 against
// 23.6 us, 2048 x 3072 x 2048 22.9 against 30.7 us)
inline bool mid128_shape_ok(const GemmArgs& g) {
    if (!tiled_shape_ok(g) || (g.k & 127) != 0 || g.k < 128 || g.out_kind != OUT_BF16) return false;
    const int64_t tiles = (int64_t)((g.m + 127) / 128) * ((g.n + 127) / 128);
    return tiles >= 140;
}

template <class Op, int ScaleKind>
inline void launch_mid128(const GemmArgs& g, hipStream_t stream) {
    using Cfg = Mid128Cfg;
    const int tiles = ((g.m + Cfg::BM - 1) / Cfg::BM) * ((g.n + Cfg::BN - 1) / Cfg::BN);
    auto kern = gemm_mid128_kernel<Op, ScaleKind>;
    static std::atomic<uint64_t> lds_allowed{0};
    allow_dynamic_lds(reinterpret_cast<const void*>(kern), Cfg::LDS_BYTES, lds_allowed);
    note_kernel(ScaleKind == SCALE_BLOCK128 ? "mid128_block128" : "mid128");
    kern<<<dim3((unsigned)tiles), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream>>>(g);
}

}  // namespace w8a8
