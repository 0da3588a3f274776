// 256x256x128 "ping-pong" 8-bit NT GEMM for gfx950, the large-shape kernel.
//
// Why this shape. On gfx950 the full-rate 8-bit MFMAs are the 32x32 ones
// (v_mfma_f32_32x32x64_f8f6f4, v_mfma_i32_32x32x32_i8); LDS delivers roughly
// 160-175 B/clk/CU to ds_read_b128, and a 128-byte L1 line fetched half at a
// time is fetched twice. A 256x256 output tile with 128-byte K slabs keeps
// L2->L1 traffic at 32 B/clk/CU and, with 128(m) x 64(n) wave tiles, LDS traffic
// at ~125 B/clk/CU when the MFMA pipe is saturated.
//
// Structure. Eight waves, two per SIMD, form two groups (waves 0-3 / 4-7) that
// alternate between a MEMORY phase (read all MFMA operands of one K slab from
// LDS into registers) and a COMPUTE phase (issue that slab's MFMAs, nothing
// else), half a slab out of step with each other, separated by workgroup
// barriers: while one group's wave keeps a SIMD's MFMA pipe busy, the other
// wave on that SIMD refills its registers. K slabs land in a two-stage LDS ring
// by direct-to-LDS buffer loads (no staging registers; rows past M / N and
// bytes past K read as zero), each issued two phases before its first reader.
//
// LDS layout of a stage: 256 activation rows then 256 weight rows, 128 bytes
// each, as eight 16-byte chunks; chunk c of row r sits at position c ^ f(r),
// f(r) = (r & 7) ^ ((r >> 3) & 1), which makes both the 8-rows-per-instruction
// direct loads and the 32-rows-per-instruction operand reads conflict-free.
//
// MFMA operand roles: weight rows are the first operand, activation rows the
// second, so an accumulator lane holds, for one m, n = 8q + 4*(lane>>5) + 0..3
// (q = 0..3): four consecutive n per register quad.
#pragma once

#include <type_traits>

#include "common.cuh"
#include "gemm_tile.cuh"
#include "launchers.h"

namespace w8a8 {

typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// 32x32 operators: `frag` is the lane's 64 bytes of one row of one slab (four
// 16-byte chunks, K-group g = lane>>5 owns chunks 4g..4g+3).
struct Op32I8 {
    using Acc = i32x16;
    using AccScalar = int;
    using Op16 = OpI8;
    // a slab is four K=32 steps; step q uses chunk q of both fragments
    static constexpr int STEPS = 4;
    static __device__ __forceinline__ Acc mma_step(int q, const u32x4 (&w)[4], const u32x4 (&x)[4], Acc c) {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8((i32x4)w[q], (i32x4)x[q], c, 0, 0, 0);
    }
    // half a slab (two chunks per row) is two K=32 steps; step s uses chunk s
    static constexpr int HALF_STEPS = 2;
    static __device__ __forceinline__ Acc mma_half(int s, const u32x4 (&w)[2], const u32x4 (&x)[2], Acc c) {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8((i32x4)w[s], (i32x4)x[s], c, 0, 0, 0);
    }
};

template <int Fmt>
struct Op32F8 {
    using Acc = f32x16;
    using AccScalar = float;
    using Op16 = OpF8<Fmt>;
    // a slab is two K=64 steps; step h uses chunks 2h, 2h+1 of both fragments
    static constexpr int STEPS = 2;
    static __device__ __forceinline__ Acc mma_step(int h, const u32x4 (&w)[4], const u32x4 (&x)[4], Acc c) {
        const u32x4 w0 = w[2 * h], w1 = w[2 * h + 1], x0 = x[2 * h], x1 = x[2 * h + 1];
        i32x8 a = {(int)w0.x, (int)w0.y, (int)w0.z, (int)w0.w,
                   (int)w1.x, (int)w1.y, (int)w1.z, (int)w1.w};
        i32x8 b = {(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w,
                   (int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
        return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, Fmt, Fmt, 0, 0, 0, 0);
    }
    // half a slab (two chunks per row) is one K=64 step
    static constexpr int HALF_STEPS = 1;
    static __device__ __forceinline__ Acc mma_half(int, const u32x4 (&w)[2], const u32x4 (&x)[2], Acc c) {
        i32x8 a = {(int)w[0].x, (int)w[0].y, (int)w[0].z, (int)w[0].w,
                   (int)w[1].x, (int)w[1].y, (int)w[1].z, (int)w[1].w};
        i32x8 b = {(int)x[0].x, (int)x[0].y, (int)x[0].z, (int)x[0].w,
                   (int)x[1].x, (int)x[1].y, (int)x[1].z, (int)x[1].w};
        return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, Fmt, Fmt, 0, 0, 0, 0);
    }
};

// MI_ 32-row activation sub-tiles by NI_ 32-row weight sub-tiles per wave; the
// eight wave tiles cover the 256 x 256 output tile
template <int MI_, int NI_>
struct PingPongShape {
    static constexpr int BM = 256, BN = 256, BK = 128;
    static constexpr int THREADS = 512;
    static constexpr int MI = MI_, NI = NI_;
    static constexpr int WAVE_M = 32 * MI, WAVE_N = 32 * NI;  // rows of m, n per wave
    static constexpr int WAVES_M = BM / WAVE_M;               // waves along m
    static_assert(MI * NI == 8 && WAVES_M * (BN / WAVE_N) == 8, "eight waves, eight sub-tiles each");
    static constexpr int OPERAND_STAGE_BYTES = 256 * BK;   // one operand's slab: 32 KiB
    static constexpr int X_STAGES = 3, W_STAGES = 2;
    static constexpr int W_BASE = X_STAGES * OPERAND_STAGE_BYTES;  // weights after activations
    static constexpr int STAGES_BYTES = (X_STAGES + W_STAGES) * OPERAND_STAGE_BYTES;  // 160 KiB
    static constexpr int EPI_ROW_BYTES = 2 * WAVE_N + 16;  // a row of bf16 + 16 bytes of padding
    static constexpr int EPI_WAVE_BYTES = WAVE_M * EPI_ROW_BYTES;
    // all 160 KiB of the CU's LDS; the epilogue re-uses the space
    static constexpr int LDS_BYTES = STAGES_BYTES;
    static_assert(8 * EPI_WAVE_BYTES <= LDS_BYTES, "epilogue staging must fit");
};
using PingPongCfg = PingPongShape<4, 2>;     // 128 (m) x 64 (n) wave tiles
// Block scales: a lane keeps one scale, one ratio and one load in flight per
// activation sub-tile, so the wave tile is 64 (m) x 128 (n): two sub-tiles of m
// instead of four, and the 128 columns are exactly one weight block.
using PingPongCfgBlock = PingPongShape<2, 4>;

// s_waitcnt vmcnt(N) alone: all but the N most recently issued vector-memory
// loads of this wave have landed (gfx9 encoding: vmcnt in bits 3:0 and 15:14,
// expcnt / lgkmcnt fields left at "no wait"). Loads return in issue order.
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}
// s_waitcnt lgkmcnt(0) alone: every LDS read of this wave has returned
__device__ __forceinline__ void wait_lgkmcnt0() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0xc07f);
}
// raw buffer descriptor words for inline assembly (same contents as make_rsrc)
__device__ __forceinline__ i32x4 raw_rsrc(const void* p, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(p);
    i32x4 r = {(int)(uint32_t)a, (int)((uint32_t)(a >> 32) & 0xffffu), (int)bytes, 0x00020000};
    return r;
}

// workgroup barrier that the instruction scheduler may not move MFMAs or LDS reads across
__device__ __forceinline__ void phase_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ void lds_dma16(__amdgpu_buffer_rsrc_t r, uint8_t* lds_wave_base,
                                          uint32_t voff, uint32_t soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        r, (__attribute__((address_space(3))) void*)lds_wave_base, 16, voff, soff, 0, 0);
}

// Phase-timestamp hooks for the kernel's own profiling harness; compiled out
// of the library.
#ifdef W8A8_PP_TIMING
#ifndef PP_BLOCK
#define PP_BLOCK 0  // the workgroup whose waves record their stamps
#endif
__device__ unsigned long long* g_pp_dbg;
#define PP_STAMP_INIT()                                                                   \
    const bool pp_rec = (blockIdx.x == PP_BLOCK) && ((threadIdx.x & 63) == 0);                   \
    unsigned long long* pp_my = g_pp_dbg + (threadIdx.x >> 6) * 256;                      \
    int pp_ti = 0;
#define PP_STAMP()                                              \
    do {                                                        \
        __builtin_amdgcn_sched_barrier(0);                      \
        if (pp_rec && pp_ti < 250) pp_my[pp_ti] = clock64();    \
        pp_ti++;                                                \
        __builtin_amdgcn_sched_barrier(0);                      \
    } while (0)
#else
#define PP_STAMP_INIT()
#define PP_STAMP()
#endif

template <class Op, int ScaleKind, class Cfg = PingPongCfg>
__global__ __launch_bounds__(Cfg::THREADS) void gemm_pingpong_kernel(GemmArgs g) {
    PP_STAMP_INIT();
    using Acc = typename Op::Acc;
    constexpr int MI = Cfg::MI, NI = Cfg::NI;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int group = wave >> 2;       // 0: memory phase on even steps, 1: on odd steps
    const int wave_m = wave % Cfg::WAVES_M;  // which WAVE_M rows of m
    const int wave_n = wave / Cfg::WAVES_M;  // which WAVE_N rows of n
    const int lrow = lane & 31;
    const int lgrp = lane >> 5;

    const int tiles_m = (g.m + Cfg::BM - 1) / Cfg::BM;
    const int tiles_n = (g.n + Cfg::BN - 1) / Cfg::BN;
    const TileCoord tc = map_tile(tiles_m, tiles_n);
    const int m0 = tc.tm * Cfg::BM, n0 = tc.tn * Cfg::BN;
    const int K = g.k;
    const int ksteps = K >> 7;

    // ---- direct-to-LDS load plan. Group 0 loads the weight rows, group 1 the
    // activation rows, each in its own memory phase: wave w fills rows
    // 64(w&3)..+63 of its operand's 256, 8 rows per instruction, 8 instructions
    // per slab. Lane l lands at row (l>>3), position (l&7) of its 1 KiB block, so
    // it fetches logical chunk (l&7) ^ f(row); with row = 8i + (l>>3) (mod 16)
    // that is c0 = (l&7)^(l>>3) for even i and c0 ^ 1 for odd i. Rows past M / N
    // need no predicate: their byte offset is past the buffer's num_records and
    // the load returns zeros.
    const bool loads_w = group == 0;
    const void* const ld_ptr = loads_w ? g.b : g.a;
    const uint32_t ld_bytes = (uint32_t)(loads_w ? g.n : g.m) * (uint32_t)K;
    const __amdgpu_buffer_rsrc_t rld = make_rsrc(ld_ptr, ld_bytes);
    const int ld_row0 = (loads_w ? n0 : m0) + (wave & 3) * 64;
    uint32_t ld_off_even, ld_off_odd;
    {
        const int c0 = (lane & 7) ^ (lane >> 3);
        const uint32_t rowoff = (uint32_t)(ld_row0 + (lane >> 3)) * (uint32_t)K;
        ld_off_even = rowoff + (uint32_t)c0 * 16;
        ld_off_odd = rowoff + (uint32_t)(c0 ^ 1) * 16;
    }
    const uint32_t row8 = 8u * (uint32_t)K;  // byte distance of 8 rows
    // LDS map: three activation stages (32 KiB each), then two weight stages
    uint8_t* const ld_base = lds + (loads_w ? Cfg::W_BASE : 0) + (wave & 3) * (64 * 128);

    auto issue_loads = [&](int kstep, int stage) {
        const uint32_t k0 = (uint32_t)kstep << 7;
        uint8_t* dst = ld_base + stage * Cfg::OPERAND_STAGE_BYTES;
        // the two lane offsets pass through an opaque statement so that the eight
        // per-instruction offsets are re-added here (one v_add each) instead of
        // living in eight registers across the whole loop as hoisted invariants
        uint32_t off_e = ld_off_even, off_o = ld_off_odd;
        if constexpr (ScaleKind == SCALE_BLOCK128) {
            // one register fewer: rows start at multiples of 128 bytes, so the odd
            // instructions' chunk c0 ^ 1 is the even offset with bit 4 flipped
            asm volatile("" : "+v"(off_e));
            off_o = off_e ^ 16u;
        } else {
            asm volatile("" : "+v"(off_e), "+v"(off_o));
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
            lds_dma16(rld, dst + i * 1024, ((i & 1) ? off_o : off_e) + (uint32_t)i * row8, k0);
    };

    // ---- L2 prefetch plan. The 32 workgroups of an XCD walk K in step, so a
    // slab's first request always goes out to the fabric; one dword per 128-byte
    // line, touched kPrefetch slabs ahead and never read, turns the later
    // direct-to-LDS loads into L2 hits. Lane l of wave w owns row l of the wave's
    // 64. The touch is a raw instruction with a pinned destination register so
    // that nothing ever waits on it; the compiler not knowing about it can only
    // make its own waits longer, never shorter.
    constexpr int kPrefetch = 3;
    const uint32_t pf_off = (uint32_t)(ld_row0 + lane) * (uint32_t)K;
    const i32x4 rld_raw = raw_rsrc(ld_ptr, ld_bytes);
    uint32_t pf_reg = 0;
    // (not with block scales: measured slower there with the touches than without)
    constexpr bool kBlk = ScaleKind == SCALE_BLOCK128;
    constexpr int kTouch = kBlk ? 0 : 1;  // touches per phase
    auto prefetch = [&](int kstep) {
        if constexpr (kTouch == 0) return;
        const uint32_t k0 = (uint32_t)kstep << 7;
        asm volatile("buffer_load_dword %0, %1, %2, %3 offen"
                     : "+v"(pf_reg) : "v"(pf_off), "s"(rld_raw), "s"(k0) : "memory");
    };

    // ---- operand read plan: chunk positions of this lane (row swizzle depends
    // on the low four row bits only, sub-tile bases are multiples of 32)
    int frag_off[4];
    {
        const int sw = (lrow & 7) ^ ((lrow >> 3) & 1);
#pragma unroll
        for (int j = 0; j < 4; ++j) frag_off[j] = lrow * 128 + (((4 * lgrp + j) ^ sw) << 4);
    }
    const int x_base = (wave_m * Cfg::WAVE_M) * 128;                // activation rows of this wave
    const int w_base = Cfg::W_BASE + (wave_n * Cfg::WAVE_N) * 128;  // weight rows of this wave

    Acc acc[NI][MI];
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[ni][mi][j] = 0;

    u32x4 xf[MI][4], wf[NI][4];

    auto read_frags = [&](int xstage, int wstage) {
        const uint8_t* xb = lds + x_base + xstage * Cfg::OPERAND_STAGE_BYTES;
        const uint8_t* wb = lds + w_base + wstage * Cfg::OPERAND_STAGE_BYTES;
        if constexpr (ScaleKind == SCALE_BLOCK128) {
            // registers are scarce in this variant: chunk j's position is chunk 0's
            // with j xor-ed into its two low chunk bits, re-derived at every use
            int f0 = frag_off[0];
            asm volatile("" : "+v"(f0));
#pragma unroll
            for (int j = 1; j < 4; ++j) frag_off[j] = f0 ^ (j << 4);
        }
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                wf[ni][j] = *reinterpret_cast<const u32x4*>(wb + ni * 4096 + frag_off[j]);
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                xf[mi][j] = *reinterpret_cast<const u32x4*>(xb + mi * 4096 + frag_off[j]);
    };
    // K step outermost: the eight accumulators are touched round-robin, so an
    // MFMA never waits on the result of the one issued just before it
    auto compute = [&]() {
#pragma unroll
        for (int st = 0; st < Op::STEPS; ++st)
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int ni = 0; ni < NI; ++ni)
                    acc[ni][mi] = Op::mma_step(st, wf[ni], xf[mi], acc[ni][mi]);
    };

    // ---- 128-block scales (SCALE_BLOCK128 only; wave tile of two activation
    // sub-tiles by one 128-column weight block). The promotion
    //   out += P_kb * sa[m,kb] * sb[n/128,kb]
    // is run in place on the accumulator: it is kept divided by the current
    // block's scale s_kb = sa*sb, i.e. before slab kb's MFMAs the accumulator is
    // multiplied by s_{kb-1}/s_kb and after the last slab by s_last. That needs no
    // second register tile for P_kb. Scales below 1e-20 are taken as 1e-20.
    // A lane owns one m per 32-row sub-tile and the wave one weight block.
    //
    // The multiplies run inside the MFMA stream: eight independent ones fit in the
    // shadow of one 32x32x64 MFMA. While the eight MFMAs of sub-tile 0 issue,
    // sub-tile 1 (not yet touched in this slab) is brought to this slab's scale;
    // while those of sub-tile 1 issue, sub-tile 0 (finished for this slab) is
    // brought to the next slab's. The scales are therefore requested two slabs
    // ahead, after the phase's slab loads (a wait in front of a slab load would
    // delay it), and turned into factors at the start of the next operand-read
    // phase, when every load older than them has landed long ago: a scale load
    // issued in the phase that needs it leaves ~1000 cycles of latency exposed.
    static_assert(!kBlk || (MI == 2 && NI == 4 && Op::STEPS == 2),
                  "block scales need the 64 (m) x 128 (n) wave tile and two K steps per slab");
    [[maybe_unused]] float blk_s[2] = {1.0f, 1.0f};  // latest scale consumed, per sub-tile
    [[maybe_unused]] float blk_r0 = 1.0f;       // sub-tile 0: this slab's scale -> the next slab's
    [[maybe_unused]] float blk_r1 = 1.0f;       // sub-tile 1: the previous slab's scale -> this slab's
    [[maybe_unused]] float blk_r1_next = 1.0f;  // the same for the next slab
    [[maybe_unused]] const int kblocks = ksteps;
    // lane l asks for the activation scale of row l of the wave's 64 (rows past M
    // read as zero and are clamped like any tiny scale); the halves of the wave
    // exchange them at use
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t rsa =
        make_rsrc(g.sa, kBlk ? (uint32_t)g.m * (uint32_t)kblocks * 4u : 0u);
    [[maybe_unused]] const uint32_t sa_off =
        (uint32_t)(m0 + wave_m * Cfg::WAVE_M + lane) * (uint32_t)kblocks * 4u;
    // (a wave whose columns all lie past N clamps to the last block: its outputs are dropped)
    [[maybe_unused]] const float* const sb_row =
        kBlk ? g.sb + (size_t)min((n0 + wave_n * Cfg::WAVE_N) >> 7, ((g.n + 127) >> 7) - 1) * kblocks : nullptr;
    [[maybe_unused]] float blk_sa_ld = 1.0f, blk_sb_ld = 1.0f;  // scales in flight
    [[maybe_unused]] auto load_block_scales = [&](int kb) {
        if constexpr (kBlk) {
            kb = min(kb, kblocks - 1);  // past the end: a harmless re-read
            blk_sb_ld = sb_row[kb];
            blk_sa_ld = __builtin_bit_cast(
                float, __builtin_amdgcn_raw_buffer_load_b32(rsa, sa_off, (uint32_t)kb * 4u, 0));
        }
    };
    // the scales in flight, per sub-tile
    [[maybe_unused]] auto landed_scales = [&](float (&next)[2]) {
        // v_permlane32_swap of a register with itself: first result = the low
        // half's values in both halves (rows 0..31), second = the high half's
        const auto both = __builtin_amdgcn_permlane32_swap(
            __float_as_uint(blk_sa_ld), __float_as_uint(blk_sa_ld), false, false);
        next[0] = fmaxf(__uint_as_float(both[0]) * blk_sb_ld, 1e-20f);
        next[1] = fmaxf(__uint_as_float(both[1]) * blk_sb_ld, 1e-20f);
    };
    // at the start of slab k's operand-read phase: slab k+1's scales become factors
    [[maybe_unused]] auto next_factors = [&](int k) {
        if constexpr (kBlk) {
            float next[2];
            landed_scales(next);
            const bool last = k + 1 >= ksteps;  // no slab follows: stay at this scale
            blk_r1 = blk_r1_next;
            // hardware reciprocal (1 ulp) against a 1e-2 output tolerance
            blk_r0 = last ? 1.0f : blk_s[0] * __builtin_amdgcn_rcpf(next[0]);
            blk_r1_next = last ? 1.0f : blk_s[1] * __builtin_amdgcn_rcpf(next[1]);
            blk_s[0] = last ? blk_s[0] : next[0];
            blk_s[1] = last ? blk_s[1] : next[1];
        }
    };
    // one slab's MFMAs with the rescaling multiplies between them
    [[maybe_unused]] auto compute_block = [&]() {
        if constexpr (kBlk) {
#pragma unroll
            for (int mi = 0; mi < 2; ++mi) {
                const float r = mi ? blk_r0 : blk_r1;
#pragma unroll
                for (int st = 0; st < 2; ++st)
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni) {
                        acc[ni][mi] = Op::mma_step(st, wf[ni], xf[mi], acc[ni][mi]);
#pragma unroll
                        for (int j = 0; j < 8; ++j) {
                            const int f = (st * NI + ni) * 8 + j;
                            float t = acc[f >> 4][mi ^ 1][f & 15] * r;
                            asm volatile("" : "+v"(t));  // here, not sunk towards its use
                            acc[f >> 4][mi ^ 1][f & 15] = t;
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
            }
        }
    };

    // ---- prologue: slabs 0 and 1 of both operands in flight, then visible
    PP_STAMP();
    issue_loads(0, 0);
    if (ksteps > 1) issue_loads(1, 1);
    load_block_scales(0);
    __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0) lgkmcnt(0) expcnt(0)
    if constexpr (kBlk) {
        landed_scales(blk_s);  // the accumulators start out at slab 0's scale
        load_block_scales(1);
    }
    __syncthreads();
    PP_STAMP();

    // Main loop, one workgroup barrier per K slab. Barrier B_k guarantees that
    // slab k is complete in LDS and visible, and that nobody reads slab k-1 any
    // more. Between B_k and B_{k+1}:
    //   group 0: read slab k's operands (memory phase), then issue its MFMAs;
    //   group 1: issue slab k-1's MFMAs, then read slab k's operands.
    // The groups therefore start every slab in opposite phases and, the two
    // phases being about equally long, stay that way without a second barrier.
    // Loads: group 0 issues the weight rows of slab k+1 (2 stages, stage of slab
    // k-1) right after its operand reads; group 1 issues the activation rows of
    // slab k+2 (3 stages) likewise. A wave waits for its own loads just before
    // the barrier that must publish them: weights of slab k+1 at B_{k+1},
    // activations of slab k+2 at B_{k+2} -- every load has a full slab time
    // (weights) or two (activations) to land.
    if (group == 0) {
        int xs = 0;  // k % 3
        for (int k = 0; k < ksteps; ++k) {
            read_frags(xs, k & 1);
            next_factors(k);
            if (k >= 1 && k + 1 < ksteps) issue_loads(k + 1, (k + 1) & 1);
            load_block_scales(k + 2);
            // always one touch, so that "all but the last one" below means the slab
            // loads; past the end it re-touches the last slab (an L2 hit)
            prefetch(min(k + kPrefetch, ksteps - 1));
            wait_lgkmcnt0();
            // lower MFMA priority than group 1: if group 1's wave on this SIMD still
            // has MFMAs of the previous slab to issue it goes first (the hardware
            // otherwise favours this, older, wave and starves the other one)
            __builtin_amdgcn_s_setprio(1);
            if constexpr (kBlk) compute_block();
            else compute();
            __builtin_amdgcn_s_setprio(0);
            // the slab loads; the prefetch touch (if any) may stay in flight
            wait_vmcnt<kTouch>();
            phase_barrier();  // B_{k+1}
            xs = (xs == 2) ? 0 : xs + 1;
        }
        phase_barrier();  // matches group 1's final barrier
    } else {
        // memory phase of slab k and the barrier that ends it
        auto memory_phase = [&](int k, int xs) {
            read_frags(xs, k & 1);
            next_factors(k);
            const int xs2 = (xs == 0) ? 2 : xs - 1;  // (k + 2) % 3
            const bool more = k + 2 < ksteps;
            if (more) issue_loads(k + 2, xs2);
            load_block_scales(k + 2);
            prefetch(min(k + 2 + kPrefetch, ksteps - 1));
            wait_lgkmcnt0();
            // slab k+1 (issued one slab ago) must have landed; this slab's eight
            // loads and the two latest touches may stay in flight
            // (block scales: and this phase's two scale loads)
            if (more) wait_vmcnt<8 + 2 * kTouch + (kBlk ? 2 : 0)>();
            else wait_vmcnt<kTouch>();
            phase_barrier();  // B_{k+1}
        };
        int xs = 0;  // k % 3
        if constexpr (kBlk) {
            // slab 0 has no predecessor to compute: kept out of the loop, whose MFMAs
            // are then unconditional (under "if (k > 0)" the compiler moved the second
            // half's multiplies out of the MFMA stream, behind the join)
            memory_phase(0, 0);
            xs = 1;
        }
        for (int k = kBlk ? 1 : 0; k < ksteps; ++k) {
            __builtin_amdgcn_s_setprio(2);
            if constexpr (kBlk) {
                compute_block();  // slab k-1
            } else {
                if (k > 0) compute();  // slab k-1
            }
            __builtin_amdgcn_s_setprio(0);
            memory_phase(k, xs);
            xs = (xs == 2) ? 0 : xs + 1;
        }
        if constexpr (kBlk) compute_block();  // last slab
        else compute();
        phase_barrier();
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): no prefetch touch outlives the loop
    asm volatile("" :: "v"(pf_reg));

    // ---------------- epilogue ----------------
    PP_STAMP();
    const EpilogueScalars es = load_epilogue_scalars<ScaleKind>(g);
    using Op16 = typename Op::Op16;
    if (g.out_kind == OUT_BF16 && (g.n & 7) == 0) {
        // bf16 through LDS: each wave lays its 128(m) x 64(n) tile down row-major
        // (144-byte rows), then streams it out as full 128-byte lines, 16 bytes a
        // lane. The K-slab stages are dead by now; the region is wave-private, so
        // no workgroup barrier is needed (group 1 is still computing while group
        // 0 is here, on registers only).
        uint8_t* const mine = lds + wave * Cfg::EPI_WAVE_BYTES;
        const uint16_t* bias = static_cast<const uint16_t*>(g.bias);
        const int nw = n0 + wave_n * Cfg::WAVE_N;
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int nl = ni * 32 + q * 8 + lgrp * 4;  // first of this lane's four n
                const int n = nw + nl;
                f32x4 sw4 = {1.0f, 1.0f, 1.0f, 1.0f};
                f32x4 b4 = {0.0f, 0.0f, 0.0f, 0.0f};
                if (n < g.n) {  // N % 8 == 0: the four are in range together
                    if constexpr (ScaleKind == SCALE_ROWCOL)
                        sw4 = *reinterpret_cast<const f32x4*>(g.sb + n);
                    if (bias) {
                        const u32x2 raw = *reinterpret_cast<const u32x2*>(bias + n);
                        b4 = f32x4{__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u),
                                   __uint_as_float(raw.y << 16), __uint_as_float(raw.y & 0xffff0000u)};
                    }
                }
#pragma unroll
                for (int mi = 0; mi < MI; ++mi) {
                    const int ml = mi * 32 + lrow;
                    const int m = m0 + wave_m * Cfg::WAVE_M + ml;
                    float sx = 1.0f;
                    if constexpr (ScaleKind == SCALE_ROWCOL) sx = (m < g.m) ? g.sa[m] : 0.0f;
                    float v[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        float f = (float)acc[ni][mi][4 * q + j];
                        if constexpr (ScaleKind == SCALE_TENSOR) f = f * (es.sa * es.sb);
                        else if constexpr (ScaleKind == SCALE_ROWCOL) f = f * sx * sw4[j];
                        else f = f * blk_s[mi];
                        v[j] = f + b4[j];
                    }
                    u32x2 pk;
                    pk.x = pack_bf16x2(v[0], v[1]);
                    pk.y = pack_bf16x2(v[2], v[3]);
                    *reinterpret_cast<u32x2*>(mine + ml * Cfg::EPI_ROW_BYTES + nl * 2) = pk;
                }
            }
        }
        // same wave reads back: LDS operations of one wave complete in order
        uint16_t* out = static_cast<uint16_t*>(g.out);
        constexpr int kRowLanes = Cfg::WAVE_N / 8;   // lanes per row, 16 bytes each
        constexpr int kRowsPer = 64 / kRowLanes;     // rows per store instruction
        const int rr = lane / kRowLanes, cc = lane % kRowLanes;
#pragma unroll
        for (int i = 0; i < Cfg::WAVE_M / kRowsPer; ++i) {
            const int ml = i * kRowsPer + rr;
            const u32x4 v = *reinterpret_cast<const u32x4*>(mine + ml * Cfg::EPI_ROW_BYTES + cc * 16);
            const int m = m0 + wave_m * Cfg::WAVE_M + ml;
            const int n = nw + cc * 8;
            // non-temporal: the output streams to memory during the epilogue instead of
            // sitting dirty in L2 until the end-of-kernel write-back
            if (m < g.m && n < g.n)
                __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(out + (size_t)m * g.n + n));
        }
    } else {
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            const int m = m0 + wave_m * Cfg::WAVE_M + mi * 32 + lrow;
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int n = n0 + wave_n * Cfg::WAVE_N + ni * 32 + q * 8 + lgrp * 4;
                    typename Op16::Acc v = {acc[ni][mi][4 * q], acc[ni][mi][4 * q + 1],
                                            acc[ni][mi][4 * q + 2], acc[ni][mi][4 * q + 3]};
                    store_subtile<Op16, ScaleKind>(g, es, v, m, n);
                }
            }
        }
    }
    PP_STAMP();
}

inline bool pingpong_shape_ok(const GemmArgs& g) {
    if (!tiled_shape_ok(g) || (g.k & 127) != 0) return false;
    // worth it only when 256x256 tiles fill most of the chip
    const int64_t tiles = (int64_t)((g.m + 255) / 256) * ((g.n + 255) / 256);
    return tiles >= 192 && g.k >= 256;
}

template <class Op, int ScaleKind, class Cfg = PingPongCfg>
inline void launch_pingpong(const GemmArgs& g, hipStream_t stream) {
    const int tiles = ((g.m + Cfg::BM - 1) / Cfg::BM) * ((g.n + Cfg::BN - 1) / Cfg::BN);
    auto kern = gemm_pingpong_kernel<Op, ScaleKind, Cfg>;
    static std::atomic<uint64_t> lds_allowed{0};
    allow_dynamic_lds(reinterpret_cast<const void*>(kern), Cfg::LDS_BYTES, lds_allowed);
    note_kernel(ScaleKind == SCALE_BLOCK128 ? "pingpong_block128" : "pingpong");
    kern<<<dim3((unsigned)tiles), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream>>>(g);
}

}  // namespace w8a8
