// 256x256x128 8-bit NT GEMM for gfx950 with four waves and 128x128 register
// tiles, software-pipelined inside each wave.
//
// Why. With 32x32 MFMAs a 128(m) x 128(n) wave tile reads (128+128) x 128 bytes
// of operands from LDS per K slab for 2048 MFMA cycles: 128 KiB per workgroup
// and slab against the 192 KiB of eight 128x64 wave tiles. LDS serves both the
// operand reads and the incoming direct-to-LDS loads (64 KiB a slab), so that
// third less read traffic is what lets the MFMA pipe stay busy. The price: the
// 256 accumulator registers of a wave leave room for one wave per SIMD only, so
// nothing can hide one wave's memory phase behind another wave's MFMAs -- each
// wave interleaves its own LDS reads and loads between its own MFMAs instead.
//
// Pipeline of one wave, K slab k (two register sets F0, F1 of half a slab each;
// a slab's half h is chunks 2h, 2h+1 of every row, 64 bytes of K):
//   first half:   MFMAs on F0 = (k, half 0)   | LDS reads (k, half 1)   -> F1
//                                             | loads: activation rows of slab k+2
//   -- own loads of slab k+1 landed, own reads of slab k done; barrier --
//   second half:  MFMAs on F1 = (k, half 1)   | LDS reads (k+1, half 0) -> F0
//                                             | loads: weight rows of slab k+2
// The instruction order is written out and pinned (one MFMA, then at most two
// LDS reads and one load) so that the MFMA pipe always has the next instruction
// waiting. Three activation stages and two weight stages (all 160 KiB): the
// activation rows of slab k+2 may be fetched before the barrier that retires
// slab k, which spreads the loads evenly over the slab -- the CU's single load
// path is the scarce resource, see the comment at the main loop. No L2 prefetch
// touches here: a touch pulls its whole line through that same path a second
// time, which costs more than the L2 misses it saves.
//
// LDS layout of a stage, operand roles and accumulator layout are those of the
// ping-pong kernel: 256 activation rows then 256 weight rows of 128 bytes, chunk
// c of row r at position c ^ (r & 7) ^ ((r >> 3) & 1); weight rows are the
// first MFMA operand.
#pragma once
#include "gemm_pingpong.cuh"

namespace w8a8 {

struct Wave128Cfg {
    static constexpr int BM = 256, BN = 256, BK = 128;
    static constexpr int THREADS = 256;
    static constexpr int MI = 4, NI = 4;  // 32-row sub-tiles per wave: 128 m x 128 n
    static constexpr int OPERAND_BYTES = 256 * BK;       // one operand's slab: 32 KiB
    static constexpr int X_STAGES = 3, W_STAGES = 2;
    static constexpr int W_BASE = X_STAGES * OPERAND_BYTES;  // weights after activations
    static constexpr int EPI_ROW_BYTES = 272;            // 128 bf16 + 16 bytes of padding
    static constexpr int EPI_PASS_BYTES = 32 * EPI_ROW_BYTES;  // one 32-row pass of a wave
    static constexpr int LDS_BYTES = (X_STAGES + W_STAGES) * OPERAND_BYTES;  // all 160 KiB
    static_assert(4 * 2 * EPI_PASS_BYTES <= LDS_BYTES, "epilogue staging must fit");
};

// order in which a half slab's sixteen 16-byte operand pieces are read from LDS:
// the first MFMAs need weight sub-tile 0 and activation sub-tile 0, then the
// other weight sub-tiles, then the other activation sub-tiles (m is the outer
// MFMA loop)
__device__ constexpr int kReadIsW[8] = {1, 0, 1, 1, 1, 0, 0, 0};
__device__ constexpr int kReadSub[8] = {0, 0, 1, 2, 3, 1, 2, 3};

// silu(g) = g / (1 + exp(-g)) on the hardware's exp2 and reciprocal, the arithmetic of the
// SwiGLU producer kernel (quantize.hip)
__device__ __forceinline__ float silu_hw(float g) {
    return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.44269504088896340736f));
}

enum : int { EPI_PLAIN = 0, EPI_SWIGLU = 1, EPI_ROPE = 2, EPI_RESID = 3 };

// Knock-outs for the phase microbenchmark (ubench/wave128_phases.hip): each bit removes one
// class of instructions so that its share of the kernel's time -- issue slots and, under the
// power cap, clock -- can be read off a timing. The library instantiates KO = 0 only; a
// knocked-out kernel computes nothing meaningful.
enum : int { KO_LDS_READS = 1, KO_LOADS = 2, KO_MFMA = 4, KO_STORES = 8, KO_BARRIER = 16, KO_WAITS = 32 };

template <class Op, int ScaleKind, int Epi = EPI_PLAIN, int KO = 0>
__global__ __launch_bounds__(Wave128Cfg::THREADS) void gemm_wave128_kernel(GemmArgs g, RopeCacheArgs rc) {
    static_assert(ScaleKind != SCALE_BLOCK128, "block scales run on the ping-pong kernel");
    static_assert(Epi == EPI_PLAIN || ScaleKind == SCALE_ROWCOL, "the SwiGLU, rotary and residual epilogues are the int8 decoder's");
    PP_STAMP_INIT();
    using Cfg = Wave128Cfg;
    using Acc = typename Op::Acc;
    constexpr int MI = Cfg::MI, NI = Cfg::NI;
    constexpr int HS = Op::HALF_STEPS;
    constexpr int NM = HS * MI * NI;  // MFMAs per half slab
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave & 1;
    const int wave_n = wave >> 1;
    const int lrow = lane & 31;
    const int lgrp = lane >> 5;

    const int tiles_m = (g.m + Cfg::BM - 1) / Cfg::BM;
    const int tiles_n = (g.n + Cfg::BN - 1) / Cfg::BN;
    const TileCoord tc = map_tile(tiles_m, tiles_n);
    const int m0 = tc.tm * Cfg::BM, n0 = tc.tn * Cfg::BN;
    const int K = g.k;
    const int ksteps = K >> 7;
    // requested now, used in the epilogue: the latency hides under the main loop
    const EpilogueScalars es = load_epilogue_scalars<ScaleKind>(g);
    [[maybe_unused]] const float s_tensor = es.sa * es.sb;
    float sx[Cfg::MI];  // per-row scales of this lane's four rows (SCALE_ROWCOL)
#pragma unroll
    for (int mi = 0; mi < Cfg::MI; ++mi) {
        sx[mi] = 1.0f;
        if constexpr (ScaleKind == SCALE_ROWCOL) {
            const int m = m0 + wave_m * 128 + mi * 32 + lrow;
            sx[mi] = (m < g.m) ? g.sa[m] : 0.0f;
        }
    }

    // ---- direct-to-LDS load plan: wave w fills rows 64w..64w+63 of both
    // operands, 8 rows per instruction, 8 + 8 instructions per slab. Lane l lands
    // at row (l>>3), position (l&7) of its 1 KiB block and so fetches logical chunk
    // (l&7) ^ f(row): c0 = (l&7)^(l>>3) for even instructions, c0 ^ 1 for odd ones.
    // Rows past M / N are past the buffer's num_records and read as zero; a slab
    // past K is switched off by a zero-length descriptor.
    const uint32_t x_bytes = (uint32_t)g.m * (uint32_t)K, w_bytes = (uint32_t)g.n * (uint32_t)K;
    uint32_t x_off[2], w_off[2];
    {
        const int c0 = (lane & 7) ^ (lane >> 3);
        const uint32_t xr = (uint32_t)(m0 + wave * 64 + (lane >> 3)) * (uint32_t)K;
        const uint32_t wr = (uint32_t)(n0 + wave * 64 + (lane >> 3)) * (uint32_t)K;
        x_off[0] = xr + (uint32_t)c0 * 16;
        x_off[1] = xr + (uint32_t)(c0 ^ 1) * 16;
        w_off[0] = wr + (uint32_t)c0 * 16;
        w_off[1] = wr + (uint32_t)(c0 ^ 1) * 16;
    }
    const uint32_t row8 = 8u * (uint32_t)K;
    uint8_t* const dma_base = lds + wave * (64 * 128);

    // instruction r of 8 of one operand's slab
    auto dma_x = [&](int r, __amdgpu_buffer_rsrc_t rx, int xstage, uint32_t k0) {
        lds_dma16(rx, dma_base + xstage * Cfg::OPERAND_BYTES + r * 1024,
                  x_off[r & 1] + (uint32_t)r * row8, k0);
    };
    auto dma_w = [&](int r, __amdgpu_buffer_rsrc_t rw, int wstage, uint32_t k0) {
        lds_dma16(rw, dma_base + Cfg::W_BASE + wstage * Cfg::OPERAND_BYTES + r * 1024,
                  w_off[r & 1] + (uint32_t)r * row8, k0);
    };

    // ---- operand read plan
    int frag_off[4];
    {
        const int sw = (lrow & 7) ^ ((lrow >> 3) & 1);
#pragma unroll
        for (int j = 0; j < 4; ++j) frag_off[j] = lrow * 128 + (((4 * lgrp + j) ^ sw) << 4);
    }
    const int x_rd = (wave_m * 128) * 128;
    const int w_rd = Cfg::W_BASE + (wave_n * 128) * 128;

    // piece r of 16 of half h of the slab in activation stage xs / weight stage ws
    auto read_one = [&](int r, int xs, int ws, int h, u32x4 (&xf)[MI][2], u32x4 (&wf)[NI][2]) {
        const int which = r >> 1, c = r & 1, sub = kReadSub[which];
        if (kReadIsW[which])
            wf[sub][c] = *reinterpret_cast<const u32x4*>(
                lds + w_rd + ws * Cfg::OPERAND_BYTES + sub * 4096 + frag_off[2 * h + c]);
        else
            xf[sub][c] = *reinterpret_cast<const u32x4*>(
                lds + x_rd + xs * Cfg::OPERAND_BYTES + sub * 4096 + frag_off[2 * h + c]);
    };

    Acc acc[NI][MI];
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[ni][mi][j] = 0;

    u32x4 xf0[MI][2], wf0[NI][2], xf1[MI][2], wf1[NI][2];

    // MFMA number i of a half slab: K step outermost, then m, then n -- sixteen
    // accumulators in turn, never two MFMAs in a row on the same one
    auto mfma_one = [&](int i, const u32x4 (&xf)[MI][2], const u32x4 (&wf)[NI][2]) {
        const int s = i / (MI * NI), mi = (i / NI) % MI, ni = i % NI;
        acc[ni][mi] = Op::mma_half(s, wf[ni], xf[mi], acc[ni][mi]);
    };

    // ---- prologue: slabs 0 and 1 in flight; slab 0 visible; first half of slab 0 in F0
    PP_STAMP();
    {
        const __amdgpu_buffer_rsrc_t rx = make_rsrc(g.a, x_bytes), rw = make_rsrc(g.b, w_bytes);
        const __amdgpu_buffer_rsrc_t rx1 = make_rsrc(g.a, ksteps > 1 ? x_bytes : 0u);
        const __amdgpu_buffer_rsrc_t rw1 = make_rsrc(g.b, ksteps > 1 ? w_bytes : 0u);
#pragma unroll
        for (int r = 0; r < 8; ++r) dma_x(r, rx, 0, 0u);
#pragma unroll
        for (int r = 0; r < 8; ++r) dma_w(r, rw, 0, 0u);
#pragma unroll
        for (int r = 0; r < 8; ++r) dma_x(r, rx1, 1, 128u);
#pragma unroll
        for (int r = 0; r < 8; ++r) dma_w(r, rw1, 1, 128u);
        if constexpr (KO & KO_LOADS) {  // every stage holds operand bytes once and for all
#pragma unroll
            for (int r = 0; r < 8; ++r) dma_x(r, rx1, 2, 256u);
            wait_vmcnt<0>();
        } else {
            wait_vmcnt<16>();  // slab 0
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 16; ++r) read_one(r, 0, 0, 0, xf0, wf0);
        if constexpr (KO & KO_LDS_READS) {  // both register sets hold operand bytes once and for all
#pragma unroll
            for (int r = 0; r < 16; ++r) read_one(r, 0, 0, 1, xf1, wf1);
        }
    }

    // reads are spread over the first three quarters of a half's MFMAs so that the
    // last one has returned by the time the half ends; the eight loads of a half
    // over all of them, one every other MFMA -- the CU's one load path takes a
    // 1 KiB instruction every 16 cycles, so four waves issuing one per 64-cycle
    // MFMA would saturate it and stall their own instruction streams
    constexpr int kReadSpan = (3 * NM) / 4;

    int xs = 0;  // k % 3
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(g.a, x_bytes), rw = make_rsrc(g.b, w_bytes);

    // one K slab; LOADS: slab k+2 exists and is fetched during this one
    auto slab = [&](auto loads_c, int k) {
        constexpr bool LOADS = decltype(loads_c)::value;
        const int ws = k & 1;
        const int xs1 = (xs == 2) ? 0 : xs + 1;   // (k + 1) % 3
        const int xs2 = (xs == 0) ? 2 : xs - 1;   // (k + 2) % 3
        const uint32_t k2 = (uint32_t)(k + 2) << 7;

        // first half: MFMAs on F0, reads of (k, half 1) into F1, activation rows
        // of slab k+2 into the stage slab k-1 left at the previous barrier
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < NM; ++i) {
            if constexpr (!(KO & KO_MFMA)) mfma_one(i, xf0, wf0);
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if constexpr (!(KO & KO_LDS_READS))
                    if ((r * kReadSpan) / 16 == i) read_one(r, xs, ws, 1, xf1, wf1);
            if constexpr (LOADS && !(KO & KO_LOADS)) {
#pragma unroll
                for (int d = 0; d < 8; ++d)
                    if ((d * NM) / 8 == i) dma_x(d, rx, xs2, k2);
            }
            __builtin_amdgcn_sched_barrier(0);
        }

        // Slab k+1 has landed for this wave -- all but this half's eight loads are
        // older -- and this wave is done reading slab k; after the barrier both
        // hold for every wave.
        wait_vmcnt<(LOADS && !(KO & KO_LOADS)) ? 8 : 0>();
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
        phase_barrier();

        // second half: MFMAs on F1, reads of (k+1, half 0) into F0 (stale bytes
        // after the last slab, never used), weight rows of slab k+2 into the stage
        // slab k occupied
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < NM; ++i) {
            if constexpr (!(KO & KO_MFMA)) mfma_one(i, xf1, wf1);
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if constexpr (!(KO & KO_LDS_READS))
                    if ((r * kReadSpan) / 16 == i) read_one(r, xs1, ws ^ 1, 0, xf0, wf0);
            if constexpr (LOADS && !(KO & KO_LOADS)) {
#pragma unroll
                for (int d = 0; d < 8; ++d)
                    if ((d * NM) / 8 == i) dma_w(d, rw, ws, k2);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        xs = xs1;
    };

    int k = 0;
    PP_STAMP();
    for (; k + 2 < ksteps; ++k) slab(std::true_type{}, k);
    for (; k < ksteps; ++k) slab(std::false_type{}, k);
    // no load outlives the loop; the stages are dead for every wave
    PP_STAMP();
    __builtin_amdgcn_s_waitcnt(0x0070);
    phase_barrier();

    // ---------------- epilogue ----------------
    // bf16 only, N % 8 == 0 (the launcher sends everything else to the ping-pong
    // kernel). Through LDS: the wave lays 32(m) x 128(n) values down row-major
    // (272-byte rows) in a private staging buffer and streams them out as full
    // 128-byte lines, 16 bytes a lane; four such passes over two buffers in turn, so
    // the first stores leave after a quarter of the conversions. Per-column operands
    // are all requested before the first one is used: one memory latency, not one
    // per use. Output rows go through a buffer descriptor: rows past M and (by the
    // offset chosen below) columns past N are dropped by the bounds check -- no
    // predicates, no 64-bit address arithmetic per store; the row step goes into the
    // checked (vector) offset because the scalar offset of a buffer instruction
    // takes no part in the check. The stores are non-temporal (aux bit 1): the
    // 2 M N output bytes stream to memory while the epilogue still computes instead
    // of sitting dirty in L2 until the end-of-kernel write-back (-1.5 us at 4096^3).
    if constexpr (Epi == EPI_ROPE) {
        // The rows are the fused q|k|v projection of a decoder layer, head_dim 128: the 128
        // columns of a wave tile are one head. The epilogue goes on where the separate rotary /
        // cache-write kernel would start: the bf16-rounded value pairs of q and k are rotated
        // (fp32 products and sums rounded one by one, one rounding to bf16 -- the arithmetic of
        // rope_cache.hip on the same rounded inputs), a pass of 32 tokens x 128 dims is staged
        // through LDS and leaves as whole 256-byte head rows: q to [batch, heads, seq, 128], k
        // and v into the cache at the tokens' positions (a position outside the cache: nothing).
        constexpr int ROWB = Cfg::EPI_ROW_BYTES, PASS_BYTES = Cfg::EPI_PASS_BYTES;
        uint8_t* const mine = lds + wave * (2 * PASS_BYTES);
        const int nwv = n0 + wave_n * 128;
        const int hh = nwv >> 7;                         // head among q heads | k heads | v heads
        const bool live_head = nwv < g.n;
        const bool is_q = hh < rc.n_heads, rotate = hh < rc.n_heads + rc.n_kv_heads;
        const int hk = hh - rc.n_heads - (rotate ? 0 : rc.n_kv_heads);
        const int mw = m0 + wave_m * 128;                // first token of this wave
        f32x4 sw4[NI][4];
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = nwv + ni * 32 + q * 8 + lgrp * 4;
                sw4[ni][q] = (n < g.n) ? *reinterpret_cast<const f32x4*>(g.sb + n) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
        void* const dst_base = is_q ? rc.q_out : (rotate ? rc.k_cache : rc.v_cache);
        const uint32_t dst_bytes = is_q ? (uint32_t)g.m * (uint32_t)rc.n_heads * 256u
                                        : (uint32_t)rc.batch * (uint32_t)rc.n_kv_heads * (uint32_t)rc.max_len * 256u;
        const __amdgpu_buffer_rsrc_t rout = make_rsrc(dst_base, live_head ? dst_bytes : 0u);
        const int r4 = lane >> 4, c16 = lane & 15;
        // One wave per SIMD: nothing hides a memory round trip inside the epilogue, so everything
        // it reads is requested ahead of its use -- the destinations of all 32 rows this lane will
        // store (cache slots: one lookup of the token's position each) now, the (cos, sin) pairs of
        // a group of 32 columns two groups before the group that uses them.
        // token index -> (sequence, token in sequence) without an integer division per row: the
        // float quotient of m < 2^23 is off by at most one, which the remainder shows
        const float inv_seq = 1.0f / (float)rc.seq;
        auto split_token = [&](int m, int& bt, int& sq) {
            bt = (int)((float)m * inv_seq);
            sq = m - bt * rc.seq;
            if (sq < 0) { --bt; sq += rc.seq; }
            else if (sq >= rc.seq) { ++bt; sq -= rc.seq; }
        };
        uint32_t dst_off[MI][8];
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int m = mw + mi * 32 + i * 4 + r4;
                int bt, sq;
                split_token(m, bt, sq);
                dst_off[mi][i] = kOutOfRange;
                if (m < g.m) {
                    if (is_q) {
                        dst_off[mi][i] = (uint32_t)((bt * rc.n_heads + hh) * rc.seq + sq) * 256u + (uint32_t)c16 * 16u;
                    } else {
                        const int64_t pos = rc.positions[sq];
                        if (pos >= 0 && pos < rc.max_len)
                            dst_off[mi][i] = (uint32_t)((int64_t)(bt * rc.n_kv_heads + hk) * rc.max_len + pos) * 256u +
                                             (uint32_t)c16 * 16u;
                    }
                }
            }
        // group gi = mi * NI + ni: the lane's token of pass mi, columns 32 ni .. 32 ni + 31
        constexpr int kAhead = 2;
        f32x4 cs[kAhead + 1][4];
        const float* cs_row[MI];
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            int bt, sq;
            split_token(mw + mi * 32 + lrow, bt, sq);
            cs_row[mi] = rc.freqs + ((int64_t)sq * 64 + (lgrp * 2)) * 2;
        }
        auto request_cs = [&](int gi) {
            if (!rotate || gi >= MI * NI) return;
            const int mi = gi / NI, ni = gi % NI;
#pragma unroll
            for (int q = 0; q < 4; ++q)  // d = 32 ni + 8 q + 4 lgrp: pair index d / 2
                cs[gi % (kAhead + 1)][q] = *reinterpret_cast<const f32x4*>(cs_row[mi] + (ni * 16 + q * 4) * 2);
        };
#pragma unroll
        for (int gi = 0; gi < kAhead; ++gi) request_cs(gi);
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            uint8_t* const buf = mine + (mi & 1) * PASS_BYTES;
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) {
                const int gi = mi * NI + ni;
                request_cs(gi + kAhead);
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float v[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
#pragma clang fp contract(off)
                        v[j] = (float)acc[ni][mi][4 * q + j] * sx[mi] * sw4[ni][q][j];
                    }
                    u32x2 pk;
                    pk.x = pack_bf16x2(v[0], v[1]);
                    pk.y = pack_bf16x2(v[2], v[3]);
                    if (rotate) {
                        const f32x4 c4 = cs[gi % (kAhead + 1)][q];
                        const float x[4] = {__uint_as_float(pk.x << 16), __uint_as_float(pk.x & 0xffff0000u),
                                            __uint_as_float(pk.y << 16), __uint_as_float(pk.y & 0xffff0000u)};
                        float y[4];
#pragma unroll
                        for (int p = 0; p < 2; ++p) {
#pragma clang fp contract(off)
                            const float c = c4[2 * p], sn = c4[2 * p + 1];
                            const float xe = x[2 * p], xo = x[2 * p + 1];
                            const float a0 = xe * c, a1 = xo * sn, b0 = xe * sn, b1 = xo * c;
                            y[2 * p] = a0 - a1;
                            y[2 * p + 1] = b0 + b1;
                        }
                        pk.x = pack_bf16x2(y[0], y[1]);
                        pk.y = pack_bf16x2(y[2], y[3]);
                    }
                    *reinterpret_cast<u32x2*>(buf + lrow * ROWB + (ni * 32 + q * 8 + lgrp * 4) * 2) = pk;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const u32x4 v = *reinterpret_cast<const u32x4*>(buf + (i * 4 + r4) * ROWB + c16 * 16);
                __builtin_amdgcn_raw_buffer_store_b128(v, rout, dst_off[mi][i], 0, 0);
            }
        }
    } else
    if constexpr (Epi == EPI_SWIGLU) {
        // The wave's 128 columns are 64 gate columns (sub-tiles 0, 1) and the 64 up columns
        // (sub-tiles 2, 3) of the same 64 columns of h, so a lane holds every pair in its own
        // registers. gate and up are rounded to bf16 as the plain epilogue would have stored
        // them, then h = bf16(up * bf16(silu(gate))) -- the arithmetic of the SwiGLU producer
        // kernel on the same rounded inputs. A pass is 32 rows x 64 columns of h (one 128-byte
        // line per row) staged through wave-private LDS (144-byte rows) and stored as whole
        // lines; the maximum of |h| over the wave's 64 columns goes to row_max[m, piece] (bf16
        // magnitudes order like their bit patterns, so the maximum is taken on the packed bits).
        constexpr int ROWB = 144, PASS_BYTES = 32 * ROWB;
        uint8_t* const mine = lds + wave * (2 * PASS_BYTES);
        const int rows_here = min(Cfg::BM, g.m - m0);
        const int hw = g.n >> 1;                       // width of h
        const uint32_t row_bytes = (uint32_t)hw * 2u;
        const __amdgpu_buffer_rsrc_t rout =
            make_rsrc(static_cast<uint16_t*>(g.out) + (size_t)m0 * hw, (uint32_t)rows_here * row_bytes);
        const int nwv = n0 + wave_n * 128;             // first fused column of this wave
        const int piece = nwv >> 7;                    // its 64-column piece of h
        const int pieces = g.n >> 7;
        f32x4 sw4[NI][4];
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = nwv + ni * 32 + q * 8 + lgrp * 4;
                sw4[ni][q] = (n < g.n) ? *reinterpret_cast<const f32x4*>(g.sb + n) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
        const int r8 = lane >> 3, c8 = lane & 7;
        const uint32_t lane_off = (nwv < g.n)
            ? (uint32_t)(wave_m * 128 + r8) * row_bytes + (uint32_t)(piece * 64 + c8 * 8) * 2u
            : kOutOfRange;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            uint8_t* const buf = mine + (mi & 1) * PASS_BYTES;
            uint32_t mx = 0u;
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float gt[4], up[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
#pragma clang fp contract(off)
                        gt[j] = (float)acc[ni][mi][4 * q + j] * sx[mi] * sw4[ni][q][j];
                        up[j] = (float)acc[ni + 2][mi][4 * q + j] * sx[mi] * sw4[ni + 2][q][j];
                    }
                    u32x2 pk;
#pragma unroll
                    for (int p = 0; p < 2; ++p) {
                        const uint32_t gb = pack_bf16x2(gt[2 * p], gt[2 * p + 1]);
                        const uint32_t ub = pack_bf16x2(up[2 * p], up[2 * p + 1]);
                        const uint32_t sb2 = pack_bf16x2(silu_hw(__uint_as_float(gb << 16)),
                                                         silu_hw(__uint_as_float(gb & 0xffff0000u)));
                        const uint32_t hb = pack_bf16x2(
                            __uint_as_float(ub << 16) * __uint_as_float(sb2 << 16),
                            __uint_as_float(ub & 0xffff0000u) * __uint_as_float(sb2 & 0xffff0000u));
                        pk[p] = hb;
                        const uint32_t mag = hb & 0x7fff7fffu;
                        mx = max(mx, max(mag & 0xffffu, mag >> 16));
                    }
                    *reinterpret_cast<u32x2*>(buf + lrow * ROWB + (ni * 32 + q * 8 + lgrp * 4) * 2) = pk;
                }
            // the other half of the row's columns sits in lane ^ 32
            mx = max(mx, (uint32_t)__shfl_xor((int)mx, 32, 64));
            const int m = m0 + wave_m * 128 + mi * 32 + lrow;
            if (lgrp == 0 && m < g.m && nwv < g.n) g.row_max[(size_t)m * pieces + piece] = __uint_as_float(mx << 16);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const u32x4 v = *reinterpret_cast<const u32x4*>(buf + (i * 8 + r8) * ROWB + c8 * 16);
                __builtin_amdgcn_raw_buffer_store_b128(
                    v, rout, lane_off + (uint32_t)(mi * 32 + i * 8) * row_bytes, 0, 2);
            }
        }
    } else
    {
        constexpr int ROWB = Cfg::EPI_ROW_BYTES, PASS_BYTES = Cfg::EPI_PASS_BYTES;
        uint8_t* const mine = lds + wave * (2 * PASS_BYTES);
        const uint16_t* bias = static_cast<const uint16_t*>(g.bias);
        const int rows_here = min(Cfg::BM, g.m - m0);
        const uint32_t row_bytes = (uint32_t)g.n * 2u;
        const __amdgpu_buffer_rsrc_t rout =
            make_rsrc(static_cast<uint16_t*>(g.out) + (size_t)m0 * g.n, (uint32_t)rows_here * row_bytes);
        const int nwv = n0 + wave_n * 128;
        f32x4 sw4[NI][4];
        u32x2 braw[NI][4];
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = nwv + ni * 32 + q * 8 + lgrp * 4;
                sw4[ni][q] = f32x4{1.0f, 1.0f, 1.0f, 1.0f};
                braw[ni][q] = u32x2{0u, 0u};
                if (n < g.n) {
                    if constexpr (ScaleKind == SCALE_ROWCOL)
                        sw4[ni][q] = *reinterpret_cast<const f32x4*>(g.sb + n);
                    if constexpr (Epi != EPI_RESID)   // (no bias with the residual epilogue: registers)
                        if (bias) braw[ni][q] = *reinterpret_cast<const u32x2*>(bias + n);
                }
            }
        const int r4 = lane >> 4, c16 = lane & 15;
        const int nst = nwv + c16 * 8;
        const uint32_t lane_off = (nst < g.n)
            ? (uint32_t)(wave_m * 128 + r4) * row_bytes + (uint32_t)nst * 2u
            : kOutOfRange;
        // EPI_RESID: the residual rows of this tile, addressed like the output
        [[maybe_unused]] const __amdgpu_buffer_rsrc_t rres = make_rsrc(
            static_cast<const uint16_t*>(Epi == EPI_RESID ? g.resid : g.out) + (size_t)m0 * g.n,
            (uint32_t)rows_here * row_bytes);
        // the eight residual pieces of a pass live in a ring: each is requested again for the
        // next pass as soon as it has been used, a whole pass ahead of its use
        [[maybe_unused]] u32x4 rr[8];
        if constexpr (Epi == EPI_RESID) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                rr[i] = buf_load16(rres, lane_off + (uint32_t)(i * 4) * row_bytes, 0);
        }
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            uint8_t* const buf = mine + (mi & 1) * PASS_BYTES;
#pragma unroll
            for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int nl = ni * 32 + q * 8 + lgrp * 4;
                    const u32x2 raw = Epi == EPI_RESID ? u32x2{0u, 0u} : braw[ni][q];
                    const f32x4 b4 = {__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u),
                                      __uint_as_float(raw.y << 16), __uint_as_float(raw.y & 0xffff0000u)};
                    float v[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float f = (float)acc[ni][mi][4 * q + j];
                        if constexpr (ScaleKind == SCALE_TENSOR) {
                            v[j] = f * s_tensor + b4[j];
                        } else {
#pragma clang fp contract(off)
                            const float scaled = f * sx[mi] * sw4[ni][q][j];
                            v[j] = scaled + b4[j];
                        }
                    }
                    u32x2 pk;
                    pk.x = pack_bf16x2(v[0], v[1]);
                    pk.y = pack_bf16x2(v[2], v[3]);
                    *reinterpret_cast<u32x2*>(buf + lrow * ROWB + nl * 2) = pk;
                }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                u32x4 v = *reinterpret_cast<const u32x4*>(buf + (i * 4 + r4) * ROWB + c16 * 16);
                if constexpr (Epi == EPI_RESID) {
                    // bf16(y + residual) on the rounded y, element by element
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t y2 = v[e], r2 = rr[i][e];
                        v[e] = pack_bf16x2(__uint_as_float(y2 << 16) + __uint_as_float(r2 << 16),
                                           __uint_as_float(y2 & 0xffff0000u) + __uint_as_float(r2 & 0xffff0000u));
                    }
                    if (mi + 1 < MI)
                        rr[i] = buf_load16(rres, lane_off + (uint32_t)((mi + 1) * 32 + i * 4) * row_bytes, 0);
                }
                if constexpr (!(KO & KO_STORES))
                    __builtin_amdgcn_raw_buffer_store_b128(
                        v, rout, lane_off + (uint32_t)(mi * 32 + i * 4) * row_bytes, 0, 2);
            }
        }
    }
    PP_STAMP();
}

// bf16 output with whole 16-byte output pieces only; other outputs keep the
// ping-pong kernel, whose epilogue handles every case
inline bool wave128_shape_ok(const GemmArgs& g) {
    // (a tile's 256 output rows are addressed with 32-bit byte offsets)
    return pingpong_shape_ok(g) && g.out_kind == OUT_BF16 && (g.n & 7) == 0 && g.n <= (1 << 22);
}

// A token count a little above a multiple of 256 (M = 256 q + r, 0 < r <= 128) can cost the
// large-tile kernel a whole extra round of workgroups for r rows (4100 x 4096 x 4096: 272 tiles on
// 256 compute units, 96 us against 69 us at 4096 rows). When it does, and the weight-streaming
// decode kernel takes the shape, those rows are better served by it in a launch of their own
// (70 us for the two). Returns r then, else 0.
inline int ragged_tail_rows(const GemmArgs& g) {
    const int r = g.m & 255;
    if (r == 0 || r > 128 || g.m < 256 || (g.k & 255) != 0) return 0;
    const int64_t tn = (g.n + 255) / 256;
    const int64_t full = (int64_t)((g.m + 255) / 256) * tn, cut = (int64_t)(g.m / 256) * tn;
    return (full + 255) / 256 > (cut + 255) / 256 ? r : 0;
}

// the first m - r rows and the last r rows of a product as calls of their own (bf16 output;
// `rowcol`: sa holds one step per row)
inline void split_rows(const GemmArgs& g, int r, bool rowcol, GemmArgs& head, GemmArgs& tail) {
    head = g;
    head.m = g.m - r;
    tail = g;
    tail.m = r;
    const size_t row0 = (size_t)head.m;
    tail.a = static_cast<const uint8_t*>(g.a) + row0 * (size_t)g.k;
    if (rowcol) tail.sa = g.sa + row0;
    tail.out = static_cast<uint8_t*>(g.out) + row0 * (size_t)g.n * 2;
    if (g.resid) tail.resid = static_cast<const uint8_t*>(g.resid) + row0 * (size_t)g.n * 2;
}

template <class Op, int ScaleKind, int Epi = EPI_PLAIN>
inline void launch_wave128(const GemmArgs& g, hipStream_t stream, const RopeCacheArgs& rc = RopeCacheArgs{}) {
    using Cfg = Wave128Cfg;
    const int tiles = ((g.m + Cfg::BM - 1) / Cfg::BM) * ((g.n + Cfg::BN - 1) / Cfg::BN);
    auto kern = gemm_wave128_kernel<Op, ScaleKind, Epi>;
    static std::atomic<uint64_t> lds_allowed{0};
    allow_dynamic_lds(reinterpret_cast<const void*>(kern), Cfg::LDS_BYTES, lds_allowed);
    note_kernel(Epi == EPI_SWIGLU ? "wave128_swiglu" : Epi == EPI_ROPE ? "wave128_rope" : Epi == EPI_RESID ? "wave128_resid" : "wave128");
    kern<<<dim3((unsigned)tiles), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream>>>(g, rc);
}

}  // namespace w8a8
