// The four-wave 256x256x128 fp8 NT GEMM on the 16x16x128 MFMA
// (v_mfma_f32_16x16x128_f8f6f4) instead of the 32x32x64 one.
//
// Why. Under the board's power cap a register-resident loop of the 16x16x128
// instruction sustains a few percent more than the 32x32x64 one on toggling
// operands; the tile, the LDS ring, the direct-to-LDS load plan, the barrier per
// slab and the bytes moved per slab are those of gemm_wave128_kernel.
//
// What changes. One 16x16x128 MFMA consumes a whole 128-byte K slab of its 16 + 16
// rows, so a slab cannot be halved along K. It is cut into quadrants instead: the
// 128(m) x 128(n) wave tile = 2 x 2 quadrants of 64 x 64 = 4 x 4 MFMAs of 32
// cycles each. A quadrant needs one half of the wave's activation rows (4 sub-tiles
// of 16 rows: 32 registers) and one half of its weight rows (32 registers). The
// quadrants are walked so that consecutive ones share one of the two halves, and
// during a quadrant the one half the next quadrant is missing is read from LDS into
// the buffer that is idle: four 32-register buffers XA, XB (activation halves 0, 1)
// and WA, WB (weight halves 0, 1) -- 128 operand registers, as in the 32x32 kernel.
// The walk has period two slabs (Q<x half><w half>, what is read meanwhile):
//   even slab k:   Q00 | W1(k) -> WB     Q01 | X1(k) -> XB      -- barrier --
//                  Q11 | X0(k+1) -> XA   Q10 | W1(k+1) -> WB
//   odd slab k+1:  Q01 | W0(k+1) -> WA   Q00 | X1(k+1) -> XB    -- barrier --
//                  Q10 | X0(k+2) -> XA   Q11 | W0(k+2) -> WA
// Every phase is 16 MFMAs (512 cycles) with 8 LDS reads of 1 KiB and 4 direct-to-LDS
// loads between them: the per-cycle rates of the 32x32 kernel. All of a slab's
// operands have been read when its second phase ends, which is where the 32x32
// kernel has its barrier too: the stage lifetimes, and with them the load plan
// (activation rows of slab k+2 in the first half of slab k, weight rows in the second
// half) carry over unchanged.
//
// Operand roles and layouts: weight rows are the first MFMA operand; lane l supplies
// row (l & 15) of a sub-tile and the 32 bytes of K-group (l >> 4) (chunks 2g, 2g+1
// of the row's eight 16-byte chunks; any assignment of K bytes to lanes is a valid
// contraction as long as both operands share it); the accumulator lane holds, for
// token m = l & 15, the four outputs n = 4 (l >> 4) .. + 3 of the sub-tile.
#pragma once
#include "gemm_wave128.cuh"

namespace w8a8 {

template <int Fmt, int ScaleKind, int KO = 0>
__global__ __launch_bounds__(Wave128Cfg::THREADS) void gemm_wave128_q16_kernel(GemmArgs g) {
    static_assert(ScaleKind == SCALE_TENSOR || ScaleKind == SCALE_ROWCOL, "per-tensor or row x column scales");
    PP_STAMP_INIT();
    using Cfg = Wave128Cfg;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave & 1;
    const int wave_n = wave >> 1;
    const int lrow = lane & 15;
    const int lgrp = lane >> 4;

    const int tiles_m = (g.m + Cfg::BM - 1) / Cfg::BM;
    const int tiles_n = (g.n + Cfg::BN - 1) / Cfg::BN;
    const TileCoord tc = map_tile(tiles_m, tiles_n);
    const int m0 = tc.tm * Cfg::BM, n0 = tc.tn * Cfg::BN;
    const int K = g.k;
    const int ksteps = K >> 7;
    // requested now, used in the epilogue: the latency hides under the main loop
    const EpilogueScalars es = load_epilogue_scalars<ScaleKind>(g);
    [[maybe_unused]] const float s_tensor = es.sa * es.sb;
    float sx[8];  // per-row scales of this lane's eight rows (SCALE_ROWCOL)
#pragma unroll
    for (int mi = 0; mi < 8; ++mi) {
        sx[mi] = 1.0f;
        if constexpr (ScaleKind == SCALE_ROWCOL) {
            const int m = m0 + wave_m * 128 + mi * 16 + lrow;
            sx[mi] = (m < g.m) ? g.sa[m] : 0.0f;
        }
    }

    // ---- direct-to-LDS load plan (that of gemm_wave128_kernel): wave w fills rows
    // 64w..64w+63 of both operands, 8 rows per instruction, 8 + 8 instructions per slab
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
    auto dma_x = [&](int r, __amdgpu_buffer_rsrc_t rx, int xstage, uint32_t k0) __attribute__((always_inline)) {
        lds_dma16(rx, dma_base + xstage * Cfg::OPERAND_BYTES + r * 1024,
                  x_off[r & 1] + (uint32_t)r * row8, k0);
    };
    auto dma_w = [&](int r, __amdgpu_buffer_rsrc_t rw, int wstage, uint32_t k0) __attribute__((always_inline)) {
        lds_dma16(rw, dma_base + Cfg::W_BASE + wstage * Cfg::OPERAND_BYTES + r * 1024,
                  w_off[r & 1] + (uint32_t)r * row8, k0);
    };

    // ---- operand read plan: the lane's two chunks of its row of a 16-row sub-tile
    int frag_off[2];
    {
        const int sw = (lrow & 7) ^ ((lrow >> 3) & 1);
#pragma unroll
        for (int j = 0; j < 2; ++j) frag_off[j] = lrow * 128 + (((2 * lgrp + j) ^ sw) << 4);
    }
    const int x_rd = (wave_m * 128) * 128;
    const int w_rd = Cfg::W_BASE + (wave_n * 128) * 128;
    // piece r of 8 of half h of an operand: sub-tile 4h + r/2, chunk r%2
    auto read_x = [&](int r, int stage, int h, u32x4 (&f)[4][2]) __attribute__((always_inline)) {
        f[r >> 1][r & 1] = *reinterpret_cast<const u32x4*>(
            lds + x_rd + stage * Cfg::OPERAND_BYTES + (4 * h + (r >> 1)) * 2048 + frag_off[r & 1]);
    };
    auto read_w = [&](int r, int stage, int h, u32x4 (&f)[4][2]) __attribute__((always_inline)) {
        f[r >> 1][r & 1] = *reinterpret_cast<const u32x4*>(
            lds + w_rd + stage * Cfg::OPERAND_BYTES + (4 * h + (r >> 1)) * 2048 + frag_off[r & 1]);
    };

    f32x4 acc[8][8];  // [n sub-tile][m sub-tile]
#pragma unroll
    for (int ni = 0; ni < 8; ++ni)
#pragma unroll
        for (int mi = 0; mi < 8; ++mi) acc[ni][mi] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    u32x4 xa[4][2], xb[4][2], wa[4][2], wb[4][2];

    // MFMA i of 16 of quadrant (activation half xh, weight half wh): m outer, n inner
    auto mfma_one = [&](int i, const u32x4 (&xf)[4][2], const u32x4 (&wf)[4][2], int xh, int wh) __attribute__((always_inline)) {
        const int mi = i >> 2, ni = i & 3;
        const i32x8 a = {(int)wf[ni][0].x, (int)wf[ni][0].y, (int)wf[ni][0].z, (int)wf[ni][0].w,
                         (int)wf[ni][1].x, (int)wf[ni][1].y, (int)wf[ni][1].z, (int)wf[ni][1].w};
        const i32x8 b = {(int)xf[mi][0].x, (int)xf[mi][0].y, (int)xf[mi][0].z, (int)xf[mi][0].w,
                         (int)xf[mi][1].x, (int)xf[mi][1].y, (int)xf[mi][1].z, (int)xf[mi][1].w};
        acc[4 * wh + ni][4 * xh + mi] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
            a, b, acc[4 * wh + ni][4 * xh + mi], Fmt, Fmt, 0, 0, 0, 0);
    };

    // ---- prologue: slabs 0 and 1 in flight; slab 0 visible; halves 0 of slab 0 in XA, WA
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
        for (int r = 0; r < 8; ++r) read_x(r, 0, 0, xa);
#pragma unroll
        for (int r = 0; r < 8; ++r) read_w(r, 0, 0, wa);
        if constexpr (KO & KO_LDS_READS) {  // all four buffers hold operand bytes once and for all
#pragma unroll
            for (int r = 0; r < 8; ++r) read_x(r, 0, 1, xb);
#pragma unroll
            for (int r = 0; r < 8; ++r) read_w(r, 0, 1, wb);
        }
    }

    int xs = 0;  // k % 3

    // One quadrant: 16 MFMAs on (xf, wf); between them the 8 reads `rd(r)` of the half the
    // next quadrant is missing, spread over the first twelve MFMAs so that the last has
    // returned when the phase ends, and the 4 loads `ld(d)` of this quarter slab, one every
    // fourth MFMA (the CU's one load path takes a 1 KiB instruction every 16 cycles: four
    // waves must not issue them faster than one per 128 cycles each).
    auto phase = [&](const u32x4 (&xf)[4][2], const u32x4 (&wf)[4][2], int xh, int wh, auto&& rd, auto&& ld) __attribute__((always_inline)) {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            if constexpr (!(KO & KO_MFMA)) mfma_one(i, xf, wf, xh, wh);
            if constexpr (!(KO & KO_LDS_READS)) {
#pragma unroll
                for (int r = 0; r < 8; ++r)
                    if ((r * 12) / 8 == i) rd(r);
            }
#pragma unroll
            for (int d = 0; d < 4; ++d)
                if (d * 4 + 2 == i) ld(d);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // one K slab; ODD: its place in the two-slab walk. Past the end of K the loads of slab k+2
    // run on a zero-length descriptor: no memory traffic, zeros into a stage nobody reads again.
    auto slab = [&](auto odd_c, int k) __attribute__((always_inline)) {
        constexpr bool ODD = decltype(odd_c)::value;
        constexpr bool LOADS = !(KO & KO_LOADS);
        const int ws = k & 1;
        const int xs1 = (xs == 2) ? 0 : xs + 1;   // (k + 1) % 3
        const int xs2 = (xs == 0) ? 2 : xs - 1;   // (k + 2) % 3
        const uint32_t k2 = (uint32_t)(k + 2) << 7;
        const bool more = k + 2 < ksteps;
        const __amdgpu_buffer_rsrc_t rx = make_rsrc(g.a, more ? x_bytes : 0u);
        const __amdgpu_buffer_rsrc_t rw = make_rsrc(g.b, more ? w_bytes : 0u);
        auto ldx = [&](int base) __attribute__((always_inline)) { return [&, base](int d) __attribute__((always_inline)) { (void)base; if constexpr (LOADS) dma_x(base + d, rx, xs2, k2); }; };
        auto ldw = [&](int base) __attribute__((always_inline)) { return [&, base](int d) __attribute__((always_inline)) { (void)base; if constexpr (LOADS) dma_w(base + d, rw, ws, k2); }; };

        if constexpr (!ODD) {
            phase(xa, wa, 0, 0, [&](int r) __attribute__((always_inline)) { read_w(r, ws, 1, wb); }, ldx(0));
            phase(xa, wb, 0, 1, [&](int r) __attribute__((always_inline)) { read_x(r, xs, 1, xb); }, ldx(4));
        } else {
            phase(xa, wb, 0, 1, [&](int r) __attribute__((always_inline)) { read_w(r, ws, 0, wa); }, ldx(0));
            phase(xa, wa, 0, 0, [&](int r) __attribute__((always_inline)) { read_x(r, xs, 1, xb); }, ldx(4));
        }
        // Slab k+1 has landed for this wave -- all but this half's eight loads are older --
        // and this wave is done reading slab k; after the barrier both hold for every wave.
        if constexpr (!(KO & KO_WAITS)) {
            wait_vmcnt<LOADS ? 8 : 0>();
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
        }
        if constexpr (!(KO & KO_BARRIER)) phase_barrier();
        // (after the last slab the reads below fetch stale bytes that are never used)
        if constexpr (!ODD) {
            phase(xb, wb, 1, 1, [&](int r) __attribute__((always_inline)) { read_x(r, xs1, 0, xa); }, ldw(0));
            phase(xb, wa, 1, 0, [&](int r) __attribute__((always_inline)) { read_w(r, ws ^ 1, 1, wb); }, ldw(4));
        } else {
            phase(xb, wa, 1, 0, [&](int r) __attribute__((always_inline)) { read_x(r, xs1, 0, xa); }, ldw(0));
            phase(xb, wb, 1, 1, [&](int r) __attribute__((always_inline)) { read_w(r, ws ^ 1, 0, wa); }, ldw(4));
        }
        xs = xs1;
    };

    // the launcher sends only even slab counts here: the loop body is the two-slab walk
    PP_STAMP();
    for (int k = 0; k < ksteps; k += 2) {
        slab(std::false_type{}, k);
        slab(std::true_type{}, k + 1);
    }
    // no load outlives the loop; the stages are dead for every wave
    PP_STAMP();
    __builtin_amdgcn_s_waitcnt(0x0070);
    phase_barrier();

    // ---------------- epilogue ----------------
    // bf16, N % 8 == 0. A pass is 32 tokens (two m sub-tiles) x 128 columns, laid down
    // row-major in a wave-private staging buffer (272-byte rows: the 8-byte writes of 32
    // lanes cover all 64 banks once) and streamed out as whole 256-byte row pieces, 16
    // bytes a lane, through a bounds-checked buffer descriptor; two buffers in turn.
    {
        constexpr int ROWB = Cfg::EPI_ROW_BYTES, PASS_BYTES = Cfg::EPI_PASS_BYTES;
        uint8_t* const mine = lds + wave * (2 * PASS_BYTES);
        const uint16_t* bias = static_cast<const uint16_t*>(g.bias);
        const int rows_here = min(Cfg::BM, g.m - m0);
        const uint32_t row_bytes = (uint32_t)g.n * 2u;
        const __amdgpu_buffer_rsrc_t rout =
            make_rsrc(static_cast<uint16_t*>(g.out) + (size_t)m0 * g.n, (uint32_t)rows_here * row_bytes);
        const int nwv = n0 + wave_n * 128;
        f32x4 sw4[8];
        u32x2 braw[8];
#pragma unroll
        for (int ni = 0; ni < 8; ++ni) {
            const int n = nwv + ni * 16 + lgrp * 4;
            sw4[ni] = f32x4{1.0f, 1.0f, 1.0f, 1.0f};
            braw[ni] = u32x2{0u, 0u};
            if (n < g.n) {
                if constexpr (ScaleKind == SCALE_ROWCOL) sw4[ni] = *reinterpret_cast<const f32x4*>(g.sb + n);
                if (bias) braw[ni] = *reinterpret_cast<const u32x2*>(bias + n);
            }
        }
        const int r4 = lane >> 4, c16 = lane & 15;
        const int nst = nwv + c16 * 8;
        const uint32_t lane_off = (nst < g.n)
            ? (uint32_t)(wave_m * 128 + r4) * row_bytes + (uint32_t)nst * 2u
            : kOutOfRange;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            uint8_t* const buf = mine + (p & 1) * PASS_BYTES;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int mi = 2 * p + h;
#pragma unroll
                for (int ni = 0; ni < 8; ++ni) {
                    const u32x2 raw = braw[ni];
                    const f32x4 b4 = {__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u),
                                      __uint_as_float(raw.y << 16), __uint_as_float(raw.y & 0xffff0000u)};
                    float v[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float f = acc[ni][mi][j];
                        if constexpr (ScaleKind == SCALE_TENSOR) {
                            v[j] = f * s_tensor + b4[j];
                        } else {
#pragma clang fp contract(off)
                            const float scaled = f * sx[mi] * sw4[ni][j];
                            v[j] = scaled + b4[j];
                        }
                    }
                    u32x2 pk;
                    pk.x = pack_bf16x2(v[0], v[1]);
                    pk.y = pack_bf16x2(v[2], v[3]);
                    *reinterpret_cast<u32x2*>(buf + (h * 16 + lrow) * ROWB + (ni * 16 + lgrp * 4) * 2) = pk;
                }
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const u32x4 v = *reinterpret_cast<const u32x4*>(buf + (i * 4 + r4) * ROWB + c16 * 16);
                if constexpr (!(KO & KO_STORES))
                    __builtin_amdgcn_raw_buffer_store_b128(
                        v, rout, lane_off + (uint32_t)(p * 32 + i * 4) * row_bytes, 0, 2);
            }
        }
    }
    PP_STAMP();
}

template <int Fmt, int ScaleKind>
inline void launch_wave128_q16(const GemmArgs& g, hipStream_t stream) {
    using Cfg = Wave128Cfg;
    const int tiles = ((g.m + Cfg::BM - 1) / Cfg::BM) * ((g.n + Cfg::BN - 1) / Cfg::BN);
    auto kern = gemm_wave128_q16_kernel<Fmt, ScaleKind>;
    static std::atomic<uint64_t> lds_allowed{0};
    allow_dynamic_lds(reinterpret_cast<const void*>(kern), Cfg::LDS_BYTES, lds_allowed);
    note_kernel("wave128_q16");
    kern<<<dim3((unsigned)tiles), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream>>>(g);
}

}  // namespace w8a8
