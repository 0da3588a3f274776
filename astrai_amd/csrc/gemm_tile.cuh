// Tiled 8-bit "NT" GEMM for gfx950: out[M,N] = epilogue(A[M,K] . B[N,K]^T).
//
// One workgroup computes a BM x BN output tile, stepping K in 128-byte slabs.
// Each slab of A and of B is staged in LDS (double buffered) as rows of eight
// 16-byte chunks; the chunk position is XOR-swizzled with the row so that the
// 16-byte-per-lane fragment reads of a wave hit distinct banks. HBM/L2 reads
// are buffer loads (zero past the end of the tensor, which handles ragged M
// and N), 128 contiguous bytes per 8 lanes.
//
// Waves are laid out WM x WN over the tile. The weight rows feed the MFMA's
// first operand and the activation rows the second, so an accumulator lane
// holds four consecutive n for one m: the epilogue scales, adds bias, rounds
// once and stores 8 bytes (4 bf16) per lane per sub-tile.
#pragma once

#include "common.cuh"
#include "launchers.h"

namespace w8a8 {

template <int BM_, int BN_, int WM_, int WN_>
struct TileCfg {
    static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_;
    static constexpr int BK = 128;  // bytes of K per slab
    static constexpr int THREADS = 64 * WM * WN;
    static constexpr int MI = BM / WM / 16;  // 16-row activation sub-tiles per wave
    static constexpr int NI = BN / WN / 16;  // 16-row weight sub-tiles per wave
    static constexpr int A_LOADS = BM * 8 / THREADS;  // 16-byte chunks per thread per slab
    static constexpr int B_LOADS = BN * 8 / THREADS;
    static constexpr int STAGE_BYTES = (BM + BN) * BK;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
    static_assert(BM % (WM * 16) == 0 && BN % (WN * 16) == 0, "wave tile");
    static_assert((BM * 8) % THREADS == 0 && (BN * 8) % THREADS == 0, "load split");
};

// byte offset of logical 16-byte chunk `c` of `row` inside a slab
__device__ __forceinline__ int lds_chunk_off(int row, int c) {
    const int sw = (row & 7) ^ ((row >> 3) & 1);
    return row * 128 + ((c ^ sw) << 4);
}

// ---------------------------------------------------------------------------
// Epilogue shared by the tiled and the generic kernel. A lane owns four
// consecutive n (n..n+3) of one row m. Order of operations follows the CPU
// kernel (astrai/extension/ops/fp8.py:118-121): ((acc * sa) * sb) [* out_scale],
// bias added in fp32 before the single rounding (csrc/kernels/fp8/gemm.cuh:405-435).
// ---------------------------------------------------------------------------
struct EpilogueScalars {
    float sa, sb, so;
};

template <int ScaleKind>
__device__ __forceinline__ EpilogueScalars load_epilogue_scalars(const GemmArgs& g) {
    EpilogueScalars e{1.0f, 1.0f, 1.0f};
    if (g.out_kind == OUT_ACC) return e;
    if constexpr (ScaleKind == SCALE_TENSOR) {
        e.sa = g.sa[0];
        e.sb = g.sb[0];
    }
    if (g.out_kind == OUT_E4M3) e.so = g.out_scale[0];
    return e;
}

template <class Op, int ScaleKind>
__device__ __forceinline__ void store_subtile(const GemmArgs& g, const EpilogueScalars& es,
                                              typename Op::Acc a, int m, int n) {
    if (m >= g.m || n >= g.n) return;
    const size_t o = (size_t)m * g.n + n;
    if (g.out_kind == OUT_ACC) {
        using S = typename Op::AccScalar;
        S* out = static_cast<S*>(g.out);
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (n + j < g.n) out[o + j] = a[j];
        return;
    }
    const uint16_t* bias = static_cast<const uint16_t*>(g.bias);
    float sx = 1.0f;
    if constexpr (ScaleKind == SCALE_ROWCOL) sx = g.sa[m];
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float f = (float)a[j];
        if constexpr (ScaleKind == SCALE_TENSOR) {
            f = f * (es.sa * es.sb);  // one combined output scale, as csrc/kernels/fp8/gemm.cuh:583
        } else if constexpr (ScaleKind == SCALE_ROWCOL) {
            const float sw = (n + j < g.n) ? g.sb[n + j] : 0.0f;
            f = f * sx * sw;
        }
        if (bias && n + j < g.n) f += bf16_to_f32(bias[n + j]);
        v[j] = f;
    }
    const bool n_vec = (g.n & 3) == 0;
    if (g.out_kind == OUT_E4M3) {
        uint8_t* out = static_cast<uint8_t*>(g.out);
        const uint32_t p = cvt_pk_fp8<0>(v[0] * es.so, v[1] * es.so) |
                           (cvt_pk_fp8<0>(v[2] * es.so, v[3] * es.so) << 16);
        if (n_vec) {
            *reinterpret_cast<uint32_t*>(out + o) = p;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (n + j < g.n) out[o + j] = (uint8_t)(p >> (8 * j));
        }
    } else {
        uint16_t* out = static_cast<uint16_t*>(g.out);
        if (n_vec) {
            u32x2 p;
            p.x = pack_bf16x2(v[0], v[1]);
            p.y = pack_bf16x2(v[2], v[3]);
            *reinterpret_cast<u32x2*>(out + o) = p;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (n + j < g.n) out[o + j] = f32_to_bf16(v[j]);
        }
    }
}

struct TileCoord {
    int tm, tn;
};

// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2). Give
// each XCD a contiguous run of tile ids, then walk tiles in groups of GROUP
// tile-rows so that the ~32 tiles resident on one XCD share A rows and B rows.
__device__ __forceinline__ TileCoord map_tile(int tiles_m, int tiles_n) {
    const int nwg = tiles_m * tiles_n;
    int pid = blockIdx.x;
    if ((nwg & 7) == 0) pid = (pid & 7) * (nwg >> 3) + (pid >> 3);
    constexpr int GROUP = 4;
    const int width = GROUP * tiles_n;
    const int group = pid / width;
    const int first_m = group * GROUP;
    const int gsz = min(tiles_m - first_m, GROUP);
    const int in_group = pid - group * width;
    TileCoord t;
    t.tm = first_m + in_group % gsz;
    t.tn = in_group / gsz;
    return t;
}

template <class Op, class Cfg, int ScaleKind>
__global__ __launch_bounds__(Cfg::THREADS) void gemm_tiled_kernel(GemmArgs g) {
    using Acc = typename Op::Acc;
    constexpr int BM = Cfg::BM, BN = Cfg::BN, MI = Cfg::MI, NI = Cfg::NI;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_m = wave % Cfg::WM;
    const int wave_n = wave / Cfg::WM;
    const int lrow = lane & 15;  // operand row inside a 16-row sub-tile
    const int lgrp = lane >> 4;  // K-group 0..3

    const int tiles_m = (g.m + BM - 1) / BM;
    const int tiles_n = (g.n + BN - 1) / BN;
    const TileCoord tc = map_tile(tiles_m, tiles_n);
    const int m0 = tc.tm * BM, n0 = tc.tn * BN;
    const int K = g.k;
    const int ksteps = (K + 127) >> 7;

    const __amdgpu_buffer_rsrc_t ra = make_rsrc(g.a, (uint32_t)g.m * (uint32_t)K);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(g.b, (uint32_t)g.n * (uint32_t)K);

    // per-thread chunk assignment: q = tid + i*THREADS -> row q>>3, chunk q&7
    const int ld_chunk = tid & 7;
    const int ld_row = tid >> 3;
    constexpr int ROWS_PER_PASS = Cfg::THREADS / 8;
    uint32_t a_off[Cfg::A_LOADS], b_off[Cfg::B_LOADS];
    int a_lds[Cfg::A_LOADS], b_lds[Cfg::B_LOADS];
#pragma unroll
    for (int i = 0; i < Cfg::A_LOADS; ++i) {
        const int r = ld_row + i * ROWS_PER_PASS;
        a_off[i] = (uint32_t)(m0 + r) * (uint32_t)K + ld_chunk * 16;
        if (m0 + r >= g.m) a_off[i] = kOutOfRange;
        a_lds[i] = lds_chunk_off(r, ld_chunk);
    }
#pragma unroll
    for (int i = 0; i < Cfg::B_LOADS; ++i) {
        const int r = ld_row + i * ROWS_PER_PASS;
        b_off[i] = (uint32_t)(n0 + r) * (uint32_t)K + ld_chunk * 16;
        if (n0 + r >= g.n) b_off[i] = kOutOfRange;
        b_lds[i] = BM * 128 + lds_chunk_off(r, ld_chunk);
    }
    const bool k_ragged = (K & 127) != 0;

    u32x4 a_reg[Cfg::A_LOADS], b_reg[Cfg::B_LOADS];

    auto global_load = [&](int kstep) {
        const uint32_t k0 = (uint32_t)kstep << 7;
        // chunks past K in the last slab must read as zero
        const bool dead = k_ragged && (int)(k0 + ld_chunk * 16) >= K;
#pragma unroll
        for (int i = 0; i < Cfg::A_LOADS; ++i)
            a_reg[i] = buf_load16(ra, dead ? kOutOfRange : a_off[i], k0);
#pragma unroll
        for (int i = 0; i < Cfg::B_LOADS; ++i)
            b_reg[i] = buf_load16(rb, dead ? kOutOfRange : b_off[i], k0);
    };
    auto lds_store = [&](int stage) {
        uint8_t* base = lds + stage * Cfg::STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < Cfg::A_LOADS; ++i)
            *reinterpret_cast<u32x4*>(base + a_lds[i]) = a_reg[i];
#pragma unroll
        for (int i = 0; i < Cfg::B_LOADS; ++i)
            *reinterpret_cast<u32x4*>(base + b_lds[i]) = b_reg[i];
    };

    Acc acc[NI][MI];
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) acc[ni][mi] = Acc{0, 0, 0, 0};

    // fragment read offsets (row part); chunk pair of this lane is (2*lgrp, 2*lgrp+1)
    int xa_off[MI][2], wb_off[NI][2];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
        const int r = wave_m * (MI * 16) + mi * 16 + lrow;
        xa_off[mi][0] = lds_chunk_off(r, 2 * lgrp);
        xa_off[mi][1] = lds_chunk_off(r, 2 * lgrp + 1);
    }
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
        const int r = wave_n * (NI * 16) + ni * 16 + lrow;
        wb_off[ni][0] = BM * 128 + lds_chunk_off(r, 2 * lgrp);
        wb_off[ni][1] = BM * 128 + lds_chunk_off(r, 2 * lgrp + 1);
    }

    // block-scale bookkeeping (ScaleKind == SCALE_BLOCK128): sa[m, kb] for this
    // lane's m of every sub-tile, sb[n/128, kb] for the wave's n range
    const int kblocks = K >> 7;

    global_load(0);
    lds_store(0);
    __syncthreads();

    for (int ks = 0; ks < ksteps; ++ks) {
        const int stage = ks & 1;
        const bool more = ks + 1 < ksteps;
        if (more) global_load(ks + 1);

        const uint8_t* base = lds + stage * Cfg::STAGE_BYTES;
        u32x4 wf[NI][2];
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
            wf[ni][0] = *reinterpret_cast<const u32x4*>(base + wb_off[ni][0]);
            wf[ni][1] = *reinterpret_cast<const u32x4*>(base + wb_off[ni][1]);
        }
        if constexpr (ScaleKind == SCALE_BLOCK128) {
            // wave n range lies inside one 128-row weight block (NI*16 <= 128)
            const int nb = (n0 + wave_n * (NI * 16)) >> 7;
            const float sbv = g.sb[(size_t)nb * kblocks + ks];
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
                const u32x4 x0 = *reinterpret_cast<const u32x4*>(base + xa_off[mi][0]);
                const u32x4 x1 = *reinterpret_cast<const u32x4*>(base + xa_off[mi][1]);
                const int m = m0 + wave_m * (MI * 16) + mi * 16 + lrow;
                const float sav = (m < g.m) ? g.sa[(size_t)m * kblocks + ks] : 0.0f;
                const float sc = sav * sbv;
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) {
                    const Acc part = Op::mma(wf[ni][0], wf[ni][1], x0, x1, Acc{0, 0, 0, 0});
                    acc[ni][mi] += part * sc;
                }
            }
        } else {
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
                const u32x4 x0 = *reinterpret_cast<const u32x4*>(base + xa_off[mi][0]);
                const u32x4 x1 = *reinterpret_cast<const u32x4*>(base + xa_off[mi][1]);
#pragma unroll
                for (int ni = 0; ni < NI; ++ni)
                    acc[ni][mi] = Op::mma(wf[ni][0], wf[ni][1], x0, x1, acc[ni][mi]);
            }
        }

        if (more) lds_store(stage ^ 1);
        __syncthreads();
    }

    // ---------------- epilogue ----------------
    const EpilogueScalars es = load_epilogue_scalars<ScaleKind>(g);
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
        const int m = m0 + wave_m * (MI * 16) + mi * 16 + lrow;
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
            const int n = n0 + wave_n * (NI * 16) + ni * 16 + lgrp * 4;
            store_subtile<Op, ScaleKind>(g, es, acc[ni][mi], m, n);
        }
    }
}

// Accepts the shape if the kernel's addressing assumptions hold.
inline bool tiled_shape_ok(const GemmArgs& g) {
    if (g.m <= 0 || g.n <= 0 || g.k <= 0) return false;
    if (g.k % 16 != 0) return false;
    const int64_t lim = (int64_t)1 << 31;  // byte offsets must stay below kOutOfRange
    return (int64_t)g.m * g.k < lim && (int64_t)g.n * g.k < lim;
}

template <class Op, class Cfg, int ScaleKind>
inline void launch_tiled(const GemmArgs& g, hipStream_t stream) {
    const int tiles = ((g.m + Cfg::BM - 1) / Cfg::BM) * ((g.n + Cfg::BN - 1) / Cfg::BN);
    auto kern = gemm_tiled_kernel<Op, Cfg, ScaleKind>;
    static std::atomic<uint64_t> lds_allowed{0};
    allow_dynamic_lds(reinterpret_cast<const void*>(kern), Cfg::LDS_BYTES, lds_allowed);
    note_kernel(Cfg::BM == 256 ? "tiled_256" : Cfg::BM == 128 ? "tiled_128" : "tiled_64");
    kern<<<dim3((unsigned)tiles), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream>>>(g);
}

// Tile selection: the large tile when it fills the chip, a smaller one otherwise.
using CfgBig = TileCfg<256, 256, 2, 4>;    // 8 waves, wave tile 128(m) x 64(n)
using CfgMid = TileCfg<128, 128, 2, 2>;    // 4 waves, wave tile 64 x 64
using CfgSmall = TileCfg<64, 64, 2, 2>;    // 4 waves, wave tile 32 x 32

template <class Op, int ScaleKind>
inline void launch_tiled_auto(const GemmArgs& g, hipStream_t stream) {
    auto tiles = [&](int bm, int bn) {
        return (int64_t)((g.m + bm - 1) / bm) * ((g.n + bn - 1) / bn);
    };
    if (tiles(256, 256) >= 192)
        launch_tiled<Op, CfgBig, ScaleKind>(g, stream);
    else if (tiles(128, 128) >= 192)
        launch_tiled<Op, CfgMid, ScaleKind>(g, stream);
    else
        launch_tiled<Op, CfgSmall, ScaleKind>(g, stream);
}

}  // namespace w8a8
