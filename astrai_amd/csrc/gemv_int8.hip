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
//  * 2 <= M <= 64: gemv_int8_rows_kernel (gemv_rows.cuh), about one workgroup per
//    compute unit with an equal share of the rows, a rolling ring of loads per wave.
//  * 65 <= M <= 128: skinny_int8_kernel, up to 48 rows per workgroup, weights through
//    LDS by direct-to-LDS loads.
// Measured at N=11008, K=4096 (weights from HBM, graph replay): M=1 8.6 us, M=2..16
// 9.3-9.9, M=32 11.2, M=64 13.9.
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
    float e_sx = 0.0f, e_sw = 0.0f, e_b = 0.0f;
    if (writer && g.out_kind != OUT_ACC) {
        e_sx = g.sa[0];
        e_sw = g.sb[en];
        if (g.bias) e_b = bf16_to_f32(static_cast<const uint16_t*>(g.bias)[en]);
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
            static_cast<uint16_t*>(g.out)[en] = f32_to_bf16(scaled + e_b);
        }
    }
}

void launch_dot(const GemmArgs& g, hipStream_t stream) {
    // a short matrix has too few rows to fill the chip with two-row waves' small windows
    if (g.n < 4096)
        gemv_int8_dot_kernel<4><<<dim3((unsigned)((g.n + 3) / 4)), dim3(64), 0, stream>>>(g);
    else
        gemv_int8_dot_kernel<2><<<dim3((unsigned)((g.n + 1) / 2)), dim3(64), 0, stream>>>(g);
}

// Skinny kernel for 2 <= M <= 128 (batched decode). The weight matrix is streamed
// once; what limits such shapes besides HBM is how often the activation block
// X[M,K] is pulled from L2 again: every workgroup needs all of it. So a
// workgroup takes as many weight rows as still leaves ~200 workgroups (RG groups
// of 16 rows, RG = 1..3) and keeps all M tokens of its rows.
//   * Four waves split K in 512-byte steps (wave w takes steps w, w+4, ...): a
//     2048-wide K already keeps all four busy.
//   * Weights go straight to LDS, one instruction per 2 rows x 512 bytes (whole
//     lines, in order). Rows are 512 bytes apart; the lane that lands at 16-byte
//     position p of row r fetches logical chunk p ^ (r & 15), which makes the
//     16-rows-per-instruction operand reads conflict-free without padding.
//   * Activations come from L2 in MFMA layout, at most four token groups (64
//     tokens, 128 registers) at a time; with more tokens the weight operands are
//     cut out of LDS again for the next four groups.
//   * int32 partials of the four waves are summed through LDS (exact), then the
//     dequant epilogue.
//
// ROPE: the rows are the fused q|k|v projection of a decoder layer and the epilogue
// goes on where the separate rotary / cache-write kernel would start: the bf16-rounded
// value pairs of q and k are rotated (fp32 products and sums rounded one by one, one
// rounding to bf16 -- the arithmetic of rope_cache.hip on the same rounded inputs),
// q goes to [batch, heads, seq, head_dim], k and v into the cache at the tokens'
// positions. A lane's four consecutive columns are two rotation pairs of one head.
template <int RG, int MB, int NW, bool ROPE>
__global__ __launch_bounds__(NW * 64) void skinny_int8_kernel(GemmArgs g, RopeCacheArgs rc) {
    constexpr int R = RG * 16;
    constexpr int XB = MB < 4 ? MB : 4;
    constexpr int PASSES = (MB + XB - 1) / XB;
    constexpr int WAVE_BYTES = R * 512;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lrow = lane & 15, lgrp = lane >> 4;
    const int K = g.k;
    const int nsteps = (K + 511) >> 9;
    const int n0 = blockIdx.x * R;

    const __amdgpu_buffer_rsrc_t rw = make_rsrc(g.b, (uint32_t)g.n * (uint32_t)K);
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(g.a, (uint32_t)g.m * (uint32_t)K);

    i32x4 acc[RG][MB];
#pragma unroll
    for (int r = 0; r < RG; ++r)
#pragma unroll
        for (int b = 0; b < MB; ++b) acc[r][b] = i32x4{0, 0, 0, 0};

    // epilogue operands of the (row group, token group) tasks this wave will write,
    // requested now so that their latency hides under the weight stream
    constexpr int TASKS = (RG * MB + NW - 1) / NW;
    float e_sx[TASKS], e_sw[TASKS][4], e_b[TASKS][4];
#pragma unroll
    for (int ti = 0; ti < TASKS; ++ti) {
        const int t = wave + ti * NW;
        const int m = (t % MB) * 16 + lrow;
        const int en = n0 + (t / MB) * 16 + lgrp * 4;
        const bool live = t < RG * MB && g.out_kind != OUT_ACC;
        e_sx[ti] = (live && m < g.m) ? g.sa[m] : 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool in = live && en + j < g.n;
            e_sw[ti][j] = in ? g.sb[en + j] : 0.0f;
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
            const int en = n0 + (t / MB) * 16 + lgrp * 4;
            e_cs[ti] = f32x4{1.0f, 0.0f, 1.0f, 0.0f};
            e_pos[ti] = -1;
            if (t < RG * MB && m < g.m && en < g.n) {
                const int sq = m % rc.seq;
                const int d = en % rc.head_dim;
                e_pos[ti] = rc.positions[sq];
                if (en < (rc.n_heads + rc.n_kv_heads) * rc.head_dim)
                    e_cs[ti] = *reinterpret_cast<const f32x4*>(
                        rc.freqs + ((int64_t)sq * (rc.head_dim >> 1) + (d >> 1)) * 2);
            }
        }
    }

    uint8_t* const mine = smem + wave * WAVE_BYTES;
    // load plan: instruction i covers rows 2i, 2i+1; lane -> row 2i + (lane>>5),
    // position lane&31, logical chunk (lane&31) ^ ((2i + (lane>>5)) & 15)
    const int r2 = lane >> 5;
    const uint32_t w_row_off = (uint32_t)(n0 + r2) * (uint32_t)K;  // rows past N: past num_records, zeros
    const int cx = (lane & 31) ^ r2;
    // operand plan: lane (lrow, lgrp) of row group rg reads chunk 4j+lgrp of row 16rg+lrow
    const uint32_t x_row_off = (uint32_t)lrow * (uint32_t)K + lgrp * 16;

    for (int s = wave; s < nsteps; s += NW) {
        const uint32_t k0 = (uint32_t)s << 9;
#pragma unroll
        for (int i = 0; i < R / 2; ++i) {
            const int chunk = cx ^ ((2 * i) & 15);
            const bool in = (int)(k0 + chunk * 16) < K;
            const uint32_t off = w_row_off + (uint32_t)(2 * i) * (uint32_t)K + (uint32_t)chunk * 16;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                rw, (__attribute__((address_space(3))) void*)(mine + i * 1024), 16,
                in ? off : kOutOfRange, k0, 0, 0);
        }
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            u32x4 xf[XB][8];
#pragma unroll
            for (int b = 0; b < XB; ++b) {
                // tokens past M start past num_records: zeros
                const uint32_t xo = x_row_off + (uint32_t)((p * XB + b) * 16) * (uint32_t)K;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const bool in = (int)(k0 + j * 64 + lgrp * 16) < K;
                    xf[b][j] = (p * XB + b < MB) ? buf_load16(rx, in ? xo + j * 64 : kOutOfRange, k0)
                                                 : u32x4{0, 0, 0, 0};
                }
            }
            __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): own rows in LDS, activations in registers
#pragma unroll
            for (int j = 0; j < 8; ++j)
#pragma unroll
                for (int r = 0; r < RG; ++r) {
                    const u32x4 wf = *reinterpret_cast<const u32x4*>(
                        mine + (r * 16 + lrow) * 512 + (((4 * j + lgrp) ^ lrow) << 4));
#pragma unroll
                    for (int b = 0; b < XB; ++b)
                        if (p * XB + b < MB)
                            acc[r][p * XB + b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(
                                (i32x4)wf, (i32x4)xf[b][j], acc[r][p * XB + b], 0, 0, 0);
                }
        }
        __builtin_amdgcn_sched_barrier(0);  // the next step's loads overwrite what was just read
    }

    // sum the waves' partials through LDS (the staging space is free now)
    __syncthreads();
    i32x4* const red = reinterpret_cast<i32x4*>(smem);  // [NW][RG * MB][64]
#pragma unroll
    for (int r = 0; r < RG; ++r)
#pragma unroll
        for (int b = 0; b < MB; ++b) red[(wave * RG * MB + r * MB + b) * 64 + lane] = acc[r][b];
    __syncthreads();
#pragma unroll
    for (int ti = 0; ti < TASKS; ++ti) {
        const int t = wave + ti * NW;
        if (t >= RG * MB) break;
        i32x4 sum = red[t * 64 + lane];
#pragma unroll
        for (int w = 1; w < NW; ++w) sum += red[(w * RG * MB + t) * 64 + lane];
        const int r = t / MB, b = t % MB;
        const int m = b * 16 + lrow;
        const int en = n0 + r * 16 + lgrp * 4;
        if (m >= g.m || en >= g.n) continue;
        const size_t o = (size_t)m * g.n + en;
        if (g.out_kind == OUT_ACC) {
            int* out = static_cast<int*>(g.out);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (en + j < g.n) out[o + j] = sum[j];
            continue;
        }
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // product and bias add rounded separately (no fused multiply-add): the
            // int8 epilogue is specified as elementwise fp32 on the exact integer
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
            *reinterpret_cast<u32x2*>(out + o) = pk;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (en + j < g.n) out[o + j] = f32_to_bf16(v[j]);
        }
    }
}

template <int RG, int MB, int NW, bool ROPE = false>
void launch_skinny(const GemmArgs& g, hipStream_t stream, const RopeCacheArgs& rc = RopeCacheArgs{}) {
    constexpr int lds_bytes = NW * RG * 16 * 512;
    static_assert(MB <= 8, "the reduction re-uses the staging space: NW * RG * MB KiB must fit");
    static_assert(lds_bytes <= 160 * 1024, "staging space of all waves must fit in LDS");
    auto kern = skinny_int8_kernel<RG, MB, NW, ROPE>;
    static std::atomic<uint64_t> lds_allowed{0};
    allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_allowed);
    const int blocks = (g.n + RG * 16 - 1) / (RG * 16);
    kern<<<dim3((unsigned)blocks), dim3(NW * 64), lds_bytes, stream>>>(g, rc);
}

// the q|k|v projection with rotary and cache write in the epilogue: up to 64 tokens
template <int RG, int NW>
void launch_skinny_mb(const GemmArgs& g, hipStream_t stream) {
    switch ((g.m + 15) / 16) {
        case 5: launch_skinny<RG, 5, NW>(g, stream); break;
        case 6: launch_skinny<RG, 6, NW>(g, stream); break;
        case 7: launch_skinny<RG, 7, NW>(g, stream); break;
        default: launch_skinny<RG, 8, NW>(g, stream); break;
    }
}

// As many rows per workgroup as still leaves ~200 workgroups. A matrix too short
// for that (16-row workgroups, fewer of them than CUs) makes up for it with more
// waves per workgroup when K is long, so that every 512-byte K-step still has a
// wave of its own and all of the matrix is requested at once.
void launch_skinny_auto(const GemmArgs& g, hipStream_t stream) {
    const int nsteps = (g.k + 511) >> 9;
    if ((g.n + 47) / 48 >= 192) launch_skinny_mb<3, 4>(g, stream);
    else if ((g.n + 31) / 32 >= 192) launch_skinny_mb<2, 4>(g, stream);
    else if (nsteps <= 4 || (g.n + 15) / 16 >= 512) launch_skinny_mb<1, 4>(g, stream);
    else if (nsteps <= 8) launch_skinny_mb<1, 8>(g, stream);
    else launch_skinny_mb<1, 16>(g, stream);
}

// Rows kernel launch plan. The rows are dealt out over 256 x rounds workgroups, rounds
// being the smallest count that keeps a workgroup's range within 48 rows (three MFMA
// row groups); ranges are rounded up to four rows (one load instruction). Four waves
// split K; a short matrix with a long K (one row group, K >= 4096) takes eight so that
// enough bytes are in flight (2048 x 5632: 5.7 us against 6.6 at M = 16). Measured per
// shape against deeper rings (IB = 2..4), fewer / more waves and one workgroup per
// sixteen rows: this plan was the fastest or within 2% of it on every decoder shape.
struct RowsPlan { int rows_per_wg, rg, nw, blocks; };

RowsPlan plan_rows(const GemmArgs& g) {
    RowsPlan p;
    const int rounds = (g.n + 256 * 48 - 1) / (256 * 48);
    const int wgs = 256 * rounds;
    p.rows_per_wg = (((g.n + wgs - 1) / wgs) + 3) & ~3;
    p.rg = (p.rows_per_wg + 15) / 16;
    p.nw = (p.rg == 1 && g.k >= 4096) ? 8 : 4;
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
    kern<<<dim3((unsigned)p.blocks), dim3(NW * 64), lds_bytes, stream>>>(g, rc, p.rows_per_wg);
}

template <int RG, int NW, bool ROPE>
void launch_rows_mb(const GemmArgs& g, const RopeCacheArgs& rc, const RowsPlan& p, hipStream_t stream) {
    switch ((g.m + 15) / 16) {
        case 1: launch_rows_inst<RG, 1, NW, ROPE>(g, rc, p, stream); break;
        case 2: launch_rows_inst<RG, 2, NW, ROPE>(g, rc, p, stream); break;
        case 3: launch_rows_inst<RG, 3, NW, ROPE>(g, rc, p, stream); break;
        default: launch_rows_inst<RG, 4, NW, ROPE>(g, rc, p, stream); break;
    }
}

// M <= 64
template <bool ROPE>
void launch_rows(const GemmArgs& g, const RopeCacheArgs& rc, hipStream_t stream) {
    const RowsPlan p = plan_rows(g);
    if (p.rg == 3) launch_rows_mb<3, 4, ROPE>(g, rc, p, stream);
    else if (p.rg == 2) launch_rows_mb<2, 4, ROPE>(g, rc, p, stream);
    else if (p.nw == 8) launch_rows_mb<1, 8, ROPE>(g, rc, p, stream);
    else launch_rows_mb<1, 4, ROPE>(g, rc, p, stream);
}

}  // namespace

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
    if (g.m == 1)
        launch_dot(g, stream);
    else if (g.m <= 64)
        launch_rows<false>(g, RopeCacheArgs{}, stream);
    else
        launch_skinny_auto(g, stream);
    return true;
}

}  // namespace w8a8
