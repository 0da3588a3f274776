// Skinny int8 W8A8 kernels for decode shapes (M <= 128): bandwidth-bound, the
// weight matrix is streamed from HBM exactly once and the MFMA pipe is almost
// idle -- speed is set by bytes in flight and by how whole the memory requests
// are. The int32 partials of the waves that split K are summed through LDS
// (integer addition is associative, so the split keeps the accumulator
// bit-exact) and the first waves run the dequant epilogue.
//
//  * M = 1: gemv_int8_dot_kernel, one wave per four weight rows, whole 1 KiB row
//    pieces straight into registers and v_dot4 on the vector ALU -- no LDS, no
//    barrier, every wave of the launch resident and loading at once.
//  * 2 <= M <= 16: gemv_int8_lds_kernel, 16 rows per workgroup, weights through
//    LDS in 1 KiB row pieces, every load of the workgroup issued at once.
//  * 17 <= M <= 128: skinny_int8_kernel, up to 48 rows per workgroup so that the
//    activation block is pulled from L2 by as few workgroups as possible.
// Measured at N=11008, K=4096 (weights from HBM): M=1 10.4 us, M=2..16 11.0-13.4,
// M=32 16.6, M=64 21.2 (the tiled GEMM kernel needs 29 us for any M <= 128).
#include "gemm_tile.cuh"

namespace w8a8 {

namespace {

// Single-token kernel (M = 1). A workgroup is one wave and owns R = 4 weight
// rows; lane l holds bytes [16 l, 16 l + 16) of every 1 KiB K-step of its rows and
// of the token, so each load instruction moves one whole 1 KiB row piece (the
// request pattern HBM and the address coalescer like best) and the matching
// activation bytes sit in the same lane. The dot products run on the vector ALU
// (v_dot4_i32_i8, exact int32), which frees the kernel of LDS, barriers and
// operand shuffles: a wave needs ~60 registers, so the ~2750 waves of an
// 11008-row matrix are all resident at once and the whole matrix is requested in
// the first microsecond. Lane partials are summed across the wave at the end
// (integer addition: the split over lanes keeps the accumulator bit-exact). The
// vector ALU's dot4 rate carries one token comfortably, not several: from two
// tokens on the MFMA kernel below is faster.
__global__ __launch_bounds__(64) void gemv_int8_dot_kernel(GemmArgs g) {
    constexpr int R = 4;
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

    int acc[R] = {0, 0, 0, 0};
#pragma unroll 2
    for (int k0 = 0; k0 < K; k0 += 1024) {
        const bool in = k0 + lane * 16 < K;
        u32x4 wv[R];
#pragma unroll
        for (int r = 0; r < R; ++r) wv[r] = buf_load16(rw, in ? w_off[r] : kOutOfRange, (uint32_t)k0);
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

// Variant that streams the weights through LDS: every load instruction moves
// 1 KiB of ONE weight row (64 lanes x 16 contiguous bytes) straight into LDS, so
// HBM, L2 and the address coalescer all see whole 128-byte lines in order; the
// MFMA operands (16 rows x 16 bytes per K-group) are then cut out of LDS, where
// the strided access is free. A workgroup of four waves owns 16 weight rows, wave
// w takes the 1 KiB K-steps w, w+4, ...; rows are laid down 1040 bytes apart so
// that the 16 rows of an operand read fall in distinct banks.
constexpr int kLdsRow = 1040;

template <int MB>
__global__ __launch_bounds__(256) void gemv_int8_lds_kernel(GemmArgs g) {
    __shared__ __attribute__((aligned(16))) uint8_t wbuf[4][16 * kLdsRow];
    __shared__ i32x4 red[4][MB][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lrow = lane & 15, lgrp = lane >> 4;
    const int K = g.k;
    const int nsteps = (K + 1023) >> 10;
    const int n0 = blockIdx.x * 16;

    const __amdgpu_buffer_rsrc_t rw = make_rsrc(g.b, (uint32_t)g.n * (uint32_t)K);
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(g.a, (uint32_t)g.m * (uint32_t)K);

    // epilogue operands first: their latency hides under the weight stream
    const int en = n0 + lgrp * 4;
    f32x4 sw4 = {0.0f, 0.0f, 0.0f, 0.0f};
    float sxv[MB];
    if (g.out_kind != OUT_ACC && wave < MB) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (en + j < g.n) sw4[j] = g.sb[en + j];
    }
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        const int m = b * 16 + lrow;
        sxv[b] = (g.out_kind != OUT_ACC && m < g.m) ? g.sa[m] : 0.0f;
    }

    i32x4 acc[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[b] = i32x4{0, 0, 0, 0};
    uint8_t* const mine = wbuf[wave];

    for (int s = wave; s < nsteps; s += 4) {
        const uint32_t k0 = (uint32_t)s << 10;
        // weights: 16 rows x 1 KiB, one instruction per row
        const bool k_in = (int)(k0 + lane * 16) < K;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t off = (uint32_t)(n0 + r) * (uint32_t)K + lane * 16;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                rw, (__attribute__((address_space(3))) void*)(mine + r * kLdsRow), 16,
                k_in ? off : kOutOfRange, k0, 0, 0);
        }
        // activations: MFMA layout straight from L2 (they are a few KiB, shared by
        // every workgroup)
        u32x4 xf[MB][16];
#pragma unroll
        for (int b = 0; b < MB; ++b) {
            const uint32_t xo = (uint32_t)(b * 16 + lrow) * (uint32_t)K + lgrp * 16;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const bool in = (int)(k0 + j * 64 + lgrp * 16) < K;
                xf[b][j] = buf_load16(rx, in ? xo + j * 64 : kOutOfRange, k0);
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the wave's own rows are in LDS
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const u32x4 wf = *reinterpret_cast<const u32x4*>(mine + lrow * kLdsRow + j * 64 + lgrp * 16);
#pragma unroll
            for (int b = 0; b < MB; ++b)
                acc[b] = __builtin_amdgcn_mfma_i32_16x16x64_i8((i32x4)wf, (i32x4)xf[b][j], acc[b], 0, 0, 0);
        }
    }

#pragma unroll
    for (int b = 0; b < MB; ++b) red[wave][b][lane] = acc[b];
    __syncthreads();
    if (wave < MB) {
        const int b = wave;
        const i32x4 sum = red[0][b][lane] + red[1][b][lane] + red[2][b][lane] + red[3][b][lane];
        const int m = b * 16 + lrow;
        if (m < g.m && en < g.n) {
            const size_t o = (size_t)m * g.n + en;
            if (g.out_kind == OUT_ACC) {
                int* out = static_cast<int*>(g.out);
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (en + j < g.n) out[o + j] = sum[j];
            } else {
                const uint16_t* bias = static_cast<const uint16_t*>(g.bias);
                float sx = 0.0f;
#pragma unroll
                for (int bb = 0; bb < MB; ++bb)
                    if (bb == b) sx = sxv[bb];
                float v[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float f = (float)sum[j] * sx * sw4[j];
                    if (bias && en + j < g.n) f += bf16_to_f32(bias[en + j]);
                    v[j] = f;
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
    }
}

void launch_dot(const GemmArgs& g, hipStream_t stream) {
    const int blocks = (g.n + 3) / 4;
    gemv_int8_dot_kernel<<<dim3((unsigned)blocks), dim3(64), 0, stream>>>(g);
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
void launch_skinny_rope_mb(const GemmArgs& g, const RopeCacheArgs& rc, hipStream_t stream) {
    switch ((g.m + 15) / 16) {
        case 1: launch_skinny<RG, 1, NW, true>(g, stream, rc); break;
        case 2: launch_skinny<RG, 2, NW, true>(g, stream, rc); break;
        case 3: launch_skinny<RG, 3, NW, true>(g, stream, rc); break;
        default: launch_skinny<RG, 4, NW, true>(g, stream, rc); break;
    }
}

template <int RG, int NW>
void launch_skinny_mb(const GemmArgs& g, hipStream_t stream) {
    switch ((g.m + 15) / 16) {
        case 1: launch_skinny<RG, 1, NW>(g, stream); break;
        case 2: launch_skinny<RG, 2, NW>(g, stream); break;
        case 3: launch_skinny<RG, 3, NW>(g, stream); break;
        case 4: launch_skinny<RG, 4, NW>(g, stream); break;
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

template <int MB>
void launch_lds(const GemmArgs& g, hipStream_t stream) {
    const int blocks = (g.n + 15) / 16;
    gemv_int8_lds_kernel<MB><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(g);
}

}  // namespace

bool launch_gemm_int8_rope_cache(const GemmArgs& g, const RopeCacheArgs& rc, hipStream_t stream) {
    if (g.m <= 0 || g.m > 64 || g.n <= 0 || g.k <= 0 || (g.k & 255) != 0 || (g.n & 3) != 0) return false;
    if (g.out_kind != OUT_BF16 || g.bias != nullptr || (rc.head_dim & 3) != 0) return false;
    if (g.m != rc.batch * rc.seq || g.n != (rc.n_heads + 2 * rc.n_kv_heads) * rc.head_dim) return false;
    if ((int64_t)g.n * g.k >= ((int64_t)1 << 31)) return false;
    // the same workgroup shapes as the plain skinny launch
    const int nsteps = (g.k + 511) >> 9;
    if ((g.n + 47) / 48 >= 192) launch_skinny_rope_mb<3, 4>(g, rc, stream);
    else if ((g.n + 31) / 32 >= 192) launch_skinny_rope_mb<2, 4>(g, rc, stream);
    else if (nsteps <= 4 || (g.n + 15) / 16 >= 512) launch_skinny_rope_mb<1, 4>(g, rc, stream);
    else if (nsteps <= 8) launch_skinny_rope_mb<1, 8>(g, rc, stream);
    else launch_skinny_rope_mb<1, 16>(g, rc, stream);
    return true;
}

bool launch_gemv_int8(const GemmArgs& g, hipStream_t stream) {
    if (g.m <= 0 || g.m > 128 || g.n <= 0 || g.k <= 0 || (g.k & 255) != 0) return false;
    const int64_t lim = (int64_t)1 << 31;
    if ((int64_t)g.n * g.k >= lim) return false;
    if (g.m == 1)
        launch_dot(g, stream);
    else if (g.m <= 16)
        launch_lds<1>(g, stream);
    else
        launch_skinny_auto(g, stream);
    return true;
}

}  // namespace w8a8
