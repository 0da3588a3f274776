// Skinny int8 W8A8 kernels for decode shapes (M <= 64): bandwidth-bound, the
// weight matrix is streamed from HBM exactly once and the MFMA pipe is almost
// idle -- speed is set by bytes in flight and by how whole the memory requests
// are. The int32 partials of the waves that split K are summed through LDS
// (integer addition is associative, so the split keeps the accumulator
// bit-exact) and the first waves run the dequant epilogue.
//
//  * M = 1: gemv_int8_dot_kernel, one wave per four weight rows, whole 1 KiB row
//    pieces straight into registers and v_dot4 on the vector ALU -- no LDS, no
//    barrier, every wave of the launch resident and loading at once.
//  * 1 < M <= 32: gemv_int8_lds_kernel streams the weights through LDS with 1 KiB
//    contiguous row pieces per instruction (see the comment on the kernel).
//  * 32 < M <= 64: gemv_int8_kernel loads MFMA-shaped operands straight into
//    registers (64 contiguous bytes of 16 rows per instruction).
#include "gemm_tile.cuh"

namespace w8a8 {

namespace {

template <int RG, int MB, int NW>
__global__ __launch_bounds__(NW * 64) void gemv_int8_kernel(GemmArgs g) {
    __shared__ i32x4 red[NW][RG * MB][64];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int lrow = lane & 15, lgrp = lane >> 4;
    const int K = g.k;
    const int nchunks = K >> 8;
    const int n0 = blockIdx.x * (RG * 16);

    const __amdgpu_buffer_rsrc_t rw = make_rsrc(g.b, (uint32_t)g.n * (uint32_t)K);
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(g.a, (uint32_t)g.m * (uint32_t)K);

    // Lane (row r, K-group q) takes bytes [64j + 16q, +16) of each 256-byte chunk
    // for j = 0..3: one instruction touches 64 contiguous bytes of each of its 16
    // rows, two instructions a whole 128-byte line. Rows past N / M read as zero
    // (their offset is past the buffer's num_records).
    uint32_t w_off[RG], x_off[MB];
#pragma unroll
    for (int r = 0; r < RG; ++r)
        w_off[r] = (uint32_t)(n0 + r * 16 + lrow) * (uint32_t)K + lgrp * 16;
#pragma unroll
    for (int b = 0; b < MB; ++b) x_off[b] = (uint32_t)(b * 16 + lrow) * (uint32_t)K + lgrp * 16;

    i32x4 acc[RG][MB];
#pragma unroll
    for (int r = 0; r < RG; ++r)
#pragma unroll
        for (int b = 0; b < MB; ++b) acc[r][b] = i32x4{0, 0, 0, 0};

    for (int c = wave; c < nchunks; c += NW) {
        const uint32_t k0 = (uint32_t)c << 8;
        u32x4 wf[RG][4], xf[MB][4];
#pragma unroll
        for (int r = 0; r < RG; ++r)
#pragma unroll
            for (int j = 0; j < 4; ++j) wf[r][j] = buf_load16(rw, w_off[r] + j * 64, k0);
#pragma unroll
        for (int b = 0; b < MB; ++b)
#pragma unroll
            for (int j = 0; j < 4; ++j) xf[b][j] = buf_load16(rx, x_off[b] + j * 64, k0);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < RG; ++r)
#pragma unroll
                for (int b = 0; b < MB; ++b)
                    acc[r][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(
                        (i32x4)wf[r][j], (i32x4)xf[b][j], acc[r][b], 0, 0, 0);
    }

#pragma unroll
    for (int r = 0; r < RG; ++r)
#pragma unroll
        for (int b = 0; b < MB; ++b) red[wave][r * MB + b][lane] = acc[r][b];
    __syncthreads();

    const EpilogueScalars es = load_epilogue_scalars<SCALE_ROWCOL>(g);
    for (int t = wave; t < RG * MB; t += NW) {
        i32x4 sum = red[0][t][lane];
#pragma unroll
        for (int w = 1; w < NW; ++w) sum += red[w][t][lane];
        const int r = t / MB, b = t % MB;
        store_subtile<OpI8, SCALE_ROWCOL>(g, es, sum, b * 16 + lrow, n0 + r * 16 + lgrp * 4);
    }
}

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

template <int MB>
void launch_lds(const GemmArgs& g, hipStream_t stream) {
    const int blocks = (g.n + 15) / 16;
    gemv_int8_lds_kernel<MB><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(g);
}

template <int RG, int MB, int NW>
void launch(const GemmArgs& g, hipStream_t stream) {
    const int blocks = (g.n + RG * 16 - 1) / (RG * 16);
    gemv_int8_kernel<RG, MB, NW><<<dim3((unsigned)blocks), dim3(NW * 64), 0, stream>>>(g);
}

template <int RG, int MB>
void launch_nw(const GemmArgs& g, hipStream_t stream) {
    if ((g.k >> 8) >= 16)
        launch<RG, MB, 16>(g, stream);
    else
        launch<RG, MB, 4>(g, stream);
}

}  // namespace

bool launch_gemv_int8(const GemmArgs& g, hipStream_t stream) {
    if (g.m <= 0 || g.m > 64 || g.n <= 0 || g.k <= 0 || (g.k & 255) != 0) return false;
    const int64_t lim = (int64_t)1 << 31;
    if ((int64_t)g.n * g.k >= lim) return false;
    if (g.m == 1) {
        launch_dot(g, stream);
        return true;
    }
    const int mb = (g.m + 15) / 16;
    switch (mb) {
        case 1: launch_lds<1>(g, stream); break;
        case 2: launch_lds<2>(g, stream); break;
        case 3: launch_nw<1, 3>(g, stream); break;
        default: launch_nw<1, 4>(g, stream); break;
    }
    return true;
}

}  // namespace w8a8
