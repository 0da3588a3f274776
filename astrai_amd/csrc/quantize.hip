// bf16 -> fp8 / int8 quantization kernels for gfx950.
//
// All kernels are bandwidth-bound elementwise passes: 16-byte loads (8 bf16 per
// lane), the correctly rounded fp32 quotient by the step (the CPU kernel's arithmetic,
// astrai/extension/ops/fp8.py:80; formed without a division sequence per element where the
// step is shared, see quant8_fp8), hardware RNE conversion, 8-byte stores.
#include "common.cuh"
#include "launchers.h"
#include "row_ops.cuh"

namespace w8a8 {

namespace {

constexpr int kThreads = kRowThreads;

// Eight saturating fp8 codes of RN32(f / step), the oracle's arithmetic: an IEEE division per
// element and a NaN-preserving clamp.
template <int Fmt>
__device__ __forceinline__ u32x2 quant8_fp8_div(const float (&f)[8], float step) {
    u32x2 o;
    o.x = cvt_pk_fp8<Fmt>(f[0] / step, f[1] / step) |
          (cvt_pk_fp8<Fmt>(f[2] / step, f[3] / step) << 16);
    o.y = cvt_pk_fp8<Fmt>(f[4] / step, f[5] / step) |
          (cvt_pk_fp8<Fmt>(f[6] / step, f[7] / step) << 16);
    return o;
}

// The same eight codes without eight IEEE division sequences (a quantizer is otherwise bound by
// them: ~11 of its ~18 vector instructions per element). The step is shared by the tensor, so
// the correctly rounded reciprocal inv = RN(1 / step) is formed once, and per element
//   q0 = f * inv,  e0 = fma(-q0, step, f),  q1 = fma(e0, inv, q0)     (q1: RN of t + 2^-22 ulp,
//   e1 = fma(-q1, step, f),  q = fma(e1, inv, q1)                      a faithful quotient)
// is the correctly rounded quotient RN32(f / step): Markstein's theorem -- a faithful quotient
// corrected once with its exact remainder and the correctly rounded reciprocal rounds
// correctly, unless the divisor's significand is all ones. The remainders are exact unless they
// underflow, which needs |f| < 2^-102: a zero code for every step >= 2^-60. So steps outside
// [2^-60, 2^60] or with an all-ones significand take the division throughout, and so do lanes
// whose quotient is not finite (infinite or NaN inputs, products that overflow), which also
// keeps NaN out of the clamp below.
template <int Fmt>
__device__ __forceinline__ u32x2 quant8_fp8(const float (&f)[8], float step) {
    constexpr float lim = Fmt ? 57344.0f : 448.0f;
    const float inv = 1.0f / step;
    const bool step_ok = step >= 0x1p-60f && step <= 0x1p60f && (__float_as_uint(step) & 0x7fffffu) != 0x7fffffu;
    float q[8];
    bool finite = true;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float q0 = f[j] * inv;
        const float e0 = __builtin_fmaf(-q0, step, f[j]);
        const float q1 = __builtin_fmaf(e0, inv, q0);
        const float e1 = __builtin_fmaf(-q1, step, f[j]);
        // (a zero quotient takes the sign of f, as the division gives it: the corrections add
        // +0 to a -0; everywhere else the sign bit is already f's, the step being positive)
        q[j] = __uint_as_float(__float_as_uint(__builtin_fmaf(e1, inv, q1)) | (__float_as_uint(f[j]) & 0x80000000u));
        finite = finite && fabsf(q[j]) < __builtin_inff();
    }
    if (__builtin_expect(!step_ok || !finite, 0)) {
        // (the empty statement keeps this a branch: the compiler otherwise evaluates the
        // divisions for every lane and selects)
        asm volatile("");
        return quant8_fp8_div<Fmt>(f, step);
    }
    u32x2 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) q[j] = __builtin_amdgcn_fmed3f(q[j], -lim, lim);
    // (the converter writes the half of its destination word that the last operand names)
    if constexpr (Fmt) {
        o.x = (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(q[2], q[3], __builtin_amdgcn_cvt_pk_bf8_f32(q[0], q[1], 0, false), true);
        o.y = (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(q[6], q[7], __builtin_amdgcn_cvt_pk_bf8_f32(q[4], q[5], 0, false), true);
    } else {
        o.x = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], 0, false), true);
        o.y = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q[6], q[7], __builtin_amdgcn_cvt_pk_fp8_f32(q[4], q[5], 0, false), true);
    }
    return o;
}

__device__ __forceinline__ uint32_t quant1_int8(float f, float step) {
    float q = rintf(f / step);
    q = fminf(fmaxf(q, -127.0f), 127.0f);
    return (uint32_t)(int)q & 0xffu;
}

// ---- per-tensor fp8 -------------------------------------------------------
// Kernels that report a tensor-wide amax end in an atomic per workgroup on one
// address, and those are served one after the other (~10 ns each: thousands of
// workgroups finishing together queue for tens of microseconds). So one workgroup
// in kEarlyEvery publishes the maximum of its first group of vectors early -- a few
// dozen atomics that have drained long before the tensor has streamed -- and at the
// end a workgroup touches the slot only if its share has outgrown what the slot
// holds by then, which a few dozen out of a thousand do on unsorted data.
constexpr int kAmaxBlocks = kAmaxPartials;  // grid cap: the workgroups stride over the tensor
constexpr int kUnroll = 4;         // independent 16-byte loads in flight per thread
constexpr int kEarlyEvery = 16;

// The other way to report the maximum: every workgroup stores its own into slot blockIdx.x of
// a kAmaxBlocks-wide array (workgroup 0 zeroes the slots no workgroup owns) and the kernel
// that consumes the maximum -- the ring push, one wave -- reduces the array. No atomics, no
// slot to clear beforehand, nothing that waits at the end of the kernel: 3-4 us less than
// the atomic form on a 4096 x 4096 tensor, and the cleared slot's fill launch besides.
__device__ __forceinline__ void store_partial(float* partials, float local, float* slots) {
    const float m = block_max(local, slots);
    if (threadIdx.x == 0) partials[blockIdx.x] = m;
    if (blockIdx.x == 0)
        for (int i = gridDim.x + threadIdx.x; i < kAmaxBlocks; i += kThreads) partials[i] = 0.0f;
}

__device__ __forceinline__ void publish_early(float* amax, float local, float* slots) {
    const float m = block_max(local, slots);
    if (threadIdx.x == 0 && m > 0.0f)
        atomicMax(reinterpret_cast<unsigned int*>(amax), __float_as_uint(m));
}

template <int Fmt>
__global__ __launch_bounds__(kThreads) void quantize_fp8_kernel(
    const uint16_t* __restrict__ x, uint8_t* __restrict__ x8, const float* __restrict__ scale,
    float* __restrict__ amax, float* __restrict__ partials, int64_t total) {
    __shared__ float slots[kThreads / kWave];
    const float step = *scale;
    float local = 0.0f;
    const int64_t nvec = total >> 3;
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    int64_t v = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    auto group = [&](int64_t v0) {
        u32x4 raw[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) raw[u] = *reinterpret_cast<const u32x4*>(x + (v0 + u * stride) * 8);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            float f[8];
            unpack8(raw[u], f);
            local = fmaxf(local, amax8(f));
            // streamed out: the codes' next reader is another kernel, and leaving them out of this
            // kernel's cache footprint is worth 1.5-3 us at 4096 x 4096
            __builtin_nontemporal_store(quant8_fp8<Fmt>(f, step), reinterpret_cast<u32x2*>(x8 + (v0 + u * stride) * 8));
        }
    };
    if (v + (kUnroll - 1) * stride < nvec) {
        group(v);
        v += kUnroll * stride;
    }
    if (amax && !partials && gridDim.x >= 64 && blockIdx.x % kEarlyEvery == 0) publish_early(amax, local, slots);
    for (; v + (kUnroll - 1) * stride < nvec; v += kUnroll * stride) group(v);
    for (; v < nvec; v += stride) {
        float f[8];
        unpack8(*reinterpret_cast<const u32x4*>(x + v * 8), f);
        local = fmaxf(local, amax8(f));
        *reinterpret_cast<u32x2*>(x8 + v * 8) = quant8_fp8<Fmt>(f, step);
    }
    if (blockIdx.x == 0) {  // ragged tail (< 8 elements)
        const int64_t i = nvec * 8 + threadIdx.x;
        if (i < total) {
            const float f = bf16_to_f32(x[i]);
            local = fmaxf(local, fabsf(f));
            x8[i] = (uint8_t)cvt_pk_fp8<Fmt>(f / step, 0.0f);
        }
    }
    if (partials) {
        store_partial(partials, local, slots);
    } else if (amax) {
        const float m = block_max(local, slots);
        if (threadIdx.x == 0) atomic_max_nonneg(amax, m);
    }
}

// ---- max |x| alone ---------------------------------------------------------
// Dynamic scaling measures a tensor before it quantizes it
// (astrai/extension/fp8.py:289-292: t.abs().amax()); this is that reduction as one
// read of the tensor, without the intermediate |x| tensor.
__global__ __launch_bounds__(kThreads) void amax_bf16_kernel(
    const uint16_t* __restrict__ x, float* __restrict__ amax, float* __restrict__ partials, int64_t total) {
    __shared__ float slots[kThreads / kWave];
    float local = 0.0f;
    const int64_t nvec = total >> 3;
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    int64_t v = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    auto group = [&](int64_t v0) {
        u32x4 raw[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) raw[u] = *reinterpret_cast<const u32x4*>(x + (v0 + u * stride) * 8);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            float f[8];
            unpack8(raw[u], f);
            local = fmaxf(local, amax8(f));
        }
    };
    if (v + (kUnroll - 1) * stride < nvec) {
        group(v);
        v += kUnroll * stride;
    }
    if (amax && gridDim.x >= 64 && blockIdx.x % kEarlyEvery == 0) publish_early(amax, local, slots);
    for (; v + (kUnroll - 1) * stride < nvec; v += kUnroll * stride) group(v);
    for (; v < nvec; v += stride) {
        float f[8];
        unpack8(*reinterpret_cast<const u32x4*>(x + v * 8), f);
        local = fmaxf(local, amax8(f));
    }
    if (blockIdx.x == 0) {
        const int64_t i = nvec * 8 + threadIdx.x;
        if (i < total) local = fmaxf(local, fabsf(bf16_to_f32(x[i])));
    }
    if (partials) {
        store_partial(partials, local, slots);
        return;
    }
    const float m = block_max(local, slots);
    if (threadIdx.x == 0) atomic_max_nonneg(amax, m);
}

// ---- delayed scaling: record one amax, refresh the step -------------------
// hist[idx] = amax; *scale = max((max(hist) / fmax) / pow2_margin, 1e-12), the
// record-then-refresh of FP8TensorMeta (astrai/extension/fp8.py:147-173, formula
// :87-89) as one single-wave launch instead of six tiny ones.
// (amax may be the ring's own slot: dynamic scaling is a ring of length one)
// (partials: the fresh value is the maximum of a quantizer's kAmaxBlocks per-workgroup maxima
// instead of *amax; amax_out, when given, receives it)
__global__ __launch_bounds__(kWave) void amax_ring_push_kernel(
    float* hist, int n, int idx, const float* amax, const float* partials, float* amax_out,
    float* scale, float fmax, float pow2_margin) {
    float fresh;
    if (partials) {
        float m = 0.0f;
#pragma unroll
        for (int i = 0; i < kAmaxBlocks / kWave; ++i) m = fmaxf(m, partials[i * kWave + threadIdx.x]);
        fresh = wave_max(m);
        if (amax_out && threadIdx.x == 0) *amax_out = fresh;
    } else {
        fresh = *amax;
    }
    float peak = 0.0f;
    for (int i = threadIdx.x; i < n; i += kWave) {
        float h = hist[i];
        if (i == idx) hist[i] = h = fresh;
        peak = fmaxf(peak, h);
    }
    peak = wave_max(peak);
    if (threadIdx.x == 0) *scale = fmaxf((peak / fmax) / pow2_margin, 1e-12f);
}

// ---- per-tensor fp8, row-major and transposed codes in one pass -----------
// The backward of a Linear contracts the gradient over both of its axes
// (dX = g.w over N, dW = g^T.x over M; csrc/kernels/fp8/mm.cu:298-312 makes
// transposed-contiguous copies first). Here one read of a [R,C] bf16 matrix
// yields its codes row-major (optional) and transposed [C,R]. Tile 128 x 128:
// 256-byte runs in, 128-byte runs out in both layouts. A thread converts 4 rows
// x 8 columns per pass, packs the four rows of each column into a dword and
// writes it to a column-major LDS tile (pitch 132 bytes); the tile then leaves
// as 16-byte pieces of the transposed rows.
constexpr int kTrRows = 128, kTrCols = 128, kTrPitch = kTrRows + 4;

template <int Fmt>
__global__ __launch_bounds__(kThreads) void quantize_transpose_fp8_kernel(
    const uint16_t* __restrict__ x, uint8_t* __restrict__ x8, uint8_t* __restrict__ x8t,
    const float* __restrict__ scale, float* __restrict__ amax, int64_t rows, int64_t cols) {
    __shared__ __attribute__((aligned(16))) uint8_t tile[kTrCols * kTrPitch];
    __shared__ float slots[kThreads / kWave];
    const int cc = threadIdx.x & 15, r4 = threadIdx.x >> 4;
    const float step = *scale;
    const bool vec = (cols & 7) == 0;
    const bool runs = (rows & 15) == 0;  // 16-byte pieces stay aligned and inside the matrix
    const int64_t tiles_x = (cols + kTrCols - 1) / kTrCols;
    const int64_t ntiles = tiles_x * ((rows + kTrRows - 1) / kTrRows);
    float local = 0.0f;
    for (int64_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
        const int64_t r0 = (t / tiles_x) * kTrRows, c0 = (t % tiles_x) * kTrCols;
        const int64_t c = c0 + cc * 8;
        // all eight 16-byte pieces of the thread requested before the first is converted
        u32x4 raw[2][4];
        const bool col_in = vec && c < cols;
#pragma unroll
        for (int pass = 0; pass < 2; ++pass)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int64_t r = r0 + pass * 64 + r4 * 4 + i;
                raw[pass][i] = u32x4{0u, 0u, 0u, 0u};
                if (col_in && r < rows) raw[pass][i] = *reinterpret_cast<const u32x4*>(x + r * cols + c);
            }
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            u32x2 q[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int64_t r = r0 + pass * 64 + r4 * 4 + i;
                float f[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
                const bool whole = col_in && r < rows;
                if (whole) {
                    unpack8(raw[pass][i], f);
                } else if (r < rows) {
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (c + j < cols) f[j] = bf16_to_f32(x[r * cols + c + j]);
                }
                local = fmaxf(local, amax8(f));
                q[i] = quant8_fp8<Fmt>(f, step);
                if (x8) {
                    if (whole) {
                        __builtin_nontemporal_store(q[i], reinterpret_cast<u32x2*>(x8 + r * cols + c));
                    } else if (r < rows) {
#pragma unroll
                        for (int j = 0; j < 8; ++j)
                            if (c + j < cols)
                                x8[r * cols + c + j] =
                                    (uint8_t)(((j < 4 ? q[i].x : q[i].y) >> ((j & 3) * 8)) & 0xffu);
                    }
                }
            }
            // 4 rows x 8 columns of bytes -> 8 dwords of one column each: two 4 x 4 byte
            // transposes of two v_perm_b32 stages (byte selectors: 0-3 second source, 4-7 first)
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const uint32_t a0 = half ? q[0].y : q[0].x, a1 = half ? q[1].y : q[1].x;
                const uint32_t a2 = half ? q[2].y : q[2].x, a3 = half ? q[3].y : q[3].x;
                const uint32_t lo01 = __builtin_amdgcn_perm(a1, a0, 0x05010400u), hi01 = __builtin_amdgcn_perm(a1, a0, 0x07030602u);
                const uint32_t lo23 = __builtin_amdgcn_perm(a3, a2, 0x05010400u), hi23 = __builtin_amdgcn_perm(a3, a2, 0x07030602u);
                const uint32_t d[4] = {__builtin_amdgcn_perm(lo23, lo01, 0x05040100u), __builtin_amdgcn_perm(lo23, lo01, 0x07060302u),
                                       __builtin_amdgcn_perm(hi23, hi01, 0x05040100u), __builtin_amdgcn_perm(hi23, hi01, 0x07060302u)};
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    *reinterpret_cast<uint32_t*>(tile + (cc * 8 + half * 4 + j) * kTrPitch + pass * 64 + r4 * 4) = d[j];
            }
        }
        __syncthreads();
#pragma unroll
        for (int h = 0; h < 4; ++h) {
            const int cl = (threadIdx.x >> 3) + 32 * h;
            const int64_t ct = c0 + cl, rt = r0 + (threadIdx.x & 7) * 16;
            if (ct >= cols || rt >= rows) continue;
            const uint8_t* src = tile + cl * kTrPitch + (threadIdx.x & 7) * 16;
            u32x4 v;
            v.x = *reinterpret_cast<const uint32_t*>(src);
            v.y = *reinterpret_cast<const uint32_t*>(src + 4);
            v.z = *reinterpret_cast<const uint32_t*>(src + 8);
            v.w = *reinterpret_cast<const uint32_t*>(src + 12);
            if (runs) {
                __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(x8t + ct * rows + rt));
            } else {
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int b = 0; b < 16; ++b)
                    if (rt + b < rows)
                        x8t[ct * rows + rt + b] = (uint8_t)((w[b >> 2] >> ((b & 3) * 8)) & 0xffu);
            }
        }
        // the first tile's maximum goes out early when more tiles follow (block_max also
        // separates this tile's LDS reads from the next tile's writes)
        if (amax && t == blockIdx.x && t + gridDim.x < ntiles && gridDim.x >= 64 &&
            blockIdx.x % kEarlyEvery == 0)
            publish_early(amax, local, slots);
        else
            __syncthreads();
    }
    if (amax) {
        const float m = block_max(local, slots);
        if (threadIdx.x == 0) atomic_max_nonneg(amax, m);
    }
}

// ---- per-row int8 ---------------------------------------------------------
// One workgroup per row; up to kCache 16-byte vectors per thread stay in
// registers between the amax pass and the quantize pass (K <= 8192), longer
// rows are re-read (they hit L2).
constexpr int kCache = 4;

__global__ __launch_bounds__(kThreads) void quantize_int8_rows_kernel(
    const uint16_t* __restrict__ x, int8_t* __restrict__ xq, float* __restrict__ s, int64_t k) {
    __shared__ float slots[kThreads / kWave];
    const int64_t row = blockIdx.x;
    const uint16_t* xr = x + row * k;
    int8_t* qr = xq + row * k;
    const bool vec_ok = (k & 7) == 0;
    const int64_t nvec = vec_ok ? (k >> 3) : 0;
    u32x4 cache[kCache];
    float local = 0.0f;
#pragma unroll
    for (int c = 0; c < kCache; ++c) {
        const int64_t v = threadIdx.x + (int64_t)c * kThreads;
        if (v < nvec) {
            cache[c] = *reinterpret_cast<const u32x4*>(xr + v * 8);
            float f[8];
            unpack8(cache[c], f);
            local = fmaxf(local, amax8(f));
        }
    }
    for (int64_t v = threadIdx.x + (int64_t)kCache * kThreads; v < nvec; v += kThreads) {
        float f[8];
        unpack8(*reinterpret_cast<const u32x4*>(xr + v * 8), f);
        local = fmaxf(local, amax8(f));
    }
    for (int64_t i = nvec * 8 + threadIdx.x; i < k; i += kThreads)
        local = fmaxf(local, fabsf(bf16_to_f32(xr[i])));

    const float amax = fmaxf(block_max(local, slots), 1e-12f);
    const float step = amax / 127.0f;
    if (threadIdx.x == 0) s[row] = step;

#pragma unroll
    for (int c = 0; c < kCache; ++c) {
        const int64_t v = threadIdx.x + (int64_t)c * kThreads;
        if (v < nvec) {
            float f[8];
            unpack8(cache[c], f);
            *reinterpret_cast<u32x2*>(qr + v * 8) = quant8_int8(f, step);
        }
    }
    for (int64_t v = threadIdx.x + (int64_t)kCache * kThreads; v < nvec; v += kThreads) {
        float f[8];
        unpack8(*reinterpret_cast<const u32x4*>(xr + v * 8), f);
        *reinterpret_cast<u32x2*>(qr + v * 8) = quant8_int8(f, step);
    }
    for (int64_t i = nvec * 8 + threadIdx.x; i < k; i += kThreads)
        qr[i] = (int8_t)quant1_int8(bf16_to_f32(xr[i]), step);
}

// ---- producers fused with the per-row int8 quantizer -------------------------
// The activation of every int8 Linear in the decoder comes out of an RMSNorm
// (after a residual add) or out of the SwiGLU product. Fusing the per-token
// quantizer into those removes a write and a read of the bf16 activation and a
// launch per Linear. One workgroup per row, the row stays in registers
// (width <= kCache * kThreads * 8 = 8192, a multiple of 8).

__device__ __forceinline__ u32x4 pack8(const float (&f)[8]) {
    u32x4 o;
    o.x = pack_bf16x2(f[0], f[1]);
    o.y = pack_bf16x2(f[2], f[3]);
    o.z = pack_bf16x2(f[4], f[5]);
    o.w = pack_bf16x2(f[6], f[7]);
    return o;
}

// out = bf16(y + resid) (the plain-GEMM route of a projection whose output joins the
// residual stream, for shapes without a fused epilogue); out may be y
__global__ __launch_bounds__(kThreads) void add_bf16_kernel(
    const uint16_t* y, const uint16_t* __restrict__ resid, uint16_t* out, int64_t total) {
    const int64_t nvec = total >> 3;
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    const int64_t first = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    for (int64_t i = first; i < nvec; i += stride) {
        float a[8], b[8];
        unpack8(*reinterpret_cast<const u32x4*>(y + i * 8), a);
        unpack8(*reinterpret_cast<const u32x4*>(resid + i * 8), b);
#pragma unroll
        for (int j = 0; j < 8; ++j) a[j] += b[j];
        *reinterpret_cast<u32x4*>(out + i * 8) = pack8(a);
    }
    const int64_t t = nvec * 8 + first;   // the last total % 8 elements
    if (t < total) out[t] = f32_to_bf16(bf16_to_f32(y[t]) + bf16_to_f32(resid[t]));
}

// s = bf16(x + res) (when res is given; written to sum_out), y = bf16(w * (rstd * s))
// with rstd = rsqrt(mean(s^2) + eps) in fp32 -- one rounding, the arithmetic of
// F.rms_norm on a bf16 tensor (model/components/norm.py:7-15) -- then the per-row
// int8 quantizer on y.
__global__ __launch_bounds__(kThreads) void add_rmsnorm_quantize_int8_rows_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ res,
    const uint16_t* __restrict__ w, float eps, uint16_t* __restrict__ sum_out,
    uint16_t* __restrict__ y_out, int8_t* __restrict__ xq, float* __restrict__ s, int64_t k) {
    __shared__ float slots[kThreads / kWave];
    const int64_t row = blockIdx.x;
    const int64_t nvec = k >> 3;
    float v[kCache][8];
    // the norm weights are requested with the row, not after the reduction's barrier (a load does
    // not move across it by itself, and its latency would then sit in the middle of the chain)
    u32x4 wr[kCache];
#pragma unroll
    for (int c = 0; c < kCache; ++c) {
        const int64_t i = threadIdx.x + (int64_t)c * kThreads;
        wr[c] = i < nvec ? *reinterpret_cast<const u32x4*>(w + i * 8) : u32x4{0u, 0u, 0u, 0u};
    }
    float ss = 0.0f;
#pragma unroll
    for (int c = 0; c < kCache; ++c) {
        const int64_t i = threadIdx.x + (int64_t)c * kThreads;
        if (i < nvec) {
            unpack8(*reinterpret_cast<const u32x4*>(x + row * k + i * 8), v[c]);
            if (res) {
                float r[8];
                unpack8(*reinterpret_cast<const u32x4*>(res + row * k + i * 8), r);
#pragma unroll
                for (int j = 0; j < 8; ++j) v[c][j] = round_bf16(v[c][j] + r[j]);
                if (sum_out) *reinterpret_cast<u32x4*>(sum_out + row * k + i * 8) = pack8(v[c]);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) ss += v[c][j] * v[c][j];
        }
    }
    const float rstd = rsqrtf(block_sum(ss, slots) / (float)k + eps);
    float local = 0.0f;
#pragma unroll
    for (int c = 0; c < kCache; ++c) {
        const int64_t i = threadIdx.x + (int64_t)c * kThreads;
        if (i < nvec) {
            float g[8];
            unpack8(wr[c], g);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[c][j] = g[j] * (rstd * v[c][j]);
            const u32x4 packed = round8_bf16(v[c]);
            local = fmaxf(local, amax8(v[c]));
            if (y_out) *reinterpret_cast<u32x4*>(y_out + row * k + i * 8) = packed;
        }
    }
    const float step = fmaxf(block_max(local, slots), 1e-12f) / 127.0f;
    if (threadIdx.x == 0) s[row] = step;
#pragma unroll
    for (int c = 0; c < kCache; ++c) {
        const int64_t i = threadIdx.x + (int64_t)c * kThreads;
        if (i < nvec) *reinterpret_cast<u32x2*>(xq + row * k + i * 8) = quant8_int8(v[c], step);
    }
}

// The same two producers for many rows (a prefill block): one wave per row instead of one
// workgroup. A row of up to 4096 elements is KC 16-byte pieces per lane, the reductions are
// wave-wide shuffles with no workgroup barrier, and every wave walks over several rows with
// the next row's pieces requested before the current row is reduced -- with one workgroup
// per row and a barrier after each reduction the kernel is bound by the latency of its
// load -> reduce -> store chain (16,384 x 2048: 32 us for 100 MB), not by memory bandwidth.
// NORM: y = bf16(w * (rstd * x)), rstd = rsqrt(mean(x^2) + eps), then the per-row int8
// quantizer on y; otherwise the quantizer on x itself. The sum of squares is taken in the
// order of the one-workgroup-per-row kernel, so both kernels give a row the same bits.
template <int KC, bool NORM>
__global__ __launch_bounds__(kThreads) void wave_rows_int8_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, float eps,
    uint16_t* __restrict__ y_out, int8_t* __restrict__ xq, float* __restrict__ s, int64_t rows, int64_t k) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t nvec = k >> 3;
    const int64_t stride = (int64_t)gridDim.x * (kThreads / kWave);
    int64_t row = (int64_t)blockIdx.x * (kThreads / kWave) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const u32x4 zero = {0u, 0u, 0u, 0u};
    [[maybe_unused]] u32x4 wr[KC];
    if constexpr (NORM) {
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            const int64_t i = lane + (int64_t)c * kWave;
            wr[c] = i < nvec ? *reinterpret_cast<const u32x4*>(w + i * 8) : zero;
        }
    }
    u32x4 cur[KC], nxt[KC];
#pragma unroll
    for (int c = 0; c < KC; ++c) {
        const int64_t i = lane + (int64_t)c * kWave;
        cur[c] = i < nvec ? *reinterpret_cast<const u32x4*>(x + row * k + i * 8) : zero;
    }
    for (; row < rows; row += stride) {
        const int64_t nr = row + stride;
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            const int64_t i = lane + (int64_t)c * kWave;
            nxt[c] = (nr < rows && i < nvec) ? *reinterpret_cast<const u32x4*>(x + nr * k + i * 8) : zero;
        }
        float v[KC][8];
        float local = 0.0f;
        if constexpr (NORM) {
            // The sum of squares in the order of the one-workgroup-per-row kernel, so that a row's
            // rstd -- and with it y and every code -- does not depend on how many rows a launch
            // holds: there thread t = i mod 256 sums the pieces i = t, t + 256, ... as they come,
            // each of the four waves reduces its 64 threads by the same butterfly, and the four
            // results are added in wave order. Lane l holds the pieces of threads l, l + 64,
            // l + 128, l + 192: four running sums, four butterflies, the same three additions.
            float ssw[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                unpack8(cur[c], v[c]);
#pragma unroll
                for (int j = 0; j < 8; ++j) ssw[c & 3] += v[c][j] * v[c][j];
            }
#pragma unroll
            for (int wv = 0; wv < 4; ++wv)
#pragma unroll
                for (int off = 32; off; off >>= 1) ssw[wv] += __shfl_xor(ssw[wv], off, kWave);
            float ss = ssw[0];
#pragma unroll
            for (int wv = 1; wv < 4; ++wv) ss += ssw[wv];
            const float rstd = rsqrtf(ss / (float)k + eps);
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                float g[8];
                unpack8(wr[c], g);
#pragma unroll
                for (int j = 0; j < 8; ++j) v[c][j] = g[j] * (rstd * v[c][j]);
                const u32x4 packed = round8_bf16(v[c]);
                local = fmaxf(local, amax8(v[c]));
                const int64_t i = lane + (int64_t)c * kWave;
                if (y_out && i < nvec) *reinterpret_cast<u32x4*>(y_out + row * k + i * 8) = packed;
            }
        } else {
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                unpack8(cur[c], v[c]);
                local = fmaxf(local, amax8(v[c]));
            }
        }
        const float step = fmaxf(wave_max(local), 1e-12f) / 127.0f;
        if (lane == 0) s[row] = step;
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            const int64_t i = lane + (int64_t)c * kWave;
            // streaming store: the codes are read next by a GEMM, long after this block has left the caches
            if (i < nvec)
                __builtin_nontemporal_store(quant8_int8(v[c], step), reinterpret_cast<u32x2*>(xq + row * k + i * 8));
        }
#pragma unroll
        for (int c = 0; c < KC; ++c) cur[c] = nxt[c];
    }
}

constexpr int64_t kWaveRowsMin = 512;     // rows from which a wave per row is the faster plan
constexpr int64_t kWaveRowsMaxK = 4096;

inline bool wave_rows_fit(int64_t rows, int64_t k) {
    return rows >= kWaveRowsMin && k <= kWaveRowsMaxK && (k & 7) == 0;
}

template <bool NORM>
void launch_wave_rows(const uint16_t* x, const uint16_t* w, float eps, uint16_t* y_out, int8_t* xq,
                      float* s, int64_t rows, int64_t k, hipStream_t stream) {
    // The norm kernel keeps the norm weights in registers: four workgroups of four waves per compute
    // unit, each wave walking over its share of rows. The plain quantizer has nothing to keep and is
    // fastest with a wave per row (16,384 x 2048: 22.0 us against 25.1 us; the norm 22.7 against 25.0).
    const int64_t want = (rows + 3) / 4;
    const int64_t cap = NORM ? 1024 : 4096;
    const dim3 grid((unsigned)(want < cap ? want : cap)), block(kThreads);
    const int64_t pieces = (k / 8 + kWave - 1) / kWave;
    if (pieces <= 1) wave_rows_int8_kernel<1, NORM><<<grid, block, 0, stream>>>(x, w, eps, y_out, xq, s, rows, k);
    else if (pieces <= 2) wave_rows_int8_kernel<2, NORM><<<grid, block, 0, stream>>>(x, w, eps, y_out, xq, s, rows, k);
    else if (pieces <= 4) wave_rows_int8_kernel<4, NORM><<<grid, block, 0, stream>>>(x, w, eps, y_out, xq, s, rows, k);
    else wave_rows_int8_kernel<8, NORM><<<grid, block, 0, stream>>>(x, w, eps, y_out, xq, s, rows, k);
}

// silu(g) = g / (1 + exp(-g)) on the hardware's exp2 and reciprocal (each within one ulp
// in fp32, far inside the bf16 rounding that follows): the library expf and an IEEE division
// made this bandwidth kernel compute-bound.
__device__ __forceinline__ float silu_f32(float g) {
    return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.44269504088896340736f));
}

// h = bf16(up * bf16(silu(gate))), silu(g) = g / (1 + exp(-g)) in fp32: the bf16
// arithmetic of ``up(x) * F.silu(gate(x))`` (model/components/mlp.py:41); then the
// per-row int8 quantizer on h. gate and up rows are `ld` elements apart (they may
// be the two halves of one fused gate|up GEMM output). With block > 0 the columns of
// gate and of up come in pieces of `block` columns that lie 2 * block apart (a fused
// output whose columns alternate between `block` gate and `block` up columns, `up`
// pointing at the first up piece).
// T threads per row: 256 with up to four pieces a thread, or -- for the few rows of a decode step,
// where the row's chain of loads, exponentials and reductions is all there is to wait for -- 1024
// with one piece each (the maximum does not depend on who holds which piece: same bits).
template <int T>
__global__ __launch_bounds__(T) void silu_mul_quantize_int8_rows_kernel(
    const uint16_t* __restrict__ gate, const uint16_t* __restrict__ up, int64_t ld, int64_t block,
    uint16_t* __restrict__ h_out, int8_t* __restrict__ hq, float* __restrict__ s, int64_t width) {
    constexpr int kThreads = T;
    constexpr int kCache = w8a8::kCache * 256 / T;
    __shared__ float slots[kThreads / kWave];
    const int64_t row = blockIdx.x;
    const int64_t nvec = width >> 3;
    float v[kCache][8];
    float local = 0.0f;
#pragma unroll
    for (int c = 0; c < kCache; ++c) {
        const int64_t i = threadIdx.x + (int64_t)c * kThreads;
        if (i < nvec) {
            float g[8];
            const int64_t col = i * 8;
            const int64_t src = block ? (col / block) * (2 * block) + col % block : col;
            unpack8(*reinterpret_cast<const u32x4*>(gate + row * ld + src), g);
            unpack8(*reinterpret_cast<const u32x4*>(up + row * ld + src), v[c]);
#pragma unroll
            for (int j = 0; j < 8; ++j)
                v[c][j] = round_bf16(v[c][j] * round_bf16(silu_f32(g[j])));
            local = fmaxf(local, amax8(v[c]));
            if (h_out) *reinterpret_cast<u32x4*>(h_out + row * width + i * 8) = pack8(v[c]);
        }
    }
    const float step = fmaxf(block_max_t<T>(local, slots), 1e-12f) / 127.0f;
    if (threadIdx.x == 0) s[row] = step;
#pragma unroll
    for (int c = 0; c < kCache; ++c) {
        const int64_t i = threadIdx.x + (int64_t)c * kThreads;
        if (i < nvec) *reinterpret_cast<u32x2*>(hq + row * width + i * 8) = quant8_int8(v[c], step);
    }
}

// Per-tensor fp8 twins of the two producers above, for a Linear under delayed scaling: the
// step is known before the tensor exists (astrai/extension/fp8.py:147-173), so the codes
// are written in the pass that forms the values and the pass reports max |y| for the ring.
// Same value arithmetic as the int8 producers, the quantizer of quantize_fp8_kernel.
template <int Fmt>
__global__ __launch_bounds__(kThreads) void add_rmsnorm_quantize_fp8_rows_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ res,
    const uint16_t* __restrict__ w, float eps, uint16_t* __restrict__ sum_out,
    uint16_t* __restrict__ y_out, uint8_t* __restrict__ x8, const float* __restrict__ scale,
    float* __restrict__ amax, int64_t k) {
    __shared__ float slots[kThreads / kWave];
    const int64_t row = blockIdx.x;
    const int64_t nvec = k >> 3;
    const float step = *scale;
    float v[kCache][8];
    float ss = 0.0f;
#pragma unroll
    for (int c = 0; c < kCache; ++c) {
        const int64_t i = threadIdx.x + (int64_t)c * kThreads;
        if (i < nvec) {
            unpack8(*reinterpret_cast<const u32x4*>(x + row * k + i * 8), v[c]);
            if (res) {
                float r[8];
                unpack8(*reinterpret_cast<const u32x4*>(res + row * k + i * 8), r);
#pragma unroll
                for (int j = 0; j < 8; ++j) v[c][j] = round_bf16(v[c][j] + r[j]);
                if (sum_out) *reinterpret_cast<u32x4*>(sum_out + row * k + i * 8) = pack8(v[c]);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) ss += v[c][j] * v[c][j];
        }
    }
    const float rstd = rsqrtf(block_sum(ss, slots) / (float)k + eps);
    float local = 0.0f;
#pragma unroll
    for (int c = 0; c < kCache; ++c) {
        const int64_t i = threadIdx.x + (int64_t)c * kThreads;
        if (i < nvec) {
            float g[8];
            unpack8(*reinterpret_cast<const u32x4*>(w + i * 8), g);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[c][j] = round_bf16(g[j] * (rstd * v[c][j]));
            local = fmaxf(local, amax8(v[c]));
            if (y_out) *reinterpret_cast<u32x4*>(y_out + row * k + i * 8) = pack8(v[c]);
            *reinterpret_cast<u32x2*>(x8 + row * k + i * 8) = quant8_fp8<Fmt>(v[c], step);
        }
    }
    if (amax) {
        const float m = block_max(local, slots);
        if (threadIdx.x == 0) atomic_max_nonneg(amax, m);
    }
}

template <int Fmt>
__global__ __launch_bounds__(kThreads) void silu_mul_quantize_fp8_rows_kernel(
    const uint16_t* __restrict__ gate, const uint16_t* __restrict__ up, int64_t ld,
    uint16_t* __restrict__ h_out, uint8_t* __restrict__ h8, const float* __restrict__ scale,
    float* __restrict__ amax, int64_t width) {
    __shared__ float slots[kThreads / kWave];
    const int64_t row = blockIdx.x;
    const int64_t nvec = width >> 3;
    const float step = *scale;
    float local = 0.0f;
    for (int64_t i = threadIdx.x; i < nvec; i += kThreads) {
        float g[8], v[8];
        unpack8(*reinterpret_cast<const u32x4*>(gate + row * ld + i * 8), g);
        unpack8(*reinterpret_cast<const u32x4*>(up + row * ld + i * 8), v);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = round_bf16(v[j] * round_bf16(silu_f32(g[j])));
        local = fmaxf(local, amax8(v));
        if (h_out) *reinterpret_cast<u32x4*>(h_out + row * width + i * 8) = pack8(v);
        *reinterpret_cast<u32x2*>(h8 + row * width + i * 8) = quant8_fp8<Fmt>(v, step);
    }
    if (amax) {
        const float m = block_max(local, slots);
        if (threadIdx.x == 0) atomic_max_nonneg(amax, m);
    }
}

// Per-row int8 quantizer for rows whose maximum is already known in pieces: row_max holds
// `pieces` partial maxima of |h| per row (written by the SwiGLU epilogue of the gate|up
// GEMM), so the row is read once. Same codes and steps as quantize_int8_rows_kernel.
__global__ __launch_bounds__(kThreads) void quantize_int8_rows_pmax_kernel(
    const uint16_t* __restrict__ h, const float* __restrict__ row_max, int64_t pieces,
    int8_t* __restrict__ hq, float* __restrict__ s, int64_t width) {
    __shared__ float slots[kThreads / kWave];
    const int64_t row = blockIdx.x;
    const int64_t nvec = width >> 3;
    // the row's data is requested before the maxima are reduced
    u32x4 raw[kCache];
#pragma unroll
    for (int c = 0; c < kCache; ++c) {
        const int64_t i = threadIdx.x + (int64_t)c * kThreads;
        if (i < nvec) raw[c] = *reinterpret_cast<const u32x4*>(h + row * width + i * 8);
    }
    float local = 0.0f;
    for (int64_t i = threadIdx.x; i < pieces; i += kThreads) local = fmaxf(local, row_max[row * pieces + i]);
    const float step = fmaxf(block_max(local, slots), 1e-12f) / 127.0f;
    if (threadIdx.x == 0) s[row] = step;
#pragma unroll
    for (int c = 0; c < kCache; ++c) {
        const int64_t i = threadIdx.x + (int64_t)c * kThreads;
        if (i < nvec) {
            float v[8];
            unpack8(raw[c], v);
            *reinterpret_cast<u32x2*>(hq + row * width + i * 8) = quant8_int8(v, step);
        }
    }
}

// ---- 1x128 activation groups ----------------------------------------------
// One 16-byte vector per lane; 16 consecutive lanes own one 128-wide group.
__global__ __launch_bounds__(kThreads) void quantize_fp8_act128_kernel(
    const uint16_t* __restrict__ x, uint8_t* __restrict__ x8, float* __restrict__ sa,
    int64_t nvec) {
    const int64_t v = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    float f[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    const bool live = v < nvec;  // nvec is a multiple of 16, so groups are all-or-nothing
    if (live) unpack8(*reinterpret_cast<const u32x4*>(x + v * 8), f);
    float a = amax8(f);
#pragma unroll
    for (int off = 8; off; off >>= 1) a = fmaxf(a, __shfl_xor(a, off, kWave));
    const float step = fmaxf(a, 1e-12f) / 448.0f;
    if (live) {
        *reinterpret_cast<u32x2*>(x8 + v * 8) = quant8_fp8<0>(f, step);
        if ((threadIdx.x & 15) == 0) sa[v >> 4] = step;
    }
}

// ---- 128x128 weight blocks ------------------------------------------------
// One workgroup per block: 128 rows x 16 vectors = 2048 vectors, 8 per thread.
__global__ __launch_bounds__(kThreads) void quantize_fp8_weight128_kernel(
    const uint16_t* __restrict__ w, uint8_t* __restrict__ w8, float* __restrict__ sb, int64_t n,
    int64_t k) {
    __shared__ float slots[kThreads / kWave];
    const int64_t kb = blockIdx.x, nb = blockIdx.y;
    const int64_t kblocks = gridDim.x;
    u32x4 cache[8];
    float local = 0.0f;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int q = threadIdx.x + c * kThreads;  // 0..2047
        const int64_t row = nb * 128 + (q >> 4);
        const int64_t col = kb * 128 + (q & 15) * 8;
        if (row < n) {
            cache[c] = *reinterpret_cast<const u32x4*>(w + row * k + col);
            float f[8];
            unpack8(cache[c], f);
            local = fmaxf(local, amax8(f));
        }
    }
    const float step = fmaxf(block_max(local, slots), 1e-12f) / 448.0f;
    if (threadIdx.x == 0) sb[nb * kblocks + kb] = step;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int q = threadIdx.x + c * kThreads;
        const int64_t row = nb * 128 + (q >> 4);
        const int64_t col = kb * 128 + (q & 15) * 8;
        if (row < n) {
            float f[8];
            unpack8(cache[c], f);
            *reinterpret_cast<u32x2*>(w8 + row * k + col) = quant8_fp8<0>(f, step);
        }
    }
}

}  // namespace

void launch_quantize_fp8(const void* x, void* x8, const float* scale, float* amax, float* partials,
                         int64_t total, int fmt, hipStream_t stream) {
    if (total <= 0) return;
    const int64_t nvec = (total + 7) / 8;
    // two groups of kUnroll vectors per thread where the tensor is large enough
    int64_t blocks = (nvec + 2 * kUnroll * kThreads - 1) / (2 * kUnroll * kThreads);
    if (blocks > kAmaxBlocks) blocks = kAmaxBlocks;
    auto xs = static_cast<const uint16_t*>(x);
    auto xo = static_cast<uint8_t*>(x8);
    if (fmt)
        quantize_fp8_kernel<1><<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(
            xs, xo, scale, amax, partials, total);
    else
        quantize_fp8_kernel<0><<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(
            xs, xo, scale, amax, partials, total);
}

void launch_amax_ring_push(float* hist, int n, int idx, const float* amax, const float* partials,
                           float* amax_out, float* scale, float fmax, float pow2_margin,
                           hipStream_t stream) {
    amax_ring_push_kernel<<<dim3(1), dim3(kWave), 0, stream>>>(hist, n, idx, amax, partials, amax_out,
                                                               scale, fmax, pow2_margin);
}

void launch_amax_bf16(const void* x, float* amax, float* partials, int64_t total, hipStream_t stream) {
    if (total <= 0) return;
    int64_t blocks = ((total + 7) / 8 + 2 * kUnroll * kThreads - 1) / (2 * kUnroll * kThreads);
    if (blocks > kAmaxBlocks) blocks = kAmaxBlocks;
    amax_bf16_kernel<<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(
        static_cast<const uint16_t*>(x), amax, partials, total);
}

void launch_quantize_transpose_fp8(const void* x, void* x8, void* x8t, const float* scale,
                                   float* amax, int64_t rows, int64_t cols, int fmt,
                                   hipStream_t stream) {
    if (rows <= 0 || cols <= 0) return;
    // a workgroup per tile while they are all resident at once (eight per compute unit)
    const int64_t ntiles = ((cols + kTrCols - 1) / kTrCols) * ((rows + kTrRows - 1) / kTrRows);
    const dim3 grid((unsigned)(ntiles <= 2048 ? ntiles : 2048));
    auto* xi = static_cast<const uint16_t*>(x);
    auto* o = static_cast<uint8_t*>(x8);
    auto* ot = static_cast<uint8_t*>(x8t);
    if (fmt == 0)
        quantize_transpose_fp8_kernel<0><<<grid, dim3(kThreads), 0, stream>>>(xi, o, ot, scale, amax, rows, cols);
    else
        quantize_transpose_fp8_kernel<1><<<grid, dim3(kThreads), 0, stream>>>(xi, o, ot, scale, amax, rows, cols);
}

void launch_quantize_int8_rows(const void* x, void* xq, float* s, int64_t rows, int64_t k,
                               hipStream_t stream) {
    if (rows <= 0 || k <= 0) return;
    if (wave_rows_fit(rows, k)) {
        launch_wave_rows<false>(static_cast<const uint16_t*>(x), nullptr, 0.0f, nullptr,
                                static_cast<int8_t*>(xq), s, rows, k, stream);
        return;
    }
    quantize_int8_rows_kernel<<<dim3((unsigned)rows), dim3(kThreads), 0, stream>>>(
        static_cast<const uint16_t*>(x), static_cast<int8_t*>(xq), s, k);
}

void launch_add_bf16(const void* y, const void* resid, void* out, int64_t total, hipStream_t stream) {
    if (total <= 0) return;
    const int64_t want = ((total >> 3) + kThreads - 1) / kThreads;
    const int64_t blocks = want < 1 ? 1 : (want > 4096 ? 4096 : want);
    add_bf16_kernel<<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(
        static_cast<const uint16_t*>(y), static_cast<const uint16_t*>(resid), static_cast<uint16_t*>(out), total);
}

void launch_add_rmsnorm_quantize_int8_rows(const void* x, const void* res, const void* w, float eps,
                                           void* sum_out, void* y_out, void* xq, float* s,
                                           int64_t rows, int64_t k, hipStream_t stream) {
    if (rows <= 0 || k <= 0) return;
    if (!res && wave_rows_fit(rows, k)) {
        launch_wave_rows<true>(static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(w), eps,
                               static_cast<uint16_t*>(y_out), static_cast<int8_t*>(xq), s, rows, k, stream);
        return;
    }
    add_rmsnorm_quantize_int8_rows_kernel<<<dim3((unsigned)rows), dim3(kThreads), 0, stream>>>(
        static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(res),
        static_cast<const uint16_t*>(w), eps, static_cast<uint16_t*>(sum_out),
        static_cast<uint16_t*>(y_out), static_cast<int8_t*>(xq), s, k);
}

void launch_silu_mul_quantize_int8_rows(const void* gate, const void* up, int64_t ld, int64_t block,
                                        void* h_out, void* hq, float* s, int64_t rows, int64_t width,
                                        hipStream_t stream) {
    if (rows <= 0 || width <= 0) return;
    if (rows <= 64)
        silu_mul_quantize_int8_rows_kernel<1024><<<dim3((unsigned)rows), dim3(1024), 0, stream>>>(
            static_cast<const uint16_t*>(gate), static_cast<const uint16_t*>(up), ld, block,
            static_cast<uint16_t*>(h_out), static_cast<int8_t*>(hq), s, width);
    else
        silu_mul_quantize_int8_rows_kernel<256><<<dim3((unsigned)rows), dim3(256), 0, stream>>>(
            static_cast<const uint16_t*>(gate), static_cast<const uint16_t*>(up), ld, block,
            static_cast<uint16_t*>(h_out), static_cast<int8_t*>(hq), s, width);
}

void launch_add_rmsnorm_quantize_fp8_rows(const void* x, const void* res, const void* w, float eps,
                                          void* sum_out, void* y_out, void* x8, const float* scale,
                                          float* amax, int64_t rows, int64_t k, int fmt,
                                          hipStream_t stream) {
    if (rows <= 0 || k <= 0) return;
    auto kern = fmt ? add_rmsnorm_quantize_fp8_rows_kernel<1> : add_rmsnorm_quantize_fp8_rows_kernel<0>;
    kern<<<dim3((unsigned)rows), dim3(kThreads), 0, stream>>>(
        static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(res),
        static_cast<const uint16_t*>(w), eps, static_cast<uint16_t*>(sum_out),
        static_cast<uint16_t*>(y_out), static_cast<uint8_t*>(x8), scale, amax, k);
}

void launch_silu_mul_quantize_fp8_rows(const void* gate, const void* up, int64_t ld, void* h_out,
                                       void* h8, const float* scale, float* amax, int64_t rows,
                                       int64_t width, int fmt, hipStream_t stream) {
    if (rows <= 0 || width <= 0) return;
    auto kern = fmt ? silu_mul_quantize_fp8_rows_kernel<1> : silu_mul_quantize_fp8_rows_kernel<0>;
    kern<<<dim3((unsigned)rows), dim3(kThreads), 0, stream>>>(
        static_cast<const uint16_t*>(gate), static_cast<const uint16_t*>(up), ld,
        static_cast<uint16_t*>(h_out), static_cast<uint8_t*>(h8), scale, amax, width);
}

void launch_quantize_int8_rows_pmax(const void* h, const float* row_max, int64_t pieces, void* hq,
                                    float* s, int64_t rows, int64_t width, hipStream_t stream) {
    if (rows <= 0 || width <= 0) return;
    quantize_int8_rows_pmax_kernel<<<dim3((unsigned)rows), dim3(kThreads), 0, stream>>>(
        static_cast<const uint16_t*>(h), row_max, pieces, static_cast<int8_t*>(hq), s, width);
}

void launch_quantize_fp8_block128_act(const void* x, void* x8, float* sa, int64_t m,
                                      int64_t k, hipStream_t stream) {
    const int64_t nvec = m * k / 8;
    if (nvec <= 0) return;
    const int64_t blocks = (nvec + kThreads - 1) / kThreads;
    quantize_fp8_act128_kernel<<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(
        static_cast<const uint16_t*>(x), static_cast<uint8_t*>(x8), sa, nvec);
}

void launch_quantize_fp8_block128_weight(const void* w, void* w8, float* sb, int64_t n,
                                         int64_t k, hipStream_t stream) {
    if (n <= 0 || k <= 0) return;
    dim3 grid((unsigned)(k / 128), (unsigned)((n + 127) / 128));
    quantize_fp8_weight128_kernel<<<grid, dim3(kThreads), 0, stream>>>(
        static_cast<const uint16_t*>(w), static_cast<uint8_t*>(w8), sb, n, k);
}

}  // namespace w8a8
