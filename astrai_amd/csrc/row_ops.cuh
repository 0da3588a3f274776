// Row-wise building blocks of the quantizing producers (RMSNorm / per-row int8), shared by the
// producer kernels and by the decode kernels that run a producer as their prologue: the same
// functions in both places, so both give the same bits.
#pragma once

#include "common.cuh"

namespace w8a8 {

constexpr int kRowThreads = 256;   // workgroup size the block-wide reductions below are written for

__device__ __forceinline__ void unpack8(u32x4 raw, float (&f)[8]) {
    f[0] = __uint_as_float(raw.x << 16);
    f[1] = __uint_as_float(raw.x & 0xffff0000u);
    f[2] = __uint_as_float(raw.y << 16);
    f[3] = __uint_as_float(raw.y & 0xffff0000u);
    f[4] = __uint_as_float(raw.z << 16);
    f[5] = __uint_as_float(raw.z & 0xffff0000u);
    f[6] = __uint_as_float(raw.w << 16);
    f[7] = __uint_as_float(raw.w & 0xffff0000u);
}

__device__ __forceinline__ float amax8(const float (&f)[8]) {
    float a = fmaxf(fabsf(f[0]), fabsf(f[1]));
    float b = fmaxf(fabsf(f[2]), fabsf(f[3]));
    float c = fmaxf(fabsf(f[4]), fabsf(f[5]));
    float d = fmaxf(fabsf(f[6]), fabsf(f[7]));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

// Eight codes, exactly rint(f / step) clamped to +-127, without eight IEEE divisions:
// t = f * (1 / step) is within two ulps of the quotient and |t| stays below 2^8 where a
// code can still change, so rint(t) can differ from rint(f / step) only when t lies within
// 2^-14 of a half-integer. Lanes that see such a value (about one vector in a thousand)
// redo their eight with the division.
__device__ __forceinline__ u32x2 quant8_int8(const float (&f)[8], float step) {
    const float inv = 1.0f / step;
    float r[8];
    bool risky = false;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float t = f[j] * inv;
        r[j] = rintf(t);
        risky |= fabsf(t - r[j]) > 0.5f - 0x1p-14f;
    }
    if (risky) {
#pragma unroll
        for (int j = 0; j < 8; ++j) r[j] = rintf(f[j] / step);
    }
    // an integer in [-127, 127] added to 1.5 * 2^23 leaves its two's-complement byte in the
    // low byte of the sum's bit pattern; byte permutes gather the eight low bytes
    uint32_t c[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
        c[j] = __float_as_uint(__builtin_amdgcn_fmed3f(r[j], -127.0f, 127.0f) + 12582912.0f);
    u32x2 o;
    o.x = __builtin_amdgcn_perm(__builtin_amdgcn_perm(c[3], c[2], 0x0c0c0400u),
                                __builtin_amdgcn_perm(c[1], c[0], 0x0c0c0400u), 0x05040100u);
    o.y = __builtin_amdgcn_perm(__builtin_amdgcn_perm(c[7], c[6], 0x0c0c0400u),
                                __builtin_amdgcn_perm(c[5], c[4], 0x0c0c0400u), 0x05040100u);
    return o;
}

// block-wide max of a per-thread value; result valid in every thread
__device__ __forceinline__ float block_max(float v, float* slots) {
    v = wave_max(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) slots[wave] = v;
    __syncthreads();
    float r = slots[0];
#pragma unroll
    for (int w = 1; w < kRowThreads / kWave; ++w) r = fmaxf(r, slots[w]);
    __syncthreads();
    return r;
}

// the same for a workgroup of T threads
template <int T>
__device__ __forceinline__ float block_max_t(float v, float* slots) {
    v = wave_max(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) slots[wave] = v;
    __syncthreads();
    float r = slots[0];
#pragma unroll
    for (int w = 1; w < T / kWave; ++w) r = fmaxf(r, slots[w]);
    __syncthreads();
    return r;
}

// block-wide sum of a per-thread value; result valid in every thread
__device__ __forceinline__ float block_sum(float v, float* slots) {
#pragma unroll
    for (int off = 32; off; off >>= 1) v += __shfl_xor(v, off, kWave);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) slots[wave] = v;
    __syncthreads();
    float r = slots[0];
#pragma unroll
    for (int w = 1; w < kRowThreads / kWave; ++w) r += slots[w];
    __syncthreads();
    return r;
}

__device__ __forceinline__ float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }

// eight values rounded to bf16 (one converter instruction per pair); returns them packed
__device__ __forceinline__ u32x4 round8_bf16(float (&f)[8]) {
    u32x4 o;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const uint32_t u = pack_bf16x2(f[2 * p], f[2 * p + 1]);
        f[2 * p] = __uint_as_float(u << 16);
        f[2 * p + 1] = __uint_as_float(u & 0xffff0000u);
        o[p] = u;
    }
    return o;
}

}  // namespace w8a8
