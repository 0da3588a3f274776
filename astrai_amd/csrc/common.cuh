// Shared device helpers for the gfx950 W8A8 kernels: vector types, MFMA
// wrappers, buffer-resource loads, bf16 / fp8 conversion, wave reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace w8a8 {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// ---------------------------------------------------------------------------
// Buffer resources: out-of-range reads return zero, which is how ragged M / N
// edges are handled without per-load predicates. Raw (stride 0) buffer,
// num_records in bytes; dword3 0x00020000 = 32-bit data format for gfx9.
// ---------------------------------------------------------------------------
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

__device__ __forceinline__ u32x4 buf_load16(__amdgpu_buffer_rsrc_t r, uint32_t voff,
                                            uint32_t soff) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0);
}

constexpr uint32_t kOutOfRange = 0x80000000u;  // any offset >= num_records reads as 0

// ---------------------------------------------------------------------------
// MFMA operators. Lane l of a wave supplies row (l & 15) of its operand and
// K-group (l >> 4); the accumulator lane holds D[4*(l>>4) + j][l & 15], j=0..3
// (D rows follow the first operand's rows). The K position of a byte inside a
// lane's registers is the same function of (K-group, byte) for both operands,
// so any consistent assignment of K bytes to lanes is a valid contraction.
// One "step" consumes 128 bytes of K per row: a lane holds two 16-byte chunks.
// ---------------------------------------------------------------------------
struct OpI8 {
    using Acc = i32x4;
    using AccScalar = int;
    static constexpr bool kIsInt = true;
    // two v_mfma_i32_16x16x64_i8 per 128-byte step
    static __device__ __forceinline__ Acc mma(u32x4 a0, u32x4 a1, u32x4 b0, u32x4 b1, Acc c) {
        c = __builtin_amdgcn_mfma_i32_16x16x64_i8((i32x4)a0, (i32x4)b0, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_i32_16x16x64_i8((i32x4)a1, (i32x4)b1, c, 0, 0, 0);
        return c;
    }
};

template <int Fmt>  // 0 = e4m3fn, 1 = e5m2
struct OpF8 {
    using Acc = f32x4;
    using AccScalar = float;
    static constexpr bool kIsInt = false;
    // one v_mfma_f32_16x16x128_f8f6f4 per 128-byte step (zero scale operands
    // select the unscaled instruction)
    static __device__ __forceinline__ Acc mma(u32x4 a0, u32x4 a1, u32x4 b0, u32x4 b1, Acc c) {
        i32x8 a = {(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w,
                   (int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
        i32x8 b = {(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w,
                   (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
        return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, Fmt, Fmt, 0, 0, 0, 0);
    }
};

// ---------------------------------------------------------------------------
// Scalar conversions
// ---------------------------------------------------------------------------
__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
    return __uint_as_float((uint32_t)h << 16);
}

// round-to-nearest-even fp32 -> bf16 on the hardware converter
// (v_cvt_pk_bf16_f32; NaN stays NaN)
typedef __bf16 bf16x2_hw __attribute__((ext_vector_type(2)));
typedef float f32x2_hw __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    const f32x2_hw v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_hw));
}

__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
    return (uint16_t)(pack_bf16x2(f, 0.0f) & 0xffffu);
}

// Saturating fp32 -> fp8 pair (low 16 bits of the result). The hardware
// converter rounds to nearest even; magnitudes are clamped to the finite max
// first (NaN passes through the clamp untouched and converts to NaN).
template <int Fmt>
__device__ __forceinline__ uint32_t cvt_pk_fp8(float a, float b) {
    constexpr float lim = Fmt ? 57344.0f : 448.0f;
    a = (a != a) ? a : fminf(fmaxf(a, -lim), lim);
    b = (b != b) ? b : fminf(fmaxf(b, -lim), lim);
    if constexpr (Fmt)
        return (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(a, b, 0, false) & 0xffffu;
    else
        return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xffffu;
}

// ---------------------------------------------------------------------------
// Wave / block reductions
// ---------------------------------------------------------------------------
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

__device__ __forceinline__ int wave_sum_i32(int v) {
#pragma unroll
    for (int off = 32; off; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// max into a non-negative float slot through its bit pattern
// (non-negative floats order like their bits). Device-scope atomics on one address
// are served one at a time, about 10 ns each, so a workgroup first looks at the slot
// and leaves it alone when its own maximum cannot raise it: thousands of workgroups
// would otherwise queue for tens of microseconds behind one another.
__device__ __forceinline__ void atomic_max_nonneg(float* dst, float v) {
    unsigned int* p = reinterpret_cast<unsigned int*>(dst);
    const unsigned int bits = __float_as_uint(v);
    if (__hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < bits) atomicMax(p, bits);
}

}  // namespace w8a8
