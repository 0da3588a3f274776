// One-wave probes of the MFMA instructions the kernels are built on, for known-answer
// tests of the lane layouts (the analogue of the reference's single-instruction test,
// csrc/tests/fp8_mma_test.cu:81-145). A probe loads the two operands the way the kernels'
// wrappers expect them -- lane l supplies row l % R of its operand and the K bytes of
// K-group l / R -- issues ONE instruction on a zero accumulator and stores every lane's
// accumulator registers as they are: d_raw[lane][reg]. The test computes A * B^T on the
// host and places it by the layout the kernels assume:
//   16-row shapes: register j of lane l is D[4 * (l / 16) + j][l % 16]
//   32-row shapes: register r of lane l is D[8 * (r / 4) + 4 * (l / 32) + r % 4][l % 32]
// (D rows follow the first operand's rows, columns the second's). A wrong row mapping, a
// transposed result or K bytes of the two operands that do not meet each other all fail.
#include "gemm_pingpong.cuh"

namespace w8a8 {

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

// operands are row-major [R][KB] bytes; a lane's chunk c is 16 bytes at K offset koff(c)
template <int KIND>
__global__ __launch_bounds__(64) void mfma_probe_kernel(const uint8_t* a, const uint8_t* b, uint32_t* d) {
    const int lane = threadIdx.x;
    auto chunk = [&](const uint8_t* p, int row, int kb, int koff) {
        return *reinterpret_cast<const u32x4*>(p + row * kb + koff);
    };
    if constexpr (KIND == 0) {  // v_mfma_i32_16x16x64_i8, operands [16][64]
        const int r = lane & 15, g = lane >> 4;
        i32x4 c = {0, 0, 0, 0};
        c = __builtin_amdgcn_mfma_i32_16x16x64_i8((i32x4)chunk(a, r, 64, 16 * g), (i32x4)chunk(b, r, 64, 16 * g), c, 0, 0, 0);
        for (int j = 0; j < 4; ++j) d[lane * 4 + j] = (uint32_t)c[j];
    } else if constexpr (KIND == 1 || KIND == 2) {  // v_mfma_f32_16x16x128_f8f6f4 through OpF8, [16][128]
        const int r = lane & 15, g = lane >> 4;
        f32x4 c = {0.0f, 0.0f, 0.0f, 0.0f};
        c = OpF8<KIND - 1>::mma(chunk(a, r, 128, 16 * g), chunk(a, r, 128, 64 + 16 * g),
                                chunk(b, r, 128, 16 * g), chunk(b, r, 128, 64 + 16 * g), c);
        for (int j = 0; j < 4; ++j) d[lane * 4 + j] = __float_as_uint(c[j]);
    } else if constexpr (KIND == 3) {  // v_mfma_i32_32x32x32_i8 through Op32I8, [32][32]
        const int r = lane & 31, g = lane >> 5;
        Op32I8::Acc c;
        for (int j = 0; j < 16; ++j) c[j] = 0;
        const u32x4 w[2] = {chunk(a, r, 32, 16 * g), chunk(a, r, 32, 16 * g)};
        const u32x4 x[2] = {chunk(b, r, 32, 16 * g), chunk(b, r, 32, 16 * g)};
        c = Op32I8::mma_half(0, w, x, c);
        for (int j = 0; j < 16; ++j) d[lane * 16 + j] = (uint32_t)c[j];
    } else if constexpr (KIND == 4 || KIND == 5) {  // v_mfma_f32_32x32x64_f8f6f4 through Op32F8, [32][64]
        const int r = lane & 31, g = lane >> 5;
        typename Op32F8<KIND - 4>::Acc c;
        for (int j = 0; j < 16; ++j) c[j] = 0.0f;
        const u32x4 w[2] = {chunk(a, r, 64, 32 * g), chunk(a, r, 64, 32 * g + 16)};
        const u32x4 x[2] = {chunk(b, r, 64, 32 * g), chunk(b, r, 64, 32 * g + 16)};
        c = Op32F8<KIND - 4>::mma_half(0, w, x, c);
        for (int j = 0; j < 16; ++j) d[lane * 16 + j] = __float_as_uint(c[j]);
    } else if constexpr (KIND == 6) {  // v_mfma_f32_16x16x32_bf16, operands [16][32] bf16
        const int r = lane & 15, g = lane >> 4;
        f32x4 c = {0.0f, 0.0f, 0.0f, 0.0f};
        c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, chunk(a, r, 64, 16 * g)),
                                                    __builtin_bit_cast(bf16x8_t, chunk(b, r, 64, 16 * g)), c, 0, 0, 0);
        for (int j = 0; j < 4; ++j) d[lane * 4 + j] = __float_as_uint(c[j]);
    } else {  // v_mfma_f32_32x32x16_bf16, operands [32][16] bf16
        const int r = lane & 31, g = lane >> 5;
        f32x16 c;
        for (int j = 0; j < 16; ++j) c[j] = 0.0f;
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, chunk(a, r, 32, 16 * g)),
                                                    __builtin_bit_cast(bf16x8_t, chunk(b, r, 32, 16 * g)), c, 0, 0, 0);
        for (int j = 0; j < 16; ++j) d[lane * 16 + j] = __float_as_uint(c[j]);
    }
}

}  // namespace

bool launch_mfma_probe(int kind, const void* a, const void* b, void* d_raw, hipStream_t stream) {
    const uint8_t* pa = static_cast<const uint8_t*>(a);
    const uint8_t* pb = static_cast<const uint8_t*>(b);
    uint32_t* pd = static_cast<uint32_t*>(d_raw);
    switch (kind) {
        case 0: mfma_probe_kernel<0><<<1, 64, 0, stream>>>(pa, pb, pd); break;
        case 1: mfma_probe_kernel<1><<<1, 64, 0, stream>>>(pa, pb, pd); break;
        case 2: mfma_probe_kernel<2><<<1, 64, 0, stream>>>(pa, pb, pd); break;
        case 3: mfma_probe_kernel<3><<<1, 64, 0, stream>>>(pa, pb, pd); break;
        case 4: mfma_probe_kernel<4><<<1, 64, 0, stream>>>(pa, pb, pd); break;
        case 5: mfma_probe_kernel<5><<<1, 64, 0, stream>>>(pa, pb, pd); break;
        case 6: mfma_probe_kernel<6><<<1, 64, 0, stream>>>(pa, pb, pd); break;
        case 7: mfma_probe_kernel<7><<<1, 64, 0, stream>>>(pa, pb, pd); break;
        default: return false;
    }
    return true;
}

}  // namespace w8a8
