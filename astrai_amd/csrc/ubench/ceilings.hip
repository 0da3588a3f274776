// Measured ceilings of one MI355X for the three resources the W8A8 kernels are
// bound by, to read the kernels' roofline fractions against:
//   1. MFMA issue rate of the 8-bit instructions with register-resident operands,
//      once with all-zero and once with random operand bits (the chip is power
//      managed: with toggling operands the clock drops and so does the ceiling);
//   2. HBM read bandwidth for one 45 MB weight matrix per launch, rotating through
//      1 GiB so that neither L2 nor the 256 MB Infinity Cache can serve it;
//   3. L2 -> LDS streaming rate with the GEMM's sharing pattern (256 workgroups,
//      each pulling its 256+256 operand rows, 128 bytes per row per step).
// Build: make -C astrai_amd/csrc ubench     Run: astrai_amd/csrc/ubench/ceilings
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

#define CK(x)                                                                          \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);      \
            exit(1);                                                                   \
        }                                                                              \
    } while (0)

__device__ unsigned hash32(unsigned x) {
    x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
    return x;
}
// four e4m3 bytes: random sign and mantissa, exponent field in [4, 9] so that sums stay finite
__device__ unsigned random_fp8x4(unsigned seed, int random) {
    if (!random) return 0;
    const unsigned h = hash32(seed);
    unsigned r = 0;
    for (int i = 0; i < 4; ++i) {
        const unsigned b = (h >> (8 * i)) & 0xff;
        r |= ((b & 0x80) | ((4 + ((b >> 3) % 6)) << 3) | (b & 7)) << (8 * i);
    }
    return r;
}

// WHICH: 0 fp8 16x16x128, 1 fp8 32x32x64, 2 i8 32x32x32, 3 i8 16x16x64
template <int WHICH>
__global__ __launch_bounds__(256) void mfma_loop(int iters, float* out, unsigned long long* t,
                                                 int random) {
    i32x8 a[4], b[4];
    i32x4 a4[4], b4[4];
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 8; ++j) {
            a[i][j] = random_fp8x4(threadIdx.x * 131 + i * 17 + j + blockIdx.x * 7919, random);
            b[i][j] = random_fp8x4(threadIdx.x * 257 + i * 29 + j + 1000003, random);
        }
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j) {
            a4[i][j] = random ? (int)hash32(threadIdx.x * 131 + i * 17 + j) : 0;
            b4[i][j] = random ? (int)hash32(threadIdx.x * 257 + i * 29 + j + 99) : 0;
        }
    const unsigned long long w0 = wall_clock64(), c0 = clock64();
    float s = 0;
    if constexpr (WHICH == 0) {
        f32x4 c[8];
        for (int i = 0; i < 8; ++i) c[i] = f32x4{0, 0, 0, 0};
        for (int it = 0; it < iters; ++it)
#pragma unroll
            for (int i = 0; i < 8; ++i)
                c[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[i & 3], b[(i >> 1) & 3], c[i], 0, 0, 0, 0, 0, 0);
        for (int i = 0; i < 8; ++i) s += c[i][0];
    } else if constexpr (WHICH == 1) {
        f32x16 c[4];
        for (int i = 0; i < 4; ++i)
            for (int j = 0; j < 16; ++j) c[i][j] = 0;
        for (int it = 0; it < iters; ++it)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                c[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i], b[(i + 1) & 3], c[i], 0, 0, 0, 0, 0, 0);
        for (int i = 0; i < 4; ++i) s += c[i][0];
    } else if constexpr (WHICH == 2) {
        i32x16 c[4];
        for (int i = 0; i < 4; ++i)
            for (int j = 0; j < 16; ++j) c[i][j] = 0;
        for (int it = 0; it < iters; ++it)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                c[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a4[i], b4[(i + 1) & 3], c[i], 0, 0, 0);
        for (int i = 0; i < 4; ++i) s += c[i][0];
    } else {
        i32x4 c[8];
        for (int i = 0; i < 8; ++i) c[i] = i32x4{0, 0, 0, 0};
        for (int it = 0; it < iters; ++it)
#pragma unroll
            for (int i = 0; i < 8; ++i)
                c[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a4[i & 3], b4[(i >> 1) & 3], c[i], 0, 0, 0);
        for (int i = 0; i < 8; ++i) s += c[i][0];
    }
    const unsigned long long w1 = wall_clock64(), c1 = clock64();
    out[blockIdx.x * 256 + threadIdx.x] = s;
    if (threadIdx.x == 0) {
        t[blockIdx.x * 2] = w1 - w0;   // 100 MHz ticks
        t[blockIdx.x * 2 + 1] = c1 - c0;  // shader clocks
    }
}

template <int W>
void run_mfma(const char* name, double ops_per_iter, float* out, unsigned long long* t) {
    for (int random : {0, 1}) {
        const int iters = 100000, blocks_per_cu = 2;
        mfma_loop<W><<<256 * blocks_per_cu, 256>>>(iters, out, t, random);  // warm the clocks
        CK(hipDeviceSynchronize());
        hipEvent_t e0, e1;
        CK(hipEventCreate(&e0));
        CK(hipEventCreate(&e1));
        CK(hipEventRecord(e0));
        mfma_loop<W><<<256 * blocks_per_cu, 256>>>(iters, out, t, random);
        CK(hipEventRecord(e1));
        CK(hipEventSynchronize(e1));
        float ms;
        CK(hipEventElapsedTime(&ms, e0, e1));
        unsigned long long h[2];
        CK(hipMemcpy(h, t, 16, hipMemcpyDeviceToHost));
        printf("mfma %-16s operands %-6s: %6.0f Tops/s, shader clock %4.0f MHz\n", name,
               random ? "random" : "zeros", 256.0 * blocks_per_cu * 4 * iters * ops_per_iter / ms / 1e9,
               h[1] / (h[0] / 100.0));
    }
}

template <int LOADS>
__global__ __launch_bounds__(256) void hbm_read(const u32x4* __restrict__ p, size_t n16, unsigned* out) {
    const size_t base = (size_t)blockIdx.x * 256 * LOADS + threadIdx.x;
    u32x4 v[LOADS];
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
        const size_t i = base + (size_t)j * 256;
        v[j] = i < n16 ? p[i] : u32x4{0, 0, 0, 0};
    }
    u32x4 acc = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < LOADS; ++j) acc += v[j];
    const unsigned s = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (s == 0x12345678u) out[0] = s;
}

// workgroup b of 256: XCD b%8, 4 x 8 tile block per XCD, like the GEMM's tile map
__global__ __launch_bounds__(512) void l2_stream(const unsigned char* A, const unsigned char* B, int ld,
                                                 int ksteps, unsigned* out) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int b = blockIdx.x, pid = (b & 7) * 32 + (b >> 3);
    const int tm = (pid / 64) * 4 + pid % 4, tn = (pid % 64) / 4;
    const unsigned char* base = (wave < 4) ? A + (size_t)tm * 256 * ld : B + (size_t)tn * 256 * ld;
    __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, (unsigned)(256u * (unsigned)ld), 0x00020000);
    const unsigned off0 = (unsigned)(((wave & 3) * 64 + (lane >> 3)) * ld + (lane & 7) * 16);
    for (int k = 0; k < ksteps; ++k) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                r, (__attribute__((address_space(3))) void*)(lds + ((k & 1) * 65536) + (wave * 8 + i) * 1024),
                16, off0 + i * 8 * ld, (unsigned)k << 7, 0, 0);
        __builtin_amdgcn_s_waitcnt(0x0f70 | 8);  // at most one step in flight beyond this one
    }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    const unsigned s = ((unsigned*)lds)[threadIdx.x];
    if (s == 0x12345678u) out[0] = s;
}

// The GEMM epilogue's store pattern with nothing before it: workgroup b owns a 256 x 256 bf16 tile
// of a 4096 x 4096 matrix (tile map as above), each of its four waves a 128 x 128 quadrant, a store
// instruction = four rows x 256 bytes, 16 bytes a lane. AUX: the cache-policy bits of the store.
template <int AUX>
__global__ __launch_bounds__(256) void tile_write(unsigned short* out, int ld) {
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int b = blockIdx.x, pid = (b & 7) * 32 + (b >> 3);
    const int tm = (pid / 64) * 4 + pid % 4, tn = (pid % 64) / 4;
    const unsigned row_bytes = (unsigned)ld * 2u;
    __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(out + (size_t)tm * 256 * ld), 0, 256u * row_bytes, 0x00020000);
    const unsigned off = (unsigned)((wave & 1) * 128 + (lane >> 4)) * row_bytes +
                         (unsigned)(tn * 256 + (wave >> 1) * 128 + (lane & 15) * 8) * 2u;
    const u32x4 v = {(unsigned)lane, (unsigned)b, 3u, 4u};
#pragma unroll
    for (int i = 0; i < 32; ++i)
        __builtin_amdgcn_raw_buffer_store_b128(v, r, off + (unsigned)(i * 4) * row_bytes, 0, AUX);
}

template <class F>
float time_ms(F f, int iters) {
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    for (int i = 0; i < 3; ++i) f();
    CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0));
    for (int i = 0; i < iters; ++i) f();
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    return ms / iters;
}

int main() {
    float* out;
    unsigned long long* t;
    CK(hipMalloc(&out, 1 << 24));
    CK(hipMalloc(&t, 8192 * 16));
    run_mfma<1>("fp8 32x32x64", 4 * 2.0 * 32 * 32 * 64, out, t);
    run_mfma<0>("fp8 16x16x128", 8 * 2.0 * 16 * 16 * 128, out, t);
    run_mfma<2>("i8 32x32x32", 4 * 2.0 * 32 * 32 * 32, out, t);
    run_mfma<3>("i8 16x16x64", 8 * 2.0 * 16 * 16 * 64, out, t);

    const size_t big = (size_t)1 << 30;
    void* buf;
    CK(hipMalloc(&buf, big));
    CK(hipMemset(buf, 1, big));
    unsigned* o2 = (unsigned*)out;
    const size_t chunk = (size_t)11008 * 4096, n16 = chunk / 16;
    const int nchunk = (int)(big / chunk);
    int c = 0;
    float ms = time_ms([&] {
        hbm_read<8><<<(unsigned)((n16 + 256 * 8 - 1) / (256 * 8)), 256>>>(
            (const u32x4*)((char*)buf + (size_t)(c % nchunk) * chunk), n16, o2);
        ++c;
    }, 200);
    printf("hbm read, 45.1 MB per launch rotating through 1 GiB: %.2f us per launch, %.0f GB/s\n", ms * 1e3, chunk / ms / 1e6);
    ms = time_ms([&] { hbm_read<8><<<(unsigned)((big / 16 + 256 * 8 - 1) / (256 * 8)), 256>>>((const u32x4*)buf, big / 16, o2); }, 10);
    printf("hbm read, 1 GiB per launch: %.1f us, %.0f GB/s\n", ms * 1e3, big / ms / 1e6);
    ms = time_ms([&] { hbm_read<4><<<1, 256>>>((const u32x4*)buf, 1, o2); }, 500);
    printf("back-to-back launch of an empty kernel: %.2f us\n", ms * 1e3);

    {
        unsigned short* o16 = (unsigned short*)buf;
        const float gap = ms;
        ms = time_ms([&] { tile_write<0><<<256, 256>>>(o16, 4096); }, 500);
        const float ms_nt = time_ms([&] { tile_write<2><<<256, 256>>>(o16, 4096); }, 500);
        printf("GEMM epilogue store pattern alone (33.5 MB, 256 workgroups x 128 KiB): %.2f us per launch with default "
               "stores, %.2f us non-temporal (launch gap %.2f us included) -> %.1f / %.1f TB/s net of the gap\n",
               ms * 1e3, ms_nt * 1e3, gap * 1e3, 33.554432 / ((ms - gap) * 1e3), 33.554432 / ((ms_nt - gap) * 1e3));
    }

    CK(hipFuncSetAttribute((const void*)l2_stream, hipFuncAttributeMaxDynamicSharedMemorySize, 131072));
    const int ld = 4096, ksteps = 32;
    ms = time_ms([&] { l2_stream<<<256, 512, 131072>>>((const unsigned char*)buf, (const unsigned char*)buf + (size_t)4096 * ld, ld, ksteps, o2); }, 200);
    const double bytes = 256.0 * ksteps * 65536;
    printf("L2->LDS stream, GEMM pattern (4096^3, 256x256x128 tiles): %.1f us for 32 K-slabs, %.1f TB/s aggregate, %.1f B/clk/CU at 2.4 GHz\n",
           ms * 1e3, bytes / ms / 1e9, bytes / 256 / (ms * 1e-3 * 2.4e9));
    return 0;
}
