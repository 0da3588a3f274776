// extern "C" entry points of libastrai_w8a8.so (declared in
// include/astrai_w8a8.h): argument validation, kernel selection, launch check.
// Nothing here allocates, frees or synchronises.
#include "../../include/astrai_w8a8.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>

#include "launchers.h"

namespace {

thread_local char g_err[256] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return fail(ASTRAI_W8A8_LAUNCH_FAILED, "%s: %s", what, hipGetErrorString(e));
    return ASTRAI_W8A8_OK;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int64_t kMaxDim = (int64_t)1 << 30;

int check_gemm(const char* what, const void* a, const void* b, const void* out, int64_t m,
               int64_t n, int64_t k) {
    if (!a || !b || !out) return fail(ASTRAI_W8A8_BAD_ARG, "%s: null operand pointer", what);
    if (m < 0 || n < 0 || k < 0 || m > kMaxDim || n > kMaxDim || k > kMaxDim)
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: bad dims m=%lld n=%lld k=%lld", what, (long long)m,
                    (long long)n, (long long)k);
    if (!aligned16(a) || !aligned16(b) || !aligned16(out))
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: operands must be 16-byte aligned", what);
    return ASTRAI_W8A8_OK;
}

w8a8::GemmArgs pack(const void* a, const void* b, const float* sa, const float* sb,
                    const float* out_scale, const void* bias, void* out, int64_t m, int64_t n,
                    int64_t k, int out_kind) {
    w8a8::GemmArgs g;
    g.a = a;
    g.b = b;
    g.sa = sa;
    g.sb = sb;
    g.out_scale = out_scale;
    g.bias = bias;
    g.out = out;
    g.m = (int)m;
    g.n = (int)n;
    g.k = (int)k;
    g.out_kind = out_kind;
    g.row_max = nullptr;
    return g;
}

// ---- library-owned scratch for the entry point that takes no workspace ----------
// Every GPU the library runs on holds its own copy of this array, at its own address,
// until the process ends. In host code the array's name is only a handle for
// hipGetSymbolAddress: what kernels and copies get is the address that call returns
// for the current device, looked up once per device and kept in scratch_addr.
constexpr int64_t kScratchFloats = ASTRAI_W8A8_STATIC_SCRATCH_FLOATS;
static __device__ __align__(256) float scratch[kScratchFloats];

constexpr int kMaxDevices = 64;
std::atomic<float*> scratch_addr[kMaxDevices];

int scratch_of_current_device(const char* what, float** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return fail(ASTRAI_W8A8_LAUNCH_FAILED, "%s: hipGetDevice: %s", what, hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices)
        return fail(ASTRAI_W8A8_UNSUPPORTED, "%s: device ordinal %d outside 0..%d", what, dev, kMaxDevices - 1);
    float* p = scratch_addr[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(ASTRAI_W8A8_LAUNCH_FAILED, "%s: hipGetSymbolAddress(scratch): %s", what,
                        hipGetErrorString(e));
        scratch_addr[dev].store(p, std::memory_order_release);  // two threads racing store the same address
    }
    *out = p;
    return ASTRAI_W8A8_OK;
}

}  // namespace

namespace w8a8 {
thread_local const char* g_last_kernel = "";
}

extern "C" {

int astrai_w8a8_abi_version(void) { return ASTRAI_W8A8_ABI_VERSION; }

const char* astrai_w8a8_last_error(void) { return g_err; }

const char* astrai_w8a8_last_kernel(void) { return w8a8::g_last_kernel; }

int astrai_w8a8_quantize_bf16_fp8(const void* x, void* x8, const float* scale, float* amax,
                                  int64_t total, int fmt, void* stream) {
    if (!x || !x8 || !scale) return fail(ASTRAI_W8A8_BAD_ARG, "quantize_bf16_fp8: null pointer");
    if (total < 0) return fail(ASTRAI_W8A8_BAD_ARG, "quantize_bf16_fp8: negative size");
    if (fmt != ASTRAI_W8A8_E4M3 && fmt != ASTRAI_W8A8_E5M2)
        return fail(ASTRAI_W8A8_BAD_ARG, "quantize_bf16_fp8: fmt must be 0 (e4m3) or 1 (e5m2)");
    if (!aligned16(x) || !aligned16(x8))
        return fail(ASTRAI_W8A8_BAD_ARG, "quantize_bf16_fp8: pointers must be 16-byte aligned");
    if (total == 0) return ASTRAI_W8A8_OK;
    w8a8::launch_quantize_fp8(x, x8, scale, amax, nullptr, total, fmt, static_cast<hipStream_t>(stream));
    return check_launch("quantize_bf16_fp8");
}

int astrai_w8a8_quantize_bf16_fp8_partials(const void* x, void* x8, const float* scale, float* partials,
                                           int64_t total, int fmt, void* stream) {
    if (!x || !x8 || !scale || !partials)
        return fail(ASTRAI_W8A8_BAD_ARG, "quantize_bf16_fp8_partials: null pointer");
    if (total <= 0) return fail(ASTRAI_W8A8_BAD_ARG, "quantize_bf16_fp8_partials: size must be positive");
    if (fmt != ASTRAI_W8A8_E4M3 && fmt != ASTRAI_W8A8_E5M2)
        return fail(ASTRAI_W8A8_BAD_ARG, "quantize_bf16_fp8_partials: fmt must be 0 (e4m3) or 1 (e5m2)");
    if (!aligned16(x) || !aligned16(x8))
        return fail(ASTRAI_W8A8_BAD_ARG, "quantize_bf16_fp8_partials: pointers must be 16-byte aligned");
    w8a8::launch_quantize_fp8(x, x8, scale, nullptr, partials, total, fmt, static_cast<hipStream_t>(stream));
    return check_launch("quantize_bf16_fp8_partials");
}

int astrai_w8a8_amax_bf16_partials(const void* x, float* partials, int64_t total, void* stream) {
    if (!x || !partials) return fail(ASTRAI_W8A8_BAD_ARG, "amax_bf16_partials: null pointer");
    if (total <= 0) return fail(ASTRAI_W8A8_BAD_ARG, "amax_bf16_partials: size must be positive");
    if (!aligned16(x)) return fail(ASTRAI_W8A8_BAD_ARG, "amax_bf16_partials: x must be 16-byte aligned");
    w8a8::launch_amax_bf16(x, nullptr, partials, total, static_cast<hipStream_t>(stream));
    return check_launch("amax_bf16_partials");
}

int astrai_w8a8_amax_ring_push_partials(float* hist, int n, int idx, const float* partials, float* amax_out,
                                        float* scale, float fmax, float pow2_margin, void* stream) {
    if (!hist || !partials || !scale)
        return fail(ASTRAI_W8A8_BAD_ARG, "amax_ring_push_partials: null pointer");
    if (n <= 0 || idx < 0 || idx >= n)
        return fail(ASTRAI_W8A8_BAD_ARG, "amax_ring_push_partials: idx must lie in [0, n)");
    if (!(fmax > 0.0f) || !(pow2_margin > 0.0f))
        return fail(ASTRAI_W8A8_BAD_ARG, "amax_ring_push_partials: fmax and pow2_margin must be positive");
    w8a8::launch_amax_ring_push(hist, n, idx, nullptr, partials, amax_out, scale, fmax, pow2_margin,
                                static_cast<hipStream_t>(stream));
    return check_launch("amax_ring_push_partials");
}

int astrai_w8a8_amax_bf16(const void* x, float* amax, int64_t total, void* stream) {
    if (!x || !amax) return fail(ASTRAI_W8A8_BAD_ARG, "amax_bf16: null pointer");
    if (total < 0) return fail(ASTRAI_W8A8_BAD_ARG, "amax_bf16: negative size");
    if (!aligned16(x)) return fail(ASTRAI_W8A8_BAD_ARG, "amax_bf16: x must be 16-byte aligned");
    if (total == 0) return ASTRAI_W8A8_OK;
    w8a8::launch_amax_bf16(x, amax, nullptr, total, static_cast<hipStream_t>(stream));
    return check_launch("amax_bf16");
}

int astrai_w8a8_amax_ring_push(float* hist, int n, int idx, const float* amax, float* scale,
                               float fmax, float pow2_margin, void* stream) {
    if (!hist || !amax || !scale) return fail(ASTRAI_W8A8_BAD_ARG, "amax_ring_push: null pointer");
    if (n <= 0 || idx < 0 || idx >= n)
        return fail(ASTRAI_W8A8_BAD_ARG, "amax_ring_push: idx must lie in [0, n)");
    if (!(fmax > 0.0f) || !(pow2_margin > 0.0f))
        return fail(ASTRAI_W8A8_BAD_ARG, "amax_ring_push: fmax and pow2_margin must be positive");
    w8a8::launch_amax_ring_push(hist, n, idx, amax, nullptr, nullptr, scale, fmax, pow2_margin,
                                static_cast<hipStream_t>(stream));
    return check_launch("amax_ring_push");
}

int astrai_w8a8_quantize_transpose_bf16_fp8(const void* x, void* x8, void* x8t, const float* scale,
                                            float* amax, int64_t rows, int64_t cols, int fmt,
                                            void* stream) {
    if (!x || !x8t || !scale)
        return fail(ASTRAI_W8A8_BAD_ARG, "quantize_transpose_bf16_fp8: null pointer");
    if (rows < 0 || cols < 0 || rows > (int64_t)65535 * 128 || cols > ((int64_t)1 << 31) - 64)
        return fail(ASTRAI_W8A8_BAD_ARG, "quantize_transpose_bf16_fp8: bad dims");
    if (fmt != ASTRAI_W8A8_E4M3 && fmt != ASTRAI_W8A8_E5M2)
        return fail(ASTRAI_W8A8_BAD_ARG,
                    "quantize_transpose_bf16_fp8: fmt must be 0 (e4m3) or 1 (e5m2)");
    if (!aligned16(x) || !aligned16(x8t) || (x8 && !aligned16(x8)))
        return fail(ASTRAI_W8A8_BAD_ARG,
                    "quantize_transpose_bf16_fp8: pointers must be 16-byte aligned");
    if (rows == 0 || cols == 0) return ASTRAI_W8A8_OK;
    w8a8::launch_quantize_transpose_fp8(x, x8, x8t, scale, amax, rows, cols, fmt,
                                        static_cast<hipStream_t>(stream));
    return check_launch("quantize_transpose_bf16_fp8");
}

int astrai_w8a8_quantize_bf16_int8_rows(const void* x, void* xq, float* s, int64_t rows,
                                        int64_t k, void* stream) {
    if (!x || !xq || !s) return fail(ASTRAI_W8A8_BAD_ARG, "quantize_bf16_int8_rows: null pointer");
    if (rows < 0 || k < 0 || rows > 0x7fffffff)
        return fail(ASTRAI_W8A8_BAD_ARG, "quantize_bf16_int8_rows: bad dims");
    if (!aligned16(x) || !aligned16(xq))
        return fail(ASTRAI_W8A8_BAD_ARG, "quantize_bf16_int8_rows: pointers must be 16-byte aligned");
    if (rows == 0 || k == 0) return ASTRAI_W8A8_OK;
    w8a8::launch_quantize_int8_rows(x, xq, s, rows, k, static_cast<hipStream_t>(stream));
    return check_launch("quantize_bf16_int8_rows");
}

int astrai_w8a8_add_rmsnorm_quantize_int8_rows(const void* x, const void* res, const void* weight,
                                               float eps, void* sum_out, void* y_out, void* xq,
                                               float* s, int64_t rows, int64_t k, void* stream) {
    if (!x || !weight || !xq || !s)
        return fail(ASTRAI_W8A8_BAD_ARG, "add_rmsnorm_quantize_int8_rows: null pointer");
    if (rows < 0 || k < 0 || rows > 0x7fffffff)
        return fail(ASTRAI_W8A8_BAD_ARG, "add_rmsnorm_quantize_int8_rows: bad dims");
    if (!(eps >= 0.0f)) return fail(ASTRAI_W8A8_BAD_ARG, "add_rmsnorm_quantize_int8_rows: eps must be >= 0");
    if ((k & 7) != 0 || k > w8a8::kFusedRowMax)
        return fail(ASTRAI_W8A8_UNSUPPORTED,
                    "add_rmsnorm_quantize_int8_rows: K must be a multiple of 8 and at most 8192");
    if (!aligned16(x) || !aligned16(weight) || !aligned16(xq) || (res && !aligned16(res)) ||
        (sum_out && !aligned16(sum_out)) || (y_out && !aligned16(y_out)))
        return fail(ASTRAI_W8A8_BAD_ARG, "add_rmsnorm_quantize_int8_rows: pointers must be 16-byte aligned");
    if (rows == 0 || k == 0) return ASTRAI_W8A8_OK;
    w8a8::launch_add_rmsnorm_quantize_int8_rows(x, res, weight, eps, sum_out, y_out, xq, s, rows, k,
                                                static_cast<hipStream_t>(stream));
    return check_launch("add_rmsnorm_quantize_int8_rows");
}

int astrai_w8a8_silu_mul_quantize_int8_rows(const void* gate, const void* up, int64_t ld, void* h_out,
                                            void* hq, float* s, int64_t rows, int64_t width,
                                            void* stream) {
    if (!gate || !up || !hq || !s)
        return fail(ASTRAI_W8A8_BAD_ARG, "silu_mul_quantize_int8_rows: null pointer");
    if (rows < 0 || width < 0 || rows > 0x7fffffff || ld < width)
        return fail(ASTRAI_W8A8_BAD_ARG, "silu_mul_quantize_int8_rows: bad dims");
    if ((width & 7) != 0 || (ld & 7) != 0 || width > w8a8::kFusedRowMax)
        return fail(ASTRAI_W8A8_UNSUPPORTED,
                    "silu_mul_quantize_int8_rows: width and ld must be multiples of 8, width at most 8192");
    if (!aligned16(gate) || !aligned16(up) || !aligned16(hq) || (h_out && !aligned16(h_out)))
        return fail(ASTRAI_W8A8_BAD_ARG, "silu_mul_quantize_int8_rows: pointers must be 16-byte aligned");
    if (rows == 0 || width == 0) return ASTRAI_W8A8_OK;
    w8a8::launch_silu_mul_quantize_int8_rows(gate, up, ld, 0, h_out, hq, s, rows, width,
                                             static_cast<hipStream_t>(stream));
    return check_launch("silu_mul_quantize_int8_rows");
}

int astrai_w8a8_silu_mul_quantize_int8_rows_blocked(const void* gu, int64_t ld, int64_t block,
                                                    void* h_out, void* hq, float* s, int64_t rows,
                                                    int64_t width, void* stream) {
    const char* what = "silu_mul_quantize_int8_rows_blocked";
    if (!gu || !hq || !s) return fail(ASTRAI_W8A8_BAD_ARG, "%s: null pointer", what);
    if (rows < 0 || width < 0 || rows > 0x7fffffff || block <= 0 || ld < 2 * width)
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: bad dims", what);
    if ((width & 7) != 0 || (ld & 7) != 0 || (block & 7) != 0 || width % block != 0 ||
        width > w8a8::kFusedRowMax)
        return fail(ASTRAI_W8A8_UNSUPPORTED,
                    "%s: width, ld and block must be multiples of 8, width a multiple of block and at most 8192",
                    what);
    if (!aligned16(gu) || !aligned16(hq) || (h_out && !aligned16(h_out)))
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: pointers must be 16-byte aligned", what);
    if (rows == 0 || width == 0) return ASTRAI_W8A8_OK;
    w8a8::launch_silu_mul_quantize_int8_rows(gu, static_cast<const uint16_t*>(gu) + block, ld, block,
                                             h_out, hq, s, rows, width,
                                             static_cast<hipStream_t>(stream));
    return check_launch(what);
}

int astrai_w8a8_add_rmsnorm_quantize_fp8_rows(const void* x, const void* res, const void* weight,
                                              float eps, void* sum_out, void* y_out, void* x8,
                                              const float* scale, float* amax, int64_t rows,
                                              int64_t k, int fmt, void* stream) {
    const char* what = "add_rmsnorm_quantize_fp8_rows";
    if (!x || !weight || !x8 || !scale) return fail(ASTRAI_W8A8_BAD_ARG, "%s: null pointer", what);
    if (rows < 0 || k < 0 || rows > 0x7fffffff) return fail(ASTRAI_W8A8_BAD_ARG, "%s: bad dims", what);
    if (fmt != ASTRAI_W8A8_E4M3 && fmt != ASTRAI_W8A8_E5M2)
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: fmt must be 0 (e4m3) or 1 (e5m2)", what);
    if ((k & 7) != 0 || k > w8a8::kFusedRowMax)
        return fail(ASTRAI_W8A8_UNSUPPORTED, "%s: K must be a multiple of 8 and at most 8192", what);
    if (!aligned16(x) || !aligned16(weight) || !aligned16(x8) || (res && !aligned16(res)) ||
        (sum_out && !aligned16(sum_out)) || (y_out && !aligned16(y_out)))
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: pointers must be 16-byte aligned", what);
    if (rows == 0 || k == 0) return ASTRAI_W8A8_OK;
    w8a8::launch_add_rmsnorm_quantize_fp8_rows(x, res, weight, eps, sum_out, y_out, x8, scale, amax,
                                               rows, k, fmt, static_cast<hipStream_t>(stream));
    return check_launch(what);
}

int astrai_w8a8_silu_mul_quantize_fp8_rows(const void* gate, const void* up, int64_t ld, void* h_out,
                                           void* h8, const float* scale, float* amax, int64_t rows,
                                           int64_t width, int fmt, void* stream) {
    const char* what = "silu_mul_quantize_fp8_rows";
    if (!gate || !up || !h8 || !scale) return fail(ASTRAI_W8A8_BAD_ARG, "%s: null pointer", what);
    if (rows < 0 || width < 0 || rows > 0x7fffffff || ld < width)
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: bad dims", what);
    if (fmt != ASTRAI_W8A8_E4M3 && fmt != ASTRAI_W8A8_E5M2)
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: fmt must be 0 (e4m3) or 1 (e5m2)", what);
    if ((width & 7) != 0 || (ld & 7) != 0)
        return fail(ASTRAI_W8A8_UNSUPPORTED, "%s: width and ld must be multiples of 8", what);
    if (!aligned16(gate) || !aligned16(up) || !aligned16(h8) || (h_out && !aligned16(h_out)))
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: pointers must be 16-byte aligned", what);
    if (rows == 0 || width == 0) return ASTRAI_W8A8_OK;
    w8a8::launch_silu_mul_quantize_fp8_rows(gate, up, ld, h_out, h8, scale, amax, rows, width, fmt,
                                            static_cast<hipStream_t>(stream));
    return check_launch(what);
}

int astrai_w8a8_quantize_int8_rows_pmax(const void* h, const float* row_max, int64_t pieces,
                                        void* hq, float* s, int64_t rows, int64_t width,
                                        void* stream) {
    const char* what = "quantize_int8_rows_pmax";
    if (!h || !row_max || !hq || !s) return fail(ASTRAI_W8A8_BAD_ARG, "%s: null pointer", what);
    if (rows < 0 || width < 0 || pieces <= 0 || rows > 0x7fffffff)
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: bad dims", what);
    if ((width & 7) != 0 || width > w8a8::kFusedRowMax)
        return fail(ASTRAI_W8A8_UNSUPPORTED, "%s: width must be a multiple of 8 and at most 8192", what);
    if (!aligned16(h) || !aligned16(hq))
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: pointers must be 16-byte aligned", what);
    if (rows == 0 || width == 0) return ASTRAI_W8A8_OK;
    w8a8::launch_quantize_int8_rows_pmax(h, row_max, pieces, hq, s, rows, width,
                                         static_cast<hipStream_t>(stream));
    return check_launch(what);
}

int astrai_w8a8_rope_cache_write_bf16(const void* qkv, int64_t ld, const float* freqs,
                                      const int64_t* positions, void* q_out, void* k_cache,
                                      void* v_cache, int64_t batch, int64_t seq, int64_t n_heads,
                                      int64_t n_kv_heads, int64_t head_dim, int64_t max_len,
                                      void* stream) {
    if (!qkv || !freqs || !positions || !q_out || !k_cache || !v_cache)
        return fail(ASTRAI_W8A8_BAD_ARG, "rope_cache_write_bf16: null pointer");
    if (batch < 0 || seq < 0 || n_heads <= 0 || n_kv_heads <= 0 || head_dim <= 0 || max_len <= 0 ||
        batch > 0x7fffffff || seq > 0x7fffffff || n_heads > 65535 || n_kv_heads > 65535)
        return fail(ASTRAI_W8A8_BAD_ARG, "rope_cache_write_bf16: bad dims");
    if (head_dim % 8 || head_dim > 65536)
        return fail(ASTRAI_W8A8_UNSUPPORTED, "rope_cache_write_bf16: head_dim must be a multiple of 8");
    if (ld < (n_heads + 2 * n_kv_heads) * head_dim || ld % 8)
        return fail(ASTRAI_W8A8_BAD_ARG, "rope_cache_write_bf16: ld must cover q|k|v and be a multiple of 8");
    if (!aligned16(qkv) || !aligned16(freqs) || !aligned16(q_out) || !aligned16(k_cache) || !aligned16(v_cache))
        return fail(ASTRAI_W8A8_BAD_ARG, "rope_cache_write_bf16: pointers must be 16-byte aligned");
    if (batch == 0 || seq == 0) return ASTRAI_W8A8_OK;
    w8a8::RopeCacheArgs a{qkv, ld, freqs, positions, q_out, k_cache, v_cache,
                          (int)batch, (int)seq, (int)n_heads, (int)n_kv_heads, (int)head_dim, max_len};
    w8a8::launch_rope_cache_write(a, static_cast<hipStream_t>(stream));
    return check_launch("rope_cache_write_bf16");
}

int astrai_w8a8_rotary_emb_bf16(const void* x, const float* freqs_cis, void* out, int64_t tokens,
                                int64_t n_heads, int64_t head_dim, void* stream) {
    if (!x || !freqs_cis || !out) return fail(ASTRAI_W8A8_BAD_ARG, "rotary_emb_bf16: null pointer");
    if (tokens < 0 || n_heads <= 0 || head_dim <= 0 || n_heads > 65535 || head_dim > 65536 ||
        tokens > ((int64_t)1 << 40))
        return fail(ASTRAI_W8A8_BAD_ARG, "rotary_emb_bf16: bad dims");
    if (head_dim % 2) return fail(ASTRAI_W8A8_BAD_ARG, "rotary_emb_bf16: head_dim must be even");
    const uintptr_t need = head_dim % 8 ? 3 : 15;  // pair-wise or 16-byte accesses
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out) |
         reinterpret_cast<uintptr_t>(freqs_cis)) & need)
        return fail(ASTRAI_W8A8_BAD_ARG, "rotary_emb_bf16: pointers must be %d-byte aligned", (int)need + 1);
    if (tokens == 0) return ASTRAI_W8A8_OK;
    if (!w8a8::launch_rotary_emb(x, freqs_cis, out, tokens, (int)n_heads, (int)head_dim,
                                 static_cast<hipStream_t>(stream)))
        return fail(ASTRAI_W8A8_UNSUPPORTED, "rotary_emb_bf16: shape not supported");
    return check_launch("rotary_emb_bf16");
}

int64_t astrai_w8a8_attn_decode_workspace_floats(int64_t batch, int64_t n_kv_heads, int64_t nsplit,
                                                 int64_t n_query_rows) {
    if (batch <= 0 || n_kv_heads <= 0 || nsplit <= 0 || n_query_rows <= 0 || n_query_rows > 8) return 0;
    return w8a8::attn_decode_workspace_floats((int)batch, (int)n_kv_heads, (int)nsplit, (int)n_query_rows);
}

// shared by the two dense decode entries; `ws` is device memory of `ws_floats` floats
static int attn_decode_common(const char* what, const void* q, const void* k_cache, const void* v_cache,
                              const int64_t* positions, float* ws, int64_t ws_floats, bool ws_is_static,
                              void* out, void* out_q, float* out_scale, int64_t batch, int64_t seq,
                              int64_t n_heads, int64_t n_kv_heads, int64_t head_dim, int64_t max_len,
                              int64_t nsplit, float scale, void* stream) {
    if (!q || !k_cache || !v_cache || !positions || (!ws && !ws_is_static) || (!out && !out_q) ||
        (out_q && !out_scale))
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: null pointer", what);
    if (batch < 0 || seq < 0 || n_heads <= 0 || n_kv_heads <= 0 || max_len <= 0 || nsplit <= 0 ||
        nsplit > 64 || batch > 65535 || n_heads % n_kv_heads)
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: bad dims", what);
    if (head_dim != 128 || (n_heads / n_kv_heads) * seq > 8 || n_heads > 64)
        return fail(ASTRAI_W8A8_UNSUPPORTED,
                    "%s: needs head_dim 128, (n_heads / n_kv_heads) * seq <= 8, n_heads <= 64", what);
    if (max_len * 256 >= ((int64_t)1 << 32))
        return fail(ASTRAI_W8A8_UNSUPPORTED, "%s: one head of the cache must stay under 4 GiB", what);
    if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || (out && !aligned16(out)) ||
        (out_q && !aligned16(out_q)))
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: pointers must be 16-byte aligned", what);
    if (batch == 0 || seq == 0) return ASTRAI_W8A8_OK;
    const int64_t need = w8a8::attn_decode_workspace_floats((int)batch, (int)n_kv_heads, (int)nsplit,
                                                            (int)((n_heads / n_kv_heads) * seq));
    if (ws_is_static) {
        if (need > kScratchFloats)
            return fail(ASTRAI_W8A8_UNSUPPORTED,
                        "%s: batch * n_kv_heads * nsplit too large for the library's scratch array "
                        "(%lld floats needed, %lld held); lower nsplit or call attn_decode_bf16 with a workspace",
                        what, (long long)need, (long long)kScratchFloats);
        if (int rc = scratch_of_current_device(what, &ws)) return rc;
    } else if (ws_floats < need) {
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: workspace too small (%lld floats needed)", what,
                    (long long)need);
    }
    w8a8::AttnDecodeArgs a{q, k_cache, v_cache, positions, ws, out, out_q, out_scale, (int)batch, (int)seq,
                           (int)n_heads, (int)n_kv_heads, (int)head_dim, max_len, (int)nsplit, scale};
    if (!w8a8::launch_attn_decode(a, static_cast<hipStream_t>(stream)))
        return fail(ASTRAI_W8A8_UNSUPPORTED, "%s: shape not supported", what);
    return check_launch(what);
}

int astrai_w8a8_attn_decode_bf16(const void* q, const void* k_cache, const void* v_cache,
                                 const int64_t* positions, float* workspace, int64_t workspace_floats,
                                 void* out, void* out_q, float* out_scale, int64_t batch,
                                 int64_t seq, int64_t n_heads,
                                 int64_t n_kv_heads, int64_t head_dim, int64_t max_len,
                                 int64_t nsplit, float scale, void* stream) {
    return attn_decode_common("attn_decode_bf16", q, k_cache, v_cache, positions, workspace, workspace_floats,
                              false, out, out_q, out_scale, batch, seq, n_heads, n_kv_heads, head_dim,
                              max_len, nsplit, scale, stream);
}

int astrai_w8a8_attn_decode_bf16_static_scratch(const void* q, const void* k_cache, const void* v_cache,
                                                const int64_t* positions, void* out, void* out_q,
                                                float* out_scale, int64_t batch, int64_t seq,
                                                int64_t n_heads, int64_t n_kv_heads, int64_t head_dim,
                                                int64_t max_len, int64_t nsplit, float scale,
                                                void* stream) {
    return attn_decode_common("attn_decode_bf16_static_scratch", q, k_cache, v_cache, positions, nullptr, 0,
                              true, out, out_q, out_scale, batch, seq, n_heads, n_kv_heads, head_dim,
                              max_len, nsplit, scale, stream);
}

int astrai_w8a8_attn_paged_decode_bf16(const void* q, const void* k_pool, const void* v_pool,
                                       const int32_t* req_to_token, const int32_t* req_pool_indices,
                                       const int32_t* kv_indptr, float* workspace,
                                       int64_t workspace_floats, void* out, int64_t batch,
                                       int64_t n_heads, int64_t n_kv_heads, int64_t head_dim,
                                       int64_t num_slots, int64_t num_requests,
                                       int64_t max_context_len, int64_t nsplit, float scale,
                                       void* stream) {
    return astrai_w8a8_attn_paged_decode_masked_bf16(q, k_pool, v_pool, req_to_token, req_pool_indices,
                                                     kv_indptr, nullptr, 0, 0, workspace, workspace_floats,
                                                     out, batch, n_heads, n_kv_heads, head_dim, num_slots,
                                                     num_requests, max_context_len, nsplit, scale, stream);
}

int astrai_w8a8_attn_paged_decode_masked_bf16(const void* q, const void* k_pool, const void* v_pool,
                                              const int32_t* req_to_token,
                                              const int32_t* req_pool_indices, const int32_t* kv_indptr,
                                              const uint8_t* mask, int64_t mask_row_stride,
                                              int64_t mask_width, float* workspace,
                                              int64_t workspace_floats, void* out, int64_t batch,
                                              int64_t n_heads, int64_t n_kv_heads, int64_t head_dim,
                                              int64_t num_slots, int64_t num_requests,
                                              int64_t max_context_len, int64_t nsplit, float scale,
                                              void* stream) {
    if (mask && (mask_width <= 0 || mask_width > INT32_MAX || mask_row_stride < 0))
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_decode_bf16: bad mask dims");
    if (!q || !k_pool || !v_pool || !req_to_token || !req_pool_indices || !kv_indptr || !workspace || !out)
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_decode_bf16: null pointer");
    if (batch < 0 || n_heads <= 0 || n_kv_heads <= 0 || num_slots <= 0 || num_requests <= 0 ||
        max_context_len <= 0 || nsplit <= 0 || nsplit > 64 || batch > 65535 || n_heads % n_kv_heads ||
        num_slots > INT32_MAX || max_context_len > INT32_MAX)
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_decode_bf16: bad dims");
    if (head_dim != 128 || n_heads / n_kv_heads > 8 || n_heads > 64)
        return fail(ASTRAI_W8A8_UNSUPPORTED,
                    "attn_paged_decode_bf16: needs head_dim 128, n_heads / n_kv_heads <= 8, n_heads <= 64");
    if (!aligned16(q) || !aligned16(k_pool) || !aligned16(v_pool) || !aligned16(out))
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_decode_bf16: pointers must be 16-byte aligned");
    if (batch == 0) return ASTRAI_W8A8_OK;
    const int64_t need = w8a8::attn_decode_workspace_floats((int)batch, (int)n_kv_heads, (int)nsplit,
                                                            (int)(n_heads / n_kv_heads));
    if (workspace_floats < need)
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_decode_bf16: workspace too small (%lld floats needed)",
                    (long long)need);
    w8a8::AttnDecodeArgs a{q, k_pool, v_pool, nullptr, workspace, out, nullptr, nullptr, (int)batch, 1,
                           (int)n_heads, (int)n_kv_heads, (int)head_dim, max_context_len, (int)nsplit, scale,
                           req_to_token, req_pool_indices, kv_indptr, max_context_len, num_slots, num_requests,
                           mask, mask_row_stride, (int)mask_width};
    if (!w8a8::launch_attn_decode(a, static_cast<hipStream_t>(stream)))
        return fail(ASTRAI_W8A8_UNSUPPORTED, "attn_paged_decode_bf16: shape not supported");
    return check_launch("attn_paged_decode_bf16");
}

int astrai_w8a8_attn_prefill_bf16(const void* q, const void* k_cache, const void* v_cache,
                                  const int64_t* positions, void* out, int64_t batch, int64_t seq,
                                  int64_t n_heads, int64_t n_kv_heads, int64_t head_dim,
                                  int64_t max_len, float scale, void* stream) {
    if (!q || !k_cache || !v_cache || !positions || !out)
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_prefill_bf16: null pointer");
    if (batch < 0 || seq < 0 || n_heads <= 0 || n_kv_heads <= 0 || max_len <= 0 ||
        n_heads % n_kv_heads || seq > (1 << 24) || batch > (1 << 20))
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_prefill_bf16: bad dims");
    if (!w8a8::attn_prefill_supported((int)n_heads, (int)n_kv_heads, (int)head_dim))
        return fail(ASTRAI_W8A8_UNSUPPORTED,
                    "attn_prefill_bf16: needs head_dim 128 and n_heads / n_kv_heads in {2, 4, 8}");
    if (max_len * 256 >= ((int64_t)1 << 32))
        return fail(ASTRAI_W8A8_UNSUPPORTED, "attn_prefill_bf16: one head of the cache must stay under 4 GiB");
    if (!(scale > 0.0f))
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_prefill_bf16: scale must be positive");
    if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(out))
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_prefill_bf16: pointers must be 16-byte aligned");
    if (batch == 0 || seq == 0) return ASTRAI_W8A8_OK;
    w8a8::AttnPrefillArgs a{q, k_cache, v_cache, positions, out, (int)batch, (int)seq, (int)n_heads,
                            (int)n_kv_heads, (int)head_dim, max_len, scale};
    if (!w8a8::launch_attn_prefill(a, static_cast<hipStream_t>(stream)))
        return fail(ASTRAI_W8A8_UNSUPPORTED, "attn_prefill_bf16: shape not supported");
    return check_launch("attn_prefill_bf16");
}

int astrai_w8a8_attn_paged_prefill_bf16(const void* q, const void* k_pool, const void* v_pool,
                                        const int32_t* req_to_token, const int32_t* req_pool_indices,
                                        const int32_t* kv_indptr, const int32_t* qo_indptr,
                                        const int32_t* q_tile_to_batch, const int32_t* q_tile_to_index,
                                        void* out, int64_t num_q_tiles, int64_t n_heads,
                                        int64_t n_kv_heads, int64_t head_dim, int64_t num_slots,
                                        int64_t num_requests, int64_t max_context_len, int causal,
                                        float scale, void* stream) {
    return astrai_w8a8_attn_paged_prefill_masked_bf16(
        q, k_pool, v_pool, req_to_token, req_pool_indices, kv_indptr, qo_indptr, q_tile_to_batch,
        q_tile_to_index, nullptr, 0, 0, 0, 0, 0, out, num_q_tiles, n_heads, n_kv_heads, head_dim, num_slots,
        num_requests, max_context_len, causal, scale, stream);
}

int astrai_w8a8_attn_paged_prefill_masked_bf16(
    const void* q, const void* k_pool, const void* v_pool, const int32_t* req_to_token,
    const int32_t* req_pool_indices, const int32_t* kv_indptr, const int32_t* qo_indptr,
    const int32_t* q_tile_to_batch, const int32_t* q_tile_to_index, const uint8_t* mask,
    int64_t mask_seq_stride, int64_t mask_head_stride, int64_t mask_row_stride, int64_t mask_rows,
    int64_t mask_width, void* out, int64_t num_q_tiles, int64_t n_heads, int64_t n_kv_heads,
    int64_t head_dim, int64_t num_slots, int64_t num_requests, int64_t max_context_len, int causal,
    float scale, void* stream) {
    if (mask && (mask_width <= 0 || mask_rows <= 0 || mask_width > INT32_MAX || mask_rows > INT32_MAX ||
                 mask_seq_stride < 0 || mask_head_stride < 0 || mask_row_stride < 0))
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_prefill_bf16: bad mask dims");
    if (!q || !k_pool || !v_pool || !req_to_token || !req_pool_indices || !kv_indptr || !qo_indptr ||
        !q_tile_to_batch || !q_tile_to_index || !out)
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_prefill_bf16: null pointer");
    if (num_q_tiles < 0 || n_heads <= 0 || n_kv_heads <= 0 || num_slots <= 0 || num_requests <= 0 ||
        max_context_len <= 0 || n_heads % n_kv_heads || num_q_tiles > (1 << 24) ||
        max_context_len > INT32_MAX)
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_prefill_bf16: bad dims");
    if (!w8a8::attn_prefill_supported((int)n_heads, (int)n_kv_heads, (int)head_dim))
        return fail(ASTRAI_W8A8_UNSUPPORTED,
                    "attn_paged_prefill_bf16: needs head_dim 128 and n_heads / n_kv_heads in {2, 4, 8}");
    if (num_slots * n_kv_heads * 256 >= ((int64_t)1 << 32))
        return fail(ASTRAI_W8A8_UNSUPPORTED, "attn_paged_prefill_bf16: a pool must stay under 4 GiB");
    if (!(scale > 0.0f)) return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_prefill_bf16: scale must be positive");
    if (!aligned16(q) || !aligned16(k_pool) || !aligned16(v_pool) || !aligned16(out))
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_prefill_bf16: pointers must be 16-byte aligned");
    if (num_q_tiles == 0) return ASTRAI_W8A8_OK;
    w8a8::AttnPrefillArgs a{};
    a.q = q; a.k_cache = k_pool; a.v_cache = v_pool; a.out = out;
    a.n_heads = (int)n_heads; a.n_kv_heads = (int)n_kv_heads; a.head_dim = (int)head_dim;
    a.scale = scale;
    a.req_to_token = req_to_token; a.req_pool_indices = req_pool_indices;
    a.kv_indptr = kv_indptr; a.qo_indptr = qo_indptr;
    a.q_tile_to_batch = q_tile_to_batch; a.q_tile_to_index = q_tile_to_index;
    a.num_q_tiles = (int)num_q_tiles; a.causal = causal ? 1 : 0;
    a.rtt_stride = max_context_len; a.num_slots = num_slots; a.num_requests = num_requests;
    a.mask = mask; a.mask_b_stride = mask_seq_stride; a.mask_h_stride = mask_head_stride;
    a.mask_l_stride = mask_row_stride; a.mask_rows = (int)mask_rows; a.mask_width = (int)mask_width;
    if (!w8a8::launch_attn_prefill(a, static_cast<hipStream_t>(stream)))
        return fail(ASTRAI_W8A8_UNSUPPORTED, "attn_paged_prefill_bf16: shape not supported");
    return check_launch("attn_paged_prefill_bf16");
}

int64_t astrai_w8a8_attn_paged_rows_workspace_floats(int64_t batch_or_tiles, int64_t n_heads,
                                                     int64_t n_kv_heads, int64_t head_dim,
                                                     int64_t nsplit, int prefill) {
    if (batch_or_tiles < 0 || nsplit <= 0 || nsplit > 64 || n_heads <= 0 || n_kv_heads <= 0 ||
        n_heads > 65535 || !w8a8::attn_rows_supported((int)n_heads, (int)n_kv_heads, (int)head_dim))
        return -1;
    return w8a8::attn_rows_workspace_floats(batch_or_tiles, (int)n_heads, (int)n_kv_heads, (int)head_dim,
                                            (int)nsplit, prefill != 0);
}

int astrai_w8a8_attn_paged_rows_bf16(
    const void* q, const void* k_pool, const void* v_pool, const int32_t* req_to_token,
    const int32_t* req_pool_indices, const int32_t* kv_indptr, const int32_t* qo_indptr,
    const int32_t* q_tile_to_batch, const int32_t* q_tile_to_index, const uint8_t* mask,
    int64_t mask_seq_stride, int64_t mask_head_stride, int64_t mask_row_stride, int64_t mask_rows,
    int64_t mask_width, float* workspace, int64_t workspace_floats, void* out, int64_t batch_or_tiles,
    int64_t n_heads, int64_t n_kv_heads, int64_t head_dim, int64_t num_slots, int64_t num_requests,
    int64_t max_context_len, int causal, int64_t nsplit, float scale, void* stream) {
    if (!q || !k_pool || !v_pool || !req_to_token || !req_pool_indices || !kv_indptr || !out ||
        (nsplit > 1 && !workspace))
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_rows_bf16: null pointer");
    const bool prefill = qo_indptr != nullptr;
    if (prefill && (!q_tile_to_batch || !q_tile_to_index))
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_rows_bf16: a prefill call needs the tile schedule");
    if (batch_or_tiles < 0 || n_heads <= 0 || n_kv_heads <= 0 || n_heads > 65535 || num_slots <= 0 ||
        num_requests <= 0 || max_context_len <= 0 || nsplit <= 0 || nsplit > 64 || n_heads % n_kv_heads ||
        num_slots > INT32_MAX || max_context_len > INT32_MAX || batch_or_tiles > (1 << 24))
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_rows_bf16: bad dims");
    if (!w8a8::attn_rows_supported((int)n_heads, (int)n_kv_heads, (int)head_dim))
        return fail(ASTRAI_W8A8_UNSUPPORTED,
                    "attn_paged_rows_bf16: needs head_dim in {32, 64, 128, 256} and n_heads / n_kv_heads <= 16");
    if (mask && (mask_width <= 0 || mask_rows <= 0 || mask_width > INT32_MAX || mask_rows > INT32_MAX ||
                 mask_seq_stride < 0 || mask_head_stride < 0 || mask_row_stride < 0))
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_rows_bf16: bad mask dims");
    if (!(scale > 0.0f)) return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_rows_bf16: scale must be positive");
    if (!aligned16(q) || !aligned16(k_pool) || !aligned16(v_pool) || !aligned16(out))
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_rows_bf16: pointers must be 16-byte aligned");
    if (batch_or_tiles == 0) return ASTRAI_W8A8_OK;
    const int64_t need = w8a8::attn_rows_workspace_floats(batch_or_tiles, (int)n_heads, (int)n_kv_heads,
                                                          (int)head_dim, (int)nsplit, prefill);
    if (need > 0 && workspace_floats < need)
        return fail(ASTRAI_W8A8_BAD_ARG, "attn_paged_rows_bf16: workspace too small (%lld floats needed)",
                    (long long)need);
    w8a8::AttnRowsArgs a{};
    a.q = q; a.k_cache = k_pool; a.v_cache = v_pool; a.req_to_token = req_to_token;
    a.req_pool_indices = req_pool_indices; a.kv_indptr = kv_indptr; a.qo_indptr = qo_indptr;
    a.q_tile_to_batch = q_tile_to_batch; a.q_tile_to_index = q_tile_to_index;
    a.ws = workspace; a.out = out; a.num_blocks = batch_or_tiles;
    a.n_heads = (int)n_heads; a.n_kv_heads = (int)n_kv_heads; a.head_dim = (int)head_dim; a.nsplit = (int)nsplit;
    a.causal = (prefill && causal) ? 1 : 0;
    a.scale = scale;
    a.rtt_stride = max_context_len; a.num_slots = num_slots; a.num_requests = num_requests;
    a.mask = mask; a.mask_b_stride = mask_seq_stride; a.mask_h_stride = mask_head_stride;
    a.mask_l_stride = mask_row_stride; a.mask_rows = (int)mask_rows; a.mask_width = (int)mask_width;
    if (!w8a8::launch_attn_rows(a, static_cast<hipStream_t>(stream)))
        return fail(ASTRAI_W8A8_UNSUPPORTED, "attn_paged_rows_bf16: shape not supported");
    return check_launch("attn_paged_rows_bf16");
}

int astrai_w8a8_quantize_bf16_fp8_block128_act(const void* x, void* x8, float* sa, int64_t m,
                                               int64_t k, void* stream) {
    if (!x || !x8 || !sa) return fail(ASTRAI_W8A8_BAD_ARG, "quantize_block128_act: null pointer");
    if (m < 0 || k < 0) return fail(ASTRAI_W8A8_BAD_ARG, "quantize_block128_act: bad dims");
    if (k % 128) return fail(ASTRAI_W8A8_UNSUPPORTED, "quantize_block128_act: K must be a multiple of 128");
    if (!aligned16(x) || !aligned16(x8))
        return fail(ASTRAI_W8A8_BAD_ARG, "quantize_block128_act: pointers must be 16-byte aligned");
    if (m == 0 || k == 0) return ASTRAI_W8A8_OK;
    w8a8::launch_quantize_fp8_block128_act(x, x8, sa, m, k, static_cast<hipStream_t>(stream));
    return check_launch("quantize_block128_act");
}

int astrai_w8a8_quantize_bf16_fp8_block128_weight(const void* w, void* w8, float* sb, int64_t n,
                                                  int64_t k, void* stream) {
    if (!w || !w8 || !sb) return fail(ASTRAI_W8A8_BAD_ARG, "quantize_block128_weight: null pointer");
    if (n < 0 || k < 0) return fail(ASTRAI_W8A8_BAD_ARG, "quantize_block128_weight: bad dims");
    if (k % 128) return fail(ASTRAI_W8A8_UNSUPPORTED, "quantize_block128_weight: K must be a multiple of 128");
    if ((n + 127) / 128 > 65535)
        return fail(ASTRAI_W8A8_UNSUPPORTED, "quantize_block128_weight: N too large");
    if (!aligned16(w) || !aligned16(w8))
        return fail(ASTRAI_W8A8_BAD_ARG, "quantize_block128_weight: pointers must be 16-byte aligned");
    if (n == 0 || k == 0) return ASTRAI_W8A8_OK;
    w8a8::launch_quantize_fp8_block128_weight(w, w8, sb, n, k, static_cast<hipStream_t>(stream));
    return check_launch("quantize_block128_weight");
}

int astrai_w8a8_gemm_fp8_pt(const void* a8, const void* b8, const float* sa, const float* sb,
                            const float* out_scale, const void* bias, void* out, int64_t m,
                            int64_t n, int64_t k, int fmt, int out_dtype, void* stream) {
    if (int rc = check_gemm("gemm_fp8_pt", a8, b8, out, m, n, k)) return rc;
    if (fmt != ASTRAI_W8A8_E4M3 && fmt != ASTRAI_W8A8_E5M2)
        return fail(ASTRAI_W8A8_BAD_ARG, "gemm_fp8_pt: fmt must be 0 (e4m3) or 1 (e5m2)");
    if (out_dtype < 0 || out_dtype > 2)
        return fail(ASTRAI_W8A8_BAD_ARG, "gemm_fp8_pt: out_dtype must be 0 (bf16), 1 (e4m3) or 2 (fp32 acc)");
    if (out_dtype != ASTRAI_W8A8_OUT_ACC && (!sa || !sb))
        return fail(ASTRAI_W8A8_BAD_ARG, "gemm_fp8_pt: null scale pointer");
    if (out_dtype == ASTRAI_W8A8_OUT_E4M3 && !out_scale)
        return fail(ASTRAI_W8A8_BAD_ARG, "gemm_fp8_pt: fp8 output requires out_scale");
    if (out_dtype == ASTRAI_W8A8_OUT_E4M3 && bias)
        return fail(ASTRAI_W8A8_BAD_ARG, "gemm_fp8_pt: bias is not supported with fp8 output");
    if (m == 0 || n == 0) return ASTRAI_W8A8_OK;
    if (k == 0) return fail(ASTRAI_W8A8_UNSUPPORTED, "gemm_fp8_pt: K must be >= 1");
    auto s = static_cast<hipStream_t>(stream);
    const w8a8::GemmArgs g = pack(a8, b8, sa, sb, out_scale, bias, out, m, n, k, out_dtype);
    if (!w8a8::launch_gemv_fp8(g, fmt, w8a8::SCALE_TENSOR, s) && !w8a8::launch_gemm_fp8_tiled(g, fmt, s))
        w8a8::launch_gemm_generic(g, fmt ? 2 : 1, w8a8::SCALE_TENSOR, s);
    return check_launch("gemm_fp8_pt");
}

int astrai_w8a8_gemm_fp8_ptpc(const void* a8, const void* b8, const float* sa, const float* sb,
                              const void* bias, void* out, int64_t m, int64_t n, int64_t k,
                              int fmt, void* stream) {
    if (int rc = check_gemm("gemm_fp8_ptpc", a8, b8, out, m, n, k)) return rc;
    if (fmt != ASTRAI_W8A8_E4M3 && fmt != ASTRAI_W8A8_E5M2)
        return fail(ASTRAI_W8A8_BAD_ARG, "gemm_fp8_ptpc: fmt must be 0 (e4m3) or 1 (e5m2)");
    if (!sa || !sb) return fail(ASTRAI_W8A8_BAD_ARG, "gemm_fp8_ptpc: null scale pointer");
    if (m == 0 || n == 0) return ASTRAI_W8A8_OK;
    if (k == 0) return fail(ASTRAI_W8A8_UNSUPPORTED, "gemm_fp8_ptpc: K must be >= 1");
    auto s = static_cast<hipStream_t>(stream);
    const w8a8::GemmArgs g = pack(a8, b8, sa, sb, nullptr, bias, out, m, n, k, w8a8::OUT_BF16);
    if (!w8a8::launch_gemv_fp8(g, fmt, w8a8::SCALE_ROWCOL, s) && !w8a8::launch_gemm_fp8_rowcol_tiled(g, fmt, s))
        w8a8::launch_gemm_generic(g, fmt ? 2 : 1, w8a8::SCALE_ROWCOL, s);
    return check_launch("gemm_fp8_ptpc");
}

int astrai_w8a8_gemm_fp8_block128(const void* a8, const void* b8, const float* sa,
                                  const float* sb, const void* bias, void* out, int64_t m,
                                  int64_t n, int64_t k, void* stream) {
    if (int rc = check_gemm("gemm_fp8_block128", a8, b8, out, m, n, k)) return rc;
    if (!sa || !sb) return fail(ASTRAI_W8A8_BAD_ARG, "gemm_fp8_block128: null scale pointer");
    if (k == 0 || k % 128)
        return fail(ASTRAI_W8A8_UNSUPPORTED, "gemm_fp8_block128: K must be a positive multiple of 128");
    if (m == 0 || n == 0) return ASTRAI_W8A8_OK;
    auto s = static_cast<hipStream_t>(stream);
    const w8a8::GemmArgs g =
        pack(a8, b8, sa, sb, nullptr, bias, out, m, n, k, w8a8::OUT_BF16);
    if (!w8a8::launch_gemv_fp8_block128(g, s) && !w8a8::launch_gemm_fp8_block128_tiled(g, s))
        w8a8::launch_gemm_generic(g, 1, w8a8::SCALE_BLOCK128, s);
    return check_launch("gemm_fp8_block128");
}

static int int8_common(const char* what, const void* a, const void* b, const float* sa,
                       const float* sb, void* out, int64_t m, int64_t n, int64_t k,
                       int out_dtype) {
    if (int rc = check_gemm(what, a, b, out, m, n, k)) return rc;
    if (out_dtype != ASTRAI_W8A8_OUT_BF16 && out_dtype != ASTRAI_W8A8_OUT_ACC)
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: out_dtype must be 0 (bf16) or 2 (int32 acc)", what);
    if (out_dtype == ASTRAI_W8A8_OUT_BF16 && (!sa || !sb))
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: null scale pointer", what);
    if (k == 0 && m > 0 && n > 0) return fail(ASTRAI_W8A8_UNSUPPORTED, "%s: K must be >= 1", what);
    return ASTRAI_W8A8_OK;
}

int astrai_w8a8_gemm_int8_ptpc(const void* a, const void* b, const float* sa, const float* sb,
                               const void* bias, void* out, int64_t m, int64_t n, int64_t k,
                               int out_dtype, void* stream) {
    if (int rc = int8_common("gemm_int8_ptpc", a, b, sa, sb, out, m, n, k, out_dtype)) return rc;
    if (m == 0 || n == 0) return ASTRAI_W8A8_OK;
    auto s = static_cast<hipStream_t>(stream);
    const w8a8::GemmArgs g = pack(a, b, sa, sb, nullptr, bias, out, m, n, k, out_dtype);
    if (m <= 128 && w8a8::launch_gemv_int8(g, s)) return check_launch("gemv_int8_ptpc");
    if (!w8a8::launch_gemm_int8_tiled(g, s))
        w8a8::launch_gemm_generic(g, 0, w8a8::SCALE_ROWCOL, s);
    return check_launch("gemm_int8_ptpc");
}

int astrai_w8a8_gemm_int8_ptpc_resid(const void* a, const void* b, const float* sa, const float* sb,
                                     const void* bias, const void* resid, void* out, int64_t m,
                                     int64_t n, int64_t k, void* stream) {
    const char* what = "gemm_int8_ptpc_resid";
    if (int rc = int8_common(what, a, b, sa, sb, out, m, n, k, ASTRAI_W8A8_OUT_BF16)) return rc;
    if (!resid) return fail(ASTRAI_W8A8_BAD_ARG, "%s: null residual pointer", what);
    if (!aligned16(resid)) return fail(ASTRAI_W8A8_BAD_ARG, "%s: resid must be 16-byte aligned", what);
    if (m == 0 || n == 0) return ASTRAI_W8A8_OK;
    {
        const auto lo = reinterpret_cast<uintptr_t>(out), ro = reinterpret_cast<uintptr_t>(resid);
        const uintptr_t bytes = (uintptr_t)m * (uintptr_t)n * 2u;
        if (lo < ro + bytes && ro < lo + bytes)
            return fail(ASTRAI_W8A8_BAD_ARG, "%s: out overlaps resid", what);
    }
    auto s = static_cast<hipStream_t>(stream);
    w8a8::GemmArgs g = pack(a, b, sa, sb, nullptr, bias, out, m, n, k, ASTRAI_W8A8_OUT_BF16);
    g.resid = resid;
    if (w8a8::launch_gemm_int8_resid(g, s)) return check_launch(what);
    // shapes without a fused epilogue: the plain product, then the addition in place
    g.resid = nullptr;
    if (!(m <= 128 && w8a8::launch_gemv_int8(g, s)) && !w8a8::launch_gemm_int8_tiled(g, s))
        w8a8::launch_gemm_generic(g, 0, w8a8::SCALE_ROWCOL, s);
    w8a8::launch_add_bf16(out, resid, out, m * n, s);
    return check_launch(what);
}

int astrai_w8a8_gemv_int8_ptpc(const void* a, const void* b, const float* sa, const float* sb,
                               const void* bias, void* out, int64_t m, int64_t n, int64_t k,
                               int out_dtype, void* stream) {
    if (int rc = int8_common("gemv_int8_ptpc", a, b, sa, sb, out, m, n, k, out_dtype)) return rc;
    if (m > 128 || k % 256 || k == 0)
        return fail(ASTRAI_W8A8_UNSUPPORTED,
                    "gemv_int8_ptpc: needs M <= 128 and K a positive multiple of 256 (got m=%lld k=%lld)",
                    (long long)m, (long long)k);
    if (m == 0 || n == 0) return ASTRAI_W8A8_OK;
    const w8a8::GemmArgs g = pack(a, b, sa, sb, nullptr, bias, out, m, n, k, out_dtype);
    if (!w8a8::launch_gemv_int8(g, static_cast<hipStream_t>(stream)))
        return fail(ASTRAI_W8A8_UNSUPPORTED, "gemv_int8_ptpc: weight matrix of 2 GiB or more");
    return check_launch("gemv_int8_ptpc");
}

int astrai_w8a8_gemm_int8_ptpc_rope_cache(const void* a, const void* b, const float* sa,
                                          const float* sb, const float* freqs,
                                          const int64_t* positions, void* q_out, void* k_cache,
                                          void* v_cache, int64_t batch, int64_t seq,
                                          int64_t n_heads, int64_t n_kv_heads, int64_t head_dim,
                                          int64_t max_len, int64_t k, void* stream) {
    const char* what = "gemm_int8_ptpc_rope_cache";
    if (!a || !b || !sa || !sb || !freqs || !positions || !q_out || !k_cache || !v_cache)
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: null pointer", what);
    if (batch < 0 || seq < 0 || n_heads <= 0 || n_kv_heads <= 0 || head_dim <= 0 || max_len <= 0 ||
        k <= 0 || n_heads > 65535 || n_kv_heads > 65535 || head_dim > 65536 || k > kMaxDim ||
        batch > kMaxDim || seq > kMaxDim)
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: bad dims", what);
    if (!aligned16(a) || !aligned16(b) || !aligned16(freqs) || !aligned16(q_out) || !aligned16(k_cache) ||
        !aligned16(v_cache))
        return fail(ASTRAI_W8A8_BAD_ARG, "%s: pointers must be 16-byte aligned", what);
    const int64_t m = batch * seq, n = (n_heads + 2 * n_kv_heads) * head_dim;
    if (m == 0) return ASTRAI_W8A8_OK;
    if (n * k >= ((int64_t)1 << 31) || m * k >= ((int64_t)1 << 31))
        return fail(ASTRAI_W8A8_UNSUPPORTED, "%s: operands must stay under 2 GiB", what);
    const w8a8::GemmArgs g = pack(a, b, sa, sb, nullptr, nullptr, nullptr, m, n, k, w8a8::OUT_BF16);
    const w8a8::RopeCacheArgs rc{nullptr, 0, freqs, positions, q_out, k_cache, v_cache,
                                 (int)batch, (int)seq, (int)n_heads, (int)n_kv_heads, (int)head_dim, max_len};
    const bool small = m <= 64 && k % 256 == 0 && head_dim % 4 == 0;
    if (!(small && w8a8::launch_gemm_int8_rope_cache(g, rc, static_cast<hipStream_t>(stream))) &&
        !w8a8::launch_gemm_int8_rope_cache_large(g, rc, static_cast<hipStream_t>(stream)))
        return fail(ASTRAI_W8A8_UNSUPPORTED,
                    "%s: needs either batch * seq <= 64 with K a multiple of 256 and head_dim a multiple of 4, "
                    "or head_dim 128 with at least 192 output tiles of 256 x 256 and K a multiple of 128, at "
                    "least 256 (got m=%lld k=%lld head_dim=%lld)",
                    what, (long long)m, (long long)k, (long long)head_dim);
    return check_launch(what);
}

int astrai_w8a8_gemm_int8_ptpc_swiglu(const void* a, const void* b, const float* sa, const float* sb,
                                      void* h_out, float* row_max, int64_t m, int64_t n, int64_t k,
                                      void* stream) {
    const char* what = "gemm_int8_ptpc_swiglu";
    if (int rc = int8_common(what, a, b, sa, sb, h_out, m, n, k, ASTRAI_W8A8_OUT_BF16)) return rc;
    if (!row_max) return fail(ASTRAI_W8A8_BAD_ARG, "%s: null pointer", what);
    if (n % 128)
        return fail(ASTRAI_W8A8_UNSUPPORTED, "%s: N (gate and up rows together) must be a multiple of 128", what);
    if (m == 0 || n == 0) return ASTRAI_W8A8_OK;
    w8a8::GemmArgs g = pack(a, b, sa, sb, nullptr, nullptr, h_out, m, n, k, w8a8::OUT_BF16);
    g.row_max = row_max;
    if (!w8a8::launch_gemm_int8_swiglu(g, static_cast<hipStream_t>(stream)))
        return fail(ASTRAI_W8A8_UNSUPPORTED,
                    "%s: needs at least 192 output tiles of 256 x 256, K a multiple of 128 and at least 256",
                    what);
    return check_launch(what);
}

int astrai_w8a8_mfma_probe(int kind, const void* a, const void* b, void* d_raw, void* stream) {
    if (!a || !b || !d_raw) return fail(ASTRAI_W8A8_BAD_ARG, "mfma_probe: null pointer");
    if (!aligned16(a) || !aligned16(b)) return fail(ASTRAI_W8A8_BAD_ARG, "mfma_probe: pointers must be 16-byte aligned");
    if (!w8a8::launch_mfma_probe(kind, a, b, d_raw, static_cast<hipStream_t>(stream)))
        return fail(ASTRAI_W8A8_BAD_ARG, "mfma_probe: kind must be 0..7");
    return check_launch("mfma_probe");
}

int astrai_w8a8_gemm_int8_ptpc_tiled(const void* a, const void* b, const float* sa,
                                     const float* sb, const void* bias, void* out, int64_t m,
                                     int64_t n, int64_t k, int out_dtype, void* stream) {
    if (int rc = int8_common("gemm_int8_ptpc_tiled", a, b, sa, sb, out, m, n, k, out_dtype))
        return rc;
    if (m == 0 || n == 0) return ASTRAI_W8A8_OK;
    const w8a8::GemmArgs g = pack(a, b, sa, sb, nullptr, bias, out, m, n, k, out_dtype);
    if (!w8a8::launch_gemm_int8_tiled(g, static_cast<hipStream_t>(stream), false))
        return fail(ASTRAI_W8A8_UNSUPPORTED,
                    "gemm_int8_ptpc_tiled: needs K %% 16 == 0 and operands under 2 GiB");
    return check_launch("gemm_int8_ptpc_tiled");
}

}  // extern "C"
