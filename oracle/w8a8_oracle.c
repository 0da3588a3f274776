/*
 * Plain-C restatement of the W8A8 linear arithmetic. TEST INFRASTRUCTURE ONLY:
 * loaded by tests/ (and built by __graft_entry__.build()) as an independent
 * check of oracle/w8a8_oracle.py; never linked into or called by the product.
 *
 * The fp8 codecs are written from the OCP 8-bit floating point definition
 * (e4m3fn: bias 7, no infinities, S.1111.111 = NaN, max 448; e5m2: bias 15,
 * IEEE-like inf/NaN, max 57344), with round-to-nearest-even and the overflow
 * behaviour of a plain cast (e4m3fn: NaN past the rounding boundary 464;
 * e5m2: inf at and past 61440), i.e. what `Tensor.to(torch.float8_*)` does in
 * astrai/extension/ops/fp8.py:80. The saturating variants clamp to the finite
 * maximum first, i.e. what the device kernels do with __NV_SATFINITE
 * (csrc/kernels/fp8/gemm.cuh:35-42).
 *
 * The GEMM loops follow the CPU loop of csrc/tests/fp8_mma_test.cu:105-116
 * (decode, fmaf-accumulate in k order, scale afterwards) and, for int8, exact
 * int32 accumulation.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float bits_to_float(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static uint32_t float_to_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

/* Generic small-float decode: ebits exponent bits, mbits mantissa bits. */
static float decode_small(uint8_t code, int ebits, int mbits, int bias, int fn) {
    int sign = code >> 7;
    int e = (code >> mbits) & ((1 << ebits) - 1);
    int m = code & ((1 << mbits) - 1);
    float v;
    if (fn) {
        if (e == (1 << ebits) - 1 && m == (1 << mbits) - 1) return NAN;
    } else if (e == (1 << ebits) - 1) {
        if (m) return NAN;
        return sign ? -INFINITY : INFINITY;
    }
    if (e == 0)
        v = ldexpf((float)m, 1 - bias - mbits);
    else
        v = ldexpf((float)((1 << mbits) | m), e - bias - mbits);
    return sign ? -v : v;
}

float oracle_e4m3fn_decode(uint8_t c) { return decode_small(c, 4, 3, 7, 1); }
float oracle_e5m2_decode(uint8_t c) { return decode_small(c, 5, 2, 15, 0); }

/* Round-to-nearest-even encode by exact arithmetic on the float's fields. */
static uint8_t encode_small(float f, int ebits, int mbits, int bias, int fn) {
    uint32_t u = float_to_bits(f);
    uint8_t sign = (uint8_t)((u >> 31) << 7);
    uint32_t mag = u & 0x7fffffffu;
    int emax_field = (1 << ebits) - 1;
    uint8_t nan_code = fn ? (uint8_t)(sign | 0x7f) : (uint8_t)(sign | 0x7f);
    if (mag > 0x7f800000u) return nan_code; /* NaN in */
    if (mag == 0x7f800000u) {               /* inf in */
        if (fn) return nan_code;
        return (uint8_t)(sign | (emax_field << mbits));
    }
    float a = bits_to_float(mag);
    if (a == 0.0f) return sign;
    int e;
    (void)frexpf(a, &e); /* a = frac * 2^e, frac in [0.5,1) -> unbiased exp e-1 */
    int ue = e - 1;
    int emin = 1 - bias; /* exponent of the smallest normal */
    int q_exp = (ue < emin ? emin : ue) - mbits; /* weight of one mantissa ulp */
    /* scaled = a / 2^q_exp is exact in float (power-of-two scaling) unless it
       underflows far below half an ulp, in which case it rounds to 0 anyway. */
    float scaled = ldexpf(a, -q_exp);
    float r = rintf(scaled); /* default rounding mode = nearest-even */
    uint32_t q = (uint32_t)r;
    /* q counts ulps: for normals q in [2^mbits, 2^(mbits+1)] */
    int field_e;
    uint32_t field_m;
    if (ue < emin) {
        if (q >= (1u << mbits)) { /* rounded up into the smallest normal */
            field_e = 1;
            field_m = q - (1u << mbits);
        } else {
            field_e = 0;
            field_m = q;
        }
    } else {
        field_e = ue + bias;
        if (q == (2u << mbits)) { /* mantissa overflow -> next binade */
            field_e += 1;
            q = 1u << mbits;
        }
        field_m = q - (1u << mbits);
    }
    if (fn) {
        /* all-ones exponent is a normal binade except mantissa 111 = NaN */
        if (field_e > emax_field ||
            (field_e == emax_field && field_m == (1u << mbits) - 1))
            return nan_code;
    } else {
        if (field_e >= emax_field) return (uint8_t)(sign | (emax_field << mbits));
    }
    return (uint8_t)(sign | (field_e << mbits) | field_m);
}

uint8_t oracle_e4m3fn_encode(float f) { return encode_small(f, 4, 3, 7, 1); }
uint8_t oracle_e5m2_encode(float f) { return encode_small(f, 5, 2, 15, 0); }

uint8_t oracle_e4m3fn_encode_sat(float f) {
    if (f > 448.0f) f = 448.0f;
    if (f < -448.0f) f = -448.0f;
    return encode_small(f, 4, 3, 7, 1);
}
uint8_t oracle_e5m2_encode_sat(float f) {
    if (f > 57344.0f) f = 57344.0f;
    if (f < -57344.0f) f = -57344.0f;
    return encode_small(f, 5, 2, 15, 0);
}

static float bf16_to_float(uint16_t h) { return bits_to_float((uint32_t)h << 16); }

/* x8 = fp8(x / scale) elementwise over bf16 input; returns max |x|.
 * astrai/extension/ops/fp8.py:80-81 (saturate=0) / gemm.cuh:128-146 (saturate=1,
 * but with the true division of the CPU path, not the reciprocal multiply). */
float oracle_fp8_quantize(const uint16_t* x, uint8_t* x8, float scale, int64_t total,
                          int fmt, int saturate) {
    float amax = 0.0f;
    for (int64_t i = 0; i < total; ++i) {
        float f = bf16_to_float(x[i]);
        float a = fabsf(f);
        if (a > amax) amax = a;
        float q = f / scale;
        if (fmt)
            x8[i] = saturate ? oracle_e5m2_encode_sat(q) : oracle_e5m2_encode(q);
        else
            x8[i] = saturate ? oracle_e4m3fn_encode_sat(q) : oracle_e4m3fn_encode(q);
    }
    return amax;
}

/* c[m,n] = sum_k dec(a[m,k]) * dec(b[n,k]), fmaf in k order, no scaling.
 * csrc/tests/fp8_mma_test.cu:105-113. */
void oracle_fp8_gemm_f32(const uint8_t* a, const uint8_t* b, float* c, int64_t m,
                         int64_t n, int64_t k, int fmt) {
    float table[256];
    for (int i = 0; i < 256; ++i)
        table[i] = fmt ? oracle_e5m2_decode((uint8_t)i) : oracle_e4m3fn_decode((uint8_t)i);
    for (int64_t i = 0; i < m; ++i)
        for (int64_t j = 0; j < n; ++j) {
            float sum = 0.0f;
            for (int64_t p = 0; p < k; ++p)
                sum = fmaf(table[a[i * k + p]], table[b[j * k + p]], sum);
            c[i * n + j] = sum;
        }
}

/* 128-block-scaled variant: per K-block partial dot (fmaf), then
 * acc += partial * sa[m,kb] * sb[n/128,kb]. */
void oracle_fp8_gemm_block128_f32(const uint8_t* a, const uint8_t* b, const float* sa,
                                  const float* sb, float* c, int64_t m, int64_t n,
                                  int64_t k) {
    float table[256];
    int64_t kb = k / 128;
    for (int i = 0; i < 256; ++i) table[i] = oracle_e4m3fn_decode((uint8_t)i);
    for (int64_t i = 0; i < m; ++i)
        for (int64_t j = 0; j < n; ++j) {
            float acc = 0.0f;
            for (int64_t q = 0; q < kb; ++q) {
                float part = 0.0f;
                for (int64_t p = q * 128; p < q * 128 + 128; ++p)
                    part = fmaf(table[a[i * k + p]], table[b[j * k + p]], part);
                acc += part * sa[i * kb + q] * sb[(j / 128) * kb + q];
            }
            c[i * n + j] = acc;
        }
}

/* Exact int32 accumulator c[m,n] = sum_k a[m,k]*b[n,k]. */
void oracle_int8_gemm_i32(const int8_t* a, const int8_t* b, int32_t* c, int64_t m,
                          int64_t n, int64_t k) {
    for (int64_t i = 0; i < m; ++i)
        for (int64_t j = 0; j < n; ++j) {
            int32_t sum = 0;
            const int8_t* ar = a + i * k;
            const int8_t* br = b + j * k;
            for (int64_t p = 0; p < k; ++p) sum += (int32_t)ar[p] * (int32_t)br[p];
            c[i * n + j] = sum;
        }
}

/* Symmetric per-row int8 quantization of bf16 rows:
 * s = max(|row|, 1e-12)/127, q = clamp(rne(x/s), +-127). */
void oracle_int8_quantize_rows(const uint16_t* x, int8_t* q, float* s, int64_t rows,
                               int64_t k) {
    for (int64_t r = 0; r < rows; ++r) {
        float amax = 0.0f;
        for (int64_t p = 0; p < k; ++p) {
            float a = fabsf(bf16_to_float(x[r * k + p]));
            if (a > amax) amax = a;
        }
        if (amax < 1e-12f) amax = 1e-12f;
        float sc = amax / 127.0f;
        s[r] = sc;
        for (int64_t p = 0; p < k; ++p) {
            float v = rintf(bf16_to_float(x[r * k + p]) / sc);
            if (v > 127.0f) v = 127.0f;
            if (v < -127.0f) v = -127.0f;
            q[r * k + p] = (int8_t)v;
        }
    }
}
