// Rotary embedding of the q / k projections and the KV-cache write of one decoder
// layer in one pass over the fused q|k|v projection output.
//
// The reference rotates adjacent (even, odd) pairs of each head in fp32 and casts
// back (astrai/extension/backend/rotary.py:25-33), permutes q/k/v to
// [batch, heads, seq, head_dim] and writes k, v into the cache at the tokens'
// positions (astrai/model/components/attention.py:19-85). Done with tensor ops
// that is a dozen small kernels per layer and decode step; here it is one:
//   q_out[b, h, s, :]            = rope(q[b, s, h, :])
//   k_cache[b, hk, pos[s], :]    = rope(k[b, s, hk, :])
//   v_cache[b, hk, pos[s], :]    = v[b, s, hk, :]
// with rope(x)[2i] = x[2i] cos_i - x[2i+1] sin_i, rope(x)[2i+1] = x[2i] sin_i +
// x[2i+1] cos_i, products and sums each rounded in fp32 (no fused multiply-add), one
// rounding to bf16 -- bit for bit what the tensor ops give. A lane handles 8
// elements (16 bytes, four pairs). A position outside [0, max_len) writes nothing.
#include <algorithm>

#include "common.cuh"
#include "launchers.h"

namespace w8a8 {

namespace {

__device__ __forceinline__ void unpack8_bf16(u32x4 raw, float (&f)[8]) {
    f[0] = __uint_as_float(raw.x << 16);
    f[1] = __uint_as_float(raw.x & 0xffff0000u);
    f[2] = __uint_as_float(raw.y << 16);
    f[3] = __uint_as_float(raw.y & 0xffff0000u);
    f[4] = __uint_as_float(raw.z << 16);
    f[5] = __uint_as_float(raw.z & 0xffff0000u);
    f[6] = __uint_as_float(raw.w << 16);
    f[7] = __uint_as_float(raw.w & 0xffff0000u);
}

__global__ __launch_bounds__(256) void rope_cache_write_kernel(RopeCacheArgs a) {
    const int vec_per_head = a.head_dim >> 3;
    const int heads_all = a.n_heads + 2 * a.n_kv_heads;
    const int64_t vec_per_row = (int64_t)heads_all * vec_per_head;
    const int64_t total = (int64_t)a.batch * a.seq * vec_per_row;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int64_t row = idx / vec_per_row;
    const int v = (int)(idx - row * vec_per_row);
    const int b = (int)(row / a.seq), s = (int)(row - (int64_t)b * a.seq);
    const int hh = v / vec_per_head, dv = v - hh * vec_per_head;

    const uint16_t* src = static_cast<const uint16_t*>(a.qkv) + row * a.ld + (int64_t)hh * a.head_dim + dv * 8;
    float x[8];
    unpack8_bf16(*reinterpret_cast<const u32x4*>(src), x);

    u32x4 outv;
    if (hh < a.n_heads + a.n_kv_heads) {
        // four (cos, sin) pairs of this token's position: 32 contiguous bytes
        const float* fr = a.freqs + ((int64_t)s * (a.head_dim >> 1) + dv * 4) * 2;
        const f32x4 f0 = *reinterpret_cast<const f32x4*>(fr);
        const f32x4 f1 = *reinterpret_cast<const f32x4*>(fr + 4);
        const float cs[8] = {f0[0], f0[1], f0[2], f0[3], f1[0], f1[1], f1[2], f1[3]};
        float y[8];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
#pragma clang fp contract(off)
            const float c = cs[2 * p], sn = cs[2 * p + 1];
            const float xe = x[2 * p], xo = x[2 * p + 1];
            const float a0 = xe * c, a1 = xo * sn, b0 = xe * sn, b1 = xo * c;
            y[2 * p] = a0 - a1;
            y[2 * p + 1] = b0 + b1;
        }
        outv.x = pack_bf16x2(y[0], y[1]);
        outv.y = pack_bf16x2(y[2], y[3]);
        outv.z = pack_bf16x2(y[4], y[5]);
        outv.w = pack_bf16x2(y[6], y[7]);
    } else {
        outv = *reinterpret_cast<const u32x4*>(src);
    }

    if (hh < a.n_heads) {
        uint16_t* dst = static_cast<uint16_t*>(a.q_out) +
                        (((int64_t)b * a.n_heads + hh) * a.seq + s) * a.head_dim + dv * 8;
        *reinterpret_cast<u32x4*>(dst) = outv;
    } else {
        const int64_t pos = a.positions[s];
        if (pos < 0 || pos >= a.max_len) return;
        const bool is_k = hh < a.n_heads + a.n_kv_heads;
        const int hk = hh - a.n_heads - (is_k ? 0 : a.n_kv_heads);
        uint16_t* base = static_cast<uint16_t*>(is_k ? a.k_cache : a.v_cache);
        uint16_t* dst = base + (((int64_t)b * a.n_kv_heads + hk) * a.max_len + pos) * a.head_dim + dv * 8;
        *reinterpret_cast<u32x4*>(dst) = outv;
    }
}

// Rotary embedding alone: x and out bf16 [tokens, heads, head_dim], freqs fp32
// [tokens, head_dim / 2, 2] holding each token's own (cos, sin) -- the contract of the
// reference's rotary_emb kernel (csrc/kernels/rotary/rotary_emb.cu:6-45), same pair
// arithmetic as above. PAIRS pairs per lane: 4 (16-byte accesses) or 1.
template <int PAIRS>
__global__ __launch_bounds__(256) void rotary_emb_kernel(const uint16_t* __restrict__ x,
                                                         const float* __restrict__ freqs,
                                                         uint16_t* __restrict__ out, int64_t tokens,
                                                         int heads, int head_dim) {
    const int per_head = (head_dim >> 1) / PAIRS;  // lanes per head
    const int64_t total = tokens * heads * per_head;
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
        const int64_t th = idx / per_head;  // token * heads + head
        const int dv = (int)(idx - th * per_head);
        const int64_t token = th / heads;
        const int64_t xo = th * head_dim + (int64_t)dv * 2 * PAIRS;
        const float* fr = freqs + (token * (head_dim >> 1) + (int64_t)dv * PAIRS) * 2;
        float xv[2 * PAIRS], cs[2 * PAIRS], y[2 * PAIRS];
        if constexpr (PAIRS == 4) {
            unpack8_bf16(*reinterpret_cast<const u32x4*>(x + xo), xv);
            const f32x4 f0 = *reinterpret_cast<const f32x4*>(fr);
            const f32x4 f1 = *reinterpret_cast<const f32x4*>(fr + 4);
            cs[0] = f0[0]; cs[1] = f0[1]; cs[2] = f0[2]; cs[3] = f0[3];
            cs[4] = f1[0]; cs[5] = f1[1]; cs[6] = f1[2]; cs[7] = f1[3];
        } else {
            const uint32_t raw = *reinterpret_cast<const uint32_t*>(x + xo);
            xv[0] = __uint_as_float(raw << 16);
            xv[1] = __uint_as_float(raw & 0xffff0000u);
            cs[0] = fr[0];
            cs[1] = fr[1];
        }
#pragma unroll
        for (int p = 0; p < PAIRS; ++p) {
#pragma clang fp contract(off)
            const float c = cs[2 * p], sn = cs[2 * p + 1];
            const float xe = xv[2 * p], xod = xv[2 * p + 1];
            const float a0 = xe * c, a1 = xod * sn, b0 = xe * sn, b1 = xod * c;
            y[2 * p] = a0 - a1;
            y[2 * p + 1] = b0 + b1;
        }
        if constexpr (PAIRS == 4) {
            u32x4 o;
            o.x = pack_bf16x2(y[0], y[1]);
            o.y = pack_bf16x2(y[2], y[3]);
            o.z = pack_bf16x2(y[4], y[5]);
            o.w = pack_bf16x2(y[6], y[7]);
            *reinterpret_cast<u32x4*>(out + xo) = o;
        } else {
            *reinterpret_cast<uint32_t*>(out + xo) = pack_bf16x2(y[0], y[1]);
        }
    }
}

}  // namespace

bool launch_rotary_emb(const void* x, const float* freqs, void* out, int64_t tokens, int heads,
                       int head_dim, hipStream_t stream) {
    if (tokens < 0 || heads <= 0 || head_dim <= 0 || (head_dim & 1)) return false;
    const bool wide = head_dim % 8 == 0;
    const int64_t total = tokens * heads * ((head_dim >> 1) / (wide ? 4 : 1));
    if (total == 0) return true;
    const int64_t blocks = std::min<int64_t>((total + 255) / 256, (int64_t)1 << 20);
    const auto* xp = static_cast<const uint16_t*>(x);
    auto* op = static_cast<uint16_t*>(out);
    if (wide)
        rotary_emb_kernel<4><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(xp, freqs, op, tokens, heads, head_dim);
    else
        rotary_emb_kernel<1><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(xp, freqs, op, tokens, heads, head_dim);
    return true;
}

void launch_rope_cache_write(const RopeCacheArgs& a, hipStream_t stream) {
    const int64_t total = (int64_t)a.batch * a.seq * (a.n_heads + 2 * a.n_kv_heads) * (a.head_dim >> 3);
    if (total <= 0) return;
    const int64_t blocks = (total + 255) / 256;
    rope_cache_write_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(a);
}

}  // namespace w8a8
