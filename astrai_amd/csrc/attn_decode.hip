// Grouped-query attention of a few new tokens against a dense bf16 KV cache
// (decode step), split over the context ("flash decoding"), head_dim 128.
//
// The reference's decode attention expands the KV heads and calls SDPA on
// [batch, heads, seq, head_dim] tensors (astrai/extension/backend/attention.py:
// 244-253,443-498); causality comes from the tokens' positions. Here the n_rep
// query heads of a KV group times the S new tokens form up to 8 query rows that
// share every key/value row read from the cache, the mask is `key <= position`
// computed in the kernel (no mask tensor), and the output is written as
// [batch, seq, heads*head_dim], the layout the output projection reads.
//
// Kernel 1 (one workgroup per batch x KV head x context split, four waves taking
// 16-key tiles in turn):
//   scores: v_mfma_f32_16x16x32_bf16 with the 16 keys of a tile as rows (16 bytes
//     per lane straight from the cache) and the query rows as columns, so a lane
//     ends up with the scores of one query for keys 4g..4g+3 (g = lane / 16);
//   online softmax per query in fp32 (running max and sum, shared by the four
//     lanes of a query through two butterfly steps);
//   P.V on the vector ALU: lane (g, c) owns dims 8c..8c+7 of keys 4g..4g+3 -- one
//     16-byte load covers four whole 256-byte value rows -- and fetches the four
//     probabilities it needs from the lanes that hold them (same 16-lane group).
//   The waves' and lane groups' partial (max, sum, acc) are merged through LDS and
//   written to a workspace.
// Kernel 2 merges the splits of a token and writes bf16.
#include "common.cuh"
#include "launchers.h"

namespace w8a8 {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kD = 128;
constexpr float kNegBig = -1e30f;  // finite stand-in for -inf: no inf - inf

__device__ __forceinline__ float lane_read(float v, int src_lane) {
    return __int_as_float(__builtin_amdgcn_ds_bpermute(src_lane << 2, __float_as_int(v)));
}

// workspace per (batch, kv head, split): NQ rows of [kD values | max | sum]
constexpr int kWsRow = kD + 2;

__device__ __forceinline__ int lane_read_i(int v, int src_lane) {
    return __builtin_amdgcn_ds_bpermute(src_lane << 2, v);
}

// PAGED: the caches are token-granular pools [slots, n_kv_heads, 128] and key j of
// sequence b lives in slot req_to_token[req_pool_indices[b]][j]
// (csrc/kernels/attention/layout_policies.cuh:174-232); every sequence has its own
// length kv_indptr[b+1] - kv_indptr[b] and one query token, the newest.
// MASK (paged only): a bool tensor [batch, mask_width] picks the positions a sequence may
// attend on top of its length (csrc/kernels/attention/mma_utils.cuh:196-199)
template <int NQ, bool PAGED, bool MASK = false>
__global__ __launch_bounds__(256) void attn_decode_partial_kernel(AttnDecodeArgs a) {
    __shared__ float sh_acc[4][NQ][kD];
    __shared__ float sh_ml[4][NQ][2];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c16 = lane & 15, g = lane >> 4;
    const int n_rep = a.n_heads / a.n_kv_heads;
    const int nq = n_rep * a.seq;  // <= NQ
    int wg = blockIdx.x;
    const int split = wg % a.nsplit;
    wg /= a.nsplit;
    const int hk = wg % a.n_kv_heads, b = wg / a.n_kv_heads;

    // this lane's query row (for the score columns): rep, token, position
    const bool q_live = c16 < nq;
    const int q_rep = q_live ? c16 / a.seq : 0, q_s = q_live ? c16 % a.seq : 0;
    int64_t q_pos, kmax = -1;
    [[maybe_unused]] const int* table = nullptr;
    if constexpr (PAGED) {
        const int64_t len = (int64_t)a.kv_indptr[b + 1] - a.kv_indptr[b];
        const int64_t req = a.req_pool_indices[b];
        const bool req_ok = req >= 0 && req < a.num_requests;  // a bad row reads as an empty sequence
        kmax = req_ok ? min(len, a.rtt_stride) - 1 : -1;
        q_pos = q_live ? kmax : -1;
        table = a.req_to_token + (req_ok ? req : 0) * a.rtt_stride;
    } else {
        q_pos = q_live ? a.positions[q_s] : -1;
        for (int s = 0; s < a.seq; ++s) kmax = max(kmax, (int64_t)a.positions[s]);
        kmax = min(kmax, (int64_t)a.max_len - 1);
    }
    const int tiles_total = (int)((kmax + 16) >> 4);  // keys 0..kmax
    const int tps = (tiles_total + a.nsplit - 1) / a.nsplit;
    const int t0 = split * tps, t1 = min(t0 + tps, tiles_total);

    // query operand: 4 steps x 16 bytes: dims 32*step + 8g .. +7 of query c16
    u32x4 qf[4];
    {
        const uint16_t* qrow = static_cast<const uint16_t*>(a.q) +
                               (((int64_t)b * a.n_heads + hk * n_rep + q_rep) * a.seq + q_s) * kD;
#pragma unroll
        for (int st = 0; st < 4; ++st)
            qf[st] = q_live ? *reinterpret_cast<const u32x4*>(qrow + 32 * st + 8 * g) : u32x4{0, 0, 0, 0};
    }
    const int64_t head_off = PAGED ? 0 : ((int64_t)b * a.n_kv_heads + hk) * a.max_len * kD;
    const uint32_t head_bytes = PAGED ? 0u : (uint32_t)a.max_len * kD * 2u;
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(static_cast<const uint16_t*>(a.k_cache) + head_off, head_bytes);
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(static_cast<const uint16_t*>(a.v_cache) + head_off, head_bytes);

    float m = kNegBig, l = 0.0f;  // of query c16, equal in its four lanes
    float acc[NQ][8];
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
        for (int d = 0; d < 8; ++d) acc[q][d] = 0.0f;

    // paged: slot of key 16t + c16, looked up one tile ahead of its use. -1: nothing is
    // fetched, key and value read as zeros; a position inside the sequence whose table
    // entry is negative ("empty padding") is still attended, with score 0, as in the
    // reference, which gates the load on the slot and the mask on the position only
    // (csrc/kernels/attention/layout_policies.cuh:104-110,212-219; decode_split_kv_mma.cuh:75-82,107-110)
    auto key_slot = [&](int t) -> int {
        const int key = (t << 4) + c16;
        const int slot = (t < t1 && key <= kmax) ? table[key] : -1;
        return slot < a.num_slots ? slot : -1;
    };
    [[maybe_unused]] int slot_next = -1;
    if constexpr (PAGED) slot_next = key_slot(t0 + wave);
    const int64_t pool_row = (int64_t)a.n_kv_heads * kD;  // elements from one slot to the next
    [[maybe_unused]] const uint8_t* mask_row = nullptr;
    if constexpr (MASK) mask_row = a.mask + (int64_t)b * a.mask_b_stride;

    for (int t = t0 + wave; t < t1; t += 4) {
        const int kb = t << 4;
        u32x4 kf[4], vf[4];
        [[maybe_unused]] uint8_t keep[4] = {1, 1, 1, 1};
        if constexpr (MASK) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = kb + 4 * g + i;
                keep[i] = key < a.mask_width ? mask_row[key] : (uint8_t)0;
            }
        }
        [[maybe_unused]] int vslot[4] = {0, 0, 0, 0};
        if constexpr (PAGED) {
            const int slot = slot_next;
            slot_next = key_slot(t + 4);
            const u32x4 zero = {0u, 0u, 0u, 0u};
            const uint16_t* kr = static_cast<const uint16_t*>(a.k_cache) +
                                 (int64_t)max(slot, 0) * pool_row + hk * kD + 8 * g;
#pragma unroll
            for (int st = 0; st < 4; ++st)
                kf[st] = slot >= 0 ? *reinterpret_cast<const u32x4*>(kr + 32 * st) : zero;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                vslot[i] = lane_read_i(slot, 4 * g + i);  // lanes 0..15 hold keys kb..kb+15
                const uint16_t* vr = static_cast<const uint16_t*>(a.v_cache) +
                                     (int64_t)max(vslot[i], 0) * pool_row + hk * kD + c16 * 8;
                vf[i] = vslot[i] >= 0 ? *reinterpret_cast<const u32x4*>(vr) : zero;
            }
        } else {
            // keys as MFMA rows: lane -> key kb + c16, dims 32*step + 8g. A dense cache row is read by
            // exactly one workgroup per step: loaded with the streaming hint (aux 2: not kept once
            // delivered), 0.56 us per layer at 32 x 4 heads x 530 keys; pool rows may be shared between
            // sequences and keep the default policy.
#pragma unroll
            for (int st = 0; st < 4; ++st)
                kf[st] = __builtin_amdgcn_raw_buffer_load_b128(rk, (uint32_t)(kb + c16) * (kD * 2) + (32 * st + 8 * g) * 2, 0, 2);
            // values: lane -> key kb + 4g + i, dims 8*c16
#pragma unroll
            for (int i = 0; i < 4; ++i)
                vf[i] = __builtin_amdgcn_raw_buffer_load_b128(rv, (uint32_t)(kb + 4 * g + i) * (kD * 2) + c16 * 16, 0, 2);
        }

        f32x4 sc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int st = 0; st < 4; ++st)
            sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf[st]),
                                                         __builtin_bit_cast(bf16x8, qf[st]), sc, 0, 0, 0);
        // sc[i] = q(c16) . k(kb + 4g + i)
        float tm = kNegBig;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            bool ok = q_live && (int64_t)(kb + 4 * g + i) <= q_pos;
            if constexpr (MASK) ok = ok && keep[i] != 0;
            sc[i] = ok ? sc[i] * a.scale : kNegBig;
            tm = fmaxf(tm, sc[i]);
        }
        tm = fmaxf(tm, __shfl_xor(tm, 16, kWave));
        tm = fmaxf(tm, __shfl_xor(tm, 32, kWave));
        const float m_new = fmaxf(m, tm);
        const float alpha = __expf(m - m_new);
        float p[4], ps = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            p[i] = (sc[i] > 0.5f * kNegBig) ? __expf(sc[i] - m_new) : 0.0f;
            ps += p[i];
        }
        ps += __shfl_xor(ps, 16, kWave);
        ps += __shfl_xor(ps, 32, kWave);
        l = l * alpha + ps;
        m = m_new;

        // P.V: this lane needs alpha and p[i] of query q from lane 16g + q
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const float aq = lane_read(alpha, 16 * g + q);
#pragma unroll
            for (int d = 0; d < 8; ++d) acc[q][d] *= aq;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // rows past the newest position were never written: keep them out even at p = 0
            if ((int64_t)(kb + 4 * g + i) > kmax) vf[i] = u32x4{0, 0, 0, 0};
            float v[8];
            v[0] = __uint_as_float(vf[i].x << 16); v[1] = __uint_as_float(vf[i].x & 0xffff0000u);
            v[2] = __uint_as_float(vf[i].y << 16); v[3] = __uint_as_float(vf[i].y & 0xffff0000u);
            v[4] = __uint_as_float(vf[i].z << 16); v[5] = __uint_as_float(vf[i].z & 0xffff0000u);
            v[6] = __uint_as_float(vf[i].w << 16); v[7] = __uint_as_float(vf[i].w & 0xffff0000u);
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                const float pq = lane_read(p[i], 16 * g + q);
#pragma unroll
                for (int d = 0; d < 8; ++d) acc[q][d] += pq * v[d];
            }
        }
    }

    // the four key groups of the wave hold sums over different keys: add them up
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            float v = acc[q][d];
            v += __shfl_xor(v, 16, kWave);
            v += __shfl_xor(v, 32, kWave);
            acc[q][d] = v;
        }
    if (g == 0) {
#pragma unroll
        for (int q = 0; q < NQ; ++q)
#pragma unroll
            for (int d = 0; d < 8; ++d) sh_acc[wave][q][c16 * 8 + d] = acc[q][d];
        if (c16 < NQ) {
            sh_ml[wave][c16][0] = m;
            sh_ml[wave][c16][1] = l;
        }
    }
    __syncthreads();
    // merge the four waves; thread -> (query, dim)
    float* ws = a.ws + (int64_t)blockIdx.x * NQ * kWsRow;
    for (int e = threadIdx.x; e < NQ * kD; e += 256) {
        const int q = e / kD, d = e - q * kD;
        float mm = kNegBig;
#pragma unroll
        for (int w = 0; w < 4; ++w) mm = fmaxf(mm, sh_ml[w][q][0]);
        float v = 0.0f, ll = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float f = __expf(sh_ml[w][q][0] - mm);
            v += sh_acc[w][q][d] * f;
            ll += sh_ml[w][q][1] * f;
        }
        ws[q * kWsRow + d] = v;
        if (d == 0) {
            ws[q * kWsRow + kD] = mm;
            ws[q * kWsRow + kD + 1] = ll;
        }
    }
}

// One workgroup per (batch, token): all heads, 8 output values per thread and
// pass. Besides (or instead of) the bf16 row it can emit the per-token int8
// quantization of that row -- the input of the int8 output projection -- computed
// on the bf16-rounded values, i.e. what the separate quantizer would produce.
constexpr int kMergeCache = 4;  // rows up to 4 * 256 * 8 = 8192 wide stay in registers

__device__ __forceinline__ float merge_block_max(float v, float* slots) {
    v = wave_max(v);
    if ((threadIdx.x & 63) == 0) slots[threadIdx.x >> 6] = v;
    __syncthreads();
    return fmaxf(fmaxf(slots[0], slots[1]), fmaxf(slots[2], slots[3]));
}

template <int NQ>
__global__ __launch_bounds__(256) void attn_decode_merge_kernel(AttnDecodeArgs a) {
    __shared__ float slots[4];
    const int n_rep = a.n_heads / a.n_kv_heads;
    const int b = blockIdx.x / a.seq, s = blockIdx.x % a.seq;
    const int width = a.n_heads * kD;
    float keep[kMergeCache][8];
    float local = 0.0f;
#pragma unroll
    for (int c = 0; c < kMergeCache; ++c) {
        const int e = (threadIdx.x + c * 256) * 8;
        if (e >= width) break;
        const int h = e / kD, d0 = e - h * kD;
        const int hk = h / n_rep, q = (h - hk * n_rep) * a.seq + s;
        const float* base = a.ws + ((int64_t)(b * a.n_kv_heads + hk) * a.nsplit) * NQ * kWsRow + q * kWsRow;
        float mm = kNegBig;
        for (int j = 0; j < a.nsplit; ++j) mm = fmaxf(mm, base[(int64_t)j * NQ * kWsRow + kD]);
        float v[8] = {0, 0, 0, 0, 0, 0, 0, 0}, ll = 0.0f;
        for (int j = 0; j < a.nsplit; ++j) {
            const float* r = base + (int64_t)j * NQ * kWsRow;
            const float f = __expf(r[kD] - mm);
            ll += r[kD + 1] * f;
#pragma unroll
            for (int d = 0; d < 8; ++d) v[d] += r[d0 + d] * f;
        }
        const float inv = ll > 0.0f ? 1.0f / ll : 0.0f;  // a token with no visible key yields zeros
        u32x4 o;
        o.x = pack_bf16x2(v[0] * inv, v[1] * inv);
        o.y = pack_bf16x2(v[2] * inv, v[3] * inv);
        o.z = pack_bf16x2(v[4] * inv, v[5] * inv);
        o.w = pack_bf16x2(v[6] * inv, v[7] * inv);
        if (a.out) *reinterpret_cast<u32x4*>(static_cast<uint16_t*>(a.out) + (int64_t)blockIdx.x * width + e) = o;
        keep[c][0] = __uint_as_float(o.x << 16); keep[c][1] = __uint_as_float(o.x & 0xffff0000u);
        keep[c][2] = __uint_as_float(o.y << 16); keep[c][3] = __uint_as_float(o.y & 0xffff0000u);
        keep[c][4] = __uint_as_float(o.z << 16); keep[c][5] = __uint_as_float(o.z & 0xffff0000u);
        keep[c][6] = __uint_as_float(o.w << 16); keep[c][7] = __uint_as_float(o.w & 0xffff0000u);
#pragma unroll
        for (int d = 0; d < 8; ++d) local = fmaxf(local, fabsf(keep[c][d]));
    }
    if (!a.out_q) return;
    // per-token int8: step = max(amax, 1e-12) / 127, round half to even, clamp
    const float step = fmaxf(merge_block_max(local, slots), 1e-12f) / 127.0f;
    if (threadIdx.x == 0) a.out_scale[blockIdx.x] = step;
#pragma unroll
    for (int c = 0; c < kMergeCache; ++c) {
        const int e = (threadIdx.x + c * 256) * 8;
        if (e >= width) break;
        uint32_t w[2] = {0u, 0u};
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            float qv = rintf(keep[c][d] / step);
            qv = fminf(fmaxf(qv, -127.0f), 127.0f);
            w[d >> 2] |= ((uint32_t)(int)qv & 0xffu) << (8 * (d & 3));
        }
        u32x2 pk;
        pk.x = w[0];
        pk.y = w[1];
        *reinterpret_cast<u32x2*>(static_cast<int8_t*>(a.out_q) + (int64_t)blockIdx.x * width + e) = pk;
    }
}

}  // namespace

int64_t attn_decode_workspace_floats(int batch, int n_kv_heads, int nsplit, int nq) {
    const int NQ = nq <= 4 ? 4 : 8;
    return (int64_t)batch * n_kv_heads * nsplit * NQ * kWsRow;
}

bool launch_attn_decode(const AttnDecodeArgs& a, hipStream_t stream) {
    const int n_rep = a.n_heads / a.n_kv_heads;
    const int nq = n_rep * a.seq;
    if (a.head_dim != kD || nq > 8 || nq <= 0 || a.nsplit <= 0) return false;
    if (a.n_heads * kD > kMergeCache * 256 * 8) return false;  // the merge kernel keeps a token's row in registers
    const unsigned grid1 = (unsigned)(a.batch * a.n_kv_heads * a.nsplit);
    const unsigned grid2 = (unsigned)(a.batch * a.seq);
    const bool paged = a.req_to_token != nullptr;
    if (paged && (a.seq != 1 || !a.req_pool_indices || !a.kv_indptr || a.rtt_stride <= 0)) return false;
    if (a.mask && (!paged || a.mask_width <= 0)) return false;
    if (nq <= 4) {
        if (paged && a.mask)
            attn_decode_partial_kernel<4, true, true><<<dim3(grid1), dim3(256), 0, stream>>>(a);
        else if (paged)
            attn_decode_partial_kernel<4, true><<<dim3(grid1), dim3(256), 0, stream>>>(a);
        else
            attn_decode_partial_kernel<4, false><<<dim3(grid1), dim3(256), 0, stream>>>(a);
        attn_decode_merge_kernel<4><<<dim3(grid2), dim3(256), 0, stream>>>(a);
    } else {
        if (paged && a.mask)
            attn_decode_partial_kernel<8, true, true><<<dim3(grid1), dim3(256), 0, stream>>>(a);
        else if (paged)
            attn_decode_partial_kernel<8, true><<<dim3(grid1), dim3(256), 0, stream>>>(a);
        else
            attn_decode_partial_kernel<8, false><<<dim3(grid1), dim3(256), 0, stream>>>(a);
        attn_decode_merge_kernel<8><<<dim3(grid2), dim3(256), 0, stream>>>(a);
    }
    return true;
}

}  // namespace w8a8
