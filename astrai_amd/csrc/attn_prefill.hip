// Causal grouped-query attention of a block of new tokens against the dense bf16
// KV cache (prefill, chunked or whole), head_dim 128, bf16 MFMAs, fp32 softmax.
//
// The reference expands the KV heads and calls SDPA on [batch, heads, seq, head_dim]
// tensors with a mask tensor (astrai/extension/backend/attention.py:244-253,443-498,
// cached branch of astrai/model/components/attention.py:19-85). Here the mask is
// `key <= position` computed in the kernel, key blocks wholly above a query block
// are never visited, the n_rep query heads of a KV group share every key/value tile,
// and the output is written token-major [batch, seq, heads*head_dim], the layout the
// output projection reads.
//
// One workgroup per (batch, KV head, 32 query tokens); wave r takes query head
// hk*n_rep + r. Per 64-key block:
//   S^T = K.Q^T on v_mfma_f32_32x32x16_bf16 with keys as rows and queries as columns,
//     so a lane owns ONE query (column lane%32) and 2x16 of its 64 scores: row maxima
//     and sums are per-lane reductions plus one exchange with lane^32;
//   O^T += V^T.P^T with the same instruction: P^T is the S^T accumulator itself,
//     rounded to bf16 in place (its register order fixes which 8 keys a lane half
//     contributes per 16-key step), and V^T comes from LDS, where the value tile is
//     stored transposed with its key slots permuted to that order, 136-byte rows
//     (conflict-free for the transposing 4-byte writes and the 16-byte operand reads);
//   keys sit in LDS as 256-byte rows of 16-byte chunks XOR-swizzled by row.
// The next block's keys and values are fetched from the cache into registers while
// the current block is multiplied.
#include <climits>

#include "common.cuh"
#include "launchers.h"

namespace w8a8 {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kD = 128;    // head_dim
constexpr int kQB = 32;    // query tokens per workgroup
constexpr int kKB = 64;    // keys per block
constexpr int kKRow = 256;                 // bytes per key row in LDS
constexpr int kVtRow = 136;                // bytes per value-dim row of V^T in LDS
constexpr int kKBytes = kKB * kKRow;       // 16 KiB
constexpr int kVtBytes = kD * kVtRow;      // 17 KiB
constexpr float kNegBig = -1e30f;          // finite stand-in for -inf: no inf - inf

// slot of key w (0..31 within a 32-key tile) in a V^T row: the S^T accumulator of
// lane half h holds keys 8g' + 4h + j at register 4g' + j; a 16-key MFMA step t takes
// registers 8t..8t+7, i.e. keys 16t + 8g + 4h + j (g = 0,1) as its k-index 8h + 4g + j.
__device__ __forceinline__ int vt_slot(int w) {
    return (w & 16) | ((w & 4) << 1) | ((w & 8) >> 1) | (w & 3);
}

template <int NREP>
__global__ __launch_bounds__(64 * NREP, 2) void attn_prefill_kernel(AttnPrefillArgs a) {
    constexpr int THREADS = 64 * NREP;
    constexpr int K_ITEMS = kKB * 16 / THREADS;        // 16-byte key chunks per thread
    constexpr int V_ITEMS = (kKB / 2) * 16 / THREADS;  // (key pair, 8-dim chunk) items per thread
    __shared__ __attribute__((aligned(16))) uint8_t lds[kKBytes + kVtBytes];
    uint8_t* const ks_lds = lds;
    uint8_t* const vt_lds = lds + kKBytes;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int qi = lane & 31, h = lane >> 5;
    const int nqb = (a.seq + kQB - 1) / kQB;
    const int groups = a.batch * a.n_kv_heads;
    const int qb = nqb - 1 - (int)(blockIdx.x / groups);  // longest key ranges first
    const int bk = (int)(blockIdx.x % groups);
    const int b = bk / a.n_kv_heads, hk = bk % a.n_kv_heads;
    const int head = hk * NREP + wave;

    // this lane's query token and what it may see
    const int s_row = qb * kQB + qi;
    const bool row_live = s_row < a.seq;
    int pq = row_live ? (int)a.positions[s_row] : -1;
    int kmax = pq, pmin = row_live ? pq : INT_MAX;
#pragma unroll
    for (int off = 16; off; off >>= 1) {
        kmax = max(kmax, __shfl_xor(kmax, off, kWave));
        pmin = min(pmin, __shfl_xor(pmin, off, kWave));
    }
    kmax = min(kmax, (int)a.max_len - 1);
    if (!row_live) pq = kmax;  // rows past the end see everything and are never stored
    const int nkb = kmax / kKB + 1;

    const uint16_t* qrow = static_cast<const uint16_t*>(a.q) +
        (((size_t)b * a.n_heads + head) * a.seq + min(s_row, a.seq - 1)) * kD;
    u32x4 qf[8];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qf[ks] = *reinterpret_cast<const u32x4*>(qrow + ks * 16 + h * 8);

    const size_t cache_off = ((size_t)b * a.n_kv_heads + hk) * (size_t)a.max_len * kD;
    const uint16_t* kc = static_cast<const uint16_t*>(a.k_cache) + cache_off;
    const uint16_t* vc = static_cast<const uint16_t*>(a.v_cache) + cache_off;

    u32x4 kreg[K_ITEMS], vreg[V_ITEMS][2];
    auto fetch = [&](int kb) {
        const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < K_ITEMS; ++i) {
            const int item = tid + i * THREADS;
            const int key = kb * kKB + (item >> 4);
            kreg[i] = key <= kmax
                ? *reinterpret_cast<const u32x4*>(kc + (size_t)key * kD + (item & 15) * 8) : zero;
        }
#pragma unroll
        for (int i = 0; i < V_ITEMS; ++i) {
            const int item = tid + i * THREADS;
            const int chunk = ((item >> 7) << 2) | (item & 3);
            const int key = kb * kKB + 2 * ((item >> 2) & 31);
            const uint16_t* src = vc + (size_t)key * kD + chunk * 8;
            // keys past kmax may never have been written: they must not reach P.V as 0 * garbage
            vreg[i][0] = key <= kmax ? *reinterpret_cast<const u32x4*>(src) : zero;
            vreg[i][1] = key + 1 <= kmax ? *reinterpret_cast<const u32x4*>(src + kD) : zero;
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < K_ITEMS; ++i) {
            const int item = tid + i * THREADS;
            const int row = item >> 4, chunk = item & 15;
            *reinterpret_cast<u32x4*>(ks_lds + row * kKRow + ((chunk ^ (row & 15)) << 4)) = kreg[i];
        }
#pragma unroll
        for (int i = 0; i < V_ITEMS; ++i) {
            const int item = tid + i * THREADS;
            const int chunk = ((item >> 7) << 2) | (item & 3);
            const int w = 2 * ((item >> 2) & 31);  // even key of the pair within the block
            uint8_t* dst = vt_lds + (chunk * 8) * kVtRow + ((w & 32) + vt_slot(w & 31)) * 2;
            const uint32_t lo[4] = {vreg[i][0].x, vreg[i][0].y, vreg[i][0].z, vreg[i][0].w};
            const uint32_t hi[4] = {vreg[i][1].x, vreg[i][1].y, vreg[i][1].z, vreg[i][1].w};
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                // dims 2p and 2p+1 of the chunk: (key w, key w+1) side by side
                *reinterpret_cast<uint32_t*>(dst + (2 * p) * kVtRow) = (lo[p] & 0xffffu) | (hi[p] << 16);
                *reinterpret_cast<uint32_t*>(dst + (2 * p + 1) * kVtRow) = (lo[p] >> 16) | (hi[p] & 0xffff0000u);
            }
        }
    };

    f32x16 o[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[dt][e] = 0.0f;
    float m_run = kNegBig, l_run = 0.0f;
    const float c = a.scale * 1.44269504088896340736f;  // scores in log2 units

    fetch(0);
    for (int kb = 0; kb < nkb; ++kb) {
        __syncthreads();  // every wave is done reading the previous block
        stage();
        __syncthreads();
        if (kb + 1 < nkb) fetch(kb + 1);

        // ---- S^T = K.Q^T for two 32-key tiles
        f32x16 s[2];
#pragma unroll
        for (int ti = 0; ti < 2; ++ti)
#pragma unroll
            for (int e = 0; e < 16; ++e) s[ti][e] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
#pragma unroll
            for (int ti = 0; ti < 2; ++ti) {
                const int row = ti * 32 + qi;
                const u32x4 kf = *reinterpret_cast<const u32x4*>(
                    ks_lds + row * kKRow + (((2 * ks + h) ^ (row & 15)) << 4));
                s[ti] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                    __builtin_bit_cast(bf16x8, kf), __builtin_bit_cast(bf16x8, qf[ks]), s[ti], 0, 0, 0);
            }

        // ---- online softmax for this lane's query
        const bool need_mask = kb * kKB + kKB - 1 > pmin;  // uniform over the wave
        float m_loc = kNegBig;
#pragma unroll
        for (int ti = 0; ti < 2; ++ti)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                float v = s[ti][e] * c;
                if (need_mask) {
                    const int key = kb * kKB + ti * 32 + (e >> 2) * 8 + h * 4 + (e & 3);
                    v = key <= pq ? v : kNegBig;
                }
                s[ti][e] = v;
                m_loc = fmaxf(m_loc, v);
            }
        m_loc = fmaxf(m_loc, __shfl_xor(m_loc, 32, kWave));
        const float m_new = fmaxf(m_run, m_loc);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        float l_add = 0.0f;
        uint32_t pk[2][8];
#pragma unroll
        for (int ti = 0; ti < 2; ++ti)
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
                const float p0 = __builtin_amdgcn_exp2f(s[ti][e] - m_new);
                const float p1 = __builtin_amdgcn_exp2f(s[ti][e + 1] - m_new);
                l_add += p0 + p1;
                pk[ti][e >> 1] = pack_bf16x2(p0, p1);
            }
        l_run = l_run * alpha + l_add;
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                for (int e = 0; e < 16; ++e) o[dt][e] *= alpha;
        }

        // ---- O^T += V^T.P^T, four 16-key steps x four 32-dim tiles
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            const int ti = st >> 1, t = st & 1;
            const u32x4 pf = {pk[ti][4 * t], pk[ti][4 * t + 1], pk[ti][4 * t + 2], pk[ti][4 * t + 3]};
#pragma unroll
            for (int dt = 0; dt < 4; ++dt) {
                const uint8_t* src = vt_lds + (dt * 32 + qi) * kVtRow + ti * 64 + t * 32 + h * 16;
                const u32x2 v0 = *reinterpret_cast<const u32x2*>(src);
                const u32x2 v1 = *reinterpret_cast<const u32x2*>(src + 8);
                const u32x4 vf = {v0.x, v0.y, v1.x, v1.y};
                o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                    __builtin_bit_cast(bf16x8, vf), __builtin_bit_cast(bf16x8, pf), o[dt], 0, 0, 0);
            }
        }
    }

    // ---- normalise and write [batch, seq, heads*128]
    l_run += __shfl_xor(l_run, 32, kWave);
    const float inv = 1.0f / l_run;
    if (row_live) {
        uint16_t* orow = static_cast<uint16_t*>(a.out) +
            (((size_t)b * a.seq + s_row) * a.n_heads + head) * kD;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                u32x2 w;
                w.x = pack_bf16x2(o[dt][4 * g] * inv, o[dt][4 * g + 1] * inv);
                w.y = pack_bf16x2(o[dt][4 * g + 2] * inv, o[dt][4 * g + 3] * inv);
                *reinterpret_cast<u32x2*>(orow + dt * 32 + g * 8 + h * 4) = w;
            }
    }
}

}  // namespace

bool attn_prefill_supported(int n_heads, int n_kv_heads, int head_dim) {
    if (head_dim != kD || n_kv_heads <= 0 || n_heads % n_kv_heads) return false;
    const int n_rep = n_heads / n_kv_heads;
    return n_rep == 2 || n_rep == 4 || n_rep == 8;
}

bool launch_attn_prefill(const AttnPrefillArgs& a, hipStream_t stream) {
    if (!attn_prefill_supported(a.n_heads, a.n_kv_heads, a.head_dim)) return false;
    if (a.batch <= 0 || a.seq <= 0 || a.max_len <= 0) return false;
    const int n_rep = a.n_heads / a.n_kv_heads;
    const int64_t wgs = (int64_t)((a.seq + kQB - 1) / kQB) * a.batch * a.n_kv_heads;
    if (wgs > INT_MAX) return false;
    const dim3 grid((unsigned)wgs);
    if (n_rep == 2)
        attn_prefill_kernel<2><<<grid, dim3(128), 0, stream>>>(a);
    else if (n_rep == 4)
        attn_prefill_kernel<4><<<grid, dim3(256), 0, stream>>>(a);
    else
        attn_prefill_kernel<8><<<grid, dim3(512), 0, stream>>>(a);
    return true;
}

}  // namespace w8a8
