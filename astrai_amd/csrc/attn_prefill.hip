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
// Two LDS buffers: while a block is multiplied, the next one arrives (keys by
// direct-to-LDS loads, values through registers) and the values of the one after are
// requested; one barrier per block. Blocks that every query of the wave sees whole skip the masking code.
#include <climits>
#include <type_traits>

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
constexpr int kBufBytes = kKBytes + kVtBytes;
constexpr float kNegBig = -1e30f;          // finite stand-in for -inf: no inf - inf

// slot of key w (0..31 within a 32-key tile) in a V^T row: the S^T accumulator of
// lane half h holds keys 8g' + 4h + j at register 4g' + j; a 16-key MFMA step t takes
// registers 8t..8t+7, i.e. keys 16t + 8g + 4h + j (g = 0,1) as its k-index 8h + 4g + j.
__device__ __forceinline__ void lds_dma16(__amdgpu_buffer_rsrc_t r, uint8_t* lds_wave_base,
                                          uint32_t voff, uint32_t soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        r, (__attribute__((address_space(3))) void*)lds_wave_base, 16, voff, soff, 0, 0);
}

__device__ __forceinline__ int vt_slot(int w) {
    return (w & 16) | ((w & 4) << 1) | ((w & 8) >> 1) | (w & 3);
}

template <int NREP>
__global__ __launch_bounds__(64 * NREP, NREP >= 4 ? 2 : 1) void attn_prefill_kernel(AttnPrefillArgs a) {
    constexpr int THREADS = 64 * NREP;
    constexpr int K_DMA = kKB / 4 / NREP;              // 1 KiB key loads per wave and block
    constexpr int V_ITEMS = (kKB / 2) * 16 / THREADS;  // (key pair, 8-dim chunk) items per thread
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * kBufBytes];

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

    // keys: straight from the cache into LDS, 1 KiB (four rows) per instruction; lane l
    // lands at row l/16, chunk position l%16 and therefore asks for chunk (l%16) ^ (row%16).
    // The descriptor ends after key kmax: later rows arrive as zeros.
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(kc, (uint32_t)(kmax + 1) * (uint32_t)kKRow);
    uint32_t k_voff[K_DMA];
#pragma unroll
    for (int j = 0; j < K_DMA; ++j) {
        const int row = (wave * K_DMA + j) * 4 + (lane >> 4);
        k_voff[j] = (uint32_t)row * kKRow + (uint32_t)(((lane & 15) ^ (row & 15)) << 4);
    }
    auto dma_k = [&](int kb, int buf) {
#pragma unroll
        for (int j = 0; j < K_DMA; ++j)
            lds_dma16(rk, lds + buf * kBufBytes + (wave * K_DMA + j) * 4 * kKRow,
                      k_voff[j] + (uint32_t)kb * (kKB * kKRow), 0);
    };
    // values: through registers, because they are stored transposed
    u32x4 vreg[V_ITEMS][2];
    auto fetch_v = [&](int kb) {
        const u32x4 zero = {0u, 0u, 0u, 0u};
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
    auto stage_v = [&](int buf) {
        uint8_t* const vt_lds = lds + buf * kBufBytes + kKBytes;
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
                // dims 2p and 2p+1 of the chunk: (key w, key w+1) side by side, one byte permute each
                *reinterpret_cast<uint32_t*>(dst + (2 * p) * kVtRow) =
                    __builtin_amdgcn_perm(hi[p], lo[p], 0x05040100u);
                *reinterpret_cast<uint32_t*>(dst + (2 * p + 1) * kVtRow) =
                    __builtin_amdgcn_perm(hi[p], lo[p], 0x07060302u);
            }
        }
    };

    f32x16 o[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[dt][e] = 0.0f;
    // m_run is the reference maximum the probabilities are taken against, in log2 units.
    // It follows the true running maximum lazily: only when some query of the wave has
    // outgrown it by more than kSlack does the wave pay for rescaling its 64 accumulators;
    // until then probabilities may reach 2^kSlack, which fp32 sums and bf16 operands hold.
    constexpr float kSlack = 8.0f;
    float m_run = kNegBig, l_run = 0.0f;
    const float c = a.scale * 1.44269504088896340736f;  // scores to log2 units

    // one 64-key block out of LDS buffer `buf`; MASK: some key of it lies past some query
    auto block = [&](auto mask_tag, int kb, const uint8_t* kbuf, const uint8_t* vbuf) {
        constexpr bool MASK = decltype(mask_tag)::value;
        // ---- S^T = K.Q^T for two 32-key tiles
        f32x16 s[2];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
#pragma unroll
            for (int ti = 0; ti < 2; ++ti) {
                const int row = ti * 32 + qi;
                const u32x4 kf = *reinterpret_cast<const u32x4*>(
                    kbuf + row * kKRow + (((2 * ks + h) ^ (row & 15)) << 4));
                if (ks == 0) {
                    const f32x16 zero = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f,
                                         0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
                    s[ti] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(bf16x8, kf), __builtin_bit_cast(bf16x8, qf[ks]), zero, 0, 0, 0);
                } else {
                    s[ti] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(bf16x8, kf), __builtin_bit_cast(bf16x8, qf[ks]), s[ti], 0, 0, 0);
                }
            }

        // ---- online softmax for this lane's query (raw scores; c > 0 keeps their order)
        float m_loc = kNegBig;
#pragma unroll
        for (int ti = 0; ti < 2; ++ti)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                if (MASK) {
                    const int key = kb * kKB + ti * 32 + (e >> 2) * 8 + h * 4 + (e & 3);
                    s[ti][e] = key <= pq ? s[ti][e] : kNegBig;
                }
                m_loc = fmaxf(m_loc, s[ti][e]);
            }
        m_loc = fmaxf(m_loc, __shfl_xor(m_loc, 32, kWave)) * c;
        if (__any(m_loc > m_run + kSlack)) {
            const float m_new = fmaxf(m_run, m_loc);
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                for (int e = 0; e < 16; ++e) o[dt][e] *= alpha;
        }
        float l_add = 0.0f;
        uint32_t pk[2][8];
#pragma unroll
        for (int ti = 0; ti < 2; ++ti)
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
                const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[ti][e], c, -m_run));
                const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[ti][e + 1], c, -m_run));
                l_add += p0 + p1;
                pk[ti][e >> 1] = pack_bf16x2(p0, p1);
            }
        l_run += l_add;

        // ---- O^T += V^T.P^T, four 16-key steps x four 32-dim tiles
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            const int ti = st >> 1, t = st & 1;
            const u32x4 pf = {pk[ti][4 * t], pk[ti][4 * t + 1], pk[ti][4 * t + 2], pk[ti][4 * t + 3]};
#pragma unroll
            for (int dt = 0; dt < 4; ++dt) {
                const uint8_t* src = vbuf + (dt * 32 + qi) * kVtRow + ti * 64 + t * 32 + h * 16;
                const u32x2 v0 = *reinterpret_cast<const u32x2*>(src);
                const u32x2 v1 = *reinterpret_cast<const u32x2*>(src + 8);
                const u32x4 vf = {v0.x, v0.y, v1.x, v1.y};
                o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                    __builtin_bit_cast(bf16x8, vf), __builtin_bit_cast(bf16x8, pf), o[dt], 0, 0, 0);
            }
        }
    };

    // Two LDS buffers: while block kb is multiplied out of one, block kb+1 goes into the
    // other (keys by DMA, values from the registers filled an iteration earlier) and the
    // values of block kb+2 are requested; one barrier per block.
    const int nfull = min(nkb, (__builtin_amdgcn_readfirstlane(pmin) + 1) / kKB);  // blocks every query sees whole
    dma_k(0, 0);
    fetch_v(0);
    stage_v(0);
    if (nkb > 1) fetch_v(1);
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0): the DMA has landed
    __syncthreads();
    for (int kb = 0; kb < nkb; ++kb) {
        const int cur = kb & 1;
        if (kb + 1 < nkb) {
            dma_k(kb + 1, cur ^ 1);
            stage_v(cur ^ 1);
        }
        if (kb + 2 < nkb) fetch_v(kb + 2);
        const uint8_t* kbuf = lds + cur * kBufBytes;
        if (kb < nfull)
            block(std::false_type{}, kb, kbuf, kbuf + kKBytes);
        else
            block(std::true_type{}, kb, kbuf, kbuf + kKBytes);
        __builtin_amdgcn_s_waitcnt(0x0070);
        __syncthreads();
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
