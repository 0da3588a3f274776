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
// hk*n_rep + r. Keys are handled in 32-key tiles:
//   S^T = K.Q^T on v_mfma_f32_32x32x16_bf16 with keys as rows and queries as columns,
//     so a lane owns ONE query (column lane%32) and 16 of a tile's 32 scores: row maxima
//     and sums are per-lane reductions plus one exchange with lane^32;
//   O^T += V^T.P^T with the same instruction: P^T is the S^T accumulator itself,
//     rounded to bf16 in place (its register order fixes which 8 keys a lane half
//     contributes per 16-key step), and the V^T operand is read out of the row-major
//     value tile with ds_read_b64_tr_b16, the LDS read that hands each lane of a
//     16-lane group four values down a column (four keys of one dim);
//   keys and values sit in LDS as 256-byte rows of 16-byte chunks XOR-swizzled by row
//     (keys by row%16 for the 32-row operand reads, values by 4*(row%4) for the
//     transposing reads, which touch four consecutive rows at a time).
// A wave's instruction stream is a software pipeline over tiles, written out and
// pinned with sched_barrier: the eight score MFMAs of tile T+1 are interleaved with
// the exponentials of tile T, and the eight P.V MFMAs of tile T with the masking and
// row maximum of tile T+1, so the matrix pipe and the vector ALU work at the same
// time inside one wave (a wave issues in order: a softmax phase between two MFMA
// phases leaves each unit idle while the other runs). Keys and values arrive by
// direct-to-LDS loads, keys into a ring of four tiles, values into two 64-key buffers,
// both one 64-key block ahead; one workgroup barrier per block; no staging registers. Tiles that every
// query of the wave sees whole skip the masking code; the accumulators are rescaled
// only when a row maximum has outgrown the reference maximum by 2^8.
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
constexpr int kKTileBytes = 32 * kKRow;    // 8 KiB: one 32-key tile
constexpr int kKRingBytes = 4 * kKTileBytes;
constexpr int kVBytes = kKB * kKRow;        // 16 KiB: 64 value rows
constexpr float kNegBig = -1e30f;          // finite stand-in for -inf: no inf - inf

typedef short i16x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void lds_dma16(__amdgpu_buffer_rsrc_t r, uint8_t* lds_wave_base,
                                          uint32_t voff, uint32_t soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        r, (__attribute__((address_space(3))) void*)lds_wave_base, 16, voff, soff, 0, 0);
}

// PAGED: the queries are packed [total_q, heads, 128] with per-request row ranges
// (qo_indptr), the caches are token-granular pools [slots, kv_heads, 128] reached through
// req_to_token, and a 64-row query tile t of the caller's schedule belongs to request
// q_tile_to_batch[t], rows 64 * q_tile_to_index[t] .. of it (csrc/kernels/attention/
// paged_prefill.cu:4-34, layout_policies.cuh:67-93,174-232; the schedule is built in
// astrai/inference/cache/pool.py:219-234). Two workgroups share a tile. Query row i of a
// request of q_len rows and kv_len keys sees keys 0 .. kv_len - q_len + i (all of them
// without the causal flag), so nothing has to be fetched to know the key range.
// MASK (paged only): a bool tensor says, per sequence, (head,) (query row,) and position,
// what may be attended on top of the causal range (csrc/kernels/attention/mma_utils.cuh:190-199);
// every tile then takes the masking path.
template <int NREP, bool PAGED, bool MASK = false>
__global__ __launch_bounds__(64 * NREP, NREP >= 4 ? 2 : 1) void attn_prefill_kernel(AttnPrefillArgs a) {
    constexpr int K_DMA = kKB / 4 / NREP;              // 1 KiB key loads per wave and block
    __shared__ __attribute__((aligned(16))) uint8_t lds[kKRingBytes + 2 * kVBytes];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int qi = lane & 31, h = lane >> 5;

    int hk, rows_total, row0;   // KV head; query rows of the sequence; first row of this block
    int64_t tok0;               // index of row 0 of the sequence in the token-major output
    const uint16_t* qbase;      // row 0 of the sequence, this wave's head
    int64_t q_row_stride;       // elements between consecutive query rows
    int pq, kmax, pmin;         // this lane's newest visible key; the block's extremes
    [[maybe_unused]] const int* table = nullptr;
    [[maybe_unused]] int kv_len = 0, b_dense = 0, seq_index = 0;
    if constexpr (PAGED) {
        const int idx = (int)blockIdx.x;
        hk = idx % a.n_kv_heads;
        const int sub = (idx / a.n_kv_heads) & 1, tile = idx / (2 * a.n_kv_heads);
        const int req_i = a.q_tile_to_batch[tile];
        seq_index = req_i;
        const int q_start = a.qo_indptr[req_i];
        rows_total = a.qo_indptr[req_i + 1] - q_start;
        row0 = a.q_tile_to_index[tile] * 64 + sub * kQB;
        if (row0 >= rows_total) return;  // the tile's second half lies past the request
        const int64_t req = a.req_pool_indices[req_i];
        const bool req_ok = req >= 0 && req < a.num_requests;  // a bad row reads as an empty sequence
        kv_len = req_ok ? (int)min((int64_t)(a.kv_indptr[req_i + 1] - a.kv_indptr[req_i]), a.rtt_stride) : 0;
        table = a.req_to_token + (req_ok ? req : 0) * a.rtt_stride;
        tok0 = q_start;
        q_row_stride = (int64_t)a.n_heads * kD;
        qbase = static_cast<const uint16_t*>(a.q) + ((int64_t)q_start * a.n_heads + hk * NREP + wave) * kD;
        const int last = min(row0 + kQB, rows_total) - 1;
        const int shift = a.causal ? kv_len - rows_total : INT_MIN;
        pq = a.causal ? min(shift + row0 + qi, kv_len - 1) : kv_len - 1;
        kmax = a.causal ? min(shift + last, kv_len - 1) : kv_len - 1;
        pmin = a.causal ? min(shift + row0, kv_len - 1) : kv_len - 1;
    } else {
        const int nqb = (a.seq + kQB - 1) / kQB;
        const int groups = a.batch * a.n_kv_heads;
        const int qb = nqb - 1 - (int)(blockIdx.x / groups);  // longest key ranges first
        const int bk = (int)(blockIdx.x % groups);
        const int b = bk / a.n_kv_heads;
        b_dense = b;
        hk = bk % a.n_kv_heads;
        rows_total = a.seq;
        row0 = qb * kQB;
        tok0 = (int64_t)b * a.seq;
        q_row_stride = kD;
        qbase = static_cast<const uint16_t*>(a.q) + ((int64_t)b * a.n_heads + hk * NREP + wave) * a.seq * kD;
        // The position is requested first and looked at last: the query rows and the first
        // key tiles do not depend on it.
        pq = row0 + qi < a.seq ? (int)a.positions[row0 + qi] : -1;
        kmax = pmin = 0;
    }
    const int head = hk * NREP + wave;
    const int s_row = row0 + qi;
    const bool row_live = s_row < rows_total;
    // this lane's row of the mask and how many of its positions the mask covers (none for a
    // query row the mask has no row for: nothing is read there and nothing attended)
    [[maybe_unused]] const uint8_t* mask_row = nullptr;
    [[maybe_unused]] int mask_keys = 0;
    if constexpr (MASK) {
        const bool covered = row_live && (a.mask_l_stride == 0 || s_row < a.mask_rows);
        mask_row = a.mask + (int64_t)seq_index * a.mask_b_stride + (int64_t)head * a.mask_h_stride +
                   (int64_t)(covered ? s_row : 0) * a.mask_l_stride;
        mask_keys = covered ? a.mask_width : 0;
    }

    const uint16_t* qrow = qbase + (int64_t)min(s_row, rows_total - 1) * q_row_stride;
    u32x4 qf[8];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qf[ks] = *reinterpret_cast<const u32x4*>(qrow + ks * 16 + h * 8);

    // keys: straight from the cache into LDS, 1 KiB (four rows) per instruction; lane l
    // lands at row l/16, chunk position l%16 and therefore asks for chunk (l%16) ^ (row%16).
    // Dense cache: the descriptor covers the whole row range of this (batch, KV head):
    // whatever a row past the newest position holds, its scores are replaced (not scaled)
    // by the mask. Paged: the descriptor covers the pool and each lane looks up the slot of
    // its row; rows past the sequence ask for an offset outside it and arrive as zeros.
    const int64_t pool_row = (int64_t)a.n_kv_heads * kKRow;  // bytes from one slot to the next
    const size_t cache_off = PAGED ? (size_t)hk * kD
                                   : ((size_t)b_dense * a.n_kv_heads + hk) * (size_t)a.max_len * kD;
    const uint16_t* kc = static_cast<const uint16_t*>(a.k_cache) + cache_off;
    const uint16_t* vc = static_cast<const uint16_t*>(a.v_cache) + cache_off;
    const uint32_t pool_bytes = PAGED ? (uint32_t)(a.num_slots * pool_row - hk * kKRow) : 0u;
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(kc, PAGED ? pool_bytes : (uint32_t)a.max_len * (uint32_t)kKRow);
    // Paged: one load per wave fetches the slots of all rows its next loads cover (lane l <
    // RPW: this wave's l-th key row; the next RPW lanes: its value rows); the loads take each
    // row's slot from the lane that holds it. Looked up one block ahead, so that the table
    // access is not a second memory round trip in front of every load.
    constexpr int RPW = 4 * K_DMA;  // rows of a 64-row block that this wave loads
    auto lookup = [&](int t0, int kbv) -> int {
        const int l = lane & (2 * RPW - 1);  // (lanes past 2 RPW repeat the pattern, unused)
        const int key = l < RPW ? t0 * 32 + wave * RPW + l : kbv * kKB + wave * RPW + (l - RPW);
        int slot = (key <= kmax) ? table[key] : -1;
        return slot < a.num_slots ? slot : -1;
    };
    auto paged_off = [&](int slots, int src_lane, int swz) -> uint32_t {
        const int slot = __builtin_amdgcn_ds_bpermute(src_lane << 2, slots);
        return slot >= 0 ? (uint32_t)(slot * pool_row) + (uint32_t)(((lane & 15) ^ swz) << 4) : kOutOfRange;
    };
    [[maybe_unused]] uint32_t k_voff[K_DMA];
    if constexpr (!PAGED) {
#pragma unroll
        for (int j = 0; j < K_DMA; ++j) {
            const int row = (wave * K_DMA + j) * 4 + (lane >> 4);
            k_voff[j] = (uint32_t)row * kKRow + (uint32_t)(((lane & 15) ^ (row & 15)) << 4);
        }
    }
    // tiles t0 and t0+1 (64 keys) into their ring slots
    auto dma_k = [&](int t0, [[maybe_unused]] int slots) {
#pragma unroll
        for (int j = 0; j < K_DMA; ++j) {
            const int inst = wave * K_DMA + j;  // 16 instructions of 4 rows; 8 per tile
            const int row = inst * 4 + (lane >> 4);
            const uint32_t off = PAGED ? paged_off(slots, j * 4 + (lane >> 4), row & 15)
                                       : k_voff[j] + (uint32_t)t0 * kKTileBytes;
            lds_dma16(rk, lds + ((t0 + (inst >> 3)) & 3) * kKTileBytes + (inst & 7) * 4 * kKRow, off, 0);
        }
    };
    [[maybe_unused]] int slots = 0;
    if constexpr (PAGED) {
        dma_k(0, lookup(0, 0));
        slots = lookup(1, 0);  // tiles 1, 2 and value block 0
    } else {
        dma_k(0, 0);
    }
    dma_k(1, slots);

    if constexpr (!PAGED) {
        // what the block's queries may see
        kmax = pq;
        pmin = row_live ? pq : INT_MAX;
#pragma unroll
        for (int off = 16; off; off >>= 1) {
            kmax = max(kmax, __shfl_xor(kmax, off, kWave));
            pmin = min(pmin, __shfl_xor(pmin, off, kWave));
        }
        // every lane holds the same extremes by now: keep them in scalar registers (loop
        // bounds, the value descriptor's size)
        kmax = min(__builtin_amdgcn_readfirstlane(kmax), (int)a.max_len - 1);
        pmin = __builtin_amdgcn_readfirstlane(pmin);
    }
    const bool sees_a_key = pq >= 0;
    if (!row_live) pq = kmax;  // rows past the end see everything and are never stored
    const int nkb = kmax / kKB + 1;  // (kmax = -1, an empty sequence: one block of masked keys)

    // values: the same way into a 64-row buffer; chunk position (l%16) holds chunk
    // (l%16) ^ 4*(row%4). Rows past kmax arrive as zeros, so a stale cache row can never
    // meet a zero probability as 0 * NaN.
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(vc, PAGED ? pool_bytes : (uint32_t)(kmax + 1) * (uint32_t)kKRow);
    [[maybe_unused]] uint32_t v_voff[K_DMA];
    if constexpr (!PAGED) {
#pragma unroll
        for (int j = 0; j < K_DMA; ++j) {
            const int row = (wave * K_DMA + j) * 4 + (lane >> 4);
            v_voff[j] = (uint32_t)row * kKRow + (uint32_t)(((lane & 15) ^ (4 * (row & 3))) << 4);
        }
    }
    auto dma_v = [&](int kb, [[maybe_unused]] int slots) {
#pragma unroll
        for (int j = 0; j < K_DMA; ++j) {
            const int row = (wave * K_DMA + j) * 4 + (lane >> 4);
            const uint32_t off = PAGED ? paged_off(slots, RPW + j * 4 + (lane >> 4), 4 * (row & 3))
                                       : v_voff[j] + (uint32_t)kb * kVBytes;
            lds_dma16(rv, lds + kKRingBytes + (kb & 1) * kVBytes + (wave * K_DMA + j) * 4 * kKRow, off, 0);
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
    const f32x16 zero16 = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f,
                           0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    // byte offset of this lane's k-step 0 key chunk inside a tile, and of its V^T row
    const int k_lane = qi * kKRow;
    // V^T operand of 32 dims x 16 keys: two transposing reads. In each 16-lane group, lane
    // 4j+q points at row j, dims 4q..4q+3 of a 4-row x 16-dim patch and receives dim (its
    // index in the group) of rows 0..3. Lane half h takes rows 4h..4h+3 and 8+4h..8+4h+3 of
    // the 16-key step: the keys its P^T registers hold (register 4g+j = key 8g + 4h + j).
    // (bits 6-7 of the offset are dt ^ j: the dim tile is XORed into the offset as well)
    const int v_lane0 = [&] {
        const int sl = lane & 15, j = sl >> 2, q = sl & 3, g1 = (lane >> 4) & 1;
        return (4 * h + j) * kKRow + ((((2 * g1 + (q >> 1)) ^ (4 * j)) << 4) | ((q & 1) << 3));
    }();
    // key operand of k-step ks: chunk (2ks + h) ^ (row % 16) of this lane's row. The tile
    // offset and the row offset are multiples of 256, so the k-step can be XORed into the
    // whole byte offset: one address register per tile instead of eight.
    const int k_lane0 = k_lane + ((h ^ (qi & 15)) << 4);
    auto k_frag = [&](int tile_off, int ks) -> u32x4 {
        return *reinterpret_cast<const u32x4*>(lds + ((tile_off + k_lane0) ^ (ks << 5)));
    };
    auto v_frag = [&](int vt_off, int t, int dt) -> u32x4 {
        typedef __attribute__((address_space(3))) i16x4 lds_i16x4;
        const uint8_t* src = lds + ((vt_off + v_lane0) ^ (dt << 6)) + t * 16 * kKRow;
        const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(src));
        const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(src + 8 * kKRow));
        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
        return u32x4{l2.x, l2.y, h2.x, h2.y};
    };
    // masking and this lane's share of the row maximum of tile T (raw scores; c > 0 keeps order)
    auto mask_max4 = [&](auto mask_tag, int T, f32x16& s, int g, float m) -> float {
        constexpr bool PARTIAL = decltype(mask_tag)::value;  // some score of the tile may be hidden
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = 4 * g + j;
            if (PARTIAL) {
                const int key = T * 32 + g * 8 + h * 4 + j;
                bool visible = key <= pq;
                if constexpr (MASK) {
                    // (the byte is fetched whether or not it is needed, from a clamped index:
                    // four independent loads per group instead of four dependent branches)
                    const uint8_t keep = mask_row[max(min(key, mask_keys - 1), 0)];
                    visible = visible && key < mask_keys && keep != 0;
                }
                s[e] = visible ? s[e] : kNegBig;
            }
            m = fmaxf(m, s[e]);
        }
        return m;
    };

    // One tile step. In: s_in = raw (masked) scores of tile T, m_in = its row maximum (both lane
    // halves). Out: P.V of tile T added to o; s_out = scores of tile T+1, m_out = their maximum.
    auto step = [&](auto mask_tag, int T, f32x16& s_in, float m_in, f32x16& s_out, float& m_out,
                    int vt /* LDS offset of the 32 value rows of tile T */) {
        const float m_sc = m_in * c;
        if (__any(m_sc > m_run + kSlack)) {
            const float m_new = fmaxf(m_run, m_sc);
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                for (int e = 0; e < 16; ++e) o[dt][e] *= alpha;
        }
        const int kt = ((T + 1) & 3) * kKTileBytes;
        uint32_t pk[8];
        float l_add = 0.0f;
        u32x4 kf[8], vf[8];
        kf[0] = k_frag(kt, 0);
        kf[1] = k_frag(kt, 1);
        __builtin_amdgcn_sched_barrier(0);
        // ---- eight score MFMAs of tile T+1, each followed by two exponentials of tile T
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            if (ks + 2 < 8) kf[ks + 2] = k_frag(kt, ks + 2);
            if (ks >= 6) vf[ks - 6] = v_frag(vt, 0, ks - 6);
            s_out = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                __builtin_bit_cast(bf16x8, kf[ks]), __builtin_bit_cast(bf16x8, qf[ks]),
                ks == 0 ? zero16 : s_out, 0, 0, 0);
            const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_in[2 * ks], c, -m_run));
            const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_in[2 * ks + 1], c, -m_run));
            l_add += p0 + p1;
            pk[ks] = pack_bf16x2(p0, p1);
            __builtin_amdgcn_sched_barrier(0);
        }
        l_run += l_add;
        // ---- eight P.V MFMAs of tile T, the later ones followed by the maximum of tile T+1
        float m = kNegBig;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int t = i >> 2, dt = i & 3;
            if (i + 2 < 8) vf[i + 2] = v_frag(vt, (i + 2) >> 2, (i + 2) & 3);
            const u32x4 pf = {pk[4 * t], pk[4 * t + 1], pk[4 * t + 2], pk[4 * t + 3]};
            o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                __builtin_bit_cast(bf16x8, vf[i]), __builtin_bit_cast(bf16x8, pf), o[dt], 0, 0, 0);
            if (i >= 4) m = mask_max4(mask_tag, T + 1, s_out, i - 4, m);
            __builtin_amdgcn_sched_barrier(0);
        }
        m_out = fmaxf(m, __shfl_xor(m, 32, kWave));
    };

    // ---- prologue: tiles 0..2 and the first value block; scores of tile 0
    const int tfull = (__builtin_amdgcn_readfirstlane(pmin) + 1) / 32;  // tiles every query sees whole
    const int nfast = MASK ? 0 : max(tfull - 1, 0) / 2;  // blocks whose steps only produce unmasked tiles
    dma_v(0, slots);
    if constexpr (PAGED) slots = lookup(3, 1);  // what the first block's loads will ask for
    // tile 0 needs the queries and the key tiles, not the values: wait for everything but
    // this wave's K_DMA value loads (the newest), which get the scores of tile 0 to land
    __builtin_amdgcn_s_waitcnt(0x0f70 | K_DMA);  // vmcnt(K_DMA)
    __syncthreads();
    f32x16 sa, sb;
    float ma, mb;
    {
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
            sa = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                __builtin_bit_cast(bf16x8, k_frag(0, ks)), __builtin_bit_cast(bf16x8, qf[ks]),
                ks == 0 ? zero16 : sa, 0, 0, 0);
        float m = kNegBig;
#pragma unroll
        for (int g = 0; g < 4; ++g) m = mask_max4(std::true_type{}, 0, sa, g, m);
        ma = fmaxf(m, __shfl_xor(m, 32, kWave));
    }
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
    __syncthreads();  // values landed; tile 0's ring slot is overwritten by the first block's loads
    for (int kb = 0; kb < nkb; ++kb) {
        const int cur = kb & 1;
        dma_k(2 * kb + 3, slots);  // tiles 2kb+3, 2kb+4: their ring slots held tiles 2kb-1 and 2kb
        if (kb + 1 < nkb) dma_v(kb + 1, slots);
        if constexpr (PAGED) slots = lookup(2 * kb + 5, kb + 2);  // for the next block's loads
        const int vt = kKRingBytes + cur * kVBytes;
        if (kb < nfast) {
            step(std::false_type{}, 2 * kb, sa, ma, sb, mb, vt);
            step(std::false_type{}, 2 * kb + 1, sb, mb, sa, ma, vt + 32 * kKRow);
        } else {
            step(std::true_type{}, 2 * kb, sa, ma, sb, mb, vt);
            step(std::true_type{}, 2 * kb + 1, sb, mb, sa, ma, vt + 32 * kKRow);
        }
        __builtin_amdgcn_s_waitcnt(0x0070);
        __syncthreads();
    }
    // ---- normalise and write [batch, seq, heads*128]: through this wave's quarter of the
    // (now idle) key ring, so that the 32 x 128 tile leaves as whole 256-byte rows
    l_run += __shfl_xor(l_run, 32, kWave);
    // a row that sees no key at all (empty sequence, or more queries than keys) yields zeros
    // (with a mask tensor a row may have met nothing but masked scores: its reference maximum
    // then still is the stand-in for -inf, times c once it has been through a rescale)
    const bool met_a_key = !MASK || m_run > 0.5f * kNegBig * fminf(c, 1.0f);
    const float inv = (l_run > 0.0f && sees_a_key && met_a_key) ? 1.0f / l_run : 0.0f;
    {
        uint8_t* const mine = lds + wave * kKTileBytes;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                u32x2 w;
                w.x = pack_bf16x2(o[dt][4 * g] * inv, o[dt][4 * g + 1] * inv);
                w.y = pack_bf16x2(o[dt][4 * g + 2] * inv, o[dt][4 * g + 3] * inv);
                // row qi, dims 32dt + 8g + 4h ..+3: chunk 4dt+g (XOR-swizzled by row), half h
                *reinterpret_cast<u32x2*>(mine + qi * kKRow + (((4 * dt + g) ^ (qi & 15)) << 4) + h * 8) = w;
            }
        uint16_t* const obase = static_cast<uint16_t*>(a.out) + ((tok0 + row0) * a.n_heads + head) * kD;
        const int r4 = lane >> 4, c16 = lane & 15;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int row = i * 4 + r4;
            const u32x4 v = *reinterpret_cast<const u32x4*>(mine + row * kKRow + ((c16 ^ (row & 15)) << 4));
            if (row0 + row < rows_total)
                *reinterpret_cast<u32x4*>(obase + (size_t)row * a.n_heads * kD + c16 * 8) = v;
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
    const bool paged = a.req_to_token != nullptr;
    if (a.mask && (!paged || a.mask_width <= 0 || a.mask_rows <= 0)) return false;
    const int n_rep = a.n_heads / a.n_kv_heads;
    int64_t wgs;
    if (paged) {
        if (!a.req_pool_indices || !a.kv_indptr || !a.qo_indptr || !a.q_tile_to_batch || !a.q_tile_to_index ||
            a.num_q_tiles <= 0 || a.rtt_stride <= 0 || a.num_slots <= 0 || a.num_requests <= 0)
            return false;
        if (a.num_slots * (int64_t)a.n_kv_heads * kKRow >= ((int64_t)1 << 32)) return false;  // 32-bit pool offsets
        wgs = (int64_t)a.num_q_tiles * 2 * a.n_kv_heads;
    } else {
        if (a.batch <= 0 || a.seq <= 0 || a.max_len <= 0) return false;
        wgs = (int64_t)((a.seq + kQB - 1) / kQB) * a.batch * a.n_kv_heads;
    }
    if (wgs > INT_MAX) return false;
    const dim3 grid((unsigned)wgs);
#define W8A8_LAUNCH_PREFILL(R)                                                          \
    do {                                                                                \
        if (paged && a.mask)                                                            \
            attn_prefill_kernel<R, true, true><<<grid, dim3(64 * R), 0, stream>>>(a);   \
        else if (paged)                                                                 \
            attn_prefill_kernel<R, true><<<grid, dim3(64 * R), 0, stream>>>(a);         \
        else                                                                            \
            attn_prefill_kernel<R, false><<<grid, dim3(64 * R), 0, stream>>>(a);        \
    } while (0)
    if (n_rep == 2)
        W8A8_LAUNCH_PREFILL(2);
    else if (n_rep == 4)
        W8A8_LAUNCH_PREFILL(4);
    else
        W8A8_LAUNCH_PREFILL(8);
#undef W8A8_LAUNCH_PREFILL
    return true;
}

}  // namespace w8a8
