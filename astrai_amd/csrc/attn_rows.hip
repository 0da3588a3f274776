// Paged grouped-query attention for the shapes the two tuned kernels do not take:
// head_dim 32, 64, 128 or 256, any n_heads / n_kv_heads up to 16, decode (one query
// row per sequence) and ragged prefill (row ranges per sequence) alike. The
// reference's paged kernels accept head_dim in {32, 64, 128, 256} and any head
// grouping (astrai/extension/backend/attention.py:518-527,
// csrc/kernels/attention/entry_utils.cuh:13-22); its own tests run head_dim 64
// (tests/extension/conftest.py:9-20).
//
// One wave per (block of query rows, KV head, context split). The query rows that share a
// KV head -- n_rep heads times up to 16 / n_rep consecutive rows of a sequence, at most
// 16 in all -- are the columns of 16-key MFMA tiles:
//   scores  v_mfma_f32_16x16x32_bf16, keys as rows (16 bytes per lane straight from the
//           pool), so a lane ends up with the scores of one query for keys 4g..4g+3;
//   softmax online, fp32, per query (its four lanes share through two butterfly steps);
//   P.V     v_mfma_f32_16x16x16_bf16 per 16 dims with V^T as the row operand -- the 16
//           value rows of the tile pass through a wave-private LDS patch and come back
//           transposed (ds_read_tr16_b64) -- and P, already in the column operand's
//           layout, split into a bf16 head and a bf16 remainder (two MFMAs), so that the
//           probabilities enter with 16 bits of mantissa.
// Every query row carries its own causal limit and mask row, so a block of prefill rows is
// a decode step with several newest tokens. Without a context split the wave normalises
// and writes bf16 itself; with one it leaves (max, sum, acc) in a workspace for the merge
// kernel. Prefill without a split runs workgroups of four row blocks that share each key /
// value tile through LDS. Correct for every shape, not tuned like the head_dim-128 kernels.
#include <climits>

#include "common.cuh"
#include "launchers.h"

namespace w8a8 {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kNQ = 16;            // query rows per wave (MFMA columns)
constexpr float kNegBig = -1e30f;  // finite stand-in for -inf: no inf - inf

typedef short i16x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int lane_read_i(int v, int src_lane) {
    return __builtin_amdgcn_ds_bpermute(src_lane << 2, v);
}

// W 32-bit words (2 W bf16 values) on their way from the pool to LDS; addresses are aligned to
// the piece's size (16 bytes at most). Vector members, no arrays: the pieces stay in registers.
template <int W>
struct Piece;
template <>
struct Piece<1> {
    uint32_t v;
    __device__ __forceinline__ void load(const uint16_t* p) { v = *reinterpret_cast<const uint32_t*>(p); }
    __device__ __forceinline__ void store(uint8_t* p) const { *reinterpret_cast<uint32_t*>(p) = v; }
    __device__ __forceinline__ void zero() { v = 0u; }
};
template <>
struct Piece<2> {
    u32x2 v;
    __device__ __forceinline__ void load(const uint16_t* p) { v = *reinterpret_cast<const u32x2*>(p); }
    __device__ __forceinline__ void store(uint8_t* p) const { *reinterpret_cast<u32x2*>(p) = v; }
    __device__ __forceinline__ void zero() { v = u32x2{0u, 0u}; }
};
template <>
struct Piece<4> {
    u32x4 v;
    __device__ __forceinline__ void load(const uint16_t* p) { v = *reinterpret_cast<const u32x4*>(p); }
    __device__ __forceinline__ void store(uint8_t* p) const { *reinterpret_cast<u32x4*>(p) = v; }
    __device__ __forceinline__ void zero() { v = u32x4{0u, 0u, 0u, 0u}; }
};
template <>
struct Piece<8> {
    u32x4 lo, hi;
    __device__ __forceinline__ void load(const uint16_t* p) {
        lo = *reinterpret_cast<const u32x4*>(p);
        hi = *reinterpret_cast<const u32x4*>(p + 8);
    }
    __device__ __forceinline__ void store(uint8_t* p) const {
        *reinterpret_cast<u32x4*>(p) = lo;
        *reinterpret_cast<u32x4*>(p + 16) = hi;
    }
    __device__ __forceinline__ void zero() { lo = hi = u32x4{0u, 0u, 0u, 0u}; }
};

// the row block a wave (or a merge workgroup's row) belongs to
struct RowBlock {
    int seq;      // sequence (index into req_pool_indices, kv_indptr, qo_indptr, the mask)
    int q_start;  // first packed query row of the sequence
    int q_len;    // query rows of the sequence
    int r0;       // first row of the block inside the sequence
};

__device__ __forceinline__ RowBlock row_block(const AttnRowsArgs& a, int block) {
    RowBlock rb;
    if (a.qo_indptr) {
        const int tile = block / a.blocks_per_tile, sub = block - tile * a.blocks_per_tile;
        rb.seq = a.q_tile_to_batch[tile];
        rb.q_start = a.qo_indptr[rb.seq];
        rb.q_len = a.qo_indptr[rb.seq + 1] - rb.q_start;
        rb.r0 = a.q_tile_to_index[tile] * 64 + sub * a.rows_per_block;
    } else {  // decode: sequence b owns packed row b
        rb.seq = block;
        rb.q_start = block;
        rb.q_len = 1;
        rb.r0 = 0;
    }
    return rb;
}

// One 16-key tile for the 16 query columns of a wave. kf: the keys as MFMA rows (lane -> key
// c16, dims 32 step + 8g); qf: the queries likewise; keep: mask bytes of this lane's four keys;
// v_tr: where this lane's transposing reads of the staged value rows point (chunk 0); key0: the
// position of this lane's first key (tile start + 4g). Updates the running maximum m of query
// c16 (equal in its four lanes), this lane's share l of its running sum (finish with query_sum)
// and its accumulators o[c][i] (dim 16c + 4g + i).
template <int D, bool MASK>
__device__ __forceinline__ void tile_step(const u32x4 (&kf)[D / 32], const u32x4 (&qf)[D / 32],
                                          const uint8_t (&keep)[4], const uint8_t* v_tr, int key0, bool q_live,
                                          int q_pos, float scale, float& m, float& l, f32x4 (&o)[D / 16]) {
    f32x4 sc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int st = 0; st < D / 32; ++st)
        sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf[st]),
                                                     __builtin_bit_cast(bf16x8, qf[st]), sc, 0, 0, 0);
    // sc[i] = q(c16) . k(key0 + i)
    float tm = kNegBig;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        bool ok = q_live && key0 + i <= q_pos;
        if constexpr (MASK) ok = ok && keep[i] != 0;
        sc[i] = ok ? sc[i] * scale : kNegBig;
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
    l = l * alpha + ps;  // this lane's four keys only: the four lanes of a query are added up at the end
    m = m_new;

    // P as the column operand (query c16, keys key0 .. key0+3): bf16 head and bf16 remainder
    const uint32_t h01 = pack_bf16x2(p[0], p[1]), h23 = pack_bf16x2(p[2], p[3]);
    const uint32_t r01 = pack_bf16x2(p[0] - __uint_as_float(h01 << 16), p[1] - __uint_as_float(h01 & 0xffff0000u));
    const uint32_t r23 = pack_bf16x2(p[2] - __uint_as_float(h23 << 16), p[3] - __uint_as_float(h23 & 0xffff0000u));
    const i16x4 p_hi = __builtin_bit_cast(i16x4, u32x2{h01, h23});
    const i16x4 p_lo = __builtin_bit_cast(i16x4, u32x2{r01, r23});
#pragma unroll
    for (int c = 0; c < D / 16; ++c) {
        typedef __attribute__((address_space(3))) i16x4 lds_i16x4;
        const i16x4 vt = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(v_tr + c * 32));
        f32x4 acc = o[c] * alpha;
        acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vt, p_hi, acc, 0, 0, 0);
        o[c] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vt, p_lo, acc, 0, 0, 0);
    }
}

__device__ __forceinline__ float query_sum(float l) {
    l += __shfl_xor(l, 16, kWave);
    return l + __shfl_xor(l, 32, kWave);
}

// workspace per (row block, kv head, split): kNQ rows of [D values | max | sum]
template <int D, bool MASK>
__global__ __launch_bounds__(256) void attn_rows_partial_kernel(AttnRowsArgs a) {
    constexpr int STEPS = D / 32;           // score MFMAs per key tile
    constexpr int CHUNKS = D / 16;          // 16-dim output chunks
    constexpr int DV = D / 16;              // value dims a lane fetches per key
    constexpr int WS_ROW = D + 2;
    constexpr int V_STRIDE = D * 2 + 32;    // bytes per staged value row: the 4 rows of a transposing read hit distinct banks
    __shared__ __attribute__((aligned(16))) uint8_t v_stage[4][16 * V_STRIDE];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c16 = lane & 15, g = lane >> 4;
    const int n_rep = a.n_heads / a.n_kv_heads;
    const int rows = a.rows_per_block;
    const int nq = n_rep * rows;  // <= kNQ
    int64_t item = (int64_t)blockIdx.x * 4 + wave;
    if (item >= a.num_items) return;
    const int split = (int)(item % a.nsplit);
    item /= a.nsplit;
    const int hk = (int)(item % a.n_kv_heads);
    const int block = (int)(item / a.n_kv_heads);
    const RowBlock rb = row_block(a, block);
    if (rb.r0 >= rb.q_len) return;  // the schedule's tile reaches past the sequence: nothing reads this block

    const int64_t req = a.req_pool_indices[rb.seq];
    const bool req_ok = req >= 0 && req < a.num_requests;  // a bad row reads as an empty sequence
    const int kv_len =
        req_ok ? (int)min((int64_t)(a.kv_indptr[rb.seq + 1] - a.kv_indptr[rb.seq]), a.rtt_stride) : 0;
    const int* table = a.req_to_token + (req_ok ? req : 0) * a.rtt_stride;
    // row i of the sequence sees keys 0 .. kv_len - q_len + i (all of them without the causal flag)
    const int shift = kv_len - rb.q_len;
    const int last_row = min(rb.r0 + rows, rb.q_len) - 1;
    const int kmax = max(a.causal ? min(shift + last_row, kv_len - 1) : kv_len - 1, -1);

    // this lane's query row (a score column): head replica, row, newest visible key
    const int q_rep = c16 / rows, q_s = c16 - q_rep * rows;
    const int row = rb.r0 + q_s;
    const bool q_live = c16 < nq && row < rb.q_len;
    const int head = hk * n_rep + (q_live ? q_rep : 0);
    const int q_pos = !q_live ? -1 : (a.causal ? min(shift + row, kv_len - 1) : kv_len - 1);

    const int tiles_total = (kmax + 16) >> 4;  // keys 0..kmax
    const int tps = (tiles_total + a.nsplit - 1) / a.nsplit;
    const int t0 = split * tps, t1 = min(t0 + tps, tiles_total);

    // query operand: STEPS x 16 bytes: dims 32*step + 8g .. +7 of query c16
    u32x4 qf[STEPS];
    {
        const uint16_t* qrow = static_cast<const uint16_t*>(a.q) +
                               ((int64_t)(rb.q_start + (q_live ? row : rb.r0)) * a.n_heads + head) * D;
#pragma unroll
        for (int st = 0; st < STEPS; ++st)
            qf[st] = q_live ? *reinterpret_cast<const u32x4*>(qrow + 32 * st + 8 * g) : u32x4{0, 0, 0, 0};
    }
    [[maybe_unused]] const uint8_t* mask_row = nullptr;
    [[maybe_unused]] int mask_keys = 0;  // positions of this lane's query row that the mask covers
    if constexpr (MASK) {
        const bool covered = q_live && (a.mask_l_stride == 0 || row < a.mask_rows);
        mask_row = a.mask + (int64_t)rb.seq * a.mask_b_stride + (int64_t)head * a.mask_h_stride +
                   (int64_t)(covered ? row : 0) * a.mask_l_stride;
        mask_keys = covered ? a.mask_width : 0;
    }

    float m = kNegBig, l = 0.0f;  // running maximum of query c16 (equal in its four lanes); this lane's share of its sum
    // o[c][i] = sum over keys of p * v for query c16, dim 16c + 4g + i
    f32x4 o[CHUNKS];
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) o[c] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    // slot of key 16t + c16, looked up one tile ahead of its use. -1 (past the newest visible
    // key, or a negative or out-of-pool table entry): nothing is fetched, key and value read
    // as zeros; a negative entry inside the sequence is attended all the same, as in the
    // reference, which gates the load on the slot and the mask on the position
    // (csrc/kernels/attention/layout_policies.cuh:104-110,212-219)
    auto key_slot = [&](int t) -> int {
        const int key = (t << 4) + c16;
        const int slot = (t < t1 && key <= kmax) ? table[key] : -1;
        return slot < a.num_slots ? slot : -1;
    };
    const int64_t pool_row = (int64_t)a.n_kv_heads * D;  // elements from one slot to the next
    uint8_t* const stage = v_stage[wave];
    // where this lane stores the value pieces it fetches (key 4g + i, dims DV c16 ..) and where
    // its transposing reads point (key 4g + c16 / 4, dims 16c + 4 (c16 % 4) ..: the lane gets
    // dim 16c + c16 of keys 4g .. 4g+3 back)
    uint8_t* const st_mine = stage + (4 * g) * V_STRIDE + c16 * DV * 2;
    const uint8_t* const tr_mine = stage + (4 * g + (c16 >> 2)) * V_STRIDE + (c16 & 3) * 8;

    // operands of one key tile, requested a tile ahead of their use: keys as MFMA rows (lane ->
    // key 16t + c16, dims 32 step + 8g), values (lane -> keys 16t + 4g + i, dims DV c16 ..), mask bytes
    u32x4 kf_n[STEPS];
    Piece<DV / 2> vw_n[4];
    [[maybe_unused]] uint8_t keep_n[4] = {1, 1, 1, 1};
    auto fetch = [&](int t, int slot) {
        const uint16_t* kr = static_cast<const uint16_t*>(a.k_cache) + (int64_t)max(slot, 0) * pool_row + hk * D + 8 * g;
#pragma unroll
        for (int st = 0; st < STEPS; ++st)
            kf_n[st] = slot >= 0 ? *reinterpret_cast<const u32x4*>(kr + 32 * st) : u32x4{0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int vslot = lane_read_i(slot, 4 * g + i);  // lanes 0..15 hold the slots of keys 16t..16t+15
            const uint16_t* vr = static_cast<const uint16_t*>(a.v_cache) + (int64_t)max(vslot, 0) * pool_row +
                                 hk * D + c16 * DV;
            if (vslot >= 0)
                vw_n[i].load(vr);
            else
                vw_n[i].zero();
        }
        if constexpr (MASK) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = (t << 4) + 4 * g + i;
                keep_n[i] = key < mask_keys ? mask_row[key] : (uint8_t)0;
            }
        }
    };
    fetch(t0, key_slot(t0));
    int slot_next = key_slot(t0 + 1);

    for (int t = t0; t < t1; ++t) {
        const int kb = t << 4;
        u32x4 kf[STEPS];
        [[maybe_unused]] uint8_t keep[4];
#pragma unroll
        for (int st = 0; st < STEPS; ++st) kf[st] = kf_n[st];
#pragma unroll
        for (int i = 0; i < 4; ++i) keep[i] = keep_n[i];
        // values of the tile into the wave's patch (the previous tile's reads are done: same wave, in order)
        __asm__ volatile("" ::: "memory");
#pragma unroll
        for (int i = 0; i < 4; ++i) vw_n[i].store(st_mine + i * V_STRIDE);
        __asm__ volatile("" ::: "memory");
        fetch(t + 1, slot_next);  // (past the last tile every slot is -1: nothing is requested)
        slot_next = key_slot(t + 2);

        tile_step<D, MASK>(kf, qf, keep, tr_mine, kb + 4 * g, q_live, q_pos, a.scale, m, l, o);
    }

    l = query_sum(l);
    if (a.nsplit == 1) {
        // the whole context was this wave's: normalise and write out[row, head, 16c + 4g ..+3]
        if (!q_live) return;
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;  // a row with no visible key yields zeros
        uint16_t* orow = static_cast<uint16_t*>(a.out) + ((int64_t)(rb.q_start + row) * a.n_heads + head) * D + 4 * g;
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c)
            *reinterpret_cast<u32x2*>(orow + 16 * c) =
                u32x2{pack_bf16x2(o[c][0] * inv, o[c][1] * inv), pack_bf16x2(o[c][2] * inv, o[c][3] * inv)};
        return;
    }
    float* ws = a.ws + (((int64_t)block * a.n_kv_heads + hk) * a.nsplit + split) * kNQ * WS_ROW + c16 * WS_ROW;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {  // (a workspace row starts on an 8-byte boundary only)
        *reinterpret_cast<f32x2_hw*>(ws + 16 * c + 4 * g) = f32x2_hw{o[c][0], o[c][1]};
        *reinterpret_cast<f32x2_hw*>(ws + 16 * c + 4 * g + 2) = f32x2_hw{o[c][2], o[c][3]};
    }
    if (g == 0) {
        ws[D] = m;
        ws[D + 1] = l;
    }
}

// Ragged prefill without a context split: a workgroup takes four consecutive row blocks of one
// sequence and KV head, one per wave, and its waves share every key / value tile. Wave w
// fetches keys and values 4w .. 4w+3 of a tile (one piece of D / 8 bytes per lane and tensor),
// the tile passes through one of two LDS buffers (one barrier per tile), and each wave takes its
// key operand and its transposed value operand from there: a quarter of the global traffic of
// four independent waves. Same arithmetic (tile_step), same results.
template <int D, bool MASK>
__global__ __launch_bounds__(256) void attn_rows_shared_kernel(AttnRowsArgs a) {
    constexpr int STEPS = D / 32, CHUNKS = D / 16;
    constexpr int PIECE = D / 16;             // bf16 values a lane fetches per tensor and tile
    constexpr int ROW = D * 2 + 32;           // bytes per staged row (see V_STRIDE above)
    __shared__ __attribute__((aligned(16))) uint8_t k_stage[2][16 * ROW];
    __shared__ __attribute__((aligned(16))) uint8_t v_stage[2][16 * ROW];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c16 = lane & 15, g = lane >> 4;
    const int n_rep = a.n_heads / a.n_kv_heads;
    const int rows = a.rows_per_block;
    const int nq = n_rep * rows;
    const int hk = blockIdx.x % a.n_kv_heads;
    const int super = blockIdx.x / a.n_kv_heads;  // four row blocks
    const RowBlock first = row_block(a, super * 4);
    if (first.r0 >= first.q_len) return;  // the whole workgroup lies past the sequence
    RowBlock rb = first;
    rb.r0 = first.r0 + wave * rows;
    const bool wave_live = rb.r0 < rb.q_len;

    const int64_t req = a.req_pool_indices[rb.seq];
    const bool req_ok = req >= 0 && req < a.num_requests;
    const int kv_len =
        req_ok ? (int)min((int64_t)(a.kv_indptr[rb.seq + 1] - a.kv_indptr[rb.seq]), a.rtt_stride) : 0;
    const int* table = a.req_to_token + (req_ok ? req : 0) * a.rtt_stride;
    const int shift = kv_len - rb.q_len;
    // newest key any row of the workgroup sees / of this wave sees
    const int wg_last = min(first.r0 + 4 * rows, rb.q_len) - 1;
    const int kmax_wg = max(a.causal ? min(shift + wg_last, kv_len - 1) : kv_len - 1, -1);
    const int my_last = min(rb.r0 + rows, rb.q_len) - 1;
    const int kmax = !wave_live ? -1 : max(a.causal ? min(shift + my_last, kv_len - 1) : kv_len - 1, -1);

    const int q_rep = c16 / rows, q_s = c16 - q_rep * rows;
    const int row = rb.r0 + q_s;
    const bool q_live = c16 < nq && row < rb.q_len;
    const int head = hk * n_rep + (q_live ? q_rep : 0);
    const int q_pos = !q_live ? -1 : (a.causal ? min(shift + row, kv_len - 1) : kv_len - 1);
    const int tiles = (kmax_wg + 16) >> 4;

    u32x4 qf[STEPS];
    {
        const uint16_t* qrow = static_cast<const uint16_t*>(a.q) +
                               ((int64_t)(rb.q_start + (q_live ? row : first.r0)) * a.n_heads + head) * D;
#pragma unroll
        for (int st = 0; st < STEPS; ++st)
            qf[st] = q_live ? *reinterpret_cast<const u32x4*>(qrow + 32 * st + 8 * g) : u32x4{0, 0, 0, 0};
    }
    [[maybe_unused]] const uint8_t* mask_row = nullptr;
    [[maybe_unused]] int mask_keys = 0;
    if constexpr (MASK) {
        const bool covered = q_live && (a.mask_l_stride == 0 || row < a.mask_rows);
        mask_row = a.mask + (int64_t)rb.seq * a.mask_b_stride + (int64_t)head * a.mask_h_stride +
                   (int64_t)(covered ? row : 0) * a.mask_l_stride;
        mask_keys = covered ? a.mask_width : 0;
    }
    float m = kNegBig, l = 0.0f;
    f32x4 o[CHUNKS];
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) o[c] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    // this lane's share of a tile's loads: key 16t + 4 wave + g, values PIECE c16 .. of both tensors
    const int my_key = 4 * wave + g;
    auto key_slot = [&](int t) -> int {
        const int key = (t << 4) + my_key;
        const int slot = (t < tiles && key <= kmax_wg) ? table[key] : -1;
        return slot < a.num_slots ? slot : -1;
    };
    const int64_t pool_row = (int64_t)a.n_kv_heads * D;
    // operands are requested AHEAD tiles before their use. Measured (32 x 512 tokens): three tiles
    // ahead gains 10% at head_dim 64 and loses 10% at 128, where the registers it takes cost a
    // resident wave per SIMD
    constexpr int AHEAD = D <= 64 ? 3 : 1;
    Piece<PIECE / 2> kw[AHEAD], vw[AHEAD];
    [[maybe_unused]] uint8_t keep_n[AHEAD][4];
    int slot_q[AHEAD];
    auto fetch = [&](int t, int slot, Piece<PIECE / 2>& kwj, Piece<PIECE / 2>& vwj, uint8_t (&kj)[4]) {
        const int64_t off = (int64_t)max(slot, 0) * pool_row + hk * D + c16 * PIECE;
        if (slot >= 0) {
            kwj.load(static_cast<const uint16_t*>(a.k_cache) + off);
            vwj.load(static_cast<const uint16_t*>(a.v_cache) + off);
        } else {
            kwj.zero();
            vwj.zero();
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = (t << 4) + 4 * g + i;
            kj[i] = !MASK ? (uint8_t)1 : (key < mask_keys ? mask_row[key] : (uint8_t)0);
        }
    };
#pragma unroll
    for (int j = 0; j < AHEAD; ++j) fetch(j, key_slot(j), kw[j], vw[j], keep_n[j]);
#pragma unroll
    for (int j = 0; j < AHEAD; ++j) slot_q[j] = key_slot(AHEAD + j);
    const int put = my_key * ROW + c16 * PIECE * 2;                    // where this lane's pieces go
    const int k_get = c16 * ROW + 16 * g;                              // key c16, dims 32 step + 8g
    const int v_get = (4 * g + (c16 >> 2)) * ROW + (c16 & 3) * 8;      // transposing reads, chunk 0

    for (int t0 = 0; t0 < tiles; t0 += AHEAD) {
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) {
            const int t = t0 + j;
            if (t >= tiles) continue;  // (the same for every wave of the workgroup)
            const int buf = t & 1;
            kw[j].store(k_stage[buf] + put);
            vw[j].store(v_stage[buf] + put);
            uint8_t keep[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) keep[i] = keep_n[j][i];
            __syncthreads();  // tile t is in place; everyone is done with the buffer tile t+1 will use
            fetch(t + AHEAD, slot_q[j], kw[j], vw[j], keep_n[j]);
            slot_q[j] = key_slot(t + 2 * AHEAD);
            if ((t << 4) <= kmax) {  // (wave-uniform) some row of this wave sees the tile
                u32x4 kf[STEPS];
#pragma unroll
                for (int st = 0; st < STEPS; ++st)
                    kf[st] = *reinterpret_cast<const u32x4*>(k_stage[buf] + k_get + 64 * st);
                tile_step<D, MASK>(kf, qf, keep, v_stage[buf] + v_get, (t << 4) + 4 * g, q_live, q_pos, a.scale, m, l,
                                   o);
            }
        }
    }
    l = query_sum(l);
    if (!q_live) return;
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;  // a row with no visible key yields zeros
    uint16_t* orow = static_cast<uint16_t*>(a.out) + ((int64_t)(rb.q_start + row) * a.n_heads + head) * D + 4 * g;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
        *reinterpret_cast<u32x2*>(orow + 16 * c) =
            u32x2{pack_bf16x2(o[c][0] * inv, o[c][1] * inv), pack_bf16x2(o[c][2] * inv, o[c][3] * inv)};
}

// With a context split: one workgroup per query row slot of the schedule (decode: per
// sequence) merges the splits of every head of the row and writes out[row, head, :] in bf16.
template <int D>
__global__ __launch_bounds__(256) void attn_rows_merge_kernel(AttnRowsArgs a) {
    constexpr int WS_ROW = D + 2;
    const int n_rep = a.n_heads / a.n_kv_heads;
    const int rows = a.rows_per_block;
    const int slots_per_block = a.qo_indptr ? rows : 1;
    const int block = blockIdx.x / slots_per_block, q_s = blockIdx.x - block * slots_per_block;
    const RowBlock rb = row_block(a, block);
    const int row = rb.r0 + q_s;
    if (row >= rb.q_len) return;
    const int width = a.n_heads * D;
    uint16_t* out = static_cast<uint16_t*>(a.out) + (int64_t)(rb.q_start + row) * width;
    for (int e = threadIdx.x * 8; e < width; e += 256 * 8) {
        const int h = e / D, d0 = e - h * D;
        const int hk = h / n_rep, q = (h - hk * n_rep) * rows + q_s;
        const float* base = a.ws + (((int64_t)block * a.n_kv_heads + hk) * a.nsplit) * kNQ * WS_ROW + q * WS_ROW;
        float mm = kNegBig;
        for (int j = 0; j < a.nsplit; ++j) mm = fmaxf(mm, base[(int64_t)j * kNQ * WS_ROW + D]);
        float v[8] = {0, 0, 0, 0, 0, 0, 0, 0}, ll = 0.0f;
        for (int j = 0; j < a.nsplit; ++j) {
            const float* r = base + (int64_t)j * kNQ * WS_ROW;
            const float f = __expf(r[D] - mm);
            ll += r[D + 1] * f;
#pragma unroll
            for (int d = 0; d < 8; ++d) v[d] += r[d0 + d] * f;
        }
        const float inv = ll > 0.0f ? 1.0f / ll : 0.0f;  // a row with no visible key yields zeros
        u32x4 ov;
        ov.x = pack_bf16x2(v[0] * inv, v[1] * inv);
        ov.y = pack_bf16x2(v[2] * inv, v[3] * inv);
        ov.z = pack_bf16x2(v[4] * inv, v[5] * inv);
        ov.w = pack_bf16x2(v[6] * inv, v[7] * inv);
        *reinterpret_cast<u32x4*>(out + e) = ov;
    }
}

template <int D>
void launch_for_dim(const AttnRowsArgs& a, unsigned grid1, unsigned grid2, hipStream_t stream) {
    if (a.qo_indptr && a.nsplit == 1) {
        // prefill without a split: four row blocks to a workgroup, sharing the key / value tiles
        const unsigned grid = (unsigned)(a.num_items / 4);  // (blocks per tile is a multiple of 4)
        if (a.mask)
            attn_rows_shared_kernel<D, true><<<dim3(grid), dim3(256), 0, stream>>>(a);
        else
            attn_rows_shared_kernel<D, false><<<dim3(grid), dim3(256), 0, stream>>>(a);
        return;
    }
    if (a.mask)
        attn_rows_partial_kernel<D, true><<<dim3(grid1), dim3(256), 0, stream>>>(a);
    else
        attn_rows_partial_kernel<D, false><<<dim3(grid1), dim3(256), 0, stream>>>(a);
    if (a.nsplit > 1) attn_rows_merge_kernel<D><<<dim3(grid2), dim3(256), 0, stream>>>(a);
}

}  // namespace

int attn_rows_per_block(int n_heads, int n_kv_heads) {
    if (n_kv_heads <= 0 || n_heads % n_kv_heads) return 0;
    const int n_rep = n_heads / n_kv_heads;
    if (n_rep > kNQ) return 0;
    int rows = 1;
    while (rows * 2 * n_rep <= kNQ) rows *= 2;  // 1, 2, 4 or 8: divides the schedule's 64-row tiles
    return rows;
}

bool attn_rows_supported(int n_heads, int n_kv_heads, int head_dim) {
    return (head_dim == 32 || head_dim == 64 || head_dim == 128 || head_dim == 256) &&
           attn_rows_per_block(n_heads, n_kv_heads) > 0;
}

int64_t attn_rows_blocks(int64_t batch_or_tiles, int n_heads, int n_kv_heads, bool prefill) {
    const int rows = attn_rows_per_block(n_heads, n_kv_heads);
    if (rows <= 0) return 0;
    return prefill ? batch_or_tiles * (64 / rows) : batch_or_tiles;
}

int64_t attn_rows_workspace_floats(int64_t batch_or_tiles, int n_heads, int n_kv_heads, int head_dim,
                                   int nsplit, bool prefill) {
    if (!attn_rows_supported(n_heads, n_kv_heads, head_dim)) return -1;
    if (nsplit <= 1) return 0;  // each wave owns a whole context and writes the output itself
    return attn_rows_blocks(batch_or_tiles, n_heads, n_kv_heads, prefill) * n_kv_heads * nsplit * kNQ *
           (head_dim + 2);
}

bool launch_attn_rows(AttnRowsArgs a, hipStream_t stream) {
    if (!attn_rows_supported(a.n_heads, a.n_kv_heads, a.head_dim) || a.nsplit <= 0 || a.num_blocks <= 0) return false;
    if (!a.req_to_token || !a.req_pool_indices || !a.kv_indptr || a.rtt_stride <= 0) return false;
    if (a.nsplit > 1 && !a.ws) return false;
    const bool prefill = a.qo_indptr != nullptr;
    if (prefill && (!a.q_tile_to_batch || !a.q_tile_to_index)) return false;
    if (a.mask && (a.mask_width <= 0 || a.mask_rows <= 0)) return false;
    a.rows_per_block = prefill ? attn_rows_per_block(a.n_heads, a.n_kv_heads) : 1;
    a.blocks_per_tile = prefill ? 64 / a.rows_per_block : 1;
    const int64_t blocks = attn_rows_blocks(a.num_blocks, a.n_heads, a.n_kv_heads, prefill);
    a.num_items = blocks * a.n_kv_heads * a.nsplit;  // one wave each, four to a workgroup
    const int64_t grid1 = (a.num_items + 3) / 4;
    const int64_t grid2 = prefill ? blocks * a.rows_per_block : blocks;
    if (grid1 > INT_MAX || grid2 > INT_MAX) return false;
    switch (a.head_dim) {
        case 32: launch_for_dim<32>(a, (unsigned)grid1, (unsigned)grid2, stream); break;
        case 64: launch_for_dim<64>(a, (unsigned)grid1, (unsigned)grid2, stream); break;
        case 128: launch_for_dim<128>(a, (unsigned)grid1, (unsigned)grid2, stream); break;
        default: launch_for_dim<256>(a, (unsigned)grid1, (unsigned)grid2, stream); break;
    }
    return true;
}

}  // namespace w8a8
