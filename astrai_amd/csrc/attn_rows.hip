// Paged grouped-query attention for the shapes the two tuned kernels do not take:
// head_dim 32, 64, 128 or 256, any n_heads / n_kv_heads up to 8, decode (one query
// row per sequence) and ragged prefill (row ranges per sequence) alike. The
// reference's paged kernels accept head_dim in {32, 64, 128, 256} and any head
// grouping (astrai/extension/backend/attention.py:518-527,
// csrc/kernels/attention/dispatchers.cuh); its own tests run head_dim 64
// (tests/extension/conftest.py:9-20).
//
// Same scheme as the decode kernel: the query rows that share a KV head -- n_rep heads
// times up to 8 / n_rep consecutive rows of a sequence, at most 8 in all -- are the
// columns of v_mfma_f32_16x16x32_bf16 score tiles whose rows are 16 keys; online
// softmax in fp32; P.V on the vector ALU; the four waves of a workgroup take key
// tiles in turn and merge through LDS; the context can be split over workgroups,
// merged by a second kernel. Every query row carries its own causal limit, so a
// block of prefill rows is a decode step with several newest tokens. Correct for
// every shape, not tuned: prefill re-reads the keys once per row block.
#include <climits>

#include "common.cuh"
#include "launchers.h"

namespace w8a8 {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kNQ = 8;             // query rows per workgroup (MFMA columns in use)
constexpr float kNegBig = -1e30f;  // finite stand-in for -inf: no inf - inf

__device__ __forceinline__ float lane_read(float v, int src_lane) {
    return __int_as_float(__builtin_amdgcn_ds_bpermute(src_lane << 2, __float_as_int(v)));
}
__device__ __forceinline__ int lane_read_i(int v, int src_lane) {
    return __builtin_amdgcn_ds_bpermute(src_lane << 2, v);
}

// W 32-bit words (2 W bf16 values) from an address aligned to their size (16 bytes at most)
template <int W>
__device__ __forceinline__ void load_words(const uint16_t* p, uint32_t (&w)[W]) {
    if constexpr (W == 1) {
        w[0] = *reinterpret_cast<const uint32_t*>(p);
    } else if constexpr (W == 2) {
        const u32x2 v = *reinterpret_cast<const u32x2*>(p);
        w[0] = v.x; w[1] = v.y;
    } else {
#pragma unroll
        for (int i = 0; i < W / 4; ++i) {
            const u32x4 v = *reinterpret_cast<const u32x4*>(p + 8 * i);
            w[4 * i] = v.x; w[4 * i + 1] = v.y; w[4 * i + 2] = v.z; w[4 * i + 3] = v.w;
        }
    }
}

// the row block a workgroup (or a merge workgroup's row) belongs to
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

// workspace per (row block, kv head, split): kNQ rows of [D values | max | sum]
template <int D, bool MASK>
__global__ __launch_bounds__(256) void attn_rows_partial_kernel(AttnRowsArgs a) {
    constexpr int STEPS = D / 32;  // score MFMAs per key tile
    constexpr int DV = D / 16;     // value dims per lane
    constexpr int WS_ROW = D + 2;
    __shared__ float sh_acc[4][kNQ][D];
    __shared__ float sh_ml[4][kNQ][2];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c16 = lane & 15, g = lane >> 4;
    const int n_rep = a.n_heads / a.n_kv_heads;
    const int rows = a.rows_per_block;
    const int nq = n_rep * rows;  // <= kNQ
    int wg = blockIdx.x;
    const int split = wg % a.nsplit;
    wg /= a.nsplit;
    const int hk = wg % a.n_kv_heads;
    const RowBlock rb = row_block(a, wg / a.n_kv_heads);
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

    float m = kNegBig, l = 0.0f;  // of query c16, equal in its four lanes
    float acc[kNQ][DV];
#pragma unroll
    for (int q = 0; q < kNQ; ++q)
#pragma unroll
        for (int d = 0; d < DV; ++d) acc[q][d] = 0.0f;

    // slot of key 16t + c16, looked up one tile ahead of its use. -1 (a negative or
    // out-of-pool table entry): nothing is fetched, key and value read as zeros, and the
    // position is attended all the same, as in the reference, which gates the load on the
    // slot and the mask on the position (csrc/kernels/attention/layout_policies.cuh:104-110,212-219)
    auto key_slot = [&](int t) -> int {
        const int key = (t << 4) + c16;
        const int slot = (t < t1 && key <= kmax) ? table[key] : -1;
        return slot < a.num_slots ? slot : -1;
    };
    int slot_next = key_slot(t0 + wave);
    const int64_t pool_row = (int64_t)a.n_kv_heads * D;  // elements from one slot to the next

    for (int t = t0 + wave; t < t1; t += 4) {
        const int kb = t << 4;
        const int slot = slot_next;
        slot_next = key_slot(t + 4);
        u32x4 kf[STEPS];
        uint32_t vw[4][DV / 2];
        [[maybe_unused]] uint8_t keep[4] = {1, 1, 1, 1};
        if constexpr (MASK) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = kb + 4 * g + i;
                keep[i] = key < mask_keys ? mask_row[key] : (uint8_t)0;
            }
        }
        {
            const uint16_t* kr = static_cast<const uint16_t*>(a.k_cache) + (int64_t)max(slot, 0) * pool_row +
                                 hk * D + 8 * g;
#pragma unroll
            for (int st = 0; st < STEPS; ++st)
                kf[st] = slot >= 0 ? *reinterpret_cast<const u32x4*>(kr + 32 * st) : u32x4{0, 0, 0, 0};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int vslot = lane_read_i(slot, 4 * g + i);  // lanes 0..15 hold keys kb..kb+15
                const uint16_t* vr = static_cast<const uint16_t*>(a.v_cache) + (int64_t)max(vslot, 0) * pool_row +
                                     hk * D + c16 * DV;
                if (vslot >= 0) {
                    load_words<DV / 2>(vr, vw[i]);
                } else {
#pragma unroll
                    for (int w = 0; w < DV / 2; ++w) vw[i][w] = 0u;
                }
            }
        }

        f32x4 sc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int st = 0; st < STEPS; ++st)
            sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf[st]),
                                                         __builtin_bit_cast(bf16x8, qf[st]), sc, 0, 0, 0);
        // sc[i] = q(c16) . k(kb + 4g + i)
        float tm = kNegBig;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            bool ok = q_live && kb + 4 * g + i <= q_pos;
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
        for (int q = 0; q < kNQ; ++q) {
            const float aq = lane_read(alpha, 16 * g + q);
#pragma unroll
            for (int d = 0; d < DV; ++d) acc[q][d] *= aq;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float v[DV];
#pragma unroll
            for (int w = 0; w < DV / 2; ++w) {
                // a row past the newest visible position was never written: keep it out even at p = 0
                const uint32_t raw = (kb + 4 * g + i) > kmax ? 0u : vw[i][w];
                v[2 * w] = __uint_as_float(raw << 16);
                v[2 * w + 1] = __uint_as_float(raw & 0xffff0000u);
            }
#pragma unroll
            for (int q = 0; q < kNQ; ++q) {
                const float pq = lane_read(p[i], 16 * g + q);
#pragma unroll
                for (int d = 0; d < DV; ++d) acc[q][d] += pq * v[d];
            }
        }
    }

    // the four key groups of the wave hold sums over different keys: add them up
#pragma unroll
    for (int q = 0; q < kNQ; ++q)
#pragma unroll
        for (int d = 0; d < DV; ++d) {
            float v = acc[q][d];
            v += __shfl_xor(v, 16, kWave);
            v += __shfl_xor(v, 32, kWave);
            acc[q][d] = v;
        }
    if (g == 0) {
#pragma unroll
        for (int q = 0; q < kNQ; ++q)
#pragma unroll
            for (int d = 0; d < DV; ++d) sh_acc[wave][q][c16 * DV + d] = acc[q][d];
        if (c16 < kNQ) {
            sh_ml[wave][c16][0] = m;
            sh_ml[wave][c16][1] = l;
        }
    }
    __syncthreads();
    // merge the four waves; thread -> (query, dim)
    float* ws = a.ws + (int64_t)blockIdx.x * kNQ * WS_ROW;
    for (int e = threadIdx.x; e < kNQ * D; e += 256) {
        const int q = e / D, d = e - q * D;
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
        ws[q * WS_ROW + d] = v;
        if (d == 0) {
            ws[q * WS_ROW + D] = mm;
            ws[q * WS_ROW + D + 1] = ll;
        }
    }
}

// One workgroup per query row slot of the schedule (decode: per sequence): merges the
// splits of every head of the row and writes out[row, head, :] in bf16.
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
        u32x4 o;
        o.x = pack_bf16x2(v[0] * inv, v[1] * inv);
        o.y = pack_bf16x2(v[2] * inv, v[3] * inv);
        o.z = pack_bf16x2(v[4] * inv, v[5] * inv);
        o.w = pack_bf16x2(v[6] * inv, v[7] * inv);
        *reinterpret_cast<u32x4*>(out + e) = o;
    }
}

template <int D>
void launch_for_dim(const AttnRowsArgs& a, unsigned grid1, unsigned grid2, hipStream_t stream) {
    if (a.mask)
        attn_rows_partial_kernel<D, true><<<dim3(grid1), dim3(256), 0, stream>>>(a);
    else
        attn_rows_partial_kernel<D, false><<<dim3(grid1), dim3(256), 0, stream>>>(a);
    attn_rows_merge_kernel<D><<<dim3(grid2), dim3(256), 0, stream>>>(a);
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
    return attn_rows_blocks(batch_or_tiles, n_heads, n_kv_heads, prefill) * n_kv_heads * nsplit * kNQ *
           (head_dim + 2);
}

bool launch_attn_rows(AttnRowsArgs a, hipStream_t stream) {
    if (!attn_rows_supported(a.n_heads, a.n_kv_heads, a.head_dim) || a.nsplit <= 0 || a.num_blocks <= 0) return false;
    if (!a.req_to_token || !a.req_pool_indices || !a.kv_indptr || a.rtt_stride <= 0) return false;
    const bool prefill = a.qo_indptr != nullptr;
    if (prefill && (!a.q_tile_to_batch || !a.q_tile_to_index)) return false;
    if (a.mask && (a.mask_width <= 0 || a.mask_rows <= 0)) return false;
    a.rows_per_block = prefill ? attn_rows_per_block(a.n_heads, a.n_kv_heads) : 1;
    a.blocks_per_tile = prefill ? 64 / a.rows_per_block : 1;
    const int64_t blocks = attn_rows_blocks(a.num_blocks, a.n_heads, a.n_kv_heads, prefill);
    const int64_t grid1 = blocks * a.n_kv_heads * a.nsplit;
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
