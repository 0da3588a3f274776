// Host-side launch functions, one group per kernel family. Each launches
// asynchronously on `stream` and returns nothing; the C ABI layer (abi.hip)
// validates arguments first and checks hipGetLastError() afterwards.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace w8a8 {

// Opt a kernel into more than 64 KiB of dynamic LDS. The attribute belongs to the
// (kernel, device) pair and a process may drive several devices from several
// threads, so `done` (one per kernel, static at the call site) keeps one bit per
// device; setting the attribute twice is harmless.
inline void allow_dynamic_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done) {
    int dev = 0;
    const bool known = hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64;
    const uint64_t bit = known ? (uint64_t)1 << dev : 0;
    if (known && (done.load(std::memory_order_acquire) & bit)) return;
    (void)hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (known) done.fetch_or(bit, std::memory_order_release);
}

// Diagnostic: every GEMM launcher leaves the family name of the kernel it launched here (per
// host thread); astrai_w8a8_last_kernel() reads it back. A product sent out as two launches
// (whole 256-row tiles + a ragged tail on the decode kernel) reports the tile kernel.
extern thread_local const char* g_last_kernel;
inline void note_kernel(const char* name) { g_last_kernel = name; }

enum OutKind : int { OUT_BF16 = 0, OUT_E4M3 = 1, OUT_ACC = 2 };
enum ScaleKind : int { SCALE_TENSOR = 0, SCALE_ROWCOL = 1, SCALE_BLOCK128 = 2 };

struct GemmArgs {
    const void* a;        // [M,K] 8-bit activations
    const void* b;        // [N,K] 8-bit weights
    const float* sa;      // per-tensor [1] | per-token [M] | block [M,K/128]
    const float* sb;      // per-tensor [1] | per-channel [N] | block [ceil(N/128),K/128]
    const float* out_scale;  // OUT_E4M3 only
    const void* bias;     // bf16 [N] or null
    void* out;            // [M,N]
    int m, n, k;
    int out_kind;
    float* row_max = nullptr;  // SwiGLU epilogue only: fp32 [M, N/128] partial row maxima of |h|
    const void* resid = nullptr;  // residual epilogue only: bf16 [M,N]; out = bf16(bf16(y) + resid)
};

// quantize.hip
// The maximum of |x| leaves a quantizer either by atomic max into *amax or, when `partials` is
// given, as kAmaxPartials per-workgroup maxima (every slot written) for the ring push to reduce.
constexpr int kAmaxPartials = 1024;
void launch_quantize_fp8(const void* x, void* x8, const float* scale, float* amax, float* partials,
                         int64_t total, int fmt, hipStream_t stream);
// hist[idx] = fresh; *scale = max((max(hist) / fmax) / pow2_margin, 1e-12), with fresh = *amax or
// the maximum of the kAmaxPartials partials (then also stored to *amax_out when that is given)
void launch_amax_ring_push(float* hist, int n, int idx, const float* amax, const float* partials,
                           float* amax_out, float* scale, float fmax, float pow2_margin,
                           hipStream_t stream);
// *amax = max(*amax, max |x|), or the partial maxima
void launch_amax_bf16(const void* x, float* amax, float* partials, int64_t total, hipStream_t stream);
// codes of a [rows, cols] matrix row-major (x8, may be null) and transposed (x8t, [cols, rows])
void launch_quantize_transpose_fp8(const void* x, void* x8, void* x8t, const float* scale,
                                   float* amax, int64_t rows, int64_t cols, int fmt,
                                   hipStream_t stream);
void launch_quantize_int8_rows(const void* x, void* xq, float* s, int64_t rows, int64_t k,
                               hipStream_t stream);
// fused producers: (residual add +) RMSNorm + per-row int8; SwiGLU product + per-row
// int8. Row width must be a multiple of 8 and at most kFusedRowMax.
constexpr int64_t kFusedRowMax = 8192;
void launch_add_rmsnorm_quantize_int8_rows(const void* x, const void* res, const void* w, float eps,
                                           void* sum_out, void* y_out, void* xq, float* s,
                                           int64_t rows, int64_t k, hipStream_t stream);
// block > 0: gate and up columns come in pieces of `block` columns, 2 * block apart
void launch_silu_mul_quantize_int8_rows(const void* gate, const void* up, int64_t ld, int64_t block,
                                        void* h_out, void* hq, float* s, int64_t rows, int64_t width,
                                        hipStream_t stream);
// per-tensor fp8 twins (step known ahead; *amax = max(*amax, max |value|) when amax is given)
void launch_add_rmsnorm_quantize_fp8_rows(const void* x, const void* res, const void* w, float eps,
                                          void* sum_out, void* y_out, void* x8, const float* scale,
                                          float* amax, int64_t rows, int64_t k, int fmt,
                                          hipStream_t stream);
void launch_silu_mul_quantize_fp8_rows(const void* gate, const void* up, int64_t ld, void* h_out,
                                       void* h8, const float* scale, float* amax, int64_t rows,
                                       int64_t width, int fmt, hipStream_t stream);
// per-row int8 of bf16 rows whose |maximum| is known as `pieces` partial maxima per row
void launch_quantize_int8_rows_pmax(const void* h, const float* row_max, int64_t pieces, void* hq,
                                    float* s, int64_t rows, int64_t width, hipStream_t stream);
void launch_quantize_fp8_block128_act(const void* x, void* x8, float* sa, int64_t m,
                                      int64_t k, hipStream_t stream);
void launch_quantize_fp8_block128_weight(const void* w, void* w8, float* sb, int64_t n,
                                         int64_t k, hipStream_t stream);

// rope_cache.hip: rotary embedding of q / k and the KV-cache write, one pass over
// the fused q|k|v projection output
struct RopeCacheArgs {
    const void* qkv;          // bf16 [batch*seq, ld], columns q heads | k heads | v heads
    int64_t ld;               // row pitch of qkv in elements
    const float* freqs;       // fp32 [seq, head_dim/2, 2] (cos, sin) of the tokens' positions
    const int64_t* positions; // int64 [seq]: cache slot of each token
    void* q_out;              // bf16 [batch, n_heads, seq, head_dim]
    void* k_cache;            // bf16 [batch, n_kv_heads, max_len, head_dim]
    void* v_cache;            // same
    int batch, seq, n_heads, n_kv_heads, head_dim;
    int64_t max_len;
};
void launch_rope_cache_write(const RopeCacheArgs& a, hipStream_t stream);
// x, out bf16 [tokens, heads, head_dim]; freqs fp32 [tokens, head_dim/2, 2] (cos, sin) per token.
// head_dim must be even; false if it is not.
bool launch_rotary_emb(const void* x, const float* freqs, void* out, int64_t tokens, int heads,
                       int head_dim, hipStream_t stream);

// attn_decode.hip: grouped-query attention of a few new tokens against the dense
// bf16 KV cache, split over the context; head_dim 128, n_rep * seq <= 8
struct AttnDecodeArgs {
    const void* q;             // bf16 [batch, n_heads, seq, 128]
    const void* k_cache;       // bf16 [batch, n_kv_heads, max_len, 128]
    const void* v_cache;       // same
    const int64_t* positions;  // int64 [seq]: position of each new token (keys <= it are attended)
    float* ws;                 // attn_decode_workspace_floats(...) floats
    void* out;                 // bf16 [batch, seq, n_heads * 128], or null
    void* out_q;               // int8 [batch*seq, n_heads * 128] per-token quantization of `out`, or null
    float* out_scale;          // fp32 [batch*seq] steps of out_q
    int batch, seq, n_heads, n_kv_heads, head_dim;
    int64_t max_len;
    int nsplit;
    float scale;
    // paged mode (req_to_token != null): seq == 1, the caches are pools [slots, n_kv_heads, 128],
    // positions is unused and every sequence has its own length
    const int* req_to_token;      // int32 [requests, rtt_stride]: slot of (request, position)
    const int* req_pool_indices;  // int32 [batch]: row of req_to_token of each sequence
    const int* kv_indptr;         // int32 [batch + 1]: prefix sums of the sequence lengths
    int64_t rtt_stride;
    int64_t num_slots, num_requests;  // table entries / rows outside these are treated as absent
    // paged mode only, optional: bool [batch, mask_width] with row stride mask_b_stride; position
    // j of sequence b is attended only where mask[b][j] is non-zero, positions at or past
    // mask_width are not attended (csrc/kernels/attention/entry_utils.cuh:226-237, mma_utils.cuh:196-199)
    const uint8_t* mask;
    int64_t mask_b_stride;
    int mask_width;
};
int64_t attn_decode_workspace_floats(int batch, int n_kv_heads, int nsplit, int nq);
bool launch_attn_decode(const AttnDecodeArgs& a, hipStream_t stream);

// attn_prefill.hip: causal grouped-query attention of a block of new tokens against
// the dense bf16 KV cache; head_dim 128, n_heads / n_kv_heads in {2, 4, 8}
struct AttnPrefillArgs {
    const void* q;             // bf16 [batch, n_heads, seq, 128]
    const void* k_cache;       // bf16 [batch, n_kv_heads, max_len, 128]
    const void* v_cache;       // same
    const int64_t* positions;  // int64 [seq]: position of each new token (keys <= it are attended)
    void* out;                 // bf16 [batch, seq, n_heads * 128]
    int batch, seq, n_heads, n_kv_heads, head_dim;
    int64_t max_len;
    float scale;
    // paged mode (req_to_token != null): q and out are packed [total_q, n_heads, 128], the
    // caches are pools [slots, n_kv_heads, 128]; positions, batch, seq and max_len are unused
    const int* req_to_token;      // int32 [requests, rtt_stride]: slot of (request, position)
    const int* req_pool_indices;  // int32 [batch]: row of req_to_token of each sequence
    const int* kv_indptr;         // int32 [batch + 1]: prefix sums of the key counts
    const int* qo_indptr;         // int32 [batch + 1]: prefix sums of the query row counts
    const int* q_tile_to_batch;   // int32 [num_q_tiles]: sequence of each 64-row query tile
    const int* q_tile_to_index;   // int32 [num_q_tiles]: index of the tile within its sequence
    int num_q_tiles;
    int causal;                   // row i of a sequence sees keys 0 .. kv_len - q_len + i; else all keys
    int64_t rtt_stride, num_slots, num_requests;
    // paged mode only, optional: bool mask addressed as mask[b * mask_b_stride + head *
    // mask_h_stride + row * mask_l_stride + key] with b the sequence, row the query row inside
    // the sequence and key the position (csrc/kernels/attention/entry_utils.cuh:326-346,
    // mma_utils.cuh:190-199). A stride of 0 broadcasts that axis. Rows at or past mask_rows (when
    // mask_l_stride != 0) and keys at or past mask_width are not attended.
    const uint8_t* mask;
    int64_t mask_b_stride, mask_h_stride, mask_l_stride;
    int mask_rows, mask_width;
};
bool attn_prefill_supported(int n_heads, int n_kv_heads, int head_dim);
bool launch_attn_prefill(const AttnPrefillArgs& a, hipStream_t stream);

// attn_rows.hip: paged attention for every head_dim in {32, 64, 128, 256} and every
// n_heads / n_kv_heads <= 8; decode (qo_indptr == null: sequence b owns packed row b) and
// ragged prefill (row ranges and the 64-row tile schedule, as for attn_prefill's paged mode)
struct AttnRowsArgs {
    const void* q;                // bf16 [total_q, n_heads, head_dim]
    const void* k_cache;          // bf16 [num_slots, n_kv_heads, head_dim]
    const void* v_cache;          // same
    const int* req_to_token;      // int32 [num_requests, rtt_stride]
    const int* req_pool_indices;  // int32 [batch]
    const int* kv_indptr;         // int32 [batch + 1]
    const int* qo_indptr;         // int32 [batch + 1], or null for decode
    const int* q_tile_to_batch;   // int32 [num_blocks] (prefill)
    const int* q_tile_to_index;   // int32 [num_blocks] (prefill)
    float* ws;                    // attn_rows_workspace_floats(...) floats
    void* out;                    // bf16 [total_q, n_heads, head_dim]
    int64_t num_blocks;           // decode: batch; prefill: 64-row tiles of the schedule
    int n_heads, n_kv_heads, head_dim, nsplit;
    int causal;                   // prefill: row i of a sequence sees keys 0 .. kv_len - q_len + i
    float scale;
    int64_t rtt_stride, num_slots, num_requests;
    // optional bool mask, addressed as for AttnPrefillArgs (decode: row 0 of every sequence)
    const uint8_t* mask;
    int64_t mask_b_stride, mask_h_stride, mask_l_stride;
    int mask_rows, mask_width;
    int rows_per_block, blocks_per_tile;  // filled in by the launcher
    int64_t num_items;                    // (row block, kv head, split) triples, filled in by the launcher
};
bool attn_rows_supported(int n_heads, int n_kv_heads, int head_dim);
int64_t attn_rows_workspace_floats(int64_t batch_or_tiles, int n_heads, int n_kv_heads, int head_dim,
                                   int nsplit, bool prefill);
bool launch_attn_rows(AttnRowsArgs a, hipStream_t stream);

// gemm_int8.hip / gemm_fp8.hip / gemm_fp8_block.hip: tiled MFMA kernels.
// Require k % 16 == 0 and m*k, n*k < 2^31 bytes; return false if the shape is
// not accepted (the caller then uses the generic kernel).
// `tail_on_decode_kernel`: a token tail that would cost the large-tile kernel a round of its own may
// run on the decode kernel in a second launch (false: the tiled kernels only)
bool launch_gemm_int8_tiled(const GemmArgs& g, hipStream_t stream, bool tail_on_decode_kernel = true);
// gate|up projection with the SwiGLU product in the epilogue. Weight rows come in blocks of
// 128: 64 gate rows, then the 64 up rows of the same columns of h. g.out is h = bf16(up *
// bf16(silu(gate))) [M, N/2], g.row_max[m, N/128] the maximum of |h| over each 64-column piece.
// Large shapes only (those of the four-wave 256x256 kernel, N % 128 == 0, no bias); false otherwise.
bool launch_gemm_int8_swiglu(const GemmArgs& g, hipStream_t stream);
// a projection whose output is added to the residual stream in the epilogue:
// g.out = bf16(bf16(dequantized product + bias) + g.resid), the bf16 arithmetic of `linear(x) + residual`.
// Row-range kernel for up to 128 tokens (K % 256 == 0), four-wave 256x256 kernel for the large
// shapes it takes; false otherwise (the caller runs the plain GEMM and an addition pass).
bool launch_gemm_int8_resid(const GemmArgs& g, hipStream_t stream);
// out = bf16(y + resid) over `total` bf16 elements; out may be y
void launch_add_bf16(const void* y, const void* resid, void* out, int64_t total, hipStream_t stream);
bool launch_gemm_fp8_tiled(const GemmArgs& g, int fmt, hipStream_t stream);
// sa per activation row [M], sb per weight row [N], bf16 output
bool launch_gemm_fp8_rowcol_tiled(const GemmArgs& g, int fmt, hipStream_t stream);
bool launch_gemm_fp8_block128_tiled(const GemmArgs& g, hipStream_t stream);

// gemm_generic.hip: any shape, guarded byte loads, one wave per 16x16 tile.
void launch_gemm_generic(const GemmArgs& g, int op /*0=i8,1=e4m3,2=e5m2*/, int scale_kind,
                         hipStream_t stream);

// gemv_int8.hip: decode-shape int8 kernels (one token: dot kernel; 2..128 tokens: row-range kernel), k % 256 == 0.
bool launch_gemv_int8(const GemmArgs& g, hipStream_t stream);
// the row-range kernel on fp8 operands: at most 128 tokens, k % 256 == 0, bf16 or fp32-accumulator
// output, per-tensor or per-row / per-column steps; false when the shape does not fit
bool launch_gemv_fp8(const GemmArgs& g, int fmt /*0=e4m3,1=e5m2*/, int scale_kind, hipStream_t stream);
// the same kernel on e4m3fn operands with 128-block steps (sa [M, K/128], sb [ceil(N/128), K/128]):
// at most 64 tokens, k % 256 == 0, bf16 output
bool launch_gemv_fp8_block128(const GemmArgs& g, hipStream_t stream);
// the fused q|k|v projection of up to 64 tokens with rotary embedding and KV-cache write
// in the epilogue (g.out unused; rc.qkv / rc.ld unused); false when the shape does not fit
bool launch_gemm_int8_rope_cache(const GemmArgs& g, const RopeCacheArgs& rc, hipStream_t stream);
// gemm_int8.hip: the same for long blocks of tokens (prefill) on the large-tile kernel: head_dim 128,
// at least 192 output tiles of 256 x 256, K % 128 == 0; false when the shape does not fit
bool launch_gemm_int8_rope_cache_large(const GemmArgs& g, const RopeCacheArgs& rc, hipStream_t stream);

// mfma_probe.hip: one instruction of MFMA shape `kind` on a zero accumulator, one wave;
// d_raw[lane][reg] are the accumulator registers as they are (4 or 16 per lane)
bool launch_mfma_probe(int kind, const void* a, const void* b, void* d_raw, hipStream_t stream);

}  // namespace w8a8
