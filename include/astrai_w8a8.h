/*
 * astrai_w8a8 -- C ABI of the gfx950 (MI355X) backend for AstrAI's quantized
 * linear-layer GEMM path.
 *
 * These entry points are what the reference's `fp8_mm` pybind module
 * (csrc/kernels/fp8/mm.cu:350-369) binds, restated as a plain C ABI: raw device
 * pointers, sizes, a HIP stream, an int status. The host adapter
 * (astrai_amd/extension/_cabi.py) owns tensor checks and output allocation, as
 * the reference binding does (mm.cu:99-126,128-184,186-234).
 *
 * Conventions shared by every call
 *   - All pointers are device pointers on the current HIP device, 16-byte
 *     aligned, into contiguous row-major storage. Nothing is allocated, freed,
 *     or synchronised; every launch is asynchronous on `stream` (a hipStream_t
 *     passed as void*; NULL = the default stream) and reads its scales on the
 *     device, so the calls are HIP-graph capturable
 *     (reference: at::cuda::getCurrentCUDAStream(), mm.cu:108-109,147-148).
 *   - A scale is the quantization STEP: q = x / scale, dequantization multiplies
 *     by it (astrai/extension/ops/fp8.py:10-13).
 *   - GEMMs are "NT": A is [M,K], B is [N,K] (the weight layout, no transpose),
 *     both K-contiguous; out is [M,N] (mm.cu:150-152).
 *   - Return value: ASTRAI_W8A8_OK or an error code; the message for the calling
 *     thread's last error is available from astrai_w8a8_last_error().
 */
#ifndef ASTRAI_W8A8_H
#define ASTRAI_W8A8_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ASTRAI_W8A8_ABI_VERSION 1

/* status codes */
#define ASTRAI_W8A8_OK 0
#define ASTRAI_W8A8_BAD_ARG 1       /* null pointer, negative size, bad enum  */
#define ASTRAI_W8A8_UNSUPPORTED 2   /* shape outside what the kernels accept  */
#define ASTRAI_W8A8_LAUNCH_FAILED 3 /* hipGetLastError() after the launch     */

/* fp8 formats: FP8Format in csrc/kernels/fp8/common.h:10-13 */
#define ASTRAI_W8A8_E4M3 0 /* OCP e4m3fn, max 448 */
#define ASTRAI_W8A8_E5M2 1 /* OCP e5m2, max 57344 */

/* output element types */
#define ASTRAI_W8A8_OUT_BF16 0
#define ASTRAI_W8A8_OUT_E4M3 1 /* fp8 GEMM only; needs out_scale (mm.cu:152-161) */
#define ASTRAI_W8A8_OUT_ACC 2  /* raw accumulator: int32 (int8 GEMM) / fp32 (fp8 GEMM) */

/* ABI version of the loaded library (== ASTRAI_W8A8_ABI_VERSION at build time). */
int astrai_w8a8_abi_version(void);

/* Message of the calling thread's most recent failing call ("" if none). */
const char* astrai_w8a8_last_error(void);

/*
 * bf16 -> fp8 quantize with fused amax.
 * Replaces quantize_bf16 (csrc/kernels/fp8/mm.cu:99-126) and
 * fp8_quantize_kernel (csrc/kernels/fp8/gemm.cuh:128-158).
 *   x8[i]  = sat_fp8(float(x[i]) / *scale)   (true division, as the CPU kernel
 *            astrai/extension/ops/fp8.py:80; saturating like the device kernel)
 *   *amax  = max(*amax, max_i |x[i]|) over the raw values. The caller zeroes
 *            *amax beforehand (the reference binding does, mm.cu:115); NULL skips it.
 */
int astrai_w8a8_quantize_bf16_fp8(const void* x_bf16, void* x8, const float* scale,
                                  float* amax, int64_t total, int fmt, void* stream);

/*
 * *amax = max(*amax, max_i |x[i]|) over a bf16 tensor, one read and no temporary.
 * Replaces the t.abs().amax() with which dynamic scaling measures each operand
 * before quantizing it (astrai/extension/fp8.py:289-292). The caller zeroes *amax.
 */
int astrai_w8a8_amax_bf16(const void* x_bf16, float* amax, int64_t total, void* stream);

/*
 * Delayed scaling's record-then-refresh (FP8TensorMeta.update_*,
 * astrai/extension/fp8.py:147-173, step formula :87-89) in one launch:
 *   hist[idx] = *amax;  *scale = max((max_i hist[i] / fmax) / pow2_margin, 1e-12)
 * hist is the fp32 ring of n recorded amax values, fmax the format's largest
 * finite value (448 or 57344), pow2_margin = 2^margin. True fp32 divisions, as
 * the reference's formula evaluates on host tensors.
 */
int astrai_w8a8_amax_ring_push(float* hist, int n, int idx, const float* amax, float* scale,
                               float fmax, float pow2_margin, void* stream);

/*
 * The three entries above with the maximum handed over as per-workgroup partial maxima
 * instead of one atomically updated slot: the producer (the quantizer of
 * csrc/kernels/fp8/mm.cu:99-126, or the amax pass) writes every one of the
 * ASTRAI_W8A8_AMAX_PARTIALS fp32 slots of `partials` (unused ones zero), and the ring push
 * reduces them -- max is order-free, so ring and step come out as with
 * astrai_w8a8_quantize_bf16_fp8 + astrai_w8a8_amax_ring_push, bit for bit. No slot to clear
 * before the producer, no atomics and nothing that waits at the producer's end: at 4096 x 4096
 * the quantizer takes 10 us against 13.8 us, and the fill launch of the slot disappears. The
 * forward of a Linear under delayed / dynamic scaling (astrai/extension/fp8.py:275-305) runs on
 * these. amax_out (may be NULL) receives the reduced maximum. total must be positive.
 */
#define ASTRAI_W8A8_AMAX_PARTIALS 1024
int astrai_w8a8_quantize_bf16_fp8_partials(const void* x_bf16, void* x8, const float* scale,
                                           float* partials, int64_t total, int fmt, void* stream);
int astrai_w8a8_amax_bf16_partials(const void* x_bf16, float* partials, int64_t total, void* stream);
int astrai_w8a8_amax_ring_push_partials(float* hist, int n, int idx, const float* partials,
                                        float* amax_out, float* scale, float fmax,
                                        float pow2_margin, void* stream);

/*
 * The same quantizer on a [rows, cols] matrix, writing the codes transposed
 * ([cols, rows], x8t) and, when x8 is not NULL, row-major as well, from one read
 * of x. Replaces the transposed-contiguous copies followed by quantize_bf16 in
 * linear_backward_fp8 (csrc/kernels/fp8/mm.cu:276-312): dX = g.w contracts
 * over the gradient's columns and dW = g^T.x over its rows, so the gradient is
 * needed in both layouts and w, x transposed. amax as above.
 */
int astrai_w8a8_quantize_transpose_bf16_fp8(const void* x_bf16, void* x8, void* x8t,
                                            const float* scale, float* amax, int64_t rows,
                                            int64_t cols, int fmt, void* stream);

/*
 * bf16 -> int8, symmetric, one scale per row (per token for activations, per
 * output channel for weights). No counterpart in the reference (it has no int8
 * path); same conventions as the fp8 quantizer.
 *   s[r]    = max(max_k |x[r,k]|, 1e-12) / 127
 *   xq[r,k] = clamp(round_half_even(float(x[r,k]) / s[r]), -127, 127)
 */
int astrai_w8a8_quantize_bf16_int8_rows(const void* x_bf16, void* xq, float* s,
                                        int64_t rows, int64_t k, void* stream);

/*
 * Producers fused with the per-row int8 quantizer: the activation of every int8
 * Linear in the decoder comes out of an RMSNorm (after a residual add) or out of
 * the SwiGLU product, and is read by nothing but the quantizer.
 *
 * add_rmsnorm: replaces the residual add of DecoderBlock.forward
 * (astrai/model/components/decoder_block.py:59-70), RMSNorm.forward = F.rms_norm
 * (astrai/model/components/norm.py:7-15) and quantize_bf16_int8_rows above.
 *   t[r,:]  = res ? bf16(x[r,:] + res[r,:]) : x[r,:]          (written to sum_out when res and sum_out are given)
 *   y[r,k]  = bf16(weight[k] * (t[r,k] * rsqrt(mean_k t[r,k]^2 + eps)))   fp32 arithmetic, one rounding
 *   s[r], xq[r,:] = the per-row int8 quantizer applied to y[r,:]
 * res, sum_out, y_out may be NULL (y_out receives y when given). K % 8 == 0, K <= 8192.
 *
 * silu_mul: replaces ``up(x) * F.silu(gate(x))`` of MLP.forward
 * (astrai/model/components/mlp.py:41) and the quantizer in front of ``down``.
 *   h[r,j]  = bf16(up[r,j] * bf16(gate[r,j] / (1 + exp(-gate[r,j]))))
 *   s[r], hq[r,:] = the per-row int8 quantizer applied to h[r,:]
 * gate and up rows are ld elements apart (the two halves of one [rows, 2*width]
 * gate|up GEMM output, or two separate tensors with ld = width); hq and h_out
 * (optional) are dense [rows, width]. width % 8 == 0, ld % 8 == 0, width <= 8192.
 */
int astrai_w8a8_add_rmsnorm_quantize_int8_rows(const void* x_bf16, const void* res_bf16,
                                               const void* weight_bf16, float eps,
                                               void* sum_out_bf16, void* y_out_bf16, void* xq,
                                               float* s, int64_t rows, int64_t k, void* stream);
int astrai_w8a8_silu_mul_quantize_int8_rows(const void* gate_bf16, const void* up_bf16, int64_t ld,
                                            void* h_out_bf16, void* hq, float* s, int64_t rows,
                                            int64_t width, void* stream);

/*
 * Per-tensor fp8 twins of the two producers, for Linear layers under the delayed-scaling
 * recipe (astrai/extension/fp8.py:147-173: the step of this call is known before the
 * activation exists; the call reports the maximum for the ring). Replace the same
 * reference code as the int8 producers plus custom::fp8_quantize
 * (astrai/extension/ops/fp8.py:60-82) on the activation.
 *   t, y, h     as above (same bf16 arithmetic)
 *   x8 / h8     = fp8(value / *scale), magnitudes clamped to the format's finite maximum
 *                 (the quantizer of quantize_bf16_fp8), [rows, K] / [rows, width]
 *   *amax       = max(*amax, max |value|) when amax is given (clear it before the first call)
 * K % 8 == 0 and K <= 8192 for add_rmsnorm; width % 8 == 0, ld % 8 == 0 for silu_mul.
 */
int astrai_w8a8_add_rmsnorm_quantize_fp8_rows(const void* x_bf16, const void* res_bf16,
                                              const void* weight_bf16, float eps,
                                              void* sum_out_bf16, void* y_out_bf16, void* x8,
                                              const float* scale, float* amax, int64_t rows,
                                              int64_t k, int fmt, void* stream);
int astrai_w8a8_silu_mul_quantize_fp8_rows(const void* gate_bf16, const void* up_bf16, int64_t ld,
                                           void* h_out_bf16, void* h8, const float* scale,
                                           float* amax, int64_t rows, int64_t width, int fmt,
                                           void* stream);

/*
 * The gate and up projections of MLP.forward (astrai/model/components/mlp.py:40-43) as one
 * GEMM whose epilogue applies the SwiGLU product, so that the [rows, 2*width] gate|up
 * matrix never reaches memory. The fused weight holds the rows of gate and up in blocks of
 * 128: rows 128t .. 128t+63 are gate rows 64t .. 64t+63, rows 128t+64 .. 128t+127 the up
 * rows of the same 64 columns of h (scales b likewise). Three entry points share that layout:
 *
 * gemm_int8_ptpc_swiglu: a int8 [M,K], b int8 [N,K] (N = 2*width, blocked as above), sa [M],
 *   sb [N]. Writes h bf16 [M, N/2] with
 *     gate = bf16(acc * sa[m] * sb[n_gate]), up = bf16(acc * sa[m] * sb[n_up])   (what
 *     gemm_int8_ptpc would have stored), h = bf16(up * bf16(gate / (1 + exp(-gate))))
 *   and row_max fp32 [M, N/128]: the maximum of |h| over each 64-column piece of the row.
 *   Shapes of the large-tile kernel only (at least 192 output tiles of 256 x 256, K % 128 == 0,
 *   K >= 256, N % 128 == 0); ASTRAI_W8A8_UNSUPPORTED otherwise -- then run gemm_int8_ptpc on
 *   the same blocked weight and silu_mul_quantize_int8_rows_blocked on its output.
 * quantize_int8_rows_pmax: the per-row int8 quantizer for rows whose maximum is known as
 *   `pieces` partial maxima per row (row_max above): one read of h, same s and hq as
 *   quantize_bf16_int8_rows. width % 8 == 0, width <= 8192.
 * silu_mul_quantize_int8_rows_blocked: silu_mul_quantize_int8_rows on a [rows, ld >= 2*width]
 *   gate|up matrix whose columns alternate between `block` gate and `block` up columns.
 * Together (GEMM + quantizer, or GEMM + blocked producer) they give bit for bit the h, s and
 * hq of gemm_int8_ptpc on an unblocked weight followed by silu_mul_quantize_int8_rows.
 */
int astrai_w8a8_gemm_int8_ptpc_swiglu(const void* a, const void* b, const float* sa, const float* sb,
                                      void* h_out_bf16, float* row_max, int64_t m, int64_t n,
                                      int64_t k, void* stream);
int astrai_w8a8_quantize_int8_rows_pmax(const void* h_bf16, const float* row_max, int64_t pieces,
                                        void* hq, float* s, int64_t rows, int64_t width,
                                        void* stream);
int astrai_w8a8_silu_mul_quantize_int8_rows_blocked(const void* gu_bf16, int64_t ld, int64_t block,
                                                    void* h_out_bf16, void* hq, float* s,
                                                    int64_t rows, int64_t width, void* stream);

/*
 * A projection whose output joins the residual stream, `attn_output + x` and
 * `mlp_output + x` of DecoderBlock.forward (astrai/model/components/decoder_block.py:67,70),
 * as one kernel: out[m,n] = bf16(bf16(acc * sa[m] * sb[n] + bias[n]) + resid[m,n]), bit for
 * bit gemm_int8_ptpc followed by the bf16 addition. resid bf16 [M,N], 16-byte aligned; out
 * must not overlap it. The addition runs in the GEMM's epilogue for up to 128 tokens with
 * K % 256 == 0 and N % 4 == 0 and for the shapes of the large-tile kernel; other shapes take
 * the plain product and an addition pass.
 */
int astrai_w8a8_gemm_int8_ptpc_resid(const void* a, const void* b, const float* sa, const float* sb,
                                     const void* bias_bf16, const void* resid_bf16, void* out_bf16,
                                     int64_t m, int64_t n, int64_t k, void* stream);

/*
 * Rotary embedding of q and k plus the KV-cache write of one decoder layer, one
 * pass over the (fused) q|k|v projection output. Replaces, between the
 * projections and the attention call of GQA.forward
 * (astrai/model/components/attention.py:19-85): the reshape/permute of q, k, v,
 * the rotation of adjacent pairs in fp32 with one cast back
 * (astrai/extension/backend/rotary.py:25-33) and the cache update.
 *   qkv        bf16 [batch*seq, ld]: per token  q (n_heads*head_dim) | k (n_kv_heads*head_dim) | v (same)
 *   freqs      fp32 [seq, head_dim/2, 2]: (cos, sin) of each token's position
 *   positions  int64 [seq] (device): cache slot of each token; a slot outside [0, max_len) is skipped
 *   q_out      bf16 [batch, n_heads, seq, head_dim]
 *   k_cache, v_cache  bf16 [batch, n_kv_heads, max_len, head_dim], written at positions[s]
 *   rope(x)[2i] = x[2i] cos_i - x[2i+1] sin_i;  rope(x)[2i+1] = x[2i] sin_i + x[2i+1] cos_i
 *   (every product and sum rounded in fp32, one rounding to bf16: identical to the tensor ops)
 * head_dim % 8 == 0, ld % 8 == 0.
 */
int astrai_w8a8_rope_cache_write_bf16(const void* qkv_bf16, int64_t ld, const float* freqs,
                                      const int64_t* positions, void* q_out_bf16,
                                      void* k_cache_bf16, void* v_cache_bf16, int64_t batch,
                                      int64_t seq, int64_t n_heads, int64_t n_kv_heads,
                                      int64_t head_dim, int64_t max_len, void* stream);

/*
 * Rotary embedding alone. Replaces rotary_emb (csrc/kernels/rotary/rotary_emb.cu:6-45 kernel,
 * :47-93 entry; Python wrapper astrai/extension/ops/rotary.py:24-39).
 *   x, out     bf16 [tokens, n_heads, head_dim], contiguous (a dense [batch, seq, ...] tensor
 *              is the same memory with tokens = batch * seq)
 *   freqs_cis  fp32 [tokens, head_dim/2, 2]: each token's own (cos, sin) rows
 *   out[t,h,2i] = x[t,h,2i] cos - x[t,h,2i+1] sin;  out[t,h,2i+1] = x[t,h,2i] sin + x[t,h,2i+1] cos
 *   with every product and sum rounded in fp32 and one rounding to bf16: bit for bit the
 *   fp32 tensor arithmetic of astrai/extension/backend/rotary.py:25-33 (the reference's own
 *   kernel leaves the contraction of a*b - c*d to its compiler).
 * head_dim even; pointers 16-byte aligned when head_dim % 8 == 0, else 4-byte.
 */
int astrai_w8a8_rotary_emb_bf16(const void* x_bf16, const float* freqs_cis, void* out_bf16,
                                int64_t tokens, int64_t n_heads, int64_t head_dim, void* stream);

/*
 * Grouped-query attention of the `seq` newest tokens of every sequence against the
 * dense KV cache (decode step; split over the context and merged). Replaces the
 * cached branch of GQA.forward / the decode attention backend
 * (astrai/model/components/attention.py:19-85,
 * astrai/extension/backend/attention.py:244-253,443-498): head expansion, mask and
 * softmax(q k^T * scale) v, with the permute back to token-major folded in.
 *   q          bf16 [batch, n_heads, seq, 128] (as written by rope_cache_write)
 *   k_cache, v_cache  bf16 [batch, n_kv_heads, max_len, 128]; entries at positions
 *              <= the largest positions[s] must have been written
 *   positions  int64 [seq] (device): token s attends keys 0..positions[s]
 *   workspace  fp32, at least astrai_w8a8_attn_decode_workspace_floats(batch,
 *              n_kv_heads, nsplit, (n_heads / n_kv_heads) * seq) floats (caller-owned scratch)
 *   out        bf16 [batch, seq, n_heads * 128], or NULL
 *   out_q, out_scale  int8 [batch*seq, n_heads * 128] and fp32 [batch*seq]: the per-token int8
 *              quantization of the bf16-rounded output rows (quantize_bf16_int8_rows applied to
 *              `out`), or NULL; at least one of out / out_q must be given
 *   nsplit     number of context splits (1..64): batch * n_kv_heads * nsplit workgroups
 * fp32 scores and softmax, fp32 accumulation of p*v, one rounding to bf16.
 * head_dim == 128, (n_heads / n_kv_heads) * seq <= 8, n_heads <= 64.
 */
int64_t astrai_w8a8_attn_decode_workspace_floats(int64_t batch, int64_t n_kv_heads, int64_t nsplit,
                                                 int64_t n_query_rows);
int astrai_w8a8_attn_decode_bf16(const void* q_bf16, const void* k_cache_bf16, const void* v_cache_bf16,
                                 const int64_t* positions, float* workspace, int64_t workspace_floats,
                                 void* out_bf16, void* out_q, float* out_scale, int64_t batch,
                                 int64_t seq, int64_t n_heads,
                                 int64_t n_kv_heads, int64_t head_dim, int64_t max_len,
                                 int64_t nsplit, float scale, void* stream);

/*
 * attn_decode_bf16 for callers that cannot allocate device memory or bring a workspace
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * It has no counterpart in the reference. Same arguments, kernels and results as
 * attn_decode_bf16 minus the workspace: the context splits' partial results go to an array
 * of ASTRAI_W8A8_STATIC_SCRATCH_FLOATS floats (4 MiB) that the library holds in static device
 * memory, one copy per GPU it runs on, until the process ends. Calls no hipMalloc / hipFree
 * or any other allocating routine. Returns ASTRAI_W8A8_UNSUPPORTED when
 * astrai_w8a8_attn_decode_workspace_floats(batch, n_kv_heads, nsplit, rows) exceeds the array.
 * The array's device address is looked up on the first call on each device (make that call
 * outside stream capture). Every call on a GPU shares that GPU's array: calls that overlap on
 * one GPU (other streams, other threads) race; calls ordered on one stream do not. Nothing in
 * the array has to be cleared between calls: every slot a call reads it has written itself.
 */
#define ASTRAI_W8A8_STATIC_SCRATCH_FLOATS (1 << 20)
int astrai_w8a8_attn_decode_bf16_static_scratch(const void* q_bf16, const void* k_cache_bf16,
                                                const void* v_cache_bf16, const int64_t* positions,
                                                void* out_bf16, void* out_q, float* out_scale,
                                                int64_t batch, int64_t seq, int64_t n_heads,
                                                int64_t n_kv_heads, int64_t head_dim, int64_t max_len,
                                                int64_t nsplit, float scale, void* stream);

/*
 * The same decode attention over a token-granular paged cache. Replaces
 * attn_paged_decode (csrc/kernels/attention/paged_decode.cu:4-67, addressing policy
 * PagedKV in csrc/kernels/attention/layout_policies.cuh:174-232; Python wrapper
 * astrai/extension/ops/attention.py:93-147) without its fused append of new_k / new_v;
 * the variant with the optional key mask follows.
 *   q          bf16 [batch, n_heads, 128]: the newest token of every sequence
 *   k_pool, v_pool  bf16 [num_slots, n_kv_heads, 128]
 *   req_to_token    int32 [num_requests, max_context_len]: pool slot of (request, position);
 *              a negative entry ("empty padding"; likewise one >= num_slots) is not
 *              fetched: its key and value read as zeros, and the position is attended like
 *              any other, as in the reference (load gated on the slot, mask on the position:
 *              layout_policies.cuh:104-110,212-219)
 *   req_pool_indices  int32 [batch]: row of req_to_token of each sequence
 *   kv_indptr  int32 [batch + 1]: prefix sums of the sequence lengths; sequence b attends
 *              positions 0 .. kv_indptr[b+1] - kv_indptr[b] - 1
 *   workspace  as for attn_decode_bf16 with n_query_rows = n_heads / n_kv_heads
 *   out        bf16 [batch, n_heads, 128]; a sequence of length 0 yields zeros
 * head_dim == 128, n_heads / n_kv_heads <= 8, n_heads <= 64.
 */
int astrai_w8a8_attn_paged_decode_bf16(const void* q_bf16, const void* k_pool_bf16,
                                       const void* v_pool_bf16, const int32_t* req_to_token,
                                       const int32_t* req_pool_indices, const int32_t* kv_indptr,
                                       float* workspace, int64_t workspace_floats, void* out_bf16,
                                       int64_t batch, int64_t n_heads, int64_t n_kv_heads,
                                       int64_t head_dim, int64_t num_slots, int64_t num_requests,
                                       int64_t max_context_len, int64_t nsplit, float scale,
                                       void* stream);

/*
 * attn_paged_decode_bf16 with the reference's optional key mask (the `mask` argument of
 * csrc/kernels/attention/paged_decode.cu:13, packed at entry_utils.cuh:226-237 and applied
 * at mma_utils.cuh:196-199).
 *   mask       bool (one byte each) [batch, mask_width], rows mask_row_stride bytes apart:
 *              position j of sequence b is attended only where mask[b][j] != 0. Positions
 *              at or past mask_width are not attended (the reference reads past the row
 *              there). A sequence with every position masked yields zeros. NULL: no mask,
 *              mask_row_stride and mask_width are ignored.
 */
int astrai_w8a8_attn_paged_decode_masked_bf16(const void* q_bf16, const void* k_pool_bf16,
                                              const void* v_pool_bf16, const int32_t* req_to_token,
                                              const int32_t* req_pool_indices, const int32_t* kv_indptr,
                                              const uint8_t* mask, int64_t mask_row_stride,
                                              int64_t mask_width, float* workspace,
                                              int64_t workspace_floats, void* out_bf16, int64_t batch,
                                              int64_t n_heads, int64_t n_kv_heads, int64_t head_dim,
                                              int64_t num_slots, int64_t num_requests,
                                              int64_t max_context_len, int64_t nsplit, float scale,
                                              void* stream);

/*
 * Causal grouped-query attention of a block of `seq` new tokens per sequence against
 * the dense KV cache (prefill, whole or chunked). Replaces the same reference code as
 * attn_decode_bf16 for long query blocks: head expansion
 * (astrai/extension/backend/attention.py:244-253), the mask tensor and SDPA
 * (:443-498), and the permute back to token-major of
 * astrai/model/components/attention.py:19-85. Key blocks that no query of a block may
 * see are skipped; the mask is computed from positions.
 *   q, k_cache, v_cache, positions  as for attn_decode_bf16 (keys at positions <= the
 *              largest positions[s] must have been written)
 *   out        bf16 [batch, seq, n_heads * 128]
 * bf16 MFMAs for q.k^T and p.v (p rounded to bf16, as SDPA's flash kernels do), fp32
 * softmax statistics and accumulation, one rounding of the output to bf16.
 * head_dim == 128, n_heads / n_kv_heads in {2, 4, 8}. Allocates nothing, no workspace.
 */
int astrai_w8a8_attn_prefill_bf16(const void* q_bf16, const void* k_cache_bf16,
                                  const void* v_cache_bf16, const int64_t* positions,
                                  void* out_bf16, int64_t batch, int64_t seq, int64_t n_heads,
                                  int64_t n_kv_heads, int64_t head_dim, int64_t max_len,
                                  float scale, void* stream);

/*
 * The same causal block attention over ragged sequences in a token-granular paged cache.
 * Replaces attn_paged_prefill (csrc/kernels/attention/paged_prefill.cu:4-52, addressing
 * policies PackedQSchedule / PagedKV in csrc/kernels/attention/layout_policies.cuh:67-93,
 * 174-232; Python wrapper astrai/extension/ops/attention.py:150-207); the variant with the
 * optional mask follows.
 *   q, out     bf16 [total_q, n_heads, 128]: the query rows of all sequences, packed
 *   k_pool, v_pool, req_to_token, req_pool_indices, kv_indptr  as for attn_paged_decode_bf16
 *   qo_indptr  int32 [batch + 1]: prefix sums of the sequences' query row counts
 *   q_tile_to_batch, q_tile_to_index  int32 [num_q_tiles]: the caller's schedule of 64-row
 *              query tiles (astrai/inference/cache/pool.py:219-234): sequence of tile t, and
 *              its index within that sequence
 *   causal     non-zero: row i of a sequence with q_len rows and kv_len keys attends keys
 *              0 .. kv_len - q_len + i (layout_policies.cuh:190-193); zero: all kv_len keys.
 *              A row that may see no key yields zeros.
 * Same arithmetic as attn_prefill_bf16. head_dim == 128, n_heads / n_kv_heads in {2, 4, 8},
 * num_slots * n_kv_heads * 256 < 2^32. Allocates nothing, no workspace.
 */
int astrai_w8a8_attn_paged_prefill_bf16(const void* q_bf16, const void* k_pool_bf16,
                                        const void* v_pool_bf16, const int32_t* req_to_token,
                                        const int32_t* req_pool_indices, const int32_t* kv_indptr,
                                        const int32_t* qo_indptr, const int32_t* q_tile_to_batch,
                                        const int32_t* q_tile_to_index, void* out_bf16,
                                        int64_t num_q_tiles, int64_t n_heads, int64_t n_kv_heads,
                                        int64_t head_dim, int64_t num_slots, int64_t num_requests,
                                        int64_t max_context_len, int causal, float scale,
                                        void* stream);

/*
 * attn_paged_prefill_bf16 with the reference's optional mask (the `mask` argument of
 * csrc/kernels/attention/paged_prefill.cu:14: 2D [batch, kv] or 4D [batch, 1 | n_heads,
 * rows, kv], packed into three strides at entry_utils.cuh:326-346 and applied at
 * mma_utils.cuh:190-199).
 *   mask       bool (one byte each); query row r (counted inside its sequence) of sequence b
 *              and head h attends position j, on top of the causal range, only where
 *              mask[b * mask_seq_stride + h * mask_head_stride + r * mask_row_stride + j] != 0.
 *              A stride of 0 broadcasts that axis (a 2D mask has head and row stride 0).
 *   mask_rows  rows the mask holds per sequence (used when mask_row_stride != 0): rows at or
 *              past it attend nothing and yield zeros
 *   mask_width positions a row of the mask holds: positions at or past it are not attended
 *              (the reference reads past the row in both cases). NULL mask: no mask.
 */
int astrai_w8a8_attn_paged_prefill_masked_bf16(
    const void* q_bf16, const void* k_pool_bf16, const void* v_pool_bf16,
    const int32_t* req_to_token, const int32_t* req_pool_indices, const int32_t* kv_indptr,
    const int32_t* qo_indptr, const int32_t* q_tile_to_batch, const int32_t* q_tile_to_index,
    const uint8_t* mask, int64_t mask_seq_stride, int64_t mask_head_stride, int64_t mask_row_stride,
    int64_t mask_rows, int64_t mask_width, void* out_bf16, int64_t num_q_tiles, int64_t n_heads,
    int64_t n_kv_heads, int64_t head_dim, int64_t num_slots, int64_t num_requests,
    int64_t max_context_len, int causal, float scale, void* stream);

/*
 * Paged attention for the shapes the tuned kernels above do not take: head_dim 32, 64, 128 or
 * 256 and any n_heads / n_kv_heads up to 16 -- the reference's paged kernels accept those
 * head_dims and any grouping (astrai/extension/backend/attention.py:518-527; its tests run
 * head_dim 64, tests/extension/conftest.py:9-20). One entry for both reference entries:
 *   qo_indptr == NULL  decode, as attn_paged_decode_masked_bf16: q / out [batch, n_heads,
 *              head_dim], batch_or_tiles = batch, causal ignored, mask rows / strides as for a
 *              2D mask (head and row stride 0)
 *   qo_indptr != NULL  ragged prefill, as attn_paged_prefill_masked_bf16: packed q / out
 *              [total_q, n_heads, head_dim], the 64-row tile schedule, batch_or_tiles = tiles
 * One wave per (block of up to 16 / (n_heads / n_kv_heads) query rows, KV head, context
 * split): bf16 MFMAs for the scores and for P.V (P as a bf16 head plus a bf16 remainder), fp32
 * softmax statistics and accumulation, one rounding of the output. Correct for every shape,
 * not tuned like the head_dim-128 kernels (prefill re-reads the keys once per row block).
 *   nsplit     in [1, 64]: 1 = every wave owns a whole context and writes the output itself,
 *              no workspace (NULL allowed); > 1 = partial results in the workspace and a
 *              merge kernel
 *   workspace  attn_paged_rows_workspace_floats(...) floats (0 for nsplit == 1; that function
 *              returns -1 for a shape this entry does not take)
 */
int64_t astrai_w8a8_attn_paged_rows_workspace_floats(int64_t batch_or_tiles, int64_t n_heads,
                                                     int64_t n_kv_heads, int64_t head_dim,
                                                     int64_t nsplit, int prefill);
int astrai_w8a8_attn_paged_rows_bf16(
    const void* q_bf16, const void* k_pool_bf16, const void* v_pool_bf16,
    const int32_t* req_to_token, const int32_t* req_pool_indices, const int32_t* kv_indptr,
    const int32_t* qo_indptr, const int32_t* q_tile_to_batch, const int32_t* q_tile_to_index,
    const uint8_t* mask, int64_t mask_seq_stride, int64_t mask_head_stride, int64_t mask_row_stride,
    int64_t mask_rows, int64_t mask_width, float* workspace, int64_t workspace_floats, void* out_bf16,
    int64_t batch_or_tiles, int64_t n_heads, int64_t n_kv_heads, int64_t head_dim, int64_t num_slots,
    int64_t num_requests, int64_t max_context_len, int causal, int64_t nsplit, float scale,
    void* stream);

/*
 * bf16 -> e4m3fn with one scale per 1x128 K-group (activations) or per 128x128
 * block (weights). No counterpart in the reference. K must be a multiple of 128.
 *   act:    sa[m,kb]  = max(max |x[m,128kb..128kb+127]|, 1e-12) / 448,   sa is [M, K/128]
 *   weight: sb[nb,kb] = max(max |w[128nb.., 128kb..]|, 1e-12) / 448,     sb is [ceil(N/128), K/128]
 */
int astrai_w8a8_quantize_bf16_fp8_block128_act(const void* x_bf16, void* x8, float* sa,
                                               int64_t m, int64_t k, void* stream);
int astrai_w8a8_quantize_bf16_fp8_block128_weight(const void* w_bf16, void* w8, float* sb,
                                                  int64_t n, int64_t k, void* stream);

/*
 * Pre-quantized fp8 GEMM with per-tensor scales.
 * Replaces mm_fp8 (csrc/kernels/fp8/mm.cu:128-184), fp8_pq_gemm_kernel
 * (gemm.cuh:447-619) and, with `bias`, the epilogue of fp8_fused_gemm_kernel
 * (gemm.cuh:405-435).
 *   acc[m,n] = sum_k a8[m,k] * b8[n,k]            fp32 accumulation
 *   OUT_BF16: out = bf16(acc * *sa * *sb + bias[n])   (bias bf16 [N] or NULL; one rounding)
 *   OUT_E4M3: out = sat_e4m3(acc * *sa * *sb * *out_scale)   (bias must be NULL)
 *   OUT_ACC : out = acc as fp32 (parity/debug surface; scales ignored)
 * a8 and b8 share `fmt`. At most 128 rows of `a8` with K % 256 == 0 (decode steps; bf16 or
 * accumulator output) run on the weight-streaming row-range kernel, as the int8 decode shapes do.
 * Any M, N, K >= 1 is accepted; the MFMA kernels fetch rows in 16-byte
 * pieces, so K % 16 != 0 (this and every other GEMM entry of this header) takes a plain any-shape
 * kernel that is some hundred times slower on large products: a caller with such a K should pad
 * both operands' rows with zero codes to a multiple of 128 (256 for at most 128 rows of `a8`),
 * which changes no sum -- the Python wrappers do so.
 */
int astrai_w8a8_gemm_fp8_pt(const void* a8, const void* b8, const float* sa,
                            const float* sb, const float* out_scale, const void* bias_bf16,
                            void* out, int64_t m, int64_t n, int64_t k, int fmt,
                            int out_dtype, void* stream);

/*
 * The per-tensor GEMM above with one scale per activation row and one per weight row:
 *   out[m,n] = bf16( (sum_k a8[m,k] * b8[n,k]) * sa[m] * sb[n] + bias[n] )
 * sa fp32 [M], sb fp32 [N]. The reference's CUDA binding takes scalars only
 * (csrc/kernels/fp8/mm.cu:49-54), but the arithmetic its ops are specified by,
 * `a.float() @ b.float().t() * sa * sb` (astrai/extension/ops/fp8.py:118), broadcasts
 * sa [M,1] and sb [N]; this entry is that broadcast on the device. bf16 output only.
 */
int astrai_w8a8_gemm_fp8_ptpc(const void* a8, const void* b8, const float* sa,
                              const float* sb, const void* bias_bf16, void* out_bf16,
                              int64_t m, int64_t n, int64_t k, int fmt, void* stream);

/*
 * Pre-quantized e4m3fn GEMM with 128-block scales. No counterpart in the
 * reference. K must be a multiple of 128.
 *   out[m,n] = bf16( sum_kb (sum_{k in kb} a8[m,k]*b8[n,k]) * sa[m,kb] * sb[n/128,kb] + bias[n] )
 * At most 64 rows of `a8` with K % 256 == 0 (decode steps) run on the weight-streaming row-range
 * kernel, as the per-tensor decode shapes do.
 */
int astrai_w8a8_gemm_fp8_block128(const void* a8, const void* b8, const float* sa,
                                  const float* sb, const void* bias_bf16, void* out,
                                  int64_t m, int64_t n, int64_t k, void* stream);

/*
 * int8 W8A8 GEMM, per-token x per-channel scales. No counterpart in the
 * reference; same NT layout and epilogue order as the fp8 path.
 *   acc[m,n] = sum_k a[m,k] * b[n,k]              exact int32
 *   OUT_BF16: out = bf16(float(acc) * sa[m] * sb[n] + bias[n])
 *   OUT_ACC : out = acc as int32 (bit-exact parity surface)
 * Picks a decode kernel for M <= 128 when K % 256 == 0 (one token: a dot-product kernel;
 * 2..128 tokens: the row-range MFMA kernel), the tiled MFMA kernels otherwise.
 */
int astrai_w8a8_gemm_int8_ptpc(const void* a, const void* b, const float* sa,
                               const float* sb, const void* bias_bf16, void* out,
                               int64_t m, int64_t n, int64_t k, int out_dtype,
                               void* stream);

/*
 * The decode int8 kernels on their own: same contract as
 * astrai_w8a8_gemm_int8_ptpc but requires M <= 128 and K % 256 == 0, and
 * returns ASTRAI_W8A8_UNSUPPORTED otherwise.
 */
int astrai_w8a8_gemv_int8_ptpc(const void* a, const void* b, const float* sa,
                               const float* sb, const void* bias_bf16, void* out,
                               int64_t m, int64_t n, int64_t k, int out_dtype,
                               void* stream);

/*
 * The fused q|k|v projection of a decoder layer with what follows it in the reference done
 * in the GEMM's epilogue: the rotary embedding of q and k (astrai/extension/backend/rotary.py:25-33),
 * the permutes and the KV-cache write (astrai/model/components/attention.py:19-85).
 * Equal, bit for bit, to astrai_w8a8_gemm_int8_ptpc (bf16 out, no bias) followed by
 * astrai_w8a8_rope_cache_write_bf16 on its output:
 *   a int8 [batch*seq, K] with sa fp32 [batch*seq]; b int8 [(n_heads + 2 n_kv_heads) * head_dim, K]
 *   (rows: q heads | k heads | v heads) with sb fp32 per row; freqs, positions, q_out,
 *   k_cache, v_cache as for astrai_w8a8_rope_cache_write_bf16.
 * Two shape classes: a few new tokens (decode steps: batch * seq <= 64, K % 256 == 0,
 * head_dim % 4 == 0; the row-range kernel) and long blocks (prefill: head_dim == 128, at least
 * 192 output tiles of 256 x 256, K % 128 == 0, K >= 256, q_out and each cache under 2 GiB; the
 * large-tile GEMM, one head per 128-column wave tile). ASTRAI_W8A8_UNSUPPORTED otherwise (run
 * the two calls instead).
 */
int astrai_w8a8_gemm_int8_ptpc_rope_cache(const void* a, const void* b, const float* sa,
                                          const float* sb, const float* freqs,
                                          const int64_t* positions, void* q_out_bf16,
                                          void* k_cache_bf16, void* v_cache_bf16, int64_t batch,
                                          int64_t seq, int64_t n_heads, int64_t n_kv_heads,
                                          int64_t head_dim, int64_t max_len, int64_t k,
                                          void* stream);

/*
 * The tiled MFMA int8 kernels on their own (no decode-kernel dispatch), for tests and
 * benchmarks that must name the kernel they measure.
 */
int astrai_w8a8_gemm_int8_ptpc_tiled(const void* a, const void* b, const float* sa,
                                     const float* sb, const void* bias_bf16, void* out,
                                     int64_t m, int64_t n, int64_t k, int out_dtype,
                                     void* stream);

/*
 * Diagnostic entry, not part of the path (the library's kernels never call it and no caller
 * of the path needs it). ONE MFMA instruction on a zero accumulator in a single 64-lane wave, for
 * known-answer tests of the lane layouts the kernels assume (what the reference checks
 * with csrc/tests/fp8_mma_test.cu:81-145 for its mma.sync shape). Operands are row-major
 * [R][K] matrices a (first operand) and b (second); lane l loads row l % R and the K bytes
 * of K-group l / R exactly as the GEMM / attention kernels do; d_raw receives every lane's
 * accumulator registers unpermuted, [64][4] (16-row shapes) or [64][16] (32-row shapes)
 * 32-bit words. The kernels assume D = a * b^T with
 *   16-row shapes: d_raw[l][j] = D[4 * (l / 16) + j][l % 16]
 *   32-row shapes: d_raw[l][r] = D[8 * (r / 4) + 4 * (l / 32) + r % 4][l % 32]
 * kind: 0 i32_16x16x64_i8 ([16][64] int8) | 1, 2 f32_16x16x128_f8f6f4 e4m3 / e5m2 ([16][128])
 *     | 3 i32_32x32x32_i8 ([32][32]) | 4, 5 f32_32x32x64_f8f6f4 e4m3 / e5m2 ([32][64])
 *     | 6 f32_16x16x32_bf16 ([16][32] bf16) | 7 f32_32x32x16_bf16 ([32][16] bf16)
 */
int astrai_w8a8_mfma_probe(int kind, const void* a, const void* b, void* d_raw, void* stream);

/* Diagnostic entry, not part of the path: the family name of the kernel that the calling
 * thread's most recent GEMM entry launched ("wave128_q16", "wave128", "wave128_swiglu",
 * "wave128_rope", "wave128_resid", "pingpong", "pingpong_block128", "mid128", "mid128_block128",
 * "tiled_256", "tiled_128", "tiled_64", "generic", "gemv_dot", "gemv_rows", "gemv_rows_rope",
 * "gemv_rows_fp8", "gemv_rows_fp8_block128"; "" before the first launch). A product sent out as
 * whole 256-row tiles plus a ragged tail on the decode kernel reports the tile kernel. For tests
 * and shape surveys that record which kernel a Linear of a given shape lands on; the static
 * string lives as long as the library. No counterpart in the reference. */
const char* astrai_w8a8_last_kernel(void);

#ifdef __cplusplus
}
#endif
#endif /* ASTRAI_W8A8_H */
