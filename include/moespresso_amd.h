/*
 * C-ABI of libmoespresso_amd.so: hand-written gfx950 (MI355X) kernels for the
 * MoEspresso attention hot path.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the comment says "host";
 *   - tensors are dense row-major with the shapes given, no strides;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); the
 *     call only enqueues work, it never synchronises and never allocates;
 *   - scratch memory is passed in by the caller (`workspace`), its size comes
 *     from the matching *_workspace_bytes function;
 *   - return value 0 = enqueued; MSPR_ERR_ARG = rejected before any launch
 *     (shape / dtype / alignment / workspace too small); MSPR_ERR_LAUNCH = HIP
 *     reported a launch error. mspr_last_error() gives the reason as text.
 *
 * Each entry point cites the reference interface it stands in for (paths under
 * the reference tree). Entry points marked "extension" have the BASELINE
 * configuration shapes (batch > 1, fp8 keys, 576/512 MLA, bf16, g32 Q8) that
 * the reference's own callables reject.
 */
#ifndef MOESPRESSO_AMD_H
#define MOESPRESSO_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MSPR_OK 0
#define MSPR_ERR_ARG (-1)
#define MSPR_ERR_LAUNCH (-2)

/* element type codes */
#define MSPR_F32 0
#define MSPR_F16 1
#define MSPR_BF16 2

/* Library ABI version (bumped on any signature change). */
int mspr_abi_version(void);

/* Text of the last error raised on the calling thread ("" if none). */
const char* mspr_last_error(void);

/* ------------------------------------------------------------------ DS4 indexer */

/* Hadamard-128 + e2m1 activation round trip over 128-wide rows, float32 out.
 * Replaces indexer_qat_rows, src/moespresso/runtime/deepseek_v4/indexer_score_kernel.py:284
 * (= _dsv4_indexer_qat, model.py:745). x: [n_rows,128] of x_dtype; out: f32 [n_rows,128]. */
int mspr_indexer_qat_rows(const void* x, int x_dtype, int64_t n_rows, float* out, void* stream);

/* Decode score row with the query QAT applied in-kernel:
 *   scores[r] = sum_h max(qat(q_h) . pooled[r], 0) * scale * weights[h]
 * Replaces fused_qat_indexer_scores, indexer_score_kernel.py:354.
 * q: [n_heads,128] of q_dtype (1..64 heads); pooled_qat: f32 [n_rows,128];
 * weights: f32 [n_heads]; scores: f32 [n_rows]. */
int mspr_fused_qat_indexer_scores(const void* q, int q_dtype, int n_heads, const float* pooled_qat,
                                  int64_t n_rows, const float* weights, float scale, float* scores,
                                  void* stream);

/* relu, score scale, head-weight cast and n_heads^-1/2 scale, head sum, capacity pad, negate.
 * Replaces fused_score_tail, indexer_score_kernel.py:562.
 * scores: f32 [n_heads,capacity] (32..64 heads); weights_raw: [n_heads] of w_dtype;
 * params: int32 [>=2], params[1] = valid columns; neg: f32 [capacity]. */
int mspr_indexer_score_tail(const float* scores, int n_heads, int64_t capacity, const void* weights_raw,
                            int w_dtype, const int32_t* params, float scale, float* neg, void* stream);

/* E4M3FN round trip of dims [0,448) in 64-blocks of 512-wide float32 rows, tail copied.
 * Replaces fp8_kv_prefix_rows, decode_attention_kernel.py:587
 * (= _deepseek_v4_fp8_kv_roundtrip, model.py:559). x/out: f32 [n_rows,512]. */
int mspr_fp8_kv_prefix_rows(const float* x, int64_t n_rows, float* out, void* stream);

/* Deterministic top-k over float32 score rows: rows whose monotone key is strictly above the
 * k-th value in ascending row order, then the lowest-index rows tied with it.
 * Stands in for mx.argpartition(-scores, kth=k-1)[..., :k] (model.py:1003,1057,1443) with the
 * emission order of the prep kernel's phase C, decode_attention_kernel.py:295-375.
 * scores: f32 [batch,n_rows] (row b at scores + b*score_stride); sel: int32 [batch,topk];
 * 0 < topk <= n_rows. No 16-bit row limit. */
int mspr_topk_select(const float* scores, int64_t score_stride, int batch, int64_t n_rows, int topk,
                     int32_t* sel, void* stream);

/* One ratio-4 decode token: in-kernel query QAT (staged as float16), score row, deterministic
 * top-k, and the prepared KV row (rope tail + E4M3FN prefix round trip).
 * Replaces fused_decode_prep, decode_attention_kernel.py:669.
 * q_idx: [n_heads,128] of q_dtype; pooled_qat: f32 [n_rows,128]; weights: f32 [n_heads];
 * kv_row: f16 [512]; inv_freq: f32 [32]; params: int32, params[0] = position;
 * outputs sel: int32 [topk], row_out: f16 [512], scores: f32 [n_rows]. 0 < topk < n_rows. */
int mspr_fused_decode_prep(const void* q_idx, int q_dtype, int n_heads, const float* pooled_qat,
                           int64_t n_rows, const float* weights, const void* kv_row,
                           const float* inv_freq, const int32_t* params, float scale, int topk,
                           int32_t* sel, void* row_out, float* scores, void* stream);

/* fused_decode_prep over a fixed-capacity pool: pooled_qat holds `capacity` rows of which the first
 * params[2] are in use; params: int32 [position, ring write index, pool rows in use] ON THE DEVICE, so a
 * launch recorded into a HIP graph follows the pool as it grows (the caller appends rows to the buffer
 * and rewrites params between replays). Rows not in use score -inf; with topk <= rows in use the
 * selection and its order equal mspr_fused_decode_prep on the first params[2] rows bit for bit, with
 * fewer rows in use the surplus ids name unused rows, which mspr_fused_decode_sdpa_fixed skips.
 * The counterpart of the fixed-capacity decode state, runtime/deepseek_v4/fixed_decode_state.py:186-206
 * (decode_step_params, pad_scores_to_capacity) and :215-288 (capacity buffers of the derived caches).
 * scores: f32 [capacity]; 0 < topk < capacity. */
int mspr_fused_decode_prep_fixed(const void* q_idx, int q_dtype, int n_heads, const float* pooled_qat,
                                 int64_t capacity, const float* weights, const void* kv_row,
                                 const float* inv_freq, const int32_t* params, float scale, int topk,
                                 int32_t* sel, void* row_out, float* scores, void* stream);

/* Extension (BASELINE config 4): batched lightning-indexer scores with FP8 keys.
 *   scores[b,r] = sum_h w[b,h] * relu(q[b,h] . e4m3(keys[b,r])) * key_scales[b,r]
 * q: bf16 [batch,n_heads,128] (n_heads <= 64); keys: E4M3FN bytes [batch,n_rows,128];
 * key_scales: f32 [batch,n_rows] (> 0); weights: f32 [batch,n_heads]; scores: f32 [batch,n_rows]. */
int mspr_indexer_scores_fp8(const void* q, const void* keys, const float* key_scales,
                            const float* weights, int batch, int n_heads, int64_t n_rows,
                            float* scores, void* stream);

/* Prefill-side QAT of query rows: the Hadamard of mspr_indexer_qat_rows with the group scale
 * 2^ceil(log2(amax/6)) and ties in the lattice search going to the even lattice index.
 * Replaces indexer_q_qat_live, indexed_attention_kernel.py:1989 (kernel :1125-1202).
 * q/out: f32 [n_rows,128] (the [batch,n_heads,tokens,128] tensor, contiguous). */
int mspr_indexer_q_qat_live(const float* q, int64_t n_rows, float* out, void* stream);

/* Prefill-side indexer scores over a chunk:
 *   scores[b,t,c] = sum_h max(q[b,h,t] . comp[b,c], 0) * weights[b,t,h], -inf where c >= (pos0+t+1)/ratio
 * with both operands staged as float16 (ratio 0 = whole pool visible).
 * Replaces indexer_scores_tiled_live, indexed_attention_kernel.py:1888 (kernel :1028-1122).
 * q: [batch,n_heads,n_tokens,128], index_comp: [batch,n_comp,128], both of dtype (f32|f16);
 * weights: f32 [batch,n_tokens,n_heads]; scores: f32 [batch,n_tokens,n_comp]. n_heads <= 64. */
int mspr_indexer_scores_tiled_live(const void* q, const float* weights, const void* index_comp, int dtype,
                                   int batch, int n_heads, int n_tokens, int64_t n_comp, int64_t pos0,
                                   int ratio, float* scores, void* stream);

/* ------------------------------------------------------------------ DS4 sparse attention */

/* Scratch bytes for the gathered-attention entry points below. */
size_t mspr_sparse_attention_workspace_bytes(int batch, int n_heads, int64_t n_keys);

/* Scratch bytes for mspr_indexed_mixed_attention_prefill: the per-range partials of calls that take one workgroup
 * per token, or the half-precision copy of float32 queries (batch*n_tokens*n_heads*512*2 bytes), whichever is
 * larger. window_rows is the largest number of ring rows a token attends. No counterpart in the reference
 * (its kernels allocate through MLX). */
size_t mspr_indexed_mixed_attention_prefill_workspace_bytes(int q_dtype, int batch, int n_heads, int n_tokens,
                                                            int window_rows, int top_k);

/* One-token indexed mixed attention over a ring of raw rows plus gathered pool rows, K == V.
 * Replaces indexed_mixed_attention_decode, indexed_attention_kernel.py:1496 (kernel :61-174).
 * q: f32 [n_heads,512] (rounded to half on load); raw_kv: f16 [raw_cap,512];
 * comp_kv: f16 [n_comp,512]; topk: int32 [top_k]; sinks: f32 [n_heads]; out: f32 [n_heads,512].
 * Ids < 0 are skipped; the first id >= min((pos0+1)/ratio, n_comp) ends the walk
 * (ratio 0 = whole pool visible). */
int mspr_indexed_mixed_attention_decode(const float* q, int n_heads, const void* raw_kv, int raw_cap,
                                        const void* comp_kv, int64_t n_comp, const int32_t* topk,
                                        int top_k, const float* sinks, int64_t pos0, int window,
                                        int ratio, int raw_start, float* out, void* workspace,
                                        size_t workspace_bytes, void* stream);

/* Indexed mixed attention for every token of a prefill chunk: token t (position pos0+t) attends
 * the ring rows for positions [max(first_raw, pos0+t+1-window), pos0+t], where the newest ring
 * row holds position pos0+n_tokens-1, then its own topk ids under the rules of the decode form
 * with visible = min((pos0+t+1)/ratio, n_comp).
 * Replaces indexed_mixed_attention_prefill (:2030), indexed_mixed_attention_prefill_live_f16
 * (:1571), _live_f32 (:1679) and banded_prefill_attention_live (:1782) of
 * indexed_attention_kernel.py; the three layouts differ only in strides.
 * q: element (b,t,head,:) at b*q_batch_stride + t*q_token_stride + head*q_head_stride (elements),
 * 512 contiguous values of q_dtype (f32 rounded to half on load, or f16); raw_kv: f16
 * [batch,raw_cap,512]; comp_kv: f16 [batch,n_comp,512]; topk: int32 [batch,n_tokens,top_k]
 * (top_k may be 0); sinks: f32 [n_heads]; out: f32 with the strides of q.
 * Calls whose slot count fits 22 tiles of 32 (window and ids each rounded up to whole tiles) run on one
 * persistent workgroup per CU that streams consecutive tokens; float32 queries are first rounded to half into
 * the workspace. Other calls take one workgroup per token and key range (every call does with
 * MSPR_PREFILL_PERSISTENT=0 in the environment, read per call). The arguments and the workspace size asked
 * for are the same either way.
 * Workspace: mspr_indexed_mixed_attention_prefill_workspace_bytes(q_dtype, batch, n_heads, n_tokens,
 * min(window or raw_cap, raw_cap), top_k). */
int mspr_indexed_mixed_attention_prefill(const void* q, int q_dtype, int batch, int n_heads, int n_tokens,
                                         int64_t q_batch_stride, int64_t q_head_stride,
                                         int64_t q_token_stride, const void* raw_kv, int raw_cap,
                                         const void* comp_kv, int64_t n_comp, const int32_t* topk, int top_k,
                                         const float* sinks, int64_t pos0, int window, int ratio,
                                         int raw_start, float* out, void* workspace, size_t workspace_bytes,
                                         void* stream);

/* Decode SDPA of the fused island: rope(q), softmax over the window (row substituted at
 * params[1]) + pooled[sel] + per-head sink, float16 output, inverse rope.
 * Replaces fused_decode_sdpa, decode_attention_kernel.py:733.
 * q: f16 [n_heads,512]; window: f16 [window_rows,512]; row: f16 [512]; pooled: f16 [n_rows,512];
 * sel: int32 [n_sel]; sinks: f16 [n_heads]; inv_freq: f32 [32]; params: int32 [position, write_idx];
 * out: f16 [n_heads,512]. */
int mspr_fused_decode_sdpa(const void* q, int n_heads, const void* window, int window_rows,
                           const void* row, const void* pooled, int64_t n_rows, const int32_t* sel,
                           int n_sel, const void* sinks, const float* inv_freq, const int32_t* params,
                           float scale, void* out, void* workspace, size_t workspace_bytes,
                           void* stream);

/* fused_decode_sdpa over a fixed-capacity pool: pooled holds `capacity` rows, params is int32
 * [position, ring write index, pool rows in use] on the device; ids in sel that are negative or name a
 * row not in use are skipped. Same arithmetic as mspr_fused_decode_sdpa otherwise (fixed-capacity decode
 * state, fixed_decode_state.py:186-206). */
int mspr_fused_decode_sdpa_fixed(const void* q, int n_heads, const void* window, int window_rows,
                                 const void* row, const void* pooled, int64_t capacity, const int32_t* sel,
                                 int n_sel, const void* sinks, const float* inv_freq, const int32_t* params,
                                 float scale, void* out, void* workspace, size_t workspace_bytes,
                                 void* stream);

/* Extension (BASELINE config 5): batched sparse multi-head latent decode attention.
 * Every head of batch b attends rows kv[b, rows[b, :]] of a shared latent cache; K is the whole
 * k_dim-wide row and V its first v_dim columns.
 * q: [batch,n_heads,k_dim] of dtype (f16|bf16); kv: [batch,n_pool,k_dim] same dtype;
 * rows: int32 [batch,n_rows] gathered ids, pool row = id*row_mul + row_add (negative ids and rows
 * outside the pool are skipped; row_mul 1, row_add 0 for plain row ids); the contiguous
 * window kv[b, win_start : win_start+win_rows] is attended as well (win_rows may be 0);
 * sinks: f32 [n_heads] or NULL; out: [batch,n_heads,v_dim] same dtype.
 * k_dim in {512,576}, v_dim = 512, n_heads <= 128. */
int mspr_sparse_mla_decode(const void* q, const void* kv, const int32_t* rows, const float* sinks,
                           int dtype, int batch, int n_heads, int k_dim, int v_dim, int64_t n_pool,
                           int n_rows, int row_mul, int row_add, int64_t win_start, int win_rows,
                           float scale, void* out, void* workspace, size_t workspace_bytes, void* stream);

/* mspr_sparse_mla_decode without a workspace argument and without any allocation, for callers that
 * cannot allocate: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * No counterpart in the reference. The per-range partials live in a scratch array that is
 * part of the library's device image (mspr_sparse_mla_decode_static_max_bytes() = 16,908,288 bytes, held
 * by every GPU the library runs on until the process ends), which bounds the call to 256 key ranges:
 * every shape with batch * ceil(n_heads/64) <= 256 whose rows fit 960 per range (batch 16 at 2176 rows,
 * batch 256 at 960) is accepted, anything larger is rejected with MSPR_ERR_ARG before any launch.
 * All calls on one GPU share the array: calls that overlap on a GPU (two streams, two threads) race. */
int mspr_sparse_mla_decode_static(const void* q, const void* kv, const int32_t* rows, const float* sinks,
                                  int dtype, int batch, int n_heads, int k_dim, int v_dim, int64_t n_pool,
                                  int n_rows, int row_mul, int row_add, int64_t win_start, int win_rows,
                                  float scale, void* out, void* stream);
size_t mspr_sparse_mla_decode_static_max_bytes(void);

/* Partial rotary embedding of the last 64 channels of rows laid out [n_outer, seq_len, width]
 * (interleaved pairs); the leading channels copy through.
 * Replaces fused_partial_rope, runtime/deepseek_v4/attention_seam_kernel.py:247 (the composed
 * _apply_partial_rope sequence at element-type rounding; kernel source :80-118).
 * x/out: dtype f32|f16|bf16, 16-byte aligned; inv_freq: float32 [32]; positions: float32 [seq_len] or
 * NULL (then row l of the sequence axis sits at position offset + l, offset + seq_len <= 2^24);
 * inverse != 0 negates the sine. */
int mspr_fused_partial_rope(const void* x, int dtype, int64_t n_outer, int64_t seq_len, int width,
                            const float* inv_freq, const float* positions, int64_t offset, int inverse,
                            void* out, void* stream);

/* ------------------------------------------------------------------ Qwen/Ornith GQA attention, 8-bit KV */

/* Affine 8-bit quantisation in groups of 64 over the last axis and its inverse: the cache write
 * path in front of the two attention operators below.
 * Stands in for mx.quantize / mx.dequantize (group_size=64, bits=8) as used by the quantised KV
 * cache's update and by the self-chunk round trip, runtime/qwen/full_attention.py:352-369.
 * x/out: [n_groups*64] of dtype (f32|f16|bf16); wq: uint32 [n_groups*16], four codes per word,
 * lowest byte first; scales, biases: [n_groups] of dtype; value = code*scale + bias. */
int mspr_affine_q8_quantize(const void* x, int dtype, int64_t n_groups, void* wq, void* scales,
                            void* biases, int group_size, int bits, void* stream);
int mspr_affine_q8_dequantize(const void* wq, const void* scales, const void* biases, int dtype,
                              int64_t n_groups, void* out, int group_size, int bits, void* stream);

/* Workspace bytes of the two Q8 decode entry points below. */
size_t mspr_sdpa_decode_q8_workspace_bytes(int batch, int n_kv_heads, int64_t n_keys);

/* One-token GQA decode attention over an MLX affine 8-bit KV cache, dequantised in-kernel.
 * Replaces mlx_kquant.sdpa_decode_q8 as called from runtime/qwen/full_attention.py:323
 * (third-party Metal operator, not vendored; arguments follow that call site).
 * queries: f32 [batch,n_q_heads,1,256]; k_wq/v_wq: uint32 [batch,n_kv_heads,kv_rows,64] (four codes
 * per word, lowest byte first); scales and biases: [batch,n_kv_heads,kv_rows,4] of sb_dtype,
 * value = code*scale + bias per 64 elements; out: f32 [batch,n_q_heads,1,256].
 * kv_rows >= n_keys is the row capacity of the cache buffers: the first n_keys rows of every head are
 * attended, so a cache that grows in blocks is passed as it lies in memory, without a trimmed copy.
 * group_size must be 64 and bits 8; n_q_heads/n_kv_heads <= 16. */
int mspr_sdpa_decode_q8(const void* queries, int q_dtype, const void* k_wq, const void* k_scales,
                        const void* k_biases, const void* v_wq, const void* v_scales,
                        const void* v_biases, int sb_dtype, int batch, int n_q_heads, int n_kv_heads,
                        int head_dim, int64_t n_keys, int64_t kv_rows, float scale, int group_size, int bits,
                        void* out, void* workspace, size_t workspace_bytes, void* stream);

/* Extension (BASELINE config 3): the same decode over a Q8_0 cache — int8 codes
 * [batch,n_kv_heads,kv_rows,256] with one float16 scale per 32 elements
 * [batch,n_kv_heads,kv_rows,8], value = code*scale (the first n_keys rows of every head are attended).
 * queries/out: [batch,n_q_heads,256] of q_dtype (f32|f16|bf16). */
int mspr_sdpa_decode_q8_0(const void* queries, int q_dtype, const void* k_codes, const void* k_scales,
                          const void* v_codes, const void* v_scales, int batch, int n_q_heads,
                          int n_kv_heads, int head_dim, int64_t n_keys, int64_t kv_rows, float scale,
                          void* out, void* workspace, size_t workspace_bytes, void* stream);

/* Causal chunked-prefill GQA attention over a dense 16-bit KV cache that already holds the chunk:
 * query row i (position past_len + i) attends keys [0, past_len + i].
 * Stands in for mx.fast.scaled_dot_product_attention(mask="causal") over the fetched cache, the
 * composed prefill route of runtime/qwen/full_attention.py:399-409, at BASELINE config 2.
 * q/out: [batch,n_q_heads,q_len,256] of dtype (f16|bf16); k, v: [batch,n_kv_heads,kv_rows,256]
 * same dtype, rows [0, past_len+q_len) valid; n_q_heads/n_kv_heads in {1,2,4,8}. */
int mspr_flash_prefill(const void* q, const void* k, const void* v, int dtype, int batch, int n_q_heads,
                       int n_kv_heads, int head_dim, int q_len, int64_t past_len, int64_t kv_rows,
                       float scale, void* out, void* workspace, size_t workspace_bytes, void* stream);

/* Workspace bytes of mspr_flash_prefill (key-range partials of short chunks; 256 when none are needed). */
size_t mspr_flash_prefill_workspace_bytes(int batch, int n_q_heads, int n_kv_heads, int q_len,
                                          int64_t past_len);

/* Workspace bytes of mspr_sdpa_fa_prefill_q8 (float16 copies of the chunk's own K/V rows, plus the
 * key-range partials when a short chunk over a deep prefix is split to fill the device). */
size_t mspr_sdpa_fa_prefill_q8_workspace_bytes(int batch, int n_q_heads, int n_kv_heads, int q_len,
                                               int64_t past_len);

/* Causal flash prefill over an affine 8-bit prefix plus the dense chunk itself: query row i attends
 * every prefix key and chunk keys [0, i].
 * Replaces mlx_kquant.sdpa_fa_prefill_q8 as called from runtime/qwen/full_attention.py:372
 * (third-party Metal operator, not vendored; arguments follow that call site and the helper at
 * tests/test_qwen_flash_prefill_attention.py:361-375).
 * queries/out: f32 [batch,n_q_heads,q_len,256]; pk_wq/pv_wq: uint32 [batch,n_kv_heads,past_rows,64];
 * their scales and biases: [batch,n_kv_heads,past_rows,4] of sb_dtype, past_rows >= past_len being the
 * row capacity of the prefix buffers (the first past_len rows of every head are the prefix);
 * self_k/self_v: [batch,n_kv_heads,q_len,256] of self_dtype (already passed through the 8-bit round
 * trip by the caller). past_len may be 0 (the prefix pointers are then ignored).
 * The chunk's own rows, the last past_len % 32 prefix rows and the queries are staged as float16 MFMA
 * operands whatever self_dtype is: chunk rows beyond +-65504 saturate there, queries beyond it become
 * infinite, and everything keeps 11 significant bits. */
int mspr_sdpa_fa_prefill_q8(const void* queries, const void* pk_wq, const void* pk_scales,
                            const void* pk_biases, const void* pv_wq, const void* pv_scales,
                            const void* pv_biases, int sb_dtype, const void* self_k, const void* self_v,
                            int self_dtype, int batch, int n_q_heads, int n_kv_heads, int head_dim,
                            int q_len, int64_t past_len, int64_t past_rows, float scale, int group_size,
                            int bits, void* out, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ measurement */

/* Per-kernel GPU timing for benchmarks. Bit k of kernel_mask brackets every later launch of kernel
 * k with HIP events on the launch stream (0 switches it off; it must be off under stream capture).
 * Kernel ids: 1 fp8 indexer scores, 2 top-k, 3 sparse attention split, 4 sparse attention merge,
 * 5 float32 indexer scores, 6 Q8 decode split, 7 Q8 decode merge, 8 flash prefill.
 * No counterpart in the reference (its probes time whole calls on the host). These two are the
 * exception to "never allocates, never synchronises": enabling makes the launchers create HIP events
 * (kept and reused), and mspr_profile_collect waits for the recorded launches. */
int mspr_profile_enable(int kernel_mask);

/* Waits for the recorded launches of kernel_id, writes their durations in milliseconds to the HOST
 * array ms_out (at most max_n) and forgets them; returns how many were written. */
int mspr_profile_collect(int kernel_id, float* ms_out, int max_n);

#ifdef __cplusplus
}
#endif
#endif /* MOESPRESSO_AMD_H */
