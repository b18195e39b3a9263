// Host entry of the fused ratio-4 decode prep: two launches on one stream (score row with the query
// QAT staged as float16, with the prepared KV row as one more workgroup of the same launch; radix
// top-k). The reference runs the same phases inside a single 1024-thread workgroup; here the score
// row is spread over the whole device.
#include "common.h"

int mspr_launch_scores_f32(const void* q, int q_dtype, int n_heads, const float* pooled, int64_t n_rows,
                           const float* weights, float scale, float* scores, bool stage_half, const void* kv_row,
                           const float* inv_freq, const int32_t* params, void* row_out, const int32_t* valid_rows,
                           hipStream_t st);
int mspr_launch_topk(const float* scores, int64_t score_stride, int batch, int64_t n_rows, int topk, int32_t* sel,
                     hipStream_t st);

static int decode_prep(const void* q_idx, int q_dtype, int n_heads, const float* pooled_qat, int64_t n_rows,
                       const float* weights, const void* kv_row, const float* inv_freq, const int32_t* params,
                       float scale, int topk, int32_t* sel, void* row_out, float* scores, bool fixed, void* stream) {
  MSPR_REQUIRE(q_idx && pooled_qat && weights && kv_row && inv_freq && params && sel && row_out && scores,
               "fused_decode_prep: null pointer");
  MSPR_REQUIRE(n_heads >= 1 && n_heads <= 64, "fused_decode_prep: q_idx must carry between 1 and 64 heads");
  MSPR_REQUIRE(q_dtype >= MSPR_F32 && q_dtype <= MSPR_BF16, "fused_decode_prep: q_idx must be f32, f16 or bf16");
  MSPR_REQUIRE(n_rows >= 1 && n_rows < (int64_t)1 << 31, "fused_decode_prep: n_rows out of range");
  MSPR_REQUIRE(topk > 0 && topk < n_rows, "fused_decode_prep: topk must be positive and smaller than n_rows");
  MSPR_REQUIRE(mspr_aligned(q_idx, 16) && mspr_aligned(pooled_qat, 16) && mspr_aligned(kv_row, 16) &&
                   mspr_aligned(row_out, 16),
               "fused_decode_prep: q_idx, pooled_qat, kv_row and row_out must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  int rc = mspr_launch_scores_f32(q_idx, q_dtype, n_heads, pooled_qat, n_rows, weights, scale, scores, true, kv_row,
                                  inv_freq, params, row_out, fixed ? params + 2 : nullptr, st);
  if (rc != MSPR_OK) return rc;
  return mspr_launch_topk(scores, n_rows, 1, n_rows, topk, sel, st);
}

extern "C" int mspr_fused_decode_prep(const void* q_idx, int q_dtype, int n_heads, const float* pooled_qat,
                                      int64_t n_rows, const float* weights, const void* kv_row,
                                      const float* inv_freq, const int32_t* params, float scale, int topk,
                                      int32_t* sel, void* row_out, float* scores, void* stream) {
  return decode_prep(q_idx, q_dtype, n_heads, pooled_qat, n_rows, weights, kv_row, inv_freq, params, scale, topk, sel,
                     row_out, scores, false, stream);
}

extern "C" int mspr_fused_decode_prep_fixed(const void* q_idx, int q_dtype, int n_heads, const float* pooled_qat,
                                            int64_t capacity, const float* weights, const void* kv_row,
                                            const float* inv_freq, const int32_t* params, float scale, int topk,
                                            int32_t* sel, void* row_out, float* scores, void* stream) {
  return decode_prep(q_idx, q_dtype, n_heads, pooled_qat, capacity, weights, kv_row, inv_freq, params, scale, topk,
                     sel, row_out, scores, true, stream);
}
