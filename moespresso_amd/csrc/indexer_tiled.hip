// Prefill-side lightning-indexer scores over a chunk of tokens:
//   scores[b,t,c] = sum_h max(q[b,h,t] . comp[b,c], 0) * w[b,t,h],  -inf where c >= (pos0+t+1)/ratio
// Operands are staged as float16 (float32 inputs are rounded on load), products accumulate in float32
// on v_mfma_f32_32x32x16_f16 with heads = M and pool rows = N, so the relu / weight / head sum runs on
// the accumulator registers of one lane column per pool row.
//
// Workgroup = 4 waves = 4 consecutive tokens of one batch entry walking the same block of pool rows
// (the rows are re-used out of L1/L2); the token's 64 x 128 query block stays in registers.
#include "common.h"
#include "profile.h"

namespace {

constexpr int kRowsPerBlock = 256;  // pool rows per workgroup (8 tiles of 32)

__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
  typedef __attribute__((ext_vector_type(2))) _Float16 h2_t;
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{a, b}, h2_t));
}

// eight consecutive elements starting at element offset `off` as packed float16
template <int DT>
__device__ __forceinline__ u32x4_t load8_as_f16(const void* base, int64_t off) {
  if constexpr (DT == MSPR_F16) {
    return *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const uint16_t*>(base) + off);
  } else {
    const f32x4_t* p = reinterpret_cast<const f32x4_t*>(reinterpret_cast<const float*>(base) + off);
    const f32x4_t a = p[0], b = p[1];
    return u32x4_t{pack_h2(a.x, a.y), pack_h2(a.z, a.w), pack_h2(b.x, b.y), pack_h2(b.z, b.w)};
  }
}

template <int DT>
__global__ __launch_bounds__(256) void scores_tiled_kernel(const void* __restrict__ q, const float* __restrict__ w,
                                                           const void* __restrict__ comp, int n_heads, int n_tokens,
                                                           int64_t n_comp, uint32_t pos0, uint32_t ratio,
                                                           float* __restrict__ scores) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n = lane & 31;
  const int g = lane >> 5;
  const int b = blockIdx.z;
  int t = blockIdx.y * 4 + wave;
  const bool t_live = t < n_tokens;
  if (!t_live) t = n_tokens - 1;

  // A operand: q[b, head, t, 16 s + 8 g .. +7] for head = n (+32), zero rows past n_heads
  u32x4_t qa[2][8];
#pragma unroll
  for (int hb = 0; hb < 2; hb++) {
    const int head = 32 * hb + n;
    const bool live = head < n_heads;
    const int64_t off = (((int64_t)b * n_heads + (live ? head : 0)) * n_tokens + t) * 128 + 8 * g;
#pragma unroll
    for (int s = 0; s < 8; s++) {
      u32x4_t v = load8_as_f16<DT>(q, off + 16 * s);
      qa[hb][s] = live ? v : u32x4_t{0, 0, 0, 0};
    }
  }
  // weights of the heads this lane's accumulator registers hold: head = 32 hb + 8 (i/4) + 4 g + i%4
  float wv[2][16];
#pragma unroll
  for (int hb = 0; hb < 2; hb++)
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int head = 32 * hb + 8 * (i / 4) + 4 * g + (i % 4);
      wv[hb][i] = head < n_heads ? w[((int64_t)b * n_tokens + t) * n_heads + head] : 0.0f;
    }
  const uint32_t qpos1 = pos0 + (uint32_t)t + 1u;
  const int64_t visible_raw = ratio == 0u ? n_comp : (int64_t)(qpos1 / ratio);
  const int64_t visible = visible_raw < n_comp ? visible_raw : n_comp;

  const int64_t row_begin = (int64_t)blockIdx.x * kRowsPerBlock;
  int64_t row_end = row_begin + kRowsPerBlock;
  if (row_end > n_comp) row_end = n_comp;
  const void* comp_b = DT == MSPR_F16
                           ? static_cast<const void*>(reinterpret_cast<const uint16_t*>(comp) + (int64_t)b * n_comp * 128)
                           : static_cast<const void*>(reinterpret_cast<const float*>(comp) + (int64_t)b * n_comp * 128);
  for (int64_t r0 = row_begin; r0 < row_end; r0 += 32) {
    int64_t row = r0 + n;
    if (row >= n_comp) row = n_comp - 1;
    u32x4_t kb[8];
#pragma unroll
    for (int s = 0; s < 8; s++) kb[s] = load8_as_f16<DT>(comp_b, row * 128 + 16 * s + 8 * g);
    f32x16_t acc0 = {0}, acc1 = {0};
#pragma unroll
    for (int s = 0; s < 8; s++) {
      acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, qa[0][s]),
                                                    __builtin_bit_cast(f16x8_t, kb[s]), acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, qa[1][s]),
                                                    __builtin_bit_cast(f16x8_t, kb[s]), acc1, 0, 0, 0);
    }
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      sum += fmaxf(acc0[i], 0.0f) * wv[0][i];
      sum += fmaxf(acc1[i], 0.0f) * wv[1][i];
    }
    sum += __shfl_xor(sum, 32, MSPR_WAVE);
    const int64_t c = r0 + n;
    if (t_live && g == 0 && c < row_end)
      scores[((int64_t)b * n_tokens + t) * n_comp + c] = c < visible ? sum : -__builtin_inff();
  }
}

}  // namespace

extern "C" int mspr_indexer_scores_tiled_live(const void* q, const float* weights, const void* index_comp, int dtype,
                                              int batch, int n_heads, int n_tokens, int64_t n_comp, int64_t pos0,
                                              int ratio, float* scores, void* stream) {
  MSPR_REQUIRE(q && weights && index_comp && scores, "indexer_scores_tiled_live: null pointer");
  MSPR_REQUIRE(dtype == MSPR_F32 || dtype == MSPR_F16,
               "indexer_scores_tiled_live: q and index_comp must both be float32 or both be float16");
  MSPR_REQUIRE(batch >= 1 && n_tokens >= 1, "indexer_scores_tiled_live: q must contain at least one batch and token");
  MSPR_REQUIRE(n_heads >= 1 && n_heads <= 64, "indexer_scores_tiled_live: between 1 and 64 heads");
  MSPR_REQUIRE(n_comp >= 1, "indexer_scores_tiled_live: index_comp must contain at least one compressed row");
  MSPR_REQUIRE(pos0 >= 0 && ratio >= 0 && pos0 + n_tokens < ((int64_t)1 << 31) && batch <= 65535,
               "indexer_scores_tiled_live: bad size argument");
  MSPR_REQUIRE(mspr_aligned(q, 16) && mspr_aligned(index_comp, 16),
               "indexer_scores_tiled_live: pointers must be 16-byte aligned");
  const int64_t row_blocks = (n_comp + kRowsPerBlock - 1) / kRowsPerBlock;
  const int64_t tok_blocks = (n_tokens + 3) / 4;
  MSPR_REQUIRE(row_blocks < ((int64_t)1 << 31) && tok_blocks <= 65535, "indexer_scores_tiled_live: grid too large");
  dim3 grid((unsigned)row_blocks, (unsigned)tok_blocks, (unsigned)batch), block(256);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MSPR_F16)
    scores_tiled_kernel<MSPR_F16><<<grid, block, 0, st>>>(q, weights, index_comp, n_heads, n_tokens, n_comp,
                                                          (uint32_t)pos0, (uint32_t)ratio, scores);
  else
    scores_tiled_kernel<MSPR_F32><<<grid, block, 0, st>>>(q, weights, index_comp, n_heads, n_tokens, n_comp,
                                                          (uint32_t)pos0, (uint32_t)ratio, scores);
  MSPR_CHECK_LAUNCH("indexer_scores_tiled_live");
  return MSPR_OK;
}
