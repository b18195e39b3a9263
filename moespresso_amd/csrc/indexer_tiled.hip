// Prefill-side lightning-indexer scores over a chunk of tokens:
//   scores[b,t,c] = sum_h max(q[b,h,t] . comp[b,c], 0) * w[b,t,h],  -inf where c >= (pos0+t+1)/ratio
// Operands are staged as float16 (float32 inputs are rounded on load), products accumulate in float32
// on v_mfma_f32_32x32x16_f16 with heads = M and pool rows = N, so the relu / weight / head sum runs on
// the accumulator registers of one lane column per pool row.
//
// Workgroup = 4 waves = 4 consecutive tokens of one batch entry walking the same block of pool rows, which
// it stages tile by tile in LDS; the token's 64 x 128 query block stays in registers.
#include "common.h"
#include "profile.h"

namespace {

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

// A workgroup = 4 waves = 4 consecutive tokens walks `rows_per_block` pool rows (a multiple of 32) in tiles of 32.
// A tile is fetched once per workgroup (every thread 32 bytes of it, rounded to float16) into one of two LDS buffers,
// a tile ahead of its use, and the four waves read their B operands from there: fetched by each wave for itself, the
// 16-byte pieces of 32 rows keep a CU's address path busier than its matrix pipes. Rows past a token's visible
// prefix score -inf whatever the products are, so a wave multiplies only the tiles that hold a row it sees.
constexpr int kTilePitch = 272;  // bytes between rows of a tile in LDS: 256 + 16, operand reads of 32 rows x 2 pieces
                                 // and the 16-byte writes of two rows at a time both without bank conflicts

template <int DT>
__global__ __launch_bounds__(256, 2) void scores_tiled_kernel(const void* __restrict__ q, const float* __restrict__ w,
                                                           const void* __restrict__ comp, int n_heads, int n_tokens,
                                                           int64_t n_comp, uint32_t pos0, uint32_t ratio,
                                                           int rows_per_block, float* __restrict__ scores) {
  __shared__ __attribute__((aligned(16))) unsigned char tile_lds[2][32 * kTilePitch];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n = lane & 31;
  const int g = lane >> 5;
  const int b = blockIdx.z;
  int t = blockIdx.y * 4 + wave;
  const bool t_live = t < n_tokens;
  if (!t_live) t = n_tokens - 1;

  const int64_t row_begin = (int64_t)blockIdx.x * rows_per_block;
  int64_t row_end = row_begin + rows_per_block;
  if (row_end > n_comp) row_end = n_comp;
  // tiles of this block that hold a row visible to token `tok`
  auto visible_of = [&](int tok) -> int64_t {
    const uint32_t qpos1 = pos0 + (uint32_t)tok + 1u;
    const int64_t v = ratio == 0u ? n_comp : (int64_t)(qpos1 / ratio);
    return v < n_comp ? v : n_comp;
  };
  auto live_tiles = [&](int64_t vis) -> int {
    const int64_t live_end = vis < row_end ? vis : row_end;
    return live_end > row_begin ? (int)((live_end - row_begin + 31) / 32) : 0;
  };
  const int64_t visible = visible_of(t);
  const int n_live = live_tiles(visible);
  // the workgroup's last token sees the most rows: it sets the number of tiles the workgroup fetches
  int t_last = blockIdx.y * 4 + 3;
  if (t_last > n_tokens - 1) t_last = n_tokens - 1;
  const int n_fetch = live_tiles(visible_of(t_last));
  float* out_row = scores + ((int64_t)b * n_tokens + t) * n_comp;

  if (n_fetch > 0) {  // (the same in every wave of the workgroup: the barriers below are met by all)
    const void* comp_b =
        DT == MSPR_F16 ? static_cast<const void*>(reinterpret_cast<const uint16_t*>(comp) + (int64_t)b * n_comp * 128)
                       : static_cast<const void*>(reinterpret_cast<const float*>(comp) + (int64_t)b * n_comp * 128);
    // this thread's share of a tile: row tid / 8, columns [16 (tid % 8), +16)
    const int f_row = tid >> 3, f_col = (tid & 7) * 16;
    auto fetch = [&](int64_t r0, u32x4_t (&st)[2]) {
      int64_t row = r0 + f_row;
      if (row >= n_comp) row = n_comp - 1;
      st[0] = load8_as_f16<DT>(comp_b, row * 128 + f_col);
      st[1] = load8_as_f16<DT>(comp_b, row * 128 + f_col + 8);
    };
    auto stash = [&](int buf, const u32x4_t (&st)[2]) {
      unsigned char* p = tile_lds[buf] + f_row * kTilePitch + f_col * 2;
      *reinterpret_cast<u32x4_t*>(p) = st[0];
      *reinterpret_cast<u32x4_t*>(p + 16) = st[1];
    };
    u32x4_t st[2];
    fetch(row_begin, st);  // (in flight while the query block and the weights arrive)

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
    const float* w_row = w + ((int64_t)b * n_tokens + t) * n_heads;
    if (n_heads == 64 && (reinterpret_cast<uintptr_t>(w) & 15u) == 0) {  // (four consecutive heads per load)
#pragma unroll
      for (int hb = 0; hb < 2; hb++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const f32x4_t v = *reinterpret_cast<const f32x4_t*>(w_row + 32 * hb + 8 * j + 4 * g);
          wv[hb][4 * j] = v.x;
          wv[hb][4 * j + 1] = v.y;
          wv[hb][4 * j + 2] = v.z;
          wv[hb][4 * j + 3] = v.w;
        }
    } else {
#pragma unroll
      for (int hb = 0; hb < 2; hb++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int head = 32 * hb + 8 * (i / 4) + 4 * g + (i % 4);
          wv[hb][i] = head < n_heads ? w_row[head] : 0.0f;
        }
    }
    stash(0, st);
    __syncthreads();

    for (int i = 0; i < n_fetch; i++) {
      if (i + 1 < n_fetch) fetch(row_begin + 32 * (int64_t)(i + 1), st);
      if (i < n_live) {
        // B operand: lane (n, g) holds comp[row r0 + n][16 s + 8 g .. +7] for k-step s
        const unsigned char* kt = tile_lds[i & 1] + n * kTilePitch + 16 * g;
        f32x16_t acc0 = {0}, acc1 = {0};
#pragma unroll
        for (int s = 0; s < 8; s++) {
          const u32x4_t kb = *reinterpret_cast<const u32x4_t*>(kt + 32 * s);
          acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, qa[0][s]),
                                                        __builtin_bit_cast(f16x8_t, kb), acc0, 0, 0, 0);
          acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, qa[1][s]),
                                                        __builtin_bit_cast(f16x8_t, kb), acc1, 0, 0, 0);
        }
        float sum = 0.0f;
#pragma unroll
        for (int k = 0; k < 16; k++) {
          sum += fmaxf(acc0[k], 0.0f) * wv[0][k];
          sum += fmaxf(acc1[k], 0.0f) * wv[1][k];
        }
        sum += __shfl_xor(sum, 32, MSPR_WAVE);
        const int64_t c = row_begin + 32 * (int64_t)i + n;
        if (t_live && g == 0 && c < row_end) out_row[c] = c < visible ? sum : -__builtin_inff();
      }
      if (i + 1 < n_fetch) stash((i + 1) & 1, st);
      __syncthreads();  // tile i+1 written by every thread; tile i read by every wave
    }
  }
  // rows of the block behind the last multiplied tile: not visible to this token
  if (t_live) {
    for (int64_t c = row_begin + (int64_t)n_live * 32 + lane; c < row_end; c += 64) out_row[c] = -__builtin_inff();
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
  // Four tokens per workgroup; the pool rows are split over several workgroups only as far as it takes to have
  // about three workgroups for each of the 256 CUs (every workgroup fetches its tokens' query blocks anew).
  const int64_t tok_blocks = (n_tokens + 3) / 4;
  int64_t row_blocks = (768 + tok_blocks * batch - 1) / (tok_blocks * batch);
  const int64_t row_tiles = (n_comp + 31) / 32;
  if (row_blocks > row_tiles) row_blocks = row_tiles;
  if (row_blocks < 1) row_blocks = 1;
  const int64_t rows_per_block = (row_tiles + row_blocks - 1) / row_blocks * 32;
  row_blocks = (n_comp + rows_per_block - 1) / rows_per_block;
  MSPR_REQUIRE(row_blocks < ((int64_t)1 << 31) && tok_blocks <= 65535 && rows_per_block < ((int64_t)1 << 31),
               "indexer_scores_tiled_live: grid too large");
  dim3 grid((unsigned)row_blocks, (unsigned)tok_blocks, (unsigned)batch), block(256);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MSPR_F16)
    scores_tiled_kernel<MSPR_F16><<<grid, block, 0, st>>>(q, weights, index_comp, n_heads, n_tokens, n_comp,
                                                          (uint32_t)pos0, (uint32_t)ratio, (int)rows_per_block, scores);
  else
    scores_tiled_kernel<MSPR_F32><<<grid, block, 0, st>>>(q, weights, index_comp, n_heads, n_tokens, n_comp,
                                                          (uint32_t)pos0, (uint32_t)ratio, (int)rows_per_block, scores);
  MSPR_CHECK_LAUNCH("indexer_scores_tiled_live");
  return MSPR_OK;
}
