// Batched lightning-indexer score row with FP8 (E4M3FN) keys and one float32 scale per key:
//   score[b, r] = sum_h w[b, h] * relu(q[b, h] . e4m3(keys[b, r])) * key_scale[b, r]
//
// The 64-head x 128-wide contraction against each key runs on the bf16 MFMA (32x32x16): heads
// are the M dimension, keys the N dimension, so the relu-weighted head sum of one key stays in one
// lane's accumulator registers (plus one xor-32 shuffle). E4M3 values are exact in bf16, and a
// bf16 x bf16 product is exact in the float32 accumulator, so the only rounding is the
// accumulation itself. Keys stream from HBM straight into the B-operand registers: a lane owns
// 64 contiguous bytes of its key row, a wave 4 KB of contiguous memory per 32-key tile, and the
// next two tiles are in flight while the current one is multiplied.
#include "common.h"
#include "profile.h"

namespace {

// Two E4M3FN bytes (the low or high half of `w`) to two bf16 values packed in one register: one
// conversion instruction (the scale operand is 1; every E4M3 value is exact in bf16).
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t fp8x2_to_bf16x2(uint32_t w, bool hi) {
  bf16x2_t r = hi ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true)
                  : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false);
  return __builtin_bit_cast(uint32_t, r);
}

// max(x, 0) on the bit pattern: a float with the sign bit set is a negative integer. One instruction,
// where the float maximum first spends another one on quieting its operand.
__device__ __forceinline__ float relu_bits(float x) {
  const int v = __float_as_int(x);
  return __int_as_float(v > 0 ? v : 0);
}

// PAIRS: a wave takes its keys in units of two consecutive 32-key tiles, so that the key scales come in
// and the scores go out 64 rows (256 bytes) at a time, one row per lane; a per-tile 128-byte load and
// store each cost a DRAM page of their own for 3 % of the bytes and measurably more of the time. The
// single-tile form spreads short rows and small batches over more waves.
template <bool PAIRS>
__global__ __launch_bounds__(256, 2) void indexer_scores_fp8_kernel(const uint16_t* __restrict__ q,
                                                                    const uint8_t* __restrict__ keys,
                                                                    const float* __restrict__ key_scales,
                                                                    const float* __restrict__ weights, int n_heads,
                                                                    int64_t n_rows, int blocks_per_batch,
                                                                    float* __restrict__ scores) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int m = lane & 31;
  const int g = lane >> 5;
  const int b = blockIdx.x / blocks_per_batch;
  const int blk = blockIdx.x % blocks_per_batch;

  const uint16_t* qb = q + (int64_t)b * n_heads * 128;
  const uint8_t* kb = keys + (int64_t)b * n_rows * 128;
  const float* ksb = key_scales + (int64_t)b * n_rows;
  const float* wb = weights + (int64_t)b * n_heads;
  float* sb = scores + (int64_t)b * n_rows;

  // work items: tiles, or units of two tiles
  const int64_t n_tiles = PAIRS ? (n_rows + 63) / 64 : (n_rows + 31) / 32;
  const int64_t stride = (int64_t)blocks_per_batch * 4;
  int64_t tile = (int64_t)blk * 4 + wave;
  const bool has_work = tile < n_tiles;  // a wave without work still brings its share of the query block

  // a tile image: the lane's 64 key bytes and the key's scale (loaded with the tile so that the wait
  // for it in the epilogue does not have to drain the tiles fetched behind it)
  auto load_tile = [&](int64_t t, u32x4_t (&raw)[4], float& ks) {
    int64_t row = t * 32 + m;
    if (row >= n_rows) row = n_rows - 1;
    ks = ksb[row];
    const u32x4_t* p = reinterpret_cast<const u32x4_t*>(kb + row * 128 + 64 * g);
#pragma unroll
    for (int j = 0; j < 4; j++) raw[j] = p[j];
  };
  // half h of unit u: rows [64 u + 32 h, +32); the unit's 64 scales, one per lane, travel with half 0
  auto load_half = [&](int64_t u, int h, u32x4_t (&raw)[4]) {
    int64_t row = u * 64 + 32 * h + m;
    if (row >= n_rows) row = n_rows - 1;
    const u32x4_t* p = reinterpret_cast<const u32x4_t*>(kb + row * 128 + 64 * g);
#pragma unroll
    for (int j = 0; j < 4; j++) raw[j] = p[j];
  };
  auto load_unit_scales = [&](int64_t u) -> float {
    int64_t row = u * 64 + lane;
    if (row >= n_rows) row = n_rows - 1;
    return ksb[row];
  };

  // Prologue. The query block and the head weights are the same for every wave of the workgroup: each
  // thread requests its share once (64 bytes of q, lanes of wave 0 one weight each), the first two
  // tiles go out right behind, and while those fly the shares meet in LDS and every wave reads its
  // A-operand registers back from there. (Every wave fetching all of q and its 32 weights itself kept
  // the address units of a CU busy for about 3 us before the first tile could be multiplied.)
  // [head tile][k-step] register images, lane (m, g) at 33 g + m of an image of 66 entries: an image starts 32 bytes
  // further on in the banks than the one before and its second half 16 bytes further than its first, so that the
  // sixteen pieces of one head (eight k-steps x two halves, what sixteen consecutive threads write) fall on
  // sixteen different 16-byte bank groups; the reads are lane-contiguous either way
  constexpr int kImg = 66;
  __shared__ __attribute__((aligned(16))) u32x4_t q_lds[2 * 8 * kImg];
  __shared__ float w_lds[64];
  u32x4_t qpiece[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int pc = tid + 256 * i;  // piece (head h, 8-column group c)
    const int h = pc >> 4, c = pc & 15;
    qpiece[i] = *reinterpret_cast<const u32x4_t*>(qb + (int64_t)(h < n_heads ? h : 0) * 128 + c * 8);
  }
  float wmine = wb[lane < n_heads ? lane : 0];
  u32x4_t ra[4], rb[4], rc[4], rd[4];
  float sa, sb_, sc;
  const int64_t last = n_tiles - 1;
  if constexpr (PAIRS) {
    const int64_t u0 = has_work ? tile : last;
    sa = load_unit_scales(u0);
    load_half(u0, 0, ra);
    load_half(u0, 1, rb);
  } else {
    load_tile(has_work ? tile : last, ra, sa);
    load_tile(tile + stride < n_tiles ? tile + stride : last, rb, sb_);
  }
  // (pinned here: the waits for the shares then leave the tile loads in flight, and the compiler cannot
  // sink the share loads into the conditional stores below, behind the tile loads)
#pragma unroll
  for (int i = 0; i < 4; i++) asm volatile("" : "+v"(qpiece[i]));
  asm volatile("" : "+v"(wmine));
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int pc = tid + 256 * i;
    const int h = pc >> 4, c = pc & 15;
    // slot of lane (m = h % 32, g = c / 8) in the image of (head tile h / 32, k-step c % 8)
    q_lds[((h >> 5) * 8 + (c & 7)) * kImg + 33 * (c >> 3) + (h & 31)] = h < n_heads ? qpiece[i] : u32x4_t{0u, 0u, 0u, 0u};
  }
  if (wave == 0) w_lds[lane] = lane < n_heads ? wmine : 0.0f;
  __syncthreads();
  if (!has_work) return;
  // A operand: lane (m -> head, g) holds q[head][64g + 8s .. +7] for k-step s; heads past the end are zero
  u32x4_t qa[2][8];
#pragma unroll
  for (int mt = 0; mt < 2; mt++)
#pragma unroll
    for (int s = 0; s < 8; s++) qa[mt][s] = q_lds[(mt * 8 + s) * kImg + 33 * g + m];
  // weights of this lane's accumulator rows: head = 32mt + 8(i/4) + 4g + i%4
  float wl[2][16];
#pragma unroll
  for (int mt = 0; mt < 2; mt++)
#pragma unroll
    for (int i = 0; i < 16; i++) wl[mt][i] = w_lds[32 * mt + 8 * (i / 4) + 4 * g + (i % 4)];

  // relu-weighted head sum of the 32 keys of one tile image: lane (m, either g) gets the sum of key m
  auto tile_sums = [&](const u32x4_t (&cur)[4]) -> float {
    f32x16_t acc0 = {0}, acc1 = {0};
#pragma unroll
    for (int s = 0; s < 8; s++) {
      // bytes 8s..8s+7 of this lane's 64: two dwords of cur[s/2]
      const uint32_t w0 = cur[s >> 1][(s & 1) * 2], w1 = cur[s >> 1][(s & 1) * 2 + 1];
      u32x4_t kf = {fp8x2_to_bf16x2(w0, false), fp8x2_to_bf16x2(w0, true), fp8x2_to_bf16x2(w1, false),
                    fp8x2_to_bf16x2(w1, true)};
      bf16x8_t kfb = __builtin_bit_cast(bf16x8_t, kf);
      acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, qa[0][s]), kfb, acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, qa[1][s]), kfb, acc1, 0, 0, 0);
    }
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) sum = fmaf(relu_bits(acc0[i]), wl[0][i], sum);
#pragma unroll
    for (int i = 0; i < 16; i++) sum = fmaf(relu_bits(acc1[i]), wl[1][i], sum);
    sum += __shfl_xor(sum, 32, MSPR_WAVE);
    return sum;
  };
  auto compute_tile = [&](int64_t t, const u32x4_t (&cur)[4], float ks) {
    const int64_t row = t * 32 + m;
    const float sum = tile_sums(cur);
    if (g == 0 && row < n_rows) sb[row] = sum * ks;
  };
  // both halves of a unit, then one 64-lane store: lane (m, g) holds row 64 u + 32 g + m
  auto compute_unit = [&](int64_t u, const u32x4_t (&h0)[4], const u32x4_t (&h1)[4], float ks_lane) {
    const float s0 = tile_sums(h0);
    const float s1 = tile_sums(h1);
    const int64_t row = u * 64 + lane;
    if (row < n_rows) sb[row] = (g ? s1 : s0) * ks_lane;
  };

  if constexpr (PAIRS) {
    // Two units' images alternate: while a unit is multiplied the next one (8 KB) is in flight. Loads past
    // the wave's last unit are clamped re-reads and are never consumed.
    while (true) {
      int64_t nu = tile + stride < n_tiles ? tile + stride : last;
      sb_ = load_unit_scales(nu);
      load_half(nu, 0, rc);
      load_half(nu, 1, rd);
      compute_unit(tile, ra, rb, sa);
      tile += stride;
      if (tile >= n_tiles) break;
      nu = tile + stride < n_tiles ? tile + stride : last;
      sa = load_unit_scales(nu);
      load_half(nu, 0, ra);
      load_half(nu, 1, rb);
      compute_unit(tile, rc, rd, sb_);
      tile += stride;
      if (tile >= n_tiles) break;
    }
    return;
  }
  // Three tile images rotate through registers: while one is multiplied the next two are in flight
  // (8 KB per wave). Loads past the wave's last tile are clamped re-reads and are never consumed.
  while (true) {
    load_tile(tile + 2 * stride < n_tiles ? tile + 2 * stride : last, rc, sc);
    compute_tile(tile, ra, sa);
    tile += stride;
    if (tile >= n_tiles) break;
    load_tile(tile + 2 * stride < n_tiles ? tile + 2 * stride : last, ra, sa);
    compute_tile(tile, rb, sb_);
    tile += stride;
    if (tile >= n_tiles) break;
    load_tile(tile + 2 * stride < n_tiles ? tile + 2 * stride : last, rb, sb_);
    compute_tile(tile, rc, sc);
    tile += stride;
    if (tile >= n_tiles) break;
  }
}

}  // namespace

int mspr_launch_indexer_scores_fp8(const void* q, const void* keys, const float* key_scales, const float* weights,
                                   int batch, int n_heads, int64_t n_rows, float* scores, hipStream_t st) {
  // units of two tiles once every wave of a full grid (2 workgroups per CU) still gets at least two of them
  const bool pairs = (int64_t)batch * ((n_rows + 63) / 64) >= 2 * 2048;
  const int64_t n_tiles = pairs ? (n_rows + 63) / 64 : (n_rows + 31) / 32;
  // 2 workgroups per CU in total and not one more, every wave with at least one work item
  int64_t per_batch = 512 / batch;  // (256 and 768 in total both measured 3 us slower at batch 16)
  int64_t max_blocks = (n_tiles + 3) / 4;
  if (per_batch > max_blocks) per_batch = max_blocks;
  if (per_batch < 1) per_batch = 1;
  dim3 grid((unsigned)(per_batch * batch)), block(256);
  {
    MsprProfScope prof(MSPR_K_INDEXER_FP8, st);
    if (pairs)
      indexer_scores_fp8_kernel<true><<<grid, block, 0, st>>>(reinterpret_cast<const uint16_t*>(q),
                                                               reinterpret_cast<const uint8_t*>(keys), key_scales, weights,
                                                               n_heads, n_rows, (int)per_batch, scores);
    else
      indexer_scores_fp8_kernel<false><<<grid, block, 0, st>>>(reinterpret_cast<const uint16_t*>(q),
                                                                reinterpret_cast<const uint8_t*>(keys), key_scales, weights,
                                                                n_heads, n_rows, (int)per_batch, scores);
  }
  MSPR_CHECK_LAUNCH("indexer_scores_fp8");
  return MSPR_OK;
}

extern "C" int mspr_indexer_scores_fp8(const void* q, const void* keys, const float* key_scales,
                                       const float* weights, int batch, int n_heads, int64_t n_rows, float* scores,
                                       void* stream) {
  MSPR_REQUIRE(q && keys && key_scales && weights && scores, "indexer_scores_fp8: null pointer");
  MSPR_REQUIRE(batch >= 1, "indexer_scores_fp8: batch must be positive");
  MSPR_REQUIRE(n_heads >= 1 && n_heads <= 64, "indexer_scores_fp8: between 1 and 64 heads");
  MSPR_REQUIRE(n_rows >= 1 && n_rows < ((int64_t)1 << 31), "indexer_scores_fp8: n_rows out of range");
  MSPR_REQUIRE(mspr_aligned(q, 16) && mspr_aligned(keys, 16), "indexer_scores_fp8: q and keys must be 16-byte aligned");
  return mspr_launch_indexer_scores_fp8(q, keys, key_scales, weights, batch, n_heads, n_rows, scores,
                                        (hipStream_t)stream);
}
