// DS4 lightning-indexer kernels with float32 pool rows: query QAT, score row, score tail,
// E4M3FN row round trip and the prepared KV row of the fused decode island.
//
// Layout notes (wave64): one 128-wide row lives in one half-wave, four elements per lane, so the
// Hadamard butterflies of strides 4..64 are xor shuffles inside the half. The score row runs on
// the float32 MFMA (32x32x2): heads are the M dimension, pool rows the N dimension, so the
// per-row head sum stays inside a lane (plus one xor-32 shuffle) and pool rows stream from HBM
// straight into the B operand registers, 256 contiguous bytes per lane.
#include "common.h"
#include "profile.h"

// The kernels in this file reproduce float32 operation sequences bit for bit: a multiply followed
// by an add must round twice, so fused multiply-add contraction is off for the whole file.
#pragma clang fp contract(off)

namespace {

// Separately rounded float32 multiply and add. They are defined below the pragma on purpose: the
// HIP header intrinsics of the same purpose are inlined with contraction still allowed.
__device__ __forceinline__ float mul_rn(float a, float b) { return a * b; }
__device__ __forceinline__ float add_rn(float a, float b) { return a + b; }

constexpr float kHadamardScale = 0.08838834764831845f;  // float32(128^-1/2)
constexpr float kAmaxFloor = 7.052966104933725e-38f;      // 6 * 2^-126
constexpr float kFp8AmaxFloor = 1.0e-4f;

// MLX Maximum(x, floor): NaN passes through.
__device__ __forceinline__ float mx_floor_max(float x, float fl) { return isnan(x) ? x : (x > fl ? x : fl); }

// QAT of one 128-wide row held by one half-wave: lane l (0..31 inside the half) holds elements
// [4l, 4l+3]. Follows the reference's float32 operation sequence: radix-2 butterflies in
// increasing stride order, scale, per-32 group amax, power-of-two scale, clip, first-wins
// nearest lattice value.
// LIVE selects the prefill-side variant (indexed_attention_kernel.py:1125-1202 of the reference):
// scale 2^ceil(log2(amax/6)) taken exactly, ties to the even lattice index.
template <bool LIVE = false>
__device__ __forceinline__ f32x4_t qat128(f32x4_t v, int lane32) {
  float a0 = v.x + v.y, a1 = v.x - v.y, a2 = v.z + v.w, a3 = v.z - v.w;
  f32x4_t x = {a0 + a2, a1 + a3, a0 - a2, a1 - a3};
#pragma unroll
  for (int m = 1; m <= 16; m <<= 1) {
    f32x4_t o;
    o.x = __shfl_xor(x.x, m, MSPR_WAVE);
    o.y = __shfl_xor(x.y, m, MSPR_WAVE);
    o.z = __shfl_xor(x.z, m, MSPR_WAVE);
    o.w = __shfl_xor(x.w, m, MSPR_WAVE);
    x = (lane32 & m) ? (o - x) : (x + o);
  }
  x = x * kHadamardScale;
  // fmaxf drops NaN operands; carry NaN explicitly so a NaN element poisons its group
  bool any_nan = isnan(x.x) || isnan(x.y) || isnan(x.z) || isnan(x.w);
  float amax = fmaxf(fmaxf(fabsf(x.x), fabsf(x.y)), fmaxf(fabsf(x.z), fabsf(x.w)));
  if (any_nan) amax = __builtin_nanf("");
#pragma unroll
  for (int m = 1; m <= 4; m <<= 1) {
    float o = __shfl_xor(amax, m, MSPR_WAVE);
    amax = (isnan(amax) || isnan(o)) ? __builtin_nanf("") : fmaxf(amax, o);
  }
  amax = mx_floor_max(amax, kAmaxFloor);
  float scale;
  if constexpr (LIVE) {
    const float r = amax / 6.0f;
    const uint32_t u = __float_as_uint(r);
    if (isnan(r) || isinf(r)) {
      scale = r;
    } else {
      int e;
      const float m = frexpf(r, &e);  // r = m * 2^e, m in [0.5, 1)
      scale = ldexpf(1.0f, m == 0.5f ? e - 1 : e);
    }
    (void)u;
  } else {
    scale = pow2_group_scale(amax, 6.0f);
  }
  const float lattice[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
  f32x4_t out;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    float n = x[j] / scale;
    n = (isnan(n) || n > -6.0f) ? n : -6.0f;
    n = (isnan(n) || n < 6.0f) ? n : 6.0f;
    float absn = fabsf(n);
    float best = fabsf(absn - lattice[0]);
    float dq = lattice[0];
    bool best_odd = false;
#pragma unroll
    for (int k = 1; k < 8; k++) {
      float d = fabsf(absn - lattice[k]);
      if (d < best || (LIVE && d == best && (k & 1) == 0 && best_odd)) {
        best = d;
        dq = lattice[k];
        best_odd = (k & 1) != 0;
      }
    }
    dq = n < 0.0f ? -dq : dq;
    out[j] = dq * scale;
  }
  return out;
}

template <int DT>
__device__ __forceinline__ f32x4_t load_row4(const void* base, int64_t row, int lane32) {
  f32x4_t v;
  if constexpr (DT == MSPR_F32) {
    v = reinterpret_cast<const f32x4_t*>(reinterpret_cast<const float*>(base) + row * 128)[lane32];
  } else {
    const uint16_t* p = reinterpret_cast<const uint16_t*>(base) + row * 128 + 4 * lane32;
    u32x2_t w = *reinterpret_cast<const u32x2_t*>(p);
    uint16_t e0 = w.x & 0xFFFFu, e1 = w.x >> 16, e2 = w.y & 0xFFFFu, e3 = w.y >> 16;
    if constexpr (DT == MSPR_F16) {
      v = f32x4_t{f16_bits_to_f32(e0), f16_bits_to_f32(e1), f16_bits_to_f32(e2), f16_bits_to_f32(e3)};
    } else {
      v = f32x4_t{bf16_bits_to_f32(e0), bf16_bits_to_f32(e1), bf16_bits_to_f32(e2), bf16_bits_to_f32(e3)};
    }
  }
  return v;
}

// ------------------------------------------------------------------ QAT rows
template <int DT, bool LIVE = false>
__global__ __launch_bounds__(256) void qat_rows_kernel(const void* __restrict__ x, int64_t n_rows,
                                                       float* __restrict__ out) {
  int lane32 = threadIdx.x & 31;
  int64_t row = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 5);
  // rows past the end recompute the last row so every lane stays active for the shuffles
  int64_t src = row < n_rows ? row : n_rows - 1;
  f32x4_t v = load_row4<DT>(x, src, lane32);
  f32x4_t y = qat128<LIVE>(v, lane32);
  if (row < n_rows) reinterpret_cast<f32x4_t*>(out + row * 128)[lane32] = y;
}

// ------------------------------------------------------------------ score row, float32 pool rows
// Block = 4 waves. The block QATs the (up to 64) query heads into LDS once, each wave then keeps
// them in registers as the MFMA A operand and walks 32-row tiles of the pool.
template <int DT, bool STAGE_HALF>
__global__ __launch_bounds__(256) void scores_f32_kernel(const void* __restrict__ q, int n_heads,
                                                         const float* __restrict__ pooled, int64_t n_rows,
                                                         const float* __restrict__ weights, float scale,
                                                         float* __restrict__ scores) {
  __shared__ float qbuf[64 * 128];
  __shared__ float wbuf[64];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int lane32 = tid & 31;
  const int wave = tid >> 6;
  const int half = (tid >> 5) & 1;

  // QAT pass: 8 rows per step (two per wave)
  for (int h0 = 0; h0 < 64; h0 += 8) {
    int h = h0 + wave * 2 + half;
    int src = h < n_heads ? h : n_heads - 1;
    f32x4_t v = load_row4<DT>(q, src, lane32);
    f32x4_t y = qat128(v, lane32);
    if (STAGE_HALF) {
#pragma unroll
      for (int j = 0; j < 4; j++) y[j] = f16_bits_to_f32(f32_to_f16_bits(y[j]));
    }
    if (h >= n_heads) y = f32x4_t{0.f, 0.f, 0.f, 0.f};
    reinterpret_cast<f32x4_t*>(qbuf + h * 128)[lane32] = y;
  }
  if (tid < 64) wbuf[tid] = tid < n_heads ? weights[tid] : 0.0f;
  __syncthreads();

  // A operand: lane (m = lane%32 -> head, g = lane/32) supplies q[head][64g + s] at k-step s
  const int m = lane & 31;
  const int g = lane >> 5;
  float qa[2][64];
#pragma unroll
  for (int mt = 0; mt < 2; mt++) {
#pragma unroll
    for (int s = 0; s < 64; s += 4) {
      // rotate the column by the row to spread LDS banks
      f32x4_t t = *reinterpret_cast<const f32x4_t*>(qbuf + (mt * 32 + m) * 128 + 64 * g + s);
      qa[mt][s] = t.x;
      qa[mt][s + 1] = t.y;
      qa[mt][s + 2] = t.z;
      qa[mt][s + 3] = t.w;
    }
  }
  // head weights for this lane's accumulator rows: head = 32mt + 8(i/4) + 4g + i%4
  float wl[2][16];
#pragma unroll
  for (int mt = 0; mt < 2; mt++)
#pragma unroll
    for (int i = 0; i < 16; i++) wl[mt][i] = wbuf[32 * mt + 8 * (i / 4) + 4 * g + (i % 4)];

  const int64_t n_tiles = (n_rows + 31) / 32;
  const int64_t wave_global = (int64_t)blockIdx.x * 4 + wave;
  const int64_t wave_stride = (int64_t)gridDim.x * 4;
  for (int64_t tile = wave_global; tile < n_tiles; tile += wave_stride) {
    int64_t row = tile * 32 + m;
    int64_t src = row < n_rows ? row : n_rows - 1;
    const f32x4_t* kp = reinterpret_cast<const f32x4_t*>(pooled + src * 128 + 64 * g);
    float kb[64];
#pragma unroll
    for (int j = 0; j < 16; j++) {
      f32x4_t t = kp[j];
      kb[4 * j] = t.x;
      kb[4 * j + 1] = t.y;
      kb[4 * j + 2] = t.z;
      kb[4 * j + 3] = t.w;
    }
    f32x16_t acc0 = {0}, acc1 = {0};
#pragma unroll
    for (int s = 0; s < 64; s++) {
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(qa[0][s], kb[s], acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(qa[1][s], kb[s], acc1, 0, 0, 0);
    }
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      sum += mul_rn(mul_rn(fmaxf(acc0[i], 0.0f), scale), wl[0][i]);
    }
#pragma unroll
    for (int i = 0; i < 16; i++) {
      sum += mul_rn(mul_rn(fmaxf(acc1[i], 0.0f), scale), wl[1][i]);
    }
    sum += __shfl_xor(sum, 32, MSPR_WAVE);
    if (g == 0 && row < n_rows) scores[row] = sum;
  }
}

// ------------------------------------------------------------------ score tail
template <int WDT>
__global__ __launch_bounds__(256) void score_tail_kernel(const float* __restrict__ s, int n_heads,
                                                         int64_t capacity, const void* __restrict__ wraw,
                                                         const int32_t* __restrict__ params, float scale,
                                                         float head_norm, float* __restrict__ neg) {
  int lane32 = threadIdx.x & 31;
  int64_t col = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 5);
  int64_t c = col < capacity ? col : capacity - 1;
  int32_t pv = params[1];
  int64_t valid = pv < 0 ? 0 : (pv < capacity ? pv : capacity);
  float partial = 0.0f;
  for (int h = lane32; h < n_heads; h += 32) {
    float w = mul_rn(load_as_f32<WDT>(wraw, h), head_norm);
    float t = s[(int64_t)h * capacity + c];
    t = isnan(t) ? t : (t > 0.0f ? t : 0.0f);
    t = mul_rn(t, scale);
    t = mul_rn(t, w);
    partial = add_rn(partial, t);
  }
#pragma unroll
  for (int off = 16; off >= 1; off >>= 1) partial = add_rn(partial, __shfl_xor(partial, off, MSPR_WAVE));
  if (lane32 == 0 && col < capacity) neg[col] = col < valid ? -partial : __builtin_inff();
}

// ------------------------------------------------------------------ E4M3FN round trip
// Nearest non-negative E4M3FN value of a in [0, 448]; exact ties go to the lower value. Equal to
// a first-wins scan of the ascending 127-entry table: both neighbours' distances are exact in
// float32, so only they can win.
__device__ __forceinline__ float e4m3_nearest_lower_ties(float a) {
  if (isnan(a)) return 0.0f;  // a scan that compares against NaN keeps entry 0
  float lo, step;
  if (a < 0.015625f) {
    step = 0.001953125f;
    lo = floorf(a * 512.0f) * 0.001953125f;
  } else {
    uint32_t u = __float_as_uint(a);
    lo = __uint_as_float(u & 0xFFF00000u);
    step = __uint_as_float((u & 0x7F800000u) - (3u << 23));
  }
  if (lo >= 448.0f) return 448.0f;
  float hi = lo + step;
  return (hi - a) < (a - lo) ? hi : lo;
}

__device__ __forceinline__ float fp8_roundtrip(float x, float scale) {
  float n = x / scale;
  n = (isnan(n) || n > -448.0f) ? n : -448.0f;
  n = (isnan(n) || n < 448.0f) ? n : 448.0f;
  float qv = e4m3_nearest_lower_ties(fabsf(n));
  float sign = n < 0.0f ? -1.0f : (n > 0.0f ? 1.0f : 0.0f);
  return mul_rn(mul_rn(sign, qv), scale);
}

// amax over a 64-element block = 4 lanes x 16 values.
__device__ __forceinline__ float block64_amax(const float (&xv)[16]) {
  float amax = 0.0f;
#pragma unroll
  for (int j = 0; j < 16; j++) amax = fmaxf(amax, fabsf(xv[j]));
  amax = fmaxf(amax, __shfl_xor(amax, 1, MSPR_WAVE));
  amax = fmaxf(amax, __shfl_xor(amax, 2, MSPR_WAVE));
  return amax;
}

__global__ __launch_bounds__(256) void fp8_rows_kernel(const float* __restrict__ x, int64_t n_rows,
                                                       float* __restrict__ out) {
  int lane32 = threadIdx.x & 31;
  int64_t row = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 5);
  int64_t src = row < n_rows ? row : n_rows - 1;
  const f32x4_t* xp = reinterpret_cast<const f32x4_t*>(x + src * 512 + 16 * lane32);
  float xv[16];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    f32x4_t t = xp[j];
    xv[4 * j] = t.x;
    xv[4 * j + 1] = t.y;
    xv[4 * j + 2] = t.z;
    xv[4 * j + 3] = t.w;
  }
  float amax = block64_amax(xv);
  float ov[16];
  if (lane32 < 28) {
    float scale = pow2_group_scale(mx_floor_max(amax, kFp8AmaxFloor), 448.0f);
#pragma unroll
    for (int j = 0; j < 16; j++) ov[j] = fp8_roundtrip(xv[j], scale);
  } else {
#pragma unroll
    for (int j = 0; j < 16; j++) ov[j] = xv[j];
  }
  if (row < n_rows) {
    f32x4_t* op = reinterpret_cast<f32x4_t*>(out + row * 512 + 16 * lane32);
#pragma unroll
    for (int j = 0; j < 4; j++) op[j] = f32x4_t{ov[4 * j], ov[4 * j + 1], ov[4 * j + 2], ov[4 * j + 3]};
  }
}

// ------------------------------------------------------------------ prepared KV row
__device__ __forceinline__ float h_round(float v) { return f16_bits_to_f32(f32_to_f16_bits(v)); }

// One (even, odd) pair rotated with every product and sum rounded to float16.
__device__ __forceinline__ void rope_pair_f16(float x0, float x1, float c, float s, float* o0, float* o1) {
  float m0 = h_round(x0 * c), m1 = h_round(x1 * s), m2 = h_round(x0 * s), m3 = h_round(x1 * c);
  *o0 = h_round(m0 - m1);
  *o1 = h_round(m2 + m3);
}

// One half-wave: lane l holds dims [16l, 16l+16). Dims < 448 take the E4M3FN round trip of the
// float16 values widened to float32; dims >= 448 take the partial rope at float16 op rounding.
__global__ __launch_bounds__(64) void kv_row_kernel(const uint16_t* __restrict__ kv, const float* __restrict__ inv_freq,
                                                    const int32_t* __restrict__ params, uint16_t* __restrict__ row_out) {
  int lane32 = threadIdx.x & 31;
  if (threadIdx.x >= 32) return;  // the shuffles below stay inside lanes 0..31 (xor 1, 2)
  float xv[16];
#pragma unroll
  for (int j = 0; j < 16; j++) xv[j] = f16_bits_to_f32(kv[16 * lane32 + j]);
  float amax = block64_amax(xv);
  if (lane32 < 28) {
    float scale = pow2_group_scale(mx_floor_max(amax, kFp8AmaxFloor), 448.0f);
#pragma unroll
    for (int j = 0; j < 16; j++) row_out[16 * lane32 + j] = f32_to_f16_bits(fp8_roundtrip(xv[j], scale));
  } else {
    int pos = params[0];
#pragma unroll
    for (int j = 0; j < 8; j++) {
      int d0 = 16 * lane32 + 2 * j;
      int p = (d0 - 448) / 2;
      float theta = (float)pos * inv_freq[p];
      float c = h_round((float)cos((double)theta));
      float s = h_round((float)sin((double)theta));
      float r0, r1;
      rope_pair_f16(xv[2 * j], xv[2 * j + 1], c, s, &r0, &r1);
      row_out[d0] = f32_to_f16_bits(r0);
      row_out[d0 + 1] = f32_to_f16_bits(r1);
    }
  }
}

}  // namespace

// ====================================================================== C-ABI

extern "C" int mspr_indexer_qat_rows(const void* x, int x_dtype, int64_t n_rows, float* out, void* stream) {
  MSPR_REQUIRE(x && out, "indexer_qat_rows: null pointer");
  MSPR_REQUIRE(n_rows > 0, "indexer_qat_rows: expects at least one row");
  MSPR_REQUIRE(x_dtype >= MSPR_F32 && x_dtype <= MSPR_BF16, "indexer_qat_rows: dtype must be f32, f16 or bf16");
  MSPR_REQUIRE(mspr_aligned(x, 16) && mspr_aligned(out, 16), "indexer_qat_rows: pointers must be 16-byte aligned");
  dim3 grid((unsigned)((n_rows + 7) / 8)), block(256);
  hipStream_t st = (hipStream_t)stream;
  if (x_dtype == MSPR_F32) qat_rows_kernel<MSPR_F32><<<grid, block, 0, st>>>(x, n_rows, out);
  else if (x_dtype == MSPR_F16) qat_rows_kernel<MSPR_F16><<<grid, block, 0, st>>>(x, n_rows, out);
  else qat_rows_kernel<MSPR_BF16><<<grid, block, 0, st>>>(x, n_rows, out);
  MSPR_CHECK_LAUNCH("indexer_qat_rows");
  return MSPR_OK;
}

extern "C" int mspr_indexer_q_qat_live(const float* q, int64_t n_rows, float* out, void* stream) {
  MSPR_REQUIRE(q && out, "indexer_q_qat_live: null pointer");
  MSPR_REQUIRE(n_rows > 0, "indexer_q_qat_live: expects at least one row");
  MSPR_REQUIRE(mspr_aligned(q, 16) && mspr_aligned(out, 16), "indexer_q_qat_live: pointers must be 16-byte aligned");
  dim3 grid((unsigned)((n_rows + 7) / 8)), block(256);
  qat_rows_kernel<MSPR_F32, true><<<grid, block, 0, (hipStream_t)stream>>>(q, n_rows, out);
  MSPR_CHECK_LAUNCH("indexer_q_qat_live");
  return MSPR_OK;
}

int mspr_launch_scores_f32(const void* q, int q_dtype, int n_heads, const float* pooled, int64_t n_rows,
                           const float* weights, float scale, float* scores, bool stage_half, hipStream_t st) {
  int64_t n_tiles = (n_rows + 31) / 32;
  int64_t blocks = (n_tiles + 3) / 4;
  if (blocks > 2048) blocks = 2048;
  dim3 grid((unsigned)blocks), block(256);
  MsprProfScope prof(MSPR_K_SCORES_F32, st);
#define MSPR_SCORES_LAUNCH(DT)                                                                          \
  do {                                                                                                  \
    if (stage_half)                                                                                     \
      scores_f32_kernel<DT, true><<<grid, block, 0, st>>>(q, n_heads, pooled, n_rows, weights, scale, scores);  \
    else                                                                                                \
      scores_f32_kernel<DT, false><<<grid, block, 0, st>>>(q, n_heads, pooled, n_rows, weights, scale, scores); \
  } while (0)
  if (q_dtype == MSPR_F32) MSPR_SCORES_LAUNCH(MSPR_F32);
  else if (q_dtype == MSPR_F16) MSPR_SCORES_LAUNCH(MSPR_F16);
  else MSPR_SCORES_LAUNCH(MSPR_BF16);
#undef MSPR_SCORES_LAUNCH
  MSPR_CHECK_LAUNCH("indexer scores (f32 pool)");
  return MSPR_OK;
}

extern "C" int mspr_fused_qat_indexer_scores(const void* q, int q_dtype, int n_heads, const float* pooled_qat,
                                             int64_t n_rows, const float* weights, float scale, float* scores,
                                             void* stream) {
  MSPR_REQUIRE(q && pooled_qat && weights && scores, "fused_qat_indexer_scores: null pointer");
  MSPR_REQUIRE(n_heads >= 1 && n_heads <= 64, "fused_qat_indexer_scores: q must carry between 1 and 64 heads");
  MSPR_REQUIRE(n_rows > 0, "fused_qat_indexer_scores: pooled_qat must contain at least one row");
  MSPR_REQUIRE(q_dtype >= MSPR_F32 && q_dtype <= MSPR_BF16, "fused_qat_indexer_scores: q must be f32, f16 or bf16");
  MSPR_REQUIRE(mspr_aligned(q, 16) && mspr_aligned(pooled_qat, 16), "fused_qat_indexer_scores: q and pooled_qat must be 16-byte aligned");
  return mspr_launch_scores_f32(q, q_dtype, n_heads, pooled_qat, n_rows, weights, scale, scores, false,
                                (hipStream_t)stream);
}

extern "C" int mspr_indexer_score_tail(const float* scores, int n_heads, int64_t capacity, const void* weights_raw,
                                       int w_dtype, const int32_t* params, float scale, float* neg, void* stream) {
  MSPR_REQUIRE(scores && weights_raw && params && neg, "indexer_score_tail: null pointer");
  MSPR_REQUIRE(n_heads >= 32 && n_heads <= 64, "indexer_score_tail: covers 32 to 64 index heads");
  MSPR_REQUIRE(capacity > 0, "indexer_score_tail: scores must cover at least one capacity column");
  MSPR_REQUIRE(w_dtype >= MSPR_F32 && w_dtype <= MSPR_BF16, "indexer_score_tail: weights_raw must be f32, f16 or bf16");
  float head_norm = (float)(1.0 / sqrt((double)n_heads));
  dim3 grid((unsigned)((capacity + 7) / 8)), block(256);
  hipStream_t st = (hipStream_t)stream;
  if (w_dtype == MSPR_F32) score_tail_kernel<MSPR_F32><<<grid, block, 0, st>>>(scores, n_heads, capacity, weights_raw, params, scale, head_norm, neg);
  else if (w_dtype == MSPR_F16) score_tail_kernel<MSPR_F16><<<grid, block, 0, st>>>(scores, n_heads, capacity, weights_raw, params, scale, head_norm, neg);
  else score_tail_kernel<MSPR_BF16><<<grid, block, 0, st>>>(scores, n_heads, capacity, weights_raw, params, scale, head_norm, neg);
  MSPR_CHECK_LAUNCH("indexer_score_tail");
  return MSPR_OK;
}

extern "C" int mspr_fp8_kv_prefix_rows(const float* x, int64_t n_rows, float* out, void* stream) {
  MSPR_REQUIRE(x && out, "fp8_kv_prefix_rows: null pointer");
  MSPR_REQUIRE(n_rows > 0, "fp8_kv_prefix_rows: expects at least one row");
  MSPR_REQUIRE(mspr_aligned(x, 16) && mspr_aligned(out, 16), "fp8_kv_prefix_rows: pointers must be 16-byte aligned");
  dim3 grid((unsigned)((n_rows + 7) / 8)), block(256);
  fp8_rows_kernel<<<grid, block, 0, (hipStream_t)stream>>>(x, n_rows, out);
  MSPR_CHECK_LAUNCH("fp8_kv_prefix_rows");
  return MSPR_OK;
}

int mspr_launch_kv_row(const void* kv_row, const float* inv_freq, const int32_t* params, void* row_out, hipStream_t st) {
  kv_row_kernel<<<1, 64, 0, st>>>(reinterpret_cast<const uint16_t*>(kv_row), inv_freq, params,
                                  reinterpret_cast<uint16_t*>(row_out));
  MSPR_CHECK_LAUNCH("prepared kv row");
  return MSPR_OK;
}
