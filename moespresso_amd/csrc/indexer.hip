// DS4 lightning-indexer kernels with float32 pool rows: query QAT, score row, score tail,
// E4M3FN row round trip and the prepared KV row of the fused decode island.
//
// Layout notes (wave64): one 128-wide row lives in one half-wave, four elements per lane, so the
// Hadamard butterflies of strides 4..64 are lane exchanges inside the half (data-parallel-primitive
// moves up to stride 32, one swizzle for stride 64). The score row runs on the bf16 MFMA (32x32x16)
// with exact products: heads are the M dimension, pool rows the N dimension, so the per-row head sum
// stays inside a lane (plus one xor-32 shuffle) and pool rows stream from HBM straight into the B
// operand registers, 256 contiguous bytes per lane.
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
constexpr int kPow2TabLen = 321;  // entries of g_pow2_tab

// MLX Maximum(x, floor): NaN passes through.
__device__ __forceinline__ float mx_floor_max(float x, float fl) { return isnan(x) ? x : (x > fl ? x : fl); }

// QAT of one 128-wide row held by one half-wave: lane l (0..31 inside the half) holds elements
// [4l, 4l+3]. Follows the reference's float32 operation sequence: radix-2 butterflies in
// increasing stride order, scale, per-32 group amax, power-of-two scale, clip, first-wins
// nearest lattice value.
// LIVE selects the prefill-side variant (indexed_attention_kernel.py:1125-1202 of the reference):
// scale 2^ceil(log2(amax/6)) taken exactly, ties to the even lattice index.
// First half: the butterflies, the 128^-1/2 scale and the floored amax of this lane's group of 32.
struct QatRotated {
  f32x4_t x;
  float amax;
};

// One cross-lane butterfly stage: lanes with bit M clear take x + o, the others o - x, where o is the
// partner lane's value. Written as fma(x, +-1, o): the product is exact, so the single rounding is that
// of the sum or difference itself.
template <int M>
__device__ __forceinline__ f32x4_t butterfly_stage(f32x4_t x, int lane32) {
  const float sgn = (lane32 & M) ? -1.0f : 1.0f;
  return f32x4_t{__builtin_fmaf(x.x, sgn, lane_xor<M>(x.x)), __builtin_fmaf(x.y, sgn, lane_xor<M>(x.y)),
                 __builtin_fmaf(x.z, sgn, lane_xor<M>(x.z)), __builtin_fmaf(x.w, sgn, lane_xor<M>(x.w))};
}

template <int M>
__device__ __forceinline__ float amax_stage(float amax) {
  const float o = lane_xor<M>(amax);
  return (isnan(amax) || isnan(o)) ? __builtin_nanf("") : fmaxf(amax, o);
}

__device__ __forceinline__ QatRotated qat_rotate(f32x4_t v, int lane32) {
  float a0 = v.x + v.y, a1 = v.x - v.y, a2 = v.z + v.w, a3 = v.z - v.w;
  f32x4_t x = {a0 + a2, a1 + a3, a0 - a2, a1 - a3};
  x = butterfly_stage<1>(x, lane32);
  x = butterfly_stage<2>(x, lane32);
  x = butterfly_stage<4>(x, lane32);
  x = butterfly_stage<8>(x, lane32);
  x = butterfly_stage<16>(x, lane32);
  x = x * kHadamardScale;
  // fmaxf drops NaN operands; carry NaN explicitly so a NaN element poisons its group
  bool any_nan = isnan(x.x) || isnan(x.y) || isnan(x.z) || isnan(x.w);
  float amax = fmaxf(fmaxf(fabsf(x.x), fabsf(x.y)), fmaxf(fabsf(x.z), fabsf(x.w)));
  if (any_nan) amax = __builtin_nanf("");
  amax = amax_stage<1>(amax);
  amax = amax_stage<2>(amax);
  amax = amax_stage<4>(amax);
  return QatRotated{x, mx_floor_max(amax, kAmaxFloor)};
}

template <bool LIVE = false>
__device__ __forceinline__ float qat_scale(float amax, const float* tab = g_pow2_tab) {
  if constexpr (LIVE) {
    const float r = amax / 6.0f;
    if (isnan(r) || isinf(r)) return r;
    int e;
    const float m = frexpf(r, &e);  // r = m * 2^e, m in [0.5, 1)
    return ldexpf(1.0f, m == 0.5f ? e - 1 : e);
  } else {
    return pow2_group_scale(amax, 6.0f, tab);
  }
}

// Second half: clip to [-6, 6] in units of the scale and take the nearest lattice value
// {0, .5, 1, 1.5, 2, 3, 4, 6}. The reference takes the first minimum of |n - lattice[k]|; around a
// midpoint of two neighbours both differences are exact float32 values (each operand is within a factor
// of two of the other, or the lattice value is 0), so comparing |n| with the midpoints picks the same
// value, ties going to the lower neighbour. The LIVE variant breaks ties towards the even lattice index,
// which turns three of the seven comparisons into >=. NaN compares false everywhere and lands on 0.
template <bool LIVE = false>
__device__ __forceinline__ f32x4_t qat_snap(f32x4_t x, float scale) {
  f32x4_t out;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    float n = x[j] / scale;
    n = (isnan(n) || n > -6.0f) ? n : -6.0f;
    n = (isnan(n) || n < 6.0f) ? n : 6.0f;
    const float a = fabsf(n);
    float dq = 0.0f;
    dq = a > 0.25f ? 0.5f : dq;
    dq = (LIVE ? a >= 0.75f : a > 0.75f) ? 1.0f : dq;
    dq = a > 1.25f ? 1.5f : dq;
    dq = (LIVE ? a >= 1.75f : a > 1.75f) ? 2.0f : dq;
    dq = a > 2.5f ? 3.0f : dq;
    dq = (LIVE ? a >= 3.5f : a > 3.5f) ? 4.0f : dq;
    dq = a > 5.0f ? 6.0f : dq;
    dq = n < 0.0f ? -dq : dq;
    out[j] = dq * scale;
  }
  return out;
}

template <bool LIVE = false>
__device__ __forceinline__ f32x4_t qat128(f32x4_t v, int lane32) {
  const QatRotated r = qat_rotate(v, lane32);
  return qat_snap<LIVE>(r.x, qat_scale<LIVE>(r.amax));
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

// Prepared KV row of the decode island, one job for the first wave of a workgroup (every thread of the
// workgroup calls this and reaches its one barrier). Lane l of the lower half-wave holds dims
// [16l, 16l+16): dims < 448 take the E4M3FN round trip of the float16 values widened to float32, dims
// >= 448 the partial rope at float16 op rounding. The upper half-wave works out the 32 cosine / sine
// pairs, one frequency per lane, while the lower one loads the row; the four rope lanes then pick their
// eight pairs up from LDS (cs, sn: 32 floats each).
__device__ __forceinline__ void kv_row_job(int tid, float* cs, float* sn, const uint16_t* __restrict__ kv,
                                           const float* __restrict__ inv_freq, const int32_t* __restrict__ params,
                                           uint16_t* __restrict__ row_out) {
  const int lane32 = tid & 31;
  if (tid >= 32 && tid < 64) {
    const float theta = (float)params[0] * inv_freq[lane32];
    cs[lane32] = h_round((float)cos((double)theta));
    sn[lane32] = h_round((float)sin((double)theta));
  }
  float xv[16];
  if (tid < 32) {
    const u32x4_t* src = reinterpret_cast<const u32x4_t*>(kv + 16 * lane32);
    const u32x4_t w0 = src[0], w1 = src[1];
    const uint32_t w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
    for (int j = 0; j < 8; j++) {
      xv[2 * j] = f16_bits_to_f32((uint16_t)(w[j] & 0xFFFFu));
      xv[2 * j + 1] = f16_bits_to_f32((uint16_t)(w[j] >> 16));
    }
  }
  __syncthreads();
  if (tid >= 32) return;  // the shuffles below stay inside lanes 0..31 (xor 1, 2)
  float amax = block64_amax(xv);
  float ov[16];
  if (lane32 < 28) {
    float scale = pow2_group_scale(mx_floor_max(amax, kFp8AmaxFloor), 448.0f);
#pragma unroll
    for (int j = 0; j < 16; j++) ov[j] = fp8_roundtrip(xv[j], scale);
  } else {
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int p = (16 * lane32 + 2 * j - 448) / 2;
      rope_pair_f16(xv[2 * j], xv[2 * j + 1], cs[p], sn[p], &ov[2 * j], &ov[2 * j + 1]);
    }
  }
  uint32_t o[8];
#pragma unroll
  for (int j = 0; j < 8; j++) o[j] = (uint32_t)f32_to_f16_bits(ov[2 * j]) | ((uint32_t)f32_to_f16_bits(ov[2 * j + 1]) << 16);
  u32x4_t* dst = reinterpret_cast<u32x4_t*>(row_out + 16 * lane32);
  dst[0] = u32x4_t{o[0], o[1], o[2], o[3]};
  dst[1] = u32x4_t{o[4], o[5], o[6], o[7]};
}

// ------------------------------------------------------------------ score row, float32 pool rows
// Block = 8 waves. The block QATs the (up to 64) query heads into LDS once (four rows per lane, while
// the wave's first pool tile is already on its way), each wave then keeps them in registers as the
// MFMA A operand and walks 32-row tiles of the pool.
//
// The contraction runs on the bf16 MFMA (32x32x16) without giving up exact products: a QAT'd query
// value is a lattice value times a power of two (three significant bits), so it is a bf16 number, and
// so is a QAT'd pool value. A pool tile whose 32-bit words all have a zero low half is multiplied as
// it is (one bf16 piece per value); any other tile is split into three bf16 pieces per value
// (truncated high part, truncated remainder, rest: 8 + 8 + 8 significant bits, exact) and takes three
// passes. Products of two bf16 numbers are exact in the float32 accumulator either way. The float32
// MFMA (32x32x2) this replaces needed 128 instructions of 16 passes per tile against 16 of 8.
__device__ __forceinline__ uint32_t pack_hi16(float lo, float hi) {
  // the high halves of two float32 words side by side: two bf16 values by truncation
  return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}

constexpr int kScoreThreads = 512;
constexpr int kScoreWaves = kScoreThreads / 64;
// float32 row pitch of the QAT'd query block in LDS: 128 values plus 4, so that the 16-byte reads of
// 16 lanes holding 16 different heads fall into different banks
constexpr int kQPitch = 132;

template <int DT, bool STAGE_HALF>
__global__ __launch_bounds__(kScoreThreads) void scores_f32_kernel(const void* __restrict__ q, int n_heads,
                                                                   const float* __restrict__ pooled, int64_t n_rows,
                                                                   const float* __restrict__ weights, float scale,
                                                                   float* __restrict__ scores,
                                                                   const uint16_t* __restrict__ kv_row,
                                                                   const float* __restrict__ inv_freq,
                                                                   const int32_t* __restrict__ params,
                                                                   uint16_t* __restrict__ row_out,
                                                                   const int32_t* __restrict__ valid_rows) {
  __shared__ float qbuf[64 * kQPitch];
  __shared__ float wbuf[64];
  __shared__ float ptab[kPow2TabLen];
  const int tid = threadIdx.x;
  // With a KV row to prepare (the fused decode prep), the launch carries one more workgroup, the last one,
  // whose first wave does that small job next to the score workgroups instead of in a launch of its own.
  const int score_blocks = (int)gridDim.x - (kv_row ? 1 : 0);
  if ((int)blockIdx.x == score_blocks) {
    kv_row_job(tid, qbuf, qbuf + 32, kv_row, inv_freq, params, row_out);
    return;
  }
  const int lane = tid & 63;
  const int lane32 = tid & 31;
  const int wave = tid >> 6;
  const int half = (tid >> 5) & 1;
  const int m = lane & 31;
  const int g = lane >> 5;

  const int64_t n_tiles = (n_rows + 31) / 32;
  const int64_t wave_stride = (int64_t)score_blocks * kScoreWaves;
  int64_t tile = (int64_t)blockIdx.x * kScoreWaves + wave;

  // The eight waves QAT the 64 query rows, one row per half-wave and four rows per lane; the rows of a
  // lane are fetched together and the power-of-two table sits in LDS, so the pass waits for memory once.
  f32x4_t raw[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int h = 16 * i + wave * 2 + half;
    raw[i] = load_row4<DT>(q, h < n_heads ? h : n_heads - 1, lane32);
  }
  const float tab_a = g_pow2_tab[tid < kPow2TabLen ? tid : 0];
  const float w_mine = weights[tid < n_heads ? tid : 0];
  // The first pool tile of the wave is requested now and lands while the queries are prepared. Lane
  // (m = row, g) owns the 64 consecutive float32 values [64 g, 64 g + 64) of its pool row.
  float kv[64];
  auto load_tile = [&](int64_t t) {
    int64_t src = t * 32 + m;
    src = src < n_rows ? src : n_rows - 1;
    const f32x4_t* kp = reinterpret_cast<const f32x4_t*>(pooled + src * 128 + 64 * g);
#pragma unroll
    for (int j = 0; j < 16; j++) {
      const f32x4_t t4 = kp[j];
      kv[4 * j] = t4.x;
      kv[4 * j + 1] = t4.y;
      kv[4 * j + 2] = t4.z;
      kv[4 * j + 3] = t4.w;
    }
  };
  load_tile(tile < n_tiles ? tile : n_tiles - 1);

  if (tid < kPow2TabLen) ptab[tid] = tab_a;
  if (tid < 64) wbuf[tid] = tid < n_heads ? w_mine : 0.0f;
  __syncthreads();
  QatRotated rot[4];
#pragma unroll
  for (int i = 0; i < 4; i++) rot[i] = qat_rotate(raw[i], lane32);
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int h = 16 * i + wave * 2 + half;
    f32x4_t y = qat_snap(rot[i].x, qat_scale(rot[i].amax, ptab));
    if (STAGE_HALF) {
#pragma unroll
      for (int j = 0; j < 4; j++) y[j] = f16_bits_to_f32(f32_to_f16_bits(y[j]));
    }
    if (h >= n_heads) y = f32x4_t{0.f, 0.f, 0.f, 0.f};
    reinterpret_cast<f32x4_t*>(qbuf + h * kQPitch)[lane32] = y;
  }
  __syncthreads();

  // A operand: lane (m -> head, g) holds q[head][64 g + 8 s .. + 7] as bf16 for k-step s. Piece 0 is the
  // truncated value itself (all of it for a bf16 number), pieces 1 and 2 the truncated remainders.
  auto q_piece = [&](int mt, int s, int piece) -> u32x4_t {
    const f32x4_t t0 = *reinterpret_cast<const f32x4_t*>(qbuf + (mt * 32 + m) * kQPitch + 64 * g + 8 * s);
    const f32x4_t t1 = *reinterpret_cast<const f32x4_t*>(qbuf + (mt * 32 + m) * kQPitch + 64 * g + 8 * s + 4);
    float v[8] = {t0.x, t0.y, t0.z, t0.w, t1.x, t1.y, t1.z, t1.w};
    for (int p = 0; p < piece; p++)
#pragma unroll
      for (int j = 0; j < 8; j++) v[j] = v[j] - __uint_as_float(__float_as_uint(v[j]) & 0xFFFF0000u);
    return u32x4_t{pack_hi16(v[0], v[1]), pack_hi16(v[2], v[3]), pack_hi16(v[4], v[5]), pack_hi16(v[6], v[7])};
  };
  u32x4_t qa[2][8];
  uint32_t q_low = 0u;
#pragma unroll
  for (int mt = 0; mt < 2; mt++) {
#pragma unroll
    for (int s = 0; s < 8; s++) {
      const u32x4_t* src = reinterpret_cast<const u32x4_t*>(qbuf + (mt * 32 + m) * kQPitch + 64 * g + 8 * s);
      const u32x4_t t0 = src[0], t1 = src[1];
      qa[mt][s] = u32x4_t{__builtin_amdgcn_perm(t0.y, t0.x, 0x07060302u), __builtin_amdgcn_perm(t0.w, t0.z, 0x07060302u),
                          __builtin_amdgcn_perm(t1.y, t1.x, 0x07060302u), __builtin_amdgcn_perm(t1.w, t1.z, 0x07060302u)};
      q_low |= t0.x | t0.y | t0.z | t0.w | t1.x | t1.y | t1.z | t1.w;
    }
  }
  // a QAT'd value is a bf16 number (zero low half) unless the input was out of range; then the whole
  // workgroup takes the three-piece form (the pieces come from LDS again, they are not kept in registers)
  const bool q_exact = __syncthreads_and((q_low & 0xFFFFu) == 0u);
  // head weights for this lane's accumulator rows: head = 32mt + 8(i/4) + 4g + i%4
  float wl[2][16];
#pragma unroll
  for (int mt = 0; mt < 2; mt++)
#pragma unroll
    for (int i = 0; i < 16; i++) wl[mt][i] = wbuf[32 * mt + 8 * (i / 4) + 4 * g + (i % 4)];

  while (tile < n_tiles) {
    const int64_t row = tile * 32 + m;
    uint32_t low = 0u;
#pragma unroll
    for (int j = 0; j < 64; j++) low |= __float_as_uint(kv[j]);
    const bool k_exact = __all((low & 0xFFFFu) == 0u);  // wave-uniform
    f32x16_t acc0 = {0}, acc1 = {0};
    auto k_operand = [&](const float (&kk)[64], int s) -> bf16x8_t {
      const u32x4_t kf = {pack_hi16(kk[8 * s], kk[8 * s + 1]), pack_hi16(kk[8 * s + 2], kk[8 * s + 3]),
                          pack_hi16(kk[8 * s + 4], kk[8 * s + 5]), pack_hi16(kk[8 * s + 6], kk[8 * s + 7])};
      return __builtin_bit_cast(bf16x8_t, kf);
    };
    if (k_exact && q_exact) {
#pragma unroll
      for (int s = 0; s < 8; s++) {
        const bf16x8_t kfb = k_operand(kv, s);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, qa[0][s]), kfb, acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, qa[1][s]), kfb, acc1, 0, 0, 0);
      }
    } else {
      // every piece of q meets every piece of k, smallest products first
      const int q_pieces = q_exact ? 1 : 3;
      for (int kp_i = 2; kp_i >= 0; kp_i--) {
        float kk[64];
#pragma unroll
        for (int j = 0; j < 64; j++) {
          float v = kv[j];
          for (int p = 0; p < kp_i; p++) v = v - __uint_as_float(__float_as_uint(v) & 0xFFFF0000u);
          kk[j] = v;
        }
        for (int qp_i = q_pieces - 1; qp_i >= 0; qp_i--) {
#pragma unroll
          for (int s = 0; s < 8; s++) {
            const bf16x8_t kfb = k_operand(kk, s);
            const u32x4_t q0 = qp_i == 0 ? qa[0][s] : q_piece(0, s, qp_i);
            const u32x4_t q1 = qp_i == 0 ? qa[1][s] : q_piece(1, s, qp_i);
            acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, q0), kfb, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, q1), kfb, acc1, 0, 0, 0);
          }
        }
      }
    }
    tile += wave_stride;
    if (tile < n_tiles) load_tile(tile);  // lands during the epilogue
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
    // fixed-capacity form: the pool buffer holds n_rows rows of which the first *valid_rows are in use (a
    // count that lives on the device, so that a captured launch follows a growing pool); the rest score -inf
    if (g == 0 && row < n_rows) scores[row] = (valid_rows && row >= (int64_t)valid_rows[0]) ? -__builtin_inff() : sum;
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

// kv_row (with inv_freq, params, row_out) may be null: no prepared KV row in this launch
int mspr_launch_scores_f32(const void* q, int q_dtype, int n_heads, const float* pooled, int64_t n_rows,
                           const float* weights, float scale, float* scores, bool stage_half, const void* kv_row,
                           const float* inv_freq, const int32_t* params, void* row_out, const int32_t* valid_rows,
                           hipStream_t st) {
  int64_t n_tiles = (n_rows + 31) / 32;
  int64_t blocks = (n_tiles + kScoreWaves - 1) / kScoreWaves;
  if (blocks > 2048) blocks = 2048;
  dim3 grid((unsigned)(blocks + (kv_row ? 1 : 0))), block(kScoreThreads);
  const uint16_t* kvp = reinterpret_cast<const uint16_t*>(kv_row);
  uint16_t* rop = reinterpret_cast<uint16_t*>(row_out);
  MsprProfScope prof(MSPR_K_SCORES_F32, st);
#define MSPR_SCORES_LAUNCH(DT)                                                                          \
  do {                                                                                                  \
    if (stage_half)                                                                                     \
      scores_f32_kernel<DT, true><<<grid, block, 0, st>>>(q, n_heads, pooled, n_rows, weights, scale, scores, kvp, \
                                                          inv_freq, params, rop, valid_rows);            \
    else                                                                                                \
      scores_f32_kernel<DT, false><<<grid, block, 0, st>>>(q, n_heads, pooled, n_rows, weights, scale, scores, kvp, \
                                                           inv_freq, params, rop, valid_rows);            \
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
  return mspr_launch_scores_f32(q, q_dtype, n_heads, pooled_qat, n_rows, weights, scale, scores, false, nullptr,
                                nullptr, nullptr, nullptr, nullptr, (hipStream_t)stream);
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

