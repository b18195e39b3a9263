// Partial rotary embedding of the last 64 channels of rows laid out [..., seq, width]; the leading
// channels copy through. One pass replaces the composed split / angle table / cos / sin / four
// multiplies / stack / concat sequence, with that sequence's rounding: the angle is one float32
// multiply position * inv_freq[p]; cos and sin are taken at float32 and cast to the element type (the
// inverse form negates the float32 sine first); every product and every sum of the rotation is
// rounded to the element type on its own (float32 rows: float32 operations, never contracted).
//
// A workgroup owns one sequence position and a slab of the outer rows (batch x heads): the 32
// cosine / sine pairs of the position are worked out once, by the first 32 threads, and shared
// through LDS, so the transcendental work does not grow with the head count; the rows then stream
// through with 16-byte (float32) or 8-byte (16-bit) accesses.
#include "common.h"

#pragma clang fp contract(off)

namespace {

constexpr int kRopeDim = 64;
constexpr int kRopeFreqs = kRopeDim / 2;
constexpr int kThreads = 256;

template <int DT>
__device__ __forceinline__ float round_to(float v) {
  if constexpr (DT == MSPR_F32) return v;
  else if constexpr (DT == MSPR_F16) return f16_bits_to_f32(f32_to_f16_bits(v));
  else return bf16_bits_to_f32(f32_to_bf16_bits(v));
}

template <int DT>
__device__ __forceinline__ f32x4_t load_quad(const void* p, int64_t quad) {
  if constexpr (DT == MSPR_F32) {
    return reinterpret_cast<const f32x4_t*>(p)[quad];
  } else {
    const u32x2_t w = reinterpret_cast<const u32x2_t*>(p)[quad];
    if constexpr (DT == MSPR_F16)
      return f32x4_t{f16_bits_to_f32((uint16_t)(w.x & 0xFFFFu)), f16_bits_to_f32((uint16_t)(w.x >> 16)),
                     f16_bits_to_f32((uint16_t)(w.y & 0xFFFFu)), f16_bits_to_f32((uint16_t)(w.y >> 16))};
    else
      return f32x4_t{bf16_bits_to_f32((uint16_t)(w.x & 0xFFFFu)), bf16_bits_to_f32((uint16_t)(w.x >> 16)),
                     bf16_bits_to_f32((uint16_t)(w.y & 0xFFFFu)), bf16_bits_to_f32((uint16_t)(w.y >> 16))};
  }
}

template <int DT>
__device__ __forceinline__ void store_quad(void* p, int64_t quad, f32x4_t v) {
  if constexpr (DT == MSPR_F32) {
    reinterpret_cast<f32x4_t*>(p)[quad] = v;
  } else if constexpr (DT == MSPR_F16) {
    reinterpret_cast<u32x2_t*>(p)[quad] =
        u32x2_t{(uint32_t)f32_to_f16_bits(v.x) | ((uint32_t)f32_to_f16_bits(v.y) << 16),
                (uint32_t)f32_to_f16_bits(v.z) | ((uint32_t)f32_to_f16_bits(v.w) << 16)};
  } else {
    reinterpret_cast<u32x2_t*>(p)[quad] =
        u32x2_t{(uint32_t)f32_to_bf16_bits(v.x) | ((uint32_t)f32_to_bf16_bits(v.y) << 16),
                (uint32_t)f32_to_bf16_bits(v.z) | ((uint32_t)f32_to_bf16_bits(v.w) << 16)};
  }
}

// grid: (seq_len, slabs); a slab is `rows_per_wg` outer rows
template <int DT>
__global__ __launch_bounds__(kThreads) void partial_rope_kernel(const void* __restrict__ x, int64_t n_outer,
                                                               int64_t seq_len, int width,
                                                               const float* __restrict__ inv_freq,
                                                               const float* __restrict__ positions, int64_t offset,
                                                               int inverse, int rows_per_wg, void* __restrict__ out) {
  __shared__ float cs[kRopeFreqs], sn[kRopeFreqs];
  const int tid = threadIdx.x;
  const int64_t l = blockIdx.x;
  if (tid < kRopeFreqs) {
    const float pos = positions ? positions[l] : (float)(offset + l);
    const float theta = pos * inv_freq[tid];
    // float32 cosine and sine of the float32 angle, correctly rounded
    const float c = (float)cos((double)theta);
    float s = (float)sin((double)theta);
    if (inverse) s = -s;
    cs[tid] = round_to<DT>(c);
    sn[tid] = round_to<DT>(s);
  }
  __syncthreads();

  const int quads = width / 4;
  const int tail_quad = (width - kRopeDim) / 4;
  const int64_t o0 = (int64_t)blockIdx.y * rows_per_wg;
  int64_t o1 = o0 + rows_per_wg;
  if (o1 > n_outer) o1 = n_outer;
  const int64_t items = (o1 - o0) * quads;
  for (int64_t it = tid; it < items; it += kThreads) {
    const int64_t o = o0 + it / quads;
    const int qd = (int)(it % quads);
    const int64_t quad = (o * seq_len + l) * quads + qd;
    f32x4_t v = load_quad<DT>(x, quad);
    if (qd >= tail_quad) {
      const int p = 2 * (qd - tail_quad);  // first of the two pairs of this quad
      f32x4_t r;
      {
        const float c = cs[p], s = sn[p];
        const float m0 = round_to<DT>(v.x * c), m1 = round_to<DT>(v.y * s);
        const float m2 = round_to<DT>(v.x * s), m3 = round_to<DT>(v.y * c);
        r.x = round_to<DT>(m0 - m1);
        r.y = round_to<DT>(m2 + m3);
      }
      {
        const float c = cs[p + 1], s = sn[p + 1];
        const float m0 = round_to<DT>(v.z * c), m1 = round_to<DT>(v.w * s);
        const float m2 = round_to<DT>(v.z * s), m3 = round_to<DT>(v.w * c);
        r.z = round_to<DT>(m0 - m1);
        r.w = round_to<DT>(m2 + m3);
      }
      v = r;
    }
    store_quad<DT>(out, quad, v);
  }
}

}  // namespace

extern "C" int mspr_fused_partial_rope(const void* x, int dtype, int64_t n_outer, int64_t seq_len, int width,
                                       const float* inv_freq, const float* positions, int64_t offset, int inverse,
                                       void* out, void* stream) {
  MSPR_REQUIRE(x && inv_freq && out, "fused_partial_rope: null pointer");
  MSPR_REQUIRE(dtype == MSPR_F32 || dtype == MSPR_F16 || dtype == MSPR_BF16,
               "fused_partial_rope: rows must be float32, float16, or bfloat16");
  MSPR_REQUIRE(n_outer >= 1 && seq_len >= 1, "fused_partial_rope: at least one row");
  MSPR_REQUIRE(seq_len <= 0x7FFFFFFF && n_outer * seq_len <= 0x7FFFFFFF, "fused_partial_rope: too many rows");
  MSPR_REQUIRE(width >= kRopeDim && width % 4 == 0, "fused_partial_rope: width must be a multiple of 4 and at least 64");
  MSPR_REQUIRE(positions || (offset >= 0 && offset + seq_len <= ((int64_t)1 << 24)),
               "fused_partial_rope: positions must stay exact in float32");
  MSPR_REQUIRE(mspr_aligned(x, 16) && mspr_aligned(out, 16), "fused_partial_rope: rows must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  // slabs: enough workgroups to cover the chip, at least one quad per thread and pass
  const int quads = width / 4;
  int64_t rows_per_wg = (kThreads * 4 + quads - 1) / quads;  // about four passes of the thread block
  const int64_t want_wgs = 1024;
  const int64_t max_rows = (n_outer * seq_len + want_wgs - 1) / want_wgs;
  if (rows_per_wg > max_rows) rows_per_wg = max_rows;
  if (rows_per_wg < 1) rows_per_wg = 1;
  if (rows_per_wg > n_outer) rows_per_wg = n_outer;
  const int64_t slabs = (n_outer + rows_per_wg - 1) / rows_per_wg;
  MSPR_REQUIRE(slabs <= 65535, "fused_partial_rope: too many outer rows for one launch");
  dim3 grid((unsigned)seq_len, (unsigned)slabs), block(kThreads);
  if (dtype == MSPR_F32)
    partial_rope_kernel<MSPR_F32><<<grid, block, 0, st>>>(x, n_outer, seq_len, width, inv_freq, positions, offset,
                                                         inverse, (int)rows_per_wg, out);
  else if (dtype == MSPR_F16)
    partial_rope_kernel<MSPR_F16><<<grid, block, 0, st>>>(x, n_outer, seq_len, width, inv_freq, positions, offset,
                                                         inverse, (int)rows_per_wg, out);
  else
    partial_rope_kernel<MSPR_BF16><<<grid, block, 0, st>>>(x, n_outer, seq_len, width, inv_freq, positions, offset,
                                                          inverse, (int)rows_per_wg, out);
  MSPR_CHECK_LAUNCH("fused_partial_rope");
  return MSPR_OK;
}
