// Affine 8-bit quantisation of KV rows in groups of 64 (the layout mx.quantize(group_size=64, bits=8)
// produces and the Q8 attention kernels consume) and its inverse.
//
// Per group: scale = max((max - min) / 255, 1e-7), signed so that the edge of larger magnitude is
// hit exactly (edge = min if |min| > |max| else max; q0 = round(edge / scale); scale = edge / q0 and
// bias = edge unless q0 == 0, then bias = 0); code = min(round((x - bias) / scale), 255). Float32
// arithmetic, one operation per step; scales and biases are stored in the input's element type, the
// codes are taken with the unrounded float32 scale and bias.
//
// A thread owns four consecutive elements (one packed word), sixteen threads own a group; both
// kernels are pure streaming passes.
#include "common.h"

#pragma clang fp contract(off)

namespace {

template <int DT>
__device__ __forceinline__ void store_sb(void* p, int64_t i, float v) {
  if constexpr (DT == MSPR_F32) reinterpret_cast<float*>(p)[i] = v;
  else if constexpr (DT == MSPR_F16) reinterpret_cast<uint16_t*>(p)[i] = f32_to_f16_bits(v);
  else reinterpret_cast<uint16_t*>(p)[i] = f32_to_bf16_bits(v);
}

template <int DT>
__device__ __forceinline__ f32x4_t load4(const void* p, int64_t i4) {
  if constexpr (DT == MSPR_F32) {
    return reinterpret_cast<const f32x4_t*>(p)[i4];
  } else {
    const u32x2_t w = reinterpret_cast<const u32x2_t*>(p)[i4];
    if constexpr (DT == MSPR_F16)
      return f32x4_t{f16_bits_to_f32((uint16_t)(w.x & 0xFFFFu)), f16_bits_to_f32((uint16_t)(w.x >> 16)),
                     f16_bits_to_f32((uint16_t)(w.y & 0xFFFFu)), f16_bits_to_f32((uint16_t)(w.y >> 16))};
    else
      return f32x4_t{bf16_bits_to_f32((uint16_t)(w.x & 0xFFFFu)), bf16_bits_to_f32((uint16_t)(w.x >> 16)),
                     bf16_bits_to_f32((uint16_t)(w.y & 0xFFFFu)), bf16_bits_to_f32((uint16_t)(w.y >> 16))};
  }
}

template <int DT>
__global__ __launch_bounds__(256) void affine_q8_quantize_kernel(const void* __restrict__ x, int64_t n_groups,
                                                                 uint32_t* __restrict__ wq, void* __restrict__ scales,
                                                                 void* __restrict__ biases) {
  const int64_t i4 = (int64_t)blockIdx.x * 256 + threadIdx.x;  // packed word index
  const int64_t group = i4 >> 4;
  const bool live = group < n_groups;
  const f32x4_t v = load4<DT>(x, live ? i4 : 0);
  float mx = fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w));
  float mn = fminf(fminf(v.x, v.y), fminf(v.z, v.w));
#pragma unroll
  for (int m = 1; m <= 8; m <<= 1) {
    mx = fmaxf(mx, __shfl_xor(mx, m, MSPR_WAVE));
    mn = fminf(mn, __shfl_xor(mn, m, MSPR_WAVE));
  }
  float scale = fmaxf((mx - mn) / 255.0f, 1e-7f);
  const bool side = fabsf(mn) > fabsf(mx);
  scale = side ? scale : -scale;
  const float edge = side ? mn : mx;
  const float q0 = rintf(edge / scale);
  const bool at_zero = q0 == 0.0f;
  scale = at_zero ? scale : edge / q0;
  const float bias = at_zero ? 0.0f : edge;
  uint32_t word = 0;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    float c = rintf((v[j] - bias) / scale);
    c = c < 255.0f ? c : 255.0f;
    c = c > 0.0f ? c : 0.0f;
    word |= (uint32_t)c << (8 * j);
  }
  if (live) {
    wq[i4] = word;
    if ((threadIdx.x & 15) == 0) {
      store_sb<DT>(scales, group, scale);
      store_sb<DT>(biases, group, bias);
    }
  }
}

template <int DT>
__global__ __launch_bounds__(256) void affine_q8_dequantize_kernel(const uint32_t* __restrict__ wq,
                                                                   const void* __restrict__ scales,
                                                                   const void* __restrict__ biases, int64_t n_groups,
                                                                   void* __restrict__ out) {
  const int64_t i4 = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t group = i4 >> 4;
  if (group >= n_groups) return;
  const float s = load_as_f32<DT>(scales, group), b = load_as_f32<DT>(biases, group);
  const uint32_t w = wq[i4];
  float r[4];
#pragma unroll
  for (int j = 0; j < 4; j++) r[j] = (float)((w >> (8 * j)) & 0xFFu) * s + b;
  if constexpr (DT == MSPR_F32) {
    reinterpret_cast<f32x4_t*>(out)[i4] = f32x4_t{r[0], r[1], r[2], r[3]};
  } else if constexpr (DT == MSPR_F16) {
    reinterpret_cast<u32x2_t*>(out)[i4] =
        u32x2_t{(uint32_t)f32_to_f16_bits(r[0]) | ((uint32_t)f32_to_f16_bits(r[1]) << 16),
                (uint32_t)f32_to_f16_bits(r[2]) | ((uint32_t)f32_to_f16_bits(r[3]) << 16)};
  } else {
    reinterpret_cast<u32x2_t*>(out)[i4] =
        u32x2_t{(uint32_t)f32_to_bf16_bits(r[0]) | ((uint32_t)f32_to_bf16_bits(r[1]) << 16),
                (uint32_t)f32_to_bf16_bits(r[2]) | ((uint32_t)f32_to_bf16_bits(r[3]) << 16)};
  }
}

}  // namespace

extern "C" int mspr_affine_q8_quantize(const void* x, int dtype, int64_t n_groups, void* wq, void* scales,
                                       void* biases, int group_size, int bits, void* stream) {
  MSPR_REQUIRE(group_size == 64 && bits == 8, "affine_q8_quantize: only group_size=64, bits=8 is supported");
  MSPR_REQUIRE(x && wq && scales && biases, "affine_q8_quantize: null pointer");
  MSPR_REQUIRE(dtype >= MSPR_F32 && dtype <= MSPR_BF16, "affine_q8_quantize: dtype must be f32, f16 or bf16");
  MSPR_REQUIRE(n_groups >= 1 && n_groups < ((int64_t)1 << 40), "affine_q8_quantize: expects at least one group");
  MSPR_REQUIRE(mspr_aligned(x, 16) && mspr_aligned(wq, 4), "affine_q8_quantize: pointers must be 16-byte aligned");
  dim3 grid((unsigned)((n_groups * 16 + 255) / 256)), block(256);
  hipStream_t st = (hipStream_t)stream;
  uint32_t* w = reinterpret_cast<uint32_t*>(wq);
  if (dtype == MSPR_F32) affine_q8_quantize_kernel<MSPR_F32><<<grid, block, 0, st>>>(x, n_groups, w, scales, biases);
  else if (dtype == MSPR_F16) affine_q8_quantize_kernel<MSPR_F16><<<grid, block, 0, st>>>(x, n_groups, w, scales, biases);
  else affine_q8_quantize_kernel<MSPR_BF16><<<grid, block, 0, st>>>(x, n_groups, w, scales, biases);
  MSPR_CHECK_LAUNCH("affine_q8_quantize");
  return MSPR_OK;
}

extern "C" int mspr_affine_q8_dequantize(const void* wq, const void* scales, const void* biases, int dtype,
                                         int64_t n_groups, void* out, int group_size, int bits, void* stream) {
  MSPR_REQUIRE(group_size == 64 && bits == 8, "affine_q8_dequantize: only group_size=64, bits=8 is supported");
  MSPR_REQUIRE(wq && scales && biases && out, "affine_q8_dequantize: null pointer");
  MSPR_REQUIRE(dtype >= MSPR_F32 && dtype <= MSPR_BF16, "affine_q8_dequantize: dtype must be f32, f16 or bf16");
  MSPR_REQUIRE(n_groups >= 1 && n_groups < ((int64_t)1 << 40), "affine_q8_dequantize: expects at least one group");
  MSPR_REQUIRE(mspr_aligned(out, 16) && mspr_aligned(wq, 4), "affine_q8_dequantize: pointers must be 16-byte aligned");
  dim3 grid((unsigned)((n_groups * 16 + 255) / 256)), block(256);
  hipStream_t st = (hipStream_t)stream;
  const uint32_t* w = reinterpret_cast<const uint32_t*>(wq);
  if (dtype == MSPR_F32) affine_q8_dequantize_kernel<MSPR_F32><<<grid, block, 0, st>>>(w, scales, biases, n_groups, out);
  else if (dtype == MSPR_F16) affine_q8_dequantize_kernel<MSPR_F16><<<grid, block, 0, st>>>(w, scales, biases, n_groups, out);
  else affine_q8_dequantize_kernel<MSPR_BF16><<<grid, block, 0, st>>>(w, scales, biases, n_groups, out);
  MSPR_CHECK_LAUNCH("affine_q8_dequantize");
  return MSPR_OK;
}
