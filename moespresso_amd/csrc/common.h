// Shared device/host helpers for the gfx950 kernels (wave64, MFMA, LDS).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/moespresso_amd.h"

#define MSPR_WAVE 64

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

#define MSPR_LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

// ---------------------------------------------------------------- host side

void mspr_set_error(const char* fmt, ...);

#define MSPR_REQUIRE(cond, ...)          \
  do {                                   \
    if (!(cond)) {                       \
      mspr_set_error(__VA_ARGS__);       \
      return MSPR_ERR_ARG;               \
    }                                    \
  } while (0)

#define MSPR_CHECK_LAUNCH(name)                                              \
  do {                                                                       \
    hipError_t e_ = hipGetLastError();                                       \
    if (e_ != hipSuccess) {                                                  \
      mspr_set_error("%s: launch failed: %s", name, hipGetErrorString(e_));  \
      return MSPR_ERR_LAUNCH;                                                \
    }                                                                        \
  } while (0)

static inline bool mspr_aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// ---------------------------------------------------------------- device side

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// float32 -> bfloat16 bits, round to nearest even (NaN kept quiet).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) {
  _Float16 h;
  __builtin_memcpy(&h, &b, 2);
  return (float)h;
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  // v_cvt_f16_f32 (round to nearest even), written out so that the compiler cannot merge a preceding
  // float32 multiply into v_fma_mixlo_f16 with a +0 addend: that form turns a product of -0 into +0
  uint32_t r;
  asm("v_cvt_f16_f32 %0, %1" : "=v"(r) : "v"(f));
  return (uint16_t)r;
}

// Load element i of a row stored as f32 / f16 / bf16, widened to float32 (exact).
template <int DT>
__device__ __forceinline__ float load_as_f32(const void* p, int64_t i) {
  if constexpr (DT == MSPR_F32) {
    return reinterpret_cast<const float*>(p)[i];
  } else if constexpr (DT == MSPR_F16) {
    return f16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i]);
  } else {
    return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i]);
  }
}

__device__ __forceinline__ float wave_xor_f32(float v, int mask) { return __shfl_xor(v, mask, MSPR_WAVE); }

// The value lane (l ^ M) holds, for a single-bit M. Inside a row of 16 lanes the exchange is one or two
// data-parallel-primitive moves (quad permutes give l^1, l^2, l^3; the half-row and row mirrors give
// l^7 and l^15, and two of them compose to l^4 and l^8), which cost an ALU slot and no LDS round trip;
// l^16 is a bit-mask swizzle, l^32 the general lane permute.
template <int M>
__device__ __forceinline__ float lane_xor(float v) {
  static_assert(M == 1 || M == 2 || M == 4 || M == 8 || M == 16 || M == 32, "single-bit lane masks only");
  int x = __float_as_int(v);
  if constexpr (M == 1) {
    x = __builtin_amdgcn_mov_dpp(x, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
  } else if constexpr (M == 2) {
    x = __builtin_amdgcn_mov_dpp(x, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
  } else if constexpr (M == 4) {
    x = __builtin_amdgcn_mov_dpp(x, 0x141, 0xF, 0xF, true);  // row_half_mirror: l^7
    x = __builtin_amdgcn_mov_dpp(x, 0x1B, 0xF, 0xF, true);   // quad_perm [3,2,1,0]: l^3
  } else if constexpr (M == 8) {
    x = __builtin_amdgcn_mov_dpp(x, 0x140, 0xF, 0xF, true);  // row_mirror: l^15
    x = __builtin_amdgcn_mov_dpp(x, 0x141, 0xF, 0xF, true);  // row_half_mirror: l^7
  } else if constexpr (M == 16) {
    x = __builtin_amdgcn_ds_swizzle(x, 0x401F);  // and 0x1F, or 0, xor 0x10
  } else {
    x = __shfl_xor(x, 32, MSPR_WAVE);
  }
  return __int_as_float(x);
}

// max / sum of a value over the two half-waves (lane l with lane l ^ 32), the same result in both lanes.
// v_permlane32_swap exchanges the upper half of its first operand with the lower half of its second: with
// two copies of the value, each lane ends up holding its own and its partner's value in the two registers.
// A vector-ALU exchange, so no LDS round trip as with the general lane permute. (The waits around it are
// the distance the instruction needs from vector writes of its operands and to reads of its results.)
__device__ __forceinline__ void half_wave_exchange(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float half_wave_max(float v) {
  float w = v;
  half_wave_exchange(v, w);
  return fmaxf(v, w);
}
// the same over lanes l and l ^ 16 (v_permlane16_swap: odd rows of 16 lanes of the first operand with the
// even rows of the second)
__device__ __forceinline__ float row_pair_max(float v) {
  float w = v;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(v), "+v"(w));
  return fmaxf(v, w);
}
__device__ __forceinline__ float half_wave_sum(float v) {
  float w = v;
  half_wave_exchange(v, w);
  return v + w;
}

// Monotone float32 -> uint32 map: negatives inverted, positives offset. Orders -0.0 below +0.0
// and +NaN above +inf.
__device__ __forceinline__ uint32_t score_key(float s) {
  uint32_t u = __float_as_uint(s);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

#include "tables.inc"

#define MSPR_POW2_TAB_MIN (-160)
#define MSPR_LN2F 0x1.62e430p-1f

// exp(ceil(log(amax/denom)/ln2)*ln2) with every step in float32 and correctly rounded log/exp.
// g_pow2_tab holds float32(exp(float32(k*ln2f))) for k = -160..160. Away from powers of two the
// ceil is decided from the exponent field; within 2^-12 of one (and for non-finite or zero input)
// a float64 log decides it, which rounds to the same float32 value the table path assumes.
// `tab` may be a copy of the table in LDS.
__device__ __forceinline__ float pow2_group_scale(float amax, float denom, const float* tab = g_pow2_tab) {
  float r = amax / denom;
  uint32_t u = __float_as_uint(r);
  uint32_t ex = (u >> 23) & 0xFFu;
  uint32_t man = u & 0x7FFFFFu;
  bool fast = (u >> 31) == 0u && ex != 0u && ex != 0xFFu && man > 0x800u && man < 0x7FF800u;
  if (fast) {
    int k = (int)ex - 127 + 1;
    return tab[k - MSPR_POW2_TAB_MIN];
  }
  float l = (float)log((double)r);
  float l2 = l / MSPR_LN2F;
  float e = ceilf(l2) * MSPR_LN2F;
  return (float)exp((double)e);
}
