// One-token GQA decode attention over an 8-bit quantised KV cache, dequantised in-kernel.
//
// Two cache formats:
//   Q8_0   : int8 codes, one float16 scale per 32 elements          value = code * scale
//   AFFINE : uint8 codes (four per 32-bit word), one scale and one   value = code * scale + bias
//            bias per 64 elements (the MLX affine 8-bit layout)
// Head dim 256, up to 16 query heads per KV head.
//
// A workgroup owns (batch, kv head, key range); each of its waves walks 32-key tiles of that
// range on its own (private online softmax state), the waves are merged through LDS at the end and
// the per-range partials by a second kernel.
//
// Per tile and wave: K codes go from HBM straight into registers (a lane owns 64 contiguous bytes of
// its key row), are dequantised to float16 with packed ops and feed v_mfma_f32_16x16x32_f16 as the A
// operand (S^T = K.Q^T, keys x heads, so the softmax statistics of a head live in one lane column).
// V codes are dequantised to a row-major float16 tile in LDS, and the V^T operand of
// O^T = V^T.P^T comes out of it through the LDS transpose read.
#include "common.h"
#include "profile.h"

namespace {

constexpr int kD = 256;
constexpr int kTileKeys = 32;
constexpr int kQ8Waves = 4;  // waves per workgroup of the split kernel (8 measured 7-25 % slower at batch 8 / 1)
constexpr int kVPitch = kD * 2 + 16;           // bytes per key row of the float16 V tile
constexpr int kVTileBytes = kTileKeys * kVPitch;
constexpr int kFmtQ8_0 = 0;
constexpr int kFmtAffine = 1;

typedef __attribute__((ext_vector_type(2))) _Float16 h2_t;

struct Q8Args {
  const void* q;        // [B, Hq, D]
  const void* k_codes;  // [B, Hkv, N, D] bytes
  const void* k_scales;
  const void* k_biases;
  const void* v_codes;
  const void* v_scales;
  const void* v_biases;
  int batch, n_q_heads, n_kv_heads;
  int64_t n_keys;
  int64_t kv_rows;  // rows allocated per (batch, kv head); >= n_keys
  float scale_log2;
  int n_splits;
  int keys_per_split;
  float* ws_o;   // [B, Hkv, S, 16, 256]
  float* ws_ml;  // [B, Hkv, S, 16, 2]
  void* out;     // [B, Hq, D]
};

__device__ __forceinline__ f32x4_t mfma16(u32x4_t a, u32x4_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0,
                                                0);
}

__device__ __forceinline__ uint32_t h2_bits(h2_t v) { return __builtin_bit_cast(uint32_t, v); }
__device__ __forceinline__ h2_t bits_h2(uint32_t v) { return __builtin_bit_cast(h2_t, v); }

template <int SDT>
__device__ __forceinline__ _Float16 load_scale(const void* p, int64_t i) {
  return (_Float16)load_as_f32<SDT>(p, i);
}

// Four codes of one 32-bit word to four float16 values (two packed registers), exact integers:
// byte b becomes the float16 with bits 0x6400 | b = 1024 + b, then the offset is taken off.
template <int FMT>
__device__ __forceinline__ void codes4_to_h(uint32_t w, h2_t& lo, h2_t& hi) {
  if constexpr (FMT == kFmtQ8_0) {
    w ^= 0x80808080u;  // int8 -> offset binary
    lo = bits_h2(__builtin_amdgcn_perm(0x64646464u, w, 0x04010400u)) - h2_t{(_Float16)1152.0f, (_Float16)1152.0f};
    hi = bits_h2(__builtin_amdgcn_perm(0x64646464u, w, 0x04030402u)) - h2_t{(_Float16)1152.0f, (_Float16)1152.0f};
  } else {
    lo = bits_h2(__builtin_amdgcn_perm(0x64646464u, w, 0x04010400u)) - h2_t{(_Float16)1024.0f, (_Float16)1024.0f};
    hi = bits_h2(__builtin_amdgcn_perm(0x64646464u, w, 0x04030402u)) - h2_t{(_Float16)1024.0f, (_Float16)1024.0f};
  }
}

template <int FMT, int QDT, int SDT>
__global__ __launch_bounds__(64 * kQ8Waves, 1) void q8_decode_split_kernel(Q8Args a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n = lane & 15;   // MFMA column: query head of the group; MFMA row (key) for the K operand
  const int g = lane >> 4;   // 0..3
  unsigned char* vt = lds + wave * kVTileBytes;  // this wave's V tile

  const int sp = blockIdx.x;
  const int kvh = blockIdx.y;
  const int b = blockIdx.z;
  const int rep = a.n_q_heads / a.n_kv_heads;
  const int64_t N = a.n_keys;
  const int64_t k0 = (int64_t)sp * a.keys_per_split;
  int64_t k1 = k0 + a.keys_per_split;
  if (k1 > N) k1 = N;

  const int64_t kv_row0 = ((int64_t)b * a.n_kv_heads + kvh) * a.kv_rows;  // first key row of this (b, kv head)
  const uint8_t* kc = reinterpret_cast<const uint8_t*>(a.k_codes) + kv_row0 * kD;
  const uint8_t* vc = reinterpret_cast<const uint8_t*>(a.v_codes) + kv_row0 * kD;
  constexpr int kGroups = FMT == kFmtQ8_0 ? 8 : 4;  // scale groups per row

  f32x4_t oacc[16];
#pragma unroll
  for (int mt = 0; mt < 16; mt++) oacc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m_run = -__builtin_inff();
  float l_run = 0.0f;

  const int vkey = lane >> 1;   // V staging: lane owns half a key row
  const int vhalf = lane & 1;
  const int tr_s = lane & 15;
  const int tr_off = (4 * g + (tr_s >> 2)) * kVPitch + 4 * (tr_s & 3) * 2;

  // Register images of one tile's codes and scales: K for the two 16-key sub-tiles of the MFMA, V for
  // the lane's half row. Loads of the next K tile are issued before the current V tile is unpacked and
  // the V loads before the current K tile is consumed, so two tiles' worth of bytes stay in flight.
  struct KRegs {
    u32x4_t c[2][4];
    uint32_t s[2], bz[2];
  } kr;
  struct VRegs {
    u32x4_t c[8];
    uint32_t s[2], bz[2];
  } vr;
  const uint8_t* ksc = reinterpret_cast<const uint8_t*>(a.k_scales);
  const uint8_t* kbi = reinterpret_cast<const uint8_t*>(a.k_biases);
  const uint8_t* vsc = reinterpret_cast<const uint8_t*>(a.v_scales);
  const uint8_t* vbi = reinterpret_cast<const uint8_t*>(a.v_biases);
  constexpr int kSB = SDT == MSPR_F32 ? 4 : 2;  // bytes per affine scale / bias

  auto load_k = [&](int64_t key0) {
#pragma unroll
    for (int u = 0; u < 2; u++) {
      int64_t key = key0 + 16 * u + n;
      if (key >= N) key = N - 1;
      const u32x4_t* cp = reinterpret_cast<const u32x4_t*>(kc + key * kD + 64 * g);
#pragma unroll
      for (int j = 0; j < 4; j++) kr.c[u][j] = cp[j];
      if constexpr (FMT == kFmtQ8_0) {
        kr.s[u] = *reinterpret_cast<const uint32_t*>(ksc + ((kv_row0 + key) * 8 + 2 * g) * 2);
      } else if constexpr (SDT == MSPR_F32) {
        kr.s[u] = *reinterpret_cast<const uint32_t*>(ksc + ((kv_row0 + key) * 4 + g) * 4);
        kr.bz[u] = *reinterpret_cast<const uint32_t*>(kbi + ((kv_row0 + key) * 4 + g) * 4);
      } else {
        kr.s[u] = *reinterpret_cast<const uint16_t*>(ksc + ((kv_row0 + key) * 4 + g) * 2);
        kr.bz[u] = *reinterpret_cast<const uint16_t*>(kbi + ((kv_row0 + key) * 4 + g) * 2);
      }
    }
  };
  auto load_v = [&](int64_t key0) {
    int64_t key = key0 + vkey;
    if (key >= N) key = N - 1;
    const u32x4_t* cp = reinterpret_cast<const u32x4_t*>(vc + key * kD + 128 * vhalf);
#pragma unroll
    for (int j = 0; j < 8; j++) vr.c[j] = cp[j];
    if constexpr (FMT == kFmtQ8_0) {
      const u32x2_t sv = *reinterpret_cast<const u32x2_t*>(vsc + ((kv_row0 + key) * 8 + 4 * vhalf) * 2);
      vr.s[0] = sv.x;
      vr.s[1] = sv.y;
    } else if constexpr (SDT == MSPR_F32) {
      const u32x2_t sv = *reinterpret_cast<const u32x2_t*>(vsc + ((kv_row0 + key) * 4 + 2 * vhalf) * 4);
      const u32x2_t bv = *reinterpret_cast<const u32x2_t*>(vbi + ((kv_row0 + key) * 4 + 2 * vhalf) * 4);
      vr.s[0] = sv.x;
      vr.s[1] = sv.y;
      vr.bz[0] = bv.x;
      vr.bz[1] = bv.y;
    } else {
      const uint32_t sv = *reinterpret_cast<const uint32_t*>(vsc + ((kv_row0 + key) * 4 + 2 * vhalf) * 2);
      const uint32_t bv = *reinterpret_cast<const uint32_t*>(vbi + ((kv_row0 + key) * 4 + 2 * vhalf) * 2);
      vr.s[0] = sv & 0xFFFFu;
      vr.s[1] = sv >> 16;
      vr.bz[0] = bv & 0xFFFFu;
      vr.bz[1] = bv >> 16;
    }
  };
  // raw affine scale / bias bits to a packed float16 pair
  auto sb_to_h2 = [&](uint32_t bits) -> h2_t {
    _Float16 h;
    if constexpr (SDT == MSPR_F32) h = (_Float16)__builtin_bit_cast(float, bits);
    else if constexpr (SDT == MSPR_F16) h = __builtin_bit_cast(_Float16, (uint16_t)bits);
    else h = (_Float16)__builtin_bit_cast(float, bits << 16);
    return h2_t{h, h};
  };
  auto h_pair = [&](uint32_t packed, int which) -> h2_t {
    const _Float16 h = __builtin_bit_cast(_Float16, (uint16_t)(which ? packed >> 16 : packed & 0xFFFFu));
    return h2_t{h, h};
  };

  const int64_t n_tiles = k1 > k0 ? (k1 - k0 + kTileKeys - 1) / kTileKeys : 0;
  // Loads are unconditional (a wave past its last tile re-reads its current one, which hits in cache)
  // so that the outstanding-load counts are static and the waits stay partial.
  if (wave < n_tiles) {
    load_k(k0 + (int64_t)wave * kTileKeys);
    load_v(k0 + (int64_t)wave * kTileKeys);
  }
  __builtin_amdgcn_sched_barrier(0);  // the first tile is on its way before the query is fetched: one memory
                                      // round trip in front of the first MFMA instead of two

  // ---- Q^T operand: lane (n = head, g) holds q[head][64g + 8s .. +7] for k-step s, pre-multiplied by
  //      scale * log2(e) and rounded to float16
  u32x4_t qf[8];
  {
    const bool live = n < rep;
    const int64_t qoff = ((int64_t)b * a.n_q_heads + kvh * rep + (live ? n : 0)) * kD + 64 * g;
    float v[8][8];
    if constexpr (QDT == MSPR_F32) {
      const f32x4_t* p = reinterpret_cast<const f32x4_t*>(reinterpret_cast<const float*>(a.q) + qoff);
      f32x4_t raw[16];
#pragma unroll
      for (int j = 0; j < 16; j++) raw[j] = p[j];
#pragma unroll
      for (int s = 0; s < 8; s++)
#pragma unroll
        for (int j = 0; j < 8; j++) v[s][j] = raw[2 * s + (j >> 2)][j & 3];
    } else {
      const u32x4_t* p = reinterpret_cast<const u32x4_t*>(reinterpret_cast<const uint16_t*>(a.q) + qoff);
      u32x4_t raw[8];
#pragma unroll
      for (int s = 0; s < 8; s++) raw[s] = p[s];
#pragma unroll
      for (int s = 0; s < 8; s++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
          if constexpr (QDT == MSPR_F16) {
            v[s][2 * j] = f16_bits_to_f32((uint16_t)(raw[s][j] & 0xFFFFu));
            v[s][2 * j + 1] = f16_bits_to_f32((uint16_t)(raw[s][j] >> 16));
          } else {
            v[s][2 * j] = bf16_bits_to_f32((uint16_t)(raw[s][j] & 0xFFFFu));
            v[s][2 * j + 1] = bf16_bits_to_f32((uint16_t)(raw[s][j] >> 16));
          }
        }
    }
#pragma unroll
    for (int s = 0; s < 8; s++) {
      u32x4_t f;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        h2_t h = {(_Float16)(live ? v[s][2 * j] * a.scale_log2 : 0.0f), (_Float16)(live ? v[s][2 * j + 1] * a.scale_log2 : 0.0f)};
        f[j] = h2_bits(h);
      }
      qf[s] = f;
    }
  }

  for (int64_t tile = wave; tile < n_tiles; tile += kQ8Waves) {
    const int64_t key0 = k0 + tile * kTileKeys;
    const int64_t next_key0 = tile + kQ8Waves < n_tiles ? key0 + kQ8Waves * kTileKeys : key0;

    // ---- S^T = K . Q^T for the two 16-key sub-tiles
    f32x4_t sacc[2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
      h2_t s0, s1, b0, b1;
      if constexpr (FMT == kFmtQ8_0) {
        s0 = h_pair(kr.s[u], 0);
        s1 = h_pair(kr.s[u], 1);
        b0 = b1 = h2_t{(_Float16)0.0f, (_Float16)0.0f};
      } else {
        s0 = s1 = sb_to_h2(kr.s[u]);
        b0 = b1 = sb_to_h2(kr.bz[u]);
      }
      f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 8; s++) {
        // bytes 8s..8s+7 of the lane's 64: two words; the first 32 bytes use the first Q8_0 scale
        const h2_t sc = s < 4 ? s0 : s1;
        const h2_t bi = s < 4 ? b0 : b1;
        u32x4_t af;
#pragma unroll
        for (int wq = 0; wq < 2; wq++) {
          h2_t lo, hi;
          codes4_to_h<FMT>(kr.c[u][s >> 1][(s & 1) * 2 + wq], lo, hi);
          if constexpr (FMT == kFmtQ8_0) {
            lo = lo * sc;
            hi = hi * sc;
          } else {
            lo = lo * sc + bi;
            hi = hi * sc + bi;
          }
          af[2 * wq] = h2_bits(lo);
          af[2 * wq + 1] = h2_bits(hi);
        }
        acc = mfma16(af, qf[s], acc);
      }
      sacc[u] = acc;
    }
    load_k(next_key0);
    __builtin_amdgcn_sched_barrier(0);

    // ---- online softmax (log2 domain); lane (n, g) holds keys 16u + 4g + i of the tile
    float tmax = -__builtin_inff();
#pragma unroll
    for (int u = 0; u < 2; u++)
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const bool valid = key0 + 16 * u + 4 * g + i < k1;
        sacc[u][i] = valid ? sacc[u][i] : -__builtin_inff();
        tmax = fmaxf(tmax, sacc[u][i]);
      }
    tmax = half_wave_max(row_pair_max(tmax));
    const bool grow = tmax > m_run + 8.0f;
    if (__any(grow)) {
      const float m_new = grow ? tmax : m_run;
      const float alpha = grow ? __builtin_amdgcn_exp2f(m_run - m_new) : 1.0f;
      l_run *= alpha;
      m_run = m_new;
#pragma unroll
      for (int mt = 0; mt < 16; mt++) oacc[mt] = oacc[mt] * alpha;
    }
    const float m_safe = m_run == -__builtin_inff() ? 0.0f : m_run;
    u32x4_t pf;
    {
      float p[8];
#pragma unroll
      for (int u = 0; u < 2; u++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          p[4 * u + i] = __builtin_amdgcn_exp2f(sacc[u][i] - m_safe);
          l_run += p[4 * u + i];
        }
#pragma unroll
      for (int j = 0; j < 4; j++) pf[j] = h2_bits(h2_t{(_Float16)p[2 * j], (_Float16)p[2 * j + 1]});
    }

    // ---- V: dequantise this wave's 32 x 256 tile into LDS (row-major float16)
    {
      h2_t sc[4], bi[4];
      if constexpr (FMT == kFmtQ8_0) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          sc[j] = h_pair(vr.s[j >> 1], j & 1);
          bi[j] = h2_t{(_Float16)0.0f, (_Float16)0.0f};
        }
      } else {
#pragma unroll
        for (int j = 0; j < 2; j++) {
          sc[2 * j] = sc[2 * j + 1] = sb_to_h2(vr.s[j]);
          bi[2 * j] = bi[2 * j + 1] = sb_to_h2(vr.bz[j]);
        }
      }
      unsigned char* dst = vt + vkey * kVPitch + 128 * vhalf * 2;
#pragma unroll
      for (int j = 0; j < 8; j++) {
        // 16 codes (elements 16j..16j+15 of the half row): scale block (16j)/32
        const h2_t s2 = sc[j >> 1], b2 = bi[j >> 1];
        u32x4_t o0, o1;
#pragma unroll
        for (int wq = 0; wq < 4; wq++) {
          h2_t lo, hi;
          codes4_to_h<FMT>(vr.c[j][wq], lo, hi);
          if constexpr (FMT == kFmtQ8_0) {
            lo = lo * s2;
            hi = hi * s2;
          } else {
            lo = lo * s2 + b2;
            hi = hi * s2 + b2;
          }
          if (wq < 2) {
            o0[2 * wq] = h2_bits(lo);
            o0[2 * wq + 1] = h2_bits(hi);
          } else {
            o1[2 * (wq - 2)] = h2_bits(lo);
            o1[2 * (wq - 2) + 1] = h2_bits(hi);
          }
        }
        *reinterpret_cast<u32x4_t*>(dst + j * 32) = o0;
        *reinterpret_cast<u32x4_t*>(dst + j * 32 + 16) = o1;
      }
    }

    load_v(next_key0);
    __builtin_amdgcn_sched_barrier(0);

    // ---- O^T += V^T . P^T (the V tile was written by this wave only: LDS operations of one wave
    //      complete in order, the wave barrier keeps the compiler from moving the reads up)
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int mt = 0; mt < 16; mt++) {
      const unsigned char* base = vt + tr_off + mt * 32;
      s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(MSPR_LDS_PTR(s16x4_t, base));
      s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(MSPR_LDS_PTR(s16x4_t, base + 16 * kVPitch));
      u32x2_t lo2 = __builtin_bit_cast(u32x2_t, lo), hi2 = __builtin_bit_cast(u32x2_t, hi);
      oacc[mt] = mfma16(u32x4_t{lo2.x, lo2.y, hi2.x, hi2.y}, pf, oacc[mt]);
    }
    __builtin_amdgcn_wave_barrier();
  }

  // ---- merge the waves through LDS (the V tiles are free now), write this range's partial
  float l_tot = l_run;
  l_tot += __shfl_xor(l_tot, 16, MSPR_WAVE);
  l_tot += __shfl_xor(l_tot, 32, MSPR_WAVE);
  __syncthreads();
  float* xo = reinterpret_cast<float*>(lds);              // [waves][16 mt][4][64 lanes]
  float* xml = xo + kQ8Waves * 16 * 4 * 64;               // [waves][16 heads][2]
#pragma unroll
  for (int mt = 0; mt < 16; mt++)
    *reinterpret_cast<f32x4_t*>(xo + ((wave * 16 + mt) * 64 + lane) * 4) = oacc[mt];
  if (g == 0) {
    xml[(wave * 16 + n) * 2] = m_run;
    xml[(wave * 16 + n) * 2 + 1] = l_tot;
  }
  __syncthreads();
  float mw[kQ8Waves], lw[kQ8Waves];
  float m_all = -__builtin_inff();
#pragma unroll
  for (int w = 0; w < kQ8Waves; w++) {
    mw[w] = xml[(w * 16 + n) * 2];
    lw[w] = xml[(w * 16 + n) * 2 + 1];
    m_all = fmaxf(m_all, mw[w]);
  }
  const float m_safe = m_all == -__builtin_inff() ? 0.0f : m_all;
  float l_all = 0.0f;
#pragma unroll
  for (int w = 0; w < kQ8Waves; w++) {
    mw[w] = __builtin_amdgcn_exp2f(mw[w] - m_safe);
    l_all += lw[w] * mw[w];
  }
  const int64_t part = (((int64_t)b * a.n_kv_heads + kvh) * a.n_splits + sp);
  float* po = a.ws_o + part * (16 * kD);
  // every wave reduces its share of the 16 M-tiles: dims 16mt + 4g + i of head n
#pragma unroll
  for (int q4 = 0; q4 < 16 / kQ8Waves; q4++) {
    const int mt = wave * (16 / kQ8Waves) + q4;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < kQ8Waves; w++) {
      f32x4_t v = *reinterpret_cast<const f32x4_t*>(xo + ((w * 16 + mt) * 64 + lane) * 4);
      acc += v * mw[w];
    }
    if (n < rep) *reinterpret_cast<f32x4_t*>(po + n * kD + 16 * mt + 4 * g) = acc;  // (columns past the real heads are padding)
  }
  if (wave == 0 && g == 0) {
    float* pml = a.ws_ml + part * 32;
    pml[n * 2] = m_all;
    pml[n * 2 + 1] = l_all;
  }
}

// Merge of the per-range partials: one workgroup per (batch, query head); 64 lanes cover the 256
// dims four at a time, the 16 waves each take every 16th range and fetch up to 16 of them in one go
// (one memory round trip for up to 256 ranges), the wave results are combined in LDS.
constexpr int kMergeWaves = 16;
template <int ODT>
__global__ __launch_bounds__(64 * kMergeWaves) void q8_decode_merge_kernel(Q8Args a) {
  __shared__ float xm[kMergeWaves], xl[kMergeWaves];
  __shared__ __attribute__((aligned(16))) float xo[kMergeWaves][kD];
  const int lane = threadIdx.x & 63;
  const int sg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int qh = blockIdx.x;
  const int b = blockIdx.y;
  const int rep = a.n_q_heads / a.n_kv_heads;
  const int kvh = qh / rep, hn = qh % rep;
  const int64_t part0 = ((int64_t)b * a.n_kv_heads + kvh) * a.n_splits;
  const float* ml = a.ws_ml + part0 * 32 + hn * 2;
  const float* po = a.ws_o + part0 * (16 * kD) + hn * kD + 4 * lane;
  constexpr int kChunk = 16;
  float m_run = -__builtin_inff(), l = 0.0f;
  f32x4_t o = {0.f, 0.f, 0.f, 0.f};
  for (int s0 = sg; s0 < a.n_splits; s0 += kMergeWaves * kChunk) {
    float mv[kChunk], lv[kChunk];
    f32x4_t ov[kChunk];
#pragma unroll
    for (int j = 0; j < kChunk; j++) {
      const int sj = s0 + kMergeWaves * j;  // wave-uniform: ranges past the end cost no load
      mv[j] = -__builtin_inff();
      lv[j] = 0.0f;
      ov[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      if (sj < a.n_splits) {
        mv[j] = ml[(int64_t)sj * 32];
        lv[j] = ml[(int64_t)sj * 32 + 1];
        ov[j] = *reinterpret_cast<const f32x4_t*>(po + (int64_t)sj * (16 * kD));
      }
    }
    float m_new = m_run;
#pragma unroll
    for (int j = 0; j < kChunk; j++) m_new = fmaxf(m_new, mv[j]);
    const float m_safe = m_new == -__builtin_inff() ? 0.0f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_safe);  // 0 while m_run is -inf
    l *= alpha;
    o = o * alpha;
#pragma unroll
    for (int j = 0; j < kChunk; j++) {
      const float w = __builtin_amdgcn_exp2f(mv[j] - m_safe);
      l += lv[j] * w;
      o += ov[j] * w;
    }
    m_run = m_new;
  }
  if (lane == 0) {
    xm[sg] = m_run;
    xl[sg] = l;
  }
  *reinterpret_cast<f32x4_t*>(&xo[sg][4 * lane]) = o;
  __syncthreads();
  if (sg != 0) return;
  float m_all = -__builtin_inff();
#pragma unroll
  for (int w = 0; w < kMergeWaves; w++) m_all = fmaxf(m_all, xm[w]);
  const float m_safe = m_all == -__builtin_inff() ? 0.0f : m_all;
  float l_all = 0.0f;
  f32x4_t o_all = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int w = 0; w < kMergeWaves; w++) {
    const float wt = __builtin_amdgcn_exp2f(xm[w] - m_safe);
    l_all += xl[w] * wt;
    o_all += *reinterpret_cast<const f32x4_t*>(&xo[w][4 * lane]) * wt;
  }
  const float inv = l_all == 0.0f ? 0.0f : 1.0f / l_all;
  const int64_t ooff = ((int64_t)b * a.n_q_heads + qh) * kD + 4 * lane;
  if constexpr (ODT == MSPR_F32) {
    *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(a.out) + ooff) = o_all * inv;
  } else {
    uint16_t h[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
      h[i] = ODT == MSPR_BF16 ? f32_to_bf16_bits(o_all[i] * inv) : f32_to_f16_bits(o_all[i] * inv);
    u32x2_t pk = {(uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16)};
    *reinterpret_cast<u32x2_t*>(reinterpret_cast<uint16_t*>(a.out) + ooff) = pk;
  }
}

// Key ranges: keys per range (whole 32-key tiles) and number of ranges. The split kernel's workgroups are
// all resident at once and the memory system serves the CUs about evenly, so the launch ends with the CU
// that holds the most tiles: a workgroup count just above the CU count (290 on 256 CUs) nearly doubles
// the time of a short launch, and two workgroups on every CU measured slower than one with twice the
// tiles (more partials, no more bandwidth). Hence at most one workgroup per CU, and never fewer than one
// tile per wave in a range.
void q8_plan(int batch, int n_kv_heads, int64_t n_keys, int64_t* keys_per_split, int* n_splits) {
  const int64_t bh = (int64_t)batch * n_kv_heads;
  const int64_t tiles = (n_keys + kTileKeys - 1) / kTileKeys;
  int64_t ranges = 256 / bh;
  if (ranges < 1) ranges = 1;
  int64_t per = (tiles + ranges - 1) / ranges;
  if (per < kQ8Waves) per = kQ8Waves;
  *keys_per_split = per * kTileKeys;
  *n_splits = (int)((tiles + per - 1) / per);
}

size_t q8_workspace_bytes(int batch, int n_kv_heads, int64_t n_keys) {
  int64_t kps;
  int splits;
  q8_plan(batch, n_kv_heads, n_keys, &kps, &splits);
  size_t parts = (size_t)batch * n_kv_heads * splits;
  return parts * (16 * kD + 32) * sizeof(float) + 256;
}

template <int FMT, int QDT, int SDT>
int q8_launch(Q8Args a, hipStream_t st) {
  constexpr int kMergeLds = (kQ8Waves * 16 * 4 * 64 + kQ8Waves * 16 * 2) * 4;
  constexpr int kLds = kQ8Waves * kVTileBytes > kMergeLds ? kQ8Waves * kVTileBytes : kMergeLds;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&q8_decode_split_kernel<FMT, QDT, SDT>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e != hipSuccess) {
      mspr_set_error("sdpa_decode_q8: cannot reserve %d bytes of LDS: %s", kLds, hipGetErrorString(e));
      return MSPR_ERR_LAUNCH;
    }
    attr_set = true;
  }
  dim3 grid((unsigned)a.n_splits, (unsigned)a.n_kv_heads, (unsigned)a.batch), block(64 * kQ8Waves);
  {
    MsprProfScope prof(MSPR_K_Q8_DECODE, st);
    q8_decode_split_kernel<FMT, QDT, SDT><<<grid, block, kLds, st>>>(a);
  }
  MSPR_CHECK_LAUNCH("sdpa_decode_q8 (split)");
  dim3 mgrid((unsigned)a.n_q_heads, (unsigned)a.batch);
  {
    MsprProfScope prof(MSPR_K_Q8_MERGE, st);
    dim3 mblock(64 * kMergeWaves);
    if (QDT == MSPR_F32) q8_decode_merge_kernel<MSPR_F32><<<mgrid, mblock, 0, st>>>(a);
    else if (QDT == MSPR_BF16) q8_decode_merge_kernel<MSPR_BF16><<<mgrid, mblock, 0, st>>>(a);
    else q8_decode_merge_kernel<MSPR_F16><<<mgrid, mblock, 0, st>>>(a);
  }
  MSPR_CHECK_LAUNCH("sdpa_decode_q8 (merge)");
  return MSPR_OK;
}

int q8_common_checks(const char* what, const void* q, const void* kc, const void* ks, const void* vc, const void* vs,
                     void* out, int batch, int n_q_heads, int n_kv_heads, int head_dim, int64_t n_keys,
                     void* workspace, size_t ws_given) {
  MSPR_REQUIRE(q && kc && ks && vc && vs && out, "%s: null pointer", what);
  MSPR_REQUIRE(batch >= 1 && n_kv_heads >= 1 && n_q_heads >= n_kv_heads && n_q_heads % n_kv_heads == 0,
               "%s: bad head counts", what);
  MSPR_REQUIRE(n_q_heads / n_kv_heads <= 16, "%s: at most 16 query heads per KV head", what);
  MSPR_REQUIRE(head_dim == kD, "%s: head_dim must be 256", what);
  MSPR_REQUIRE(n_keys >= 1 && n_keys < ((int64_t)1 << 31), "%s: n_keys out of range", what);
  MSPR_REQUIRE(mspr_aligned(q, 16) && mspr_aligned(kc, 16) && mspr_aligned(vc, 16) && mspr_aligned(out, 16),
               "%s: pointers must be 16-byte aligned", what);
  size_t need = q8_workspace_bytes(batch, n_kv_heads, n_keys);
  MSPR_REQUIRE(workspace && ws_given >= need && mspr_aligned(workspace, 16),
               "%s: workspace of %zu bytes (16-byte aligned) needed, %zu given", what, need, ws_given);
  return MSPR_OK;
}

void q8_fill_args(Q8Args& a, int batch, int n_q_heads, int n_kv_heads, int64_t n_keys, int64_t kv_rows, float scale,
                  void* workspace) {
  a.kv_rows = kv_rows;
  a.batch = batch;
  a.n_q_heads = n_q_heads;
  a.n_kv_heads = n_kv_heads;
  a.n_keys = n_keys;
  a.scale_log2 = (float)((double)scale * 1.4426950408889634);
  int64_t kps;
  q8_plan(batch, n_kv_heads, n_keys, &kps, &a.n_splits);
  a.keys_per_split = (int)kps;
  size_t parts = (size_t)batch * n_kv_heads * a.n_splits;
  a.ws_o = reinterpret_cast<float*>(workspace);
  a.ws_ml = a.ws_o + parts * (16 * kD);
}

}  // namespace

extern "C" size_t mspr_sdpa_decode_q8_workspace_bytes(int batch, int n_kv_heads, int64_t n_keys) {
  if (batch < 1 || n_kv_heads < 1 || n_keys < 1) return 0;
  return q8_workspace_bytes(batch, n_kv_heads, n_keys);
}

extern "C" int mspr_sdpa_decode_q8(const void* queries, int q_dtype, const void* k_wq, const void* k_scales,
                                   const void* k_biases, const void* v_wq, const void* v_scales,
                                   const void* v_biases, int sb_dtype, int batch, int n_q_heads, int n_kv_heads,
                                   int head_dim, int64_t n_keys, int64_t kv_rows, float scale, int group_size,
                                   int bits, void* out, void* workspace, size_t workspace_bytes, void* stream) {
  MSPR_REQUIRE(group_size == 64 && bits == 8, "sdpa_decode_q8: only group_size=64, bits=8 is supported");
  MSPR_REQUIRE(kv_rows >= n_keys, "sdpa_decode_q8: kv_rows (rows allocated per head) must cover n_keys");
  MSPR_REQUIRE(q_dtype == MSPR_F32, "sdpa_decode_q8: queries must be float32");
  MSPR_REQUIRE(sb_dtype >= MSPR_F32 && sb_dtype <= MSPR_BF16, "sdpa_decode_q8: scales/biases must be f32, f16 or bf16");
  MSPR_REQUIRE(k_biases && v_biases, "sdpa_decode_q8: null pointer");
  int rc = q8_common_checks("sdpa_decode_q8", queries, k_wq, k_scales, v_wq, v_scales, out, batch, n_q_heads,
                            n_kv_heads, head_dim, n_keys, workspace, workspace_bytes);
  if (rc != MSPR_OK) return rc;
  Q8Args a = {};
  a.q = queries;
  a.k_codes = k_wq;
  a.k_scales = k_scales;
  a.k_biases = k_biases;
  a.v_codes = v_wq;
  a.v_scales = v_scales;
  a.v_biases = v_biases;
  a.out = out;
  q8_fill_args(a, batch, n_q_heads, n_kv_heads, n_keys, kv_rows, scale, workspace);
  hipStream_t st = (hipStream_t)stream;
  if (sb_dtype == MSPR_F32) return q8_launch<kFmtAffine, MSPR_F32, MSPR_F32>(a, st);
  if (sb_dtype == MSPR_F16) return q8_launch<kFmtAffine, MSPR_F32, MSPR_F16>(a, st);
  return q8_launch<kFmtAffine, MSPR_F32, MSPR_BF16>(a, st);
}

extern "C" int mspr_sdpa_decode_q8_0(const void* queries, int q_dtype, const void* k_codes, const void* k_scales,
                                     const void* v_codes, const void* v_scales, int batch, int n_q_heads,
                                     int n_kv_heads, int head_dim, int64_t n_keys, int64_t kv_rows, float scale,
                                     void* out, void* workspace, size_t workspace_bytes, void* stream) {
  MSPR_REQUIRE(kv_rows >= n_keys, "sdpa_decode_q8_0: kv_rows (rows allocated per head) must cover n_keys");
  MSPR_REQUIRE(q_dtype >= MSPR_F32 && q_dtype <= MSPR_BF16, "sdpa_decode_q8_0: queries must be f32, f16 or bf16");
  int rc = q8_common_checks("sdpa_decode_q8_0", queries, k_codes, k_scales, v_codes, v_scales, out, batch, n_q_heads,
                            n_kv_heads, head_dim, n_keys, workspace, workspace_bytes);
  if (rc != MSPR_OK) return rc;
  Q8Args a = {};
  a.q = queries;
  a.k_codes = k_codes;
  a.k_scales = k_scales;
  a.v_codes = v_codes;
  a.v_scales = v_scales;
  a.out = out;
  q8_fill_args(a, batch, n_q_heads, n_kv_heads, n_keys, kv_rows, scale, workspace);
  hipStream_t st = (hipStream_t)stream;
  if (q_dtype == MSPR_F32) return q8_launch<kFmtQ8_0, MSPR_F32, MSPR_F16>(a, st);
  if (q_dtype == MSPR_F16) return q8_launch<kFmtQ8_0, MSPR_F16, MSPR_F16>(a, st);
  return q8_launch<kFmtQ8_0, MSPR_BF16, MSPR_F16>(a, st);
}
