// Causal chunked-prefill GQA attention, head dim 256: a chunk of q_len new tokens attends to the
// past_len tokens already in the KV cache and, causally, to itself.
//
// Workgroup = 8 waves on one KV head, 32 query rows per wave: two groups of four waves (four query
// heads, or fewer heads times adjacent 32-row blocks), one group on a late block of the chunk and the
// other on the mirrored early block, so one K/V tile staged in LDS feeds eight waves and every
// workgroup carries the same matrix work under the causal mask.
// K/V tiles of 32 keys stream through a 4-slot LDS ring with asynchronous global->LDS copies; the
// 16-byte pieces of a row are XOR-swizzled on the way in (the copy writes LDS linearly, the global
// address of each lane is free), which makes both the K operand reads (ds_read_b128, lane = key) and
// the V^T operand reads (LDS transpose read) bank-conflict free without padding.
//
// Per wave and tile: S^T = K.Q^T on v_mfma_f32_32x32x16 (keys x queries: the softmax statistics of a
// query live in one lane column), online softmax in the log2 domain with a lazily advanced reference
// maximum, O^T += V^T.P^T. Q^T stays in registers (64 VGPRs), O^T in 128 accumulator registers.
#include "common.h"
#include "profile.h"

namespace {

constexpr int kD = 256;
constexpr int kRowBytes = kD * 2;
constexpr int kTile = 32;                       // keys per tile
constexpr int kTileBytes = kTile * kRowBytes;   // 16 KB, K and V each
constexpr int kStageBytes = 2 * kTileBytes;
constexpr int kBufs = 4;
constexpr int kThreads = 512;
constexpr int kLdsBytes = kBufs * kStageBytes;  // 128 KB

struct PrefillArgs {
  const void* q;   // [B, Hq, L, 256]
  const void* k;   // [B, Hkv, kv_rows, 256]
  const void* v;
  void* out;       // [B, Hq, L, 256]
  int batch, n_q_heads, n_kv_heads;
  int q_len;
  int64_t past_len;
  int64_t kv_rows;  // rows allocated per (batch, kv head); >= past_len + q_len
  float scale_log2;
  int rep_shift;    // log2(query heads per KV head), 0..3
  int q_blocks;     // workgroups along the query axis
  // key-range splits (short chunks over deep prefixes do not fill the device otherwise): split sp of a
  // query block takes every n_splits-th share of that block's tiles; partials are merged afterwards
  int n_splits;
  float* ws_o;      // [n_splits][B][Hq][L][256] unnormalised O relative to ws_ml's maximum
  float* ws_ml;     // [n_splits][B][Hq][L][2]   (reference maximum in log2 units, denominator)
  // quantised-prefix form only: tiles [0, q8_tiles) come from the affine 8-bit prefix below, the rest
  // from k / v, which then hold float16 rows for keys [32 q8_tiles, past_len + q_len)
  int q8_tiles;
  int64_t past_rows;  // rows allocated per (batch, kv head) in the prefix tensors; >= past_len
  const void* pk_wq;  // [B, Hkv, past_rows, 256] codes
  const void* pk_s;   // [B, Hkv, past_rows, 4]
  const void* pk_b;
  const void* pv_wq;
  const void* pv_s;
  const void* pv_b;
};

typedef __attribute__((ext_vector_type(2))) _Float16 h2_t;
__device__ __forceinline__ uint32_t h2_bits(h2_t v) { return __builtin_bit_cast(uint32_t, v); }
__device__ __forceinline__ h2_t bits_h2(uint32_t v) { return __builtin_bit_cast(h2_t, v); }
// raw affine scale / bias bits to a packed float16 pair
template <int SDT>
__device__ __forceinline__ h2_t sb_to_h2(uint32_t bits) {
  _Float16 h;
  if constexpr (SDT == MSPR_F32) h = (_Float16)__builtin_bit_cast(float, bits);
  else if constexpr (SDT == MSPR_F16) h = __builtin_bit_cast(_Float16, (uint16_t)bits);
  else h = (_Float16)__builtin_bit_cast(float, bits << 16);
  return h2_t{h, h};
}
// 16 unsigned 8-bit codes -> 16 float16 values code * scale + bias (two 16-byte pieces)
__device__ __forceinline__ void dequant16(u32x4_t c, h2_t sc, h2_t bi, u32x4_t& p0, u32x4_t& p1) {
  const h2_t k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
#pragma unroll
  for (int w = 0; w < 4; w++) {
    // byte b becomes the float16 with bits 0x6400 | b = 1024 + b, exactly
    h2_t lo = (bits_h2(__builtin_amdgcn_perm(0x64646464u, c[w], 0x04010400u)) - k1024) * sc + bi;
    h2_t hi = (bits_h2(__builtin_amdgcn_perm(0x64646464u, c[w], 0x04030402u)) - k1024) * sc + bi;
    if (w < 2) {
      p0[2 * w] = h2_bits(lo);
      p0[2 * w + 1] = h2_bits(hi);
    } else {
      p1[2 * (w - 2)] = h2_bits(lo);
      p1[2 * (w - 2) + 1] = h2_bits(hi);
    }
  }
}

template <int KDT>
__device__ __forceinline__ f32x16_t mfma32(u32x4_t a, u32x4_t b, f32x16_t c) {
  if constexpr (KDT == MSPR_BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                   c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c,
                                                  0, 0, 0);
  }
}

template <int KDT>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  if constexpr (KDT == MSPR_BF16) {
    typedef __attribute__((ext_vector_type(2))) __bf16 bf2_t;
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{a, b}, bf2_t));
  } else {
    typedef __attribute__((ext_vector_type(2))) _Float16 h2_t;
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{a, b}, h2_t));
  }
}

template <int N>
__device__ __forceinline__ void wait_vm_and_barrier() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}
// lane i's 16 bytes at `src` land at lds_base + 16 i (lds_base wave-uniform); issued through asm so
// that the compiler's wait-count pass does not drain it in front of LDS transpose reads
__device__ __forceinline__ void async_load_16(uint64_t base, uint32_t offset, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %1, %0" ::"s"(base), "v"(offset), "s"(lds_base)
               : "memory", "m0");
}

// the same with 4 bytes per lane: lane i's dword lands at lds_base + 4 i
__device__ __forceinline__ void async_load_4(uint64_t base, uint32_t offset, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %1, %0" ::"s"(base), "v"(offset), "s"(lds_base)
               : "memory", "m0");
}

// LDS byte address of a pointer into the kernel's dynamic LDS
__device__ __forceinline__ uint32_t lds_addr(const unsigned char* p) {
  return (uint32_t)(uintptr_t)MSPR_LDS_PTR(const unsigned char, p);
}

// swizzle of the 16-byte pieces of a tile row: piece p of row r sits at slot (p & 16) | ((p ^ f(r)) & 15)
__device__ __forceinline__ int swz(int r) { return ((r & 7) << 1) | ((r >> 3) & 1); }

// Q8 = false: k / v are the whole 16-bit cache, q / out have its element type.
// Q8 = true (KDT float16): float32 q / out, quantised prefix + float16 tail rows (see PrefillArgs).
template <int KDT, bool Q8, int SDT, bool IO32 = Q8>
__global__ __launch_bounds__(kThreads, 1) void flash_prefill_kernel(PrefillArgs a) {
  extern __shared__ __attribute__((aligned(256))) unsigned char lds[];  // tile bases: zero low bits under the address XORs
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31;  // MFMA column: query row of the wave's block; MFMA row (key) for the K operand
  const int g = lane >> 5;

  // ---- workgroup -> (batch, kv head, pair of query row ranges, half of the heads when eight share a KV head).
  // Waves 0-3 take 32-row blocks from the late end of the chunk (most keys), waves 4-7 the mirrored blocks from
  // the early end, so every workgroup carries the same matrix work although the causal key count grows with the
  // query position; the tile stream runs to the late block's last key and the early waves leave it when their
  // last key has passed. Four heads per group; with fewer heads per KV head a group takes 2 or 4 adjacent blocks.
  const int rep = 1 << a.rep_shift;
  const int hpg_shift = a.rep_shift < 2 ? a.rep_shift : 2;  // log2(heads per group)
  const int blocks_per_group = 4 >> hpg_shift;
  const int head_halves = 1 << (a.rep_shift - hpg_shift);
  const int n_blocks = (a.q_len + 31) / 32;
  const int n_pairs = a.q_blocks / head_halves;
  int work = blockIdx.x;
  const int sp = work % a.n_splits;
  work /= a.n_splits;
  const int pair = (work % a.q_blocks) / head_halves;  // pair 0 (longest stream) first
  const int head_half = work % head_halves;
  work /= a.q_blocks;
  const int kvh = work % a.n_kv_heads;
  const int b = work / a.n_kv_heads;
  const int wi = wave & 3;
  const int head = kvh * rep + (head_half << hpg_shift) + (wi & ((1 << hpg_shift) - 1));
  // late group: blocks [n_blocks - bpg (pair + 1), n_blocks - bpg pair); early group: blocks [bpg pair, bpg (pair + 1))
  // as far as they lie below the late groups' range [n_blocks - bpg n_pairs, n_blocks)
  const int blk = wave < 4 ? n_blocks - blocks_per_group * (pair + 1) + (wi >> hpg_shift)
                           : blocks_per_group * pair + (wi >> hpg_shift);
  const bool active = wave < 4 ? blk >= 0 : blk < n_blocks - blocks_per_group * n_pairs;  // wave-uniform
  const int q0 = active ? 32 * blk : 0;  // first query row of this wave
  const int past = (int)a.past_len;

  const unsigned char* kbase =
      reinterpret_cast<const unsigned char*>(a.k) + ((int64_t)b * a.n_kv_heads + kvh) * a.kv_rows * kRowBytes;
  const unsigned char* vbase =
      reinterpret_cast<const unsigned char*>(a.v) + ((int64_t)b * a.n_kv_heads + kvh) * a.kv_rows * kRowBytes;

  // keys needed by the workgroup: [0, past + last query row]
  int q_last = 32 * (n_blocks - blocks_per_group * pair) - 1;  // last row of the late group
  if (q_last > a.q_len - 1) q_last = a.q_len - 1;
  const int all_tiles = (int)((past + q_last) / kTile) + 1;
  // this workgroup's share of the block's tiles: [t_begin, n_tiles)
  const int tiles_per_split = (all_tiles + a.n_splits - 1) / a.n_splits;
  const int t_begin = sp * tiles_per_split < all_tiles ? sp * tiles_per_split : all_tiles;
  const int n_tiles = t_begin + tiles_per_split < all_tiles ? t_begin + tiles_per_split : all_tiles;

  // ---- asynchronous tile copies: thread handles LDS slots tid and tid + 512 of the K and of the V tile;
  //      addresses are a scalar tile base plus a per-thread 32-bit offset
  const int c_row = tid >> 5;                                  // tile row of slot `tid` (slot tid+512: row + 16)
  const int c_piece = (tid & 16) | ((tid ^ swz(c_row)) & 15);  // global 16-byte piece that lands in the slot
  const uint32_t lds0 = (uint32_t)(uintptr_t)MSPR_LDS_PTR(unsigned char, lds);
  const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(lds0) + wave * 1024;
  const int n_keys = (int)(past + a.q_len);  // keys that exist
  const int t1 = Q8 ? a.q8_tiles : 0;        // first tile served from k / v; their row 0 is key 32 t1
  auto issue_tile = [&](int t_abs, int slot) {
    // rows past the last key (only in the last tile) are masked by the causal rule; read the last key instead
    const int t = t_abs - t1;
    const int last = n_keys - 1 - t_abs * kTile;
    const uint32_t o0 = (uint32_t)((c_row < last ? c_row : last) * kRowBytes + c_piece * 16);
    const uint32_t o1 = (uint32_t)((c_row + 16 < last ? c_row + 16 : last) * kRowBytes + c_piece * 16);
    const uint64_t kt = (uint64_t)(kbase + (int64_t)t * kTileBytes);
    const uint64_t vt = (uint64_t)(vbase + (int64_t)t * kTileBytes);
    const uint32_t dst = lds_wave + slot * kStageBytes;
    async_load_16(kt, o0, dst);
    async_load_16(kt, o1, dst + 8192);
    async_load_16(vt, o0, dst + kTileBytes);
    async_load_16(vt, o1, dst + kTileBytes + 8192);
  };

  // ---- Q^T operand: lane (n, g) holds q[q0 + n][16 s + 8 g .. +7] for k-step s
  u32x4_t qf[16];
  {
    int qrow = q0 + n;
    if (qrow > a.q_len - 1) qrow = a.q_len - 1;
    if (qrow < 0) qrow = 0;
    const int64_t qoff = (((int64_t)b * a.n_q_heads + head) * a.q_len + qrow) * kD + 8 * g;
    if constexpr (!IO32) {
      const u32x4_t* qp = reinterpret_cast<const u32x4_t*>(reinterpret_cast<const uint16_t*>(a.q) + qoff);
#pragma unroll
      for (int s = 0; s < 16; s++) qf[s] = qp[2 * s];
    } else {
      const f32x4_t* qp = reinterpret_cast<const f32x4_t*>(reinterpret_cast<const float*>(a.q) + qoff);
#pragma unroll
      for (int s0 = 0; s0 < 16; s0 += 4) {
        f32x4_t raw[8];
#pragma unroll
        for (int j = 0; j < 4; j++) {
          raw[2 * j] = qp[4 * (s0 + j)];
          raw[2 * j + 1] = qp[4 * (s0 + j) + 1];
        }
#pragma unroll
        for (int j = 0; j < 4; j++)
          qf[s0 + j] = u32x4_t{pack2<KDT>(raw[2 * j][0], raw[2 * j][1]), pack2<KDT>(raw[2 * j][2], raw[2 * j][3]),
                               pack2<KDT>(raw[2 * j + 1][0], raw[2 * j + 1][1]),
                               pack2<KDT>(raw[2 * j + 1][2], raw[2 * j + 1][3])};
      }
    }
#pragma unroll
    for (int s = 0; s < 16; s++) asm volatile("" : "+v"(qf[s]));  // complete before the first asynchronous copy
  }

  f32x16_t oacc[8];
#pragma unroll
  for (int mt = 0; mt < 8; mt++) oacc[mt] = f32x16_t{0};
  float m_run = -__builtin_inff();
  float l_run = 0.0f;

  // per-lane LDS offsets inside a tile (the k-step / M-tile index enters by XOR, see swz)
  const int k_off = n * kRowBytes + 32 * (n & 7) + 16 * (g ^ ((n >> 3) & 1));
  const int tr_s = lane & 15;
  const int tr_row = 4 * g + (tr_s >> 2);            // + 8 h + 16 ks
  const int tr_piece = 2 * ((lane >> 4) & 1) + ((tr_s & 3) >> 1);  // 16-byte piece inside the 64-byte M-tile row
  int v_off[2];
#pragma unroll
  for (int h = 0; h < 2; h++) {
    const int r = tr_row + 8 * h;
    v_off[h] = kTileBytes + r * kRowBytes + 16 * ((tr_piece ^ swz(r)) & 15) + 8 * (tr_s & 1);
  }
  const int my_last_key = active ? past + q0 + 31 : -1;  // last key any query of this wave may see
  const int qpos_g = past + q0 + n - 4 * g;  // the lane's query position minus its key offset inside a tile

  // stage 1 of a tile: S^T = K . Q^T on the matrix cores
  auto qk_tile = [&](const unsigned char* st, f32x16_t& sacc) {
    // S^T = K . Q^T
    sacc = f32x16_t{0};
    {
      // all sixteen K operand reads are written out up front; the scheduling directives below make
      // the compiler keep kAhead of them in flight in front of the dependent MFMA chain instead of
      // waiting for each read right before its MFMA
#ifndef MSPR_FP_AHEAD_K
#define MSPR_FP_AHEAD_K 4
#endif
      constexpr int kAhead = MSPR_FP_AHEAD_K;
      // (the k-step enters the address by XOR on top of the tile base: formed per tile, the eight variants
      // are not carried in registers across the loop)
      const uint32_t kb = lds_addr(st) + (uint32_t)k_off;
      u32x4_t af[16];
#pragma unroll
      for (int s2 = 0; s2 < 16; s2++)
        af[s2] = *MSPR_LDS_PTR(const u32x4_t, (uintptr_t)((kb ^ (uint32_t)((s2 & 7) << 5)) + (uint32_t)((s2 >> 3) * 256)));
#pragma unroll
      for (int s2 = 0; s2 < 16; s2++) sacc = mfma32<KDT>(af[s2], qf[s2], sacc);
      __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);  // DS reads
#pragma unroll
      for (int s2 = 0; s2 < 16 - kAhead; s2++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 0);
    }
  };
  // stage 2 of a tile: online softmax on the vector units, then O^T += V^T . P^T on the matrix cores
  auto softmax_pv_tile = [&](const unsigned char* st, int key0, f32x16_t& sacc) {
    // online softmax (log2 domain); register i is key key0 + 8 (i/4) + 4 g + i%4
    // The maximum is tracked on the raw scores and the softmax scale (> 0) goes into the exponent's
    // fused multiply-add, so a score costs one max, one fma and one exp2.
    float tmax = -__builtin_inff();
    if (key0 + kTile - 1 <= past + q0) {  // wave-uniform: no query of the wave masks any key of the tile
#pragma unroll
      for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, sacc[i]);
    } else {
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const bool valid = key0 + 8 * (i / 4) + (i % 4) <= qpos_g;
        sacc[i] = valid ? sacc[i] : -__builtin_inff();
        tmax = fmaxf(tmax, sacc[i]);
      }
    }
    tmax = half_wave_max(tmax) * a.scale_log2;
    constexpr float kGrow = KDT == MSPR_BF16 ? 64.0f : 8.0f;
    const bool grow = tmax > m_run + kGrow;
    if (__any(grow)) {
      const float m_new = grow ? tmax : m_run;
      const float alpha = grow ? __builtin_amdgcn_exp2f(m_run - m_new) : 1.0f;
      l_run *= alpha;
      m_run = m_new;
#pragma unroll
      for (int mt = 0; mt < 8; mt++) oacc[mt] = oacc[mt] * alpha;
    }
    const float neg_m = m_run == -__builtin_inff() ? 0.0f : -m_run;
    float psum = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      sacc[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[i], a.scale_log2, neg_m));
      psum += sacc[i];
    }
    l_run += psum;
    u32x4_t pf[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
      pf[ks] = u32x4_t{pack2<KDT>(sacc[8 * ks], sacc[8 * ks + 1]), pack2<KDT>(sacc[8 * ks + 2], sacc[8 * ks + 3]),
                       pack2<KDT>(sacc[8 * ks + 4], sacc[8 * ks + 5]), pack2<KDT>(sacc[8 * ks + 6], sacc[8 * ks + 7])};

    // O^T += V^T . P^T; the transpose reads run kAheadV MFMAs in front of their use
    {
#ifndef MSPR_FP_AHEAD_V
#define MSPR_FP_AHEAD_V 4
#endif
      constexpr int kAheadV = MSPR_FP_AHEAD_V;
      const uint32_t vb0 = lds_addr(st) + (uint32_t)v_off[0], vb1 = lds_addr(st) + (uint32_t)v_off[1];
      u32x4_t vf[16];
#pragma unroll
      for (int mt = 0; mt < 8; mt++) {
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
          const uint32_t lo_a = (vb0 ^ (uint32_t)((mt & 3) << 6)) + (uint32_t)((mt >> 2) * 256 + ks * 16 * kRowBytes);
          const uint32_t hi_a = (vb1 ^ (uint32_t)((mt & 3) << 6)) + (uint32_t)((mt >> 2) * 256 + ks * 16 * kRowBytes);
          s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(MSPR_LDS_PTR(s16x4_t, (uintptr_t)lo_a));
          s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(MSPR_LDS_PTR(s16x4_t, (uintptr_t)hi_a));
          u32x2_t lo2 = __builtin_bit_cast(u32x2_t, lo), hi2 = __builtin_bit_cast(u32x2_t, hi);
          vf[2 * mt + ks] = u32x4_t{lo2.x, lo2.y, hi2.x, hi2.y};
        }
      }
#pragma unroll
      for (int mt = 0; mt < 8; mt++)
#pragma unroll
        for (int ks = 0; ks < 2; ks++) oacc[mt] = mfma32<KDT>(vf[2 * mt + ks], pf[ks], oacc[mt]);
      __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAheadV, 0);
#pragma unroll
      for (int i = 0; i < 16 - kAheadV; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, kAheadV, 0);
    }
  };
  auto compute_tile = [&](const unsigned char* st, int key0) {
    f32x16_t sacc;
    qk_tile(st, sacc);
    softmax_pv_tile(st, key0, sacc);
  };

  if constexpr (Q8) {
    // ---- quantised prefix. The raw bytes of a tile (8 KB of K codes, 8 KB of V codes, scales and biases)
    //      are copied asynchronously into a three-slot ring in the upper half of the LDS, three tiles ahead;
    //      tile t+1 is unpacked from there into the other float16 stage at the top of step t. No register
    //      carries raw bytes across a step (twelve more live registers did not fit next to the accumulators,
    //      and a spill of a freshly loaded value waits for the whole memory latency once per tile).
    const int p_end = n_tiles < t1 ? n_tiles : t1;  // prefix tiles of this workgroup: [t_begin, p_end)
    if (t_begin < p_end) {
      constexpr int kSB = SDT == MSPR_F32 ? 4 : 2;   // bytes per scale / bias
      constexpr int kCodeBytes = kTile * kD;         // 8 KB of codes per tile, K and V each
      constexpr int kScaleBytes = kTile * 4 * kSB;   // one tile of one scale or bias array: 256 or 512 B
      constexpr int kRawBytes = 2 * kCodeBytes + 4 * 512;
      constexpr int kRawBase = 2 * kStageBytes;      // the unpacked stages use the lower 64 KB
      static_assert(kRawBase + 3 * kRawBytes <= kLdsBytes, "raw ring does not fit");
      const int64_t row0 = ((int64_t)b * a.n_kv_heads + kvh) * a.past_rows;
      const uint8_t* kc = reinterpret_cast<const uint8_t*>(a.pk_wq) + row0 * kD;
      const uint8_t* vc = reinterpret_cast<const uint8_t*>(a.pv_wq) + row0 * kD;
      // scale / bias copies: wave w moves array w & 3 (K scale, K bias, V scale, V bias), 4 bytes per lane; with
      // float32 scales waves 4-7 move the second 256 bytes, with 16-bit ones they repeat the copy of waves 0-3
      // (every wave then issues the same number of copies and the waits below are static counts)
      const int arr = wave & 3;
      const uint8_t* sb_base = reinterpret_cast<const uint8_t*>(arr == 0 ? a.pk_s : arr == 1 ? a.pk_b : arr == 2 ? a.pv_s : a.pv_b) +
                               row0 * 4 * kSB;
      const int sb_half = kSB == 4 ? (wave >> 2) * 256 : 0;
      const uint32_t code_off = (uint32_t)tid * 16;  // K / V codes: LDS slot tid of the tile's 512
      const uint32_t sb_off = (uint32_t)(sb_half + lane * 4);
      auto issue_raw = [&](int t, int rslot) {
        if (t > p_end - 1) t = p_end - 1;  // past the end: a harmless re-read, so that the counts stay static
        const uint32_t dst = __builtin_amdgcn_readfirstlane(lds0) + kRawBase + rslot * kRawBytes;
        async_load_16((uint64_t)(kc + (int64_t)t * kCodeBytes), code_off, dst + wave * 1024);
        async_load_16((uint64_t)(vc + (int64_t)t * kCodeBytes), code_off, dst + kCodeBytes + wave * 1024);
        async_load_4((uint64_t)(sb_base + (int64_t)t * kScaleBytes), sb_off, dst + 2 * kCodeBytes + arr * 512 + sb_half);
      };
      auto unpack = [&](int rslot, int slot) {
        // (the per-thread offsets are re-derived from the thread index at each use, which the empty asm
        // enforces: carried across the loop they end up in scratch, and a reload waits behind the copies)
        int tl = tid;
        asm volatile("" : "+v"(tl));
        const int row = tl >> 4, pp = tl & 15;  // tile row and its 16 elements [16 pp, +16), scale group pp / 4
        const unsigned char* raw = lds + kRawBase + rslot * kRawBytes;
        const u32x4_t rk = *reinterpret_cast<const u32x4_t*>(raw + tl * 16);
        const u32x4_t rv = *reinterpret_cast<const u32x4_t*>(raw + kCodeBytes + tl * 16);
        uint32_t rs[4];
        const unsigned char* sp = raw + 2 * kCodeBytes + (row * 4 + (pp >> 2)) * kSB;
#pragma unroll
        for (int i = 0; i < 4; i++) {
          if constexpr (SDT == MSPR_F32) rs[i] = *reinterpret_cast<const uint32_t*>(sp + i * 512);
          else rs[i] = *reinterpret_cast<const uint16_t*>(sp + i * 512);
        }
        const int f = swz(row);
        const int w_off0 = row * kRowBytes + 16 * (((2 * pp) & 16) | (((2 * pp) ^ f) & 15));
        const int w_off1 = row * kRowBytes + 16 * (((2 * pp + 1) & 16) | (((2 * pp + 1) ^ f) & 15));
        unsigned char* st = lds + slot * kStageBytes;
        u32x4_t p0, p1;
        dequant16(rk, sb_to_h2<SDT>(rs[0]), sb_to_h2<SDT>(rs[1]), p0, p1);
        *reinterpret_cast<u32x4_t*>(st + w_off0) = p0;
        *reinterpret_cast<u32x4_t*>(st + w_off1) = p1;
        dequant16(rv, sb_to_h2<SDT>(rs[2]), sb_to_h2<SDT>(rs[3]), p0, p1);
        *reinterpret_cast<u32x4_t*>(st + kTileBytes + w_off0) = p0;
        *reinterpret_cast<u32x4_t*>(st + kTileBytes + w_off1) = p1;
      };
      issue_raw(t_begin, 0);
      issue_raw(t_begin + 1, 1);
      issue_raw(t_begin + 2, 2);
      wait_vm_and_barrier<6>();  // the raw bytes of the first tile are in LDS
      unpack(0, 0);
      for (int t = t_begin; t < p_end; t++) {
        const int i = t - t_begin;
        // this wave's copies of raw tile t+1 are done (those of t+2 may be in flight); after the barrier
        // every wave's are, stage i & 1 holds tile t, and stage (i + 1) & 1 and raw slot i % 3 are free
        wait_vm_and_barrier<3>();
        issue_raw(t + 3, i % 3);
        if (t + 1 < p_end) unpack((i + 1) % 3, (i + 1) & 1);
        if (t * kTile <= my_last_key) compute_tile(lds + (i & 1) * kStageBytes, t * kTile);
      }
      // every wave has left the last prefix tile and the trailing raw copies have landed before the ring
      // below reuses the LDS
      wait_vm_and_barrier<0>();
    }
  }

  // ---- dense tiles through the asynchronous ring: every wave issues its share of every tile
  //      (clamped past the end), so the waits are static counts. Every wave runs both stages of tile t in
  //      iteration t. (Running the two waves of a SIMD half a tile apart, one of them with stage 2 of tile
  //      t-1 in front of stage 1 of tile t, paid while the tile loop still reloaded spilled registers; without
  //      those reloads it measured 1.7 % slower than this order, and both waves deferred 5 % slower.)
#ifndef MSPR_FP_TILES_AHEAD
#define MSPR_FP_TILES_AHEAD 2
#endif
  constexpr int kTilesAhead = MSPR_FP_TILES_AHEAD;  // tiles in flight behind the one being consumed (at most kBufs - 1)
  static_assert(kTilesAhead >= 1 && kTilesAhead <= kBufs - 1, "ring too small");
  const int r0 = t_begin > t1 ? t_begin : t1;  // first tile of this workgroup that is served from k / v
  if (r0 < n_tiles) {
#pragma unroll
    for (int j = 0; j < kTilesAhead; j++) issue_tile(r0 + j < n_tiles ? r0 + j : n_tiles - 1, j);
    for (int t = r0; t < n_tiles; t++) {
      // tile t has landed once this wave's copies of it are done (those of the newer tiles may be in flight:
      // four per tile) and every wave got here; the ring slot of tile t-1 is free after the barrier
      wait_vm_and_barrier<4 * (kTilesAhead - 1)>();
      issue_tile(t + kTilesAhead < n_tiles ? t + kTilesAhead : n_tiles - 1,
                 (t - r0 + kTilesAhead) % kBufs);  // past the end: a harmless re-read
      const int key0 = t * kTile;
      if (key0 > my_last_key) continue;  // wave-uniform: this wave's queries see none of the tile
      compute_tile(lds + ((t - r0) % kBufs) * kStageBytes, key0);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the clamped trailing copies must not outlive the workgroup's LDS

  // ---- normalise and store: lane (n, g) holds dims 32 mt + 8 (i/4) + 4 g + i%4 of query row q0 + n
  const float l_tot = l_run + __shfl_xor(l_run, 32, MSPR_WAVE);
  if (a.n_splits > 1) {
    if (active && q0 + n < a.q_len) {
      const int64_t row = (((int64_t)sp * a.batch + b) * a.n_q_heads + head) * a.q_len + q0 + n;
      float* po = a.ws_o + row * kD;
#pragma unroll
      for (int mt = 0; mt < 8; mt++)
#pragma unroll
        for (int c = 0; c < 4; c++)
          *reinterpret_cast<f32x4_t*>(po + 32 * mt + 8 * c + 4 * g) =
              f32x4_t{oacc[mt][4 * c], oacc[mt][4 * c + 1], oacc[mt][4 * c + 2], oacc[mt][4 * c + 3]};
      if (g == 0) {
        a.ws_ml[row * 2] = m_run;
        a.ws_ml[row * 2 + 1] = l_tot;
      }
    }
    return;
  }
  const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
  if (active && q0 + n < a.q_len) {
    const int64_t ooff = (((int64_t)b * a.n_q_heads + head) * a.q_len + q0 + n) * kD;
#pragma unroll
    for (int mt = 0; mt < 8; mt++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        if constexpr (IO32) {
          *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(a.out) + ooff + 32 * mt + 8 * c + 4 * g) =
              f32x4_t{oacc[mt][4 * c] * inv, oacc[mt][4 * c + 1] * inv, oacc[mt][4 * c + 2] * inv,
                      oacc[mt][4 * c + 3] * inv};
        } else {
          u32x2_t w = {pack2<KDT>(oacc[mt][4 * c] * inv, oacc[mt][4 * c + 1] * inv),
                       pack2<KDT>(oacc[mt][4 * c + 2] * inv, oacc[mt][4 * c + 3] * inv)};
          *reinterpret_cast<u32x2_t*>(reinterpret_cast<uint16_t*>(a.out) + ooff + 32 * mt + 8 * c + 4 * g) = w;
        }
      }
  }
}

// Float16 tail rows of the quantised-prefix form: key 32 q8_tiles + j for j in [0, tail_rows), the
// last (past_len % 32) prefix rows dequantised, then the chunk's own rows converted.
template <int SDT, int ODT>
__global__ __launch_bounds__(256) void prefill_q8_tail_kernel(PrefillArgs a, const void* self_k, const void* self_v,
                                                              int self_dtype, uint16_t* tail_k, uint16_t* tail_v,
                                                              int tail_rows, int first_row) {
  const int d = threadIdx.x;
  const int j = first_row + blockIdx.x;
  const int kvh = blockIdx.y;
  const int b = blockIdx.z;
  const int64_t bh = (int64_t)b * a.n_kv_heads + kvh;
  const int64_t key = (int64_t)a.q8_tiles * kTile + j;
  float kx, vx;
  if (key < a.past_len) {
    const int64_t row = bh * a.past_rows + key;
    const float ks = load_as_f32<SDT>(a.pk_s, row * 4 + d / 64), kb = load_as_f32<SDT>(a.pk_b, row * 4 + d / 64);
    const float vs = load_as_f32<SDT>(a.pv_s, row * 4 + d / 64), vb = load_as_f32<SDT>(a.pv_b, row * 4 + d / 64);
    kx = (float)reinterpret_cast<const uint8_t*>(a.pk_wq)[row * kD + d] * ks + kb;
    vx = (float)reinterpret_cast<const uint8_t*>(a.pv_wq)[row * kD + d] * vs + vb;
  } else {
    const int64_t off = (bh * a.q_len + (key - a.past_len)) * kD + d;
    if (self_dtype == MSPR_F32) {
      kx = load_as_f32<MSPR_F32>(self_k, off);
      vx = load_as_f32<MSPR_F32>(self_v, off);
    } else if (self_dtype == MSPR_F16) {
      kx = load_as_f32<MSPR_F16>(self_k, off);
      vx = load_as_f32<MSPR_F16>(self_v, off);
    } else {
      kx = load_as_f32<MSPR_BF16>(self_k, off);
      vx = load_as_f32<MSPR_BF16>(self_v, off);
    }
  }
  // 16-bit staging: values beyond the range of the staging type saturate instead of becoming infinite (an
  // infinite key or value turns the whole output row into NaN)
  if constexpr (ODT == MSPR_F16) {
    kx = __builtin_amdgcn_fmed3f(kx, -65504.0f, 65504.0f);
    vx = __builtin_amdgcn_fmed3f(vx, -65504.0f, 65504.0f);
    tail_k[(bh * tail_rows + j) * kD + d] = f32_to_f16_bits(kx);
    tail_v[(bh * tail_rows + j) * kD + d] = f32_to_f16_bits(vx);
  } else {
    constexpr float kBf16Max = 0x1.fep127f;
    kx = __builtin_amdgcn_fmed3f(kx, -kBf16Max, kBf16Max);
    vx = __builtin_amdgcn_fmed3f(vx, -kBf16Max, kBf16Max);
    tail_k[(bh * tail_rows + j) * kD + d] = f32_to_bf16_bits(kx);
    tail_v[(bh * tail_rows + j) * kD + d] = f32_to_bf16_bits(vx);
  }
}

// Prefix rows [0, n_rows) of the quantised cache as float16 rows of the dense K/V buffers (the form taken for
// long chunks: the attention kernel then reads every tile as a dense one). Same arithmetic as the in-kernel
// unpacking (float16 code * scale + bias), so both forms attend the same values. A thread converts 16 codes
// of K and of V; 16 threads a row, 16 rows a workgroup.
// 16 unsigned 8-bit codes -> 16 bfloat16 values: code * scale + bias in float32 (one fused multiply-add, scale and
// bias at their float32 values), rounded once
__device__ __forceinline__ void dequant16_bf16(u32x4_t c, float sc, float bi, u32x4_t& p0, u32x4_t& p1) {
#pragma unroll
  for (int w = 0; w < 4; w++) {
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) v[j] = __builtin_fmaf((float)((c[w] >> (8 * j)) & 0xFFu), sc, bi);
    const uint32_t lo = pack2<MSPR_BF16>(v[0], v[1]), hi = pack2<MSPR_BF16>(v[2], v[3]);
    if (w < 2) {
      p0[2 * w] = lo;
      p0[2 * w + 1] = hi;
    } else {
      p1[2 * (w - 2)] = lo;
      p1[2 * (w - 2) + 1] = hi;
    }
  }
}
template <int SDT>
__device__ __forceinline__ float sb_to_f32(uint32_t bits) {
  if constexpr (SDT == MSPR_F32) return __builtin_bit_cast(float, bits);
  else if constexpr (SDT == MSPR_F16) return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
  else return __builtin_bit_cast(float, bits << 16);
}

template <int SDT, int ODT>
__global__ __launch_bounds__(256) void prefill_q8_dequant_kernel(PrefillArgs a, uint16_t* out_k, uint16_t* out_v,
                                                                 int64_t n_rows, int64_t out_rows) {
  const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  const int pp = threadIdx.x & 15;
  if (row >= n_rows) return;
  const int64_t bh = (int64_t)blockIdx.z * a.n_kv_heads + blockIdx.y;
  const int64_t src = bh * a.past_rows + row;
  const u32x4_t rk = reinterpret_cast<const u32x4_t*>(a.pk_wq)[src * 16 + pp];
  const u32x4_t rv = reinterpret_cast<const u32x4_t*>(a.pv_wq)[src * 16 + pp];
  uint32_t rs[4];
  const void* arrs[4] = {a.pk_s, a.pk_b, a.pv_s, a.pv_b};
#pragma unroll
  for (int i = 0; i < 4; i++) {
    if constexpr (SDT == MSPR_F32) rs[i] = reinterpret_cast<const uint32_t*>(arrs[i])[src * 4 + (pp >> 2)];
    else rs[i] = reinterpret_cast<const uint16_t*>(arrs[i])[src * 4 + (pp >> 2)];
  }
  u32x4_t p0, p1;
  const int64_t dst = (bh * out_rows + row) * kD + 16 * pp;
  if constexpr (ODT == MSPR_F16) dequant16(rk, sb_to_h2<SDT>(rs[0]), sb_to_h2<SDT>(rs[1]), p0, p1);
  else dequant16_bf16(rk, sb_to_f32<SDT>(rs[0]), sb_to_f32<SDT>(rs[1]), p0, p1);
  *reinterpret_cast<u32x4_t*>(out_k + dst) = p0;
  *reinterpret_cast<u32x4_t*>(out_k + dst + 8) = p1;
  if constexpr (ODT == MSPR_F16) dequant16(rv, sb_to_h2<SDT>(rs[2]), sb_to_h2<SDT>(rs[3]), p0, p1);
  else dequant16_bf16(rv, sb_to_f32<SDT>(rs[2]), sb_to_f32<SDT>(rs[3]), p0, p1);
  *reinterpret_cast<u32x4_t*>(out_v + dst) = p0;
  *reinterpret_cast<u32x4_t*>(out_v + dst + 8) = p1;
}

// Merge of the key-range partials of one query row: 64 lanes x 4 columns, four rows per workgroup.
template <int ODT>
__global__ __launch_bounds__(256) void prefill_merge_kernel(PrefillArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t n_rows = (int64_t)a.batch * a.n_q_heads * a.q_len;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= n_rows) return;
  float m_run = -__builtin_inff(), l = 0.0f;
  f32x4_t o = {0.f, 0.f, 0.f, 0.f};
  constexpr int kChunk = 8;
  for (int s0 = 0; s0 < a.n_splits; s0 += kChunk) {
    float mv[kChunk], lv[kChunk];
    f32x4_t ov[kChunk];
#pragma unroll
    for (int j = 0; j < kChunk; j++) {
      const int sj = s0 + j < a.n_splits ? s0 + j : 0;
      const int64_t r = (int64_t)sj * n_rows + row;
      mv[j] = a.ws_ml[r * 2];
      lv[j] = a.ws_ml[r * 2 + 1];
      ov[j] = *reinterpret_cast<const f32x4_t*>(a.ws_o + r * kD + 4 * lane);
      // a range that saw no key of this row contributes nothing (its O is whatever the registers held)
      if (s0 + j >= a.n_splits || !(lv[j] > 0.0f)) {
        mv[j] = -__builtin_inff();
        lv[j] = 0.0f;
        ov[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      }
    }
    float m_new = m_run;
#pragma unroll
    for (int j = 0; j < kChunk; j++) m_new = fmaxf(m_new, mv[j]);
    const float m_safe = m_new == -__builtin_inff() ? 0.0f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_safe);
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
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;
  if constexpr (ODT == MSPR_F32) {
    *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(a.out) + row * kD + 4 * lane) = o * inv;
  } else {
    u32x2_t w = {pack2<ODT>(o.x * inv, o.y * inv), pack2<ODT>(o.z * inv, o.w * inv)};
    *reinterpret_cast<u32x2_t*>(reinterpret_cast<uint16_t*>(a.out) + row * kD + 4 * lane) = w;
  }
}

// workgroups along the query axis: pairs of (late, early) row ranges, times two head halves when eight
// query heads share a KV head (see the kernel's work mapping)
int prefill_q_blocks(int rep, int q_len) {
  const int heads_per_group = rep < 4 ? rep : 4;
  const int blocks_per_group = 4 / heads_per_group;
  const int n_blocks = (q_len + 31) / 32;
  const int n_pairs = (n_blocks + 2 * blocks_per_group - 1) / (2 * blocks_per_group);
  return n_pairs * (rep / heads_per_group);
}

// enough workgroups for the 256 CUs but not more (one fits a CU, so a count just above 256 means a second
// round for a few of them), at least 16 tiles (512 keys) per range
int prefill_choose_splits(int batch, int n_kv_heads, int q_blocks, int64_t past_len, int q_len) {
  const int64_t wgs = (int64_t)batch * n_kv_heads * q_blocks;
  if (wgs >= 192) return 1;
  int64_t want = 256 / wgs;
  const int64_t tiles = (past_len + q_len + kTile - 1) / kTile;
  if (want > tiles / 16) want = tiles / 16;
  if (want > 32) want = 32;
  return want < 1 ? 1 : (int)want;
}

size_t prefill_split_bytes(int batch, int n_q_heads, int n_kv_heads, int q_len, int64_t past_len) {
  const int rep = n_q_heads / n_kv_heads;
  const int q_blocks = prefill_q_blocks(rep, q_len);
  const int splits = prefill_choose_splits(batch, n_kv_heads, q_blocks, past_len, q_len);
  if (splits == 1) return 0;
  return (size_t)splits * batch * n_q_heads * q_len * (kD + 2) * sizeof(float);
}

template <int KDT, bool Q8, int SDT, bool IO32 = Q8>
int prefill_launch(const PrefillArgs& a, hipStream_t st) {
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&flash_prefill_kernel<KDT, Q8, SDT, IO32>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    if (e != hipSuccess) {
      mspr_set_error("flash_prefill: cannot reserve %d bytes of LDS: %s", kLdsBytes, hipGetErrorString(e));
      return MSPR_ERR_LAUNCH;
    }
    attr_set = true;
  }
  dim3 grid((unsigned)(a.q_blocks * a.n_kv_heads * a.batch * a.n_splits)), block(kThreads);
  {
    MsprProfScope prof(MSPR_K_FLASH_PREFILL, st);
    flash_prefill_kernel<KDT, Q8, SDT, IO32><<<grid, block, kLdsBytes, st>>>(a);
  }
  MSPR_CHECK_LAUNCH("flash_prefill");
  if (a.n_splits > 1) {
    const int64_t n_rows = (int64_t)a.batch * a.n_q_heads * a.q_len;
    dim3 mgrid((unsigned)((n_rows + 3) / 4)), mblock(256);
    if (IO32) prefill_merge_kernel<MSPR_F32><<<mgrid, mblock, 0, st>>>(a);
    else prefill_merge_kernel<KDT><<<mgrid, mblock, 0, st>>>(a);
    MSPR_CHECK_LAUNCH("flash_prefill (merge)");
  }
  return MSPR_OK;
}

}  // namespace

extern "C" size_t mspr_flash_prefill_workspace_bytes(int batch, int n_q_heads, int n_kv_heads, int q_len,
                                                     int64_t past_len) {
  if (batch < 1 || n_kv_heads < 1 || n_q_heads < n_kv_heads || n_q_heads % n_kv_heads != 0 || q_len < 1 ||
      past_len < 0 || n_q_heads / n_kv_heads > 8)
    return 0;
  return prefill_split_bytes(batch, n_q_heads, n_kv_heads, q_len, past_len) + 256;
}

extern "C" int mspr_flash_prefill(const void* q, const void* k, const void* v, int dtype, int batch, int n_q_heads,
                                  int n_kv_heads, int head_dim, int q_len, int64_t past_len, int64_t kv_rows,
                                  float scale, void* out, void* workspace, size_t workspace_bytes, void* stream) {
  MSPR_REQUIRE(q && k && v && out, "flash_prefill: null pointer");
  MSPR_REQUIRE(dtype == MSPR_BF16 || dtype == MSPR_F16, "flash_prefill: dtype must be float16 or bfloat16");
  MSPR_REQUIRE(head_dim == kD, "flash_prefill: head_dim must be 256");
  MSPR_REQUIRE(batch >= 1 && n_kv_heads >= 1 && n_q_heads >= n_kv_heads && n_q_heads % n_kv_heads == 0,
               "flash_prefill: bad head counts");
  const int rep = n_q_heads / n_kv_heads;
  MSPR_REQUIRE(rep == 1 || rep == 2 || rep == 4 || rep == 8,
               "flash_prefill: query heads per KV head must be 1, 2, 4 or 8");
  MSPR_REQUIRE(q_len >= 1 && past_len >= 0 && past_len + q_len <= kv_rows && kv_rows < ((int64_t)1 << 31),
               "flash_prefill: need q_len >= 1, past_len >= 0 and past_len + q_len <= kv_rows");
  MSPR_REQUIRE(mspr_aligned(q, 16) && mspr_aligned(k, 16) && mspr_aligned(v, 16) && mspr_aligned(out, 16),
               "flash_prefill: pointers must be 16-byte aligned");
  PrefillArgs a = {};
  a.q = q;
  a.k = k;
  a.v = v;
  a.out = out;
  a.batch = batch;
  a.n_q_heads = n_q_heads;
  a.n_kv_heads = n_kv_heads;
  a.q_len = q_len;
  a.past_len = past_len;
  a.kv_rows = kv_rows;
  a.scale_log2 = (float)((double)scale * 1.4426950408889634);
  a.rep_shift = rep == 1 ? 0 : rep == 2 ? 1 : rep == 4 ? 2 : 3;
  a.q_blocks = prefill_q_blocks(rep, q_len);
  a.n_splits = prefill_choose_splits(batch, n_kv_heads, a.q_blocks, past_len, q_len);
  MSPR_REQUIRE((int64_t)a.q_blocks * n_kv_heads * batch * a.n_splits < ((int64_t)1 << 31), "flash_prefill: grid too large");
  if (a.n_splits > 1) {
    const size_t need = prefill_split_bytes(batch, n_q_heads, n_kv_heads, q_len, past_len);
    MSPR_REQUIRE(workspace && workspace_bytes >= need && mspr_aligned(workspace, 16),
                 "flash_prefill: workspace of %zu bytes (16-byte aligned) needed, %zu given", need, workspace_bytes);
    a.ws_o = reinterpret_cast<float*>(workspace);
    a.ws_ml = a.ws_o + (size_t)a.n_splits * batch * n_q_heads * q_len * kD;
  }
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MSPR_BF16) return prefill_launch<MSPR_BF16, false, MSPR_F32>(a, st);
  return prefill_launch<MSPR_F16, false, MSPR_F32>(a, st);
}

// Prefix tiles unpacked inside the attention kernel. Unpacking costs a fifth of a tile's time for every
// workgroup that passes the tile; converting the prefix once costs about 1.4 ns per row. From a thousand
// queries per chunk on, the prefix is therefore converted to float16 rows first (a scratch of 1 KB per key and
// KV head) and the attention kernel runs on dense tiles only.
static int prefill_q8_tiles(int q_len, int64_t past_len) { return q_len >= 1024 ? 0 : (int)(past_len / kTile); }

extern "C" size_t mspr_sdpa_fa_prefill_q8_workspace_bytes(int batch, int n_q_heads, int n_kv_heads, int q_len,
                                                          int64_t past_len) {
  if (batch < 1 || n_kv_heads < 1 || n_q_heads < n_kv_heads || n_q_heads % n_kv_heads != 0 || q_len < 1 ||
      past_len < 0 || n_q_heads / n_kv_heads > 8)
    return 0;
  const int64_t tail_rows = past_len - (int64_t)prefill_q8_tiles(q_len, past_len) * kTile + q_len;
  const size_t tail = ((size_t)batch * n_kv_heads * tail_rows * kRowBytes * 2 + 255) / 256 * 256;
  return tail + prefill_split_bytes(batch, n_q_heads, n_kv_heads, q_len, past_len) + 256;
}

extern "C" int mspr_sdpa_fa_prefill_q8(const void* queries, const void* pk_wq, const void* pk_scales,
                                       const void* pk_biases, const void* pv_wq, const void* pv_scales,
                                       const void* pv_biases, int sb_dtype, const void* self_k, const void* self_v,
                                       int self_dtype, int batch, int n_q_heads, int n_kv_heads, int head_dim,
                                       int q_len, int64_t past_len, int64_t past_rows, float scale, int group_size,
                                       int bits, void* out, void* workspace, size_t workspace_bytes, void* stream) {
  MSPR_REQUIRE(group_size == 64 && bits == 8, "sdpa_fa_prefill_q8: only group_size=64, bits=8 is supported");
  MSPR_REQUIRE(past_rows >= past_len, "sdpa_fa_prefill_q8: past_rows (rows allocated per head) must cover past_len");
  MSPR_REQUIRE(queries && self_k && self_v && out, "sdpa_fa_prefill_q8: null pointer");
  MSPR_REQUIRE(past_len == 0 || (pk_wq && pk_scales && pk_biases && pv_wq && pv_scales && pv_biases),
               "sdpa_fa_prefill_q8: null pointer");
  MSPR_REQUIRE(sb_dtype >= MSPR_F32 && sb_dtype <= MSPR_BF16 && self_dtype >= MSPR_F32 && self_dtype <= MSPR_BF16,
               "sdpa_fa_prefill_q8: scales/biases and the self chunk must be f32, f16 or bf16");
  MSPR_REQUIRE(head_dim == kD, "sdpa_fa_prefill_q8: head_dim must be 256");
  MSPR_REQUIRE(batch >= 1 && n_kv_heads >= 1 && n_q_heads >= n_kv_heads && n_q_heads % n_kv_heads == 0,
               "sdpa_fa_prefill_q8: bad head counts");
  const int rep = n_q_heads / n_kv_heads;
  MSPR_REQUIRE(rep == 1 || rep == 2 || rep == 4 || rep == 8,
               "sdpa_fa_prefill_q8: query heads per KV head must be 1, 2, 4 or 8");
  MSPR_REQUIRE(q_len >= 1 && past_len >= 0 && past_len + q_len < ((int64_t)1 << 31),
               "sdpa_fa_prefill_q8: need q_len >= 1 and past_len >= 0");
  MSPR_REQUIRE(mspr_aligned(queries, 16) && mspr_aligned(out, 16) && mspr_aligned(pk_wq, 16) && mspr_aligned(pv_wq, 16),
               "sdpa_fa_prefill_q8: pointers must be 16-byte aligned");
  // (scales and biases move to LDS four bytes per lane)
  MSPR_REQUIRE(mspr_aligned(pk_scales, 4) && mspr_aligned(pk_biases, 4) && mspr_aligned(pv_scales, 4) &&
                   mspr_aligned(pv_biases, 4),
               "sdpa_fa_prefill_q8: scales and biases must be 4-byte aligned");
  const size_t need = mspr_sdpa_fa_prefill_q8_workspace_bytes(batch, n_q_heads, n_kv_heads, q_len, past_len);
  MSPR_REQUIRE(workspace && workspace_bytes >= need && mspr_aligned(workspace, 16),
               "sdpa_fa_prefill_q8: workspace of %zu bytes (16-byte aligned) needed, %zu given", need, workspace_bytes);
  PrefillArgs a = {};
  const int q8_tiles = prefill_q8_tiles(q_len, past_len);
  const int tail_rows = (int)(past_len - (int64_t)q8_tiles * kTile) + q_len;
  uint16_t* tail_k = reinterpret_cast<uint16_t*>(workspace);
  uint16_t* tail_v = tail_k + (size_t)batch * n_kv_heads * tail_rows * kD;
  a.q = queries;
  a.k = tail_k;
  a.v = tail_v;
  a.out = out;
  a.batch = batch;
  a.n_q_heads = n_q_heads;
  a.n_kv_heads = n_kv_heads;
  a.q_len = q_len;
  a.past_len = past_len;
  a.kv_rows = tail_rows;
  a.scale_log2 = (float)((double)scale * 1.4426950408889634);
  a.rep_shift = rep == 1 ? 0 : rep == 2 ? 1 : rep == 4 ? 2 : 3;
  a.q_blocks = prefill_q_blocks(rep, q_len);
  a.q8_tiles = q8_tiles;
  a.past_rows = past_rows;
  a.n_splits = prefill_choose_splits(batch, n_kv_heads, a.q_blocks, past_len, q_len);
  if (a.n_splits > 1) {
    const size_t tail = ((size_t)batch * n_kv_heads * tail_rows * kRowBytes * 2 + 255) / 256 * 256;
    a.ws_o = reinterpret_cast<float*>(reinterpret_cast<unsigned char*>(workspace) + tail);
    a.ws_ml = a.ws_o + (size_t)a.n_splits * batch * n_q_heads * q_len * kD;
  }
  a.pk_wq = pk_wq;
  a.pk_s = pk_scales;
  a.pk_b = pk_biases;
  a.pv_wq = pv_wq;
  a.pv_s = pv_scales;
  a.pv_b = pv_biases;
  hipStream_t st = (hipStream_t)stream;
  // rows of the dense buffers: prefix rows not left to the attention kernel, then the chunk's own rows
  const int64_t dq_rows = q8_tiles == 0 ? past_len : 0;  // converted 16 codes at a time
  const int first_row = (int)dq_rows;                   // the rest element by element (at most 31 prefix rows + chunk)
#ifndef MSPR_Q8_LONG_BF16
#define MSPR_Q8_LONG_BF16 1
#endif
  // Long chunks (prefix converted beforehand) stage K/V and the queries as bfloat16 and run the bfloat16 matrix
  // instructions: the device holds a higher clock under them than under the float16 ones, and the 8-bit codes
  // leave the rounding of the staging type (2^-9 of a value) below their own step. Short chunks unpack the
  // prefix inside the attention kernel with packed float16 arithmetic and stay float16 throughout.
  const bool bf16_staging = MSPR_Q8_LONG_BF16 && q_len >= 1024;  // (then q8_tiles == 0)
#define MSPR_LAUNCH_BY_SB(KERNEL, GRID, ...)                                                          \
  do {                                                                                                \
    if (bf16_staging) {                                                                               \
      if (sb_dtype == MSPR_F32) KERNEL<MSPR_F32, MSPR_BF16><<<GRID, 256, 0, st>>>(__VA_ARGS__);        \
      else if (sb_dtype == MSPR_F16) KERNEL<MSPR_F16, MSPR_BF16><<<GRID, 256, 0, st>>>(__VA_ARGS__);   \
      else KERNEL<MSPR_BF16, MSPR_BF16><<<GRID, 256, 0, st>>>(__VA_ARGS__);                            \
    } else {                                                                                          \
      if (sb_dtype == MSPR_F32) KERNEL<MSPR_F32, MSPR_F16><<<GRID, 256, 0, st>>>(__VA_ARGS__);         \
      else if (sb_dtype == MSPR_F16) KERNEL<MSPR_F16, MSPR_F16><<<GRID, 256, 0, st>>>(__VA_ARGS__);    \
      else KERNEL<MSPR_BF16, MSPR_F16><<<GRID, 256, 0, st>>>(__VA_ARGS__);                             \
    }                                                                                                 \
  } while (0)
  if (dq_rows > 0) {
    dim3 dgrid((unsigned)((dq_rows + 15) / 16), (unsigned)n_kv_heads, (unsigned)batch);
    MSPR_LAUNCH_BY_SB(prefill_q8_dequant_kernel, dgrid, a, tail_k, tail_v, dq_rows, tail_rows);
    MSPR_CHECK_LAUNCH("sdpa_fa_prefill_q8 (prefix rows)");
  }
  dim3 tgrid((unsigned)(tail_rows - first_row), (unsigned)n_kv_heads, (unsigned)batch);
  MSPR_LAUNCH_BY_SB(prefill_q8_tail_kernel, tgrid, a, self_k, self_v, self_dtype, tail_k, tail_v, tail_rows, first_row);
#undef MSPR_LAUNCH_BY_SB
  MSPR_CHECK_LAUNCH("sdpa_fa_prefill_q8 (tail rows)");
  // (prefix converted beforehand: the dense kernel, with float32 queries and output)
  if (q8_tiles == 0) {
    if (bf16_staging) return prefill_launch<MSPR_BF16, false, MSPR_F32, true>(a, st);
    return prefill_launch<MSPR_F16, false, MSPR_F32, true>(a, st);
  }
  if (sb_dtype == MSPR_F32) return prefill_launch<MSPR_F16, true, MSPR_F32>(a, st);
  if (sb_dtype == MSPR_F16) return prefill_launch<MSPR_F16, true, MSPR_F16>(a, st);
  return prefill_launch<MSPR_F16, true, MSPR_BF16>(a, st);
}
