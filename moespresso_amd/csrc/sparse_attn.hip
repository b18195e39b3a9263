// Gathered ("indexed") decode attention over a latent KV cache shared by all heads.
//
// One query token per batch entry attends a list of key slots: first a window segment (a ring of
// raw rows, optionally with one slot replaced by a freshly prepared row), then rows gathered from
// a pool by index. K is the whole row (512 or 576 wide), V its first 512 columns.
//
// Work split: a workgroup owns (batch, 64-head block, slot range) and streams 32-slot tiles.
// Each K row is read from HBM once and staged row-major in LDS (ring of three tiles, filled by
// asynchronous global->LDS copies). The eight waves are (head group hg of 32 heads) x (quarter dh):
// for S^T = K.Q^T a wave contracts its quarter of the row width and the four quarters are summed
// through LDS; for O^T = V^T.P^T it owns 128 of the 512 output columns. Two waves share a SIMD and
// fill each other's waits (a wave has no matrix work while it stages or exchanges). V^T operands come
// out of the same row-major tile through the LDS transpose read, so no second copy of the tile
// exists.
//
// Partial (m, l, O) per key range are merged by a second kernel (log-sum-exp), which also applies the
// sink, the normalisation, the output cast and the optional inverse rope. (Merging inside the split
// launch, behind a per-sequence arrival counter, was built and measured: the device-scope release of
// the partials, the counter round trips and the partial reads are five dependent trips to memory of
// about 2 us each at the end of every workgroup, against 6 us for the second launch.)
//
// MFMA shapes: v_mfma_f32_32x32x16_{f16,bf16}. Accumulator layout (lane l, register i):
// column = l % 32, row = 8*(i/4) + 4*(l/32) + i%4. In S^T the column is the head and the row the
// key, so softmax statistics are per lane; P^T registers feed the next MFMA's B operand unchanged.
#include "common.h"
#include "profile.h"

#include <cstdlib>

// Scratch of mspr_sparse_mla_decode_static, the entry point that allocates nothing: the partials of up to 256
// key ranges (a grid of one workgroup per CU), 64 heads x 512 float16 and 64 x (m, l) float32 each. Every range
// of a call is written before it is read, so nothing in it has to start at zero. Host code never uses this
// name as an address: it asks for the device address once per device (static_scratch below).
constexpr size_t kStaticBytes = 256 * (size_t)(64 * 512 * 2 + 64 * 2 * 4);
static __device__ __align__(256) unsigned char scratch[kStaticBytes];

namespace {

constexpr int kTile = 32;
constexpr int kDV = 512;
constexpr int kThreads = 512;  // split kernel: eight waves, two per SIMD
constexpr int kWaves = kThreads / 64;

struct SparseAttnArgs {
  // query
  const void* q;
  int q_dtype;
  int64_t q_batch_stride;  // elements; q of (b, t, head) at b*q_batch_stride + t*q_token_stride + head*q_head_stride
  int64_t q_head_stride;
  int64_t q_token_stride;
  int n_heads;
  int batch;               // sequences = batch entries x tokens
  int n_tokens;            // query tokens per batch entry; they share the window and pool tensors
  // prefill form: window range and visible pool prefix follow from the token's position pos0 + t
  int prefill;
  uint32_t pos0, window, ratio;
  // window segment
  const void* win;
  int64_t win_batch_stride;
  int n_win;
  int win_first;  // logical index of the first visited ring row
  int raw_start;
  int raw_cap;
  const void* subst_row;
  int subst_slot;          // window slot replaced by subst_row (-1: none)
  int subst_from_params;   // take the slot from params[1] on the device instead
  // gathered segment
  const void* pool;
  int64_t pool_batch_stride;
  int64_t n_pool;
  const int32_t* pool_rows_dev;  // optional: rows of the pool in use, read on the device (<= n_pool, the capacity)
  const int32_t* idx;
  int64_t idx_batch_stride;
  int n_idx;
  int64_t visible;  // ids >= visible end the walk
  int check_stop;
  int row_mul;  // pool row = id * row_mul + row_add
  int row_add;
  // softmax
  const void* sinks;
  int sinks_dtype;
  float scale_log2;
  // rope
  const float* inv_freq;
  const int32_t* params;
  int rope;
  // split: range sp of a sequence owns window slots [sp*win_per_split, +win_per_split) and gathered
  // ids [sp*idx_per_split, +idx_per_split)
  int n_splits;
  uint32_t inv_splits, inv_hblk, inv_tokens;  // floor(2^32 / n) of n_splits, n_hblk, n_tokens
  int win_per_split;
  int idx_per_split;
  int n_hblk;
  uint16_t* ws_o;  // float16 partial rows, each normalised by its own range's denominator
  float* ws_ml;
  // output
  void* out;
  int out_dtype;
  int64_t out_batch_stride, out_head_stride, out_token_stride;  // elements
  int direct;  // one key range per sequence: the split kernel normalises and stores, no partials
};

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

// Two float32 values rounded (nearest even) to the KV element type, packed in one register; the
// vector conversion lowers to one v_cvt_pk_{bf16,f16}_f32.
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

// 2^x through the hardware transcendental (no denormal fix-up: results below 2^-126 flush to 0,
// which is what a softmax weight that small should do).
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <int KDT>
__device__ __forceinline__ float unpack_lo(uint32_t w) {
  if constexpr (KDT == MSPR_BF16) return bf16_bits_to_f32((uint16_t)(w & 0xFFFFu));
  else return f16_bits_to_f32((uint16_t)(w & 0xFFFFu));
}
template <int KDT>
__device__ __forceinline__ float unpack_hi(uint32_t w) {
  if constexpr (KDT == MSPR_BF16) return bf16_bits_to_f32((uint16_t)(w >> 16));
  else return f16_bits_to_f32((uint16_t)(w >> 16));
}

template <int KDT>
__device__ __forceinline__ float round_to_kdt(float v) {
  if constexpr (KDT == MSPR_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(v));
  else return f16_bits_to_f32(f32_to_f16_bits(v));
}

// Query element type of a kernel instance: the KV type itself (operands are used as loaded) or
// float32 (rounded to the KV type on load).
constexpr int kQSame = -1;

// A zero row for slots that are skipped: the asynchronous tile loads always run with every lane
// active (the wait counters below rely on a fixed number of loads per tile), so a skipped slot reads
// zeros instead of being predicated off.
__device__ __attribute__((aligned(16))) const unsigned char g_zero_row[1280] = {0};

// Where the prefill consumer's lanes without a head (a block of fewer than 64 heads) put their output stores, so
// that the store instructions run with every lane active and the same count in every wave: 512 floats per lane
// position, never read.
__device__ __attribute__((aligned(16))) float g_store_sink[64 * 512];

#define MSPR_GLB_PTR(T, p) ((__attribute__((address_space(1))) T*)(p))

// Wait until at most N of this wave's vector-memory operations are outstanding and all of its LDS
// operations are done, then meet the other waves. Written as one asm statement so that no
// compiler-inserted full drain (as a fence would add) sits between the asynchronous tile loads.
template <int N>
__device__ __forceinline__ void wait_vm_and_barrier() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}
// One wave-wide asynchronous copy global -> LDS: lane i's 16 bytes at `src` land at lds_base + 16 i
// (lds_base is wave-uniform). Issued through asm so that the compiler's wait-count pass does not
// see LDS writes in flight (it would drain them in front of every LDS transpose read); completion
// is awaited explicitly through wait_vm_and_barrier.
__device__ __forceinline__ void async_load_16(uint64_t src, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_base) : "memory", "m0");
}
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Normalised output values of four consecutive columns -> output tensor, in the output element type
// (the fused-decode form applies the inverse partial rope on the float16 values at float16 op rounding).
template <int ODT>
__device__ __forceinline__ void emit_output(const SparseAttnArgs& a, const float (&r)[4], int64_t ooff, int dim0) {
  if constexpr (ODT == MSPR_F32) {
    *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(a.out) + ooff) = f32x4_t{r[0], r[1], r[2], r[3]};
  } else if constexpr (ODT == MSPR_BF16) {
    u32x2_t w2 = {(uint32_t)f32_to_bf16_bits(r[0]) | ((uint32_t)f32_to_bf16_bits(r[1]) << 16),
                  (uint32_t)f32_to_bf16_bits(r[2]) | ((uint32_t)f32_to_bf16_bits(r[3]) << 16)};
    *reinterpret_cast<u32x2_t*>(reinterpret_cast<uint16_t*>(a.out) + ooff) = w2;
  } else {
    float h[4];
#pragma unroll
    for (int j = 0; j < 4; j++) h[j] = f16_bits_to_f32(f32_to_f16_bits(r[j]));
    if (a.rope && dim0 >= kDV - 64) {
#pragma unroll
      for (int j = 0; j < 2; j++) {
        int p = (dim0 - (kDV - 64)) / 2 + j;
        float theta = (float)a.params[0] * a.inv_freq[p];
        float cs = f16_bits_to_f32(f32_to_f16_bits((float)cos((double)theta)));
        float sn = f16_bits_to_f32(f32_to_f16_bits(-(float)sin((double)theta)));
        float x0 = h[2 * j], x1 = h[2 * j + 1];
        float m0 = f16_bits_to_f32(f32_to_f16_bits(x0 * cs)), m1 = f16_bits_to_f32(f32_to_f16_bits(x1 * sn));
        float m2 = f16_bits_to_f32(f32_to_f16_bits(x0 * sn)), m3 = f16_bits_to_f32(f32_to_f16_bits(x1 * cs));
        h[2 * j] = f16_bits_to_f32(f32_to_f16_bits(m0 - m1));
        h[2 * j + 1] = f16_bits_to_f32(f32_to_f16_bits(m2 + m3));
      }
    }
    u32x2_t w2 = {(uint32_t)f32_to_f16_bits(h[0]) | ((uint32_t)f32_to_f16_bits(h[1]) << 16),
                  (uint32_t)f32_to_f16_bits(h[2]) | ((uint32_t)f32_to_f16_bits(h[3]) << 16)};
    *reinterpret_cast<u32x2_t*>(reinterpret_cast<uint16_t*>(a.out) + ooff) = w2;
  }
}

__device__ __forceinline__ float load_sink_log2(const SparseAttnArgs& a, int head) {
  if (!a.sinks) return -__builtin_inff();
  return (a.sinks_dtype == MSPR_F16 ? f16_bits_to_f32(reinterpret_cast<const uint16_t*>(a.sinks)[head])
                                    : reinterpret_cast<const float*>(a.sinks)[head]) * 1.4426950408889634f;
}

template <int DK>
struct Geometry {
  static constexpr int kSlots = DK / 8 + 1;        // 16-byte slots per LDS row; the last one is padding, so
                                                   // 8 consecutive rows start on distinct 16B bank groups
  static constexpr int kPitch = kSlots * 16;       // bytes
  static constexpr int kTileSlots = kTile * kSlots;
  static constexpr int kInstr = (kTileSlots + 63) / 64;   // wave-wide 1 KB loads per tile
  static constexpr int kPerThread = (kInstr + kWaves - 1) / kWaves;  // loads per thread per tile
  static constexpr int kLastWaves = kInstr - kWaves * (kPerThread - 1);  // waves that issue the last of them
  static constexpr int kTileBytes = kInstr * 1024;
  static constexpr int kPart = DK / 4;             // contraction columns per dh wave
  static constexpr int kSteps = kPart / 16;        // MFMA k-steps per dh wave
  static constexpr int kBufs = 3;                  // tile ring: one in use, two in flight
  static constexpr int kSxBytes = 4 * 16 * 64 * 4; // 4 waves x 16 floats x 64 lanes (one head group)
  static constexpr int kMaxIds = 1024;             // gathered slots per workgroup
  static constexpr int kOffSx = kBufs * kTileBytes;
  static constexpr int kMaxTiles = kMaxIds / kTile; // tiles per workgroup
  static constexpr int kOffRowPtr = kOffSx + 2 * kSxBytes;       // row pointer of every slot of the workgroup
  static constexpr int kOffVmask = kOffRowPtr + kMaxIds * 8;     // one validity word per tile
  static constexpr int kOffRope = kOffVmask + kMaxTiles * 4;
  static constexpr int kOffStop = kOffRope + 64 * 4;
  static constexpr int kLdsBytes = kOffStop + 16;
  static_assert(kPart % 16 == 0, "a wave's share of the row width is a whole number of MFMA k-steps");
  static_assert(kLastWaves >= 1 && kLastWaves <= kWaves, "the last round of tile loads is issued by the first waves");
};

template <int KDT, int DK, int QDT, bool ROPE>
__global__ __launch_bounds__(kThreads, 1) void sparse_attn_split_kernel(SparseAttnArgs a) {
  using G = Geometry<DK>;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  unsigned char* kbuf = lds;                                                   // [kBufs][kTileBytes]
  float* sx = reinterpret_cast<float*>(lds + G::kOffSx);                       // [8 waves][16*64]
  uint64_t* rowptr = reinterpret_cast<uint64_t*>(lds + G::kOffRowPtr);         // [kMaxIds]
  uint32_t* vmask = reinterpret_cast<uint32_t*>(lds + G::kOffVmask);           // [kMaxTiles]
  float* rope_c = reinterpret_cast<float*>(lds + G::kOffRope);
  float* rope_s = rope_c + 32;
  int* stop_shared = reinterpret_cast<int*>(lds + G::kOffStop);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int hg = wave >> 2;  // head group of 32 heads
  const int dh = wave & 3;   // quarter of the row width (S^T) and of the output columns (O^T)
  const int n = lane & 31;  // MFMA column: head (S^T, O^T); MFMA row for A operands
  const int g = lane >> 5;

  // ---- workgroup -> (batch, head block, split); consecutive splits of one batch share an XCD
  const int total = gridDim.x;
  int work = blockIdx.x;
  if ((total & 7) == 0) work = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
  // (divisions by multiplication with floor(2^32 / n) and one correction step: a launch starts with an empty
  // instruction cache, and a software division is a hundred instructions in front of the first memory request)
  auto div_by = [](uint32_t x, uint32_t n, uint32_t inv) -> uint32_t {
    if (n == 1u) return x;
    uint32_t q = __umulhi(x, inv);  // true quotient or one less
    if (x - q * n >= n) q++;
    return q;
  };
  const int bh = (int)div_by((uint32_t)work, (uint32_t)a.n_splits, a.inv_splits);
  const int sp = work - bh * a.n_splits;
  const int seq = (int)div_by((uint32_t)bh, (uint32_t)a.n_hblk, a.inv_hblk);
  const int hb = bh - seq * a.n_hblk;
  const int b = (int)div_by((uint32_t)seq, (uint32_t)a.n_tokens, a.inv_tokens);
  const int t = seq - b * a.n_tokens;

  // window rows and visible pool prefix of this sequence; the prefill form derives them from the
  // token's position in the unsigned 32-bit arithmetic of the reference kernel
  int seq_n_win = a.n_win, seq_win_first = a.win_first;
  int64_t seq_visible = a.visible;
  if (a.prefill) {
    const uint32_t qpos = a.pos0 + (uint32_t)t, n_raw = (uint32_t)a.raw_cap;
    const uint32_t last_pos = a.pos0 + (uint32_t)a.n_tokens - 1u;
    const uint32_t first_raw_pos = last_pos + 1u - n_raw;
    const uint32_t window_first = (a.window != 0u && qpos + 1u > a.window) ? qpos + 1u - a.window : 0u;
    const uint32_t first = first_raw_pos > window_first ? first_raw_pos : window_first;
    const uint32_t last = qpos < last_pos ? qpos : last_pos;
    seq_n_win = first <= last ? (int)(last - first + 1u) : 0;
    if (seq_n_win > a.n_win) seq_n_win = a.n_win;  // the host sized the slot space for n_win window rows
    seq_win_first = first <= last ? (int)(first - first_raw_pos) : 0;
    const int64_t vis = a.ratio == 0u ? a.n_pool : (int64_t)((qpos + 1u) / a.ratio);
    seq_visible = vis < a.n_pool ? vis : a.n_pool;
  }

  // range sp: its share of the window slots, then its share of the gathered ids. Window tiles come
  // first in the tile order: their rows need no ids, so their copies leave before the id round trip.
  const int w0 = sp * a.win_per_split;
  int w1 = w0 + a.win_per_split;
  if (w1 > seq_n_win) w1 = seq_n_win;
  const int wt = w1 > w0 ? (w1 - w0 + kTile - 1) / kTile : 0;
  const int g0 = sp * a.idx_per_split;
  int g1 = g0 + a.idx_per_split;
  if (g1 > a.n_idx) g1 = a.n_idx;
  const int gt = g1 > g0 ? (g1 - g0 + kTile - 1) / kTile : 0;
  const int n_tiles = wt + gt;
  const int g_ls0 = wt * kTile;  // first local slot of the gathered part

  const uint16_t* win_b = reinterpret_cast<const uint16_t*>(a.win) + (int64_t)b * a.win_batch_stride;
  const uint16_t* pool_b = reinterpret_cast<const uint16_t*>(a.pool) + (int64_t)b * a.pool_batch_stride;
  const int32_t* idx_b = a.idx + (int64_t)seq * a.idx_batch_stride;

  // ---- query operand: lane (n = head, g) holds q[head][dh*kPart + 16ks + 8g .. +7]; its loads go out
  //      right behind the id loads below and are back by the time the row pointer table is built
  const int head = hb * 64 + hg * 32 + n;
  const bool q_live = head < a.n_heads;
  const int64_t qoff = (int64_t)b * a.q_batch_stride + (int64_t)t * a.q_token_stride +
                       (int64_t)(q_live ? head : 0) * a.q_head_stride + dh * G::kPart + 8 * g;
  u32x4_t qf[G::kSteps];
  f32x4_t qraw32[QDT == MSPR_F32 ? G::kSteps : 1][2];
  // The gathered ids of this thread's slots are requested before anything else: ids -> row pointers ->
  // rows is the longest dependency chain of the prologue. Local slot ls = tid + 512 j of the range.
  int my_id[G::kMaxIds / kThreads];
#pragma unroll
  for (int j = 0; j < G::kMaxIds / kThreads; j++) {
    const int ls = tid + kThreads * j;
    const int gi = g0 + ls - g_ls0;
    my_id[j] = (ls >= g_ls0 && gi < g1) ? idx_b[gi] : -1;
  }
  if constexpr (QDT == MSPR_F32) {
    const float* qp = reinterpret_cast<const float*>(a.q) + qoff;
#pragma unroll
    for (int ks = 0; ks < G::kSteps; ks++) {
      qraw32[ks][0] = *reinterpret_cast<const f32x4_t*>(qp + 16 * ks);
      qraw32[ks][1] = *reinterpret_cast<const f32x4_t*>(qp + 16 * ks + 4);
    }
  } else {
    const uint16_t* qp = reinterpret_cast<const uint16_t*>(a.q) + qoff;
#pragma unroll
    for (int ks = 0; ks < G::kSteps; ks++) qf[ks] = *reinterpret_cast<const u32x4_t*>(qp + 16 * ks);
  }

  // ---- static part of this thread's tile loads: LDS slot P = tid + 512 j holds (row P / kSlots, chunk P % kSlots)
  uint32_t pk[G::kPerThread];
#pragma unroll
  for (int j = 0; j < G::kPerThread; j++) {
    const int P = tid + kThreads * j;
    const int row = P / G::kSlots, chunk = P % G::kSlots;
    pk[j] = (P < G::kTileSlots && chunk != G::kSlots - 1) ? ((uint32_t)row << 16) | (uint32_t)(chunk * 16) : 0xFFFFFFFFu;
  }
  const uint64_t zero_row = reinterpret_cast<uint64_t>(&g_zero_row[0]);
  // asynchronous loads of one tile straight into its LDS ring buffer: source addresses first (LDS
  // reads of the row pointers), then one 1 KB copy per call of issue_one
  auto tile_sources = [&](int tile, uint64_t (&src)[G::kPerThread]) {
    const uint64_t* rp = rowptr + tile * kTile;
#pragma unroll
    for (int j = 0; j < G::kPerThread; j++) {
      const uint32_t p = pk[j];
      const bool act = p != 0xFFFFFFFFu;
      // lanes of the padding slot fetch a harmless duplicate so that every load is fully active
      src[j] = rp[act ? (p >> 16) : 0] + (act ? (p & 0xFFFFu) : 0u);
    }
  };
  auto tile_lds_base = [&](int tile) -> uint32_t {
    return __builtin_amdgcn_readfirstlane(
        (uint32_t)(size_t)MSPR_LDS_PTR(unsigned char, kbuf + (tile % G::kBufs) * G::kTileBytes + wave * 1024));
  };
  auto issue_one = [&](const uint64_t (&src)[G::kPerThread], uint32_t dst_lds, int j) {
    if (j < G::kPerThread - 1 || wave < G::kLastWaves) async_load_16(src[j], dst_lds + j * (kWaves * 1024));
  };
  auto issue_tile = [&](int tile) {
    uint64_t src[G::kPerThread];
    tile_sources(tile, src);
    const uint32_t dst_lds = tile_lds_base(tile);
#pragma unroll
    for (int j = 0; j < G::kPerThread; j++) issue_one(src, dst_lds, j);
  };

  // ---- row pointer and validity of the window slots (ring rows, or the substituted row); skipped slots
  //      point at a zero row so that every tile load stays fully active. The first window tiles are
  //      requested at once.
  if (wt > 0) {
    const int subst_slot = a.subst_from_params ? a.params[1] : a.subst_slot;
#pragma unroll
    for (int tj = 0; tj < G::kMaxIds / kThreads; tj++) {
      if (tj * kThreads >= g_ls0) break;
      const int ls = tj * kThreads + tid;  // (the bound is a multiple of 32: whole waves or half waves run)
      const int slot = w0 + ls;
      const bool valid = ls < g_ls0 && slot < w1;
      uint64_t ptr = zero_row;
      if (valid) {
        if (slot == subst_slot) {
          ptr = reinterpret_cast<uint64_t>(a.subst_row);
        } else {
          // (raw_start and first + slot are both below raw_cap)
          uint32_t r = (uint32_t)a.raw_start + (uint32_t)seq_win_first + (uint32_t)slot;
          if (r >= (uint32_t)a.raw_cap) r -= (uint32_t)a.raw_cap;
          ptr = reinterpret_cast<uint64_t>(win_b + (int64_t)r * DK);
        }
      }
      const uint64_t bal = __ballot(valid);
      if (ls < g_ls0) {
        rowptr[ls] = ptr;
        if ((lane & 31) == 0) vmask[ls >> 5] = (uint32_t)(bal >> (lane & 32));
      }
    }
    lds_barrier();
    issue_tile(0);
    if (wt > 1) issue_tile(1);
  }

  // ---- stop position of the gathered walk, rope table
  if (ROPE && tid < 32) {
    float theta = (float)a.params[0] * a.inv_freq[tid];
    rope_c[tid] = f16_bits_to_f32(f32_to_f16_bits((float)cos((double)theta)));
    rope_s[tid] = f16_bits_to_f32(f32_to_f16_bits((float)sin((double)theta)));
  }
  int stop_pos = a.n_idx;
  if (a.check_stop) {
    if (tid == 0) *stop_shared = a.n_idx;
    __syncthreads();
    int first = a.n_idx;
    for (int i = tid; i < a.n_idx; i += kThreads) {
      int id = idx_b[i];
      if (id >= 0 && (int64_t)id >= seq_visible && i < first) first = i;
    }
    if (first < a.n_idx) atomicMin(stop_shared, first);
    __syncthreads();
    stop_pos = *stop_shared;
  }

  // ---- row pointer and validity of the gathered slots, by all threads at once
  int64_t n_pool = a.n_pool;
  if (a.pool_rows_dev) {
    const int64_t in_use = a.pool_rows_dev[0];
    n_pool = in_use < n_pool ? (in_use > 0 ? in_use : 0) : n_pool;
  }
#pragma unroll
  for (int tj = 0; tj < G::kMaxIds / kThreads; tj++) {
    if (tj * kThreads >= n_tiles * kTile) break;
    const int ls = tj * kThreads + tid;
    const int gi = g0 + ls - g_ls0;  // index into the gathered id list
    uint64_t ptr = zero_row;
    bool valid = false;
    if (ls >= g_ls0 && gi < g1) {
      const int id = gi < stop_pos ? my_id[tj] : -1;
      if (id >= 0) {
        const int64_t r = (int64_t)id * a.row_mul + a.row_add;
        if (r >= 0 && r < n_pool) {
          valid = true;
          ptr = reinterpret_cast<uint64_t>(pool_b + r * DK);
        }
      }
    }
    const uint64_t bal = __ballot(valid);
    if (ls >= g_ls0 && ls < n_tiles * kTile) {
      rowptr[ls] = ptr;
      if ((lane & 31) == 0) vmask[ls >> 5] = (uint32_t)(bal >> (lane & 32));
    }
  }
  __syncthreads();  // row pointer table visible
  // The query loads (issued long ago) must be complete before the next asynchronous tile load goes
  // out: a wait left for their first use would otherwise also wait for (drain) the tile loads behind them.
  if constexpr (QDT == MSPR_F32) {
#pragma unroll
    for (int ks = 0; ks < G::kSteps; ks++) asm volatile("" : "+v"(qraw32[ks][0]), "+v"(qraw32[ks][1]));
  } else {
#pragma unroll
    for (int ks = 0; ks < G::kSteps; ks++) asm volatile("" : "+v"(qf[ks]));
  }
  // two tiles are in flight when the tile loop starts
  if (wt < 1 && n_tiles > 0) issue_tile(0);
  if (wt < 2 && n_tiles > 1) issue_tile(1);

  // ---- finish the query operand (type conversion, rope) while the first tiles are in flight
  if constexpr (QDT == kQSame && !ROPE) {
    if (!q_live) {
#pragma unroll
      for (int ks = 0; ks < G::kSteps; ks++) qf[ks] = u32x4_t{0u, 0u, 0u, 0u};
    }
  } else {
#pragma unroll
    for (int ks = 0; ks < G::kSteps; ks++) {
      float v[8];
      if constexpr (QDT == MSPR_F32) {
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = round_to_kdt<KDT>(qraw32[ks][j >> 2][j & 3]);
      } else {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          v[2 * j] = unpack_lo<KDT>(qf[ks][j]);
          v[2 * j + 1] = unpack_hi<KDT>(qf[ks][j]);
        }
      }
      const int d0 = dh * G::kPart + 16 * ks + 8 * g;
      if (ROPE && d0 >= DK - 64) {
        // partial rope on interleaved pairs with every product and sum rounded to the element type
#pragma unroll
        for (int j = 0; j < 4; j++) {
          int p = (d0 - (DK - 64)) / 2 + j;
          float c = rope_c[p], s = rope_s[p];
          float x0 = v[2 * j], x1 = v[2 * j + 1];
          float m0 = round_to_kdt<KDT>(x0 * c), m1 = round_to_kdt<KDT>(x1 * s);
          float m2 = round_to_kdt<KDT>(x0 * s), m3 = round_to_kdt<KDT>(x1 * c);
          v[2 * j] = round_to_kdt<KDT>(m0 - m1);
          v[2 * j + 1] = round_to_kdt<KDT>(m2 + m3);
        }
      }
      qf[ks] = q_live ? u32x4_t{pack2<KDT>(v[0], v[1]), pack2<KDT>(v[2], v[3]), pack2<KDT>(v[4], v[5]),
                                 pack2<KDT>(v[6], v[7])}
                      : u32x4_t{0u, 0u, 0u, 0u};
    }
  }

  f32x16_t oacc[4];
#pragma unroll
  for (int mt = 0; mt < 4; mt++) oacc[mt] = f32x16_t{0};
  // m_run is a lazily updated reference maximum: it only moves when a tile's maximum exceeds it by
  // more than kGrow (log2 units), so the 128 accumulator registers are rescaled a few times per kernel
  // instead of once per tile.
  float m_run = -__builtin_inff();
  float l_run = 0.0f;

  // per-lane LDS offsets
  const int a_row_off = n * G::kPitch + (dh * G::kPart + 8 * g) * 2;  // QK^T A operand
  const int tr_s = lane & 15;
  const int tr_off = (4 * g + (tr_s >> 2)) * G::kPitch + (dh * 128 + 16 * ((lane >> 4) & 1) + 4 * (tr_s & 3)) * 2;

  for (int t = 0; t < n_tiles; t++) {
    // tile t+2 goes into the ring buffer of tile t-1, which every wave has left after the barrier
    // below; its copies are issued between the matrix-core instructions of this tile, so that the time
    // a copy waits for the address unit is covered by MFMAs already in flight. The source addresses
    // (reads of the static row pointer table) are worked out before the wait, in its shadow.
    const bool more = t + 2 < n_tiles;  // workgroup-uniform
    uint64_t nsrc[G::kPerThread];
    uint32_t ndst = 0;
    if (more) {
      tile_sources(t + 2, nsrc);
      ndst = tile_lds_base(t + 2);
    }
    // tile t has landed once this wave's loads of it are done and every wave got here
    if (t + 1 < n_tiles) {
      if (wave < G::kLastWaves) wait_vm_and_barrier<G::kPerThread>();
      else wait_vm_and_barrier<G::kPerThread - 1>();
    } else {
      wait_vm_and_barrier<0>();
    }
    const int buf = t % G::kBufs;
    const unsigned char* kt = kbuf + buf * G::kTileBytes;
    const uint32_t mask_all = vmask[t];

    // S^T partial over this wave's half of the row width
    // (two accumulators, even and odd k-steps: a single chain of dependent MFMAs runs about a tenth
    // below the issue rate of independent ones)
    f32x16_t sacc = {0};
    {
      f32x16_t sodd = {0};
      constexpr int kAhead = 6;  // LDS reads in flight in front of the MFMA chains
      u32x4_t af[kAhead];
#pragma unroll
      for (int ks = 0; ks < kAhead; ks++) af[ks] = *reinterpret_cast<const u32x4_t*>(kt + a_row_off + ks * 32);
#pragma unroll
      for (int ks = 0; ks < G::kSteps; ks++) {
        u32x4_t cur = af[ks % kAhead];
        if (ks + kAhead < G::kSteps)
          af[ks % kAhead] = *reinterpret_cast<const u32x4_t*>(kt + a_row_off + (ks + kAhead) * 32);
        if (ks & 1) sodd = mfma32<KDT>(cur, qf[ks], sodd);
        else sacc = mfma32<KDT>(cur, qf[ks], sacc);
        if (more && (ks & 1) == 0 && ks / 2 < G::kPerThread) {
          issue_one(nsrc, ndst, ks / 2);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      sacc = sacc + sodd;
    }
    if (more) {
#pragma unroll
      for (int j = (G::kSteps + 1) / 2; j < G::kPerThread; j++) issue_one(nsrc, ndst, j);
    }
    // the four partial S^T of a head group meet in LDS; every wave adds them in the same order, so the
    // four waves hold bit-identical scores (one buffer is enough: the barrier at the top of the loop
    // separates these reads from the next tile's writes)
    float* sxw = sx + wave * (16 * 64);
#pragma unroll
    for (int c = 0; c < 4; c++)
      *reinterpret_cast<f32x4_t*>(sxw + (c * 64 + lane) * 4) =
          f32x4_t{sacc[4 * c], sacc[4 * c + 1], sacc[4 * c + 2], sacc[4 * c + 3]};
    lds_barrier();
    {
      const float* sxp = sx + (hg * 4) * (16 * 64);
      f32x4_t part[4][4];
#pragma unroll
      for (int d = 0; d < 4; d++)
#pragma unroll
        for (int c = 0; c < 4; c++)
          part[d][c] = *reinterpret_cast<const f32x4_t*>(sxp + d * (16 * 64) + (c * 64 + lane) * 4);
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const f32x4_t o = ((part[0][c] + part[1][c]) + part[2][c]) + part[3][c];
        sacc[4 * c] = o.x;
        sacc[4 * c + 1] = o.y;
        sacc[4 * c + 2] = o.z;
        sacc[4 * c + 3] = o.w;
      }
    }

    // online softmax in the log2 domain; key of register i is 8*(i/4) + 4g + i%4
    float tmax = -__builtin_inff();
    if (mask_all == 0xFFFFFFFFu) {
#pragma unroll
      for (int i = 0; i < 16; i++) {
        sacc[i] *= a.scale_log2;
        tmax = fmaxf(tmax, sacc[i]);
      }
    } else {
      const uint32_t mask = mask_all >> (4 * g);
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const bool valid = (mask >> (8 * (i / 4) + (i % 4))) & 1u;
        sacc[i] = valid ? sacc[i] * a.scale_log2 : -__builtin_inff();
        tmax = fmaxf(tmax, sacc[i]);
      }
    }
    tmax = half_wave_max(tmax);
    // bf16 weights keep float32's exponent range, float16 weights must stay below 2^15
    constexpr float kGrow = KDT == MSPR_BF16 ? 64.0f : 8.0f;
    const bool grow = tmax > m_run + kGrow;
    if (__any(grow)) {
      const bool fresh = __all(m_run == -__builtin_inff());  // nothing accumulated yet
      const float m_new = grow ? tmax : m_run;
      const float alpha = grow ? fast_exp2(m_run - m_new) : 1.0f;
      l_run *= alpha;
      m_run = m_new;
      if (!fresh) {
#pragma unroll
        for (int mt = 0; mt < 4; mt++) oacc[mt] = oacc[mt] * alpha;
      }
    }
    const float m_safe = m_run == -__builtin_inff() ? 0.0f : m_run;
    float psum = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      sacc[i] = fast_exp2(sacc[i] - m_safe);
      psum += sacc[i];
    }
    l_run += psum;
    u32x4_t pf[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
      pf[ks] = u32x4_t{pack2<KDT>(sacc[8 * ks], sacc[8 * ks + 1]), pack2<KDT>(sacc[8 * ks + 2], sacc[8 * ks + 3]),
                       pack2<KDT>(sacc[8 * ks + 4], sacc[8 * ks + 5]), pack2<KDT>(sacc[8 * ks + 6], sacc[8 * ks + 7])};

    // O^T += V^T . P^T ; V^T operands through the LDS transpose read of the row-major tile
    // (k-step outer, output tile inner: consecutive MFMAs never share an accumulator)
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
#pragma unroll
      for (int mt = 0; mt < 4; mt++) {
        const unsigned char* base = kt + tr_off + (16 * ks) * G::kPitch + mt * 64;
        s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(MSPR_LDS_PTR(s16x4_t, base));
        s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(MSPR_LDS_PTR(s16x4_t, base + 8 * G::kPitch));
        u32x2_t lo2 = __builtin_bit_cast(u32x2_t, lo), hi2 = __builtin_bit_cast(u32x2_t, hi);
        oacc[mt] = mfma32<KDT>(u32x4_t{lo2.x, lo2.y, hi2.x, hi2.y}, pf[ks], oacc[mt]);
      }
    }
  }

  float l_tot = l_run + __shfl_xor(l_run, 32, MSPR_WAVE);
  if (a.direct) {
    // ---- the only key range of this sequence: sink, normalise, store
    const float sink = q_live ? load_sink_log2(a, head) : -__builtin_inff();
    const float m_all = fmaxf(m_run, sink);
    const float m_safe = m_all == -__builtin_inff() ? 0.0f : m_all;
    const float w = fast_exp2(m_run - m_safe);
    const float l = l_tot * w + fast_exp2(sink - m_safe);
    const float f = l == 0.0f ? 0.0f : w / l;
    if (q_live) {
      const int64_t obase = (int64_t)b * a.out_batch_stride + (int64_t)t * a.out_token_stride +
                            (int64_t)head * a.out_head_stride;
#pragma unroll
      for (int mt = 0; mt < 4; mt++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
          const float r[4] = {oacc[mt][4 * c] * f, oacc[mt][4 * c + 1] * f, oacc[mt][4 * c + 2] * f,
                              oacc[mt][4 * c + 3] * f};
          const int dim0 = dh * 128 + 32 * mt + 8 * c + 4 * g;
          if (a.out_dtype == MSPR_F32) emit_output<MSPR_F32>(a, r, obase + dim0, dim0);
          else if (a.out_dtype == MSPR_BF16) emit_output<MSPR_BF16>(a, r, obase + dim0, dim0);
          else emit_output<MSPR_F16>(a, r, obase + dim0, dim0);
        }
    }
    return;
  }
  // ---- partial results: registers go out in their native order (coalesced), stats per head. A
  // partial row is stored normalised by its own denominator, so it is a convex combination of V rows
  // and fits float16 whenever V does; with bf16 V it saturates at the float16 range instead of
  // overflowing. Its rounding (2^-11 relative) stays below the rounding of the final output.
  const int64_t part = ((int64_t)(seq * a.n_hblk + hb) * a.n_splits + sp);
  uint16_t* wo = a.ws_o + (part * kWaves + wave) * (int64_t)(4 * 16 * 64);
  const float inv_l = l_tot == 0.0f ? 0.0f : 1.0f / l_tot;
#pragma unroll
  for (int mt = 0; mt < 4; mt++)
#pragma unroll
    for (int c = 0; c < 4; c += 2) {
      uint32_t w[4];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        float x = oacc[mt][4 * c + 2 * j] * inv_l, y = oacc[mt][4 * c + 2 * j + 1] * inv_l;
        if constexpr (KDT == MSPR_BF16) {
          x = __builtin_amdgcn_fmed3f(x, -65504.0f, 65504.0f);
          y = __builtin_amdgcn_fmed3f(y, -65504.0f, 65504.0f);
        }
        w[j] = pack2<MSPR_F16>(x, y);
      }
      // registers 4c..4c+7 of this lane: 16 bytes, lane-contiguous
      *reinterpret_cast<u32x4_t*>(wo + ((mt * 2 + c / 2) * 64 + lane) * 8) = u32x4_t{w[0], w[1], w[2], w[3]};
    }
  if (dh == 0 && g == 0) {
    float* ml = a.ws_ml + (part * 64 + hg * 32 + n) * 2;
    ml[0] = m_run;
    ml[1] = l_tot;
  }

}

// Merge of the per-split partials: one workgroup per (batch, head block, wave slot, 32-column tile).
// ---------------------------------------------------------------------------------------------------
// Prefill consumer: many query tokens against one ring of raw rows and one pool (float16 rows of 512).
//
// A workgroup is persistent: it takes every gridDim.x-th (token, head block) unit and runs their 32-slot
// tiles as one stream through a ring of four tile buffers, so that the first rows of the next token are
// requested while the last tiles of the current one are multiplied. What a token needs before its first
// tile (ids -> stop position -> row pointers; its query rows) is produced inside the tile loop of the token
// before it: ids are requested at tile 0, the row pointer table is written at tile 1 into the other of
// two table slots, the query operand is requested once the last S^T product of the current token has run.
// Every token runs at least kMinTiles tiles (the missing ones are fully masked), which is what makes those
// positions exist.
//
// The tile step differs from the split kernel's: no wave splits a contraction, so no partial sums are
// exchanged. For S^T = K.Q^T the 32 keys x 64 heads of a tile are eight 16 x 16 blocks, one per wave
// (v_mfma_f32_16x16x32_f16 over the whole row width, the query block of 16 heads in 64 registers); a wave
// takes the exponentials of its block and writes them as P^T in the element type. For O^T = V^T.P^T a wave
// owns 32 heads x 128 output columns as in the split kernel and reads the P^T of its heads from LDS. One
// barrier per tile (P^T written). The running maximum of a head has to be the same in every wave that
// touches it: a wave uses the common value as it is, and raises a flag if one of its keys exceeds it by more
// than kGrow; on a flagged tile (always the first one of a token, rarely another) the waves exchange their
// block maxima, rescale, and write P^T again. The matrix work of a step is V^T.P^T of tile s together with
// K.Q^T of tile s+1, in one stretch between two barriers.
//
// Ring: behind barrier C of step s every wave has left the V^T reads of tile s-1, so the copies of tile
// s+3 go into its buffer; every wave waits for its own copies of tile s+1 before C, so tile s+1 is complete
// when K.Q^T of it starts.
//
// Vector-memory waits. The tile copies, the id fetches and the cache warm-up of the query rows are asynchronous
// global -> LDS copies issued through asm: they write no register, so nothing the compiler does with registers
// can meet a load in flight. A wave counts them as it issues them (`issued`) and remembers the count behind each
// request (a mark); "this request has landed" is s_waitcnt vmcnt(issued - mark), since a wave's vector-memory
// operations complete in the order issued. Everything else (query rows, the sink, the output stores) is an
// ordinary load or store that the compiler sees and waits for itself; the query rows are forced complete at a
// chosen place by an empty asm statement that names their registers. Operations the count leaves out only make
// a wait longer, never shorter; the output stores are counted (sixteen per wave) so that the waits of a token's
// first steps do not cover the stores of the token before it.
// ---------------------------------------------------------------------------------------------------
struct PrefillGeometry {
  using G = Geometry<512>;
  static constexpr int kBufs = 4;                         // one tile under V^T.P^T, one under K.Q^T, two in flight
  static constexpr int kSlots = 66;                       // 16-byte slots per LDS row, two of them padding: rows 32
                                                          // bytes apart in the banks serve the 16-row operand
                                                          // reads of K.Q^T and the transpose reads best
  static constexpr int kPitch = kSlots * 16;
  static constexpr int kTileSlots = kTile * kSlots;       // = 33 wave-wide copies exactly
  static constexpr int kMaxTiles = 22;                    // 704 slots per token
  static constexpr int kMinTiles = 5;
  static constexpr int kTableSlots = kMaxTiles * kTile;
  static constexpr int kQSteps = 512 / 32;                // MFMAs of one 16 x 16 block of S^T
  static constexpr int kPPitch = 80;                      // bytes per head of P^T: 32 keys + 16 B, so that the
                                                          // heads of a read phase start on distinct banks
  static constexpr int kOffTable = kBufs * G::kTileBytes;            // [2][kTableSlots] row pointers
  static constexpr int kOffVmask = kOffTable + 2 * kTableSlots * 8;  // [2][32] validity word per tile
  static constexpr int kOffP = kOffVmask + 2 * 32 * 4;               // [2 steps][64 heads][kPPitch]
  static constexpr int kOffTmax = kOffP + 2 * 64 * kPPitch;          // [8 waves][16 heads] float
  static constexpr int kOffL = kOffTmax + kWaves * 16 * 4;           // [8 waves][16 heads] float
  static constexpr int kOffIds = kOffL + kWaves * 16 * 4;            // [2][512] ids of the unit in preparation
  static constexpr int kOffFlag = kOffIds + 2 * kThreads * 4;        // flag[2], stop[2]
  static constexpr int kOffWarm = kOffFlag + 16;                     // [64 lanes] dwords nobody reads (every wave's)
  static constexpr int kLdsBytes = kOffWarm + 256;
  static_assert(kTileSlots == G::kInstr * 64 && kOffTable % 16 == 0 && kOffP % 16 == 0 && kOffIds % 16 == 0 &&
                    kLdsBytes <= 160 * 1024,
                "LDS map of the prefill consumer");
};

__device__ __forceinline__ f32x4_t mfma16_f16(u32x4_t a, u32x4_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0,
                                                0);
}

// s_waitcnt vmcnt(n') with the largest n' <= n of a few levels, for a wave-uniform n: at most n' of this wave's
// vector-memory operations stay in flight (waiting for more than asked is always allowed). The levels are the counts
// the prefill consumer meets: 4 or 5 (a wave's copies of one tile, every step of the steady state), 6 (with the
// warm-up dword or the two id requests on top), 20 and above (with the sixteen output stores of the unit before).
// A ladder of scalar compares, the common counts first: a switch over every count compiles into a chain of some
// forty guarded blocks that a wave walks through on each wait.
__device__ __forceinline__ void wait_vm_dyn(int n) {
  n = __builtin_amdgcn_readfirstlane(n);  // (the same in every lane: keeps the selection on the scalar unit)
  if (n == 5) asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
  else if (n == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
  else if (n >= 20) asm volatile("s_waitcnt vmcnt(20)" ::: "memory");
  else if (n >= 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

struct PrefillUnit {
  int b, t, hb, seq;
  int n_win, win_first, wt;  // ring rows of the token's window, first of them (logical), their tiles
  int64_t visible;
};

__global__ __launch_bounds__(kThreads, 1) void sparse_attn_prefill_kernel(SparseAttnArgs a) {
  constexpr int KDT = MSPR_F16;
  constexpr int DK = 512;
  using G = Geometry<DK>;
  using PG = PrefillGeometry;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  unsigned char* kbuf = lds;
  uint64_t* table = reinterpret_cast<uint64_t*>(lds + PG::kOffTable);
  uint32_t* vmask = reinterpret_cast<uint32_t*>(lds + PG::kOffVmask);
  float* tmaxbuf = reinterpret_cast<float*>(lds + PG::kOffTmax);
  float* lbuf = reinterpret_cast<float*>(lds + PG::kOffL);
  int* flag = reinterpret_cast<int*>(lds + PG::kOffFlag);
  int* stop_sh = flag + 2;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // (uniform: what is derived from it stays scalar)
  // O^T = V^T.P^T: wave = (head group of 32, quarter of the output columns), lane = (head n, half g)
  const int hg = wave >> 2;
  const int dh = wave & 3;
  const int n = lane & 31;
  const int g = lane >> 5;
  // S^T = K.Q^T: wave = (key half, head quarter), lane = (row / column c16 of the block, k group kg)
  const int kh = wave & 1;
  const int hq = wave >> 1;
  const int c16 = lane & 15;
  const int kg = lane >> 4;
  unsigned char* p_wr = lds + PG::kOffP + (16 * hq + c16) * PG::kPPitch + 32 * kh + 8 * kg;  // keys 16 kh + 4 kg ..
  const unsigned char* p_rd = lds + PG::kOffP + (32 * hg + n) * PG::kPPitch + 8 * g;
  const int tmax_rd = (2 * (2 * hg + (n >> 4))) * 16 + (n & 15);  // first of the two blocks that hold head 32 hg + n
  const int k_mine = wave < G::kLastWaves ? G::kPerThread : G::kPerThread - 1;  // copies of this wave per tile
  // this wave's asynchronous copies, counted as they are issued; a mark is the count right behind a request
  int issued = 0;
  int mark_t0 = 0, mark_t1 = 0, mark_t2 = 0, mark_t3 = 0, mark_ids = 0;

  const int n_units = a.batch * a.n_hblk;
  const int stride = (int)gridDim.x;
  int unit = (int)blockIdx.x;
  if (unit >= n_units) return;

  auto div_by = [](uint32_t x, uint32_t n, uint32_t inv) -> uint32_t {
    if (n == 1u) return x;
    uint32_t q = __umulhi(x, inv);
    if (x - q * n >= n) q++;
    return q;
  };
  auto unit_of = [&](int u) -> PrefillUnit {
    PrefillUnit m;
    m.seq = (int)div_by((uint32_t)u, (uint32_t)a.n_hblk, a.inv_hblk);
    m.hb = u - m.seq * a.n_hblk;
    m.b = (int)div_by((uint32_t)m.seq, (uint32_t)a.n_tokens, a.inv_tokens);
    m.t = m.seq - m.b * a.n_tokens;
    // window rows and visible pool prefix, in the unsigned 32-bit arithmetic of the reference kernel
    const uint32_t qpos = a.pos0 + (uint32_t)m.t, n_raw = (uint32_t)a.raw_cap;
    const uint32_t last_pos = a.pos0 + (uint32_t)a.n_tokens - 1u;
    const uint32_t first_raw_pos = last_pos + 1u - n_raw;
    const uint32_t window_first = (a.window != 0u && qpos + 1u > a.window) ? qpos + 1u - a.window : 0u;
    const uint32_t first = first_raw_pos > window_first ? first_raw_pos : window_first;
    const uint32_t last = qpos < last_pos ? qpos : last_pos;
    m.n_win = first <= last ? (int)(last - first + 1u) : 0;
    if (m.n_win > a.n_win) m.n_win = a.n_win;
    m.win_first = first <= last ? (int)(first - first_raw_pos) : 0;
    const int64_t vis = a.ratio == 0u ? a.n_pool : (int64_t)((qpos + 1u) / a.ratio);
    m.visible = vis < a.n_pool ? vis : a.n_pool;
    m.wt = (m.n_win + kTile - 1) / kTile;
    return m;
  };
  auto tiles_of = [&](const PrefillUnit& m, int stop_pos) -> int {
    const int nt = m.wt + (stop_pos + kTile - 1) / kTile;
    return nt < PG::kMinTiles ? PG::kMinTiles : nt;
  };
  // ids of this thread's two table slots (slot ls = tid + 512 j; gathered part starts at slot 32 wt), fetched
  // straight into LDS: always two copies with every lane active, index clamped. A wave reads back only what it
  // fetched itself, so its own wait is all that stands between the request and the read.
  const int* ids_lds = reinterpret_cast<const int*>(lds + PG::kOffIds);
  const uint32_t ids_lds_wave = __builtin_amdgcn_readfirstlane(
      (uint32_t)(size_t)MSPR_LDS_PTR(unsigned char, lds + PG::kOffIds + wave * 256));
  auto request_ids = [&](const PrefillUnit& m) {
    const int32_t* idx_b = a.idx + (int64_t)m.seq * a.idx_batch_stride;
#pragma unroll
    for (int j = 0; j < 2; j++) {
      int gi = tid + kThreads * j - m.wt * kTile;
      gi = gi < 0 ? 0 : (gi >= a.n_idx ? a.n_idx - 1 : gi);
      const int32_t* p = idx_b + gi;
      // lane i's dword lands at ids_lds[64 wave + 512 j + i] = ids_lds[tid + 512 j]
      asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dword %0, off" ::"v"(p), "s"(ids_lds_wave + j * (kThreads * 4))
                   : "memory", "m0");
    }
    issued += 2;
    mark_ids = issued;
  };
  auto await_ids = [&](int (&ids)[2]) {
    wait_vm_dyn(issued - mark_ids);
    ids[0] = ids_lds[tid];
    ids[1] = ids_lds[tid + kThreads];
  };
  // position of the first id that ends the walk (>= the visible prefix), minimum over the workgroup
  auto scan_stop = [&](const PrefillUnit& m, const int (&ids)[2], int* stop) {
    int first = a.n_idx;
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const int gi = tid + kThreads * j - m.wt * kTile;
      if (gi >= 0 && gi < a.n_idx && ids[j] >= 0 && (int64_t)ids[j] >= m.visible && gi < first) first = gi;
    }
    if (first < a.n_idx) atomicMin(stop, first);
  };
  const uint64_t zero_row = reinterpret_cast<uint64_t>(&g_zero_row[0]);
  auto build_table = [&](const PrefillUnit& m, int slot, const int (&ids)[2], int stop_pos, int n_tiles) {
    const uint16_t* win_b = reinterpret_cast<const uint16_t*>(a.win) + (int64_t)m.b * a.win_batch_stride;
    const uint16_t* pool_b = reinterpret_cast<const uint16_t*>(a.pool) + (int64_t)m.b * a.pool_batch_stride;
    const int g_ls0 = m.wt * kTile;
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const int ls = tid + kThreads * j;
      uint64_t ptr = zero_row;
      bool valid = false;
      if (ls < g_ls0) {
        if (ls < m.n_win) {
          uint32_t r = (uint32_t)a.raw_start + (uint32_t)m.win_first + (uint32_t)ls;
          if (r >= (uint32_t)a.raw_cap) r -= (uint32_t)a.raw_cap;
          valid = true;
          ptr = reinterpret_cast<uint64_t>(win_b + (int64_t)r * DK);
        }
      } else {
        const int gi = ls - g_ls0;
        const int id = gi < stop_pos ? ids[j] : -1;
        if (id >= 0) {
          const int64_t r = (int64_t)id * a.row_mul + a.row_add;
          if (r >= 0 && r < a.n_pool) {
            valid = true;
            ptr = reinterpret_cast<uint64_t>(pool_b + r * DK);
          }
        }
      }
      const uint64_t bal = __ballot(valid);
      if (ls < n_tiles * kTile) {  // (a multiple of 32: whole or half waves)
        table[slot * PG::kTableSlots + ls] = ptr;
        if ((lane & 31) == 0) vmask[slot * 32 + (ls >> 5)] = (uint32_t)(bal >> (lane & 32));
      }
    }
  };

  // ---- tile copies (as in the split kernel): LDS slot P = tid + 512 j holds (row P / kSlots, chunk P % kSlots)
  uint32_t pk[G::kPerThread];
#pragma unroll
  for (int j = 0; j < G::kPerThread; j++) {
    const int P = tid + kThreads * j;
    const int row = P / PG::kSlots, chunk = P % PG::kSlots;
    pk[j] = (P < PG::kTileSlots && chunk < 64) ? ((uint32_t)row << 16) | (uint32_t)(chunk * 16) : 0xFFFFFFFFu;
  }
  // source address of each of this thread's 16-byte slots of a tile, from the row pointer table
  auto tile_sources = [&](int slot, int tile, uint64_t (&src)[G::kPerThread]) {
    const uint64_t* rp = table + slot * PG::kTableSlots + tile * kTile;
#pragma unroll
    for (int j = 0; j < G::kPerThread; j++) {
      const uint32_t p = pk[j];
      const bool act = p != 0xFFFFFFFFu;
      src[j] = rp[act ? (p >> 16) : 0] + (act ? (p & 0xFFFFu) : 0u);
    }
  };
  auto issue_copies = [&](const uint64_t (&src)[G::kPerThread], int flat) {
    const int buf = flat & (PG::kBufs - 1);
    const uint32_t dst_lds = __builtin_amdgcn_readfirstlane(
        (uint32_t)(size_t)MSPR_LDS_PTR(unsigned char, kbuf + buf * G::kTileBytes + wave * 1024));
#pragma unroll
    for (int j = 0; j < G::kPerThread; j++)
      if (j < G::kPerThread - 1 || wave < G::kLastWaves) async_load_16(src[j], dst_lds + j * (kWaves * 1024));
    issued += k_mine;
    mark_t0 = buf == 0 ? issued : mark_t0;
    mark_t1 = buf == 1 ? issued : mark_t1;
    mark_t2 = buf == 2 ? issued : mark_t2;
    mark_t3 = buf == 3 ? issued : mark_t3;
  };
  auto copy_tile = [&](int slot, int tile, int flat) {
    uint64_t src[G::kPerThread];
    tile_sources(slot, tile, src);
    issue_copies(src, flat);
  };
  static_assert(PG::kBufs == 4, "ring index by mask");
  // this wave's copies of flat tile j have landed
  auto await_tile = [&](int flat) {
    const int buf = flat & (PG::kBufs - 1);
    const int mark = buf == 0 ? mark_t0 : (buf == 1 ? mark_t1 : (buf == 2 ? mark_t2 : mark_t3));
    wait_vm_dyn(issued - mark);
  };

  // ---- query operand of a unit: lane (c16 = head of the quarter, kg) holds q[head][32 ks + 8 kg .. +7]
  u32x4_t qf[PG::kQSteps];
  auto request_q = [&](const PrefillUnit& m) {
    const int head = m.hb * 64 + 16 * hq + c16;
    const int64_t qoff = (int64_t)m.b * a.q_batch_stride + (int64_t)m.t * a.q_token_stride +
                         (int64_t)(head < a.n_heads ? head : 0) * a.q_head_stride + 8 * kg;
    const uint16_t* qp = reinterpret_cast<const uint16_t*>(a.q) + qoff;
    // (ordinary loads: the compiler knows these registers are in flight until it has waited for them)
#pragma unroll
    for (int ks = 0; ks < PG::kQSteps; ks++) qf[ks] = *reinterpret_cast<const u32x4_t*>(qp + 32 * ks);
  };
  // one dword of every 128-byte line of a unit's query rows (64 rows of 1 KB), requested long before the rows
  // themselves so that those come out of the L2. The dwords go to LDS nobody reads (the same 256 bytes for
  // every wave).
  const uint32_t warm_lds =
      __builtin_amdgcn_readfirstlane((uint32_t)(size_t)MSPR_LDS_PTR(unsigned char, lds + PG::kOffWarm));
  auto warm_q = [&](const PrefillUnit& m) {
    const int head = m.hb * 64 + (tid >> 3);
    const uint16_t* p = reinterpret_cast<const uint16_t*>(a.q) + (int64_t)m.b * a.q_batch_stride +
                        (int64_t)m.t * a.q_token_stride + (int64_t)(head < a.n_heads ? head : 0) * a.q_head_stride +
                        (tid & 7) * 64;
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dword %0, off" ::"v"(p), "s"(warm_lds) : "memory", "m0");
    issued += 1;
  };
  static_assert(PG::kQSteps == 16, "the query wait below names sixteen registers");
#define MSPR_QF_OPERANDS                                                                                             \
  "+v"(qf[0]), "+v"(qf[1]), "+v"(qf[2]), "+v"(qf[3]), "+v"(qf[4]), "+v"(qf[5]), "+v"(qf[6]), "+v"(qf[7]), "+v"(qf[8]), \
      "+v"(qf[9]), "+v"(qf[10]), "+v"(qf[11]), "+v"(qf[12]), "+v"(qf[13]), "+v"(qf[14]), "+v"(qf[15])
  // The query rows have to be complete here: the statement uses their registers, so the compiler puts its wait
  // in front of it (and not in front of their first use in a matrix instruction, behind tile copies that the
  // wait would then cover too).
  auto await_q = [&]() { asm volatile("" : MSPR_QF_OPERANDS : : "memory"); };
#undef MSPR_QF_OPERANDS
  auto mask_q = [&](const PrefillUnit& m) {
    if (m.hb * 64 + 16 * hq + c16 >= a.n_heads) {
#pragma unroll
      for (int ks = 0; ks < PG::kQSteps; ks++) qf[ks] = u32x4_t{0u, 0u, 0u, 0u};
    }
  };

  // ---- first unit: ids, stop position, table, query, first three tiles
  PrefillUnit cur = unit_of(unit);
  int ids[2] = {-1, -1};
  const bool have_ids = a.n_idx > 0;
  if (have_ids) request_ids(cur);
  request_q(cur);
  if (tid == 0) stop_sh[0] = a.n_idx;
  __syncthreads();
  if (have_ids) {
    await_ids(ids);
    scan_stop(cur, ids, &stop_sh[0]);
  }
  __syncthreads();
  // (read from LDS, the same in every lane: made scalar so that the tile loop's control flow is)
  int n_cur = __builtin_amdgcn_readfirstlane(tiles_of(cur, stop_sh[0]));
  build_table(cur, 0, ids, stop_sh[0], n_cur);
  await_q();
  mask_q(cur);
  // sink of this lane's head (a plain load: its wait would drain the tile copies anywhere behind this point)
  float sink_l2;
  {
    const int head = cur.hb * 64 + hg * 32 + n;
    sink_l2 = head < a.n_heads ? load_sink_log2(a, head) : -__builtin_inff();
    asm volatile("" : "+v"(sink_l2));
  }
  __syncthreads();
  copy_tile(0, 0, 0);
  copy_tile(0, 1, 1);
  copy_tile(0, 2, 2);

  f32x16_t oacc[4];
#pragma unroll
  for (int mt = 0; mt < 4; mt++) oacc[mt] = f32x16_t{0};
  // reference maximum per head, the same in every wave that holds the head: m_qk for head 16 hq + c16 (S^T
  // role), m_pv for head 32 hg + n (O^T role)
  float m_qk = -__builtin_inff(), m_pv = -__builtin_inff();
  float l_qk = 0.0f;  // denominator share of this lane: its head, its four keys of every tile

  const int a_row_off = (16 * kh + c16) * PG::kPitch + 16 * kg;
  const int tr_s = lane & 15;
  const int tr_off = (4 * g + (tr_s >> 2)) * PG::kPitch + (dh * 128 + 16 * ((lane >> 4) & 1) + 4 * (tr_s & 3)) * 2;
  constexpr float kGrow = 8.0f;  // float16 weights stay below 2^15

  // S^T block of one tile
  auto qk_block = [&](const unsigned char* kt) -> f32x4_t {
    f32x4_t se = {0.0f, 0.0f, 0.0f, 0.0f}, so = {0.0f, 0.0f, 0.0f, 0.0f};
    constexpr int kAhead = 6;
    u32x4_t af[kAhead];
#pragma unroll
    for (int ks = 0; ks < kAhead; ks++) af[ks] = *reinterpret_cast<const u32x4_t*>(kt + a_row_off + ks * 64);
#pragma unroll
    for (int ks = 0; ks < PG::kQSteps; ks++) {
      const u32x4_t cur_a = af[ks % kAhead];
      if (ks + kAhead < PG::kQSteps)
        af[ks % kAhead] = *reinterpret_cast<const u32x4_t*>(kt + a_row_off + (ks + kAhead) * 64);
      if (ks & 1) so = mfma16_f16(cur_a, qf[ks], so);
      else se = mfma16_f16(cur_a, qf[ks], se);
    }
    // The operand reads run kAhead steps in front of the matrix instructions that consume them (stated to the
    // scheduler, which otherwise keeps only two reads in flight)
    __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
#pragma unroll
    for (int ks = 0; ks < PG::kQSteps - kAhead; ks++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 0);
    return se + so;
  };

  // O^T += V^T . P^T of flat tile s (P^T of the step is in LDS behind barrier C)
  auto pv_tile = [&](int s) {
    const unsigned char* kt = kbuf + (s % PG::kBufs) * G::kTileBytes;
    const unsigned char* p_rd_s = p_rd + (s & 1) * (64 * PG::kPPitch);
    u32x4_t pf[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
      const u32x2_t lo = *reinterpret_cast<const u32x2_t*>(p_rd_s + 32 * ks);
      const u32x2_t hi = *reinterpret_cast<const u32x2_t*>(p_rd_s + 32 * ks + 16);
      pf[ks] = u32x4_t{lo.x, lo.y, hi.x, hi.y};
    }
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
#pragma unroll
      for (int mt = 0; mt < 4; mt++) {
        const unsigned char* base = kt + tr_off + (16 * ks) * PG::kPitch + mt * 64;
        s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(MSPR_LDS_PTR(s16x4_t, base));
        s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(MSPR_LDS_PTR(s16x4_t, base + 8 * PG::kPitch));
        u32x2_t lo2 = __builtin_bit_cast(u32x2_t, lo), hi2 = __builtin_bit_cast(u32x2_t, hi);
        oacc[mt] = mfma32<KDT>(u32x4_t{lo2.x, lo2.y, hi2.x, hi2.y}, pf[ks], oacc[mt]);
      }
    }
    __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
    for (int i = 0; i < 6; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
  };

  // tile 0 is complete once every wave's copies of it are (the copies of tiles 1 and 2 stay in flight)
  await_tile(0);
  lds_barrier();
  f32x4_t sacc = qk_block(kbuf);

  int s = 0;     // tiles done by this workgroup: ring buffer s % 4, flag and P^T slot s & 1
  int slot = 0;  // table slot of the current unit
  for (;;) {
    const bool have_next = unit + stride < n_units;
    PrefillUnit nxt = cur;
    int n_nxt = 0;
    int nids[2] = {-1, -1};
    if (have_next) nxt = unit_of(unit + stride);

    for (int t = 0; t < n_cur; t++, s++) {
      const bool last = t == n_cur - 1;
      // ---- what the next unit needs, at fixed places of this unit's stream
      if (have_next) {
        if (t == 1 && have_ids) {
          await_ids(nids);  // (requested a step ago; younger: the copies issued behind barrier C of that step)
          scan_stop(nxt, nids, &stop_sh[slot ^ 1]);
        }
        if (t == 0) {
          if (have_ids) request_ids(nxt);
          if (tid == 0) stop_sh[slot ^ 1] = a.n_idx;
        }
        if (t == 2) warm_q(nxt);
      }
      // ---- tile s+3 (of this unit, or one of the first three of the next): its copies go out behind barrier C.
      //      Their source addresses come out of the row pointer table in LDS; they are read here, a softmax and
      //      a barrier ahead of their use - unless the table is the next unit's and was written only a step ago
      //      (t < 3: no barrier has passed since), in which case they are read behind barrier C.
      int la_slot = slot, la_tile = t + 3;
      bool ahead = true;
      if (la_tile >= n_cur) {
        la_slot = slot ^ 1;
        la_tile -= n_cur;
        ahead = have_next;
      }
      const bool early = ahead && (la_slot == slot || t >= 3);
      uint64_t la_src[G::kPerThread];
      if (early) tile_sources(la_slot, la_tile, la_src);
      // ---- softmax weights of this wave's block: head 16 hq + c16, keys 16 kh + 4 kg + i
      float sv[4];
      {
        const uint32_t mbits = vmask[slot * 32 + t] >> (16 * kh + 4 * kg);
        sv[0] = (mbits & 1u) ? sacc[0] * a.scale_log2 : -__builtin_inff();
        sv[1] = (mbits & 2u) ? sacc[1] * a.scale_log2 : -__builtin_inff();
        sv[2] = (mbits & 4u) ? sacc[2] * a.scale_log2 : -__builtin_inff();
        sv[3] = (mbits & 8u) ? sacc[3] * a.scale_log2 : -__builtin_inff();
      }
      const float tloc = half_wave_max(row_pair_max(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]))));
      float pw[4];
      unsigned char* p_wr_s = p_wr + (s & 1) * (64 * PG::kPPitch);
      {
        const float m_safe = m_qk == -__builtin_inff() ? 0.0f : m_qk;
#pragma unroll
        for (int j = 0; j < 4; j++) pw[j] = fast_exp2(sv[j] - m_safe);
        *reinterpret_cast<u32x2_t*>(p_wr_s) = u32x2_t{pack2<KDT>(pw[0], pw[1]), pack2<KDT>(pw[2], pw[3])};
      }
      if (__any(tloc > m_qk + kGrow) && lane == 0) flag[s & 1] = s + 1;
      // tile s+1 complete behind this barrier: every wave waits for its own copies of it, leaving in flight
      // what it has issued since (the copies of tile s+2, ids, the warm-up dword, the stores of the unit before)
      if (!last || have_next) await_tile(s + 1);
      lds_barrier();  // C
      const int flagged = flag[s & 1];  // (requested here, looked at behind the copies: they do not depend on it)
      if (ahead) {
        if (!early) tile_sources(la_slot, la_tile, la_src);
        issue_copies(la_src, s + 3);
      }
      if (__builtin_amdgcn_readfirstlane(flagged) == s + 1) {
        // ---- a key above the common maximum: the waves agree on a new one and write P^T again
        if (kg == 0) tmaxbuf[wave * 16 + c16] = tloc;
        lds_barrier();
        {
          const float tq = fmaxf(tmaxbuf[(2 * hq) * 16 + c16], tmaxbuf[(2 * hq + 1) * 16 + c16]);
          const bool grow = tq > m_qk + kGrow;
          l_qk *= grow ? fast_exp2(m_qk - tq) : 1.0f;
          m_qk = grow ? tq : m_qk;
        }
        {
          const float tp = fmaxf(tmaxbuf[tmax_rd], tmaxbuf[tmax_rd + 16]);
          const bool grow = tp > m_pv + kGrow;
          if (__any(grow)) {
            const float alpha = grow ? fast_exp2(m_pv - tp) : 1.0f;
            m_pv = grow ? tp : m_pv;
#pragma unroll
            for (int mt = 0; mt < 4; mt++) oacc[mt] = oacc[mt] * alpha;
          }
        }
        const float m_safe = m_qk == -__builtin_inff() ? 0.0f : m_qk;
#pragma unroll
        for (int j = 0; j < 4; j++) pw[j] = fast_exp2(sv[j] - m_safe);
        *reinterpret_cast<u32x2_t*>(p_wr_s) = u32x2_t{pack2<KDT>(pw[0], pw[1]), pack2<KDT>(pw[2], pw[3])};
        lds_barrier();
      }
      l_qk += (pw[0] + pw[1]) + (pw[2] + pw[3]);
      if (have_next && t == 1) {
        const int stop_pos = stop_sh[slot ^ 1];
        n_nxt = __builtin_amdgcn_readfirstlane(tiles_of(nxt, stop_pos));
        build_table(nxt, slot ^ 1, nids, stop_pos, n_nxt);
      }
      // ---- O^T += V^T . P^T of tile s, and S^T of tile s+1. (The unit's last tile: behind the loop, with the
      //      request for the next unit's query rows in front of it.)
      if (!last) {
        pv_tile(s);
        sacc = qk_block(kbuf + ((s + 1) % PG::kBufs) * G::kTileBytes);
      }
    }

    // ---- K.Q^T of this unit's last tile ran a step ago, so the query registers are free: the next unit's rows
    //      are requested here and arrive while this unit's output leaves. Request, wait and first use sit in
    //      straight-line code, so no path reaches a use of these registers with the loads in flight.
    if (have_next) request_q(nxt);
    pv_tile(s - 1);
    // ---- end of the unit: the denominators meet, sink, normalise, store
    {
      float l_w = l_qk;
      l_w += __shfl_xor(l_w, 16, MSPR_WAVE);
      l_w += __shfl_xor(l_w, 32, MSPR_WAVE);
      if (kg == 0) lbuf[wave * 16 + c16] = l_w;
      lds_barrier();
      const float l_tot = lbuf[tmax_rd] + lbuf[tmax_rd + 16];
      const int head = cur.hb * 64 + hg * 32 + n;
      const bool q_live = head < a.n_heads;
      const float sink = sink_l2;
      const float m_all = fmaxf(m_pv, sink);
      const float m_safe = m_all == -__builtin_inff() ? 0.0f : m_all;
      const float w = fast_exp2(m_pv - m_safe);
      const float l = l_tot * w + fast_exp2(sink - m_safe);
      const float f = l == 0.0f ? 0.0f : w / l;
      // Sixteen stores per wave, every lane active (a lane without a head stores into g_store_sink), in straight
      // line behind the query request: the compiler's wait for the query rows then leaves exactly these stores in
      // flight (it counts what it issued itself), and the wave's own count of them below is exact.
      float* orow = q_live ? reinterpret_cast<float*>(a.out) + ((int64_t)cur.b * a.out_batch_stride +
                                                                 (int64_t)cur.t * a.out_token_stride +
                                                                 (int64_t)head * a.out_head_stride)
                           : &g_store_sink[lane * 512];
#pragma unroll
      for (int mt = 0; mt < 4; mt++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
          const int dim0 = dh * 128 + 32 * mt + 8 * c + 4 * g;
          *reinterpret_cast<f32x4_t*>(orow + dim0) = f32x4_t{oacc[mt][4 * c] * f, oacc[mt][4 * c + 1] * f,
                                                             oacc[mt][4 * c + 2] * f, oacc[mt][4 * c + 3] * f};
        }
      // The query rows requested above are forced complete on every path out of this block (also when there is
      // no next unit: then nothing is in flight and the statement costs nothing), so that the compiler never
      // sees a path into the tile loop with those loads outstanding.
      await_q();
      issued += 16;
    }
    if (!have_next) break;
    mask_q(nxt);
    unit += stride;
    if (nxt.hb != cur.hb) {  // (more than 64 heads: the wait of this load drains the copies in flight once)
      const int head = nxt.hb * 64 + hg * 32 + n;
      sink_l2 = head < a.n_heads ? load_sink_log2(a, head) : -__builtin_inff();
      asm volatile("" : "+v"(sink_l2));
    }
    cur = nxt;
    n_cur = n_nxt;
    slot ^= 1;
#pragma unroll
    for (int mt = 0; mt < 4; mt++) oacc[mt] = f32x16_t{0};
    m_qk = -__builtin_inff();
    m_pv = -__builtin_inff();
    l_qk = 0.0f;
    // S^T of the unit's first tile (its copies were awaited in the step before)
    sacc = qk_block(kbuf + (s % PG::kBufs) * G::kTileBytes);
  }
}

// Float32 query rows of a prefill chunk rounded to half (nearest even, what the consumer's operand load does to a
// float32 query) into a dense [batch][token][head][512] copy: the persistent consumer keeps the 64 x 512 query
// block of a unit in registers, which holds half-precision rows only. A thread converts eight values.
__global__ __launch_bounds__(256) void prefill_q_to_half_kernel(const float* q, int64_t batch_stride, int64_t head_stride,
                                                                int64_t token_stride, int n_heads, int n_tokens,
                                                                int64_t n_rows, uint16_t* dst) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // (batch, token, head) flattened
  if (row >= n_rows) return;
  const int col = (threadIdx.x & 63) * 8;
  const int64_t bt = row / n_heads;
  const int head = (int)(row - bt * n_heads);
  const int64_t b = bt / n_tokens;
  const int64_t t = bt - b * n_tokens;
  const float* src = q + b * batch_stride + t * token_stride + (int64_t)head * head_stride + col;
  const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(src);
  const f32x4_t hi = *reinterpret_cast<const f32x4_t*>(src + 4);
  *reinterpret_cast<u32x4_t*>(dst + row * 512 + col) = u32x4_t{pack2<MSPR_F16>(lo.x, lo.y), pack2<MSPR_F16>(lo.z, lo.w),
                                                              pack2<MSPR_F16>(hi.x, hi.y), pack2<MSPR_F16>(hi.z, hi.w)};
}

template <int ODT>
__global__ __launch_bounds__(256) void sparse_attn_merge_kernel(SparseAttnArgs a) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int c = tid >> 6;  // accumulator quad: registers 4c..4c+3 (half of a stored group of 8)
  // a sequence's partials are merged on the XCD whose workgroups wrote them (the split kernel's mapping), so
  // that they are read from that XCD's L2
  unsigned work = blockIdx.x;
  if ((gridDim.x & 7u) == 0u) work = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const int mt = work & 3;
  const int wave = (work >> 2) & 7;  // wave of the split kernel whose registers this workgroup merges
  const int bh = work >> 5;
  const int hb = bh % a.n_hblk;
  const int seq = bh / a.n_hblk;
  const int b = seq / a.n_tokens;
  const int t = seq - b * a.n_tokens;
  const int hg = wave >> 2, dh = wave & 3;
  const int n = lane & 31, g = lane >> 5;
  const int head = hb * 64 + hg * 32 + n;
  if (head >= a.n_heads) return;

  const float sink = load_sink_log2(a, head);
  const int64_t part0 = (int64_t)(seq * a.n_hblk + hb) * a.n_splits;
  const float* ml0 = a.ws_ml + (part0 * 64 + hg * 32 + n) * 2;
  const uint16_t* wo0 =
      a.ws_o + (part0 * kWaves + wave) * (int64_t)(4 * 16 * 64) + ((mt * 2 + c / 2) * 64 + lane) * 8 + (c & 1) * 4;
  // One online pass in chunks of 16 ranges: the statistics and the partial rows of a chunk are all
  // requested at once, so a sequence split into up to 16 ranges costs one memory round trip.
  constexpr int kChunk = 16;
  float m_run = sink;  // the sink joins the maximum and the denominator once
  float l = sink == -__builtin_inff() ? 0.0f : 1.0f;
  f32x4_t o = {0.f, 0.f, 0.f, 0.f};
  for (int s0 = 0; s0 < a.n_splits; s0 += kChunk) {
    float mv[kChunk], lv[kChunk];
    f16x4_t ov[kChunk];
#pragma unroll
    for (int j = 0; j < kChunk; j++) {
      const bool live = s0 + j < a.n_splits;
      const int64_t sj = live ? s0 + j : 0;
      mv[j] = ml0[sj * 128];
      lv[j] = ml0[sj * 128 + 1];
      ov[j] = *reinterpret_cast<const f16x4_t*>(wo0 + sj * (int64_t)(4 * 8 * 16 * 64));
      if (!live) mv[j] = -__builtin_inff();
    }
    float m_new = m_run;
#pragma unroll
    for (int j = 0; j < kChunk; j++) m_new = fmaxf(m_new, mv[j]);
    const float m_safe = m_new == -__builtin_inff() ? 0.0f : m_new;
    const float alpha = fast_exp2(m_run - m_safe);  // 0 while nothing has been accumulated
    l *= alpha;
    o = o * alpha;
#pragma unroll
    for (int j = 0; j < kChunk; j++) {
      const float w = lv[j] * fast_exp2(mv[j] - m_safe);  // the stored row is already divided by lv[j]
      l += w;
      o += __builtin_convertvector(ov[j], f32x4_t) * w;
    }
    m_run = m_new;
  }
  const float inv = l == 0.0f ? 0.0f : 1.0f / l;
  float r[4] = {o.x * inv, o.y * inv, o.z * inv, o.w * inv};
  const int dim0 = dh * 128 + 32 * mt + 8 * c + 4 * g;
  const int64_t ooff = (int64_t)b * a.out_batch_stride + (int64_t)t * a.out_token_stride +
                       (int64_t)head * a.out_head_stride + dim0;
  emit_output<ODT>(a, r, ooff, dim0);
}

int choose_splits(int batch_hblk, int n_keys) {
  // enough workgroups to cover the 256 CUs but not one more (all are resident at once and a CU that holds
  // two of them takes about twice as long), at least one 32-slot tile each, and never more slots per
  // workgroup than its LDS row pointer table holds (its window share and its gathered share are each
  // padded to whole tiles: at most 62 slots of padding and 2 of rounding on top of n_keys / splits)
  int tiles = (n_keys + kTile - 1) / kTile;
  if (tiles < 1) tiles = 1;
  int want = batch_hblk <= 256 ? 256 / batch_hblk : 1;
  if (want > 32) want = 32;
  if (want > tiles) want = tiles;
  int min_splits = (n_keys + 959) / 960;
  if (want < min_splits) want = min_splits;
  if (want < 1) want = 1;
  return want;
}

constexpr size_t kPartialBytes = 4 * 8 * 16 * 64 * sizeof(uint16_t);  // 64 heads x 512 columns, float16
constexpr size_t kStatBytes = 64 * 2 * sizeof(float);                 // (m, l) per head
static_assert(kStaticBytes == 256 * (kPartialBytes + kStatBytes), "static scratch: 256 key ranges");

size_t workspace_bytes(int batch, int n_heads, int64_t n_keys) {
  int n_hblk = (n_heads + 63) / 64;
  int splits = choose_splits(batch * n_hblk, (int)n_keys);
  if (splits == 1) return 256;  // one key range per sequence: stored directly, no partials
  size_t parts = (size_t)batch * n_hblk * splits;
  return parts * (kPartialBytes + kStatBytes);
}

// Address of the static scratch on the current device, looked up once per device (each GPU holds its own
// copy of the array at its own address; the array's name is never used as an address in host code).
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {nullptr};

int static_scratch(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    mspr_set_error("sparse attention: cannot identify the current device (%s)", hipGetErrorString(e));
    return MSPR_ERR_LAUNCH;
  }
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      mspr_set_error("sparse attention: no address for the static scratch on device %d (%s)", dev,
                     hipGetErrorString(e));
      return MSPR_ERR_LAUNCH;
    }
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return MSPR_OK;
}

template <int KDT, int DK, int QDT, bool ROPE>
int launch_split(const SparseAttnArgs& a, hipStream_t st) {
  using G = Geometry<DK>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sparse_attn_split_kernel<KDT, DK, QDT, ROPE>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, G::kLdsBytes);
    if (e != hipSuccess) {
      mspr_set_error("sparse attention: cannot reserve %d bytes of LDS: %s", G::kLdsBytes, hipGetErrorString(e));
      return MSPR_ERR_LAUNCH;
    }
    attr_set = true;
  }
  dim3 grid((unsigned)(a.batch * a.n_hblk * a.n_splits)), block(kThreads);
  {
    MsprProfScope prof(MSPR_K_SPARSE_SPLIT, st);
    sparse_attn_split_kernel<KDT, DK, QDT, ROPE><<<grid, block, G::kLdsBytes, st>>>(a);
  }
  MSPR_CHECK_LAUNCH("sparse attention (split)");
  return MSPR_OK;
}

// The persistent prefill consumer takes at most PrefillGeometry::kMaxTiles tiles per token (float32 queries go
// through a half-precision copy in the workspace first); longer slot lists go through the split kernel, one
// workgroup per token.
bool prefill_consumer_fits(const SparseAttnArgs& a, int kv_dtype, int k_dim) {
  if (!a.prefill || kv_dtype != MSPR_F16 || k_dim != 512 || (a.q_dtype != MSPR_F16 && a.q_dtype != MSPR_F32) || a.rope ||
      a.out_dtype != MSPR_F32)
    return false;
  // MSPR_PREFILL_PERSISTENT=0 (read per call, like the reference's consumer switches) keeps every prefill call on
  // the split kernel, one workgroup per token: the form to compare the persistent consumer with
  const char* gate = getenv("MSPR_PREFILL_PERSISTENT");
  if (gate && gate[0] == '0' && gate[1] == '\0') return false;
  if (a.subst_row || a.subst_from_params || a.pool_rows_dev) return false;
  const int tiles = (a.n_win + kTile - 1) / kTile + (a.n_idx + kTile - 1) / kTile;
  return tiles <= PrefillGeometry::kMaxTiles;
}

int launch_prefill_consumer(const SparseAttnArgs& a, hipStream_t st) {
  using PG = PrefillGeometry;
  static bool attr_set = false;
  static int n_cus = 0;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sparse_attn_prefill_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, PG::kLdsBytes);
    int dev = 0;
    if (e == hipSuccess) e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&n_cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess || n_cus < 1) {
      mspr_set_error("sparse attention (prefill): cannot set up the kernel: %s", hipGetErrorString(e));
      return MSPR_ERR_LAUNCH;
    }
    attr_set = true;
  }
  const int n_units = a.batch * a.n_hblk;
  dim3 grid((unsigned)(n_units < n_cus ? n_units : n_cus)), block(kThreads);
  {
    MsprProfScope prof(MSPR_K_SPARSE_SPLIT, st);
    sparse_attn_prefill_kernel<<<grid, block, PG::kLdsBytes, st>>>(a);
  }
  MSPR_CHECK_LAUNCH("sparse attention (prefill)");
  return MSPR_OK;
}

int run_sparse_attention(SparseAttnArgs a, int kv_dtype, int k_dim, void* workspace, size_t workspace_bytes_given,
                         hipStream_t st) {
  const int n_keys = a.n_win + a.n_idx;
  if (a.n_tokens < 1) a.n_tokens = 1;
  if (a.q_head_stride == 0) a.q_head_stride = k_dim;
  if (a.out_head_stride == 0) {
    a.out_head_stride = kDV;
    a.out_batch_stride = (int64_t)a.n_heads * kDV;
  }
  a.n_hblk = (a.n_heads + 63) / 64;
  auto magic = [](int n) -> uint32_t { return n <= 1 ? 0u : (uint32_t)(((uint64_t)1 << 32) / (uint32_t)n); };
  a.inv_hblk = magic(a.n_hblk);
  a.inv_tokens = magic(a.n_tokens);
  if (prefill_consumer_fits(a, kv_dtype, k_dim)) {
    if (a.q_dtype == MSPR_F32) {
      // (a.batch counts sequences = batch entries x tokens)
      const int64_t n_rows = (int64_t)a.batch * a.n_heads;
      const size_t need = (size_t)n_rows * 512 * sizeof(uint16_t);
      MSPR_REQUIRE(workspace && workspace_bytes_given >= need,
                   "sparse attention (prefill): workspace of %zu bytes needed for the half-precision query copy, "
                   "%zu given",
                   need, workspace_bytes_given);
      MSPR_REQUIRE(mspr_aligned(workspace, 16), "sparse attention: workspace must be 16-byte aligned");
      MSPR_REQUIRE(a.q_head_stride % 4 == 0 && a.q_token_stride % 4 == 0 && a.q_batch_stride % 4 == 0,
                   "sparse attention (prefill): float32 q strides must be multiples of 4 elements");
      prefill_q_to_half_kernel<<<dim3((unsigned)((n_rows + 3) / 4)), dim3(256), 0, st>>>(
          reinterpret_cast<const float*>(a.q), a.q_batch_stride, a.q_head_stride, a.q_token_stride, a.n_heads,
          a.n_tokens, n_rows, reinterpret_cast<uint16_t*>(workspace));
      MSPR_CHECK_LAUNCH("sparse attention (prefill, query conversion)");
      a.q = workspace;
      a.q_dtype = MSPR_F16;
      a.q_head_stride = 512;
      a.q_token_stride = (int64_t)a.n_heads * 512;
      a.q_batch_stride = (int64_t)a.n_tokens * a.n_heads * 512;
    }
    return launch_prefill_consumer(a, st);
  }
  a.n_splits = choose_splits(a.batch * a.n_hblk, n_keys);
  a.win_per_split = (a.n_win + a.n_splits - 1) / a.n_splits;
  a.idx_per_split = (a.n_idx + a.n_splits - 1) / a.n_splits;
  const int table_slots = (a.win_per_split + kTile - 1) / kTile * kTile + (a.idx_per_split + kTile - 1) / kTile * kTile;
  MSPR_REQUIRE(table_slots <= 1024, "sparse attention: too many key slots (%d)", n_keys);
  a.direct = a.n_splits == 1;
  a.inv_splits = magic(a.n_splits);
  size_t need = workspace_bytes(a.batch, a.n_heads, n_keys);
  MSPR_REQUIRE(workspace && workspace_bytes_given >= need, "sparse attention: workspace of %zu bytes needed, %zu given",
               need, workspace_bytes_given);
  MSPR_REQUIRE(mspr_aligned(workspace, 16), "sparse attention: workspace must be 16-byte aligned");
  size_t parts = (size_t)a.batch * a.n_hblk * a.n_splits;
  a.ws_o = reinterpret_cast<uint16_t*>(workspace);
  a.ws_ml = reinterpret_cast<float*>(reinterpret_cast<unsigned char*>(workspace) + parts * kPartialBytes);
  int rc;
  if (a.rope) rc = launch_split<MSPR_F16, 512, kQSame, true>(a, st);
  else if (a.q_dtype == MSPR_F32) rc = launch_split<MSPR_F16, 512, MSPR_F32, false>(a, st);
  else if (kv_dtype == MSPR_BF16 && k_dim == 576) rc = launch_split<MSPR_BF16, 576, kQSame, false>(a, st);
  else if (kv_dtype == MSPR_BF16 && k_dim == 512) rc = launch_split<MSPR_BF16, 512, kQSame, false>(a, st);
  else if (kv_dtype == MSPR_F16 && k_dim == 576) rc = launch_split<MSPR_F16, 576, kQSame, false>(a, st);
  else rc = launch_split<MSPR_F16, 512, kQSame, false>(a, st);
  if (rc != MSPR_OK || a.direct) return rc;
  dim3 grid((unsigned)(a.batch * a.n_hblk * 32)), block(256);
  {
    MsprProfScope prof(MSPR_K_SPARSE_MERGE, st);
    if (a.out_dtype == MSPR_F32) sparse_attn_merge_kernel<MSPR_F32><<<grid, block, 0, st>>>(a);
    else if (a.out_dtype == MSPR_BF16) sparse_attn_merge_kernel<MSPR_BF16><<<grid, block, 0, st>>>(a);
    else sparse_attn_merge_kernel<MSPR_F16><<<grid, block, 0, st>>>(a);
  }
  MSPR_CHECK_LAUNCH("sparse attention (merge)");
  return MSPR_OK;
}

}  // namespace

extern "C" size_t mspr_sparse_attention_workspace_bytes(int batch, int n_heads, int64_t n_keys) {
  if (batch < 1 || n_heads < 1 || n_keys < 0) return 0;
  return workspace_bytes(batch, n_heads, n_keys);
}

extern "C" size_t mspr_indexed_mixed_attention_prefill_workspace_bytes(int q_dtype, int batch, int n_heads,
                                                                       int n_tokens, int window_rows, int top_k) {
  if (batch < 1 || n_heads < 1 || n_tokens < 1 || window_rows < 0 || top_k < 0) return 0;
  // the per-range partials of the split kernel (slot lists too long for the persistent consumer), or the
  // half-precision copy of float32 queries for the persistent consumer, whichever is larger
  size_t need = workspace_bytes(batch * n_tokens, n_heads, (int64_t)window_rows + top_k);
  if (q_dtype == MSPR_F32) {
    const size_t copy = (size_t)batch * n_tokens * n_heads * 512 * sizeof(uint16_t);
    if (copy > need) need = copy;
  }
  return need;
}

extern "C" int mspr_indexed_mixed_attention_decode(const float* q, int n_heads, const void* raw_kv, int raw_cap,
                                                   const void* comp_kv, int64_t n_comp, const int32_t* topk,
                                                   int top_k, const float* sinks, int64_t pos0, int window,
                                                   int ratio, int raw_start, float* out, void* workspace,
                                                   size_t workspace_bytes_given, void* stream) {
  MSPR_REQUIRE(q && raw_kv && comp_kv && sinks && out, "indexed_mixed_attention_decode: null pointer");
  MSPR_REQUIRE(top_k == 0 || topk, "indexed_mixed_attention_decode: null topk");
  MSPR_REQUIRE(n_heads >= 1, "indexed_mixed_attention_decode: q must carry at least one head");
  MSPR_REQUIRE(raw_cap >= 1, "indexed_mixed_attention_decode: raw_kv must contain at least one row");
  MSPR_REQUIRE(raw_start >= 0 && raw_start < raw_cap, "indexed_mixed_attention_decode: raw_start must be inside raw_kv");
  MSPR_REQUIRE(n_comp >= 1 && top_k >= 0 && window >= 0 && ratio >= 0 && pos0 >= 0 && pos0 < ((int64_t)1 << 31),
               "indexed_mixed_attention_decode: bad size argument");
  MSPR_REQUIRE(mspr_aligned(q, 16) && mspr_aligned(raw_kv, 16) && mspr_aligned(comp_kv, 16) && mspr_aligned(out, 16),
               "indexed_mixed_attention_decode: pointers must be 16-byte aligned");
  // Ring rows visited, in the unsigned 32-bit arithmetic of the reference kernel
  // (indexed_attention_kernel.py:120-141): a ring deeper than pos0+1 wraps and visits nothing.
  uint32_t qpos = (uint32_t)pos0, n_raw = (uint32_t)raw_cap;
  uint32_t first_raw_pos = qpos + 1u - n_raw;
  uint32_t raw_last_pos = first_raw_pos + n_raw - 1u;
  uint32_t window_first = (window != 0 && qpos + 1u > (uint32_t)window) ? qpos + 1u - (uint32_t)window : 0u;
  uint32_t first = first_raw_pos > window_first ? first_raw_pos : window_first;
  uint32_t last = qpos < raw_last_pos ? qpos : raw_last_pos;
  SparseAttnArgs a = {};
  a.q = q;
  a.q_dtype = MSPR_F32;
  a.q_batch_stride = 0;
  a.n_heads = n_heads;
  a.batch = 1;
  a.win = raw_kv;
  a.n_win = first <= last ? (int)(last - first + 1u) : 0;
  a.win_first = first <= last ? (int)(first - first_raw_pos) : 0;
  a.raw_start = raw_start;
  a.raw_cap = raw_cap;
  a.subst_row = nullptr;
  a.subst_slot = -1;
  a.pool = comp_kv;
  a.n_pool = n_comp;
  a.idx = topk;
  a.n_idx = top_k;
  int64_t visible = ratio == 0 ? n_comp : (pos0 + 1) / ratio;
  a.visible = visible < n_comp ? visible : n_comp;
  a.check_stop = 1;
  a.row_mul = 1;
  a.row_add = 0;
  a.sinks = sinks;
  a.sinks_dtype = MSPR_F32;
  a.scale_log2 = (float)(1.4426950408889634 / sqrt(512.0));
  a.rope = 0;
  a.out = out;
  a.out_dtype = MSPR_F32;
  return run_sparse_attention(a, MSPR_F16, 512, workspace, workspace_bytes_given, (hipStream_t)stream);
}

static int decode_sdpa(const void* q, int n_heads, const void* window, int window_rows, const void* row,
                       const void* pooled, int64_t n_rows, const int32_t* sel, int n_sel, const void* sinks,
                       const float* inv_freq, const int32_t* params, float scale, void* out, void* workspace,
                       size_t workspace_bytes_given, bool fixed, void* stream) {
  MSPR_REQUIRE(q && window && row && pooled && sinks && inv_freq && params && out,
               "fused_decode_sdpa: null pointer");
  MSPR_REQUIRE(n_sel == 0 || sel, "fused_decode_sdpa: null sel");
  MSPR_REQUIRE(n_heads >= 1, "fused_decode_sdpa: q must carry at least one head");
  MSPR_REQUIRE(window_rows >= 0 && n_rows >= 1 && n_sel >= 0, "fused_decode_sdpa: bad size argument");
  MSPR_REQUIRE(mspr_aligned(q, 16) && mspr_aligned(window, 16) && mspr_aligned(row, 16) && mspr_aligned(pooled, 16) &&
                   mspr_aligned(out, 8),
               "fused_decode_sdpa: pointers must be 16-byte aligned");
  SparseAttnArgs a = {};
  a.q = q;
  a.q_dtype = MSPR_F16;
  a.n_heads = n_heads;
  a.batch = 1;
  a.win = window;
  a.n_win = window_rows;
  a.win_first = 0;
  a.raw_start = 0;
  a.raw_cap = window_rows > 0 ? window_rows : 1;
  a.subst_row = row;
  a.subst_slot = -1;
  a.subst_from_params = 1;
  a.pool = pooled;
  a.n_pool = n_rows;
  a.idx = sel;
  a.n_idx = n_sel;
  a.visible = n_rows;
  a.check_stop = 0;
  a.row_mul = 1;
  a.row_add = 0;
  a.sinks = sinks;
  a.sinks_dtype = MSPR_F16;
  a.scale_log2 = (float)((double)scale * 1.4426950408889634);
  a.inv_freq = inv_freq;
  a.params = params;
  a.rope = 1;
  a.out = out;
  a.out_dtype = MSPR_F16;
  a.pool_rows_dev = fixed ? params + 2 : nullptr;
  return run_sparse_attention(a, MSPR_F16, 512, workspace, workspace_bytes_given, (hipStream_t)stream);
}

extern "C" int mspr_fused_decode_sdpa(const void* q, int n_heads, const void* window, int window_rows,
                                      const void* row, const void* pooled, int64_t n_rows, const int32_t* sel,
                                      int n_sel, const void* sinks, const float* inv_freq, const int32_t* params,
                                      float scale, void* out, void* workspace, size_t workspace_bytes_given,
                                      void* stream) {
  return decode_sdpa(q, n_heads, window, window_rows, row, pooled, n_rows, sel, n_sel, sinks, inv_freq, params, scale,
                     out, workspace, workspace_bytes_given, false, stream);
}

extern "C" int mspr_fused_decode_sdpa_fixed(const void* q, int n_heads, const void* window, int window_rows,
                                            const void* row, const void* pooled, int64_t capacity,
                                            const int32_t* sel, int n_sel, const void* sinks, const float* inv_freq,
                                            const int32_t* params, float scale, void* out, void* workspace,
                                            size_t workspace_bytes_given, void* stream) {
  return decode_sdpa(q, n_heads, window, window_rows, row, pooled, capacity, sel, n_sel, sinks, inv_freq, params,
                     scale, out, workspace, workspace_bytes_given, true, stream);
}

static int sparse_mla_decode_impl(const void* q, const void* kv, const int32_t* rows, const float* sinks, int dtype,
                                 int batch, int n_heads, int k_dim, int v_dim, int64_t n_pool, int n_rows, int row_mul,
                                 int row_add, int64_t win_start, int win_rows, float scale, void* out,
                                 void* workspace, size_t workspace_bytes_given, void* stream) {
  MSPR_REQUIRE(q && kv && out, "sparse_mla_decode: null pointer");
  MSPR_REQUIRE(n_rows == 0 || rows, "sparse_mla_decode: null rows");
  MSPR_REQUIRE(dtype == MSPR_F16 || dtype == MSPR_BF16, "sparse_mla_decode: dtype must be f16 or bf16");
  MSPR_REQUIRE(k_dim == 512 || k_dim == 576, "sparse_mla_decode: k_dim must be 512 or 576");
  MSPR_REQUIRE(v_dim == 512, "sparse_mla_decode: v_dim must be 512");
  MSPR_REQUIRE(batch >= 1 && n_heads >= 1 && n_heads <= 128, "sparse_mla_decode: batch >= 1 and 1 <= n_heads <= 128");
  MSPR_REQUIRE(n_pool >= 1 && n_pool < ((int64_t)1 << 31) && n_rows >= 0 && win_rows >= 0,
               "sparse_mla_decode: bad size argument");
  MSPR_REQUIRE(win_rows == 0 || (win_start >= 0 && win_start + win_rows <= n_pool),
               "sparse_mla_decode: window must lie inside the pool");
  MSPR_REQUIRE(mspr_aligned(q, 16) && mspr_aligned(kv, 16) && mspr_aligned(out, 16),
               "sparse_mla_decode: pointers must be 16-byte aligned");
  SparseAttnArgs a = {};
  a.q = q;
  a.q_dtype = dtype;
  a.q_batch_stride = (int64_t)n_heads * k_dim;
  a.n_heads = n_heads;
  a.batch = batch;
  a.win = reinterpret_cast<const uint16_t*>(kv) + (win_rows > 0 ? win_start : 0) * k_dim;
  a.win_batch_stride = n_pool * k_dim;
  a.n_win = win_rows;
  a.win_first = 0;
  a.raw_start = 0;
  a.raw_cap = win_rows > 0 ? win_rows : 1;
  a.subst_row = nullptr;
  a.subst_slot = -1;
  a.pool = kv;
  a.pool_batch_stride = n_pool * k_dim;
  a.n_pool = n_pool;
  a.idx = rows;
  a.idx_batch_stride = n_rows;
  a.n_idx = n_rows;
  a.visible = n_pool;
  a.check_stop = 0;
  a.row_mul = row_mul;
  a.row_add = row_add;
  a.sinks = sinks;
  a.sinks_dtype = MSPR_F32;
  a.scale_log2 = (float)((double)scale * 1.4426950408889634);
  a.rope = 0;
  a.out = out;
  a.out_dtype = dtype;
  return run_sparse_attention(a, dtype, k_dim, workspace, workspace_bytes_given, (hipStream_t)stream);
}

extern "C" int mspr_indexed_mixed_attention_prefill(const void* q, int q_dtype, int batch, int n_heads, int n_tokens,
                                                    int64_t q_batch_stride, int64_t q_head_stride,
                                                    int64_t q_token_stride, const void* raw_kv, int raw_cap,
                                                    const void* comp_kv, int64_t n_comp, const int32_t* topk,
                                                    int top_k, const float* sinks, int64_t pos0, int window,
                                                    int ratio, int raw_start, float* out, void* workspace,
                                                    size_t workspace_bytes_given, void* stream) {
  const char* what = "indexed_mixed_attention_prefill";
  MSPR_REQUIRE(q && raw_kv && comp_kv && sinks && out, "%s: null pointer", what);
  MSPR_REQUIRE(top_k == 0 || topk, "%s: null topk", what);
  MSPR_REQUIRE(q_dtype == MSPR_F32 || q_dtype == MSPR_F16, "%s: q must be float16 or float32", what);
  MSPR_REQUIRE(batch >= 1 && n_tokens >= 1 && n_heads >= 1, "%s: q must contain at least one batch, token and head",
               what);
  MSPR_REQUIRE((int64_t)batch * n_tokens < ((int64_t)1 << 24), "%s: too many tokens", what);
  MSPR_REQUIRE(raw_cap >= 1, "%s: raw_kv must contain at least one row", what);
  MSPR_REQUIRE(raw_start >= 0 && raw_start < raw_cap, "%s: raw_start must be inside raw_kv", what);
  MSPR_REQUIRE(n_comp >= 1 && top_k >= 0 && window >= 0 && ratio >= 0 && pos0 >= 0 &&
                   pos0 + n_tokens < ((int64_t)1 << 31),
               "%s: bad size argument", what);
  MSPR_REQUIRE(q_head_stride >= 512 && q_token_stride >= 0 && q_batch_stride >= 0 && q_head_stride % 8 == 0 &&
                   q_token_stride % 8 == 0 && q_batch_stride % 8 == 0,
               "%s: q strides must be multiples of 8 elements", what);
  MSPR_REQUIRE(mspr_aligned(q, 16) && mspr_aligned(raw_kv, 16) && mspr_aligned(comp_kv, 16) && mspr_aligned(out, 16),
               "%s: pointers must be 16-byte aligned", what);
  SparseAttnArgs a = {};
  a.q = q;
  a.q_dtype = q_dtype;
  a.q_batch_stride = q_batch_stride;
  a.q_head_stride = q_head_stride;
  a.q_token_stride = q_token_stride;
  a.n_heads = n_heads;
  a.batch = batch * n_tokens;
  a.n_tokens = n_tokens;
  a.prefill = 1;
  a.pos0 = (uint32_t)pos0;
  a.window = (uint32_t)window;
  a.ratio = (uint32_t)ratio;
  a.win = raw_kv;
  a.win_batch_stride = (int64_t)raw_cap * 512;
  // slot space: at most min(window, raw_cap, tokens seen so far) ring rows per token
  int64_t max_win = window != 0 && window < raw_cap ? window : raw_cap;
  if (max_win > pos0 + n_tokens) max_win = pos0 + n_tokens;
  a.n_win = (int)max_win;
  a.win_first = 0;
  a.raw_start = raw_start;
  a.raw_cap = raw_cap;
  a.subst_row = nullptr;
  a.subst_slot = -1;
  a.pool = comp_kv;
  a.pool_batch_stride = n_comp * 512;
  a.n_pool = n_comp;
  a.idx = topk;
  a.idx_batch_stride = top_k;
  a.n_idx = top_k;
  a.visible = n_comp;
  a.check_stop = 1;
  a.row_mul = 1;
  a.row_add = 0;
  a.sinks = sinks;
  a.sinks_dtype = MSPR_F32;
  a.scale_log2 = (float)(1.4426950408889634 / sqrt(512.0));
  a.rope = 0;
  a.out = out;
  a.out_dtype = MSPR_F32;
  a.out_batch_stride = q_batch_stride;
  a.out_head_stride = q_head_stride;
  a.out_token_stride = q_token_stride;
  return run_sparse_attention(a, MSPR_F16, 512, workspace, workspace_bytes_given, (hipStream_t)stream);
}

extern "C" int mspr_sparse_mla_decode(const void* q, const void* kv, const int32_t* rows, const float* sinks,
                                      int dtype, int batch, int n_heads, int k_dim, int v_dim, int64_t n_pool,
                                      int n_rows, int row_mul, int row_add, int64_t win_start, int win_rows,
                                      float scale, void* out, void* workspace, size_t workspace_bytes_given,
                                      void* stream) {
  return sparse_mla_decode_impl(q, kv, rows, sinks, dtype, batch, n_heads, k_dim, v_dim, n_pool, n_rows, row_mul,
                                row_add, win_start, win_rows, scale, out, workspace, workspace_bytes_given, stream);
}

extern "C" size_t mspr_sparse_mla_decode_static_max_bytes(void) { return kStaticBytes; }

extern "C" int mspr_sparse_mla_decode_static(const void* q, const void* kv, const int32_t* rows, const float* sinks,
                                             int dtype, int batch, int n_heads, int k_dim, int v_dim, int64_t n_pool,
                                             int n_rows, int row_mul, int row_add, int64_t win_start, int win_rows,
                                             float scale, void* out, void* stream) {
  MSPR_REQUIRE(batch >= 1 && n_heads >= 1 && n_rows >= 0 && win_rows >= 0, "sparse_mla_decode_static: bad size argument");
  const size_t need = workspace_bytes(batch, n_heads, (int64_t)n_rows + win_rows);
  MSPR_REQUIRE(need <= kStaticBytes,
               "sparse_mla_decode_static: batch %d x %d heads x %d keys needs %zu bytes of scratch, the built-in "
               "scratch holds %zu (at most 256 key ranges): use mspr_sparse_mla_decode with a workspace",
               batch, n_heads, n_rows + win_rows, need, kStaticBytes);
  void* ws = nullptr;
  int rc = static_scratch(&ws);
  if (rc != MSPR_OK) return rc;
  return sparse_mla_decode_impl(q, kv, rows, sinks, dtype, batch, n_heads, k_dim, v_dim, n_pool, n_rows, row_mul,
                                row_add, win_start, win_rows, scale, out, ws, kStaticBytes, stream);
}
