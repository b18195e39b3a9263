// Causal chunked-prefill GQA attention, head dim 256: a chunk of q_len new tokens attends to the
// past_len tokens already in the KV cache and, causally, to itself.
//
// Workgroup = 8 waves = the query heads that share one KV head (times query sub-blocks when fewer
// than 8 heads share it) x 32 query rows each, so one K/V tile staged in LDS feeds eight waves.
// K/V tiles of 32 keys stream through a 3-deep LDS ring with asynchronous global->LDS copies; the
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
constexpr int kBufs = 3;
constexpr int kThreads = 512;
constexpr int kLdsBytes = kBufs * kStageBytes;  // 96 KB

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

// swizzle of the 16-byte pieces of a tile row: piece p of row r sits at slot (p & 16) | ((p ^ f(r)) & 15)
__device__ __forceinline__ int swz(int r) { return ((r & 7) << 1) | ((r >> 3) & 1); }

template <int KDT>
__global__ __launch_bounds__(kThreads, 1) void flash_prefill_kernel(PrefillArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31;  // MFMA column: query row of the wave's block; MFMA row (key) for the K operand
  const int g = lane >> 5;

  // ---- workgroup -> (batch, kv head, query block); late blocks (most keys) first
  const int rep = 1 << a.rep_shift;
  const int sub_blocks = 8 >> a.rep_shift;  // 32-row query sub-blocks per workgroup
  const int rows_per_wg = 32 * sub_blocks;
  int work = blockIdx.x;
  const int qb = a.q_blocks - 1 - work % a.q_blocks;
  work /= a.q_blocks;
  const int kvh = work % a.n_kv_heads;
  const int b = work / a.n_kv_heads;
  const int head = kvh * rep + (wave & (rep - 1));
  const int q0 = qb * rows_per_wg + 32 * (wave >> a.rep_shift);  // first query row of this wave
  const int past = (int)a.past_len;

  const unsigned char* kbase =
      reinterpret_cast<const unsigned char*>(a.k) + ((int64_t)b * a.n_kv_heads + kvh) * a.kv_rows * kRowBytes;
  const unsigned char* vbase =
      reinterpret_cast<const unsigned char*>(a.v) + ((int64_t)b * a.n_kv_heads + kvh) * a.kv_rows * kRowBytes;

  // keys needed by the workgroup: [0, past + last query row]
  int q_last = qb * rows_per_wg + rows_per_wg - 1;
  if (q_last > a.q_len - 1) q_last = a.q_len - 1;
  const int n_tiles = (int)((past + q_last) / kTile) + 1;

  // ---- asynchronous tile copies: thread handles LDS slots tid and tid + 512 of the K and of the V tile;
  //      addresses are a scalar tile base plus a per-thread 32-bit offset
  const int c_row = tid >> 5;                                  // tile row of slot `tid` (slot tid+512: row + 16)
  const int c_piece = (tid & 16) | ((tid ^ swz(c_row)) & 15);  // global 16-byte piece that lands in the slot
  const uint32_t lds0 = (uint32_t)(uintptr_t)MSPR_LDS_PTR(unsigned char, lds);
  const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(lds0) + wave * 1024;
  const int n_keys = (int)(past + a.q_len);  // keys that exist
  auto issue_tile = [&](int t, int slot) {
    // rows past the last key (only in the last tile) are masked by the causal rule; read the last key instead
    const int last = n_keys - 1 - t * kTile;
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
    const u32x4_t* qp = reinterpret_cast<const u32x4_t*>(
        reinterpret_cast<const unsigned char*>(a.q) + (((int64_t)b * a.n_q_heads + head) * a.q_len + qrow) * kRowBytes +
        16 * g);
#pragma unroll
    for (int s = 0; s < 16; s++) qf[s] = qp[2 * s];
#pragma unroll
    for (int s = 0; s < 16; s++) asm volatile("" : "+v"(qf[s]));  // complete before the first asynchronous copy
  }

  // every wave issues its share of every tile (clamped past the end), so waits are static counts
  issue_tile(0, 0);
  issue_tile(n_tiles > 1 ? 1 : 0, 1);

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
  const int my_last_key = past + q0 + 31;  // last key any query of this wave may see
  const int qpos = past + q0 + n;

  for (int t = 0; t < n_tiles; t++) {
    // tile t has landed once this wave's copies of it are done (4 newer ones may be in flight) and
    // every wave got here; the ring slot of tile t-1 is free after the barrier
    wait_vm_and_barrier<4>();
    issue_tile(t + 2 < n_tiles ? t + 2 : n_tiles - 1, (t + 2) % kBufs);  // past the end: a harmless re-read
    const int key0 = t * kTile;
    if (key0 > my_last_key) continue;  // wave-uniform: this wave's queries see none of the tile
    const unsigned char* st = lds + (t % kBufs) * kStageBytes;

    // S^T = K . Q^T
    f32x16_t sacc = {0};
    {
      constexpr int kAhead = 3;
      u32x4_t af[kAhead];
#pragma unroll
      for (int s = 0; s < kAhead; s++)
        af[s] = *reinterpret_cast<const u32x4_t*>(st + ((k_off ^ ((s & 7) << 5)) + (s >> 3) * 256));
#pragma unroll
      for (int s = 0; s < 16; s++) {
        u32x4_t cur = af[s % kAhead];
        if (s + kAhead < 16) {
          const int s2 = s + kAhead;
          af[s % kAhead] = *reinterpret_cast<const u32x4_t*>(st + ((k_off ^ ((s2 & 7) << 5)) + (s2 >> 3) * 256));
        }
        sacc = mfma32<KDT>(cur, qf[s], sacc);
      }
    }

    // online softmax (log2 domain); register i is key key0 + 8 (i/4) + 4 g + i%4
    float tmax = -__builtin_inff();
    if (key0 + kTile - 1 <= past + q0) {  // wave-uniform: no query of the wave masks any key of the tile
#pragma unroll
      for (int i = 0; i < 16; i++) {
        sacc[i] *= a.scale_log2;
        tmax = fmaxf(tmax, sacc[i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const bool valid = key0 + 8 * (i / 4) + 4 * g + (i % 4) <= qpos;
        sacc[i] = valid ? sacc[i] * a.scale_log2 : -__builtin_inff();
        tmax = fmaxf(tmax, sacc[i]);
      }
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, MSPR_WAVE));
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
    const float m_safe = m_run == -__builtin_inff() ? 0.0f : m_run;
    float psum = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      sacc[i] = __builtin_amdgcn_exp2f(sacc[i] - m_safe);
      psum += sacc[i];
    }
    l_run += psum;
    u32x4_t pf[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
      pf[ks] = u32x4_t{pack2<KDT>(sacc[8 * ks], sacc[8 * ks + 1]), pack2<KDT>(sacc[8 * ks + 2], sacc[8 * ks + 3]),
                       pack2<KDT>(sacc[8 * ks + 4], sacc[8 * ks + 5]), pack2<KDT>(sacc[8 * ks + 6], sacc[8 * ks + 7])};

    // O^T += V^T . P^T
#pragma unroll
    for (int mt = 0; mt < 8; mt++) {
#pragma unroll
      for (int ks = 0; ks < 2; ks++) {
        const unsigned char* lo_p = st + ((v_off[0] ^ ((mt & 3) << 6)) + (mt >> 2) * 256 + ks * 16 * kRowBytes);
        const unsigned char* hi_p = st + ((v_off[1] ^ ((mt & 3) << 6)) + (mt >> 2) * 256 + ks * 16 * kRowBytes);
        s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(MSPR_LDS_PTR(s16x4_t, lo_p));
        s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(MSPR_LDS_PTR(s16x4_t, hi_p));
        u32x2_t lo2 = __builtin_bit_cast(u32x2_t, lo), hi2 = __builtin_bit_cast(u32x2_t, hi);
        oacc[mt] = mfma32<KDT>(u32x4_t{lo2.x, lo2.y, hi2.x, hi2.y}, pf[ks], oacc[mt]);
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the clamped trailing copies must not outlive the workgroup's LDS

  // ---- normalise and store: lane (n, g) holds dims 32 mt + 8 (i/4) + 4 g + i%4 of query row q0 + n
  const float l_tot = l_run + __shfl_xor(l_run, 32, MSPR_WAVE);
  const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
  if (q0 + n < a.q_len) {
    unsigned char* op = reinterpret_cast<unsigned char*>(a.out) +
                        (((int64_t)b * a.n_q_heads + head) * a.q_len + q0 + n) * kRowBytes;
#pragma unroll
    for (int mt = 0; mt < 8; mt++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        u32x2_t w = {pack2<KDT>(oacc[mt][4 * c] * inv, oacc[mt][4 * c + 1] * inv),
                     pack2<KDT>(oacc[mt][4 * c + 2] * inv, oacc[mt][4 * c + 3] * inv)};
        *reinterpret_cast<u32x2_t*>(op + (32 * mt + 8 * c + 4 * g) * 2) = w;
      }
  }
}

template <int KDT>
int prefill_launch(const PrefillArgs& a, hipStream_t st) {
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&flash_prefill_kernel<KDT>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    if (e != hipSuccess) {
      mspr_set_error("flash_prefill: cannot reserve %d bytes of LDS: %s", kLdsBytes, hipGetErrorString(e));
      return MSPR_ERR_LAUNCH;
    }
    attr_set = true;
  }
  dim3 grid((unsigned)(a.q_blocks * a.n_kv_heads * a.batch)), block(kThreads);
  {
    MsprProfScope prof(MSPR_K_FLASH_PREFILL, st);
    flash_prefill_kernel<KDT><<<grid, block, kLdsBytes, st>>>(a);
  }
  MSPR_CHECK_LAUNCH("flash_prefill");
  return MSPR_OK;
}

}  // namespace

extern "C" int mspr_flash_prefill(const void* q, const void* k, const void* v, int dtype, int batch, int n_q_heads,
                                  int n_kv_heads, int head_dim, int q_len, int64_t past_len, int64_t kv_rows,
                                  float scale, void* out, void* stream) {
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
  const int rows_per_wg = 32 * (8 / rep);
  a.q_blocks = (q_len + rows_per_wg - 1) / rows_per_wg;
  MSPR_REQUIRE((int64_t)a.q_blocks * n_kv_heads * batch < ((int64_t)1 << 31), "flash_prefill: grid too large");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MSPR_BF16) return prefill_launch<MSPR_BF16>(a, st);
  return prefill_launch<MSPR_F16>(a, st);
}
