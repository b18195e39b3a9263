// Deterministic top-k over float32 score rows: select on monotone uint32 keys, then ordered emission
// (rows strictly above the k-th key in ascending row order, then the lowest-index rows tied with it).
//
// One 1024-thread workgroup per score row. Rows of up to 32768 scores are read once and kept in
// registers, every thread owning a block of consecutive rows. Two ways to the k-th key:
//  * pivot path: a 1024-row sample gives a 16-bit key prefix safely below the k-th key, the rows at
//    or above it (a few thousand) are compacted in row order and three small digit passes plus the
//    emission run on that list. The kernel checks exactly that the list contains the k-th key; the
//    sample decides how long the call takes, never what it returns.
//  * full passes (also the fallback of the pivot path): MSB radix select with four 8-bit digits over
//    all keys. Histograms are 256 bins x 64 copies in LDS, copy = lane id, laid out [bin][copy], so
//    every lane of an LDS atomic hits its own bank whatever the digit distribution is (scores of one
//    row usually share their top byte, which would serialise a single shared counter 64-fold). After
//    two digits the keys that still match the prefix are usually a handful; they are compacted into
//    an LDS list and the last two digits run on that list only.
// Longer rows use the striped kernel, which re-reads global memory each pass.
#include <cmath>

#include "common.h"
#include "profile.h"

namespace {

constexpr int kThreads = 1024;
constexpr int kWaves = kThreads / 64;
constexpr int kCopies = 64;
constexpr int kListCap = 2048;
constexpr int kFastPer = 6;                     // survivor-list entries per thread on the pivot path
constexpr int kFastCap = kFastPer * kThreads;   // survivor-list capacity

struct SelectState {
  uint32_t prefix;
  uint32_t need;
  uint32_t live;   // keys matching the current prefix
  uint32_t list_n;
};

// Wave 0: pick the bucket where the count from the top first reaches `need`. totals[b] in LDS.
__device__ __forceinline__ void choose_bucket(const uint32_t* totals, SelectState* st, uint32_t shift, int lane) {
  uint32_t t[4];
#pragma unroll
  for (int j = 0; j < 4; j++) t[j] = totals[4 * lane + j];
  uint32_t lane_sum = t[0] + t[1] + t[2] + t[3];
  uint32_t sfx = lane_sum;  // inclusive suffix sum over lanes
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    uint32_t o = __shfl_down(sfx, off, MSPR_WAVE);
    if (lane + off < 64) sfx += o;
  }
  const uint32_t need = st->need;
  const uint32_t prefix = st->prefix;
  int chosen = -1;
  uint32_t chosen_need = 0u, chosen_cnt = 0u;
  uint32_t run = sfx - lane_sum;  // keys in buckets of higher lanes
#pragma unroll
  for (int j = 3; j >= 0; j--) {
    if (chosen < 0 && run < need && run + t[j] >= need) {
      chosen = 4 * lane + j;
      chosen_need = need - run;
      chosen_cnt = t[j];
    }
    run += t[j];
  }
  uint64_t any = __ballot(chosen >= 0);
  if (any == 0ull) {
    // fewer live keys than needed cannot happen for topk <= n_rows; bucket 0 takes the rest
    if (lane == 0) {
      st->need = need - (sfx - t[0]);
      st->live = t[0];
    }
  } else if (chosen >= 0) {
    st->prefix = prefix | ((uint32_t)chosen << shift);
    st->need = chosen_need;
    st->live = chosen_cnt;
  }
}

template <int CACHE>
__global__ __launch_bounds__(kThreads) void topk_select_kernel(const float* __restrict__ scores_all,
                                                                int64_t score_stride, int64_t n_rows, int topk,
                                                                int32_t* __restrict__ sel_all) {
  __shared__ uint32_t hist[256 * kCopies];  // [bin][copy]
  __shared__ uint32_t totals[256];
  __shared__ uint32_t list[kListCap];
  __shared__ SelectState st;
  __shared__ uint32_t cnt_above[kThreads];
  __shared__ uint32_t cnt_tie[kThreads];
  __shared__ uint32_t wave_tot[2 * kWaves];
  __shared__ uint32_t carry[2];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const float* scores = scores_all + (int64_t)blockIdx.x * score_stride;
  int32_t* sel = sel_all + (int64_t)blockIdx.x * topk;
  const int64_t n_chunks = (n_rows + kThreads - 1) / kThreads;

  uint32_t kreg[CACHE > 0 ? CACHE : 1];
  if constexpr (CACHE > 0) {
#pragma unroll
    for (int i = 0; i < CACHE; i++) {
      int64_t r = (int64_t)i * kThreads + tid;
      kreg[i] = r < n_rows ? score_key(scores[r]) : 0u;
    }
  }
  if (tid == 0) {
    st.prefix = 0u;
    st.need = (uint32_t)topk;
    st.live = (uint32_t)n_rows;
    st.list_n = 0u;
  }

  // one digit over every key: count keys whose higher digits equal the prefix
  auto full_pass = [&](int pass) {
    const uint32_t shift = 24u - 8u * pass;
    u32x4_t* h4 = reinterpret_cast<u32x4_t*>(hist);
    for (int i = tid; i < 256 * kCopies / 4; i += kThreads) h4[i] = u32x4_t{0u, 0u, 0u, 0u};
    __syncthreads();
    const uint32_t prefix = st.prefix;
    const uint32_t mask_hi = pass == 0 ? 0u : (0xFFFFFFFFu << (shift + 8u));
    if constexpr (CACHE > 0) {
#pragma unroll
      for (int i = 0; i < CACHE; i++) {
        int64_t r = (int64_t)i * kThreads + tid;
        uint32_t key = kreg[i];
        if (r < n_rows && (key & mask_hi) == prefix) atomicAdd(&hist[((key >> shift) & 0xFFu) * kCopies + lane], 1u);
      }
    } else {
      for (int64_t c = 0; c < n_chunks; c++) {
        int64_t r = c * kThreads + tid;
        if (r < n_rows) {
          uint32_t key = score_key(scores[r]);
          if ((key & mask_hi) == prefix) atomicAdd(&hist[((key >> shift) & 0xFFu) * kCopies + lane], 1u);
        }
      }
    }
    __syncthreads();
    // totals[bin] = sum over copies: four threads per bin, 16 copies each, rotated to spread banks
    {
      const int bin = tid >> 2, q = tid & 3;
      uint32_t s = 0u;
#pragma unroll
      for (int j = 0; j < 16; j++) s += hist[bin * kCopies + q * 16 + ((j + lane) & 15)];
      s += __shfl_xor(s, 1, MSPR_WAVE);
      s += __shfl_xor(s, 2, MSPR_WAVE);
      if (q == 0) totals[bin] = s;
    }
    __syncthreads();
    if (wave == 0) choose_bucket(totals, &st, shift, lane);
    __syncthreads();
  };

  full_pass(0);
  full_pass(1);

  if (st.live <= (uint32_t)kListCap) {
    // compact the keys that match the 16-bit prefix; their order does not matter here
    const uint32_t prefix = st.prefix;
    if constexpr (CACHE > 0) {
#pragma unroll
      for (int i = 0; i < CACHE; i++) {
        int64_t r = (int64_t)i * kThreads + tid;
        uint32_t key = kreg[i];
        if (r < n_rows && (key & 0xFFFF0000u) == prefix) list[atomicAdd(&st.list_n, 1u)] = key;
      }
    } else {
      for (int64_t c = 0; c < n_chunks; c++) {
        int64_t r = c * kThreads + tid;
        if (r < n_rows) {
          uint32_t key = score_key(scores[r]);
          if ((key & 0xFFFF0000u) == prefix) list[atomicAdd(&st.list_n, 1u)] = key;
        }
      }
    }
    __syncthreads();
    const uint32_t n_list = st.list_n;
    for (int pass = 2; pass < 4; pass++) {
      const uint32_t shift = 24u - 8u * pass;
      if (tid < 256) totals[tid] = 0u;
      __syncthreads();
      const uint32_t pfx = st.prefix;
      const uint32_t mask_hi = 0xFFFFFFFFu << (shift + 8u);
      for (uint32_t i = tid; i < n_list; i += kThreads) {
        uint32_t key = list[i];
        if ((key & mask_hi) == pfx) atomicAdd(&totals[(key >> shift) & 0xFFu], 1u);
      }
      __syncthreads();
      if (wave == 0) choose_bucket(totals, &st, shift, lane);
      __syncthreads();
    }
  } else {
    full_pass(2);
    full_pass(3);
  }

  const uint32_t threshold = st.prefix;
  const uint32_t need_ties = st.need;
  const uint32_t n_above = (uint32_t)topk - need_ties;
  if (tid == 0) {
    carry[0] = 0u;
    carry[1] = 0u;
  }
  __syncthreads();

  // Emission in groups of 64 chunks (65536 rows): per (chunk, wave) counts -> one block scan.
  const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  auto count_chunk = [&](int ci, bool live, uint32_t key) {
    uint64_t ba = __ballot(live && key > threshold);
    uint64_t bt = __ballot(live && key == threshold);
    if (lane == 0) {
      cnt_above[ci * kWaves + wave] = (uint32_t)__popcll(ba);
      cnt_tie[ci * kWaves + wave] = (uint32_t)__popcll(bt);
    }
  };
  auto emit_chunk = [&](int ci, int64_t r, bool live, uint32_t key) {
    bool is_above = live && key > threshold;
    bool is_tie = live && key == threshold;
    uint64_t ba = __ballot(is_above);
    uint64_t bt = __ballot(is_tie);
    if (is_above) {
      uint32_t slot = cnt_above[ci * kWaves + wave] + (uint32_t)__popcll(ba & lt_mask);
      sel[slot] = (int32_t)r;
    } else if (is_tie) {
      uint32_t rank = cnt_tie[ci * kWaves + wave] + (uint32_t)__popcll(bt & lt_mask);
      if (rank < need_ties) sel[n_above + rank] = (int32_t)r;
    }
  };
  for (int64_t g0 = 0; g0 < n_chunks; g0 += 64) {
    const int gchunks = (int)((n_chunks - g0) < 64 ? (n_chunks - g0) : 64);
    if constexpr (CACHE > 0) {
#pragma unroll
      for (int ci = 0; ci < CACHE; ci++) {
        if (ci < gchunks) {
          int64_t r = (int64_t)ci * kThreads + tid;
          count_chunk(ci, r < n_rows, kreg[ci]);
        }
      }
    } else {
      for (int ci = 0; ci < gchunks; ci++) {
        int64_t r = (g0 + ci) * kThreads + tid;
        bool live = r < n_rows;
        count_chunk(ci, live, live ? score_key(scores[r]) : 0u);
      }
    }
    for (int i = gchunks * kWaves + tid; i < kThreads; i += kThreads) {
      cnt_above[i] = 0u;
      cnt_tie[i] = 0u;
    }
    __syncthreads();
    // exclusive scan over the (chunk, wave) entries, one per thread
    uint32_t va = cnt_above[tid], vt = cnt_tie[tid];
    uint32_t ia = va, it = vt;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      uint32_t oa = __shfl_up(ia, off, MSPR_WAVE);
      uint32_t ot = __shfl_up(it, off, MSPR_WAVE);
      if (lane >= off) {
        ia += oa;
        it += ot;
      }
    }
    if (lane == 63) {
      wave_tot[wave] = ia;
      wave_tot[kWaves + wave] = it;
    }
    __syncthreads();
    uint32_t base_a = carry[0], base_t = carry[1];
    for (int w = 0; w < wave; w++) {
      base_a += wave_tot[w];
      base_t += wave_tot[kWaves + w];
    }
    __syncthreads();
    cnt_above[tid] = base_a + ia - va;
    cnt_tie[tid] = base_t + it - vt;
    if (tid == kThreads - 1) {
      carry[0] = base_a + ia;
      carry[1] = base_t + it;
    }
    __syncthreads();
    if constexpr (CACHE > 0) {
#pragma unroll
      for (int ci = 0; ci < CACHE; ci++) {
        if (ci < gchunks) {
          int64_t r = (int64_t)ci * kThreads + tid;
          emit_chunk(ci, r, r < n_rows, kreg[ci]);
        }
      }
    } else {
      for (int ci = 0; ci < gchunks; ci++) {
        int64_t r = (g0 + ci) * kThreads + tid;
        bool live = r < n_rows;
        emit_chunk(ci, r, live, live ? score_key(scores[r]) : 0u);
      }
    }
    __syncthreads();
  }
}

// Every wave runs this on the same 256 totals and gets the same answer in every lane: the digit
// where the count from the top first reaches `need`, the keys still needed inside it and its size.
struct Pick {
  uint32_t digit, need, live;
};
// Inclusive prefix sum over the 64 lanes with data-parallel-primitive moves (no LDS round trips):
// four shifts inside each row of 16 lanes, then the row totals are carried across rows.
__device__ __forceinline__ uint32_t wave_prefix_sum(uint32_t x) {
  int v = (int)x;
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, false);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xF, 0xF, false);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xF, 0xF, false);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xF, 0xF, false);  // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);  // row_bcast:31 into rows 2 and 3
  return (uint32_t)v;
}

// mask = 2 mask + bit
__device__ __forceinline__ uint32_t shift_in(uint32_t mask, bool bit) { return (mask << 1) | (bit ? 1u : 0u); }

// One histogram vote per lane. Up to four rounds first count all lanes that share the bin of the
// lowest voting lane with a single atomic (digits near the top of the key are shared by most rows,
// which would serialise one atomic per lane on the same counter); what is left votes directly.
__device__ __forceinline__ void wave_hist_add(uint32_t* h, int bin, int lane) {
#pragma unroll
  for (int round = 0; round < 4; round++) {
    const uint64_t voters = __ballot(bin >= 0);
    if (voters == 0ull) break;
    const int first = (int)__builtin_ctzll(voters);
    const int d = __builtin_amdgcn_readlane(bin, first);
    const uint64_t same = __ballot(bin == d);
    if (lane == first) atomicAdd(&h[d], (uint32_t)__popcll(same));
    if (bin == d) bin = -1;
  }
  if (bin >= 0) atomicAdd(&h[bin], 1u);
}

__device__ __forceinline__ Pick pick_bucket(const uint32_t* totals, uint32_t need, int lane) {
  // lane l looks at digits 255-4l .. 252-4l, so a prefix sum over lanes counts keys from the top digit down
  uint32_t t[4];
#pragma unroll
  for (int j = 0; j < 4; j++) t[j] = totals[255 - (4 * lane + j)];
  const uint32_t lane_sum = t[0] + t[1] + t[2] + t[3];
  const uint32_t incl = wave_prefix_sum(lane_sum);
  int chosen = -1;
  uint32_t chosen_need = 0u, chosen_cnt = 0u;
  uint32_t run = incl - lane_sum;  // keys in higher digits
#pragma unroll
  for (int j = 0; j < 4; j++) {
    if (chosen < 0 && run < need && run + t[j] >= need) {
      chosen = 255 - (4 * lane + j);
      chosen_need = need - run;
      chosen_cnt = t[j];
    }
    run += t[j];
  }
  const uint64_t any = __ballot(chosen >= 0);
  Pick p;
  if (any) {
    const int src = (int)__builtin_ctzll(any);
    p.digit = (uint32_t)__builtin_amdgcn_readlane(chosen, src);
    p.need = (uint32_t)__builtin_amdgcn_readlane((int)chosen_need, src);
    p.live = (uint32_t)__builtin_amdgcn_readlane((int)chosen_cnt, src);
  } else {
    // fewer keys than needed cannot happen for topk <= rows held; digit 0 would take the rest
    const uint32_t total = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
    const uint32_t d0 = (uint32_t)__builtin_amdgcn_readlane((int)t[3], 63);
    p.digit = 0u;
    p.need = need - (total - d0);
    p.live = d0;
  }
  return p;
}

// Rows of up to C*1024 scores: thread t owns the C consecutive rows [C t, C t + C) in registers.
// With consecutive ownership the ordered emission needs no cross-lane work per row: a thread knows
// the relative order of its own rows, so one packed block scan of the per-thread counts gives every
// thread its output slots. Digit histograms over all keys use 256 bins x 64 copies (copy = lane, so
// an LDS atomic never meets a bank conflict whatever the digit distribution); the thread that sums a
// group of copies also zeroes it for the next pass. Select state lives in registers: every wave derives it
// from the same totals, which saves the broadcast barriers.
// Rows past n_rows are given key 0: they can only tie with the lowest possible key and lose every
// tie to a real row (ties go to the lower index), so no pass needs a bounds check.
template <int C>
__global__ __launch_bounds__(kThreads) void topk_blocked_kernel(const float* __restrict__ scores_all,
                                                                 int64_t score_stride, int n_rows, int topk,
                                                                 int sample_rank, int32_t* __restrict__ sel_all) {
  // The staging area for the load (C*1024 keys) is reused for the histogram copies afterwards.
  // copies of the full-pass histograms: one per lane where the staging area is that large anyway; 32 (lanes l and
  // l + 32 share one) for the short-row instance, whose LDS then lets two workgroups share a CU
  constexpr int kCp = C * kThreads >= 256 * kCopies ? kCopies : kCopies / 2;
  constexpr int kStageWords = C * kThreads > 256 * kCp ? C * kThreads : 256 * kCp;
  __shared__ __attribute__((aligned(16))) uint32_t stage[kStageWords];
  uint32_t* hist = stage;                   // [bin][copy]
  __shared__ uint32_t totals[256];
  __shared__ uint32_t small_hist[2][256];   // digits 2 and 3 on the compacted list
  // survivor rows of the pivot path (16-bit row numbers), or the compacted keys of the full passes
  __shared__ __attribute__((aligned(16))) uint32_t list_words[kFastCap / 2 > kListCap ? kFastCap / 2 : kListCap];
  uint32_t* list = list_words;
  uint16_t* fast_rows = reinterpret_cast<uint16_t*>(list_words);
  __shared__ uint32_t list_n;
  __shared__ uint32_t wave_tot[kWaves];
  __shared__ uint32_t fhist[5][256];        // pivot path: two sample digits, three digits on the survivor list
  __shared__ Pick pick_box[5];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const float* scores = scores_all + (int64_t)blockIdx.x * score_stride;
  int32_t* sel = sel_all + (int64_t)blockIdx.x * topk;
  if (sample_rank > 0)
    for (int i = tid; i < 5 * 256; i += kThreads) (&fhist[0][0])[i] = 0u;  // ordered by the barriers of the load

  // Load with lane-contiguous 16-byte reads (a wave reads 1 KB at a time), then hand every thread its
  // C consecutive rows through LDS. The 16-byte pieces of a thread's C/4-piece block are XOR-permuted
  // by the thread index so that neither the writes nor the reads pile up on a few banks.
  uint32_t kreg[C];
  constexpr int kPieces = C / 4;  // 16-byte pieces per thread
  {
    const bool vec_ok = (reinterpret_cast<uintptr_t>(scores) & 15u) == 0u && n_rows >= 4;  // uniform
    // all vector loads first, unconditionally (a piece that crosses the end of the row re-reads the
    // last whole piece and is patched element by element below)
    f32x4_t v[kPieces];
    const int last_whole = (n_rows - 4) & ~3;
    if (vec_ok) {
#pragma unroll
      for (int k = 0; k < kPieces; k++) {
        const int r = 4 * (k * kThreads + tid);
        v[k] = *reinterpret_cast<const f32x4_t*>(scores + (r < last_whole ? r : last_whole));
      }
    }
#pragma unroll
    for (int k = 0; k < kPieces; k++) {
      const int piece = k * kThreads + tid;  // global piece index: rows 4*piece .. 4*piece+3
      const int r = 4 * piece;
      u32x4_t keys;
      if (vec_ok && r + 3 < n_rows) {
        keys = u32x4_t{score_key(v[k].x), score_key(v[k].y), score_key(v[k].z), score_key(v[k].w)};
      } else {
#pragma unroll
        for (int e = 0; e < 4; e++) keys[e] = r + e < n_rows ? score_key(scores[r + e]) : 0u;
      }
      const int owner = piece / kPieces, j = piece % kPieces;
      *reinterpret_cast<u32x4_t*>(&stage[owner * C + 4 * (j ^ (owner & (kPieces - 1)))]) = keys;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kPieces; j++) {
      const u32x4_t keys = *reinterpret_cast<const u32x4_t*>(&stage[tid * C + 4 * (j ^ (tid & (kPieces - 1)))]);
#pragma unroll
      for (int e = 0; e < 4; e++) kreg[4 * j + e] = keys[e];
    }
  }

  // ---- pivot path. Every thread's first row is a sample of the (padded) row set; the 16-bit key
  // prefix at rank `sample_rank` of the sample sits, with a wide margin, below the k-th key of the
  // whole row, so the rows at or above it ("survivors", a few thousand) contain the answer. They are
  // compacted in row order and the exact select and the emission run on that list only. Whether the
  // pivot was good is checked exactly (survivors >= k, within the list capacity, k-th key less than
  // 255 prefixes above the pivot); if not, the full radix passes below take over, so the result never
  // depends on the sample. The keys stay in the staging area, which this path does not overwrite.
  // one wave works out the digit, the others wait for it: with 16 waves on 4 SIMDs a computation that
  // every wave repeats costs four times its instruction count, a barrier costs less (a slot per use,
  // so no slot is rewritten while a slow wave may still read it)
  auto shared_pick = [&](const uint32_t* h, uint32_t want, int slot) -> Pick {
    if (wave == 0) {
      const Pick p = pick_bucket(h, want, lane);
      if (lane == 0) pick_box[slot] = p;
    }
    __syncthreads();
    return pick_box[slot];
  };
  if (sample_rank > 0) {
    const uint32_t skey = kreg[0];
    wave_hist_add(fhist[0], (int)(skey >> 24), lane);  // the top byte is shared by most rows: vote per wave
    __syncthreads();
    const Pick s0 = shared_pick(fhist[0], (uint32_t)sample_rank, 0);
    if ((skey >> 24) == s0.digit) atomicAdd(&fhist[1][(skey >> 16) & 0xFFu], 1u);
    __syncthreads();
    const Pick s1 = shared_pick(fhist[1], s0.need, 1);
    const uint32_t pivot16 = (s0.digit << 8) | s1.digit;
    const uint32_t pivot = pivot16 << 16;

    uint32_t smask = 0u;
#pragma unroll
    for (int i = C - 1; i >= 0; i--) smask = shift_in(smask, kreg[i] >= pivot);
    const uint32_t cnt = (uint32_t)__popc(smask);
    const uint32_t sincl = wave_prefix_sum(cnt);
    if (lane == 63) wave_tot[wave] = sincl;
    __syncthreads();
    uint32_t sbase = 0u, total = 0u;
#pragma unroll
    for (int w = 0; w < kWaves; w++) {
      const uint32_t wt = wave_tot[w];
      sbase += w < wave ? wt : 0u;
      total += wt;
    }
    if (total >= (uint32_t)topk && total <= (uint32_t)kFastCap) {  // the same for every thread
      uint32_t pos = sbase + sincl - cnt;
      while (smask) {
        const int i = __builtin_ctz(smask);
        smask &= smask - 1u;
        fast_rows[pos++] = (uint16_t)(C * tid + i);
      }
      __syncthreads();
      // thread t takes the list entries [t E, t E + E): consecutive, so the emission order is again a
      // matter of one block scan
      const uint32_t per = (total + kThreads - 1) / kThreads;  // 1 .. kFastPer
      uint32_t lk[kFastPer], lr[kFastPer];
      uint32_t lvalid = 0u;
#pragma unroll
      for (int j = 0; j < kFastPer; j++) {
        const uint32_t idx = (uint32_t)tid * per + j;
        const bool ok = (uint32_t)j < per && idx < total;
        const uint32_t row = fast_rows[ok ? idx : 0u];
        const uint32_t owner = row / C, piece = (row % C) >> 2, e = row & 3u;
        lr[j] = row;
        lk[j] = stage[owner * C + 4 * (piece ^ (owner & (kPieces - 1))) + e];
        lvalid |= (ok ? 1u : 0u) << j;
      }
      // digit A: distance of the 16-bit prefix from the pivot's, everything 255 or more prefixes up in
      // one bin; digits B and C: the low 16 bits
      uint32_t* hA = fhist[2];
#pragma unroll
      for (int j = 0; j < kFastPer; j++) {
        const uint32_t d = (lk[j] >> 16) - pivot16;
        if ((lvalid >> j) & 1u) atomicAdd(&hA[d < 255u ? d : 255u], 1u);
      }
      __syncthreads();
      const Pick pa = shared_pick(hA, (uint32_t)topk, 2);
      if (pa.digit < 255u) {  // the same for every thread
        uint32_t fprefix = (pivot16 + pa.digit) << 16, fneed = pa.need;
#pragma unroll
        for (int pass = 2; pass < 4; pass++) {
          const uint32_t shift = 24u - 8u * pass;
          const uint32_t mask_hi = 0xFFFFFFFFu << (shift + 8u);
          uint32_t* h = fhist[1 + pass];
#pragma unroll
          for (int j = 0; j < kFastPer; j++)
            if (((lvalid >> j) & 1u) && (lk[j] & mask_hi) == fprefix) atomicAdd(&h[(lk[j] >> shift) & 0xFFu], 1u);
          __syncthreads();
          const Pick pk = shared_pick(h, fneed, 1 + pass);
          fprefix |= pk.digit << shift;
          fneed = pk.need;
        }
        const uint32_t n_above_f = (uint32_t)topk - fneed;
        uint32_t am = 0u, tm = 0u;
#pragma unroll
        for (int j = 0; j < kFastPer; j++) {
          const bool ok = (lvalid >> j) & 1u;
          am |= (ok && lk[j] > fprefix ? 1u : 0u) << j;
          tm |= (ok && lk[j] == fprefix ? 1u : 0u) << j;
        }
        const uint32_t mine_f = (uint32_t)__popc(am) | ((uint32_t)__popc(tm) << 16);
        const uint32_t incl_f = wave_prefix_sum(mine_f);
        if (lane == 63) wave_tot[wave] = incl_f;  // its earlier contents were consumed before the barriers above
        __syncthreads();
        uint32_t base_f = 0u;
        for (int w = 0; w < wave; w++) base_f += wave_tot[w];
        const uint32_t excl_f = base_f + incl_f - mine_f;
        uint32_t slot_f = excl_f & 0xFFFFu;
        uint32_t rank_f = excl_f >> 16;
#pragma unroll
        for (int j = 0; j < kFastPer; j++) {
          if ((am >> j) & 1u) sel[slot_f++] = (int32_t)lr[j];
          else if (((tm >> j) & 1u) && rank_f < fneed) sel[n_above_f + rank_f++] = (int32_t)lr[j];
        }
        return;
      }
    }
  }
  __syncthreads();  // the staging area and wave_tot have been read by every thread; the full passes reuse them

  {
    u32x4_t* h4 = reinterpret_cast<u32x4_t*>(hist);
    for (int i = tid; i < 256 * kCp / 4; i += kThreads) h4[i] = u32x4_t{0u, 0u, 0u, 0u};
    if (tid < 512) (&small_hist[0][0])[tid] = 0u;
    if (tid == 0) list_n = 0u;
  }
  __syncthreads();

  uint32_t prefix = 0u, need = (uint32_t)topk, live = (uint32_t)(C * kThreads);

  // one digit over every key of the thread
  auto full_pass = [&](int pass) {
    const uint32_t shift = 24u - 8u * pass;
    const uint32_t mask_hi = pass == 0 ? 0u : (0xFFFFFFFFu << (shift + 8u));
#pragma unroll
    for (int i = 0; i < C; i++) {
      const uint32_t key = kreg[i];
      if (pass == 0 || (key & mask_hi) == prefix)
        atomicAdd(&hist[((key >> shift) & 0xFFu) * kCp + (lane & (kCp - 1))], 1u);
    }
    __syncthreads();
    // totals[bin] = sum over copies: four threads per bin, a quarter of the copies each as 16-byte reads
    // (rotated so that 16 neighbouring lanes cover all 16 bank groups), zeroed behind the read
    {
      const int bin = tid >> 2, q = tid & 3;
      uint32_t sum = 0u;
#pragma unroll
      for (int j = 0; j < kCp / 16; j++) {
        u32x4_t* p = reinterpret_cast<u32x4_t*>(&hist[bin * kCp + q * (kCp / 4) + 4 * ((j + (tid >> 2)) & (kCp / 16 - 1))]);
        const u32x4_t v = *p;
        *p = u32x4_t{0u, 0u, 0u, 0u};
        sum += v.x + v.y + v.z + v.w;
      }
      sum += __shfl_xor(sum, 1, MSPR_WAVE);
      sum += __shfl_xor(sum, 2, MSPR_WAVE);
      if (q == 0) totals[bin] = sum;
    }
    __syncthreads();
    const Pick p = pick_bucket(totals, need, lane);
    prefix |= p.digit << shift;
    need = p.need;
    live = p.live;
  };

  full_pass(0);
  full_pass(1);

  if (live <= (uint32_t)kListCap) {
    // the keys that still match the 16-bit prefix are few: finish the select on a compacted list
#pragma unroll
    for (int i = 0; i < C; i++) {
      const uint32_t key = kreg[i];
      if ((key & 0xFFFF0000u) == prefix) list[atomicAdd(&list_n, 1u)] = key;
    }
    __syncthreads();
    const uint32_t n_list = list_n;
#pragma unroll
    for (int pass = 2; pass < 4; pass++) {
      const uint32_t shift = 24u - 8u * pass;
      const uint32_t mask_hi = 0xFFFFFFFFu << (shift + 8u);
      uint32_t* h = small_hist[pass - 2];
      for (uint32_t i = tid; i < n_list; i += kThreads) {
        const uint32_t key = list[i];
        if ((key & mask_hi) == prefix) atomicAdd(&h[(key >> shift) & 0xFFu], 1u);
      }
      __syncthreads();
      const Pick p = pick_bucket(h, need, lane);
      prefix |= p.digit << shift;
      need = p.need;
      live = p.live;
    }
  } else {
    full_pass(2);
    full_pass(3);
  }

  const uint32_t threshold = prefix;
  const uint32_t need_ties = need;
  const uint32_t n_above = (uint32_t)topk - need_ties;

  // ---- ordered emission: per-thread masks, one packed block scan (above count low, tie count high)
  uint32_t above_mask = 0u, tie_mask = 0u;
#pragma unroll
  for (int i = 0; i < C; i++) {
    above_mask |= (kreg[i] > threshold ? 1u : 0u) << i;
    tie_mask |= (kreg[i] == threshold ? 1u : 0u) << i;
  }
  const uint32_t mine = (uint32_t)__popc(above_mask) | ((uint32_t)__popc(tie_mask) << 16);
  const uint32_t incl = wave_prefix_sum(mine);
  if (lane == 63) wave_tot[wave] = incl;
  __syncthreads();
  uint32_t base = 0u;
  for (int w = 0; w < wave; w++) base += wave_tot[w];
  const uint32_t excl = base + incl - mine;
  uint32_t slot_a = excl & 0xFFFFu;
  uint32_t rank_t = excl >> 16;
  const int row0 = C * tid;
  while (above_mask) {
    const int i = __builtin_ctz(above_mask);
    above_mask &= above_mask - 1u;
    sel[slot_a++] = row0 + i;
  }
  while (tie_mask && rank_t < need_ties) {
    const int i = __builtin_ctz(tie_mask);
    tie_mask &= tie_mask - 1u;
    sel[n_above + rank_t++] = row0 + i;
  }
}

// Short rows, one row per workgroup of 256 threads. A prefill chunk selects for thousands of tokens at once over a
// pool of a few hundred to two thousand rows: with 1024 threads a row a CU holds two of them, with 256 it holds
// eight, and each spends less on barriers. Thread t owns the C consecutive rows [C t, C t + C) (read coalesced,
// handed over through LDS); four 8-bit digit passes, each with a histogram of its own (zeroed once, so a pass costs
// one barrier), votes of a wave for one bin merged into one atomic; every wave derives the select state from the
// same totals. Rows past n_rows get key 0 as in the blocked kernel. Emission as there.
constexpr int kSmallThreads = 256;
template <int C>
__global__ __launch_bounds__(kSmallThreads) void topk_small_kernel(const float* __restrict__ scores_all,
                                                                   int64_t score_stride, int n_rows, int topk,
                                                                   int32_t* __restrict__ sel_all) {
  __shared__ __attribute__((aligned(16))) uint32_t stage[C * kSmallThreads];
  __shared__ uint32_t hist[4][256];
  __shared__ uint32_t wave_tot[kSmallThreads / 64];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const float* scores = scores_all + (int64_t)blockIdx.x * score_stride;
  int32_t* sel = sel_all + (int64_t)blockIdx.x * topk;

#pragma unroll
  for (int i = 0; i < 4; i++) (&hist[0][0])[i * kSmallThreads + tid] = 0u;
#pragma unroll
  for (int j = 0; j < C; j++) {
    const int e = j * kSmallThreads + tid;
    stage[e] = e < n_rows ? score_key(scores[e]) : 0u;
  }
  __syncthreads();
  uint32_t kreg[C];
#pragma unroll
  for (int i = 0; i < C; i++) kreg[i] = stage[C * tid + i];

  uint32_t prefix = 0u, need = (uint32_t)topk;
#pragma unroll
  for (int pass = 0; pass < 4; pass++) {
    const uint32_t shift = 24u - 8u * (uint32_t)pass;
    const uint32_t mask_hi = pass == 0 ? 0u : 0xFFFFFFFFu << (shift + 8u);
#pragma unroll
    for (int i = 0; i < C; i++) {
      const int bin = (kreg[i] & mask_hi) == prefix ? (int)((kreg[i] >> shift) & 0xFFu) : -1;
      wave_hist_add(hist[pass], bin, lane);
    }
    __syncthreads();
    const Pick p = pick_bucket(hist[pass], need, lane);
    prefix |= p.digit << shift;
    need = p.need;
  }
  const uint32_t threshold = prefix;
  const uint32_t need_ties = need;
  const uint32_t n_above = (uint32_t)topk - need_ties;

  // ---- ordered emission: per-thread masks, one packed block scan (above count low, tie count high)
  uint32_t above_mask = 0u, tie_mask = 0u;
#pragma unroll
  for (int i = 0; i < C; i++) {
    above_mask |= (kreg[i] > threshold ? 1u : 0u) << i;
    tie_mask |= (kreg[i] == threshold ? 1u : 0u) << i;
  }
  const uint32_t mine = (uint32_t)__popc(above_mask) | ((uint32_t)__popc(tie_mask) << 16);
  const uint32_t incl = wave_prefix_sum(mine);
  if (lane == 63) wave_tot[wave] = incl;
  __syncthreads();
  uint32_t base = 0u;
  for (int w = 0; w < wave; w++) base += wave_tot[w];
  const uint32_t excl = base + incl - mine;
  uint32_t slot_a = excl & 0xFFFFu;
  uint32_t rank_t = excl >> 16;
  const int row0 = C * tid;
  while (above_mask) {
    const int i = __builtin_ctz(above_mask);
    above_mask &= above_mask - 1u;
    sel[slot_a++] = row0 + i;
  }
  while (tie_mask && rank_t < need_ties) {
    const int i = __builtin_ctz(tie_mask);
    tie_mask &= tie_mask - 1u;
    sel[n_above + rank_t++] = row0 + i;
  }
}

// Rank, inside the 1024-row sample, of the pivot of the pivot path; 0 switches the path off. With k of
// the C*1024 (padded) rows wanted, k/C sample rows are expected above the k-th key; the rank adds 4.5
// standard deviations so that the survivors almost always include it, and the path is used only where
// the survivors then almost always (6 more deviations) fit the list. A miss on either side costs time,
// not correctness: the kernel checks the survivor count and falls back to the full passes.
int pivot_sample_rank(int c, int topk) {
  const double expect = (double)topk / c;
  const double rank = std::ceil(expect + 4.5 * std::sqrt(expect) + 2.0);
  const double worst = rank * c + 6.0 * c * std::sqrt(rank);
  if (rank > 512.0 || worst > (double)kFastCap) return 0;
  return (int)rank;
}

}  // namespace

int mspr_launch_topk(const float* scores, int64_t score_stride, int batch, int64_t n_rows, int topk, int32_t* sel,
                     hipStream_t st) {
  dim3 grid((unsigned)batch), block(kThreads);
  MsprProfScope prof(MSPR_K_TOPK, st);
  if (n_rows <= 4 * kSmallThreads)
    topk_small_kernel<4><<<grid, dim3(kSmallThreads), 0, st>>>(scores, score_stride, (int)n_rows, topk, sel);
  else if (n_rows <= 8 * kSmallThreads)
    topk_small_kernel<8><<<grid, dim3(kSmallThreads), 0, st>>>(scores, score_stride, (int)n_rows, topk, sel);
  // (many rows of up to 4096 scores: more rows resident per CU beats more threads per row; measured at 3844 rows,
  // k = 512: 84 against 111 us at 2500 scores, 92 against 113 at 4000, but 218 against 145 at 7961)
  else if (batch >= 128 && n_rows <= 16 * kSmallThreads)
    topk_small_kernel<16><<<grid, dim3(kSmallThreads), 0, st>>>(scores, score_stride, (int)n_rows, topk, sel);
  else if (n_rows <= 8 * 1024)
    topk_blocked_kernel<8><<<grid, block, 0, st>>>(scores, score_stride, (int)n_rows, topk, pivot_sample_rank(8, topk), sel);
  else if (n_rows <= 32 * 1024)
    topk_blocked_kernel<32><<<grid, block, 0, st>>>(scores, score_stride, (int)n_rows, topk, pivot_sample_rank(32, topk), sel);
  else topk_select_kernel<0><<<grid, block, 0, st>>>(scores, score_stride, n_rows, topk, sel);
  MSPR_CHECK_LAUNCH("topk_select");
  return MSPR_OK;
}

extern "C" int mspr_topk_select(const float* scores, int64_t score_stride, int batch, int64_t n_rows, int topk,
                                int32_t* sel, void* stream) {
  MSPR_REQUIRE(scores && sel, "topk_select: null pointer");
  MSPR_REQUIRE(batch >= 1, "topk_select: batch must be positive");
  MSPR_REQUIRE(n_rows >= 1 && n_rows < (int64_t)1 << 31, "topk_select: n_rows must be in [1, 2^31)");
  MSPR_REQUIRE(topk >= 1 && topk <= n_rows, "topk_select: topk must be positive and at most n_rows");
  MSPR_REQUIRE(score_stride >= n_rows, "topk_select: score_stride must cover a row");
  return mspr_launch_topk(scores, score_stride, batch, n_rows, topk, sel, (hipStream_t)stream);
}
