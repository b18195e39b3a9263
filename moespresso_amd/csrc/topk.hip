// Deterministic top-k over float32 score rows: four-pass MSB radix select on monotone uint32
// keys, then ordered emission (rows strictly above the k-th key in ascending row order, then the
// lowest-index rows tied with it).
//
// One 1024-thread workgroup per score row. For rows of up to CACHE*1024 scores every thread keeps
// its keys in registers (striped ownership: thread t owns rows t, t+1024, ...), so HBM/L2 is read
// once; longer rows re-read global memory each pass. Histograms are private per wave (16 x 256
// counters in LDS), so an LDS atomic only ever contends inside one wave.
#include "common.h"
#include "profile.h"

namespace {

constexpr int kThreads = 1024;
constexpr int kWaves = kThreads / 64;

struct SelectState {
  uint32_t prefix;
  uint32_t need;
};

template <int CACHE>
__global__ __launch_bounds__(kThreads) void topk_select_kernel(const float* __restrict__ scores_all,
                                                                int64_t score_stride, int64_t n_rows, int topk,
                                                                int32_t* __restrict__ sel_all) {
  __shared__ uint32_t hist[kWaves * 256];
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

  // keys of padding slots never match a live prefix group and never pass the threshold tests:
  // they are skipped through the `live` flag instead of a sentinel value.
  uint32_t kreg[CACHE > 0 ? CACHE : 1];
  if (CACHE > 0) {
#pragma unroll
    for (int i = 0; i < CACHE; i++) {
      int64_t r = (int64_t)i * kThreads + tid;
      kreg[i] = r < n_rows ? score_key(scores[r]) : 0u;
    }
  }
  if (tid == 0) {
    st.prefix = 0u;
    st.need = (uint32_t)topk;
  }

  for (int pass = 0; pass < 4; pass++) {
    const uint32_t shift = 24u - 8u * pass;
    for (int i = tid; i < kWaves * 256; i += kThreads) hist[i] = 0u;
    __syncthreads();
    const uint32_t prefix = st.prefix;
    const uint32_t mask_hi = pass == 0 ? 0u : (0xFFFFFFFFu << (shift + 8u));
    uint32_t* myhist = hist + wave * 256;
    if (CACHE > 0) {
#pragma unroll
      for (int i = 0; i < CACHE; i++) {
        int64_t r = (int64_t)i * kThreads + tid;
        uint32_t key = kreg[i];
        if (r < n_rows && (key & mask_hi) == prefix) atomicAdd(&myhist[(key >> shift) & 0xFFu], 1u);
      }
    } else {
      for (int64_t c = 0; c < n_chunks; c++) {
        int64_t r = c * kThreads + tid;
        if (r < n_rows) {
          uint32_t key = score_key(scores[r]);
          if ((key & mask_hi) == prefix) atomicAdd(&myhist[(key >> shift) & 0xFFu], 1u);
        }
      }
    }
    __syncthreads();
    if (wave == 0) {
      // lane l owns buckets 4l..4l+3; suffix sums from bucket 255 downward
      uint32_t t[4];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        uint32_t s = 0u;
        for (int w = 0; w < kWaves; w++) s += hist[w * 256 + 4 * lane + j];
        t[j] = s;
      }
      uint32_t lane_sum = t[0] + t[1] + t[2] + t[3];
      // inclusive suffix scan over lanes: sfx = sum of lane_sum over lanes >= lane
      uint32_t sfx = lane_sum;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        uint32_t o = __shfl_down(sfx, off, MSPR_WAVE);
        if (lane + off < 64) sfx += o;
      }
      const uint32_t need = st.need;
      uint32_t above_lane = sfx - lane_sum;  // count in buckets of higher lanes
      // walk this lane's buckets from the top: bucket b is chosen when the count at or above b
      // first reaches `need`
      int chosen = -1;
      uint32_t chosen_need = 0u;
      uint32_t run = above_lane;
#pragma unroll
      for (int j = 3; j >= 0; j--) {
        if (chosen < 0 && run < need && run + t[j] >= need) {
          chosen = 4 * lane + j;
          chosen_need = need - run;
        }
        run += t[j];
      }
      // exactly one lane chooses when the live count >= need; otherwise bucket 0 takes the rest
      uint64_t any = __ballot(chosen >= 0);
      if (any == 0ull) {
        if (lane == 0) {
          // count above bucket 0 = total - t[0]
          uint32_t total = sfx;
          st.prefix = prefix;  // bucket 0 adds no bits
          st.need = need - (total - t[0]);
        }
      } else if (chosen >= 0) {
        st.prefix = prefix | ((uint32_t)chosen << shift);
        st.need = chosen_need;
      }
    }
    __syncthreads();
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
    // E1: ballots per chunk
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
    // E2: exclusive scan over the (chunk, wave) entries, one per thread
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
    // E3: emit
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

}  // namespace

int mspr_launch_topk(const float* scores, int64_t score_stride, int batch, int64_t n_rows, int topk, int32_t* sel,
                     hipStream_t st) {
  dim3 grid((unsigned)batch), block(kThreads);
  MsprProfScope prof(MSPR_K_TOPK, st);
  if (n_rows <= 8 * 1024) topk_select_kernel<8><<<grid, block, 0, st>>>(scores, score_stride, n_rows, topk, sel);
  else if (n_rows <= 32 * 1024) topk_select_kernel<32><<<grid, block, 0, st>>>(scores, score_stride, n_rows, topk, sel);
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
