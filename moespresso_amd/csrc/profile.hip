// Optional per-kernel timing: when switched on, the launchers bracket selected kernels with HIP
// events on the launch stream, so a benchmark can read GPU-side durations of individual kernels
// inside a multi-kernel step. Off by default; never active under stream capture.
#include <vector>

#include "common.h"
#include "profile.h"

namespace {

struct Record {
  hipEvent_t begin;
  hipEvent_t end;
  int kernel_id;
};

int g_mask = 0;
std::vector<Record> g_records;
std::vector<hipEvent_t> g_free;

hipEvent_t take_event() {
  if (!g_free.empty()) {
    hipEvent_t e = g_free.back();
    g_free.pop_back();
    return e;
  }
  hipEvent_t e = nullptr;
  if (hipEventCreate(&e) != hipSuccess) return nullptr;
  return e;
}

}  // namespace

bool mspr_prof_active(int kernel_id) { return (g_mask >> kernel_id) & 1; }

int mspr_prof_begin(int kernel_id, hipStream_t st) {
  if (!mspr_prof_active(kernel_id)) return -1;
  Record r{take_event(), take_event(), kernel_id};
  if (!r.begin || !r.end) return -1;
  if (hipEventRecord(r.begin, st) != hipSuccess) return -1;
  g_records.push_back(r);
  return (int)g_records.size() - 1;
}

void mspr_prof_end(int token, hipStream_t st) {
  if (token < 0 || token >= (int)g_records.size()) return;
  (void)hipEventRecord(g_records[token].end, st);
}

extern "C" int mspr_profile_enable(int kernel_mask) {
  g_mask = kernel_mask;
  return MSPR_OK;
}

extern "C" int mspr_profile_collect(int kernel_id, float* ms_out, int max_n) {
  int n = 0;
  std::vector<Record> keep;
  for (const Record& r : g_records) {
    if (r.kernel_id != kernel_id) {
      keep.push_back(r);
      continue;
    }
    float ms = 0.0f;
    if (hipEventSynchronize(r.end) == hipSuccess && hipEventElapsedTime(&ms, r.begin, r.end) == hipSuccess &&
        ms_out && n < max_n) {
      ms_out[n++] = ms;
    }
    g_free.push_back(r.begin);
    g_free.push_back(r.end);
  }
  g_records.swap(keep);
  return n;
}
