// Internal hooks of the optional per-kernel timing (see profile.hip).
#pragma once
#include <hip/hip_runtime.h>

// kernel ids used in the mask of mspr_profile_enable and in mspr_profile_collect
#define MSPR_K_INDEXER_FP8 1
#define MSPR_K_TOPK 2
#define MSPR_K_SPARSE_SPLIT 3
#define MSPR_K_SPARSE_MERGE 4
#define MSPR_K_SCORES_F32 5
#define MSPR_K_Q8_DECODE 6
#define MSPR_K_Q8_MERGE 7
#define MSPR_K_FLASH_PREFILL 8

bool mspr_prof_active(int kernel_id);
int mspr_prof_begin(int kernel_id, hipStream_t st);
void mspr_prof_end(int token, hipStream_t st);

// RAII bracket around one launch
struct MsprProfScope {
  int token;
  hipStream_t st;
  MsprProfScope(int kernel_id, hipStream_t s) : token(mspr_prof_begin(kernel_id, s)), st(s) {}
  ~MsprProfScope() { mspr_prof_end(token, st); }
};
