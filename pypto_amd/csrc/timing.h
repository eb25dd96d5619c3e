// Optional per-kernel timing with HIP events recorded on the launch stream (off by default).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pto {

enum KernelId { KID_INDEXER_SCORE = 0, KID_INDEXER_TOPK = 1, KID_SFA_DECODE = 2, KID_SFA_COMBINE = 3, KID_INDEXER_SELECT = 4, KID_SELECT_EXPERTS = 5, KID_GQA_DECODE = 6, KID_GQA_COMBINE = 7, KID_APQ_NORM = 8, KID_PROLOG_Q = 9, KID_APQ_GEMM = 10, KID_PROLOG_K = 11, KID_MLA_XA = 12, KID_MLA_NORM = 13, KID_MLA_QB = 14, KID_MLA_WUK = 15, KID_APQ_HEAD = 16, KID_PAGED_GATHER = 17, KID_COUNT = 18 };

bool timing_enabled();
void timing_set(bool on);
// Record an event pair around one kernel launch; no-ops while timing is off.
void timing_begin(int kid, hipStream_t s);
void timing_end(int kid, hipStream_t s);
// Wait for the recorded events, return their summed duration and count, and forget them.
hipError_t timing_collect(int kid, double* total_ms, uint64_t* launches);

// The instrument's own offset: an event pair around an empty kernel, less that kernel's duration.
hipError_t timing_pair_overhead(hipStream_t s, double* ms_out);

struct ScopedKernelTimer {
    int kid;
    hipStream_t s;
    ScopedKernelTimer(int k, hipStream_t st) : kid(k), s(st) { timing_begin(kid, s); }
    ~ScopedKernelTimer() { timing_end(kid, s); }
};

} // namespace pto
