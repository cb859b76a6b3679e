// Entry points that are not kernels: constants, the chunking rule, error strings.
#include <stdio.h>
#include "bhi_common.h"
#include "bhi_host.h"

static thread_local char g_err[256] = "";

int bhi_fail(int code, const char* msg) {
    snprintf(g_err, sizeof(g_err), "%s", msg);
    return code;
}

int bhi_launch_status(const char* what) {
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) return 0;
    snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
    return (int)e;
}

extern "C" const char* bhi_last_error_string(void) { return g_err; }

extern "C" int bhi_constants(int32_t* out, int n) {
    const int32_t v[] = {
        bhi::kFormatVersion, bhi::kLanes, bhi::kGroupRows, bhi::kStepCols, bhi::kTableBits,
        bhi::kWindowWords, bhi::kHeaderBits, bhi::kMaxBatch, bhi::kAnsPrecision,
        bhi::kAlignWords, bhi::kTailPadWords, bhi::kTargetTasks, bhi::kMaxTaskSteps,
    };
    const int total = (int)(sizeof(v) / sizeof(v[0]));
    for (int i = 0; out && i < n && i < total; ++i) out[i] = v[i];
    return total;
}

extern "C" int bhi_chunks_per_group(int M, int Ks, int split_k) {
    if (M < bhi::kGroupRows || Ks < bhi::kStepCols || split_k < 1) return bhi_fail(BHI_EINVAL, "bad shape");
    return bhi::chunks_per_group(M, Ks, split_k);
}
