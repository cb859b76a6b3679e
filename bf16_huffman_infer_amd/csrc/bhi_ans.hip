// rANS path (placeholder entry points until the kernels land).
#include "bhi_common.h"
#include "bhi_host.h"

extern "C" int bhi_gemv_bf16_ans(const void*, const void*, int64_t, const void*, void*, const void*, const void*,
                                 int, int, int, int, void*) { return bhi_fail(BHI_EINVAL, "rANS path not built"); }
extern "C" int bhi_ans_decode(const void*, const void*, int64_t, void*, const void*, const void*,
                              int, int, int, void*) { return bhi_fail(BHI_EINVAL, "rANS path not built"); }
extern "C" int bhi_ans_encode(const void*, const void*, const void*, void*, void*, int, int, int64_t, void*) {
    return bhi_fail(BHI_EINVAL, "rANS path not built");
}
extern "C" int64_t bhi_ans_encode_capacity(int) { return 0; }
