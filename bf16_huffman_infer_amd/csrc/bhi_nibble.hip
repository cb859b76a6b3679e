// Fixed-width ("nibble") exponent code: fused decode+GEMV, decode-to-BF16 and the encoder.
//
// Not one of the reference's codecs.  Entropy decoding on this GPU is bound by
// instruction issue and LDS lookups rather than by memory; storing every exponent as a
// 4-bit offset from a per-matrix base (escape list for the rest) gives up about nine
// percent of the size for a decoder without tables, cursors or serial dependencies.
// The entry points mirror the rANS ones (one int32 [256] LUT buffer: [0] base exponent,
// [1] nonzero when the matrix has escaped exponents).
#include "bhi_task.h"

namespace bhi {

constexpr uint32_t kNibbleEsc = 15;

struct NibbleCodec {
    using Cursor = NibbleCursor;
    static constexpr bool kTransformsX = false;    // kernels with RMSNorm / SiLU*mul in front of the product are built
    static constexpr int kTableWords = 4;          // base and flags, one 16-byte copy
    using Table = PlainTable<4>;
    static __device__ __forceinline__ uint32_t variant_word(const uint8_t* __restrict__ lut) {
        return constant_word((const uint32_t*)lut + 1);
    }
    static __device__ __forceinline__ bool variant_test(uint32_t w, const uint8_t* __restrict__) { return w != 0; }
    static __device__ __forceinline__ bool variant(const uint8_t* __restrict__ lut) { return variant_test(variant_word(lut), lut); }
};

// One wavefront per task: pass 1 counts escapes, pass 2 writes the rows and the escape
// list (raw exponents, (step, column, lane) order, backwards from the end of the block).
__global__ __launch_bounds__(kLanes)
void nibble_encode_kernel(const uint8_t* __restrict__ data, const uint32_t* __restrict__ lut,
                          uint32_t* __restrict__ output, uint32_t* __restrict__ output_lengths,
                          int n_tasks, int n_steps, long long out_stride) {
    const int task = blockIdx.x;
    const int lane = threadIdx.x;
    if (task >= n_tasks) return;
    const uint32_t base = lut[0] & 0xFFu;
    const uint2* dp = (const uint2*)(data + (size_t)task * n_steps * kLanes * kLaneCols) + lane;
    uint32_t* out = output + (size_t)task * out_stride;

    auto escaped = [&](uint32_t sym) { return sym - base >= kNibbleEsc; };     // unsigned: below the base wraps
    uint32_t nesc = 0;
    for (int t = 0; t < n_steps; ++t) {
        const uint2 d = dp[(size_t)t * kLanes];
#pragma unroll
        for (int j = 0; j < kLaneCols; ++j) nesc += escaped(((j < 4 ? d.x : d.y) >> (8 * (j & 3))) & 0xFFu);
    }
    for (int o = 32; o > 0; o >>= 1) nesc += __shfl_xor(nesc, o);
    const uint32_t body = (uint32_t)n_steps * kLanes + nesc;
    const uint32_t total = (body + kAlignWords - 1) / kAlignWords * kAlignWords;
    if (lane == 0) output_lengths[task] = total;
    for (uint32_t i = body + lane; i < total; i += kLanes) out[i] = 0;

    uint32_t eptr = 0;
    for (int t = 0; t < n_steps; ++t) {
        const uint2 d = dp[(size_t)t * kLanes];
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < kLaneCols; ++j) {
            const uint32_t sym = ((j < 4 ? d.x : d.y) >> (8 * (j & 3))) & 0xFFu;
            const bool esc = escaped(sym);
            const uint64_t m = ballot(esc);
            if (esc) out[total - 1 - (eptr + lane_rank(m))] = sym;
            eptr += (uint32_t)__builtin_popcountll(m);
            word |= (esc ? kNibbleEsc : sym - base) << (4 * j);
        }
        out[(size_t)t * kLanes + lane] = word;
    }
}

}  // namespace bhi

using namespace bhi;

extern "C" int bhi_gemv_bf16_nibble(const void* A_rem, const void* A_exp, int64_t exp_words,
                                    const void* X, void* Y, const void* offsets, const void* LUT,
                                    int split_k, int M, int Ks, int batch, void* stream) {
    if (!A_rem || !A_exp || !X || !Y || !offsets || !LUT) return bhi_fail(BHI_EINVAL, "null pointer");
    if (batch < 1) return bhi_fail(BHI_EINVAL, "batch must be >= 1");
    if (batch > kMaxBatch) return bhi_fail(BHI_EBATCH, "fused GEMV supports batch <= 8");
    Shape s;
    if (int rc = check_shape(split_k, M, Ks, exp_words, &s)) return rc;
    launch_gemv_batch<NibbleCodec>(batch, A_rem, A_exp, X, Y, offsets, LUT, LUT, s, (hipStream_t)stream);
    return bhi_launch_status("gemv_bf16_nibble");
}

extern "C" int bhi_gemv_bf16_nibble_grouped(const bhi_gemv_member* members, int n_members, const void* X,
                                            int split_k, int Ks, int batch, void* stream) {
    if (int rc = gemv_grouped<NibbleCodec>(members, n_members, X, split_k, Ks, batch, 0, true, (hipStream_t)stream)) return rc;
    return bhi_launch_status("gemv_bf16_nibble_grouped");
}

extern "C" int bhi_nibble_decode(const void* A_rem, const void* A_exp, int64_t exp_words,
                                 void* Y, const void* offsets, const void* LUT,
                                 int split_k, int M, int Ks, void* stream) {
    if (!A_rem || !A_exp || !Y || !offsets || !LUT) return bhi_fail(BHI_EINVAL, "null pointer");
    Shape s;
    if (int rc = check_shape(split_k, M, Ks, exp_words, &s)) return rc;
    launch_decode<NibbleCodec>(A_rem, A_exp, Y, offsets, LUT, LUT, s, (hipStream_t)stream);
    return bhi_launch_status("nibble_decode");
}

extern "C" int64_t bhi_nibble_encode_capacity(int n_steps) {
    if (n_steps < 1) return 0;
    // the rows + every exponent escaped + alignment
    return (int64_t)n_steps * kLanes + (int64_t)n_steps * kLaneCols * kLanes + kAlignWords;
}

extern "C" int bhi_nibble_encode(const void* data, const void* LUT, void* output, void* output_lengths,
                                 int n_tasks, int n_steps, int64_t out_stride, void* stream) {
    if (!data || !LUT || !output || !output_lengths) return bhi_fail(BHI_EINVAL, "null pointer");
    if (n_tasks < 1 || n_steps < 1 || n_steps > kMaxTaskSteps)
        return bhi_fail(BHI_EINVAL, "need n_tasks >= 1 and 1 <= n_steps <= 128");
    if (out_stride < bhi_nibble_encode_capacity(n_steps))
        return bhi_fail(BHI_EINVAL, "output rows shorter than bhi_nibble_encode_capacity(n_steps)");
    hipLaunchKernelGGL(nibble_encode_kernel, dim3((unsigned)n_tasks), dim3(kLanes), 0, (hipStream_t)stream,
                       (const uint8_t*)data, (const uint32_t*)LUT, (uint32_t*)output, (uint32_t*)output_lengths,
                       n_tasks, n_steps, (long long)out_stride);
    return bhi_launch_status("nibble_encode");
}
