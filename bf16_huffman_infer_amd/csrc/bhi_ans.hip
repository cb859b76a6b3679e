// rANS path: fused decode+GEMV, decode-to-BF16 and the encoder, for gfx950.
//
// Stand-ins for the reference's gemv_bf16_ans / ans_decode / ans_encode
// (bf16_huffman_infer/src/kernel.cu:686-711, 851-875, 767-811) with the reference's state
// width, precision and table words (kernel.cu:647-683).  What differs is the
// renormalisation schedule: a lane owns one state and looks at it after every four
// symbols, which keeps the refill out of the per-symbol dependency chain and makes a
// lane's words plain rows of its task block.
#include "bhi_task.h"

namespace bhi {

constexpr int kAnsTableWords = 1 << kAnsPrecision;
constexpr int kAnsHalf = 4;                     // symbols between two looks at the state
constexpr int kAnsInitRows = 2;                 // rows 0, 1 of a lane: its initial state

// The decode table in LDS: one 8-byte entry per slot, built from the table buffer's words
// ((sym<<24)|(freq<<12)|rem, the reference's format) when a block starts:
//   word 0  freq                 -- an operand of the multiply as it stands
//   word 1  (sym << 23) | rem    -- rem in the low bits; the symbol where the upper half of the
//                                   word, moved into one half of a pair word, is `sym << 7`
// Read with one ds_read_b64, this saves the two field extractions per symbol and the shift per
// pair of the packed form (eight symbols a step: the kernel is bound by instruction issue).
struct AnsTable {
    static constexpr int kLdsWords = 2 * kAnsTableWords;
    static __device__ __forceinline__ uint2 expand(uint32_t w) {
        return make_uint2((w >> 12) & 0xFFFu, ((w >> 24) << 23) | (w & 0xFFFu));
    }
    template <int THREADS>
    struct Stage {
        static_assert(THREADS >= kAnsTableWords, "one slot per thread");
        uint32_t w;
        __device__ __forceinline__ void issue(const uint32_t* __restrict__ g) {
            if (THREADS == kAnsTableWords || (int)threadIdx.x < kAnsTableWords) w = g[threadIdx.x];
        }
        __device__ __forceinline__ void commit(uint32_t* __restrict__ lds) const {
            if (THREADS == kAnsTableWords || (int)threadIdx.x < kAnsTableWords) ((uint2*)lds)[threadIdx.x] = expand(w);
        }
    };
    static __device__ __forceinline__ void fill(uint32_t* __restrict__ lds, const uint32_t* __restrict__ g) {
        for (int i = threadIdx.x; i < kAnsTableWords; i += blockDim.x) ((uint2*)lds)[i] = expand(g[i]);
    }
};

struct AnsCodec {
    using Cursor = AnsCursor;
    using Table = AnsTable;
    static constexpr bool kTransformsX = true;    // kernels with RMSNorm / SiLU*mul in front of the product are built
    static constexpr int kTableWords = kAnsTableWords;
    static __device__ __forceinline__ bool variant(const uint8_t* __restrict__) { return false; }
    static __device__ __forceinline__ uint32_t variant_word(const uint8_t* __restrict__) { return 0u; }
    static __device__ __forceinline__ bool variant_test(uint32_t, const uint8_t* __restrict__) { return false; }
};

// What the encoder does to a state for one half-step, backwards over its four symbols.
// Returns false when some intermediate state would not fit 64 bits.
__device__ __forceinline__ bool ans_push4(uint64_t& x, const uint8_t (&s)[kAnsHalf],
                                          const uint32_t* __restrict__ freq, const uint32_t* __restrict__ cum) {
    bool fits = true;
#pragma unroll
    for (int j = kAnsHalf - 1; j >= 0; --j) {
        const uint64_t f = freq[s[j]];
        const uint64_t q = x / f;
        fits = fits && q < (1ull << 56);
        x = ((q & ((1ull << 56) - 1)) << 8) + (x % f) + cum[s[j]];
    }
    return fits;
}

// One wavefront per task; a lane runs its own encoder backwards over the task, twice:
// the first pass counts its words (the block gets as many rows as the longest lane),
// the second writes them in decoding order.
__global__ __launch_bounds__(kLanes)
void ans_encode_kernel(const uint8_t* __restrict__ data, const uint32_t* __restrict__ freq,
                       const uint32_t* __restrict__ cum, uint32_t* __restrict__ output,
                       uint32_t* __restrict__ output_lengths, int n_tasks, int n_steps, long long out_stride) {
    __shared__ uint32_t sf[256], sc[256];
    for (int i = threadIdx.x; i < 256; i += kLanes) { sf[i] = freq[i]; sc[i] = cum[i]; }
    __syncthreads();
    const int task = blockIdx.x;
    const int lane = threadIdx.x;
    if (task >= n_tasks) return;
    const uint2* dp = (const uint2*)(data + (size_t)task * n_steps * kLanes * kLaneCols) + lane;
    uint32_t* out = output + (size_t)task * out_stride;

    uint32_t mine = 0, rows = 0, total = 0;
    for (int pass = 0; pass < 2; ++pass) {
        uint64_t x = 1ull << 32;
        uint32_t n = 0;                                        // words emitted so far
        auto emit = [&](uint32_t w) {
            if (pass == 1) out[(size_t)(mine - 1 - n) * kLanes + lane] = w;
            ++n;
        };
        for (int t = n_steps - 1; t >= 0; --t) {
            const uint2 d = dp[(size_t)t * kLanes];
            for (int half = 1; half >= 0; --half) {
                const uint32_t w4 = half ? d.y : d.x;
                const uint8_t s[kAnsHalf] = {(uint8_t)w4, (uint8_t)(w4 >> 8), (uint8_t)(w4 >> 16), (uint8_t)(w4 >> 24)};
                uint64_t y = x;
                const bool keep = ans_push4(y, s, sf, sc) && x >= (1ull << 32);
                if (!keep) {
                    emit((uint32_t)x);
                    y = x >> 32;
                    ans_push4(y, s, sf, sc);
                }
                x = y;
            }
        }
        emit((uint32_t)(x >> 32));
        emit((uint32_t)x);
        if (pass == 0) {
            mine = n;
            rows = n;
            for (int o = 32; o > 0; o >>= 1) {
                const uint32_t r2 = __shfl_xor(rows, o);
                rows = r2 > rows ? r2 : rows;
            }
            total = (rows * kLanes + kAlignWords - 1) / kAlignWords * kAlignWords;
            if (lane == 0) output_lengths[task] = total;
            for (uint32_t r = mine; r < rows; ++r) out[(size_t)r * kLanes + lane] = 0;
            for (uint32_t i = rows * kLanes + lane; i < total; i += kLanes) out[i] = 0;
        }
    }
}

}  // namespace bhi

using namespace bhi;

static int check_ans_args(const void* A_rem, const void* A_exp, const void* Y, const void* offsets, const void* LUT) {
    if (!A_rem || !A_exp || !Y || !offsets || !LUT) return bhi_fail(BHI_EINVAL, "null pointer");
    return 0;
}

extern "C" int bhi_gemv_bf16_ans(const void* A_rem, const void* A_exp, int64_t exp_words,
                                 const void* X, void* Y, const void* offsets, const void* LUT,
                                 int split_k, int M, int Ks, int batch, void* stream) {
    if (int rc = check_ans_args(A_rem, A_exp, Y, offsets, LUT)) return rc;
    if (!X) return bhi_fail(BHI_EINVAL, "null pointer");
    if (batch < 1) return bhi_fail(BHI_EINVAL, "batch must be >= 1");
    if (batch > kMaxBatch) return bhi_fail(BHI_EBATCH, "fused GEMV supports batch <= 8");
    Shape s;
    if (int rc = check_shape(split_k, M, Ks, exp_words, &s)) return rc;
    launch_gemv_batch<AnsCodec>(batch, A_rem, A_exp, X, Y, offsets, LUT, nullptr, s, (hipStream_t)stream);
    return bhi_launch_status("gemv_bf16_ans");
}

extern "C" int bhi_gemv_bf16_ans_grouped(const bhi_gemv_member* members, int n_members, const void* X,
                                         int split_k, int Ks, int batch, void* stream) {
    if (int rc = gemv_grouped<AnsCodec>(members, n_members, X, split_k, Ks, batch, 0, true, (hipStream_t)stream)) return rc;
    return bhi_launch_status("gemv_bf16_ans_grouped");
}

extern "C" int bhi_gemv_bf16_ans_grouped_x(const bhi_gemv_member* members, int n_members, const void* X,
                                           int split_k, int Ks, int batch, int x_mode, const void* x_aux, float eps,
                                           void* stream) {
    if (int rc = gemv_grouped<AnsCodec>(members, n_members, X, split_k, Ks, batch, 0, true, (hipStream_t)stream,
                                        x_mode, x_aux, eps)) return rc;
    return bhi_launch_status("gemv_bf16_ans_grouped_x");
}

extern "C" int bhi_gemm_bf16_ans(const bhi_gemv_member* weight, const void* X, int split_k, int Ks, int batch,
                                 void* workspace, int64_t workspace_bytes, void* stream) {
    if (int rc = launch_mma<AnsCodec>(weight, 1, X, split_k, Ks, batch, workspace, workspace_bytes, 0, true,
                                      (hipStream_t)stream)) return rc;
    return bhi_launch_status("gemm_bf16_ans");
}

extern "C" int bhi_gemm_bf16_ans_grouped(const bhi_gemv_member* members, int n_members, const void* X, int split_k,
                                         int Ks, int batch, void* stream) {
    if (int rc = launch_mma<AnsCodec>(members, n_members, X, split_k, Ks, batch, nullptr, 0, 0, true,
                                      (hipStream_t)stream)) return rc;
    return bhi_launch_status("gemm_bf16_ans_grouped");
}

extern "C" int bhi_ans_decode(const void* A_rem, const void* A_exp, int64_t exp_words,
                              void* Y, const void* offsets, const void* LUT,
                              int split_k, int M, int Ks, void* stream) {
    if (int rc = check_ans_args(A_rem, A_exp, Y, offsets, LUT)) return rc;
    Shape s;
    if (int rc = check_shape(split_k, M, Ks, exp_words, &s)) return rc;
    launch_decode<AnsCodec>(A_rem, A_exp, Y, offsets, LUT, nullptr, s, (hipStream_t)stream);
    return bhi_launch_status("ans_decode");
}

extern "C" int64_t bhi_ans_encode_capacity(int n_steps) {
    if (n_steps < 1) return 0;
    // every half-step emits a word + the two words of the final state, per lane
    return (int64_t)kLanes * (2 * (int64_t)n_steps + kAnsInitRows) + kAlignWords;
}

extern "C" int bhi_ans_encode(const void* data, const void* freq, const void* cum,
                              void* output, void* output_lengths,
                              int n_tasks, int n_steps, int64_t out_stride, void* stream) {
    if (!data || !freq || !cum || !output || !output_lengths) return bhi_fail(BHI_EINVAL, "null pointer");
    if (n_tasks < 1 || n_steps < 1 || n_steps > kMaxTaskSteps)
        return bhi_fail(BHI_EINVAL, "need n_tasks >= 1 and 1 <= n_steps <= 128");
    if (out_stride < bhi_ans_encode_capacity(n_steps))
        return bhi_fail(BHI_EINVAL, "output rows shorter than bhi_ans_encode_capacity(n_steps)");
    hipLaunchKernelGGL(ans_encode_kernel, dim3((unsigned)n_tasks), dim3(kLanes), 0, (hipStream_t)stream,
                       (const uint8_t*)data, (const uint32_t*)freq, (const uint32_t*)cum,
                       (uint32_t*)output, (uint32_t*)output_lengths, n_tasks, n_steps, (long long)out_stride);
    return bhi_launch_status("ans_encode");
}
