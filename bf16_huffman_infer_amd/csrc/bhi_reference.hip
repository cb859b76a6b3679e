// Reader for weights compressed by the reference package itself (its layout, its tables):
// decodes them to the original BF16 matrix so that they can be re-encoded in this
// library's layout.  One thread per exponent stream, straight from the reference's rules;
// a conversion-time tool, not a hot path.
//
// Reference layout (bf16_huffman_infer/functional.py:129-242,297-310): row (k, r) has 64
// streams; stream g carries the exponents of columns k*Ks + c*128 + 2g + e (chunk c, then
// e = 0, 1); word w of stream g sits at A_exp[offsets[k, r] + 64*w + g]; inside each
// 128-column chunk of rem, column h*64 + 2l + e is stored at byte 4l + 2h + e.
// Decode rules: Huffman src/kernel.cu:354-380 (refill 32 bits when fewer than 32 are valid,
// four 256-entry byte tables tried in turn, 255 = miss); rANS src/kernel.cu:652-683
// (state = first word; refill when state < 256; slot = state & 255).
#include "bhi_common.h"
#include "bhi_host.h"

namespace bhi {

constexpr int kRefStreams = 64;

__device__ __forceinline__ void ref_store(uint16_t* __restrict__ Y, const uint8_t* __restrict__ rem_row,
                                          int col, uint32_t sym) {
    // position of column `col` of the split inside the permuted rem row
    const int chunk = col >> 7, in = col & 127;
    const int h = in >> 6, l = (in & 63) >> 1, e = in & 1;
    const uint32_t r = rem_row[chunk * 128 + 4 * l + 2 * h + e];
    Y[col] = (uint16_t)(((r << 8) & 0x8000u) | (r & 0x7Fu) | (sym << 7));
}

template <bool ANS>
__global__ __launch_bounds__(256)
void ref_decode_kernel(const uint8_t* __restrict__ A_rem, const uint32_t* __restrict__ A_exp, uint32_t exp_words,
                       uint16_t* __restrict__ Y, const uint32_t* __restrict__ offsets,
                       const uint8_t* __restrict__ LUT1, const uint8_t* __restrict__ LUT2,
                       const uint8_t* __restrict__ LUT3, const uint8_t* __restrict__ LUT4,
                       const uint8_t* __restrict__ code_lengths, const uint32_t* __restrict__ ans_lut,
                       int split_k, int M, int Ks) {
    const long long id = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long total = (long long)split_k * M * kRefStreams;
    if (id >= total) return;
    const int g = (int)(id % kRefStreams);
    const long long row = id / kRefStreams;              // k * M + r
    const int k = (int)(row / M), r = (int)(row % M);
    const uint8_t* rem_row = A_rem + (size_t)row * Ks;
    uint16_t* y = Y + (size_t)r * split_k * Ks + (size_t)k * Ks;
    uint32_t p = offsets[row] + g;
    auto next_word = [&]() -> uint64_t {
        const uint32_t w = p < exp_words ? A_exp[p] : 0u;   // the Huffman rule may look one word past a stream
        p += kRefStreams;
        return w;
    };
    const int L = Ks / kRefStreams;
    if (ANS) {
        uint64_t state = next_word();
        for (int i = 0; i < L; ++i) {
            if (state < 256) state = (state << 32) | next_word();
            const uint32_t e = ans_lut[state & 255];
            state = (uint64_t)((e >> 12) & 0xFFFu) * (state >> 8) + (e & 0xFFFu);
            ref_store(y, rem_row, (i >> 1) * 128 + 2 * g + (i & 1), e >> 24);
        }
    } else {
        uint64_t state = 0;
        int valid = 0;
        for (int i = 0; i < L; ++i) {
            if (valid < 32) { state |= next_word() << valid; valid += 32; }
            uint32_t s = LUT1[state & 0xFF];
            if (s == 255) s = LUT2[(state >> 8) & 0xFF];
            if (s == 255) s = LUT3[(state >> 16) & 0xFF];
            if (s == 255) s = LUT4[(state >> 24) & 0xFF];
            const int len = code_lengths[s];
            state >>= len;
            valid -= len;
            ref_store(y, rem_row, (i >> 1) * 128 + 2 * g + (i & 1), s);
        }
    }
}

}  // namespace bhi

using namespace bhi;

static int check_ref_dims(int split_k, int M, int Ks, int64_t exp_words) {
    if (split_k < 1 || M < 1 || Ks < 128 || Ks % 128 != 0)
        return bhi_fail(BHI_EINVAL, "need split_k >= 1, M >= 1 and Ks a multiple of 128");
    if (exp_words < 1 || exp_words >= ((int64_t)1 << 32)) return bhi_fail(BHI_EINVAL, "exponent stream size out of range");
    return 0;
}

extern "C" int bhi_reference_huffman_decode(const void* A_rem, const void* A_exp, int64_t exp_words,
                                            void* Y, const void* offsets,
                                            const void* LUT1, const void* LUT2, const void* LUT3, const void* LUT4,
                                            const void* code_lengths,
                                            int split_k, int M, int Ks, void* stream) {
    if (!A_rem || !A_exp || !Y || !offsets || !LUT1 || !LUT2 || !LUT3 || !LUT4 || !code_lengths)
        return bhi_fail(BHI_EINVAL, "null pointer");
    if (int rc = check_ref_dims(split_k, M, Ks, exp_words)) return rc;
    const long long total = (long long)split_k * M * kRefStreams;
    hipLaunchKernelGGL(ref_decode_kernel<false>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint8_t*)A_rem, (const uint32_t*)A_exp, (uint32_t)exp_words, (uint16_t*)Y,
                       (const uint32_t*)offsets, (const uint8_t*)LUT1, (const uint8_t*)LUT2, (const uint8_t*)LUT3,
                       (const uint8_t*)LUT4, (const uint8_t*)code_lengths, (const uint32_t*)nullptr, split_k, M, Ks);
    return bhi_launch_status("reference_huffman_decode");
}

extern "C" int bhi_reference_ans_decode(const void* A_rem, const void* A_exp, int64_t exp_words,
                                        void* Y, const void* offsets, const void* LUT,
                                        int split_k, int M, int Ks, void* stream) {
    if (!A_rem || !A_exp || !Y || !offsets || !LUT) return bhi_fail(BHI_EINVAL, "null pointer");
    if (int rc = check_ref_dims(split_k, M, Ks, exp_words)) return rc;
    const long long total = (long long)split_k * M * kRefStreams;
    hipLaunchKernelGGL(ref_decode_kernel<true>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint8_t*)A_rem, (const uint32_t*)A_exp, (uint32_t)exp_words, (uint16_t*)Y,
                       (const uint32_t*)offsets, (const uint8_t*)nullptr, (const uint8_t*)nullptr, (const uint8_t*)nullptr,
                       (const uint8_t*)nullptr, (const uint8_t*)nullptr, (const uint32_t*)LUT, split_k, M, Ks);
    return bhi_launch_status("reference_ans_decode");
}
