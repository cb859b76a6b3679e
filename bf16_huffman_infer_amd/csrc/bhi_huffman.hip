// Huffman path: fused decode+GEMV, decode-to-BF16 and the encoder, for gfx950.
//
// Stand-ins for the reference's gemv_bf16_huffman / huffman_decode / huffman_encode
// (bf16_huffman_infer/src/kernel.cu:419-442, 510-531, 590-610).  The reference walks
// one row per 32-lane warp with two private bitstreams per lane and two dependent
// byte-table reads per exponent; here one 64-lane wavefront walks four rows and one LDS
// read resolves two exponents.
#include <mutex>
#include "bhi_task.h"

namespace bhi {

struct HuffCodec {
    using Cursor = HuffCursor;
    static constexpr bool kTransformsX = true;    // kernels with RMSNorm / SiLU*mul in front of the product are built
    static constexpr int kTableWords = kTableEntries;
    using Table = PlainTable<kTableEntries>;
    // escaped pairs need the slower walk; the header says whether the matrix has any
    static __device__ __forceinline__ bool variant(const uint8_t* __restrict__ header) { return header_has_esc(header); }
    static __device__ __forceinline__ uint32_t variant_word(const uint8_t* __restrict__ header) { return header_flag_word(header); }
    static __device__ __forceinline__ bool variant_test(uint32_t w, const uint8_t* __restrict__ header) { return header_flag_test(w, header); }
};

// ------------------------------------------------------------------ encoder
// One wavefront per task: every lane packs its own codes into its own column of the
// task block; the block gets as many rows as the longest lane needs.
__global__ __launch_bounds__(kLanes)
void huffman_encode_kernel(const uint8_t* __restrict__ data, const uint32_t* __restrict__ enc,
                           uint32_t* __restrict__ output, uint32_t* __restrict__ output_lengths,
                           int n_tasks, int n_steps, long long out_stride) {
    const int task = blockIdx.x;
    const int lane = threadIdx.x;
    if (task >= n_tasks) return;
    const uint2* dp = (const uint2*)(data + (size_t)task * n_steps * kLanes * kLaneCols) + lane;
    uint32_t* out = output + (size_t)task * out_stride;
    const uint32_t esc_entry = enc[65536];

    // pass 1: sizes
    uint32_t bits = kHeaderBits, nesc = 0;
    for (int t = 0; t < n_steps; ++t) {
        uint2 d = dp[(size_t)t * kLanes];
        uint32_t pr[4] = {d.x & 0xFFFFu, d.x >> 16, d.y & 0xFFFFu, d.y >> 16};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t en = enc[pr[q]];
            if ((en >> 16) == 0) { en = esc_entry; nesc++; }
            bits += en >> 16;
        }
    }
    uint32_t rows = (bits + 31u) >> 5, sum_esc = nesc;
    for (int o = 32; o > 0; o >>= 1) {
        uint32_t r2 = __shfl_xor(rows, o);
        rows = r2 > rows ? r2 : rows;
        sum_esc += __shfl_xor(sum_esc, o);
    }
    const uint32_t body = rows * kLanes + sum_esc;
    const uint32_t total = (body + kAlignWords - 1) / kAlignWords * kAlignWords;
    if (lane == 0) output_lengths[task] = total;
    for (uint32_t i = body + lane; i < total; i += kLanes) out[i] = 0;

    // pass 2: emit
    uint64_t acc = 0;
    uint32_t fill = kHeaderBits, row = 0, eptr = 0;
    for (int t = 0; t < n_steps; ++t) {
        uint2 d = dp[(size_t)t * kLanes];
        uint32_t pr[4] = {d.x & 0xFFFFu, d.x >> 16, d.y & 0xFFFFu, d.y >> 16};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t en = enc[pr[q]];
            bool esc = (en >> 16) == 0;
            uint64_t m = ballot(esc);
            if (esc) {
                en = esc_entry;
                out[total - 1 - (eptr + lane_rank(m))] = pr[q];
            }
            eptr += (uint32_t)__builtin_popcountll(m);
            acc |= (uint64_t)(en & 0xFFFFu) << fill;          // fill < 32, code <= 11 bits
            fill += en >> 16;
            if (fill >= 32u) {
                out[(size_t)row * kLanes + lane] = (uint32_t)acc;
                acc >>= 32;
                fill -= 32u;
                row++;
            }
        }
    }
    for (; row < rows; ++row) {
        out[(size_t)row * kLanes + lane] = (uint32_t)acc;
        acc >>= 32;
    }
}

}  // namespace bhi

using namespace bhi;

extern "C" int bhi_huffman_decode(const void* A_rem, const void* A_exp, int64_t exp_words,
                                  void* Y, const void* offsets,
                                  const void* LUT1, int64_t lut1_bytes,
                                  const void*, const void*, const void*, const void* code_lengths,
                                  int split_k, int M, int Ks, void* stream) {
    if (!A_rem || !A_exp || !Y || !offsets || !LUT1 || !code_lengths) return bhi_fail(BHI_EINVAL, "null pointer");
    Shape s;
    if (lut1_bytes != (int64_t)kTableEntries * 4)
        return bhi_fail(BHI_ELAYOUT, "LUT1 must hold 2048 four-byte pair entries");
    if (int rc = check_shape(split_k, M, Ks, exp_words, &s)) return rc;
    launch_decode<HuffCodec>(A_rem, A_exp, Y, offsets, LUT1, code_lengths, s, (hipStream_t)stream);
    return bhi_launch_status("huffman_decode");
}

extern "C" int bhi_gemv_bf16_huffman(const void* A_rem, const void* A_exp, int64_t exp_words,
                                     const void* X, void* Y, const void* offsets,
                                     const void* LUT1, int64_t lut1_bytes,
                                     const void*, const void*, const void*, const void* code_lengths,
                                     int split_k, int M, int Ks, int batch, void* stream) {
    if (!A_rem || !A_exp || !X || !Y || !offsets || !LUT1 || !code_lengths) return bhi_fail(BHI_EINVAL, "null pointer");
    if (batch < 1) return bhi_fail(BHI_EINVAL, "batch must be >= 1");
    if (batch > kMaxBatch) return bhi_fail(BHI_EBATCH, "fused GEMV supports batch <= 8");
    Shape s;
    if (lut1_bytes != (int64_t)kTableEntries * 4)
        return bhi_fail(BHI_ELAYOUT, "LUT1 must hold 2048 four-byte pair entries");
    if (int rc = check_shape(split_k, M, Ks, exp_words, &s)) return rc;
    launch_gemv_batch<HuffCodec>(batch, A_rem, A_exp, X, Y, offsets, LUT1, code_lengths, s, (hipStream_t)stream);
    return bhi_launch_status("gemv_bf16_huffman");
}

extern "C" int bhi_gemv_bf16_huffman_grouped(const bhi_gemv_member* members, int n_members, const void* X,
                                             int split_k, int Ks, int batch, void* stream) {
    if (int rc = gemv_grouped<HuffCodec>(members, n_members, X, split_k, Ks, batch, (int64_t)kTableEntries * 4, false,
                                         (hipStream_t)stream)) return rc;
    return bhi_launch_status("gemv_bf16_huffman_grouped");
}

extern "C" int bhi_gemv_bf16_huffman_grouped_x(const bhi_gemv_member* members, int n_members, const void* X,
                                               int split_k, int Ks, int batch, int x_mode, const void* x_aux, float eps,
                                               void* stream) {
    if (int rc = gemv_grouped<HuffCodec>(members, n_members, X, split_k, Ks, batch, (int64_t)kTableEntries * 4, false,
                                         (hipStream_t)stream, x_mode, x_aux, eps)) return rc;
    return bhi_launch_status("gemv_bf16_huffman_grouped_x");
}

extern "C" int bhi_gemm_bf16_huffman(const bhi_gemv_member* weight, const void* X, int split_k, int Ks, int batch,
                                     void* workspace, int64_t workspace_bytes, void* stream) {
    if (int rc = launch_mma<HuffCodec>(weight, 1, X, split_k, Ks, batch, workspace, workspace_bytes,
                                       (int64_t)kTableEntries * 4, false, (hipStream_t)stream)) return rc;
    return bhi_launch_status("gemm_bf16_huffman");
}

extern "C" int bhi_gemm_bf16_huffman_grouped(const bhi_gemv_member* members, int n_members, const void* X, int split_k,
                                             int Ks, int batch, void* stream) {
    if (int rc = launch_mma<HuffCodec>(members, n_members, X, split_k, Ks, batch, nullptr, 0,
                                       (int64_t)kTableEntries * 4, false, (hipStream_t)stream)) return rc;
    return bhi_launch_status("gemm_bf16_huffman_grouped");
}

// The workspace of bhi_gemm_bf16_huffman_static: part of the library's image on every GPU
// that loads it, zero when the image is loaded, and -- like any workspace of these kernels --
// left with its counters at zero by every launch.
constexpr int64_t kStaticWorkspaceBytes = (int64_t)kMmaCounterBytes + (2 << 20);
static __device__ __align__(256) unsigned char scratch[kStaticWorkspaceBytes];

// The array's address on the current device.  `scratch` itself is only a host-side handle:
// each GPU holds its own copy at its own address, looked up once per device.
static int static_workspace(void** out) {
    constexpr int kMaxDevices = 64;
    static std::mutex lock;
    static void* known[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return bhi_fail(BHI_EINVAL, "no usable current device");
    std::lock_guard<std::mutex> hold(lock);
    if (!known[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            (void)hipGetLastError();
            return bhi_fail(BHI_EINVAL, "the library's built-in workspace has no address on this device");
        }
        known[dev] = p;
    }
    *out = known[dev];
    return 0;
}

extern "C" int bhi_gemm_bf16_huffman_static(const bhi_gemv_member* weight, const void* X, int split_k, int Ks, int batch,
                                            void* stream) {
    if (!weight) return bhi_fail(BHI_EINVAL, "null pointer");
    if (batch < 1 || batch > kMmaMaxBatch) return bhi_fail(BHI_EBATCH, "the fused matrix product takes 1 to 32 rows of X");
    Shape s;
    if (int rc = check_shape(split_k, weight->M, Ks, weight->exp_words, &s)) return rc;
    if (mma_workspace_bytes(s, batch) > kStaticWorkspaceBytes)
        return bhi_fail(BHI_EINVAL, "this product needs more than the 2 MiB of partial sums the built-in workspace holds: "
                                    "use bhi_gemm_bf16_huffman with a workspace of bhi_gemm_workspace_bytes(...) bytes");
    void* ws = nullptr;
    if (int rc = static_workspace(&ws)) return rc;
    if (int rc = launch_mma<HuffCodec>(weight, 1, X, split_k, Ks, batch, ws, kStaticWorkspaceBytes,
                                       (int64_t)kTableEntries * 4, false, (hipStream_t)stream)) return rc;
    return bhi_launch_status("gemm_bf16_huffman_static");
}

extern "C" int64_t bhi_gemm_static_workspace_bytes(void) { return kStaticWorkspaceBytes; }

// Everything the library looks up once per device (today: the address of the built-in
// workspace), looked up now, on the current device: a caller that will first use the library
// under stream capture calls this beforehand, outside the capture.
extern "C" int bhi_device_init(void) {
    void* ws = nullptr;
    return static_workspace(&ws);
}

extern "C" int64_t bhi_gemm_workspace_bytes(int split_k, int M, int Ks, int batch) {
    Shape s;
    if (batch < 1 || batch > kMmaMaxBatch) return bhi_fail(BHI_EBATCH, "the fused matrix product takes 1 to 32 rows of X");
    if (int rc = check_shape(split_k, M, Ks, kTailPadWords, &s)) return rc;
    return mma_workspace_bytes(s, batch);
}

extern "C" int64_t bhi_encode_capacity(int n_steps) {
    if (n_steps < 1) return 0;
    // every lane full of longest codes + every pair escaped + alignment
    int64_t lane_words = ((int64_t)kHeaderBits + (int64_t)n_steps * kPairsPerStep * kTableBits + 31) / 32;
    return (int64_t)kLanes * lane_words + (int64_t)n_steps * kPairsPerStep * kLanes + kAlignWords;
}

extern "C" int bhi_huffman_encode(const void* data, const void* LUT, void* output, void* output_lengths,
                                  int n_tasks, int n_steps, int64_t out_stride, void* stream) {
    if (!data || !LUT || !output || !output_lengths) return bhi_fail(BHI_EINVAL, "null pointer");
    if (n_tasks < 1 || n_steps < 1 || n_steps > kMaxTaskSteps)
        return bhi_fail(BHI_EINVAL, "need n_tasks >= 1 and 1 <= n_steps <= 128");
    if (out_stride < bhi_encode_capacity(n_steps))
        return bhi_fail(BHI_EINVAL, "output rows shorter than bhi_encode_capacity(n_steps)");
    hipLaunchKernelGGL(huffman_encode_kernel, dim3((unsigned)n_tasks), dim3(kLanes), 0, (hipStream_t)stream,
                       (const uint8_t*)data, (const uint32_t*)LUT, (uint32_t*)output, (uint32_t*)output_lengths,
                       n_tasks, n_steps, (long long)out_stride);
    return bhi_launch_status("huffman_encode");
}
