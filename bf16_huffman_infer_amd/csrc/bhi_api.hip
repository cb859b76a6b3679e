// Entry points that are not kernels: constants, the chunking rule, error strings.
#include <stdio.h>
#include "bhi_task.h"

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
        (int32_t)sizeof(bhi_gemv_member),
    };
    const int total = (int)(sizeof(v) / sizeof(v[0]));
    for (int i = 0; out && i < n && i < total; ++i) out[i] = v[i];
    return total;
}

extern "C" int bhi_chunks_per_group(int M, int Ks, int split_k) {
    if (M < bhi::kGroupRows || Ks < bhi::kStepCols || split_k < 1) return bhi_fail(BHI_EINVAL, "bad shape");
    return bhi::chunks_per_group(M, Ks, split_k);
}

// A loop that only loads: `wavefronts` wavefronts each stream a contiguous span of `src`
// with four 16-byte loads in flight per lane and keep nothing.  It measures what this GPU
// delivers to a kernel with the fused GEMV's shape (one wavefront per task, a few KB in
// flight each) when there is no decode work at all: the ceiling the GEMV sits under.
namespace bhi {
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
template <bool NT>
__global__ __launch_bounds__(256) void stream_read_kernel(const uint32_t* __restrict__ src, long long words_per_wave,
                                                           uint32_t* __restrict__ sink) {
    const int lane = threadIdx.x & (kLanes - 1);
    const long long wave = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const uint32_t* base = src + wave * words_per_wave;
    uint32_t acc = 0;
    long long o = 0;
    for (; o + 4 * 4 * kLanes <= words_per_wave; o += 4 * 4 * kLanes) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const u32x4_t* q = (const u32x4_t*)(base + o + u * 4 * kLanes) + lane;
            const u32x4_t v = NT ? __builtin_nontemporal_load(q) : *q;
            acc += v.x ^ v.y ^ v.z ^ v.w;
        }
    }
    for (; o + 4 * kLanes <= words_per_wave; o += 4 * kLanes) {      // the last, shorter iteration
        const u32x4_t* q = (const u32x4_t*)(base + o) + lane;
        const u32x4_t v = NT ? __builtin_nontemporal_load(q) : *q;
        acc += v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9E3779B9u) sink[0] = acc;     // keeps the loads alive; not taken on real data
}
}  // namespace bhi

extern "C" int64_t bhi_stream_read(const void* src, int64_t bytes, int wavefronts, int nontemporal, void* sink, void* stream) {
    if (!src || !sink) return bhi_fail(BHI_EINVAL, "null pointer");
    if (wavefronts < 4 || wavefronts % 4 != 0 || bytes < 0) return bhi_fail(BHI_EINVAL, "wavefronts must be a positive multiple of 4");
    const long long chunk = 4 * bhi::kLanes;                           // words of one load of a wavefront
    const long long words_per_wave = bytes / 4 / wavefronts / chunk * chunk;
    if (words_per_wave > 0) {
        if (nontemporal)
            hipLaunchKernelGGL(bhi::stream_read_kernel<true>, dim3((unsigned)(wavefronts / 4)), dim3(256), 0, (hipStream_t)stream,
                               (const uint32_t*)src, words_per_wave, (uint32_t*)sink);
        else
            hipLaunchKernelGGL(bhi::stream_read_kernel<false>, dim3((unsigned)(wavefronts / 4)), dim3(256), 0, (hipStream_t)stream,
                               (const uint32_t*)src, words_per_wave, (uint32_t*)sink);
        if (int rc = bhi_launch_status("stream_read")) return -(int64_t)(rc > 0 ? rc : -rc);
    }
    return words_per_wave * 4 * wavefronts;
}

// ---------------------------------------------------------------------------------------------
// The two layer pieces the GEMV can take in front of its product, as kernels of their own: the
// unfused form of the same arithmetic (same reduction order, same roundings), used where the
// fused form does not apply (more than four rows) and as the reference the fused form is
// tested against bit for bit.
namespace bhi {
template <int BS>
__global__ __launch_bounds__(kBlockThreads) void rms_norm_kernel(const uint16_t* __restrict__ X, const uint16_t* __restrict__ gamma,
                                                                 uint16_t* __restrict__ out, int K, float eps) {
    __shared__ float part[kWavesPerBlock * BS];
    float r[BS];
    rms_scales_start<BS>(X, K, part);
    __syncthreads();
    rms_scales_finish<BS>(part, K, eps, r);
    const int p = blockIdx.x * blockDim.x + threadIdx.x;          // pair index
    if (p < K / 2) {
        const uint32_t g = ((const uint32_t*)gamma)[p];
#pragma unroll
        for (int b = 0; b < BS; ++b)
            ((uint32_t*)out)[(size_t)b * (K / 2) + p] = rms_pair(((const uint32_t*)X)[(size_t)b * (K / 2) + p], r[b], g);
    }
}

__global__ __launch_bounds__(256) void silu_mul_kernel(const uint32_t* __restrict__ gate, const uint32_t* __restrict__ up,
                                                       uint32_t* __restrict__ out, long long pairs) {
    const long long p = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (p < pairs) out[p] = silu_mul_pair(gate[p], up[p]);
}
}  // namespace bhi

extern "C" int bhi_rms_norm(const void* X, const void* gamma, void* out, int rows, int K, float eps, void* stream) {
    using namespace bhi;
    if (!X || !gamma || !out) return bhi_fail(BHI_EINVAL, "null pointer");
    if (rows < 1 || rows > 4 || K < 2 || K % 2 != 0) return bhi_fail(BHI_EINVAL, "rms_norm takes 1 to 4 rows of an even length");
    const dim3 grid((unsigned)((K / 2 + kBlockThreads - 1) / kBlockThreads)), block(kBlockThreads);
    const uint16_t *x = (const uint16_t*)X, *g = (const uint16_t*)gamma;
    uint16_t* o = (uint16_t*)out;
    switch (rows) {
        case 1: hipLaunchKernelGGL(rms_norm_kernel<1>, grid, block, 0, (hipStream_t)stream, x, g, o, K, eps); break;
        case 2: hipLaunchKernelGGL(rms_norm_kernel<2>, grid, block, 0, (hipStream_t)stream, x, g, o, K, eps); break;
        case 3: hipLaunchKernelGGL(rms_norm_kernel<3>, grid, block, 0, (hipStream_t)stream, x, g, o, K, eps); break;
        default: hipLaunchKernelGGL(rms_norm_kernel<4>, grid, block, 0, (hipStream_t)stream, x, g, o, K, eps); break;
    }
    return bhi_launch_status("rms_norm");
}

extern "C" int bhi_silu_mul(const void* gate, const void* up, void* out, int64_t n, void* stream) {
    if (!gate || !up || !out) return bhi_fail(BHI_EINVAL, "null pointer");
    if (n < 2 || n % 2 != 0) return bhi_fail(BHI_EINVAL, "silu_mul takes an even number of elements");
    const long long pairs = n / 2;
    hipLaunchKernelGGL(bhi::silu_mul_kernel, dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint32_t*)gate, (const uint32_t*)up, (uint32_t*)out, pairs);
    return bhi_launch_status("silu_mul");
}

// ---------------------------------------------------------------------------------------------
// A workspace of the fused matrix product back to the state the library expects (all zero): for
// a caller whose launch failed or was abandoned halfway, where counters may be left non-zero.
// A fill kernel, not a memset: it may be recorded into a graph.
namespace bhi {
__global__ __launch_bounds__(256) void zero_kernel(uint32_t* __restrict__ p, long long words) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += (long long)gridDim.x * blockDim.x) p[i] = 0u;
}
}  // namespace bhi

extern "C" int bhi_gemm_workspace_reset(void* workspace, int64_t workspace_bytes, void* stream) {
    if (!workspace || workspace_bytes < 0 || workspace_bytes % 4 != 0 || ((uintptr_t)workspace & 3) != 0)
        return bhi_fail(BHI_EINVAL, "workspace must be a 4-byte aligned region of whole words");
    const long long words = workspace_bytes / 4;
    if (words > 0) {
        const long long blocks = (words + 255) / 256;
        hipLaunchKernelGGL(bhi::zero_kernel, dim3((unsigned)(blocks < 1024 ? blocks : 1024)), dim3(256), 0, (hipStream_t)stream,
                           (uint32_t*)workspace, words);
    }
    return bhi_launch_status("gemm_workspace_reset");
}
