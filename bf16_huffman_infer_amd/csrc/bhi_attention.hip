// One token's attention step of a decoder layer in one launch: per-head RMSNorm and rotary
// embedding of the projected q and k heads, the write of k and v into the cache at the token's
// position, and the attention of the one query per head over the cache slots up to that
// position (grouped-query: several q heads share a k/v head).
//
// No counterpart in the reference, which leaves the attention to the model code it is given
// (transformers' attention over torch kernels).  It is here because the recorded decode step
// spends its time between the linear layers otherwise: written with torch operations this
// part is 14 kernels per layer, about 5 us each inside a graph, beside 4 launches of this
// library.  The position is read from device memory, so a recorded graph follows it.
//
// One block of 256 threads per q head.
//  1. Wavefront 0 normalises and rotates the q head, wavefront 1 the k head of the group
//     (lane l holds elements l and l + 64, the two halves the rotation pairs up); both go to
//     LDS, q in fp32 with the softmax scale applied, k rounded to BF16 as the cache holds it.
//     The group's first block writes k and v into the cache; every block takes the new
//     token's k and v from LDS / the input, so no block waits for another.
//  2. Scores: thread t owns cache slots t, t + 256, ...; a slot's k row is 256 contiguous
//     bytes, requested whole (sixteen 16-byte loads in flight) and multiplied with q from LDS
//     (broadcast reads).
//  3. Softmax over the block (fp32; maximum and sum through wavefront reductions and LDS),
//     the weights rounded to BF16 as a BF16 matrix product would take them.
//  4. Output: wavefront w sums slots w, w + 4, ...; lane l owns elements 2l and 2l + 1 of the
//     head (a v row is one 256-byte load of the wavefront); the four partial sums meet in LDS.
#include "bhi_common.h"
#include "bhi_host.h"

namespace bhi {

constexpr int kAttnDim = 128;          // head dimension the kernel is written for
constexpr int kAttnThreads = 256;
constexpr int kAttnMaxLen = 8192;      // cache slots: the weights of all of them sit in LDS

struct AttnArgs {
    const uint16_t* qk;        // bf16 [q_heads + kv_heads, 128]: the projections of the token
    const uint16_t* v;         // bf16 [kv_heads, 128]
    const uint16_t* norm_w;    // bf16 [q_heads + kv_heads, 128] RMSNorm weights per head, or null
    const float* cos;          // fp32 [max_len, 128]: cos(angle) for both halves
    const float* sin;          // fp32 [max_len, 128]: -sin for the first half, +sin for the second
    const long long* pos;      // the token's position (device memory)
    uint16_t* k_cache;         // bf16 [kv_heads, max_len, 128]
    uint16_t* v_cache;
    uint16_t* out;             // bf16 [q_heads, 128]
    int q_heads, kv_heads, max_len;
    float eps, scale;
};

__device__ __forceinline__ float bf16_lo(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t pair) { return __uint_as_float(pair & 0xFFFF0000u); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// RMSNorm (fp32, weight applied after the normalisation) and rotation of one head by one
// wavefront: returns the lane's two elements (l and l + 64), times `scale`
__device__ __forceinline__ float2 norm_rotate(const uint16_t* head, const uint16_t* w, const float* cos, const float* sin,
                                              int lane, float eps, float scale) {
    float a = __uint_as_float((uint32_t)head[lane] << 16), b = __uint_as_float((uint32_t)head[lane + 64] << 16);
    const float r = rsqrtf(wave_sum(a * a + b * b) * (1.0f / kAttnDim) + eps);
    a *= r;
    b *= r;
    if (w) {
        a *= __uint_as_float((uint32_t)w[lane] << 16);
        b *= __uint_as_float((uint32_t)w[lane + 64] << 16);
    }
    // out = x * cos + swap_halves(x) * sin, sin carrying the sign
    return make_float2((a * cos[lane] + b * sin[lane]) * scale, (b * cos[lane + 64] + a * sin[lane + 64]) * scale);
}

__global__ __launch_bounds__(kAttnThreads) void decode_attention_kernel(const AttnArgs a) {
    extern __shared__ float weights[];                 // [slots rounded up to 256]
    __shared__ float q[kAttnDim];
    __shared__ uint16_t k_new[kAttnDim];
    __shared__ float red[kAttnThreads / kLanes];
    __shared__ float part[kAttnThreads / kLanes][kAttnDim];

    const int tid = threadIdx.x, lane = tid & (kLanes - 1), wave = tid >> 6;
    const int h = blockIdx.x, group = a.q_heads / a.kv_heads, kh = h / group;
    long long p = *a.pos;
    p = p < 0 ? 0 : (p >= a.max_len ? a.max_len - 1 : p);
    const int n = (int)p + 1;                           // visible slots: 0 .. pos
    const uint16_t* kc = a.k_cache + (size_t)kh * a.max_len * kAttnDim;
    const uint16_t* vc = a.v_cache + (size_t)kh * a.max_len * kAttnDim;
    const float *cs = a.cos + (size_t)p * kAttnDim, *sn = a.sin + (size_t)p * kAttnDim;
    const bool writer = h % group == 0;

    // What depends on the position only is requested now, ahead of the q/k work and its barrier:
    // the k row of this thread's first slot and the v rows of the wavefront's first sixteen slots
    // (clamped to a valid row where there is no such slot; those values are never used).
    uint4 kk[kAttnDim / 8];
    {
        const uint4* row = (const uint4*)(kc + (size_t)(tid < n - 1 ? tid : 0) * kAttnDim);
#pragma unroll
        for (int c = 0; c < kAttnDim / 8; ++c) kk[c] = row[c];
    }
    const uint32_t* vrow = (const uint32_t*)vc + lane;
    uint32_t v_first[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        const int j = wave + 4 * u;
        v_first[u] = vrow[(size_t)(j < n - 1 ? j : 0) * (kAttnDim / 2)];
    }

    if (wave == 0) {
        const float2 r = norm_rotate(a.qk + (size_t)h * kAttnDim, a.norm_w ? a.norm_w + (size_t)h * kAttnDim : nullptr,
                                     cs, sn, lane, a.eps, a.scale);
        // the query as the BF16 value a BF16 matrix product would see
        q[lane] = __uint_as_float((uint32_t)f32_to_bf16_rne(r.x) << 16);
        q[lane + 64] = __uint_as_float((uint32_t)f32_to_bf16_rne(r.y) << 16);
    } else if (wave == 1) {
        const int row = a.q_heads + kh;
        const float2 r = norm_rotate(a.qk + (size_t)row * kAttnDim, a.norm_w ? a.norm_w + (size_t)row * kAttnDim : nullptr,
                                     cs, sn, lane, a.eps, 1.0f);
        const uint16_t lo = f32_to_bf16_rne(r.x), hi = f32_to_bf16_rne(r.y);
        k_new[lane] = lo;
        k_new[lane + 64] = hi;
        if (writer) {
            uint16_t* dst = a.k_cache + ((size_t)kh * a.max_len + p) * kAttnDim;
            dst[lane] = lo;
            dst[lane + 64] = hi;
        }
    } else if (wave == 2 && writer) {
        const uint16_t* src = a.v + (size_t)kh * kAttnDim;
        uint16_t* dst = a.v_cache + ((size_t)kh * a.max_len + p) * kAttnDim;
        dst[lane] = src[lane];
        dst[lane + 64] = src[lane + 64];
    }
    __syncthreads();

    // ---- scores: the token's own slot from LDS (wavefront 3, two elements per lane), the slots
    // before it from the cache
    const int rounds = (n + kAttnThreads - 1) / kAttnThreads;
    float best = -INFINITY;
    if (wave == 3) {
        const float own = wave_sum(__uint_as_float((uint32_t)k_new[lane] << 16) * q[lane] +
                                   __uint_as_float((uint32_t)k_new[lane + 64] << 16) * q[lane + 64]);
        if (lane == 0) weights[n - 1] = own;
        best = own;
    }
    for (int r = 0; r < rounds; ++r) {
        // one slot per thread and round, its whole row requested at once (16 loads in flight)
        const int j = r * kAttnThreads + tid;
        if (r > 0) {
            const uint4* row = (const uint4*)(kc + (size_t)(j < n - 1 ? j : 0) * kAttnDim);   // past the end: any valid row, dropped below
#pragma unroll
            for (int c = 0; c < kAttnDim / 8; ++c) kk[c] = row[c];
        }
        float s = 0.f;
#pragma unroll
        for (int c = 0; c < kAttnDim / 8; ++c) {
            const float4 q0 = *(const float4*)(q + 8 * c), q1 = *(const float4*)(q + 8 * c + 4);
            s += bf16_lo(kk[c].x) * q0.x + bf16_hi(kk[c].x) * q0.y + bf16_lo(kk[c].y) * q0.z + bf16_hi(kk[c].y) * q0.w
               + bf16_lo(kk[c].z) * q1.x + bf16_hi(kk[c].z) * q1.y + bf16_lo(kk[c].w) * q1.z + bf16_hi(kk[c].w) * q1.w;
        }
        if (j != n - 1) {
            const float v = j < n - 1 ? s : -INFINITY;
            weights[j] = v;
            best = fmaxf(best, v);
        }
    }
    best = wave_max(best);
    if (lane == 0) red[wave] = best;
    __syncthreads();
    best = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float sum = 0.f;
    for (int j = tid; j < rounds * kAttnThreads; j += kAttnThreads) {
        const float e = j < n ? __expf(weights[j] - best) : 0.f;
        weights[j] = e;
        sum += e;
    }
    sum = wave_sum(sum);
    if (lane == 0) red[wave] = sum;
    __syncthreads();
    const float inv = 1.0f / (red[0] + red[1] + red[2] + red[3]);

    // ---- weighted sum of the v rows: wavefront w takes slots w, w + 4, ...
    float o0 = 0.f, o1 = 0.f;
#pragma unroll
    for (int u = 0; u < 16; ++u) {                      // the rows requested at the start
        const int j = wave + 4 * u;
        if (j < n - 1) {
            const float w = __uint_as_float((uint32_t)f32_to_bf16_rne(weights[j] * inv) << 16);
            o0 += w * bf16_lo(v_first[u]);
            o1 += w * bf16_hi(v_first[u]);
        }
    }
    int j = wave + 64;
    for (; j + 60 < n - 1; j += 64) {                   // sixteen rows in flight per wavefront
        uint32_t x[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) x[u] = vrow[(size_t)(j + 4 * u) * (kAttnDim / 2)];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const float w = __uint_as_float((uint32_t)f32_to_bf16_rne(weights[j + 4 * u] * inv) << 16);
            o0 += w * bf16_lo(x[u]);
            o1 += w * bf16_hi(x[u]);
        }
    }
    for (; j + 12 < n - 1; j += 16) {
        uint32_t x[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) x[u] = vrow[(size_t)(j + 4 * u) * (kAttnDim / 2)];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const float w = __uint_as_float((uint32_t)f32_to_bf16_rne(weights[j + 4 * u] * inv) << 16);
            o0 += w * bf16_lo(x[u]);
            o1 += w * bf16_hi(x[u]);
        }
    }
    for (; j < n - 1; j += 4) {
        const uint32_t x = vrow[(size_t)j * (kAttnDim / 2)];
        const float w = __uint_as_float((uint32_t)f32_to_bf16_rne(weights[j] * inv) << 16);
        o0 += w * bf16_lo(x);
        o1 += w * bf16_hi(x);
    }
    if (wave == ((n - 1) & 3)) {                        // the token's own v, from the input
        const uint32_t x = ((const uint32_t*)(a.v + (size_t)kh * kAttnDim))[lane];
        const float w = __uint_as_float((uint32_t)f32_to_bf16_rne(weights[n - 1] * inv) << 16);
        o0 += w * bf16_lo(x);
        o1 += w * bf16_hi(x);
    }
    part[wave][2 * lane] = o0;
    part[wave][2 * lane + 1] = o1;
    __syncthreads();
    if (tid < kAttnDim) {
        const float v = part[0][tid] + part[1][tid] + part[2][tid] + part[3][tid];
        a.out[(size_t)h * kAttnDim + tid] = f32_to_bf16_rne(v);
    }
}

}  // namespace bhi

extern "C" int bhi_decode_attention(const void* qk, const void* v, const void* norm_weight, const void* cos, const void* sin,
                                    const void* pos, void* k_cache, void* v_cache, void* out, int q_heads, int kv_heads,
                                    int head_dim, int max_len, float eps, float scale, void* stream) {
    using namespace bhi;
    if (!qk || !v || !cos || !sin || !pos || !k_cache || !v_cache || !out) return bhi_fail(BHI_EINVAL, "null pointer");
    if (head_dim != kAttnDim) return bhi_fail(BHI_EINVAL, "decode_attention is written for a head dimension of 128");
    if (q_heads < 1 || kv_heads < 1 || q_heads % kv_heads != 0) return bhi_fail(BHI_EINVAL, "q_heads must be a multiple of kv_heads");
    if (max_len < 1 || max_len > kAttnMaxLen) return bhi_fail(BHI_EINVAL, "decode_attention takes a cache of 1 to 8192 slots");
    AttnArgs a;
    a.qk = (const uint16_t*)qk; a.v = (const uint16_t*)v; a.norm_w = (const uint16_t*)norm_weight;
    a.cos = (const float*)cos; a.sin = (const float*)sin; a.pos = (const long long*)pos;
    a.k_cache = (uint16_t*)k_cache; a.v_cache = (uint16_t*)v_cache; a.out = (uint16_t*)out;
    a.q_heads = q_heads; a.kv_heads = kv_heads; a.max_len = max_len; a.eps = eps; a.scale = scale;
    const size_t lds = (size_t)((max_len + kAttnThreads - 1) / kAttnThreads * kAttnThreads) * sizeof(float);
    hipLaunchKernelGGL(decode_attention_kernel, dim3((unsigned)q_heads), dim3(kAttnThreads), lds, (hipStream_t)stream, a);
    return bhi_launch_status("decode_attention");
}
