// Huffman path: fused decode+GEMV, decode-to-BF16 and the encoder, for gfx950.
//
// Stand-ins for the reference's gemv_bf16_huffman / huffman_decode / huffman_encode
// (bf16_huffman_infer/src/kernel.cu:419-442, 510-531, 590-610).  The reference walks
// one row per 32-lane warp with two private bitstreams per lane and two dependent
// byte-table reads per exponent; here one 64-lane wavefront walks four rows, one LDS
// read resolves two exponents, and all lanes share one refill stream.
#include "bhi_common.h"
#include "bhi_host.h"

namespace bhi {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float dot2(uint32_t w, uint32_t x, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w), __builtin_bit_cast(bf16x2_t, x), acc, false);
}

// Cooperative copy of the 16 KB pair table into LDS.
__device__ __forceinline__ void load_table(uint32_t* __restrict__ lds, const uint32_t* __restrict__ g) {
    const uint4* src = (const uint4*)g;
    uint4* dst = (uint4*)lds;
    for (int i = threadIdx.x; i < kTableEntries / 4; i += blockDim.x) dst[i] = src[i];
}

struct Shape {
    int M, Ks, split_k, nc, steps;      // steps per (split, group)
    uint32_t total_words;
};

// ------------------------------------------------------------------ decode to BF16
__global__ __launch_bounds__(kBlockThreads)
void huffman_decode_kernel(const uint8_t* __restrict__ A_rem, const uint32_t* __restrict__ A_exp,
                           uint16_t* __restrict__ Y, const uint32_t* __restrict__ offsets,
                           const uint32_t* __restrict__ table, Shape s) {
    __shared__ uint32_t lut[kTableEntries];
    load_table(lut, table);
    __syncthreads();

    const int lane = threadIdx.x & (kLanes - 1);
    const int wave = (int)uniform(threadIdx.x / kLanes);
    const int G = s.M / kGroupRows;
    const int per_group = s.split_k * s.nc;
    const long long ntasks = (long long)G * per_group;
    long long task = (long long)blockIdx.x * kWavesPerBlock + wave;
    if (task >= ntasks) return;
    const int g = (int)(task / per_group);
    const int kc = (int)(task % per_group);
    const int k = kc / s.nc, c = kc % s.nc;
    const int t0 = (s.steps * c) / s.nc, t1 = (s.steps * (c + 1)) / s.nc;

    HuffCursor cur;
    cur.init(A_exp, task_span(offsets, s.M, s.split_k, s.nc, k, g, c, s.total_words), lane);

    const int K = s.Ks * s.split_k;
    const uint2* remp = (const uint2*)(A_rem + ((size_t)k * s.M + (size_t)kGroupRows * g) * s.Ks) + (size_t)t0 * kLanes + lane;
    uint16_t* yp = Y + (size_t)(kGroupRows * g + (lane & 3)) * K + (size_t)k * s.Ks + (size_t)t0 * kStepCols + (lane >> 2) * kLaneCols;

    uint2 r_next = remp[0];
    for (int t = t0; t < t1; ++t) {
        uint2 r = r_next;
        remp += kLanes;
        if (t + 1 < t1) r_next = remp[0];
        uint32_t e[4];
        cur.step(lut, e);
        uint4 out;
        out.x = rebuild_pair(e[0], rem_lo_pair(r.x));
        out.y = rebuild_pair(e[1], rem_hi_pair(r.x));
        out.z = rebuild_pair(e[2], rem_lo_pair(r.y));
        out.w = rebuild_pair(e[3], rem_hi_pair(r.y));
        *(uint4*)yp = out;
        yp += kStepCols;
    }
}

// ------------------------------------------------------------------ fused decode + GEMV
// Block = 8 wavefronts.  The split_k*nc tasks of one row group are spread over
// P = min(split_k*nc, 8) wavefronts of the same block (a wavefront loops when there
// are more tasks than that), so the sum over splits and chunks never leaves the block.
template <int BS>
__global__ __launch_bounds__(kBlockThreads)
void gemv_huffman_kernel(const uint8_t* __restrict__ A_rem, const uint32_t* __restrict__ A_exp,
                         const uint16_t* __restrict__ X, uint16_t* __restrict__ Y,
                         const uint32_t* __restrict__ offsets, const uint32_t* __restrict__ table,
                         Shape s, int P, int groups_per_block) {
    __shared__ uint32_t lut[kTableEntries];
    __shared__ float part[kWavesPerBlock][BS][kGroupRows];
    load_table(lut, table);
    __syncthreads();

    const int lane = threadIdx.x & (kLanes - 1);
    const int wave = (int)uniform(threadIdx.x / kLanes);
    const int G = s.M / kGroupRows;
    const int per_group = s.split_k * s.nc;
    const int rg = wave / P, p = wave % P;
    const int g = blockIdx.x * groups_per_block + rg;
    const bool active = rg < groups_per_block && g < G;
    const int K = s.Ks * s.split_k;

    float acc[BS];
#pragma unroll
    for (int b = 0; b < BS; ++b) acc[b] = 0.f;

    if (active) {
        for (int kc = p; kc < per_group; kc += P) {
            const int k = kc / s.nc, c = kc % s.nc;
            const int t0 = (s.steps * c) / s.nc, t1 = (s.steps * (c + 1)) / s.nc;
            HuffCursor cur;
            cur.init(A_exp, task_span(offsets, s.M, s.split_k, s.nc, k, g, c, s.total_words), lane);
            const uint2* remp = (const uint2*)(A_rem + ((size_t)k * s.M + (size_t)kGroupRows * g) * s.Ks) + (size_t)t0 * kLanes + lane;
            const uint16_t* xp = X + (size_t)k * s.Ks + (size_t)t0 * kStepCols + (lane >> 2) * kLaneCols;

            uint2 r_next = remp[0];
            uint4 x_next[BS];
#pragma unroll
            for (int b = 0; b < BS; ++b) x_next[b] = *(const uint4*)(xp + (size_t)b * K);
            for (int t = t0; t < t1; ++t) {
                uint2 r = r_next;
                uint4 x[BS];
#pragma unroll
                for (int b = 0; b < BS; ++b) x[b] = x_next[b];
                remp += kLanes;
                xp += kStepCols;
                if (t + 1 < t1) {
                    r_next = remp[0];
#pragma unroll
                    for (int b = 0; b < BS; ++b) x_next[b] = *(const uint4*)(xp + (size_t)b * K);
                }
                uint32_t e[4];
                cur.step(lut, e);
                const uint32_t w0 = rebuild_pair(e[0], rem_lo_pair(r.x));
                const uint32_t w1 = rebuild_pair(e[1], rem_hi_pair(r.x));
                const uint32_t w2 = rebuild_pair(e[2], rem_lo_pair(r.y));
                const uint32_t w3 = rebuild_pair(e[3], rem_hi_pair(r.y));
#pragma unroll
                for (int b = 0; b < BS; ++b) {
                    float a = acc[b];
                    a = dot2(w0, x[b].x, a);
                    a = dot2(w1, x[b].y, a);
                    a = dot2(w2, x[b].z, a);
                    a = dot2(w3, x[b].w, a);
                    acc[b] = a;
                }
            }
        }
        // lanes 4*b + i hold partial sums of row i: fold the 16 column blocks
#pragma unroll
        for (int b = 0; b < BS; ++b) {
            float a = acc[b];
            a += __shfl_xor(a, 4);
            a += __shfl_xor(a, 8);
            a += __shfl_xor(a, 16);
            a += __shfl_xor(a, 32);
            if (lane < kGroupRows) part[wave][b][lane] = a;
        }
    }
    __syncthreads();
    if (active && p == 0 && lane < kGroupRows) {
#pragma unroll
        for (int b = 0; b < BS; ++b) {
            float a = 0.f;
            for (int q = 0; q < P; ++q) a += part[rg * P + q][b][lane];
            Y[(size_t)b * s.M + kGroupRows * g + lane] = f32_to_bf16_rne(a);
        }
    }
}

// ------------------------------------------------------------------ encoder
// One wavefront per task; it replays the decoder's refill schedule and writes each
// finished word at the stream position the decoder will read it from.
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
    const uint32_t nwords = (bits + 31u) >> 5;
    const uint32_t nref = nwords > (uint32_t)kInitWords ? nwords - kInitWords : 0u;
    uint32_t sum_ref = nref, sum_esc = nesc;
    for (int o = 32; o > 0; o >>= 1) {
        sum_ref += __shfl_xor(sum_ref, o);
        sum_esc += __shfl_xor(sum_esc, o);
    }
    const uint32_t body = kInitWords * kLanes + sum_ref + sum_esc;
    const uint32_t total = (body + kAlignWords - 1) / kAlignWords * kAlignWords;
    if (lane == 0) output_lengths[task] = total;
    // zero padding between refill words and escape list
    for (uint32_t i = kInitWords * kLanes + sum_ref + lane; i < total - sum_esc; i += kLanes) out[i] = 0;

    // pass 2: emit.  a0/a1 hold the bits of words m, m+1, m+2 (m = cursor word).
    uint64_t a0 = nref;
    uint32_t a1 = 0;
    uint32_t fill = kHeaderBits;                 // bit position relative to word m
    uint32_t q0 = lane, q1 = kLanes + lane, q2 = 2 * kLanes + lane;   // stream slots of words m, m+1, m+2
    const uint32_t kNone = 0xFFFFFFFFu;
    uint32_t left = nref, ptr = kInitWords * kLanes, eptr = 0;
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
            const uint32_t code = en & 0xFFFFu, len = en >> 16;
            if (fill < 64u) {
                a0 |= (uint64_t)code << fill;
                if (fill + len > 64u) a1 |= code >> (64u - fill);
            } else {
                a1 |= code << (fill - 64u);
            }
            fill += len;
        }
        for (;;) {
            bool cross = fill >= 32u + kCursorBias;
            if (ballot(cross) == 0) break;
            bool load = cross && left != 0;
            uint64_t m = ballot(load);
            if (cross) {
                if (q0 != kNone) out[q0] = (uint32_t)a0;
                a0 = (a0 >> 32) | ((uint64_t)a1 << 32);
                a1 = 0;
                fill -= 32u;
                q0 = q1; q1 = q2;
                q2 = load ? ptr + lane_rank(m) : kNone;
                if (load) left -= 1;
            }
            ptr += (uint32_t)__builtin_popcountll(m);
        }
    }
    if (q0 != kNone) out[q0] = (uint32_t)a0;
    if (q1 != kNone) out[q1] = (uint32_t)(a0 >> 32);
    if (q2 != kNone) out[q2] = a1;
}

}  // namespace bhi

using namespace bhi;

static int check_shape(int split_k, int M, int Ks, int64_t exp_words, int64_t lut1_bytes, Shape* s) {
    if (split_k < 1 || M < kGroupRows || M % kGroupRows != 0 || Ks < kStepCols || Ks % kStepCols != 0)
        return bhi_fail(BHI_EINVAL, "need split_k >= 1, M a multiple of 4 and Ks a multiple of 128");
    if (lut1_bytes != (int64_t)kTableEntries * 4)
        return bhi_fail(BHI_ELAYOUT, "LUT1 must hold 4096 four-byte pair entries");
    if (exp_words < kTailPadWords || exp_words >= ((int64_t)1 << 32))
        return bhi_fail(BHI_EINVAL, "exponent stream size out of range");
    s->M = M; s->Ks = Ks; s->split_k = split_k;
    s->nc = chunks_per_group(M, Ks, split_k);
    s->steps = Ks / kStepCols;
    if ((s->steps + s->nc - 1) / s->nc > kMaxTaskSteps)
        return bhi_fail(BHI_ELAYOUT, "more than 128 steps per task");
    s->total_words = (uint32_t)(exp_words - kTailPadWords);
    return 0;
}

extern "C" int bhi_huffman_decode(const void* A_rem, const void* A_exp, int64_t exp_words,
                                  void* Y, const void* offsets,
                                  const void* LUT1, int64_t lut1_bytes,
                                  const void*, const void*, const void*, const void*,
                                  int split_k, int M, int Ks, void* stream) {
    if (!A_rem || !A_exp || !Y || !offsets || !LUT1) return bhi_fail(BHI_EINVAL, "null pointer");
    Shape s;
    if (int rc = check_shape(split_k, M, Ks, exp_words, lut1_bytes, &s)) return rc;
    long long ntasks = (long long)(M / kGroupRows) * split_k * s.nc;
    unsigned grid = (unsigned)((ntasks + kWavesPerBlock - 1) / kWavesPerBlock);
    hipLaunchKernelGGL(huffman_decode_kernel, dim3(grid), dim3(kBlockThreads), 0, (hipStream_t)stream,
                       (const uint8_t*)A_rem, (const uint32_t*)A_exp, (uint16_t*)Y, (const uint32_t*)offsets,
                       (const uint32_t*)LUT1, s);
    return bhi_launch_status("huffman_decode");
}

template <int BS>
static void launch_gemv(const void* A_rem, const void* A_exp, const void* X, void* Y, const void* offsets,
                        const void* LUT1, const Shape& s, hipStream_t stream) {
    int per_group = s.split_k * s.nc;
    int P = per_group < kWavesPerBlock ? per_group : kWavesPerBlock;
    int gpb = kWavesPerBlock / P;
    int G = s.M / kGroupRows;
    unsigned grid = (unsigned)((G + gpb - 1) / gpb);
    hipLaunchKernelGGL(gemv_huffman_kernel<BS>, dim3(grid), dim3(kBlockThreads), 0, stream,
                       (const uint8_t*)A_rem, (const uint32_t*)A_exp, (const uint16_t*)X, (uint16_t*)Y,
                       (const uint32_t*)offsets, (const uint32_t*)LUT1, s, P, gpb);
}

extern "C" int bhi_gemv_bf16_huffman(const void* A_rem, const void* A_exp, int64_t exp_words,
                                     const void* X, void* Y, const void* offsets,
                                     const void* LUT1, int64_t lut1_bytes,
                                     const void*, const void*, const void*, const void*,
                                     int split_k, int M, int Ks, int batch, void* stream) {
    if (!A_rem || !A_exp || !X || !Y || !offsets || !LUT1) return bhi_fail(BHI_EINVAL, "null pointer");
    if (batch < 1) return bhi_fail(BHI_EINVAL, "batch must be >= 1");
    if (batch > kMaxBatch) return bhi_fail(BHI_EBATCH, "fused GEMV supports batch <= 8");
    Shape s;
    if (int rc = check_shape(split_k, M, Ks, exp_words, lut1_bytes, &s)) return rc;
    hipStream_t st = (hipStream_t)stream;
    switch (batch) {
        case 1: launch_gemv<1>(A_rem, A_exp, X, Y, offsets, LUT1, s, st); break;
        case 2: launch_gemv<2>(A_rem, A_exp, X, Y, offsets, LUT1, s, st); break;
        case 3: launch_gemv<3>(A_rem, A_exp, X, Y, offsets, LUT1, s, st); break;
        case 4: launch_gemv<4>(A_rem, A_exp, X, Y, offsets, LUT1, s, st); break;
        case 5: launch_gemv<5>(A_rem, A_exp, X, Y, offsets, LUT1, s, st); break;
        case 6: launch_gemv<6>(A_rem, A_exp, X, Y, offsets, LUT1, s, st); break;
        case 7: launch_gemv<7>(A_rem, A_exp, X, Y, offsets, LUT1, s, st); break;
        default: launch_gemv<8>(A_rem, A_exp, X, Y, offsets, LUT1, s, st); break;
    }
    return bhi_launch_status("gemv_bf16_huffman");
}

extern "C" int64_t bhi_encode_capacity(int n_steps) {
    if (n_steps < 1) return 0;
    // init words + every lane full of 12-bit codes + every pair escaped + alignment
    int64_t lane_words = ((int64_t)kHeaderBits + (int64_t)n_steps * kPairsPerStep * kTableBits + 31) / 32;
    return kInitWords * kLanes + (int64_t)kLanes * lane_words + (int64_t)n_steps * kPairsPerStep * kLanes + kAlignWords;
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
