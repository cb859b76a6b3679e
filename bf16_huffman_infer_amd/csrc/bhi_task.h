// Codec-independent part of the kernels: how a task is walked (segments, operand
// policies), the decode-to-BF16 and fused GEMV kernels, and their launch geometry.  A
// codec supplies `Cursor` (open / prime_issue / prime_commit / start / room / prefetch /
// commit / step), the size of its decode table and `variant(header)`, a wave-uniform
// choice between two instantiations of the walk.
#pragma once
#include <type_traits>
#include "bhi_common.h"
#include "bhi_host.h"

namespace bhi {

typedef float f32x4_t __attribute__((ext_vector_type(4)));

// Cooperative copy of the decode table into LDS.
template <int WORDS>
__device__ __forceinline__ void load_table(uint32_t* __restrict__ lds, const uint32_t* __restrict__ g) {
    const uint4* src = (const uint4*)g;
    uint4* dst = (uint4*)lds;
    for (int i = threadIdx.x; i < WORDS / 4; i += blockDim.x) dst[i] = src[i];
}

// The same copy in two halves: the loads are issued when a block starts, ahead of every
// other load (vector loads return in issue order, so the table arrives first), and the LDS
// writes follow once the task's own first loads are on their way.
template <int WORDS, int THREADS>
struct TableCopy {
    static constexpr int kVecs = WORDS / 4;
    static_assert(kVecs <= 2 * THREADS, "at most two 16-byte pieces per thread");
    // named registers: an array that a lambda captures by reference ends up in scratch memory
    typedef uint32_t vec_t __attribute__((ext_vector_type(4)));
    vec_t v0, v1;
    __device__ __forceinline__ void issue(const uint32_t* __restrict__ g) {
        const int i = (int)threadIdx.x;
        if (kVecs >= THREADS || i < kVecs) v0 = ((const vec_t*)g)[i];
        if (kVecs > THREADS && (kVecs == 2 * THREADS || i + THREADS < kVecs)) v1 = ((const vec_t*)g)[i + THREADS];
    }
    __device__ __forceinline__ void commit(uint32_t* __restrict__ lds) const {
        const int i = (int)threadIdx.x;
        if (kVecs >= THREADS || i < kVecs) ((vec_t*)lds)[i] = v0;
        if (kVecs > THREADS && (kVecs == 2 * THREADS || i + THREADS < kVecs)) ((vec_t*)lds)[i + THREADS] = v1;
    }
};

// A codec's decode table as LDS holds it.  The plain case: the words of the table buffer, as they are.
template <int WORDS>
struct PlainTable {
    static constexpr int kLdsWords = WORDS;
    template <int THREADS> using Stage = TableCopy<WORDS, THREADS>;
    static __device__ __forceinline__ void fill(uint32_t* __restrict__ lds, const uint32_t* __restrict__ g) { load_table<WORDS>(lds, g); }
};

struct Shape {
    int M, Ks, split_k, nc, steps;      // steps per (split, group)
    uint32_t total_words;
    int nc_log2;                        // nc is a power of two (chunks_per_group doubles it)
};

// One segment of a task: S steps whose operands a policy has loaded into `slot`.
// `Slot` holds what is loaded per step; `take(...)` hands out what the policy pipelines
// on its own inside the compute phase; `use(...)` receives the lane's four rebuilt BF16
// pairs (columns 0..7 of its row in step t).
template <bool FULL, bool HAS_ESC, int S, class Cursor, class Policy>
__device__ __forceinline__ void decode_segment(Cursor& cur, const uint32_t* lut, Policy& pol,
                                               const typename Policy::Slot (&slot)[S], int t0, int ns) {
#pragma unroll
    for (int i = 0; i < S; ++i) {
        if (FULL || t0 + i < ns) {
            const typename Policy::Piped piped = pol.take(slot[i], i, t0 + i);
            uint32_t e[4];
            cur.template step<HAS_ESC>(lut, e, i);
            uint32_t w[4];
            const uint2 r = slot[i].rem;
            w[0] = rebuild_pair(e[0], rem_lo_pair(r.x));
            w[1] = rebuild_pair(e[1], rem_hi_pair(r.x));
            w[2] = rebuild_pair(e[2], rem_lo_pair(r.y));
            w[3] = rebuild_pair(e[3], rem_hi_pair(r.y));
            pol.use(piped, t0 + i, w);
        }
    }
}

// A whole segment: stage the rows prefetched during the previous segment, prefetch the
// next ones if the ring has room, issue the operand loads of the following segment into
// `next`, decode `now`.  Every global load is thus issued a whole segment before its
// first use and is unconditional apart from the row prefetch, so the compiler can count
// the outstanding ones and make each step wait for exactly its own operands.
template <bool HAS_ESC, int S, class Cursor, class Policy>
__device__ __forceinline__ void run_segment(Cursor& cur, const uint32_t* lut, Policy& pol, bool& pending,
                                            uint32_t (&rows)[S], const typename Policy::Slot (&now)[S],
                                            typename Policy::Slot (&next)[S], int seg, int next_seg, bool spare, int ns) {
    if (pending) cur.commit(rows);
    pending = cur.template room<S>();
    if (pending) cur.prefetch(rows);
    pol.load_full(next, next_seg, spare);
    decode_segment<true, HAS_ESC>(cur, lut, pol, now, seg, ns);
}

// The walk over one task.  Its first loads (operands of the first segment, the rows that
// prime the ring) are issued before `between()` runs, which is where the first task of a
// block stores the decode table into LDS: table, rows and operands are in flight
// together.  Whole segments alternate between two operand sets (one being decoded, one in
// flight); the last whole segment reloads itself instead of running past the task.  A
// last, shorter segment clamps its step indices and guards its steps.
template <bool HAS_ESC, int S, class Cursor, class Policy, class Between>
__device__ __forceinline__ void run_task(Cursor& cur, const uint32_t* lut, Policy& pol, int ns, Between between) {
    typename Policy::Slot a[S], b[S];
    const int full_end = ns - ns % S;
    const int last_full = full_end - S;
    pol.prime();
    if (full_end > 0) {
        pol.load_full(a, 0, false);
    } else {
#pragma unroll
        for (int i = 0; i < S; ++i) pol.load(a[i], i);
    }
    {
        uint32_t first[kPrimeRows];
        cur.prime_issue(first);
        between();
        cur.prime_commit(first);
    }
    cur.start(lut);
    uint32_t rows[S];
    bool pending = cur.template room<S>();
    if (pending) cur.prefetch(rows);
    int seg = 0;
    if (full_end > 0) {
        for (;;) {
            int nx = seg + S;
            run_segment<HAS_ESC, S>(cur, lut, pol, pending, rows, a, b, seg, nx < last_full ? nx : last_full, nx > last_full, ns);
            seg = nx;
            if (seg >= full_end) break;
            nx = seg + S;
            run_segment<HAS_ESC, S>(cur, lut, pol, pending, rows, b, a, seg, nx < last_full ? nx : last_full, nx > last_full, ns);
            seg = nx;
            if (seg >= full_end) break;
        }
        if (seg < ns) {
#pragma unroll
            for (int i = 0; i < S; ++i) pol.load(a[i], seg + i);
        }
    }
    if (pending) cur.commit(rows);
    if (seg < ns) decode_segment<false, HAS_ESC, S>(cur, lut, pol, a, seg, ns);
}

// The format header (code_lengths buffer): [0] version, [1] table bits, [2] ESC code
// length, [3] nonzero when the matrix contains escaped pairs.
// The flag is read in two halves so that a kernel can issue the load early and look at the
// word late: `header_flag_word` is the aligned word that holds byte 3 (a scalar load needs a
// word address), `header_flag_test` picks the byte out of it.
__device__ __forceinline__ uint32_t header_flag_word(const uint8_t* __restrict__ header) {
    return constant_word((const uint32_t*)((uintptr_t)(header + 3) & ~(uintptr_t)3));
}
__device__ __forceinline__ bool header_flag_test(uint32_t w, const uint8_t* __restrict__ header) {
    return ((w >> (8u * (uint32_t)((uintptr_t)(header + 3) & 3))) & 0xFFu) != 0;
}
__device__ __forceinline__ bool header_has_esc(const uint8_t* __restrict__ header) {
    return header_flag_test(header_flag_word(header), header);
}

// Pins a wave-uniform value where it stands: what is computed from it cannot move above this
// point, so the wait for the load behind it lands here and not right after the load.
__device__ __forceinline__ uint32_t pin_uniform(uint32_t v) {
    asm volatile("" : "+s"(v));
    return v;
}

// decode-to-BF16: rem in, 16 bytes of weights out per lane and step
struct StorePolicy {
    struct Slot { uint2 rem; };
    struct Piped {};
    const uint2* rem0;       // this lane's 8 rem bytes of the task's first step
    uint16_t* yp;            // this lane's 8 output columns of the task's first step
    int last;

    __device__ __forceinline__ void prime() const {}
    __device__ __forceinline__ void load(Slot& s, int t) const {
        t = t < last ? t : last;
        s.rem = stream_load(rem0 + (size_t)t * kLanes);
    }
    template <int S>
    __device__ __forceinline__ void load_full(Slot (&s)[S], int t0, bool) const {
        const uint2* p = rem0 + (size_t)t0 * kLanes;
#pragma unroll
        for (int i = 0; i < S; ++i) s[i].rem = stream_load(p + i * kLanes);
    }
    __device__ __forceinline__ Piped take(const Slot&, int, int) const { return Piped{}; }
    __device__ __forceinline__ void use(const Piped&, int t, const uint32_t (&w)[4]) const {
        *(uint4*)(yp + (size_t)t * kStepCols) = make_uint4(w[0], w[1], w[2], w[3]);
    }
};

// Broadcast of lane q of every quad (dpp quad_perm:[q,q,q,q]).
template <int Q>
__device__ __forceinline__ uint32_t quad_bcast(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, Q * 0x55, 0xF, 0xF, true);
}

// fused GEMV, batch 1..8: a lane keeps the sums of its own row (lane & 3) over its 8 columns
// of every step, one fp32 accumulator per batch row, and adds four two-element dot
// products per step and batch row (v_dot2c_f32_bf16).  The four lanes of a quad own the
// same 8 columns: each loads ONE X pair per batch row (lane 4*b + i the pair 8*b + 2*i,
// 8*b + 2*i + 1), so a wavefront's X load is 256 contiguous bytes per batch row, and the
// dot products read the other lanes' pairs through their DPP operand.
//
// (The 4x4x4 matrix products this replaced need, in lane 4*b + j, all 8 columns of batch
// row j: four different rows of X inside every quad.  Those loads are not coalesced and
// cost more than everything else the batch adds: 27.9 -> 24.0 us at batch 2, 33.1 -> 27.2
// at batch 4, 44.6 -> 33.4 at batch 8 on 18944x3584.)
//
// Where the X pairs wait for their step depends on the batch:
//   batch 1..4  in the segment's operand set, loaded a segment ahead like rem (bs registers
//               per step);
//   batch 5..8  that would be 8 * bs registers: they are fetched XAHEAD steps ahead instead,
//               right after the step that used their registers (X is cache resident).
//
// acc += sum over q of x[q].lo * w[q].lo + x[q].hi * w[q].hi, where x[q] is the X pair held by
// lane q of this lane's quad: four v_dot2c_f32_bf16 with the quad broadcast folded into their
// DPP operand (the compiler keeps a separate v_mov_dpp when given the builtins).  A VALU
// write to `x` right before a DPP read of it needs two wait states, and the compiler cannot
// see the DPP reads inside the asm.  All four reads of `x` therefore sit in ONE asm statement
// behind one s_nop: nothing the compiler emits (a register copy of `x`, say) can land
// between a write of `x` and an unprotected read.  The other side of the statement has a
// hazard of its own: a VALU instruction that is not the same dot product must not read
// `acc` within three wait states of the write, and the compiler, which does not see a dot
// product here, will happily copy `acc` to another register right behind the statement
// (wrong sums, in whichever batch row the copy happened to hit).  Hence the closing s_nop.
#define BHI_DOT(ACC, X, W, Q) "v_dot2c_f32_bf16_dpp " ACC ", " X ", " W " quad_perm:[" Q "," Q "," Q "," Q "] row_mask:0xf bank_mask:0xf\n\t"
// N batch rows at once (N <= 4): acc[j] += the four products of x[j] with w[0..3].  One
// statement for all of them, so that the two s_nops are paid once per step and not once per
// batch row, and the products of different rows interleave (no instruction waits for the one
// right before it).
template <int N>
__device__ __forceinline__ void dot_rows(float* acc, const uint32_t (&x)[4], const uint32_t (&w)[4]) {
    static_assert(N >= 1 && N <= 4, "up to four batch rows per statement");
    if constexpr (N == 1) {
        asm("s_nop 1\n\t"
            BHI_DOT("%0", "%1", "%2", "0") BHI_DOT("%0", "%1", "%3", "1") BHI_DOT("%0", "%1", "%4", "2") BHI_DOT("%0", "%1", "%5", "3")
            "s_nop 2"
            : "+v"(acc[0]) : "v"(x[0]), "v"(w[0]), "v"(w[1]), "v"(w[2]), "v"(w[3]));
    } else if constexpr (N == 2) {
        asm("s_nop 1\n\t"
            BHI_DOT("%0", "%2", "%4", "0") BHI_DOT("%1", "%3", "%4", "0")
            BHI_DOT("%0", "%2", "%5", "1") BHI_DOT("%1", "%3", "%5", "1")
            BHI_DOT("%0", "%2", "%6", "2") BHI_DOT("%1", "%3", "%6", "2")
            BHI_DOT("%0", "%2", "%7", "3") BHI_DOT("%1", "%3", "%7", "3")
            "s_nop 2"
            : "+v"(acc[0]), "+v"(acc[1]) : "v"(x[0]), "v"(x[1]), "v"(w[0]), "v"(w[1]), "v"(w[2]), "v"(w[3]));
    } else if constexpr (N == 3) {
        asm("s_nop 1\n\t"
            BHI_DOT("%0", "%3", "%6", "0") BHI_DOT("%1", "%4", "%6", "0") BHI_DOT("%2", "%5", "%6", "0")
            BHI_DOT("%0", "%3", "%7", "1") BHI_DOT("%1", "%4", "%7", "1") BHI_DOT("%2", "%5", "%7", "1")
            BHI_DOT("%0", "%3", "%8", "2") BHI_DOT("%1", "%4", "%8", "2") BHI_DOT("%2", "%5", "%8", "2")
            BHI_DOT("%0", "%3", "%9", "3") BHI_DOT("%1", "%4", "%9", "3") BHI_DOT("%2", "%5", "%9", "3")
            "s_nop 2"
            : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2])
            : "v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(w[0]), "v"(w[1]), "v"(w[2]), "v"(w[3]));
    } else {
        asm("s_nop 1\n\t"
            BHI_DOT("%0", "%4", "%8", "0") BHI_DOT("%1", "%5", "%8", "0") BHI_DOT("%2", "%6", "%8", "0") BHI_DOT("%3", "%7", "%8", "0")
            BHI_DOT("%0", "%4", "%9", "1") BHI_DOT("%1", "%5", "%9", "1") BHI_DOT("%2", "%6", "%9", "1") BHI_DOT("%3", "%7", "%9", "1")
            BHI_DOT("%0", "%4", "%10", "2") BHI_DOT("%1", "%5", "%10", "2") BHI_DOT("%2", "%6", "%10", "2") BHI_DOT("%3", "%7", "%10", "2")
            BHI_DOT("%0", "%4", "%11", "3") BHI_DOT("%1", "%5", "%11", "3") BHI_DOT("%2", "%6", "%11", "3") BHI_DOT("%3", "%7", "%11", "3")
            "s_nop 2"
            : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3])
            : "v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]), "v"(w[0]), "v"(w[1]), "v"(w[2]), "v"(w[3]));
    }
}
#undef BHI_DOT

// What the GEMV multiplies the weights with: X as given, or a function of X that the layer in
// front of the linear would otherwise have to write to memory with a kernel of its own:
//   kXRms      h = x * rsqrt(mean(x^2) + eps) * gamma      (RMSNorm; gamma bf16 [K])
//   kXSiluMul  h = silu(gate) * x                          (the SwiGLU product; gate bf16 [batch, K])
// Both round as the separate kernels of this library do (bhi_rms_norm, bhi_silu_mul), so the
// fused and the unfused sequence give the same bits.
enum XMode { kXPlain = 0, kXRms = 1, kXSiluMul = 2 };

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ f32x2_t pair_to_f32(uint32_t p) {
    return f32x2_t{__uint_as_float(p << 16), __uint_as_float(p & 0xFFFF0000u)};
}
__device__ __forceinline__ uint32_t f32_to_pair(f32x2_t v) {           // round to nearest even, both halves
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
// bf16(x * r * gamma), one rounding
__device__ __forceinline__ uint32_t rms_pair(uint32_t x, float r, uint32_t gamma) {
    const f32x2_t xf = pair_to_f32(x), gf = pair_to_f32(gamma);
    return f32_to_pair(f32x2_t{xf.x * r * gf.x, xf.y * r * gf.y});
}
// bf16(bf16(silu(g)) * u): the rounding of a BF16 silu followed by a BF16 multiply
__device__ __forceinline__ uint32_t silu_mul_pair(uint32_t g, uint32_t u) {
    const f32x2_t gf = pair_to_f32(g), uf = pair_to_f32(u);
    // g * rcp(1 + 2^(-g * log2 e)): hardware exp2 and reciprocal (one unit in the last place each,
    // far below the BF16 rounding that follows); a full-precision division here costs more than
    // the rest of the step
    const float ex = __builtin_amdgcn_exp2f(gf.x * -1.4426950408889634f), ey = __builtin_amdgcn_exp2f(gf.y * -1.4426950408889634f);
    const f32x2_t sf = pair_to_f32(f32_to_pair(f32x2_t{gf.x * __builtin_amdgcn_rcpf(1.0f + ex), gf.y * __builtin_amdgcn_rcpf(1.0f + ey)}));
    return f32_to_pair(f32x2_t{sf.x * uf.x, sf.y * uf.y});
}

// rsqrt(mean(x^2) + eps) of every batch row, by a whole block: thread t squares the pairs
// t, t + T, ... of each row, a wavefront adds its lanes' sums by xor-shuffles, the
// wavefronts' sums meet in `part` ([waves][BS] floats in LDS) and are added in order after
// the caller's next barrier (rms_scales_finish).  The same code serves the stand-alone
// RMSNorm kernel, which is what makes fused and unfused results identical.
template <int BS>
__device__ __forceinline__ void rms_scales_start(const uint16_t* __restrict__ X, int K, float* part) {
    const int lane = threadIdx.x & (kLanes - 1), wave = threadIdx.x / kLanes;
    float sq[BS];
#pragma unroll
    for (int b = 0; b < BS; ++b) sq[b] = 0.f;
    for (int p = threadIdx.x; p < K / 2; p += blockDim.x) {
#pragma unroll
        for (int b = 0; b < BS; ++b) {
            const f32x2_t v = pair_to_f32(((const uint32_t*)X)[(size_t)b * (K / 2) + p]);
            sq[b] += v.x * v.x;
            sq[b] += v.y * v.y;
        }
    }
#pragma unroll
    for (int b = 0; b < BS; ++b) {
        float v = sq[b];
        for (int o = 1; o < kLanes; o <<= 1) v += __shfl_xor(v, o);
        if (lane == 0) part[wave * BS + b] = v;
    }
}
template <int BS>
__device__ __forceinline__ void rms_scales_finish(const float* part, int K, float eps, float (&r)[BS]) {
    const int waves = blockDim.x / kLanes;
#pragma unroll
    for (int b = 0; b < BS; ++b) {
        float v = 0.f;
        for (int w = 0; w < waves; ++w) v += part[w * BS + b];
        r[b] = 1.0f / sqrtf(v / (float)K + eps);
    }
}

template <int BS, int XM = kXPlain>
struct DotPolicy {
    static_assert(XM == kXPlain || BS <= 4, "transformed X is kept in the segment's operand set: batch 1..4");
    static constexpr int NSET = BS <= 4 ? 1 : 2;            // batch rows in sets of four
    static constexpr bool PIPED = BS > 4;
    static constexpr int XAHEAD = BS > 6 ? 1 : 2;            // 92 registers at batch 8: five wavefronts per SIMD
    struct Slot { uint2 rem; uint4 x; uint4 a; };            // x: the lane's X pair of batch rows 0..3; a: gamma or gate pairs
    struct Piped { uint4 x, a; int i, t; };
    const uint2* rem0;
    const uint2* spare_rem;  // kSegLong * 512 readable bytes that are cache resident (the decode table, or the start of the task's exponent stream)
    const uint32_t* xq0;     // this lane's X pair of batch row 0, first step of the task
    const uint32_t* aq0;     // the same position in gamma (kXRms) or in gate row 0 (kXSiluMul)
    float rs[BS <= 4 ? BS : 1];   // kXRms: the rows' scales
    int xrow;                // distance between batch rows of X, in pairs
    int last;
    uint4 xr[XAHEAD][NSET];  // batch 5..8: the pairs of the next XAHEAD steps
    float dot[2 * 4];
    f32x4_t acc[NSET];       // filled by fold(): the sums in the layout the epilogue stores from

    // one X pair per batch row B0 .. B0 + 3: each a 256-byte contiguous load of the wavefront
    template <int B0>
    __device__ __forceinline__ void xpairs(uint4& x, const uint32_t* p) const {
        if (BS > B0) x.x = p[(size_t)B0 * xrow];
        if (BS > B0 + 1) x.y = p[(size_t)(B0 + 1) * xrow];
        if (BS > B0 + 2) x.z = p[(size_t)(B0 + 2) * xrow];
        if (BS > B0 + 3) x.w = p[(size_t)(B0 + 3) * xrow];
    }
    __device__ __forceinline__ void xload(uint4 (&dst)[NSET], int t) const {
        t = t < last ? t : last;
        xpairs<0>(dst[0], xq0 + (size_t)t * (kStepCols / 2));
        if (NSET > 1) xpairs<4>(dst[NSET - 1], xq0 + (size_t)t * (kStepCols / 2));
    }
    __device__ __forceinline__ void prime() {
        if (PIPED) {
#pragma unroll
            for (int i = 0; i < XAHEAD; ++i) xload(xr[i], i);
        }
    }
    __device__ __forceinline__ void load(Slot& s, int t) const { load_at(s, rem0, xq0, last, t, aq0); }
    // step t (clamped to last_) of the task whose first step sits at r0 / x0 (/ a0)
    __device__ __forceinline__ void load_at(Slot& s, const uint2* r0, const uint32_t* x0, int last_, int t,
                                            const uint32_t* a0 = nullptr) const {
        t = t < last_ ? t : last_;
        s.rem = stream_load(r0 + (size_t)t * kLanes);
        if (!PIPED) xpairs<0>(s.x, x0 + (size_t)t * (kStepCols / 2));
        if (XM == kXRms) s.a.x = a0[(size_t)t * (kStepCols / 2)];
        if (XM == kXSiluMul) xpairs<0>(s.a, a0 + (size_t)t * (kStepCols / 2));
    }
    // `spare`: the loads are not needed (the last whole segment of a task has no successor) and
    // go to `spare_rem`, bytes that are in cache anyway, instead of reading the segment again
    template <int S>
    __device__ __forceinline__ void load_full(Slot (&s)[S], int t0, bool spare) const {
        const uint2* pr = spare ? spare_rem : rem0 + (size_t)t0 * kLanes;
        const uint32_t* pq = xq0 + (size_t)t0 * (kStepCols / 2);
        const uint32_t* pa = aq0 + (size_t)t0 * (kStepCols / 2);
#pragma unroll
        for (int i = 0; i < S; ++i) {
            s[i].rem = stream_load(pr + i * kLanes);
            if (!PIPED) xpairs<0>(s[i].x, pq + i * (kStepCols / 2));
            if (XM == kXRms) s[i].a.x = pa[i * (kStepCols / 2)];
            if (XM == kXSiluMul) xpairs<0>(s[i].a, pa + i * (kStepCols / 2));
        }
    }
    __device__ __forceinline__ Piped take(const Slot& s, int i, int t) const {
        Piped p;
        if (!PIPED) p.x = s.x;
        if (XM != kXPlain) p.a = s.a;
        p.i = i;
        p.t = t;
        return p;
    }
    __device__ __forceinline__ void use(const Piped& s, int, const uint32_t (&w)[4]) {
#pragma unroll
        for (int q = 0; q < NSET; ++q) {
            const uint4 xs = PIPED ? xr[s.i % XAHEAD][q] : s.x;
            uint32_t xb[4] = {xs.x, xs.y, xs.z, xs.w};
            if (XM == kXRms) {
#pragma unroll
                for (int j = 0; j < BS && j < 4; ++j) xb[j] = rms_pair(xb[j], rs[j], s.a.x);
            }
            if (XM == kXSiluMul) {
                const uint32_t gb[4] = {s.a.x, s.a.y, s.a.z, s.a.w};
#pragma unroll
                for (int j = 0; j < BS && j < 4; ++j) xb[j] = silu_mul_pair(gb[j], xb[j]);
            }
            if (q == 0) dot_rows<(BS < 4 ? BS : 4)>(dot, xb, w);
            else dot_rows<(BS > 4 ? BS - 4 : 1)>(dot + 4, xb, w);
        }
        if (PIPED) xload(xr[s.i % XAHEAD], s.t + XAHEAD);
    }
    // The epilogue stores from lanes 0..3 of the wavefront: lane 4*b + j wants, in register i
    // of set q, the sum that lane 4*b + i holds for batch row 4*q + j.
    __device__ __forceinline__ void fold() {
        const int mine = threadIdx.x & 3;
#pragma unroll
        for (int q = 0; q < NSET; ++q) {
            uint32_t r[4] = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (4 * q + j < BS) {
                    const uint32_t d = __float_as_uint(dot[4 * q + j]);
                    const uint32_t t[4] = {quad_bcast<0>(d), quad_bcast<1>(d), quad_bcast<2>(d), quad_bcast<3>(d)};
#pragma unroll
                    for (int i = 0; i < 4; ++i) r[i] = mine == j ? t[i] : r[i];
                }
            }
            acc[q] = f32x4_t{__uint_as_float(r[0]), __uint_as_float(r[1]), __uint_as_float(r[2]), __uint_as_float(r[3])};
        }
    }
};

struct TaskId { int k, c, t0, t1; };

__device__ __forceinline__ TaskId task_of(const Shape& s, int kc) {
    TaskId id;
    // shifts, not divisions: every wavefront runs this before its first load
    id.k = kc >> s.nc_log2;
    id.c = kc & (s.nc - 1);
    id.t0 = (s.steps * id.c) >> s.nc_log2;
    id.t1 = (s.steps * (id.c + 1)) >> s.nc_log2;
    return id;
}

// ------------------------------------------------------------------ decode to BF16
template <class Codec, int NW, int S>
__global__ __launch_bounds__(NW * kLanes)
void decode_kernel(const uint8_t* __restrict__ A_rem, const uint32_t* __restrict__ A_exp,
                           uint16_t* __restrict__ Y, const uint32_t* __restrict__ offsets,
                           const uint32_t* __restrict__ table, const uint8_t* __restrict__ header, Shape s) {
    __shared__ uint32_t rings[NW][kRingWords];
    __shared__ uint32_t lut[Codec::Table::kLdsWords];
    // The table's loads go out first and its LDS writes follow the task's own first loads; a
    // wavefront without a task still copies its share and joins the barrier.
    typename Codec::Table::template Stage<NW * kLanes> table_copy;
    table_copy.issue(table);
    auto stage_table = [&]() {
        table_copy.commit(lut);
        lds_barrier();
    };

    const int lane = threadIdx.x & (kLanes - 1);
    const int wave = (int)uniform(threadIdx.x / kLanes);
    const int G = s.M / kGroupRows;
    const int per_group = s.split_k * s.nc;
    const long long ntasks = (long long)G * per_group;
    const long long task = (long long)blockIdx.x * NW + wave;
    if (task >= ntasks) {
        stage_table();
        return;
    }
    const int g = (int)(task / per_group);
    const TaskId id = task_of(s, (int)(task % per_group));

    typename Codec::Cursor cur;
    cur.open(A_exp, task_span(offsets, s.M, s.split_k, s.nc, id.k, g, id.c, s.total_words), lane, rings[wave]);
    const int K = s.Ks * s.split_k;
    StorePolicy pol;
    pol.rem0 = (const uint2*)(A_rem + ((size_t)id.k * s.M + (size_t)kGroupRows * g) * s.Ks) + (size_t)id.t0 * kLanes + lane;
    pol.yp = Y + (size_t)(kGroupRows * g + (lane & 3)) * K + (size_t)id.k * s.Ks + (size_t)id.t0 * kStepCols + (lane >> 2) * kLaneCols;
    pol.last = id.t1 - id.t0 - 1;
    if (Codec::variant(header)) run_task<true, S>(cur, lut, pol, id.t1 - id.t0, stage_table);
    else run_task<false, S>(cur, lut, pol, id.t1 - id.t0, stage_table);
}

// ------------------------------------------------------------------ fused decode + GEMV
// Block = NW wavefronts.  The split_k*nc tasks of one row group are spread over
// P = min(split_k*nc, NW) wavefronts of the same block (a wavefront loops when there
// are more tasks than that), so the sum over splits and chunks never leaves the block.
// register budget: at least this many wavefronts per SIMD must stay resident
#ifndef BHI_MIN_WAVES1
#define BHI_MIN_WAVES1 6
#endif
constexpr int min_waves(int bs) { return bs <= 1 ? BHI_MIN_WAVES1 : (bs <= 2 ? 5 : (bs <= 4 ? 4 : 3)); }

// One launch can serve several weights that multiply the same X (the q/k/v or gate/up
// projections of a decoder layer): each member brings its own buffers, table and output,
// and owns a contiguous range of the grid.
constexpr int kMaxMembers = 4;
struct Member {
    const uint8_t* rem;
    const uint32_t* exp;
    uint16_t* Y;
    const uint32_t* offsets;
    const uint32_t* table;
    const uint8_t* header;
    const uint16_t* bias;    // bf16 [M] or null
    const uint16_t* residual;   // bf16 [batch, M] or null: added last, as a separate BF16 `y + residual` would
    Shape s;
    int first_block;         // this member's blocks are [first_block, next member's first_block)
};
struct Group {
    int n;
    Member m[kMaxMembers];
    const uint16_t* xaux;    // gamma (kXRms) or gate (kXSiluMul)
    float eps;               // kXRms
};

// The sum rounded to BF16; with a bias, that BF16 value plus the bias, rounded again (what a
// separate BF16 `output += bias` after the product gives).
__device__ __forceinline__ uint16_t finish_output(float sum, const uint16_t* __restrict__ bias, int row,
                                                  const uint16_t* __restrict__ residual_row = nullptr) {
    uint16_t y = f32_to_bf16_rne(sum);
    if (bias) y = f32_to_bf16_rne(__uint_as_float((uint32_t)y << 16) + __uint_as_float((uint32_t)bias[row] << 16));
    if (residual_row) y = f32_to_bf16_rne(__uint_as_float((uint32_t)y << 16) + __uint_as_float((uint32_t)residual_row[row] << 16));
    return y;
}

template <class Codec, int BS, int NW, int S, int XM = kXPlain>
__global__ __launch_bounds__(NW * kLanes, min_waves(BS))
void gemv_kernel(const uint16_t* __restrict__ X, int first1, int first2, int first3, const Group grp) {
    // The partial sums reuse the rings once every task of the block is done.
    __shared__ uint32_t rings[NW][kRingWords];
    __shared__ uint32_t lut[Codec::Table::kLdsWords];
    __shared__ float rms_part[XM == kXRms ? NW * BS : 1];
    // first1..3: first block of members 1..3 (INT_MAX when absent).  Leading scalar arguments
    // are in registers when the wavefront starts (the library is built with kernel-argument
    // preload), so the member is known without a fetch and its fields take one fetch, not two
    // dependent ones.
    static_assert(kMaxMembers == 4, "one leading argument per member after the first");
    int member = 0;
    if ((int)blockIdx.x >= first1) member = 1;
    if ((int)blockIdx.x >= first2) member = 2;
    if ((int)blockIdx.x >= first3) member = 3;
    const Member& mb = grp.m[member];
    const uint8_t* __restrict__ A_rem = mb.rem;
    const uint32_t* __restrict__ A_exp = mb.exp;
    uint16_t* __restrict__ Y = mb.Y;
    const uint32_t* __restrict__ offsets = mb.offsets;
    const uint32_t* __restrict__ table = mb.table;
    const uint8_t* __restrict__ header = mb.header;
    const uint16_t* __restrict__ bias = mb.bias;
    const uint16_t* __restrict__ residual = mb.residual;
    const Shape s = mb.s;
    const int block = (int)blockIdx.x - mb.first_block;
    // P wavefronts share one row group; a block holds NW / P row groups
    const int P = s.split_k * s.nc < NW ? s.split_k * s.nc : NW;
    static_assert(NW == 4, "the wavefront-to-task arithmetic below is written for four wavefronts");
    const int groups_per_block = P == 1 ? 4 : (P == 2 ? 2 : 1);
    // The table reaches LDS while the first task's first loads are in flight: the copy and
    // its barrier run once per wavefront, inside the first task or, for a wavefront
    // without one, right after.
    bool staged = false;
    // (the RMSNorm variant needs its registers for the sums of squares at that point and
    // copies the table in one go instead)
    constexpr bool kEarlyTable = XM != kXRms;
    typename Codec::Table::template Stage<NW * kLanes> table_copy;
    if (kEarlyTable) table_copy.issue(table);
    auto stage_table = [&]() {
        if (!staged) {
            if (kEarlyTable) table_copy.commit(lut);
            else Codec::Table::fill(lut, table);
            lds_barrier();
            staged = true;
        }
    };

    const int lane = threadIdx.x & (kLanes - 1);
    const int wave = (int)uniform(threadIdx.x / kLanes);
    const int G = s.M / kGroupRows;
    const int per_group = s.split_k * s.nc;
    // wave / P and wave % P for wave < 4 and P in 1..4 without a division
    const int rg = P == 1 ? wave : (P == 2 ? wave >> 1 : (wave >= P ? 1 : 0));
    const int p = wave - rg * P;
    const int g = block * groups_per_block + rg;
    const bool active = rg < groups_per_block && g < G;
    const int K = s.Ks * s.split_k;
    const uint32_t variant_word = Codec::variant_word(header);

    DotPolicy<BS, XM> pol;
    constexpr int NSET = DotPolicy<BS, XM>::NSET;
#pragma unroll
    for (int q = 0; q < NSET; ++q) pol.acc[q] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 8; ++j) pol.dot[j] = 0.f;
    pol.xrow = K / 2;
    // RMSNorm in front of the product: every wavefront of the block squares its share of X
    // (also one without a task) behind its first loads; the sums are complete behind the
    // barrier that ends the table copy
    auto stage_all = [&]() {
        if (!staged) {
            if constexpr (XM == kXRms) rms_scales_start<BS>(X, K, rms_part);
            stage_table();
            if constexpr (XM == kXRms) rms_scales_finish<BS>(rms_part, K, grp.eps, pol.rs);
        }
    };

    if (active) {
        for (int kc = p; kc < per_group; kc += P) {
            const TaskId id = task_of(s, kc);
            typename Codec::Cursor cur;
            const TaskSpan span = task_span(offsets, s.M, s.split_k, s.nc, id.k, g, id.c, s.total_words);
            cur.open(A_exp, span, lane, rings[wave]);
            pol.rem0 = (const uint2*)(A_rem + ((size_t)id.k * s.M + (size_t)kGroupRows * g) * s.Ks) + (size_t)id.t0 * kLanes + lane;
            pol.xq0 = (const uint32_t*)(X + (size_t)id.k * s.Ks + (size_t)id.t0 * kStepCols) + lane;
            pol.aq0 = XM == kXPlain ? nullptr
                                    : (const uint32_t*)(grp.xaux + (size_t)id.k * s.Ks + (size_t)id.t0 * kStepCols) + lane;
            pol.last = id.t1 - id.t0 - 1;
            // loads nobody needs go to bytes that are in cache anyway: the decode table where it is
            // long enough, else the start of the task's own exponent stream (read moments ago; the
            // zero tail behind the last stream keeps kSegLong * 512 bytes readable from any task's
            // start).  One region for every wavefront -- the offsets array was tried -- makes a few
            // cache lines hot and costs 4 % on the rANS block step.
            static_assert(kTailPadWords * 4 >= kSegLong * kLanes * 8, "the tail pad covers a segment's spare loads");
            if (Codec::kTableWords * 4 >= kSegLong * kLanes * 8) pol.spare_rem = (const uint2*)table + lane;
            else pol.spare_rem = (const uint2*)(A_exp + (span.base & ~1u)) + lane;
            // looked at only now: the flag's load has been in flight together with the offsets'
            const bool variant = Codec::variant_test(pin_uniform(variant_word), header);
            if (variant) run_task<true, S>(cur, lut, pol, id.t1 - id.t0, stage_all);
            else run_task<false, S>(cur, lut, pol, id.t1 - id.t0, stage_all);
            // Nothing is in flight at the end of a task.  Saying so keeps the compiler from
            // waiting at the top of the loop for loads that a previous pass might have left
            // behind: on the first pass that wait would be for the table, before the task's
            // own first loads are issued.
            __builtin_amdgcn_s_waitcnt(0x0F70);
        }
        pol.fold();
        // lane 4*b + j holds, in register i, the sum of row i for batch j over column block b
#pragma unroll
        for (int q = 0; q < NSET; ++q) {
#pragma unroll
            for (int i = 0; i < kGroupRows; ++i) {
                pol.acc[q][i] = sum_over_column_blocks(pol.acc[q][i]);
            }
        }
    }
    stage_all();
    if (P == 1) {
        // one wavefront per row group: its sums are final
        if (active && lane < 4) {
#pragma unroll
            for (int q = 0; q < NSET; ++q) {
                const int batch = lane + 4 * q;
                if (batch < BS) {
#pragma unroll
                    for (int i = 0; i < kGroupRows; ++i)
                        Y[(size_t)batch * s.M + kGroupRows * g + i] = finish_output(pol.acc[q][i], bias, kGroupRows * g + i,
                                                                                    residual ? residual + (size_t)batch * s.M : nullptr);
                }
            }
        }
        return;
    }
    // partial sums, [set][row][batch lane], go into the wavefront's own ring: nobody else
    // reads or writes it before the barrier below
    float* mine = (float*)rings[wave];
    if (active && lane < 4) {
#pragma unroll
        for (int q = 0; q < NSET; ++q)
#pragma unroll
            for (int i = 0; i < kGroupRows; ++i) mine[(q * kGroupRows + i) * 4 + lane] = pol.acc[q][i];
    }
    lds_barrier();
    if (active && p == 0 && lane < 4) {
#pragma unroll
        for (int q = 0; q < NSET; ++q) {
            const int batch = lane + 4 * q;
            if (batch < BS) {
#pragma unroll
                for (int i = 0; i < kGroupRows; ++i) {
                    float a = 0.f;
                    for (int w = 0; w < P; ++w) a += ((const float*)rings[rg * P + w])[(q * kGroupRows + i) * 4 + lane];
                    Y[(size_t)batch * s.M + kGroupRows * g + i] = finish_output(a, bias, kGroupRows * g + i,
                                                                                residual ? residual + (size_t)batch * s.M : nullptr);
                }
            }
        }
    }
}

}  // namespace bhi

static inline int check_shape(int split_k, int M, int Ks, int64_t exp_words, bhi::Shape* s) {
    using namespace bhi;
    if (split_k < 1 || M < kGroupRows || M % kGroupRows != 0 || Ks < kStepCols || Ks % kStepCols != 0)
        return bhi_fail(BHI_EINVAL, "need split_k >= 1, M a multiple of 4 and Ks a multiple of 128");
    if (exp_words < kTailPadWords || exp_words >= ((int64_t)1 << 32))
        return bhi_fail(BHI_EINVAL, "exponent stream size out of range");
    s->M = M; s->Ks = Ks; s->split_k = split_k;
    s->nc = chunks_per_group(M, Ks, split_k);
    s->steps = Ks / kStepCols;
    s->nc_log2 = 0;
    while ((1 << s->nc_log2) < s->nc) ++s->nc_log2;
    if ((1 << s->nc_log2) != s->nc) return bhi_fail(BHI_ELAYOUT, "chunks per group must be a power of two");
    if ((s->steps + s->nc - 1) / s->nc > kMaxTaskSteps)
        return bhi_fail(BHI_ELAYOUT, "more than 128 steps per task");
    s->total_words = (uint32_t)(exp_words - kTailPadWords);
    return 0;
}

// Blocks a member needs: one per NW / P row groups.
static inline int gemv_blocks(const bhi::Shape& s) {
    using namespace bhi;
    const int per_group = s.split_k * s.nc;
    const int P = per_group < kWavesPerBlock ? per_group : kWavesPerBlock, gpb = kWavesPerBlock / P;
    return (s.M / kGroupRows + gpb - 1) / gpb;
}

// Segment length of a launch.  Short segments start sooner and lose less on short tasks:
// 5-10 % faster whenever every wavefront of the launch is resident at once, and on tasks
// of 8 or 16 steps in any case.  A launch with more wavefronts than the GPU holds (a group
// of weights) runs at full contention for most of its time; there, on long tasks (28
// steps), the smaller per-step overhead of long segments wins by about 5 %.
static inline int first_block_of(const bhi::Group& g, int i) { return i < g.n ? g.m[i].first_block : 0x7FFFFFFF; }

constexpr int kLongTaskSteps = 24;
template <class Codec, int BS>
static inline void launch_gemv(const void* X, const bhi::Group& grp, int blocks, hipStream_t stream) {
    using namespace bhi;
    const dim3 grid((unsigned)blocks), block(kWavesPerBlock * kLanes);
    const Shape& s0 = grp.m[0].s;
    if ((long long)blocks * kWavesPerBlock > kTargetTasks && s0.steps / s0.nc >= kLongTaskSteps)
        hipLaunchKernelGGL((bhi::gemv_kernel<Codec, BS, kWavesPerBlock, kSegLong>), grid, block, 0, stream, (const uint16_t*)X, first_block_of(grp, 1), first_block_of(grp, 2), first_block_of(grp, 3), grp);
    else
        hipLaunchKernelGGL((bhi::gemv_kernel<Codec, BS, kWavesPerBlock, kSegShort>), grid, block, 0, stream, (const uint16_t*)X, first_block_of(grp, 1), first_block_of(grp, 2), first_block_of(grp, 3), grp);
}

// Launches with a transformed X (kXRms, kXSiluMul): batch 1..4, short segments.
template <class Codec, int XM>
static inline void launch_gemv_x(int batch, const void* X, const bhi::Group& grp, int blocks, hipStream_t stream) {
    using namespace bhi;
    const dim3 grid((unsigned)blocks), block(kWavesPerBlock * kLanes);
    const uint16_t* x = (const uint16_t*)X;
    switch (batch) {
        case 1: hipLaunchKernelGGL((gemv_kernel<Codec, 1, kWavesPerBlock, kSegShort, XM>), grid, block, 0, stream, x, first_block_of(grp, 1), first_block_of(grp, 2), first_block_of(grp, 3), grp); break;
        case 2: hipLaunchKernelGGL((gemv_kernel<Codec, 2, kWavesPerBlock, kSegShort, XM>), grid, block, 0, stream, x, first_block_of(grp, 1), first_block_of(grp, 2), first_block_of(grp, 3), grp); break;
        case 3: hipLaunchKernelGGL((gemv_kernel<Codec, 3, kWavesPerBlock, kSegShort, XM>), grid, block, 0, stream, x, first_block_of(grp, 1), first_block_of(grp, 2), first_block_of(grp, 3), grp); break;
        default: hipLaunchKernelGGL((gemv_kernel<Codec, 4, kWavesPerBlock, kSegShort, XM>), grid, block, 0, stream, x, first_block_of(grp, 1), first_block_of(grp, 2), first_block_of(grp, 3), grp); break;
    }
}

template <class Codec>
static inline void launch_gemv_batch(int batch, const void* X, const bhi::Group& grp, int blocks, hipStream_t st,
                                     int x_mode = bhi::kXPlain) {
    if constexpr (Codec::kTransformsX) {
        if (x_mode == bhi::kXRms) return launch_gemv_x<Codec, bhi::kXRms>(batch, X, grp, blocks, st);
        if (x_mode == bhi::kXSiluMul) return launch_gemv_x<Codec, bhi::kXSiluMul>(batch, X, grp, blocks, st);
    }
    switch (batch) {
        case 1: launch_gemv<Codec, 1>(X, grp, blocks, st); break;
        case 2: launch_gemv<Codec, 2>(X, grp, blocks, st); break;
        case 3: launch_gemv<Codec, 3>(X, grp, blocks, st); break;
        case 4: launch_gemv<Codec, 4>(X, grp, blocks, st); break;
        case 5: launch_gemv<Codec, 5>(X, grp, blocks, st); break;
        case 6: launch_gemv<Codec, 6>(X, grp, blocks, st); break;
        case 7: launch_gemv<Codec, 7>(X, grp, blocks, st); break;
        default: launch_gemv<Codec, 8>(X, grp, blocks, st); break;
    }
}

// A single weight is a group of one.
template <class Codec>
static inline void launch_gemv_batch(int batch, const void* A_rem, const void* A_exp, const void* X, void* Y,
                                     const void* offsets, const void* table, const void* header,
                                     const bhi::Shape& s, hipStream_t st) {
    bhi::Group grp = {};
    grp.n = 1;
    grp.m[0] = bhi::Member{(const uint8_t*)A_rem, (const uint32_t*)A_exp, (uint16_t*)Y, (const uint32_t*)offsets,
                           (const uint32_t*)table, (const uint8_t*)header, nullptr, nullptr, s, 0};
    launch_gemv_batch<Codec>(batch, X, grp, gemv_blocks(s), st);
}

static_assert(sizeof(bhi_gemv_member) == 88, "bindings mirror this struct field by field");

// The grouped entry points: members of one codec that share X, split_k and Ks.
// `table_bytes_expected` > 0 checks every member's table size (Huffman).
template <class Codec>
static inline int gemv_grouped(const bhi_gemv_member* members, int n_members, const void* X, int split_k, int Ks,
                               int batch, int64_t table_bytes_expected, bool header_is_table, hipStream_t st,
                               int x_mode = bhi::kXPlain, const void* x_aux = nullptr, float eps = 0.f) {
    using namespace bhi;
    if (!members || !X) return bhi_fail(BHI_EINVAL, "null pointer");
    if (n_members < 1 || n_members > kMaxMembers) return bhi_fail(BHI_EINVAL, "a group has 1 to 4 members");
    if (batch < 1) return bhi_fail(BHI_EINVAL, "batch must be >= 1");
    if (batch > kMaxBatch) return bhi_fail(BHI_EBATCH, "fused GEMV supports batch <= 8");
    if (x_mode != kXPlain) {
        if (x_mode != kXRms && x_mode != kXSiluMul) return bhi_fail(BHI_EINVAL, "unknown X transform");
        if (!Codec::kTransformsX) return bhi_fail(BHI_EINVAL, "this codec's kernels take X as it is");
        if (!x_aux) return bhi_fail(BHI_EINVAL, "the X transform needs its second operand (gamma or gate)");
        if (batch > 4) return bhi_fail(BHI_EBATCH, "a transformed X is fused for batch <= 4");
    }
    Group grp = {};
    grp.n = n_members;
    grp.xaux = (const uint16_t*)x_aux;
    grp.eps = eps;
    long long blocks = 0;
    for (int i = 0; i < n_members; ++i) {
        const bhi_gemv_member& m = members[i];
        if (!m.A_rem || !m.A_exp || !m.Y || !m.offsets || !m.table || (!header_is_table && !m.header))
            return bhi_fail(BHI_EINVAL, "null pointer in a group member");
        if (table_bytes_expected > 0 && m.table_bytes != table_bytes_expected)
            return bhi_fail(BHI_ELAYOUT, "decode table of a group member has the wrong size");
        Shape s;
        if (int rc = check_shape(split_k, m.M, Ks, m.exp_words, &s)) return rc;
        grp.m[i] = Member{(const uint8_t*)m.A_rem, (const uint32_t*)m.A_exp, (uint16_t*)m.Y, (const uint32_t*)m.offsets,
                          (const uint32_t*)m.table, (const uint8_t*)(header_is_table ? m.table : m.header),
                          (const uint16_t*)m.bias, (const uint16_t*)m.residual, s, (int)blocks};
        blocks += gemv_blocks(s);
    }
    if (blocks > 0x7FFFFFFFll) return bhi_fail(BHI_EINVAL, "group too large for one launch");
    launch_gemv_batch<Codec>(batch, X, grp, (int)blocks, st, x_mode);
    return 0;
}

template <class Codec>
static inline void launch_decode(const void* A_rem, const void* A_exp, void* Y, const void* offsets,
                                 const void* table, const void* header, const bhi::Shape& s, hipStream_t st) {
    using namespace bhi;
    constexpr int NW = 4;
    const long long ntasks = (long long)(s.M / kGroupRows) * s.split_k * s.nc;
    const unsigned grid = (unsigned)((ntasks + NW - 1) / NW);
    hipLaunchKernelGGL((decode_kernel<Codec, NW, kSegLong>), dim3(grid), dim3(NW * kLanes), 0, st,
                       (const uint8_t*)A_rem, (const uint32_t*)A_exp, (uint16_t*)Y, (const uint32_t*)offsets,
                       (const uint32_t*)table, (const uint8_t*)header, s);
}

#include "bhi_mma.h"
