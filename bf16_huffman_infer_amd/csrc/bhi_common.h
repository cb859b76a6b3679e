// Shared device helpers and format constants for the gfx950 kernels.
//
// Stream format in one paragraph (the numpy model under oracle/ is the executable
// statement): a task = (split k, 4-row group g, chunk c).  One wavefront decodes one
// task.  Per step every lane l = 4*b + i owns row 4g+i and the 8 columns
// 128*t + 8*b + j, i.e. four exponent pairs.  A lane's code bits start at bit 8 of its
// private bitstring (bits 0..7 = number of refill loads it will make); the bitstring is
// cut into 32-bit words; words 0..2 of lane l sit at [l], [64+l], [128+l] of the task
// stream and all later words are stored in the order the wavefront consumes them:
// after each step, while any lane's cursor has left its word, those lanes advance one
// word and the ones that still have loads left take consecutive stream words in lane
// order.  Escaped pairs keep only the ESC code in band; their two bytes are read
// backwards from the end of the task stream in (pair, lane) order.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bhi {

constexpr int kFormatVersion = 1;
constexpr int kLanes = 64;
constexpr int kGroupRows = 4;
constexpr int kLaneCols = 8;
constexpr int kStepCols = 128;
constexpr int kPairsPerStep = 4;
constexpr int kInitWords = 3;
constexpr int kHeaderBits = 8;
constexpr int kCursorBias = 2;
constexpr int kTableBits = 12;
constexpr int kTableEntries = 1 << kTableBits;
constexpr uint32_t kTableMask = (kTableEntries - 1) << 2;   // byte address mask
constexpr int kMaxBatch = 8;
constexpr int kAnsPrecision = 8;
constexpr int kAlignWords = 4;
constexpr int kTailPadWords = 1024;
constexpr int kTargetTasks = 4096;
constexpr int kMinChunkSteps = 4;
constexpr int kMaxChunks = 4;
constexpr int kMaxTaskSteps = 128;
constexpr int kWavesPerBlock = 8;
constexpr int kBlockThreads = kWavesPerBlock * kLanes;

__host__ __device__ inline int chunks_per_group(int M, int Ks, int split_k) {
    int steps = Ks / kStepCols;
    int nc = 1;
    while (nc < kMaxChunks && (long long)(M / kGroupRows) * split_k * nc < kTargetTasks &&
           steps / (nc * 2) >= kMinChunkSteps)
        nc *= 2;
    return nc;
}

__device__ __forceinline__ uint32_t lane_rank(uint64_t mask) {
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

__device__ __forceinline__ uint64_t ballot(bool p) { return __builtin_amdgcn_ballot_w64(p); }

__device__ __forceinline__ uint32_t uniform(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

// Two BF16 values from (table entry, rem bytes).  `e` holds exponent a in bits 7..0 and
// exponent b in bits 23..16; `z` holds [rb, rb, ra, ra]: the sign comes from the upper
// copy of each rem byte, the mantissa from the lower copy, the exponent from e<<7.
__device__ __forceinline__ uint32_t rebuild_pair(uint32_t e, uint32_t z) {
    return ((e << 7) & 0x7F807F80u) | (z & 0x807F807Fu);
}

__device__ __forceinline__ uint32_t rem_lo_pair(uint32_t r) { return __builtin_amdgcn_perm(r, r, 0x01010000u); }
__device__ __forceinline__ uint32_t rem_hi_pair(uint32_t r) { return __builtin_amdgcn_perm(r, r, 0x03030202u); }

// Position of a task's stream and of the stream that follows it in (k, g, c) order.
struct TaskSpan { uint32_t base, end; };

__device__ __forceinline__ TaskSpan task_span(const uint32_t* __restrict__ offsets, int M, int split_k, int nc,
                                              int k, int g, int c, uint32_t total_words) {
    TaskSpan s;
    const int G = M / kGroupRows;
    s.base = offsets[(size_t)k * M + kGroupRows * g + c];
    if (c + 1 < nc)            s.end = offsets[(size_t)k * M + kGroupRows * g + c + 1];
    else if (g + 1 < G)        s.end = offsets[(size_t)k * M + kGroupRows * (g + 1)];
    else if (k + 1 < split_k)  s.end = offsets[(size_t)(k + 1) * M];
    else                       s.end = total_words;
    return s;
}

// Per-lane Huffman bit cursor over the wavefront's shared stream.
struct HuffCursor {
    uint32_t lo, hi, nx;     // three consecutive words of this lane's bitstring
    uint32_t c;              // cursor = bit position - 2 inside `lo`, < 32 between steps
    uint32_t left;           // refill loads this lane still has to make
    uint32_t ptr;            // wave-uniform: next unread refill word of the task stream
    uint32_t eptr;           // wave-uniform: escape entries consumed so far
    const uint32_t* sp;      // task stream
    const uint32_t* ep;      // one past the task stream (escape list grows down from here)

    __device__ __forceinline__ void init(const uint32_t* __restrict__ words, TaskSpan span, int lane) {
        sp = words + span.base;
        ep = words + span.end;
        lo = sp[lane];
        hi = sp[kLanes + lane];
        nx = sp[2 * kLanes + lane];
        left = lo & 0xFFu;
        c = kHeaderBits - kCursorBias;
        ptr = kInitWords * kLanes;
        eptr = 0;
    }

    // Decode the four pairs of one step.  e[q] = a | b<<16 | (len|esc<<7)<<24.
    // `nx` is first needed after the second lookup, two LDS round trips after the
    // refill of the previous step issued its load.
    __device__ __forceinline__ void step(const uint32_t* __restrict__ table, uint32_t (&e)[4]) {
        const char* tb = (const char*)table;
        uint32_t wlo = __builtin_amdgcn_alignbit(hi, lo, c);
        e[0] = *(const uint32_t*)(tb + (wlo & kTableMask));
        uint32_t l0 = e[0] >> 24;
        uint32_t w1 = wlo >> (l0 & 31u);
        e[1] = *(const uint32_t*)(tb + (w1 & kTableMask));
        uint32_t s01 = l0 + (e[1] >> 24);
        uint32_t whi = __builtin_amdgcn_alignbit(nx, hi, c);
        uint32_t w2 = __builtin_amdgcn_alignbit(whi, wlo, s01);
        e[2] = *(const uint32_t*)(tb + (w2 & kTableMask));
        uint32_t l2 = e[2] >> 24;
        uint32_t w3 = w2 >> (l2 & 31u);
        e[3] = *(const uint32_t*)(tb + (w3 & kTableMask));
        c += s01 + l2 + (e[3] >> 24);
        if (__builtin_expect(ballot(c >= 128u) != 0, 0)) escapes(e);
        // a step consumes at most 48 bits, so a lane leaves at most two words
        if (ballot(c >= 32u) != 0) {
            refill_round();
            if (__builtin_expect(ballot(c >= 32u) != 0, 0)) refill_round();
        }
    }

    // ESC entries carry 0x80 in the length byte, so every escaped pair added 128 to c.
    __device__ __forceinline__ void escapes(uint32_t (&e)[4]) {
        c &= 127u;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            bool esc = (e[q] >> 31) != 0;
            uint64_t m = ballot(esc);
            if (esc) {
                uint32_t v = *(ep - 1 - (eptr + lane_rank(m)));
                e[q] = (v & 0xFFu) | ((v & 0xFF00u) << 8);
            }
            eptr = uniform(eptr + (uint32_t)__builtin_popcountll(m));
        }
    }

    __device__ __forceinline__ void refill_round() {
        const bool cross = c >= 32u;
        if (cross) { c -= 32u; lo = hi; hi = nx; }
        const bool load = cross && left != 0;
        const uint64_t m = ballot(load);
        if (load) { nx = sp[ptr + lane_rank(m)]; left -= 1; }
        ptr = uniform(ptr + (uint32_t)__builtin_popcountll(m));
    }
};

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);   // quiet NaN
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

}  // namespace bhi
