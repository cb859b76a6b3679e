// Shared device helpers and format constants for the gfx950 kernels.
//
// Stream format in one paragraph (the numpy model under oracle/ is the executable
// statement): a task = (split k, 4-row group g, chunk c).  One wavefront decodes one
// task.  Per step every lane l = 4*b + i owns row 4g+i and the 8 columns
// 128*t + 8*b + j, i.e. four exponent pairs.  A lane's code bits start at bit 2 of its
// private bitstring, the bitstring is cut into 32-bit words, and word w of lane l sits
// at [64*w + l] of the task block ("row" w); the block has as many rows as its longest
// lane.  Escaped pairs keep only the ESC code in band; their two bytes are read
// backwards from the end of the task block in (pair, lane) order.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bhi {

constexpr int kFormatVersion = 2;
constexpr int kLanes = 64;
constexpr int kGroupRows = 4;
constexpr int kLaneCols = 8;
constexpr int kStepCols = 128;
constexpr int kPairsPerStep = 4;
constexpr int kWindowWords = 3;
constexpr int kHeaderBits = 2;
constexpr int kTableBits = 11;
constexpr int kTableEntries = 1 << kTableBits;
constexpr uint32_t kTableMask = (kTableEntries - 1) << 2;   // byte address mask
constexpr int kMaxBatch = 8;
constexpr int kAnsPrecision = 8;
constexpr int kAlignWords = 4;
constexpr int kTailPadWords = 2048;
#ifndef BHI_TARGET_TASKS
#define BHI_TARGET_TASKS 6144
#endif
constexpr int kTargetTasks = BHI_TARGET_TASKS;      // wavefronts kept resident: 256 CUs x 4 SIMDs x 6
constexpr int kMinChunkSteps = 4;
constexpr int kMaxChunks = 4;
constexpr int kMaxTaskSteps = 128;
constexpr int kWavesPerBlock = 4;
constexpr int kBlockThreads = kWavesPerBlock * kLanes;

__host__ __device__ inline int chunks_per_group(int M, int Ks, int split_k) {
    int steps = Ks / kStepCols;
    int nc = 1;
    while (nc < kMaxChunks && (long long)(M / kGroupRows) * split_k * nc * 2 <= kTargetTasks &&
           steps / (nc * 2) >= kMinChunkSteps)
        nc *= 2;
    // The tasks of a row group are dealt to the four wavefronts of a block: six tasks would give
    // two wavefronts two tasks and two of them one (4096x12288 with three splits: 32 steps on the
    // longest wavefront where 24 would do), so a count above four that is no multiple of four
    // is doubled once more.
    if (split_k * nc > kWavesPerBlock && (split_k * nc) % kWavesPerBlock != 0 && nc < kMaxChunks &&
        steps / (nc * 2) >= kMinChunkSteps)
        nc *= 2;
    return nc;
}

__device__ __forceinline__ uint32_t lane_rank(uint64_t mask) {
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

__device__ __forceinline__ uint64_t ballot(bool p) { return __builtin_amdgcn_ballot_w64(p); }

__device__ __forceinline__ uint32_t uniform(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

// Table entry: len in bits 4..0 (bits 5, 6 clear), exponent a in bits 14..7 and exponent
// b in bits 30..23 -- where a packed pair of BF16 values keeps them -- and the ESC flag in
// bit 31.  The low six bits of a sum of raw entries are therefore the sum of their
// lengths (at most 48), and an OR of entries is negative iff one of them is an ESC.
constexpr uint32_t kEscFlag = 0x80000000u;

// Two BF16 values from (table entry, rem bytes).  `z` holds [rb, rb, ra, ra]: the sign
// comes from the upper copy of each rem byte, the mantissa from the lower copy.
__device__ __forceinline__ uint32_t rebuild_pair(uint32_t e, uint32_t z) {
    return (e & 0x7F807F80u) | (z & 0x807F807Fu);
}

__device__ __forceinline__ uint32_t rem_lo_pair(uint32_t r) { return __builtin_amdgcn_perm(r, r, 0x01010000u); }
__device__ __forceinline__ uint32_t rem_hi_pair(uint32_t r) { return __builtin_amdgcn_perm(r, r, 0x03030202u); }

// Sum over the 16 lanes that share `lane & 3` (the 16 column blocks of a step), left in every
// lane: two rotations inside the rows of 16 lanes (DPP), then the two row-swap instructions of
// gfx950 -- no trip through the LDS crossbar, which four dependent `__shfl_xor` would take.
__device__ __forceinline__ float sum_over_column_blocks(float a) {
    a += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(a), 0x124, 0xF, 0xF, false));   // row_ror:4
    a += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(a), 0x128, 0xF, 0xF, false));   // row_ror:8
    // v_permlane16_swap exchanges rows 1, 3 of its first operand with rows 0, 2 of the second:
    // from two copies of `a` come [r0 r0 r2 r2] and [r1 r1 r3 r3]
    typedef uint32_t pair_t __attribute__((ext_vector_type(2)));
    pair_t p = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(a), false, false);
    a = __uint_as_float(p.x) + __uint_as_float(p.y);
    // v_permlane32_swap exchanges the upper half of the first with the lower half of the second
    p = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(a), false, false);
    return __uint_as_float(p.x) + __uint_as_float(p.y);
}

// A word of memory that nothing writes while the kernel runs (offsets, the format header),
// read at a wave-uniform address: through the constant address space the compiler issues a
// scalar load, which neither queues behind the vector loads in flight nor has to be waited
// for with them.  At a lane-dependent address it is an ordinary vector load.
typedef __attribute__((address_space(4))) const uint32_t const_u32;
__device__ __forceinline__ uint32_t constant_word(const uint32_t* p) {
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wold-style-cast"
    return *(const_u32*)p;
#pragma clang diagnostic pop
}

// A block barrier that orders LDS traffic only.  __syncthreads() also waits for every global
// load in flight (s_waitcnt vmcnt(0)), which would drain the prefetched windows at each barrier.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xC07F);      // lgkmcnt(0): this wavefront's LDS writes have landed
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Position of a task's stream and of the stream that follows it in (k, g, c) order.
struct TaskSpan { uint32_t base, end; };

__device__ __forceinline__ TaskSpan task_span(const uint32_t* __restrict__ offsets, int M, int split_k, int nc,
                                              int k, int g, int c, uint32_t total_words) {
    // offsets[k][4 * g + c] for c < nc; the stream that follows starts at the next used slot:
    // the group's next chunk, or slot 0 of the next group (which for the last group of a split
    // is the first slot of the next split), or, for the very last task, the end of the stream.
    // Both loads are issued unconditionally (the second at a clamped index), without branches.
    TaskSpan s;
    const int at = k * M + kGroupRows * g;
    const int next = c + 1 < nc ? at + c + 1 : at + kGroupRows;
    const int slots = split_k * M;
    s.base = constant_word(offsets + (at + c));
    const uint32_t e = constant_word(offsets + (next < slots ? next : slots - 1));
    s.end = next < slots ? e : total_words;
    return s;
}

// A task is processed in segments of S steps; the global loads of a segment (all
// unconditional) are issued back to back, one whole segment before they are used.  VMEM
// loads complete in issue order, so a load issued on demand inside a segment would make
// its wait drain the whole queue.  Two steps per segment: on short tasks (7 steps) that is 6-12 %
// faster than four, on long ones 0-5 %, and it needs 14-24 registers less.
//
// Exponent rows are staged in a per-wavefront LDS ring of kRingRows rows (256 B each).
// Row r lives in slot r % kRingRows; slots 0 and 1 are mirrored behind the last slot so
// that the three rows of a window are always at +0, +256 and +512 bytes of one address.
// Lanes sit at different rows, yet row r of lane l is always in bank l % 32: window reads
// are conflict free.  A task stages kPrimeRows rows before its first step; every segment
// then prefetches the next S rows if every lane has made room for them, and the
// following segment commits them to the ring.  A lane whose window is not staged (a
// cheap per-step test) reads it from global memory instead.
// The segment length S is a template parameter of the walk: kSegShort or kSegLong steps,
// with as many rows prefetched per segment.
constexpr int kSegShort = 2;
constexpr int kSegLong = 4;
#ifndef BHI_RING_ROWS
#define BHI_RING_ROWS 16
#endif
constexpr int kRingRows = BHI_RING_ROWS;
constexpr int kRingRowsLog2 = kRingRows == 8 ? 3 : kRingRows == 16 ? 4 : kRingRows == 32 ? 5 : -1;
static_assert(kRingRowsLog2 > 0, "ring of 8, 16 or 32 rows");
#ifndef BHI_PRIME_ROWS
#define BHI_PRIME_ROWS 8
#endif
constexpr int kPrimeRows = BHI_PRIME_ROWS;      // rows staged before the first step
constexpr int kRingSlots = kRingRows + 2;   // slots 0 and 1 are mirrored behind the last one
constexpr int kRingWords = kRingSlots * kLanes;
static_assert(kRingRows % kSegLong == 0 && kSegLong % kSegShort == 0 && (kRingRows & (kRingRows - 1)) == 0 && kSegShort >= 2,
              "rows are committed in aligned groups; the group at slot 0 carries both mirrored rows");
static_assert(kPrimeRows % kSegLong == 0 && kPrimeRows >= 4 && kPrimeRows <= kRingRows, "priming stages whole groups");

// The rem plane is read once, front to back, 512 aligned bytes per wavefront and step:
// loaded with the non-temporal hint its lines leave the caches first and stop displacing
// what is read again (the table, X, the row lines two loads share).  Measured on
// 18944x3584 at batch 1: 24.2 -> 21.9 us.  The same hint on the rows gains nothing, whether
// task blocks are aligned to 16 bytes (neighbouring row loads share a line) or to 128.
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint2 stream_load(const uint2* p) {
    const u32x2_t v = __builtin_nontemporal_load((const u32x2_t*)p);
    return make_uint2(v.x, v.y);
}

// LDS pointers are kept in their own address space: a pointer that may be LDS or global
// turns every access into a flat load, which waits on the global-memory counter.
typedef __attribute__((address_space(3))) uint32_t lds_u32;

// A lane's view of its task block: a bit position in its own column of rows, and the
// wavefront's LDS ring of staged rows.  The codec cursors below build on it.
// POS_SHIFT: `pos` counts bits (5: the Huffman cursor, whose windows start at any bit) or whole
// rows (0: the rANS cursor, which only ever takes whole words -- advancing by one row is then an
// add with carry-in off the refill test instead of a select and an add).
template <int POS_SHIFT>
struct RowRingT {
    uint32_t pos;            // position of the lane's window, in bits or rows (codec specific bias)
    uint32_t rhi;            // wave-uniform: rows [0, rhi) have been staged
    uint32_t lim;            // wave-uniform: windows starting below this bit are fully staged
    uint32_t nrows;          // wave-uniform: rows of the block worth staging
    const uint32_t* bp;      // task block, this lane's column
    lds_u32* ring;           // this wavefront's LDS ring, this lane's column

    __device__ __forceinline__ void open_rows(const uint32_t* __restrict__ words, TaskSpan span, int lane, uint32_t* ring_) {
        bp = words + span.base + lane;
        ring = (lds_u32*)ring_ + lane;
        nrows = uniform((span.end - span.base + kLanes - 1) / kLanes);
        pos = 0;
        rhi = 0;
        lim = 0;
    }

    // This lane's word of row p >> POS_SHIFT; the next two rows follow at +kLanes, +2*kLanes words.
    __device__ __forceinline__ const lds_u32* slot_of(uint32_t p) const {
        // v_bfe_u32 + v_lshl_add_u32; written as shift and mask the compiler makes it three
        // instructions on the critical path of every step
        uint32_t slot;
        asm("v_bfe_u32 %0, %1, %2, %3" : "=v"(slot) : "v"(p), "n"(POS_SHIFT), "n"(kRingRowsLog2));
        return ring + slot * kLanes;
    }

    // Stage the first kRingRows rows of the block, once per task, in two halves so that the
    // caller can put other work between the loads and their use.  Rows past the end of a
    // short block are filler nobody decodes.
    __device__ __forceinline__ void prime_issue(uint32_t (&v)[kPrimeRows]) const {
#pragma unroll
        for (int j = 0; j < kPrimeRows; ++j) {
            const uint32_t r = (uint32_t)j < nrows ? (uint32_t)j : nrows - 1;
            v[j] = bp[(size_t)r * kLanes];
        }
    }
    __device__ __forceinline__ void prime_commit(const uint32_t (&v)[kPrimeRows]) {
#pragma unroll
        for (int j = 0; j < kPrimeRows; ++j) ring[j * kLanes] = v[j];
        ring[kRingRows * kLanes] = v[0];
        ring[(kRingRows + 1) * kLanes] = v[1];
        rhi = kPrimeRows;
        set_lim();
    }

    // windows read rows m..m+2; once the whole block is staged nothing can be missing
    __device__ __forceinline__ void set_lim() {
        lim = rhi >= nrows ? 0xFFFFFFFFu : (rhi - 2) << POS_SHIFT;
    }

    // Can the next R rows be staged now?  Row r may replace row r - kRingRows once
    // no window needs it, i.e. once every lane is past it: one compare and a ballot.  Rows
    // are staged in whole groups: rhi stays a multiple of R and a group never wraps
    // around the ring.  Decided before the loads are issued so that they need not be
    // issued in vain (and so that the compiler cannot sink them behind the decision).
    template <int R>
    __device__ __forceinline__ bool room() const { return room_at<R>(rhi); }
    // The same question for the R rows that start at row `first` >= rhi (a group fetched
    // further ahead than the next one): positions only advance, so room now is room later.
    template <int R>
    __device__ __forceinline__ bool room_at(uint32_t first) const {
        const uint32_t top = first + R;
        const uint32_t oldest = top > (uint32_t)kRingRows ? (top - kRingRows) << POS_SHIFT : 0u;
        return first < nrows && ballot(pos < oldest) == 0;
    }

    // The next R rows after the staged ones: one address, immediate offsets.  Rows
    // past the end of the block belong to the next block or to the zero pad that ends the
    // stream; they are loaded, staged, never decoded.
    template <int R>
    __device__ __forceinline__ void prefetch(uint32_t (&v)[R]) const { prefetch_at(v, rhi); }
    template <int R>
    __device__ __forceinline__ void prefetch_at(uint32_t (&v)[R], uint32_t first) const {
        const uint32_t* p = bp + (size_t)first * kLanes;
#pragma unroll
        for (int j = 0; j < R; ++j) v[j] = p[j * kLanes];
    }

    template <int R>
    __device__ __forceinline__ void commit(const uint32_t (&v)[R]) {
        lds_u32* dst = ring + (rhi & (kRingRows - 1)) * kLanes;
#pragma unroll
        for (int j = 0; j < R; ++j) dst[j * kLanes] = v[j];
        if ((rhi & (kRingRows - 1)) == 0) {
            ring[kRingRows * kLanes] = v[0];
            ring[(kRingRows + 1) * kLanes] = v[1];
        }
        rhi += R;
        set_lim();
    }

    // The lane's window: rows m, m+1, m+2 with m = pos >> POS_SHIFT.
    __device__ __forceinline__ void window(uint32_t& lo, uint32_t& hi, uint32_t& nx) const {
        // the ring is read unconditionally (a slot address is always valid); lanes whose
        // window is not staged there get it from global memory instead
        const lds_u32* w = slot_of(pos);
        lo = w[0];
        hi = w[kLanes];
        nx = w[2 * kLanes];
        if (__builtin_expect(ballot(pos >= lim) != 0, 0)) fetch_behind(lo, hi, nx);
    }

    // Some lane's window is not staged (it ran more than a ring ahead of the slowest lane,
    // or faster than the segments stage rows): those lanes read global memory.  The
    // address is kept in range for the others (the stream ends in a zero pad anyway).
    __device__ __forceinline__ void fetch_behind(uint32_t& lo, uint32_t& hi, uint32_t& nx) const {
        const bool staged = pos < lim;
        const uint32_t* g = bp + (size_t)(staged ? 0u : pos >> POS_SHIFT) * kLanes;
        const uint32_t g0 = g[0], g1 = g[kLanes], g2 = g[2 * kLanes];
        // vmcnt(0) here, inside the rare branch: otherwise the wait lands behind the join
        // and every step would drain the operand loads that are in flight for later steps
        __builtin_amdgcn_s_waitcnt(0x0F70);
        lo = staged ? lo : g0;
        hi = staged ? hi : g1;
        nx = staged ? nx : g2;
    }
};

// The table entry selected by bits 2..12 of a (pre-shifted) window.
__device__ __forceinline__ uint32_t table_entry(const char* tb, uint32_t w) {
    return *(const uint32_t*)(tb + (w & kTableMask));
}

// Per-lane Huffman bit cursor.  pos = bit position - 2: the window is kept shifted left
// by two so that `window & kTableMask` is the byte address of the table entry.
typedef RowRingT<5> RowRing;

struct HuffCursor : RowRing {
    uint32_t eptr;           // wave-uniform: escape entries consumed so far
    const uint32_t* ep;      // one past the task block (escape list grows down from here)

    __device__ __forceinline__ void open(const uint32_t* __restrict__ words, TaskSpan span, int lane, uint32_t* ring_) {
        open_rows(words, span, lane, ring_);
        ep = words + span.end;
        eptr = 0;
    }

    __device__ __forceinline__ void start(const uint32_t*) {}

    // Decode the four pairs of one step; e[q] are raw table entries.
    template <bool HAS_ESC>
    __device__ __forceinline__ void step(const uint32_t* __restrict__ table, uint32_t (&e)[4], int) {
        uint32_t lo, hi, nx;
        window(lo, hi, nx);
        const char* tb = (const char*)table;
        const uint32_t c = pos & 31u;
        const uint32_t wlo = __builtin_amdgcn_alignbit(hi, lo, c);
        e[0] = table_entry(tb, wlo);
        const uint32_t w1 = wlo >> (e[0] & 31u);
        e[1] = table_entry(tb, w1);
        const uint32_t whi = __builtin_amdgcn_alignbit(nx, hi, c);
        const uint32_t t01 = e[0] + e[1];
        const uint32_t w2 = __builtin_amdgcn_alignbit(whi, wlo, t01);
        e[2] = table_entry(tb, w2);
        const uint32_t w3 = w2 >> (e[2] & 31u);
        e[3] = table_entry(tb, w3);
        pos += (t01 + e[2] + e[3]) & 0x3Fu;
        if (HAS_ESC) {
            // pins the cursor update in front of the branch: the entries then die at it and
            // the rare path patches them in place, without register copies on the common one
            asm volatile("" : "+v"(pos));
            const uint32_t any = e[0] | e[1] | e[2] | e[3];
            if (__builtin_expect(ballot((int32_t)any < 0) != 0, 0)) escapes(e);
        }
    }

    // Exponents of escaped pairs come from the escape list, in (pair, lane) order.
    __device__ __forceinline__ void escapes(uint32_t (&e)[4]) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            bool esc = (int32_t)e[q] < 0;
            uint64_t m = ballot(esc);
            if (esc) {
                uint32_t v = *(ep - 1 - (eptr + lane_rank(m)));
                e[q] = ((v & 0xFFu) << 7) | ((v & 0xFF00u) << 15);
            }
            eptr = uniform(eptr + (uint32_t)__builtin_popcountll(m));
        }
    }
};

// Per-lane rANS cursor: one 64-bit state, precision 8, table words (sym<<24)|(freq<<12)|rem.
// The state is looked at after every four symbols; when it has dropped below 2**32 the
// lane's next row word is shifted in.  pos = index of the lane's next row.
struct AnsCursor : RowRingT<0> {
    uint32_t xl, xh;         // the state

    __device__ __forceinline__ void open(const uint32_t* __restrict__ words, TaskSpan span, int lane, uint32_t* ring_) {
        open_rows(words, span, lane, ring_);
    }

    // rows 0 and 1 are the initial state (call after prime_commit())
    __device__ __forceinline__ void start(const uint32_t*) {
        xl = ring[0];
        xh = ring[kLanes];
        pos = 2;
    }

    // one symbol: returns the second word of its table entry ((sym << 23) | rem), advances the state
    __device__ __forceinline__ uint32_t symbol(const uint32_t* __restrict__ table) {
        // byte 0 of the state, times eight, in one instruction (written as a mask and a shift
        // the compiler makes it two; eight symbols per step, the kernel is bound by VALU issue)
        uint32_t off;
        asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0"
            : "=v"(off) : "v"(3u), "v"(xl));
        const uint2 ent = *(const uint2*)((const char*)table + off);       // {freq, (sym << 23) | rem}
        // state >> 8 in one instruction (the compiler splits a 64-bit shift by a constant into two)
        uint64_t y;
        asm("v_lshrrev_b64 %0, 8, %1" : "=v"(y) : "v"(((uint64_t)xh << 32) | xl));
        const uint64_t lowp = (uint64_t)ent.x * (uint32_t)y + (ent.y & 0xFFFu);   // v_mad_u64_u32
        xl = (uint32_t)lowp;
        // freq <= 256 and y >> 32 < 2**24: a 24-bit multiply-add (the state is valid: < 2**64)
        xh = __umul24(ent.x, (uint32_t)(y >> 32)) + (uint32_t)(lowp >> 32);
        return ent.y;
    }

    __device__ __forceinline__ void refill(uint32_t word) {
        const bool need = xh == 0u;
        xh = need ? xl : xh;
        xl = need ? word : xl;
        pos += need ? 1u : 0u;
    }

    // two symbols -> one pair entry in the Huffman table's format (a<<7 | b<<23): the upper
    // halves of the two entry words side by side
    __device__ __forceinline__ uint32_t pair(const uint32_t* __restrict__ table) {
        const uint32_t a = symbol(table);
        const uint32_t b = symbol(table);
        return __builtin_amdgcn_perm(b, a, 0x07060302u);
    }

    template <bool UNUSED>
    __device__ __forceinline__ void step(const uint32_t* __restrict__ table, uint32_t (&e)[4], int) {
        uint32_t lo, hi, nx;
        window(lo, hi, nx);
        e[0] = pair(table);
        e[1] = pair(table);
        const bool first = xh == 0u;
        refill(lo);
        e[2] = pair(table);
        e[3] = pair(table);
        refill(first ? hi : lo);
    }
};

// Fixed-width exponent code: the eight nibbles of a lane and step sit in one word of the
// task block's row t (column j in bits 4j..4j+3); a nibble is the exponent's offset from
// `base`, 15 marks an exponent that travels in the escape list instead.  Nothing here
// is sequential: the cursor only hands out the words the segment prefetched.  It has
// the interface of the entropy cursors so that the same task walk drives it; the LDS
// ring is not used.
struct NibbleCursor {
    const uint32_t* bp;      // task block, this lane's column
    const uint32_t* ep;      // one past the task block (escape list grows down from here)
    uint32_t eptr;           // wave-uniform: escape entries consumed so far
    uint32_t next;           // wave-uniform: first step not prefetched yet
    uint32_t base4;          // wave-uniform: the base exponent in every byte
    uint32_t cur[kSegLong];  // the words of the segment being decoded (one row per step)

    __device__ __forceinline__ void open(const uint32_t* __restrict__ words, TaskSpan span, int lane, uint32_t*) {
        bp = words + span.base + lane;
        ep = words + span.end;
        eptr = 0;
        next = 0;
    }
    __device__ __forceinline__ void prime_issue(uint32_t (&)[kPrimeRows]) const {}
    __device__ __forceinline__ void prime_commit(const uint32_t (&)[kPrimeRows]) const {}
    __device__ __forceinline__ void start(const uint32_t* lut) { base4 = uniform(lut[0] & 0xFFu) * 0x01010101u; }
    template <int R>
    __device__ __forceinline__ bool room() const { return true; }

    // rows past the last step belong to the escape list, the next block or the zero pad
    template <int R>
    __device__ __forceinline__ void prefetch(uint32_t (&v)[R]) {
        const uint32_t* p = bp + (size_t)next * kLanes;
#pragma unroll
        for (int j = 0; j < R; ++j) v[j] = p[j * kLanes];
        next += R;                          // segments are prefetched in order, possibly one ahead
    }
    template <int R>
    __device__ __forceinline__ void commit(const uint32_t (&v)[R]) {
        static_assert(R <= kSegLong, "cur holds one segment");
#pragma unroll
        for (int j = 0; j < R; ++j) cur[j] = v[j];
    }

    // pair entries in the Huffman table's format (a<<7 | b<<23) for step i of the segment
    template <bool HAS_ESC>
    __device__ __forceinline__ void step(const uint32_t*, uint32_t (&e)[4], int i) {
        const uint32_t d = cur[i];
        uint32_t even = (d & 0x0F0F0F0Fu) + base4;            // exponents of columns 0, 2, 4, 6
        uint32_t odd = ((d >> 4) & 0x0F0F0F0Fu) + base4;      // exponents of columns 1, 3, 5, 7
        if (HAS_ESC) {
            uint32_t t = d & (d >> 1);
            t &= t >> 2;                                       // bit 4j set iff nibble j is 15
            if (__builtin_expect(ballot((t & 0x11111111u) != 0) != 0, 0)) escapes(t, even, odd);
        }
        e[0] = __builtin_amdgcn_perm(odd, even, 0x0C040C00u) << 7;
        e[1] = __builtin_amdgcn_perm(odd, even, 0x0C050C01u) << 7;
        e[2] = __builtin_amdgcn_perm(odd, even, 0x0C060C02u) << 7;
        e[3] = __builtin_amdgcn_perm(odd, even, 0x0C070C03u) << 7;
    }

    // escaped exponents come from the escape list, in (column, lane) order
    __device__ __forceinline__ void escapes(uint32_t t, uint32_t& even, uint32_t& odd) {
#pragma unroll
        for (int j = 0; j < kLaneCols; ++j) {
            const bool esc = ((t >> (4 * j)) & 1u) != 0;
            const uint64_t m = ballot(esc);
            if (esc) {
                const uint32_t raw = *(ep - 1 - (eptr + lane_rank(m))) & 0xFFu;
                uint32_t& half = (j & 1) ? odd : even;
                const int sh = 8 * (j >> 1);
                half = (half & ~(0xFFu << sh)) | (raw << sh);
            }
            eptr = uniform(eptr + (uint32_t)__builtin_popcountll(m));
        }
    }
};

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);   // quiet NaN
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

}  // namespace bhi
