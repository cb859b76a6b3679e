// Persistent fused decode + GEMV: a grid sized to what the GPU keeps resident, whose
// wavefronts walk MANY tasks each.
//
//   * a block stages the decode table once, for all the tasks its wavefronts will ever run;
//   * the row groups of a weight are dealt to the blocks in contiguous ranges; inside a block
//     the wavefronts pull units (a row group, or 1/upg of one) from a queue head in LDS, so a
//     SIMD's faster wavefronts take more of the block's work (an LDS atomic costs a hundred
//     clocks; one global counter serves 6144 wavefronts at 11 ns per pull, which is why the
//     queue is per block);
//   * while a task's last segment decodes, the next task's first exponent rows and first
//     operands are already in flight (their address comes from an `offsets` entry that was
//     requested a segment into the task), so a task switch costs no memory round trip;
//   * partial sums of units that share a row group meet in LDS: the partners are always in
//     the same block, the last one to arrive adds them in a fixed order and stores.
//
// Measured on MI355X at batch 1 (Huffman, interleaved A/B against the static grid, medians):
// gate+up group of two 18944x3584 40.1 us against 36.8 us, 18944x3584 alone 22.9 against
// 19.6 us, 3584x18944 28.6 against 22.0 us, 4608x3584 12.8 against 10.3 us; with tasks of half
// the length (twice the units to pull) 42.5 against 41.6 us.  The static grid is not held back
// by what this kernel removes: its middle phase already streams at the rate of a load-only
// loop, and what it loses (launch, first fill, the last blocks) a block-local queue cannot
// give back -- the hardware's own block dispatcher balances ACROSS compute units, which a
// static deal of row groups to blocks does not.  The kernel is therefore off by default
// (environment BHI_PERSIST=1 enables it for launches with more tasks than resident
// wavefronts, =2 wherever it can run) and kept for measurement.
#pragma once
// (included by bhi_task.h, after the static-grid kernels it builds on)

namespace bhi {

#ifndef BHI_PERSIST_WAVES
#define BHI_PERSIST_WAVES 12
#endif
#ifndef BHI_PERSIST_BLOCKS_PER_CU
#define BHI_PERSIST_BLOCKS_PER_CU 2
#endif
#ifndef BHI_PERSIST_SEG
#define BHI_PERSIST_SEG 2
#endif
#ifndef BHI_PERSIST_DEFAULT
#define BHI_PERSIST_DEFAULT 0
#endif
constexpr int kPersistSeg = BHI_PERSIST_SEG;
constexpr int kPersistWaves = BHI_PERSIST_WAVES;
constexpr int kPersistBlocksPerCU = BHI_PERSIST_BLOCKS_PER_CU;
constexpr int kComputeUnits = 256;
constexpr int kMaxUnitsPerGroup = 8;          // partial sums of one row group held in LDS
constexpr int kOpenGroups = 16;               // row groups whose partial sums can be open at once, per block

struct PMember {
    const uint8_t* rem;
    const uint32_t* exp;
    uint16_t* Y;
    const uint32_t* offsets;
    const uint32_t* table;
    const uint8_t* header;
    const uint16_t* bias;
    Shape s;
    int first_block, nblocks;    // this member's blocks are [first_block, first_block + nblocks)
    int upg;                     // units per row group; divides split_k * nc
};
struct PGroup {
    int n;
    PMember m[kMaxMembers];
};

// One task as the walk needs it (all wave-uniform but the two lane pointers).
// (No padding bytes: the struct is carried around a loop, and padding would travel with it
// through scratch memory.)
struct TaskCtx {
    int g, kc;                   // row group, task index inside the group (split-major, then chunk)
    int ns;                      // steps
    int end_is_total;            // nonzero: the task is the last of the stream and ends at total_words
    const uint2* rem0;           // this lane's 8 rem bytes of the task's first step
    const uint32_t* xq0;         // this lane's X pair of batch row 0, first step
    uint32_t obase, oend;        // indices into offsets[] of the task's start and of its successor's
};

__device__ __forceinline__ TaskCtx make_task(const PMember& mb, const uint16_t* __restrict__ X, int g, int kc, int lane) {
    const Shape& s = mb.s;
    const TaskId id = task_of(s, kc);
    TaskCtx t;
    t.g = g;
    t.kc = kc;
    t.ns = id.t1 - id.t0;
    t.rem0 = (const uint2*)(mb.rem + ((size_t)id.k * s.M + (size_t)kGroupRows * g) * s.Ks) + (size_t)id.t0 * kLanes + lane;
    t.xq0 = (const uint32_t*)(X + (size_t)id.k * s.Ks + (size_t)id.t0 * kStepCols) + lane;
    const int G = s.M / kGroupRows;
    t.obase = (uint32_t)id.k * s.M + kGroupRows * g + id.c;
    t.end_is_total = 0;
    if (id.c + 1 < s.nc)              t.oend = t.obase + 1;
    else if (g + 1 < G)               t.oend = (uint32_t)id.k * s.M + kGroupRows * (g + 1);
    else if (id.k + 1 < s.split_k)    t.oend = (uint32_t)(id.k + 1) * s.M;
    else { t.oend = t.obase; t.end_is_total = 1; }
    return t;
}

// What is fetched for a task before its walk begins: the rows that prime the ring and
// the operands of its first segment.
template <class Policy, int S>
struct Primed {
    uint32_t rows[kPrimeRows];
    typename Policy::Slot slot[S];
};

// The walk over one task whose first loads were issued by somebody else (the previous
// task's last segment, or the kernel's prologue).  `point_a` runs once, one whole segment
// into the task (at its start when the task has a single segment): the place to find out
// which task comes next and to request its `offsets` entries.  `point_b` runs right
// before the last segment decodes: the place to issue the next task's first loads.  Both
// sit in straight-line code, so the compiler's count of outstanding loads stays exact.
template <bool HAS_ESC, int S, class Cursor, class Policy, class PointA, class PointB>
__device__ __forceinline__ void run_task_primed(Cursor& cur, const uint32_t* lut, Policy& pol, int ns,
                                                const Primed<Policy, S>& pr, PointA point_a, PointB point_b) {
    typename Policy::Slot a[S], b[S];
#pragma unroll
    for (int i = 0; i < S; ++i) a[i] = pr.slot[i];
    pol.prime();
    cur.prime_commit(pr.rows);
    cur.start(lut);
    uint32_t rows[S];
    bool pending = cur.template room<S>();
    if (pending) cur.prefetch(rows);
    const int nfull = (ns - 1) / S;          // whole segments in front of the last one
    auto whole = [&](const typename Policy::Slot (&now)[S], typename Policy::Slot (&next)[S], int i) {
        if (pending) cur.commit(rows);
        pending = cur.template room<S>();
        if (pending) cur.prefetch(rows);
        const int t1 = (i + 1) * S;
        if (i + 1 < nfull) {
            pol.load_full(next, t1);
        } else {
#pragma unroll
            for (int j = 0; j < S; ++j) pol.load(next[j], t1 + j);      // the last segment may be short: clamped
        }
        decode_segment<true, HAS_ESC>(cur, lut, pol, now, i * S, ns);
    };
    if (nfull > 0) {
        whole(a, b, 0);
        point_a();
        int i = 1;
        for (;;) {
            if (i >= nfull) break;
            whole(b, a, i);
            ++i;
            if (i >= nfull) break;
            whole(a, b, i);
            ++i;
        }
    } else {
        point_a();
    }
    point_b();
    if (nfull & 1) {
#pragma unroll
        for (int i = 0; i < S; ++i) a[i] = b[i];
    }
    if (pending) cur.commit(rows);
    decode_segment<false, HAS_ESC, S>(cur, lut, pol, a, nfull * S, ns);
}

template <class Codec, int BS, int NWB, int S>
__global__ __launch_bounds__(NWB * kLanes, (NWB * kPersistBlocksPerCU + 3) / 4)
void gemv_persist_kernel(const uint16_t* __restrict__ X, const PGroup grp) {
    using Policy = DotPolicy<BS>;
    constexpr int NSET = Policy::NSET;
    constexpr int kSums = NSET * kGroupRows * 4;          // floats a unit hands over: [set][row][batch lane]
    __shared__ uint32_t rings[NWB][kRingWords];
    __shared__ uint32_t lut[Codec::kTableWords];
    __shared__ uint32_t qhead;
    __shared__ uint32_t arrived[kOpenGroups];
    __shared__ float partial[kOpenGroups][kMaxUnitsPerGroup][kSums];

    int member = 0;
#pragma unroll
    for (int i = 1; i < kMaxMembers; ++i)
        if (i < grp.n && (int)blockIdx.x >= grp.m[i].first_block) member = i;
    const PMember& mb = grp.m[member];
    const Shape s = mb.s;
    const int lane = threadIdx.x & (kLanes - 1);
    const int wave = (int)uniform(threadIdx.x / kLanes);
    const int blk = (int)blockIdx.x - mb.first_block;
    const int G = s.M / kGroupRows;
    const int per_group = s.split_k * s.nc;
    const int upg = mb.upg, tpu = per_group / upg;
    const int g_lo = (int)((long long)G * blk / mb.nblocks), g_hi = (int)((long long)G * (blk + 1) / mb.nblocks);
    const int nunits = (g_hi - g_lo) * upg;
    const bool variant = Codec::variant(mb.header);
    const int K = s.Ks * s.split_k;

    if (threadIdx.x == 0) qhead = NWB;
    if (threadIdx.x < kOpenGroups) arrived[threadIdx.x] = 0;

    Policy pol;
#pragma unroll
    for (int q = 0; q < NSET; ++q) pol.acc[q] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 8; ++j) pol.dot[j] = 0.f;
    pol.xrow = K / 2;

    int q = wave;                                  // the first unit of every wavefront is dealt, not pulled
    if (q >= nunits) {
        load_table<Codec::kTableWords>(lut, mb.table);
        __syncthreads();
        return;
    }

    // ---- the first task starts cold: operands, then offsets -> rows, the table alongside
    TaskCtx T = make_task(mb, X, g_lo + q / upg, (q % upg) * tpu, lane);
    int kc_end = T.kc + tpu;
    Primed<Policy, S> pr;
    // the offsets entries first: loads return in order, and the row loads wait for these
    const uint32_t first_base = mb.offsets[T.obase], first_end = mb.offsets[T.oend];
    pol.rem0 = T.rem0; pol.xq0 = T.xq0; pol.last = T.ns - 1;
#pragma unroll
    for (int i = 0; i < S; ++i) pol.load(pr.slot[i], i);
    typename Codec::Cursor cur;
    {
        TaskSpan sp;
        sp.base = first_base;
        sp.end = T.end_is_total ? s.total_words : first_end;
        cur.open(mb.exp, sp, lane, rings[wave]);
        cur.prime_issue(pr.rows);
    }
    load_table<Codec::kTableWords>(lut, mb.table);
    __syncthreads();

    for (;;) {
        TaskCtx N = T;                             // the task after T (T itself when there is none: harmless reloads)
        bool have_next = false, next_new_unit = false;
        uint32_t nb_v = 0, ne_v = 0;               // its offsets entries, in flight from point A to point B
        TaskSpan nsp;
        auto point_a = [&]() {
            if (T.kc + 1 < kc_end) {
                N = make_task(mb, X, T.g, T.kc + 1, lane);
                have_next = true;
            } else {
                uint32_t v = 0;
                if (lane == 0) v = atomicAdd(&qhead, 1u);
                const int qn = (int)uniform(v);
                if (qn < nunits) {
                    N = make_task(mb, X, g_lo + qn / upg, (qn % upg) * tpu, lane);
                    have_next = true;
                    next_new_unit = true;
                }
            }
            nb_v = mb.offsets[N.obase];
            ne_v = mb.offsets[N.oend];
        };
        auto point_b = [&]() {
            nsp.base = uniform(nb_v);
            nsp.end = N.end_is_total ? s.total_words : uniform(ne_v);
            const uint32_t* bp = mb.exp + nsp.base + lane;
            const uint32_t nrows = (nsp.end - nsp.base + kLanes - 1) / kLanes;
#pragma unroll
            for (int j = 0; j < kPrimeRows; ++j) {
                const uint32_t r = (uint32_t)j < nrows ? (uint32_t)j : nrows - 1;
                pr.rows[j] = bp[(size_t)r * kLanes];
            }
            const int last = N.ns - 1;
#pragma unroll
            for (int i = 0; i < S; ++i) pol.load_at(pr.slot[i], N.rem0, N.xq0, last, i);
        };
        pol.rem0 = T.rem0; pol.xq0 = T.xq0; pol.last = T.ns - 1;
        if (variant) run_task_primed<true, S>(cur, lut, pol, T.ns, pr, point_a, point_b);
        else run_task_primed<false, S>(cur, lut, pol, T.ns, pr, point_a, point_b);

        if (T.kc + 1 >= kc_end) {
            // ---- the unit is complete: fold the lane sums and hand them over
            pol.fold();
#pragma unroll
            for (int qq = 0; qq < NSET; ++qq) {
#pragma unroll
                for (int i = 0; i < kGroupRows; ++i) {
                    pol.acc[qq][i] = sum_over_column_blocks(pol.acc[qq][i]);
                }
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) pol.dot[j] = 0.f;
            const int g = T.g;
            if (upg == 1) {
                if (lane < 4) {
#pragma unroll
                    for (int qq = 0; qq < NSET; ++qq) {
                        const int batch = lane + 4 * qq;
                        if (batch < BS) {
#pragma unroll
                            for (int i = 0; i < kGroupRows; ++i)
                                mb.Y[(size_t)batch * s.M + kGroupRows * g + i] = finish_output(pol.acc[qq][i], mb.bias, kGroupRows * g + i);
                        }
                    }
                }
            } else {
                // Partners of a row group are pulled back to back from this block's queue, so
                // at most a few groups are open at once; a slot is reused kOpenGroups groups
                // later.  Should a partner of that older group still be decoding (it would
                // have to be kOpenGroups * upg units behind), wait for it: it does not wait
                // for anybody.
                const int slot = (g - g_lo) % kOpenGroups;
                const int j = (T.kc + 1 - tpu) / tpu;                 // which unit of the group this was
                const uint32_t round = (uint32_t)((g - g_lo) / kOpenGroups);
                while ((uniform(__hip_atomic_load(&arrived[slot], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) >> 8) != (round & 0xFFFFFFu))
                    __builtin_amdgcn_s_sleep(8);
                if (lane < 4) {
#pragma unroll
                    for (int qq = 0; qq < NSET; ++qq)
#pragma unroll
                        for (int i = 0; i < kGroupRows; ++i) partial[slot][j][(qq * kGroupRows + i) * 4 + lane] = pol.acc[qq][i];
                }
                uint32_t old = 0;
                if (lane == 0) old = __hip_atomic_fetch_add(&arrived[slot], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
                old = uniform(old);
                if ((int)(old & 0xFFu) == upg - 1) {
                    if (lane < 4) {
#pragma unroll
                        for (int qq = 0; qq < NSET; ++qq) {
                            const int batch = lane + 4 * qq;
                            if (batch < BS) {
#pragma unroll
                                for (int i = 0; i < kGroupRows; ++i) {
                                    float a = 0.f;
                                    for (int w = 0; w < upg; ++w) a += partial[slot][w][(qq * kGroupRows + i) * 4 + lane];
                                    mb.Y[(size_t)batch * s.M + kGroupRows * g + i] = finish_output(a, mb.bias, kGroupRows * g + i);
                                }
                            }
                        }
                    }
                    // the slot now belongs to the group kOpenGroups further on
                    if (lane == 0) __hip_atomic_store(&arrived[slot], ((round + 1) & 0xFFFFFFu) << 8, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            }
        }
        if (!have_next) break;
        T = N;
        if (next_new_unit) kc_end = T.kc + tpu;
        cur.open(mb.exp, nsp, lane, rings[wave]);
    }
}

// Which launches take the persistent kernel, and how a member's row groups are cut into
// units.  Returns 0 when the static grid should run instead.
static inline int persist_units_per_group(const Shape& s, long long waves) {
    const int per_group = s.split_k * s.nc;
    const long long G = s.M / kGroupRows;
    int upg = 1;
    // finer units while there are fewer than two per wavefront, as far as the streams allow
    while (upg * 2 <= per_group && per_group % (upg * 2) == 0 && upg * 2 <= kMaxUnitsPerGroup && G * upg < 2 * waves) upg *= 2;
    return upg;
}

}  // namespace bhi

#include <stdlib.h>

// 0: static grid only, 1: persistent grid where it applies (default), 2: persistent wherever it can run
static inline int persist_mode() {
    static const int mode = [] {
        const char* e = getenv("BHI_PERSIST");
        return e ? atoi(e) : BHI_PERSIST_DEFAULT;
    }();
    return mode;
}

template <class Codec, int BS>
static inline void launch_persist(const void* X, const bhi::PGroup& pg, int blocks, hipStream_t stream) {
    using namespace bhi;
    hipLaunchKernelGGL((gemv_persist_kernel<Codec, BS, kPersistWaves, kPersistSeg>), dim3((unsigned)blocks),
                       dim3(kPersistWaves * kLanes), 0, stream, (const uint16_t*)X, pg);
}

// Turns a group of the static-grid launcher into a persistent launch when that pays:
// returns false (nothing launched) when the static grid should run.
template <class Codec>
static inline bool try_launch_persist(int batch, const void* X, const bhi::Group& grp, hipStream_t stream) {
    using namespace bhi;
    const int mode = persist_mode();
    if (mode == 0 || batch > 1) return false;      // batch 2..4 would need more than the 80 registers six wavefronts allow
    const int max_blocks = kComputeUnits * kPersistBlocksPerCU;
    // work of a member in steps; blocks are dealt in proportion
    double work[kMaxMembers], total = 0;
    long long units_min = 0;
    for (int i = 0; i < grp.n; ++i) {
        const Shape& s = grp.m[i].s;
        work[i] = (double)(s.M / kGroupRows) * s.split_k * s.steps;
        total += work[i];
        units_min += (long long)(s.M / kGroupRows) * s.split_k * s.nc;
    }
    // everything resident at once and nothing to pull: the static grid is as good
    if (mode == 1 && units_min <= (long long)max_blocks * kPersistWaves) return false;
    PGroup pg = {};
    pg.n = grp.n;
    int first = 0;
    for (int i = 0; i < grp.n; ++i) {
        const Member& m = grp.m[i];
        const Shape& s = m.s;
        const int G = s.M / kGroupRows;
        int nb = (int)(max_blocks * work[i] / total + 0.5);
        if (nb < 1) nb = 1;
        const int per_group = s.split_k * s.nc;
        // never more blocks than there are units for their wavefronts
        const long long most_units = (long long)G * (per_group < kMaxUnitsPerGroup ? per_group : kMaxUnitsPerGroup);
        const long long need = (most_units + kPersistWaves - 1) / kPersistWaves;
        if (nb > need) nb = (int)need;
        if (nb > G) nb = G;
        PMember& p = pg.m[i];
        p.rem = m.rem; p.exp = m.exp; p.Y = m.Y; p.offsets = m.offsets; p.table = m.table; p.header = m.header;
        p.bias = m.bias; p.s = s; p.first_block = first; p.nblocks = nb;
        p.upg = persist_units_per_group(s, (long long)nb * kPersistWaves);
        first += nb;
    }
    launch_persist<Codec, 1>(X, pg, first, stream);
    return true;
}
