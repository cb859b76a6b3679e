// Fused decode + matrix product for up to 32 rows of X (the path for 9..32 rows, and from 3 rows on
// large layers): the weights go from the decoder's
// registers straight into matrix-core instructions, the compressed bytes are read once
// and no BF16 weight ever reaches HBM.
//
// Stands in for the reference's path above eight rows, `get_weight()` followed by
// `F.linear` (bf16_huffman_infer/functional.py:405-407, 460-462; decode kernel
// src/kernel.cu:222-310), which writes the whole BF16 matrix and reads it back through a
// library GEMM.
//
// Shape of the work.  A wavefront decodes the tasks of ONE row group (4 weight rows), as in
// the GEMV; lane 4b+i holds row i, columns 8b..8b+7 of a step: exactly the A operand of the
// sixteen 4x4x4 blocks of v_mfma_f32_4x4x4_16b_bf16 (block b = lanes 4b..4b+3, two
// instructions per step for the two halves of the 8 columns).  The B operand of block b is
// X[batch 4q+j][the same 4 columns] in lane 4b+j; lane 4b+j then accumulates, for batch
// quad q, the sums of rows 0..3 for batch 4q+j over column block b (4 registers per quad).
//
// X does not come from global memory per wavefront (at 32 rows that would be 8 KB per
// wavefront and step against 0.7 KB of weights): the block's wavefronts (8, 12 or 16 of them)
// walk the same columns in lockstep, one window of four steps at a time, and the window's
// slice of X is staged in LDS once per block in the exact order the lanes read it (conflict
// free, 16 bytes per lane and instruction), double buffered, one barrier per window (a barrier
// that orders LDS only: the global loads of the next window stay in flight across it).
//
// Measured on MI355X, Student-t weights, rotating over 640 MB of clones: 12288x4096 at 16 / 32
// rows 25.0 / 32.2 us against 56 us for decode-to-BF16 + library GEMM; 4096x12288 (2 / 3 K
// slices) 32 / 45 us against 54-56 us.  Taking the X reads out (wrong results) saves 1.6 / 3.8 us,
// the barriers 2.8 / 5.7 us; requesting rem bytes, rows and X two windows ahead instead of one
// was slower (128 registers, and nothing was waiting for those loads).  A compute unit gets
// through 1.5 times the row groups with 16 resident wavefronts that it does with 8, and no more
// with 24: the lockstep makes a block as slow as its slowest wavefront in every window, so what
// counts is that the grid covers the 256 units evenly (mma_plan below).  From 3 to 8 rows the
// kernel also beats the GEMV on large layers (37888x3584 at 4 rows 39.8 against 44.4 us, at 8
// rows 45.0 against 58.7 us): one load of X per block instead of one per wavefront, two matrix
// instructions per batch quad and step instead of four dot products per batch row.
//
// Few row groups (M < 8192) would leave most of the GPU idle, so the tasks of a row group
// can be dealt to up to 8 blocks (K slices).  Their partial sums meet in a workspace in
// device memory: every block stores its slice, the last one to arrive at the row block's
// counter adds the slices in order and writes Y; it leaves the counter at zero.
#pragma once
// (included by bhi_task.h users after the static-grid kernels)

namespace bhi {

typedef short short4_t __attribute__((ext_vector_type(4)));

#ifndef BHI_MMA_ARRIVAL_ORDER
#define BHI_MMA_ARRIVAL_ORDER __ATOMIC_RELAXED
#endif
#ifndef BHI_MMA_LAST_ACQUIRES
#define BHI_MMA_LAST_ACQUIRES 1
#endif
constexpr int kMmaSeg = 4;                   // steps per window
constexpr int kMmaSegShort = 2;              // at 5..8 rows also built with short windows: 8 KB less LDS, a third block per unit
// Wavefronts (row groups) per block.  LDS holds two windows of X (8 KB per batch quad, half of
// that with short windows) beside the table and the rings: up to 16 rows two 8-wavefront blocks
// fit a compute unit, and one block of 12 or of 16 at any batch.  Which one a launch takes is
// a matter of how evenly its blocks cover the 256 compute units (mma_plan below).
constexpr int kMmaWavesSmall = 8, kMmaWavesMid = 12, kMmaWavesLarge = 16;
constexpr int kMmaSmallUpToQ = 4;            // 8-wavefront blocks: batch quads 1..4
// Blocks of NW wavefronts that a compute unit holds at Q batch quads and windows of S steps:
// by LDS (rings 4.5 KB per wavefront, table up to 8 KB, X windows 2 KB per quad and step,
// 160 KB per unit) and by registers (65-73 up to two quads: six wavefronts per SIMD; 84-102 up
// to four quads: four; above: three or four)
constexpr int mma_resident_blocks(int Q, int NW, int S = kMmaSeg) {
    return Q == 1 ? (NW == kMmaWavesSmall ? 3 : (NW == kMmaWavesMid ? 2 : 1))
         : Q == 2 ? (NW == kMmaWavesLarge ? 1 : (NW == kMmaWavesSmall && S == kMmaSegShort ? 3 : 2))
         : Q <= 4 ? (NW == kMmaWavesSmall ? 2 : 1) : 1;
}
constexpr int kMmaMaxBatch = 32;
constexpr int kMmaMaxSlices = 8;
constexpr int kMmaSliceBelowGroups = 2048;   // weights with fewer row groups are cut along K

template <int Q>
struct MmaPolicy {
    struct Slot { uint2 rem; };
    struct Piped { int i; };
    const uint2* rem0;
    int last;
    const uint4* xw;          // this lane's 16 bytes of (step 0, quad 0) in the current window
    f32x4_t acc[Q];

    __device__ __forceinline__ void load(Slot& s, int t) const {
        t = t < last ? t : last;
        s.rem = stream_load(rem0 + (size_t)t * kLanes);
    }
    __device__ __forceinline__ Piped take(const Slot&, int i, int) const { return Piped{i}; }
    __device__ __forceinline__ void use(const Piped& p, int, const uint32_t (&w)[4]) {
        const uint2 a0 = make_uint2(w[0], w[1]), a1 = make_uint2(w[2], w[3]);
#pragma unroll
        for (int q = 0; q < Q; ++q) {
            const uint4 b = xw[(p.i * Q + q) * kLanes];
            acc[q] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(short4_t, a0), __builtin_bit_cast(short4_t, make_uint2(b.x, b.y)), acc[q], 0, 0, 0);
            acc[q] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(short4_t, a1), __builtin_bit_cast(short4_t, make_uint2(b.z, b.w)), acc[q], 0, 0, 0);
        }
    }
};

struct MmaArgs {
    const uint8_t* rem;
    const uint32_t* exp;
    uint16_t* Y;
    const uint32_t* offsets;
    const uint32_t* table;
    const uint8_t* header;
    const uint16_t* bias;
    const uint16_t* residual;
    Shape s;
    int batch;
    int slices;              // K slices (blocks per row block); divides split_k * nc
    float* partial;          // [slices][batch][M] when slices > 1
    uint32_t* counters;      // one per row block, zero between launches
};

// Up to four weights that multiply the same X in one grid (the gate and up projections of a
// decoder layer): member i owns the blocks from first[i] on.  Only a group of one is cut
// along K.
struct MmaGroup {
    MmaArgs m[kMaxMembers];
    int first[kMaxMembers];
};

// Workspace layout: the arrival counters first, at a fixed place for every shape (a launch
// relies on finding them at zero, so no other launch may ever have used those bytes for
// anything else), then the partial sums.
constexpr int kMmaCounterBytes = kMmaSliceBelowGroups / 8 * 4;       // sliced launches have fewer row blocks than this
__host__ __device__ inline long long mma_partial_floats(int M, int batch, int slices) {
    return slices > 1 ? (long long)slices * batch * M : 0;
}

template <class Codec, int Q, int NW, int S = kMmaSeg>
__global__ __launch_bounds__(NW * kLanes, mma_resident_blocks(Q, NW, S) * NW / 4)     // wavefronts per SIMD that the blocks of a compute unit add up to
void mma_kernel(const uint16_t* __restrict__ X, int first1, int first2, int first3, const MmaGroup grp) {
    constexpr int kWindow = S * Q * kLanes;                   // 16-byte units of one X window
    constexpr int kThreads = NW * kLanes;
    constexpr int kPieces = S * Q * 4 * 16;                   // 16-byte pieces of a window: (step, batch row, 8 columns)
    constexpr int kLoads = (kPieces + kThreads - 1) / kThreads;
    __shared__ uint32_t rings[NW][kRingWords];
    __shared__ uint32_t lut[Codec::Table::kLdsWords];
    __shared__ uint4 xbuf[2][kWindow];
    __shared__ uint32_t is_last;

    // first1..3: first block of members 1..3 (INT_MAX when absent); leading scalar arguments
    // are in registers when the wavefront starts, so the member is known without a fetch
    static_assert(kMaxMembers == 4, "one leading argument per member after the first");
    int member = 0;
    if ((int)blockIdx.x >= first1) member = 1;
    if ((int)blockIdx.x >= first2) member = 2;
    if ((int)blockIdx.x >= first3) member = 3;
    const MmaArgs& a = grp.m[member];
    const int block = (int)blockIdx.x - grp.first[member];
    const Shape s = a.s;
    const int lane = threadIdx.x & (kLanes - 1);
    const int wave = (int)uniform(threadIdx.x / kLanes);
    const int rb = block / a.slices, ks = block % a.slices;
    // a block past the last row group (M / 4 need not be a multiple of NW) repeats that group
    // without storing anything: its wavefronts still load their share of X and meet the barriers
    const int G = s.M / kGroupRows;
    const bool real = rb * NW + wave < G;
    const int g = real ? rb * NW + wave : G - 1;
    const int per_group = s.split_k * s.nc;
    const int tpk = per_group / a.slices;
    const int kc0 = ks * tpk, kc1 = kc0 + tpk;
    const int K = s.Ks * s.split_k;
    const bool variant = Codec::variant(a.header);
    const int B = a.batch;

    MmaPolicy<Q> pol;
#pragma unroll
    for (int q = 0; q < Q; ++q) pol.acc[q] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // ---- X staging: piece p of a window = (step i, batch row r = 4q + j, column group b); the
    // thread that loads it writes it where lane 4b + j will read it
    static_assert(kLoads <= 3, "three pieces per thread at most");
    uint4 xg0 = make_uint4(0, 0, 0, 0), xg1 = make_uint4(0, 0, 0, 0), xg2 = make_uint4(0, 0, 0, 0);     // (named registers: an array would live in scratch memory)
    auto piece_load = [&](uint4& dst, int n, int k, int t0, int t_end) __attribute__((always_inline)) {
        const int p = (int)threadIdx.x + n * kThreads;
        if (kPieces % kThreads == 0 || p < kPieces) {
            const int b = p & 15, r = (p >> 4) % (4 * Q), i = p / (64 * Q);
            const int rr = r < B ? r : B - 1;                     // rows past the batch: any valid row
            int t = t0 + i;
            t = t < t_end ? t : t_end - 1;                        // steps past the task: any valid step
            dst = *(const uint4*)(X + (size_t)rr * K + (size_t)k * s.Ks + (size_t)t * kStepCols + b * kLaneCols);
        }
    };
    auto piece_store = [&](const uint4& src, int n, int par) __attribute__((always_inline)) {
        const int p = (int)threadIdx.x + n * kThreads;
        if (kPieces % kThreads == 0 || p < kPieces) {
            const int b = p & 15, r = (p >> 4) % (4 * Q), i = p / (64 * Q);
            xbuf[par][(i * Q + (r >> 2)) * kLanes + 4 * b + (r & 3)] = src;
        }
    };
    auto x_load = [&](int k, int t0, int t_end) __attribute__((always_inline)) {       // window starting at step t0 of split k; the task ends at t_end
        piece_load(xg0, 0, k, t0, t_end);
        if (kLoads > 1) piece_load(xg1, 1, k, t0, t_end);
        if (kLoads > 2) piece_load(xg2, 2, k, t0, t_end);
    };
    auto x_store = [&](int par) __attribute__((always_inline)) {
        piece_store(xg0, 0, par);
        if (kLoads > 1) piece_store(xg1, 1, par);
        if (kLoads > 2) piece_store(xg2, 2, par);
    };

    typename Codec::Cursor cur;
    int par = 0;
    auto walk = [&](auto has_esc) __attribute__((always_inline)) {
        constexpr bool HAS_ESC = decltype(has_esc)::value;
        for (int kc = kc0; kc < kc1; ++kc) {
            const TaskId id = task_of(s, kc);
            const int ns = id.t1 - id.t0;
            cur.open(a.exp, task_span(a.offsets, s.M, s.split_k, s.nc, id.k, g, id.c, s.total_words), lane, rings[wave]);
            pol.rem0 = (const uint2*)(a.rem + ((size_t)id.k * s.M + (size_t)kGroupRows * g) * s.Ks) + (size_t)id.t0 * kLanes + lane;
            pol.last = ns - 1;
            typename MmaPolicy<Q>::Slot now[S], next[S];
#pragma unroll
            for (int i = 0; i < S; ++i) pol.load(now[i], i);
            uint32_t first[kPrimeRows];
            cur.prime_issue(first);
            if (kc == kc0) {
                // the table and the first window of X travel with the task's first loads
                x_load(id.k, id.t0, id.t1);
                Codec::Table::fill(lut, a.table);
                x_store(0);
                __syncthreads();
            }
            cur.prime_commit(first);
            cur.start(lut);
            uint32_t rows[S];
            bool pending = cur.template room<S>();
            if (pending) cur.prefetch(rows);
            const int nseg = (ns + S - 1) / S;
            for (int seg = 0; seg < nseg; ++seg) {
                // the window after this one: the task's next, or the next task's first
                const bool more_here = seg + 1 < nseg, more = more_here || kc + 1 < kc1;
                if (more_here) {
                    x_load(id.k, id.t0 + (seg + 1) * S, id.t1);
                } else if (more) {
                    const TaskId nx = task_of(s, kc + 1);
                    x_load(nx.k, nx.t0, nx.t1);
                }
                if (pending) cur.commit(rows);
                pending = cur.template room<S>();
                if (pending) cur.prefetch(rows);
#pragma unroll
                for (int i = 0; i < S; ++i) pol.load(next[i], (seg + 1) * S + i);
                pol.xw = &xbuf[par][lane];
                decode_segment<false, HAS_ESC, S>(cur, lut, pol, now, seg * S, ns);
                if (more) x_store(par ^ 1);
                lds_barrier();
                par ^= 1;
#pragma unroll
                for (int i = 0; i < S; ++i) now[i] = next[i];
            }
        }
    };
    if (variant) walk(std::true_type{});
    else walk(std::false_type{});

    // ---- sums over the 16 column blocks; lane j (< 4) then holds batch 4q + j, rows 0..3
#pragma unroll
    for (int q = 0; q < Q; ++q) {
#pragma unroll
        for (int i = 0; i < kGroupRows; ++i) {
            pol.acc[q][i] = sum_over_column_blocks(pol.acc[q][i]);
        }
    }
    if (a.slices == 1) {
        if (real && lane < 4) {
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                const int batch = 4 * q + lane;
                if (batch < B) {
#pragma unroll
                    for (int i = 0; i < kGroupRows; ++i)
                        a.Y[(size_t)batch * s.M + kGroupRows * g + i] = finish_output(pol.acc[q][i], a.bias, kGroupRows * g + i,
                                                                                      a.residual ? a.residual + (size_t)batch * s.M : nullptr);
                }
            }
        }
        return;
    }
    // ---- K slices: this block's sums go to the workspace with agent-scope stores: they are
    // written through the L2 of this die (which the other dies do not see) to the memory side
    // all dies share, and `s_waitcnt vmcnt(0)` returns once they have been acknowledged there.
    // Then the block arrives at its row block's counter.  The last block to arrive executes ONE
    // agent-scope acquire (thread 0; the barrier behind it carries the order to the other
    // threads) before it reads the other blocks' sums.  The arrival itself is a relaxed atomic:
    // a release there makes every arriving block write back its die's whole L2, which holds
    // nothing of this kernel that is not written through already, and costs 2.5-2.9 us of a
    // 17-32 us launch (measured: 4096x12288 at 16 rows 31.9 -> 34.5 us, 4096x4096 16.7 -> 19.4 us;
    // the acquire in the last block: +0.1-0.4 us).  A cache-wide fence per WAVEFRONT, 6144 of
    // them, made the launch take 270 us.  What this relies on beyond the language's memory model:
    // an acknowledged agent-scope store is visible to agent-scope loads of every die.
    if (real && lane < 4) {
#pragma unroll
        for (int q = 0; q < Q; ++q) {
            const int batch = 4 * q + lane;
            if (batch < B) {
                float* dst = a.partial + ((size_t)ks * B + batch) * s.M + kGroupRows * g;
#pragma unroll
                for (int i = 0; i < kGroupRows; ++i)
                    __hip_atomic_store(dst + i, pol.acc[q][i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0): the stores above have completed
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t old = __hip_atomic_fetch_add(a.counters + rb, 1u, BHI_MMA_ARRIVAL_ORDER, __HIP_MEMORY_SCOPE_AGENT);
        is_last = old == (uint32_t)a.slices - 1;
        if (BHI_MMA_LAST_ACQUIRES && is_last) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    }
    __syncthreads();
    if (!is_last) return;
    // the last block to arrive adds the slices in order (device-scope loads: from memory, not
    // from a stale line of this die's L2)
    const int rows_here = kGroupRows * NW;
    for (int e = threadIdx.x; e < B * rows_here; e += kThreads) {
        const int batch = e / rows_here, row = rb * rows_here + e % rows_here;
        if (row >= s.M) continue;
        float v = 0.f;
        for (int k = 0; k < a.slices; ++k)
            v += __hip_atomic_load(a.partial + ((size_t)k * B + batch) * s.M + row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        a.Y[(size_t)batch * s.M + row] = finish_output(v, a.bias, row, a.residual ? a.residual + (size_t)batch * s.M : nullptr);
    }
    if (threadIdx.x == 0) __hip_atomic_store(a.counters + rb, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace bhi

// Shape of a launch: wavefronts per block and K slices, by a small cost model in units of steps.
//
// A block of NW wavefronts covers NW row groups and walks (tasks per group / d) tasks when the
// row group's tasks are dealt to d blocks (K slices, d a divisor); it pays about six steps'
// worth of start, and every slice adds a round trip of partial sums (two steps' worth).  The
// pace of a block depends on how many wavefronts share its compute unit: measured on
// 4096-column weights at 16 rows, a unit with 8 / 12 / 16 resident wavefronts gets through
// 1 / 1.26 / 1.51 row groups in the time a lone 8-wavefront block needs for one (8192 rows,
// 256 blocks: 21.1 us; 12288 rows as 256 blocks of 12: 25.0 us; 16384 rows, 512 blocks of 8:
// 27.9 us), and 24 do no better than 16 (18944x3584 at 8 rows).  What the model is there to
// avoid is a grid that covers the 256 units unevenly: 12288 rows as 384 blocks of 8 put two
// blocks on half of the units and one on the rest and take as long as 16384 rows (27.7 us; at
// 32 rows 192 blocks of 16 leave a quarter of the units idle: 37.2 us against 32.2 us for 256
// blocks of 12).  Blocks beyond what is resident at once wait for a round; the last round runs
// at the pace of the wavefronts it puts on a unit (18944x3584 at 16 rows, 592 blocks of 8:
// 38.1 us, 395 blocks of 12: 39.5 us; at 8 rows, where two blocks of 12 fit a unit: 31.0 and
// 26.3 us).  At 5..8 rows the 8-wavefront block also comes with windows of two steps: a third
// block fits the unit and every step costs about 3 % more (37888x3584: 49.0 -> 45.1 us;
// 3584x18944, whose 448 blocks have room anyway: 28.8 -> 30.9 us).
// The 8-wavefront block (16 above 16 rows) stays unless another shape is at least
// 4 % cheaper, and so does a smaller number of slices: the model is no more exact than that.
// It reproduces the order measured at 16 / 32 rows for the slices as well: 4096x12288
// (6 tasks of 16 steps) 2 slices 32 us, 3 slices 33 us, 6 slices 41 us, none 50 us / 3 slices
// 44 us, 2 slices 55 us, 6 slices 59 us; 3584x18944 (4 tasks of 37 steps) 4 slices 36 us,
// 2 slices 42 us; 4096x4096 (4 tasks of 8 steps) 2 slices 17 us, 4 slices 20 us.
struct MmaPlan { int nw, slices, seg; };

// time of a row group on a unit that holds `waves` wavefronts, relative to a lone block of 8
static inline double mma_pace(int waves) {
    const double through = waves <= 8 ? 1.0 : (waves <= 12 ? 1.26 : 1.51);
    return waves / 8.0 / through;
}

static inline MmaPlan mma_plan(const bhi::Shape& s, int Q) {
    using namespace bhi;
    const int G = s.M / kGroupRows, per_group = s.split_k * s.nc;
    const double task_steps = (double)s.steps / s.nc;
    const int max_slices = G >= kMmaSliceBelowGroups ? 1 : kMmaMaxSlices;
    MmaPlan best = {0, 1, kMmaSeg};
    double best_cost = 0;
    const bool small = Q <= kMmaSmallUpToQ;
    struct Candidate { int nw, seg; };
    const Candidate candidates[4] = {{small ? kMmaWavesSmall : kMmaWavesLarge, kMmaSeg}, {kMmaWavesMid, kMmaSeg},
                                     {small ? kMmaWavesLarge : 0, kMmaSeg}, {Q == 2 ? kMmaWavesSmall : 0, kMmaSegShort}};
    for (const Candidate& c : candidates) {
        const int nw = c.nw;
        if (nw == 0) continue;
        const long long row_blocks = (G + nw - 1) / nw;
        const int resident = mma_resident_blocks(Q, nw, c.seg);
        const double step_cost = c.seg == kMmaSeg ? 1.0 : 1.03;
        MmaPlan here = {nw, 1, c.seg};
        double here_cost = 0;
        for (int d = 1; d <= max_slices && d <= per_group; ++d) {
            if (per_group % d != 0) continue;
            const long long blocks = row_blocks * d;
            const long long rest = blocks % (256 * resident);
            double pace = mma_pace(nw * resident) * (double)(blocks / (256 * resident));
            if (rest > 0) pace += mma_pace(nw * (int)((rest + 255) / 256));
            const double cost = step_cost * pace * (per_group / d * task_steps + 6.0) + 2.0 * d;
            if (d == 1 || cost < 0.96 * here_cost) { here = MmaPlan{nw, d, c.seg}; here_cost = cost; }
        }
        if (best.nw == 0 || here_cost < 0.96 * best_cost) { best = here; best_cost = here_cost; }
    }
    return best;
}

static inline int64_t mma_workspace_bytes(const bhi::Shape& s, int batch) {
    using namespace bhi;
    const int slices = mma_plan(s, (batch + 3) / 4).slices;
    return slices > 1 ? kMmaCounterBytes + mma_partial_floats(s.M, batch, slices) * 4 : 0;
}

template <class Codec, int Q, int NW, int S = bhi::kMmaSeg>
static inline void launch_mma_qn(bhi::MmaGroup& grp, int n, const uint16_t* x, hipStream_t stream) {
    using namespace bhi;
    long long blocks = 0;
    for (int i = 0; i < kMaxMembers; ++i) {
        grp.first[i] = i < n ? (int)blocks : 0x7FFFFFFF;
        if (i < n) blocks += (long long)((grp.m[i].s.M / kGroupRows + NW - 1) / NW) * grp.m[i].slices;
    }
    const dim3 grid((unsigned)blocks), block(NW * kLanes);
    hipLaunchKernelGGL((mma_kernel<Codec, Q, NW, S>), grid, block, 0, stream, x, grp.first[1], grp.first[2], grp.first[3], grp);
}

template <class Codec, int Q>
static inline void launch_mma_q(bhi::MmaGroup& grp, int n, const MmaPlan& plan, const uint16_t* x, hipStream_t stream) {
    using namespace bhi;
    const int nw = plan.nw;
    if constexpr (Q == 2) {
        if (plan.seg == kMmaSegShort) return launch_mma_qn<Codec, Q, kMmaWavesSmall, kMmaSegShort>(grp, n, x, stream);
    }
    if constexpr (Q <= kMmaSmallUpToQ) {
        if (nw == kMmaWavesSmall) return launch_mma_qn<Codec, Q, kMmaWavesSmall>(grp, n, x, stream);
    }
    if (nw == kMmaWavesMid) return launch_mma_qn<Codec, Q, kMmaWavesMid>(grp, n, x, stream);
    launch_mma_qn<Codec, Q, kMmaWavesLarge>(grp, n, x, stream);
}

// The plan of a group is the plan of one weight with all the members' rows.
static inline bhi::Shape mma_group_shape(const bhi::Shape& first, long long rows) {
    bhi::Shape s = first;
    s.M = (int)rows;
    return s;
}

template <class Codec>
static inline int launch_mma(const bhi_gemv_member* members, int n_members, const void* X, int split_k, int Ks, int batch,
                             void* workspace, int64_t workspace_bytes, int64_t table_bytes_expected, bool header_is_table,
                             hipStream_t stream) {
    using namespace bhi;
    if (!members || !X) return bhi_fail(BHI_EINVAL, "null pointer");
    if (n_members < 1 || n_members > kMaxMembers) return bhi_fail(BHI_EINVAL, "a group has 1 to 4 members");
    if (batch < 1 || batch > kMmaMaxBatch) return bhi_fail(BHI_EBATCH, "the fused matrix product takes 1 to 32 rows of X");
    MmaGroup grp = {};
    long long rows = 0;
    for (int i = 0; i < n_members; ++i) {
        const bhi_gemv_member& m = members[i];
        if (!m.A_rem || !m.A_exp || !m.Y || !m.offsets || !m.table || (!header_is_table && !m.header))
            return bhi_fail(BHI_EINVAL, "null pointer in a group member");
        if (table_bytes_expected > 0 && m.table_bytes != table_bytes_expected)
            return bhi_fail(BHI_ELAYOUT, "decode table has the wrong size");
        MmaArgs& a = grp.m[i];
        if (int rc = check_shape(split_k, m.M, Ks, m.exp_words, &a.s)) return rc;
        a.rem = (const uint8_t*)m.A_rem; a.exp = (const uint32_t*)m.A_exp; a.Y = (uint16_t*)m.Y;
        a.offsets = (const uint32_t*)m.offsets; a.table = (const uint32_t*)m.table;
        a.header = (const uint8_t*)(header_is_table ? m.table : m.header); a.bias = (const uint16_t*)m.bias;
        a.residual = (const uint16_t*)m.residual;
        a.batch = batch; a.slices = 1;
        a.counters = nullptr; a.partial = nullptr;
        rows += m.M;
    }
    if (rows > 0x7FFFFFFFll) return bhi_fail(BHI_EINVAL, "group too large for one launch");
    const int Q = (batch + 3) / 4;
    const Shape whole = mma_group_shape(grp.m[0].s, rows);
    const MmaPlan plan = mma_plan(whole, Q);
    if (plan.slices > 1) {
        if (n_members > 1)
            return bhi_fail(BHI_EINVAL, "a group this small would be cut along K: launch its members one by one");
        const int64_t need = mma_workspace_bytes(whole, batch);
        if (!workspace || workspace_bytes < need) return bhi_fail(BHI_EINVAL, "workspace too small: see bhi_gemm_workspace_bytes");
        grp.m[0].slices = plan.slices;
        grp.m[0].counters = (uint32_t*)workspace;
        grp.m[0].partial = (float*)((char*)workspace + kMmaCounterBytes);
    }
    const uint16_t* x = (const uint16_t*)X;
    switch (Q) {
        case 1: launch_mma_q<Codec, 1>(grp, n_members, plan, x, stream); break;
        case 2: launch_mma_q<Codec, 2>(grp, n_members, plan, x, stream); break;
        case 3: launch_mma_q<Codec, 3>(grp, n_members, plan, x, stream); break;
        case 4: launch_mma_q<Codec, 4>(grp, n_members, plan, x, stream); break;
        case 5: launch_mma_q<Codec, 5>(grp, n_members, plan, x, stream); break;
        case 6: launch_mma_q<Codec, 6>(grp, n_members, plan, x, stream); break;
        case 7: launch_mma_q<Codec, 7>(grp, n_members, plan, x, stream); break;
        default: launch_mma_q<Codec, 8>(grp, n_members, plan, x, stream); break;
    }
    return 0;
}
