// Many independent reduces of one dtype and operation in ONE launch: job j computes
// dst_j[i] = src_j0[i] OP src_j1[i] OP ... for i < count_j, every job with the same number n of inputs.  This is the
// shape of the reference's read_reduce_write (N pair-reduces per launch,
// src/coll/algorithms/reduce_scatter/sycl/reduce_scatter_large_sycl_impl.hpp:22-66), of reduce_read_write_kernel_{1..7}
// (src/kernels/kernels.cl:156-177) and, with n = 1, of copy_data (N copies per launch); it is also what makes many small
// messages cost one launch instead of one launch each.
//
// The job table (pointers, counts, first-vector offsets) travels in the kernel arguments, so nothing is allocated
// and nothing is read from memory before the payload.  Work is cut into tiles of kBlock x kBatchUnroll vectors of
// one job; a block finds its job by a binary search over the running tile counts (scalar work on kernel arguments).
// Arithmetic, chain order, head and tail elements follow reduce_multi_kernel.
#pragma once

#include "reduce_kernels.hpp"

namespace mi {

constexpr int kBatchMaxJobs = 96;       // jobs per launch
constexpr int kBatchMaxPtrs = 320;      // pointers per launch: jobs x (n + 1); 64 jobs of four inputs fit
constexpr int kBatchUnroll = 4;         // vectors per lane and tile: 16 KiB of every buffer per tile

struct BatchTable {                     // by-value kernel argument (3.8 KB of the 4 KB there are)
    const void* p[kBatchMaxPtrs];       // job j: inputs p[j * (n + 1) + 0 .. n - 1], output p[j * (n + 1) + n]
    uint64_t count[kBatchMaxJobs];      // elements
    uint32_t tile_end[kBatchMaxJobs];   // tiles of jobs 0..j together
    uint8_t head[kBatchMaxJobs];        // elements before job j's first vector (bits 0-6); bit 7: the job's last whole
                                        // vector is left to the edge lanes, so that vector nvec may be read (load_vectors)
};
static_assert(sizeof(BatchTable) + 64 <= 4096, "the job table and the other arguments must fit the kernel-argument segment");

struct BatchLaunchArgs {
    const void* const* srcs;            // host array, n_jobs x n device pointers, job after job
    void* const* dsts;                  // host array, n_jobs device pointers
    const size_t* counts;               // host array, n_jobs element counts
    int n, n_jobs, op;
    hipStream_t stream;
    Tuning tune;
    size_t skip_from_count = 0;         // > 0: jobs of this many elements or more are left out (the caller has launched them)
};

template <class TR, int OP>
__global__ void __launch_bounds__(kBlock)
reduce_batch_kernel(BatchTable tb, int n, int n_jobs, uint32_t total_tiles) {
    typedef typename TR::elem_t E;
    kernel_prologue<TR, OP>();
    constexpr uint64_t kTile = (uint64_t)kBlock * kBatchUnroll;
    for (uint32_t it = blockIdx.x; it < total_tiles; it += gridDim.x) {
        int lo = 0, hi = n_jobs - 1;                    // first job whose tiles end beyond `it`
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (tb.tile_end[mid] > it) hi = mid;
            else lo = mid + 1;
        }
        const int j = lo;
        const uint32_t t = it - (j ? tb.tile_end[j - 1] : 0u);
        const uint32_t head = tb.head[j] & 0x7fu, beyond = tb.head[j] >> 7;
        const uint64_t count = tb.count[j];
        const uint64_t nvec = (count - head) / TR::VEC - beyond;
        const uint64_t nload = nvec + beyond;
        const uint32_t tail = (uint32_t)(count - head - nvec * TR::VEC);
        const int b = j * (n + 1);                      // the job's pointers: tb.p[b .. b + n]
        unsigned char* dst = (unsigned char*)tb.p[b + n];

        uint64_t idx[kBatchUnroll];
#pragma unroll
        for (int u = 0; u < kBatchUnroll; u++) idx[u] = (uint64_t)t * kTile + threadIdx.x + (uint64_t)u * kBlock;
        if (idx[0] < nload) {
            Accs<TR> a[kBatchUnroll];
            u32x4 x[kBatchUnroll];
            load_vectors<sizeof(E), kBatchUnroll, false>((const unsigned char*)tb.p[b] + head * sizeof(E), idx, nvec, nload, x);
#pragma unroll
            for (int u = 0; u < kBatchUnroll; u++) a[u] = vec_init<TR>(x[u]);
            for (int k = 1; k < n; k++) {
                load_vectors<sizeof(E), kBatchUnroll, false>((const unsigned char*)tb.p[b + k] + head * sizeof(E), idx, nvec, nload, x);
#pragma unroll
                for (int u = 0; u < kBatchUnroll; u++) vec_step<TR, OP>(x[u], a[u]);
            }
            u32x4_u* d = (u32x4_u*)(dst + head * sizeof(E));
#pragma unroll
            for (int u = 0; u < kBatchUnroll; u++)
                if (idx[u] < nvec) st_loose(d + idx[u], vec_finish<TR>(a[u]));
        }
        // the job's elements before its first and after its last vector: lanes of its first tile
        if (t == 0 && threadIdx.x < head + tail) {
            const uint32_t e = threadIdx.x;
            const uint64_t i = (e < head) ? e : (uint64_t)head + nvec * TR::VEC + (e - head);
            typename TR::acc_t r = TR::init(ld_elem<E>(tb.p[b], i));
            for (int k = 1; k < n; k++) r = TR::template step<OP>(ld_elem<E>(tb.p[b + k], i), r);
            st_elem<E>(dst, i, TR::finish(r));
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// The phased form of the same, for batches that move enough to fill whole phases (the chunks a large reduce-scatter
// stages: N pair- or N-input reduces of a few MiB to tens of MiB each).  The jobs' vectors are laid end to end in tiles
// of kBatchPhaseTile vectors (32 KiB of every buffer of ONE job: four vectors per lane of a block, the group that
// reduce_multi_phased_kernel keeps in flight per input; a job's last tile is padded), and the tiles are dealt out as
// that kernel deals out its groups: group q of block b in a phase is tile (phase x 11 + q) x grid + b, so that at every
// step the chip reads `grid` consecutive tiles.  Which job a tile belongs to, and where in it the tile starts, is
// worked out by lane q of every wave for the block's q-th tile of a phase (batch_describe), ahead of the phase.
// Staging (registers and LDS), barrier, early arrival and arithmetic are those of
// reduce_multi_phased_kernel; the jobs' edge elements are computed between the report of the first write phase and
// the wait that follows it, job j by block j mod grid.
constexpr int kBatchPhaseG = 4;
constexpr uint64_t kBatchPhaseTile = (uint64_t)kBatchPhaseG * kPhaseBlock;

struct BatchSlot {                  // where one tile lives; the same for every lane of the block
    bool valid;                     // false: the phase has no such tile (nvec = nload = 0: nothing is read or stored)
    uint32_t job;                   // index into the table
    uint32_t p0;                    // index of the job's first pointer in BatchTable::p
    uint32_t head;                  // elements before the job's first vector
    uint64_t first;                 // the tile's first vector, counted within the job
    uint64_t nvec, nload;           // the job's vectors that are computed / that may be read
};

// What lane q of a wave knows about this block's q-th tile of the phase (batch_describe); the tile's owner-independent
// facts are then handed to all lanes with v_readlane (batch_slot), so that the walk job table -> job -> first vector
// happens once per phase and tile, beside the payload's loads instead of in front of them, and the write phase needs
// no second walk.  (Walked per tile, by scalar code in front of the tile's first load, the same table cost the types
// with more arithmetic per vector 5-8 % with four inputs per job and everything 6-17 % with two.)
struct BatchDesc {
    uint32_t job;       // index into the table; ~0u: the phase has no such tile
    uint32_t headb;     // BatchTable::head of the job
    uint64_t first;     // the tile's first vector, counted within the job
    uint64_t nvec;      // the job's vectors that are computed
};

// `kt`: the job table where the kernel's arguments live in memory (a lane-indexed read of a by-value argument would
// otherwise make the compiler copy the table to scratch memory).
template <class TR>
__device__ __forceinline__ BatchDesc batch_describe(const BatchTable* kt, int n_jobs, uint64_t tile, uint32_t total_tiles) {
    BatchDesc d = { ~0u, 0u, 0u, 0u };
    if (tile < total_tiles) {
        int lo = 0, hi = n_jobs - 1;                // first job whose tiles end beyond `tile`
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (kt->tile_end[mid] > tile) hi = mid;
            else lo = mid + 1;
        }
        const uint32_t beg = lo ? kt->tile_end[lo - 1] : 0u;
        d.job = (uint32_t)lo;
        d.headb = kt->head[lo];
        d.first = (tile - beg) * kBatchPhaseTile;
        d.nvec = (kt->count[lo] - (d.headb & 0x7fu)) / TR::VEC - (d.headb >> 7);
    }
    return d;
}
__device__ __forceinline__ uint64_t readlane64(uint64_t v, int lane) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, lane);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), lane);
    return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ BatchSlot batch_slot(const BatchDesc& d, int q, int n) {
    BatchSlot s;
    const uint32_t job = (uint32_t)__builtin_amdgcn_readlane((int)d.job, q);
    const uint32_t headb = (uint32_t)__builtin_amdgcn_readlane((int)d.headb, q);
    s.valid = job != ~0u;
    s.job = s.valid ? job : 0u;
    s.p0 = s.job * (uint32_t)(n + 1);
    s.head = headb & 0x7fu;
    s.first = readlane64(d.first, q);
    s.nvec = readlane64(d.nvec, q);
    s.nload = s.nvec + (headb >> 7);
    return s;
}

// Vector g of this lane within a tile: the four lie a quarter of the tile apart, or -- wave_runs, for buffers off the
// 128-byte lines -- 64 vectors apart, so that a wave covers 4 KiB in one run (see reduce_multi_phased_kernel).
__device__ __forceinline__ uint32_t batch_tile_vector(int g, uint32_t wave_runs) {
    return wave_runs ? (threadIdx.x & ~63u) * kBatchPhaseG + (uint32_t)g * 64u + (threadIdx.x & 63u)
                     : (uint32_t)g * kPhaseBlock + threadIdx.x;
}

template <class TR, int OP>
__device__ __forceinline__ void reduce_batch_tile(const BatchTable& tb, int n, const BatchSlot& s, uint32_t wave_runs,
                                                  u32x4 (&out)[kBatchPhaseG], PhaseSync* arrive_ps = nullptr, int arrive_k = 0) {
    typedef typename TR::elem_t E;
    constexpr int G = kBatchPhaseG;
    Accs<TR> a[G];
    u32x4 x[G];
    uint64_t idx[G];
#pragma unroll
    for (int g = 0; g < G; g++) idx[g] = s.first + batch_tile_vector(g, wave_runs);
    load_vectors<sizeof(E), G, false>((const unsigned char*)tb.p[s.p0] + s.head * sizeof(E), idx, s.nvec, s.nload, x);
#pragma unroll
    for (int g = 0; g < G; g++) a[g] = vec_init<TR>(x[g]);
    for (int k = 1; k < n; k++) {
        if (k == arrive_k && threadIdx.x == 0) phase_arrive(arrive_ps);     // arrive_k == 0: never
        load_vectors<sizeof(E), G, false>((const unsigned char*)tb.p[s.p0 + k] + s.head * sizeof(E), idx, s.nvec, s.nload, x);
#pragma unroll
        for (int g = 0; g < G; g++) vec_step<TR, OP>(x[g], a[g]);
    }
#pragma unroll
    for (int g = 0; g < G; g++) out[g] = vec_finish<TR>(a[g]);
}

// A job's elements before its first and after its last vector, one per lane (at most 127 + 2 * VEC - 1 of them).
template <class TR, int OP>
__device__ __forceinline__ void reduce_batch_edges(const BatchTable& tb, int n, int j) {
    typedef typename TR::elem_t E;
    const uint64_t count = tb.count[j];
    if (count == 0) return;
    const uint32_t head = tb.head[j] & 0x7fu, beyond = tb.head[j] >> 7;
    const uint64_t nvec = (count - head) / TR::VEC - beyond;
    const uint32_t tail = (uint32_t)(count - head - nvec * TR::VEC);
    if (threadIdx.x < head + tail) {
        const uint32_t p0 = (uint32_t)(j * (n + 1));
        const uint32_t e = threadIdx.x;
        const uint64_t i = (e < head) ? e : (uint64_t)head + nvec * TR::VEC + (e - head);
        const typename TR::acc_t r = fold_element<TR, OP>(tb.p + p0, 1, n, i, TR::init(ld_elem<E>(tb.p[p0], i)));
        st_elem<E>((void*)tb.p[p0 + n], i, TR::finish(r));
    }
}

template <class TR, int OP>
__global__ void __launch_bounds__(kPhaseBlock)
reduce_batch_phased_kernel(BatchTable tb, int n, int n_jobs, uint32_t total_tiles, PhaseSync* ps, int early_loads,
                           int early_stores, long spin_ticks, uint32_t wave_runs, uint32_t write_pace16) {
    typedef typename TR::elem_t E;
    kernel_prologue<TR, OP>();
    constexpr int G = kBatchPhaseG;
    constexpr int RG = MultiPhaseRegs<TR>::groups;
    constexpr int LG = kPhaseU / G;
    static_assert(kPhaseU % G == 0, "LDS steps must be a multiple of the group size");
    __shared__ u32x4 stage[kPhaseU * kPhaseBlock];
    const uint64_t grid = gridDim.x;
    const uint64_t per_phase = grid * (uint64_t)(RG + LG);  // tiles
    static_assert(RG + LG <= 64, "one tile description per lane of a wave");
    // the job table is the kernel's first argument: it starts the kernel-argument segment
    const BatchTable* kt = (const BatchTable*)__builtin_amdgcn_kernarg_segment_ptr();
    bool give_up = false;
    unsigned gen = 0;
    if (threadIdx.x == 0) gen = phase_generation(ps);
    // lane q of every wave describes this block's tile of group q of a phase: tile t0 + q * grid + blockIdx.x.  The
    // first phase's tiles are described here, every later phase's while the block waits at the barrier in the middle of
    // the phase before (the walk is a chain of dependent loads, about a microsecond).
    const uint32_t lane = threadIdx.x & 63u;
    auto describe = [&](uint64_t t0) {
        return batch_describe<TR>(kt, n_jobs, lane < (uint32_t)(RG + LG) ? t0 + (uint64_t)lane * grid + blockIdx.x : (uint64_t)total_tiles,
                                  total_tiles);
    };
    BatchDesc desc = describe(0);
    for (uint64_t t0 = 0; t0 < total_tiles; t0 += per_phase) {
        u32x4 rs[G * (RG > 0 ? RG : 1)];
#pragma unroll
        for (int q = 0; q < RG; q++) {
            const BatchSlot s = batch_slot(desc, q, n);
            if (s.valid) {
                u32x4 v[G];
                reduce_batch_tile<TR, OP>(tb, n, s, wave_runs, v);
#pragma unroll
                for (int g = 0; g < G; g++) rs[q * G + g] = v[g];
            }
        }
        bool arrived = false;
        for (int q = 0; q < LG; q++) {
            const BatchSlot s = batch_slot(desc, RG + q, n);
            if (!s.valid) break;                            // tiles ascend with q: nothing further in this phase
            const int rem = (LG - q) * n * G;               // loads per lane still to issue in this phase
            int arrive_k = 0;
            if (!arrived) {
                const int k = rem > early_loads ? (rem - early_loads + G - 1) / G : 0;
                if (k == 0 && threadIdx.x == 0) phase_arrive(ps);
                arrive_k = k < n ? k : 0;
                arrived = k < n;
            }
            u32x4 v[G];
            reduce_batch_tile<TR, OP>(tb, n, s, wave_runs, v, ps, arrive_k);
#pragma unroll
            for (int g = 0; g < G; g++) stage[(q * G + g) * kPhaseBlock + threadIdx.x] = v[g];
        }
        if (early_loads == 0) __syncthreads();              // "when done" means the whole block, and its loads have landed
        if (!arrived && threadIdx.x == 0) phase_arrive(ps);
        const BatchDesc next = describe(t0 + per_phase);
        phase_wait(ps, ++gen, give_up, spin_ticks);
        const bool more = t0 + per_phase < total_tiles;
        const int arrive_u = more ? kPhaseU - early_stores : -1;    // kPhaseU: after the last store
        uint64_t pace_next16 = write_pace16 ? (uint64_t)wall_clock64() << 4 : 0;
        auto paced = [&](bool valid) {
            if (write_pace16 && valid) {
                while (((uint64_t)wall_clock64() << 4) < pace_next16) __builtin_amdgcn_s_sleep(1);
                pace_next16 += write_pace16;
            }
        };
#pragma unroll
        for (int q = 0; q < RG; q++) {
            const BatchSlot s = batch_slot(desc, q, n);
            paced(s.valid);
            u32x4_u* d = (u32x4_u*)((unsigned char*)tb.p[s.p0 + n] + s.head * sizeof(E));
#pragma unroll
            for (int g = 0; g < G; g++) {
                const uint64_t i = s.first + batch_tile_vector(g, wave_runs);
                if (i < s.nvec) st_loose(d + i, rs[q * G + g]);
            }
        }
        for (int q = 0; q < LG; q++) {
            const BatchSlot s = batch_slot(desc, RG + q, n);
            paced(s.valid);
            u32x4_u* d = (u32x4_u*)((unsigned char*)tb.p[s.p0 + n] + s.head * sizeof(E));
#pragma unroll
            for (int g = 0; g < G; g++) {
                const uint64_t i = s.first + batch_tile_vector(g, wave_runs);
                if (q * G + g == arrive_u && threadIdx.x == 0) phase_arrive(ps);
                if (i < s.nvec) st_loose(d + i, stage[(q * G + g) * kPhaseBlock + threadIdx.x]);
            }
        }
        if (more && arrive_u == kPhaseU) {
            __syncthreads();                                // "when done": every wave's stores have been acknowledged
            if (threadIdx.x == 0) phase_arrive(ps);
        }
        // The jobs' edge elements, spread over the blocks, after the block's report of the first write phase and before
        // its wait: there the round trip to memory costs nothing while other blocks still write.  Inside a read phase
        // it held up the one block of a job's first tile, and with it the barrier (64 jobs of 4 x 4 MiB with 112-byte
        // heads: 241 us against 222 us); after the last phase it is the last thing the chip does.
        if (t0 == 0)
            for (int j = blockIdx.x; j < n_jobs; j += gridDim.x) reduce_batch_edges<TR, OP>(tb, n, j);
        if (more) phase_wait(ps, ++gen, give_up, spin_ticks);
        desc = next;
    }
    if (total_tiles == 0)       // no phase at all
        for (int j = blockIdx.x; j < n_jobs; j += gridDim.x) reduce_batch_edges<TR, OP>(tb, n, j);
}

// Host side: fills tables of at most kBatchMaxJobs jobs / kBatchMaxPtrs pointers and launches one kernel per table,
// in the phased form when the table's jobs together fill whole phases (the rule of the single reduce, wants_phased,
// on their total), else in the streaming form.
inline bool skipped(const BatchLaunchArgs& a, int j) {
    return a.skip_from_count > 0 && a.counts[j] >= a.skip_from_count;
}

template <class TR, int OP>
inline hipError_t launch_batch_op(const BatchLaunchArgs& a) {
    typedef typename TR::elem_t E;
    const int per_launch = (kBatchMaxPtrs / (a.n + 1)) < kBatchMaxJobs ? (kBatchMaxPtrs / (a.n + 1)) : kBatchMaxJobs;
    const uint64_t phase_grid = (uint64_t)(a.tune.num_cus / kPhaseGroups) * kPhaseGroups;
    int j0 = 0;
    while (j0 < a.n_jobs) {
        // the jobs of this table: where each one's vectors start (the 16-byte boundary of the buffer that makes the
        // loose accesses cheapest) and whether it leaves its last whole vector to the edge lanes (vector_split)
        VecSplit split[kBatchMaxJobs];
        int nj = 0;
        uint64_t small_tiles = 0, phase_tiles = 0, vectors = 0;     // tiles of the streaming form (16 KiB), of the phased form (32 KiB)
        uint32_t realigned = 0;
        for (; j0 + nj < a.n_jobs && nj < per_launch; nj++) {
            const int j = j0 + nj;
            VecSplit v = { 0, 0, 0, 0 };
            if (a.counts[j] && !skipped(a, j)) {
                LaunchArgs one;
                one.srcs = a.srcs + (size_t)j * a.n;
                one.n = a.n;
                one.dst = a.dsts[j];
                one.count = a.counts[j];
                one.tune = a.tune;
                v = vector_split<E, TR::VEC>(one);
            }
            constexpr uint64_t kSmall = (uint64_t)kBlock * kBatchUnroll;
            const bool work = a.counts[j] && !skipped(a, j);
            const uint64_t jt = work ? (v.nvec ? (v.nvec + kSmall - 1) / kSmall : 1) : 0;   // edge elements only: still a tile
            if (small_tiles + jt > 0x7fffffffull) {
                if (nj == 0) return hipErrorInvalidValue;       // one job of more than 2^31 tiles (32 TiB)
                break;                                          // the next launch takes it
            }
            small_tiles += jt;
            phase_tiles += work ? (v.nvec ? (v.nvec + kBatchPhaseTile - 1) / kBatchPhaseTile : 1) : 0;
            vectors += v.nvec;
            realigned |= v.beyond;
            split[nj] = v;
        }
        bool phased = false;
        if (a.tune.sync != nullptr && a.tune.num_cus >= kPhaseGroups) {
            if (a.tune.variant != 0) phased = a.tune.variant == 8;
            else
                phased = a.tune.max_blocks == 0 && a.n >= 2 &&
                         (uint64_t)(a.n + 1) * vectors * 16u >= (uint64_t)a.tune.phased_min_bytes &&
                         batch_phases_full_enough(vectors, phase_tiles, phase_grid * (uint64_t)(MultiPhaseRegs<TR>::groups + kPhaseU / kBatchPhaseG),
                                                  kBatchPhaseTile, a.n);
        }
        const uint64_t tile = phased ? kBatchPhaseTile : (uint64_t)kBlock * kBatchUnroll;
        BatchTable tb;
        uint64_t tiles = 0;
        uint32_t off_lines = 0;         // does any buffer's first vector start off a 128-byte line?
        for (int q = 0; q < nj; q++) {
            const int j = j0 + q;
            const bool work = a.counts[j] && !skipped(a, j);
            tiles += work ? (split[q].nvec ? (split[q].nvec + tile - 1) / tile : 1) : 0;
            for (int k = 0; k < a.n; k++) tb.p[q * (a.n + 1) + k] = a.srcs[(size_t)j * a.n + k];
            tb.p[q * (a.n + 1) + a.n] = a.dsts[j];
            tb.count[q] = work ? a.counts[j] : 0;
            tb.tile_end[q] = (uint32_t)tiles;
            tb.head[q] = (uint8_t)(split[q].head | (split[q].beyond << 7));
            if (work)
                for (int k = 0; k <= a.n; k++)
                    off_lines |= (uint32_t)((uintptr_t)tb.p[q * (a.n + 1) + k] + split[q].head * sizeof(E)) & (kLineBytes - 1);
        }
        const uint32_t wave_runs = a.tune.wave_runs == 2 || (a.tune.wave_runs == 1 && off_lines);
        const uint32_t write_pace16 = a.n >= 2 && a.n <= PhasePacedInputs<TR, OP>::value ? write_pace_ticks16(phase_grid * kBatchPhaseTile * 16u, 1.1 * (double)a.tune.write_pace, a.tune.wall_khz) : 0u;
        j0 += nj;
        if (tiles == 0) continue;
        g_realigned_launches += realigned;
        if (phased) {
            g_last_kernel = "reduce_batch_phased_kernel";
            hipLaunchKernelGGL((reduce_batch_phased_kernel<TR, OP>), dim3((unsigned)phase_grid), dim3(kPhaseBlock), 0, a.stream, tb, a.n,
                               nj, (uint32_t)tiles, a.tune.sync, phase_early_loads<TR, OP>(a.tune, a.n, write_pace16 != 0), phase_early_stores<TR>(a.tune, 1), a.tune.spin_ticks,
                               wave_runs, write_pace16);
        }
        else {
            g_last_kernel = "reduce_batch_kernel";
            hipLaunchKernelGGL((reduce_batch_kernel<TR, OP>), dim3(grid_for(tiles, a.tune)), dim3(kBlock), 0, a.stream, tb, a.n, nj,
                               (uint32_t)tiles);
        }
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// One instantiation of this per traits class lives in its own translation unit.
template <class TR>
hipError_t launch_reduce_batch(const BatchLaunchArgs& a) {
    switch (a.op) {
        case OP_SUM: return launch_batch_op<TR, OP_SUM>(a);
        case OP_PROD: return launch_batch_op<TR, OP_PROD>(a);
        case OP_MIN: return launch_batch_op<TR, OP_MIN>(a);
        case OP_MAX: return launch_batch_op<TR, OP_MAX>(a);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace mi
