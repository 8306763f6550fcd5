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
    uint8_t head[kBatchMaxJobs];        // elements before job j's first vector
};
static_assert(sizeof(BatchTable) + 64 <= 4096, "the job table and the other arguments must fit the kernel-argument segment");

struct BatchLaunchArgs {
    const void* const* srcs;            // host array, n_jobs x n device pointers, job after job
    void* const* dsts;                  // host array, n_jobs device pointers
    const size_t* counts;               // host array, n_jobs element counts
    int n, n_jobs, op;
    hipStream_t stream;
    Tuning tune;
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
        const uint32_t head = tb.head[j];
        const uint64_t count = tb.count[j];
        const uint64_t nvec = (count - head) / TR::VEC;
        const uint32_t tail = (uint32_t)(count - head - nvec * TR::VEC);
        const int b = j * (n + 1);                      // the job's pointers: tb.p[b .. b + n]
        unsigned char* dst = (unsigned char*)tb.p[b + n];

        uint64_t idx[kBatchUnroll];
#pragma unroll
        for (int u = 0; u < kBatchUnroll; u++) idx[u] = (uint64_t)t * kTile + threadIdx.x + (uint64_t)u * kBlock;
        if (idx[0] < nvec) {
            Accs<TR> a[kBatchUnroll];
            const u32x4_u* s0 = (const u32x4_u*)((const unsigned char*)tb.p[b] + head * sizeof(E));
#pragma unroll
            for (int u = 0; u < kBatchUnroll; u++)
                a[u] = vec_init<TR>((idx[u] < nvec) ? ld_loose(s0 + idx[u]) : u32x4{ 0, 0, 0, 0 });
            for (int k = 1; k < n; k++) {
                const u32x4_u* sk = (const u32x4_u*)((const unsigned char*)tb.p[b + k] + head * sizeof(E));
                u32x4 x[kBatchUnroll];
#pragma unroll
                for (int u = 0; u < kBatchUnroll; u++) x[u] = (idx[u] < nvec) ? ld_loose(sk + idx[u]) : u32x4{ 0, 0, 0, 0 };
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

// Host side: fills tables of at most kBatchMaxJobs jobs / kBatchMaxPtrs pointers and launches one kernel per table.
template <class TR, int OP>
inline hipError_t launch_batch_op(const BatchLaunchArgs& a) {
    typedef typename TR::elem_t E;
    constexpr uint64_t kTile = (uint64_t)kBlock * kBatchUnroll;
    const int per_launch = (kBatchMaxPtrs / (a.n + 1)) < kBatchMaxJobs ? (kBatchMaxPtrs / (a.n + 1)) : kBatchMaxJobs;
    int j0 = 0;
    while (j0 < a.n_jobs) {
        BatchTable tb;
        int nj = 0;
        uint64_t tiles = 0;
        for (; j0 + nj < a.n_jobs && nj < per_launch; nj++) {
            const int j = j0 + nj;
            const uint64_t count = a.counts[j];
            // the vectors of a job start on the 16-byte boundary of the buffer that makes the loose accesses cheapest (vector_head)
            LaunchArgs one;
            one.srcs = a.srcs + (size_t)j * a.n;
            one.n = a.n;
            one.dst = a.dsts[j];
            one.count = count;
            uint64_t head = count ? vector_head<E>(one) : 0;
            if (head > count) head = count;
            const uint64_t nvec = (count - head) / TR::VEC;
            const uint64_t jt = count ? (nvec ? (nvec + kTile - 1) / kTile : 1) : 0;    // a job of edge elements only still gets a tile
            if (tiles + jt > 0x7fffffffull) {
                if (nj == 0) return hipErrorInvalidValue;       // one job of more than 2^31 tiles (32 TiB)
                break;                                          // the next launch takes it
            }
            tiles += jt;
            for (int k = 0; k < a.n; k++) tb.p[nj * (a.n + 1) + k] = a.srcs[(size_t)j * a.n + k];
            tb.p[nj * (a.n + 1) + a.n] = a.dsts[j];
            tb.count[nj] = count;
            tb.tile_end[nj] = (uint32_t)tiles;
            tb.head[nj] = (uint8_t)head;
        }
        j0 += nj;
        if (tiles == 0) continue;
        const int grid = grid_for(tiles, a.tune);
        g_last_kernel = "reduce_batch_kernel";
        hipLaunchKernelGGL((reduce_batch_kernel<TR, OP>), dim3(grid), dim3(kBlock), 0, a.stream, tb, a.n, nj, (uint32_t)tiles);
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
