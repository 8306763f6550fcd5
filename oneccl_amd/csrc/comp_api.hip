// extern "C" layer of libmi_ccl_comp.so: argument checks, traits selection and the copy / converter
// kernels.  The reduce kernels themselves are instantiated one traits class per translation unit
// (inst_*.hip) from reduce_kernels.hpp.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <cctype>

#include "../../include/mi_ccl_comp.h"
#include "batch_kernels.hpp"
#include "launch_geometry.hpp"
#include "reduce_kernels.hpp"

namespace mi {

#define MI_DECLARE(TR)                                                   \
    extern template hipError_t launch_reduce<TR>(const LaunchArgs&);     \
    extern template hipError_t launch_reduce_batch<TR>(const BatchLaunchArgs&)
MI_DECLARE(I8Traits);
MI_DECLARE(U8Traits);
MI_DECLARE(I16Traits);
MI_DECLARE(U16Traits);
MI_DECLARE(I32Traits);
MI_DECLARE(U32Traits);
MI_DECLARE(I64Traits);
MI_DECLARE(U64Traits);
MI_DECLARE(F32Traits);
MI_DECLARE(F64Traits);
MI_DECLARE(Fp16PairwiseTraits);
MI_DECLARE(Fp16NativeTraits);
typedef Bf16PairwiseTraits<false, false> Bf16PairScalar;
typedef Bf16PairwiseTraits<false, true> Bf16PairAvx512f;
typedef Bf16PairwiseTraits<true, true> Bf16PairAvx512bf;
MI_DECLARE(Bf16PairScalar);
MI_DECLARE(Bf16PairAvx512f);
MI_DECLARE(Bf16PairAvx512bf);
MI_DECLARE(Bf16KeepTraits<false>);
MI_DECLARE(Bf16KeepTraits<true>);

// ---------------------------------------------------------------------------------------------------
// tuning state and device facts

thread_local const char* g_last_kernel = "";
thread_local unsigned long g_realigned_launches = 0;
thread_local unsigned long g_wide_phase_launches = 0;

static std::atomic<int> g_waves_per_cu{ 256 };
static std::atomic<int> g_max_blocks{ 0 };
static std::atomic<int> g_xcd_chunked{ 0 };
static std::atomic<int> g_variant{ 0 };
static std::atomic<long> g_phased_min_bytes{ 160L << 20 };
static std::atomic<int> g_phase_early_loads{ -1 };
static std::atomic<int> g_phase_early_stores{ -1 };
static std::atomic<long> g_phase_spin_ticks{ kPhaseSpinTicks };
static std::atomic<int> g_fp16_impl{ MI_CCL_FP16_AVX512F };
static std::atomic<int> g_realign{ 1 };
static std::atomic<int> g_line_start{ 1 };
static std::atomic<int> g_wave_runs{ 1 };
static std::atomic<int> g_write_pace{ 7300 };
static std::atomic<long> g_launch_block_limit{ 0 };     // 0: what HIP allows; smaller values are for tests of the splitting
static_assert(kGeomBlock == kBlock, "the geometry header and the kernels agree on the block size");

static uint64_t block_limit() {
    const long v = g_launch_block_limit.load(std::memory_order_relaxed);
    const uint64_t hw = hip_block_limit(kBlock);
    return (v > 0 && (uint64_t)v < hw) ? (uint64_t)v : hw;
}
static std::atomic<int> g_num_cus[64];

// Barrier words of the phased kernels: kPhaseSlots sets per device (each GPU holds its own instance of a __device__
// variable at its own address, looked up once per device).  Every call takes the next set in turn, so that launches
// which overlap on one GPU (different streams) do not count each other's arrivals: with one shared set two
// overlapping launches lose their phase alignment and run at the unaligned speed, about a quarter slower.  (A set
// comes round again after kPhaseSlots calls; launches that far apart and still overlapping share it, which costs
// speed only, never correctness.)
constexpr size_t kBatchCopyAlone = 32u << 20;      // mi_ccl_comp_reduce_batch: one-input jobs from this many bytes get copy_kernel launches of their own
constexpr int kPhaseSlots = 16;
static __device__ PhaseSync g_phase_sync[kPhaseSlots];
static std::atomic<PhaseSync*> g_phase_sync_ptr[64];
static std::atomic<unsigned> g_phase_sync_next[64];

static PhaseSync* phase_sync() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return nullptr;
    PhaseSync* p = g_phase_sync_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        void* sym = nullptr;
        if (hipGetSymbolAddress(&sym, HIP_SYMBOL(g_phase_sync)) != hipSuccess)
            return nullptr;
        p = (PhaseSync*)sym;
        g_phase_sync_ptr[dev].store(p, std::memory_order_release);
    }
    return p + g_phase_sync_next[dev].fetch_add(1, std::memory_order_relaxed) % kPhaseSlots;
}

static int num_cus() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return 256;
    int v = g_num_cus[dev].load(std::memory_order_relaxed);
    if (v == 0) {
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
            v = 256;
        g_num_cus[dev].store(v, std::memory_order_relaxed);
    }
    return v;
}

static std::atomic<int> g_wall_khz[64];
static int wall_khz() {         // the rate of wall_clock64(), which paces the write phase of the phased reduce
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return 100000;
    int v = g_wall_khz[dev].load(std::memory_order_relaxed);
    if (v == 0) {
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeWallClockRate, dev) != hipSuccess || v <= 0)
            v = 100000;
        g_wall_khz[dev].store(v, std::memory_order_relaxed);
    }
    return v;
}

Tuning current_tuning() {
    Tuning t;
    t.waves_per_cu = g_waves_per_cu.load(std::memory_order_relaxed);
    t.max_blocks = g_max_blocks.load(std::memory_order_relaxed);
    t.xcd_chunked = g_xcd_chunked.load(std::memory_order_relaxed);
    t.variant = g_variant.load(std::memory_order_relaxed);
    t.num_cus = num_cus();
    t.phased_min_bytes = g_phased_min_bytes.load(std::memory_order_relaxed);
    t.sync = phase_sync();
    t.early_loads = g_phase_early_loads.load(std::memory_order_relaxed);
    t.early_stores = g_phase_early_stores.load(std::memory_order_relaxed);
    t.spin_ticks = g_phase_spin_ticks.load(std::memory_order_relaxed);
    t.fp16_impl = g_fp16_impl.load(std::memory_order_relaxed);
    t.realign = g_realign.load(std::memory_order_relaxed);
    t.line_start = g_line_start.load(std::memory_order_relaxed);
    t.wave_runs = g_wave_runs.load(std::memory_order_relaxed);
    t.write_pace = g_write_pace.load(std::memory_order_relaxed);
    t.wall_khz = wall_khz();
    return t;
}

static const size_t kDtypeSize[MI_CCL_DATATYPE_LAST] = { 1, 1, 2, 2, 4, 4, 8, 8, 2, 4, 8, 2 };
static const char* const kDtypeName[MI_CCL_DATATYPE_LAST] = { "int8",  "uint8",  "int16",   "uint16",
                                                              "int32", "uint32", "int64",   "uint64",
                                                              "float16", "float32", "float64", "bfloat16" };

static int status_of(hipError_t e) {
    if (e == hipSuccess)
        return MI_CCL_SUCCESS;
    if (e == hipErrorOutOfMemory)
        return MI_CCL_OUT_OF_RESOURCE;
    if (e == hipErrorInvalidValue)
        return MI_CCL_INVALID_ARGUMENTS;
    return MI_CCL_RUNTIME_ERROR;
}

// One launch of the traits class that (dtype, lp_mode, bf16_impl) selects.
static hipError_t dispatch(int dtype, bool keep, int bf16_impl, const LaunchArgs& a) {
    switch (dtype) {
        case MI_CCL_INT8: return launch_reduce<I8Traits>(a);
        case MI_CCL_UINT8: return launch_reduce<U8Traits>(a);
        case MI_CCL_INT16: return launch_reduce<I16Traits>(a);
        case MI_CCL_UINT16: return launch_reduce<U16Traits>(a);
        case MI_CCL_INT32: return launch_reduce<I32Traits>(a);
        case MI_CCL_UINT32: return launch_reduce<U32Traits>(a);
        case MI_CCL_INT64: return launch_reduce<I64Traits>(a);
        case MI_CCL_UINT64: return launch_reduce<U64Traits>(a);
        case MI_CCL_FLOAT16:
            return a.tune.fp16_impl == MI_CCL_FP16_AVX512FP16 ? launch_reduce<Fp16NativeTraits>(a)
                                                              : launch_reduce<Fp16PairwiseTraits>(a);
        case MI_CCL_FLOAT32: return launch_reduce<F32Traits>(a);
        case MI_CCL_FLOAT64: return launch_reduce<F64Traits>(a);
        case MI_CCL_BFLOAT16:
            if (keep)
                return (bf16_impl == MI_CCL_BF16_AVX512BF) ? launch_reduce<Bf16KeepTraits<true>>(a)
                                                            : launch_reduce<Bf16KeepTraits<false>>(a);
            if (bf16_impl == MI_CCL_BF16_SCALAR)
                return launch_reduce<Bf16PairScalar>(a);
            if (bf16_impl == MI_CCL_BF16_AVX512F)
                return launch_reduce<Bf16PairAvx512f>(a);
            return launch_reduce<Bf16PairAvx512bf>(a);
        default: return hipErrorInvalidValue;
    }
}

// The same choice for a launch of many independent jobs.
static hipError_t dispatch_batch(int dtype, bool keep, int bf16_impl, const BatchLaunchArgs& a) {
    switch (dtype) {
        case MI_CCL_INT8: return launch_reduce_batch<I8Traits>(a);
        case MI_CCL_UINT8: return launch_reduce_batch<U8Traits>(a);
        case MI_CCL_INT16: return launch_reduce_batch<I16Traits>(a);
        case MI_CCL_UINT16: return launch_reduce_batch<U16Traits>(a);
        case MI_CCL_INT32: return launch_reduce_batch<I32Traits>(a);
        case MI_CCL_UINT32: return launch_reduce_batch<U32Traits>(a);
        case MI_CCL_INT64: return launch_reduce_batch<I64Traits>(a);
        case MI_CCL_UINT64: return launch_reduce_batch<U64Traits>(a);
        case MI_CCL_FLOAT16:
            return a.tune.fp16_impl == MI_CCL_FP16_AVX512FP16 ? launch_reduce_batch<Fp16NativeTraits>(a)
                                                              : launch_reduce_batch<Fp16PairwiseTraits>(a);
        case MI_CCL_FLOAT32: return launch_reduce_batch<F32Traits>(a);
        case MI_CCL_FLOAT64: return launch_reduce_batch<F64Traits>(a);
        case MI_CCL_BFLOAT16:
            if (keep)
                return (bf16_impl == MI_CCL_BF16_AVX512BF) ? launch_reduce_batch<Bf16KeepTraits<true>>(a)
                                                            : launch_reduce_batch<Bf16KeepTraits<false>>(a);
            if (bf16_impl == MI_CCL_BF16_SCALAR)
                return launch_reduce_batch<Bf16PairScalar>(a);
            if (bf16_impl == MI_CCL_BF16_AVX512F)
                return launch_reduce_batch<Bf16PairAvx512f>(a);
            return launch_reduce_batch<Bf16PairAvx512bf>(a);
        default: return hipErrorInvalidValue;
    }
}

static int launch_copy(const void* in, void* out, size_t bytes, bool nontemporal, hipStream_t stream);
static int launch_broadcast(const void* in, void* const* dsts, int m, size_t bytes, hipStream_t stream);

static bool fp16_impl_ok(int v) {
    return v == MI_CCL_FP16_DEFAULT || (v >= MI_CCL_FP16_F16C && v <= MI_CCL_FP16_AVX512FP16);
}

static int reduce_n_impl(int dtype, int op, const void* const* srcs, int n, void* const* dsts, int m, size_t count,
                         int lp_mode, int bf16_impl, int fp16_impl, void* stream) {
    if (count == 0)
        return MI_CCL_SUCCESS;
    if (m < 1 || m > kMaxDsts || !dsts)
        return MI_CCL_INVALID_ARGUMENTS;
    if (dtype < 0 || dtype >= MI_CCL_DATATYPE_LAST || op < MI_CCL_SUM || op > MI_CCL_MAX)
        return MI_CCL_INVALID_ARGUMENTS;
    if (n < 1 || n > kMaxSrcs || !srcs)
        return MI_CCL_INVALID_ARGUMENTS;
    if (bf16_impl < MI_CCL_BF16_SCALAR || bf16_impl > MI_CCL_BF16_AVX512BF || !fp16_impl_ok(fp16_impl))
        return MI_CCL_INVALID_ARGUMENTS;
    if (lp_mode & ~(MI_CCL_LP_KEEP_PRECISION | MI_CCL_LP_TAIL_QUIRK))
        return MI_CCL_INVALID_ARGUMENTS;
    const bool keep = (lp_mode & MI_CCL_LP_KEEP_PRECISION) != 0;
    if (keep && dtype != MI_CCL_BFLOAT16)
        return MI_CCL_INVALID_ARGUMENTS;
    if ((lp_mode & MI_CCL_LP_TAIL_QUIRK) && !keep)
        return MI_CCL_INVALID_ARGUMENTS;
    const size_t esz = kDtypeSize[dtype];
    for (int k = 0; k < m; k++)
        if (!dsts[k] || ((uintptr_t)dsts[k] % esz) != 0)
            return MI_CCL_INVALID_ARGUMENTS;
    for (int j = 0; j < n; j++)
        if (!srcs[j] || ((uintptr_t)srcs[j] % esz) != 0)
            return MI_CCL_INVALID_ARGUMENTS;

    // one input, rounded after every pair: a chain of zero pairwise steps hands the input back as it is, whatever
    // the type -- a copy to one buffer or a broadcast to several
    Tuning tune = current_tuning();
    if (fp16_impl != MI_CCL_FP16_DEFAULT)
        tune.fp16_impl = fp16_impl;     // this call's choice; the process-wide value is only the default
    if (n == 1 && !keep && tune.variant == 0) {
        if (m == 1)
            return dsts[0] == srcs[0] ? MI_CCL_SUCCESS : launch_copy(srcs[0], dsts[0], count * esz, true, (hipStream_t)stream);
        if (!broadcast_wants_phased(tune, (uint64_t)count * esz))
            return launch_broadcast(srcs[0], dsts, m, count * esz, (hipStream_t)stream);
        // large: the phased reduce with one input, on bytes (a sum over one unsigned input hands every bit back)
        LaunchArgs b;
        b.srcs = srcs;
        b.n = 1;
        b.dst = dsts[0];
        b.dsts = dsts;
        b.m = m;
        b.count = count * esz;
        b.op = MI_CCL_SUM;
        b.stream = (hipStream_t)stream;
        b.tune = tune;
        b.tune.variant = 8;
        return status_of(dispatch(MI_CCL_UINT8, false, MI_CCL_BF16_AVX512BF, b));
    }

    LaunchArgs a;
    a.srcs = srcs;
    a.n = n;
    a.dst = dsts[0];
    a.dsts = dsts;
    a.m = m;
    a.count = count;
    a.op = op;
    a.stream = (hipStream_t)stream;
    a.tune = tune;

    // keep-precision under avx512bf: the reference narrows the last count % 16 elements by truncation
    // (src/comp/bf16/bf16.cpp:144-148).  Those <= 15 elements get a launch of the truncating traits.
    if (keep && (lp_mode & MI_CCL_LP_TAIL_QUIRK) && bf16_impl == MI_CCL_BF16_AVX512BF && (count % 16) != 0) {
        const size_t limit = count - count % 16;
        if (limit) {
            a.count = limit;
            hipError_t e = dispatch(dtype, true, MI_CCL_BF16_AVX512BF, a);
            if (e != hipSuccess)
                return status_of(e);
        }
        const void* shifted[kMaxSrcs];
        for (int j = 0; j < n; j++) shifted[j] = (const char*)srcs[j] + limit * esz;
        void* shifted_dst[kMaxDsts];
        for (int k = 0; k < m; k++) shifted_dst[k] = (char*)dsts[k] + limit * esz;
        a.srcs = shifted;
        a.dst = shifted_dst[0];
        a.dsts = shifted_dst;
        a.count = count - limit;
        return status_of(dispatch(dtype, true, MI_CCL_BF16_AVX512F, a));
    }
    return status_of(dispatch(dtype, keep, bf16_impl, a));
}

// ---------------------------------------------------------------------------------------------------
// copy and converter kernels

// Vectors from the output's first 16-byte boundary on; the input is read as loose vectors (any alignment).  One
// vector per lane and one 4 KiB tile per block, however large the copy: short-lived blocks over a compact window of
// addresses measure 6.45-6.5 TB/s from 512 MiB up (6.6-6.7 with device-scope stores, st_loose_device_scope), four
// vectors per lane 5.9 and the phased one-input reduce 5.9.
template <bool NT>
__global__ void __launch_bounds__(kBlock)
copy_kernel(const unsigned char* in, unsigned char* out, uint32_t head, uint64_t nvec, uint32_t tail) {
    const u32x4_u* s = (const u32x4_u*)(in + head);
    u32x4* d = (u32x4*)(out + head);
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < nvec; i += (uint64_t)gridDim.x * kBlock) {
        if (NT)
            st_loose_device_scope((u32x4_u*)(d + i), ld_loose(s + i));
        else
            d[i] = *(s + i);
    }
    if (blockIdx.x == 0 && threadIdx.x < head + tail) {
        uint32_t t = threadIdx.x;
        uint64_t i = (t < head) ? t : (uint64_t)head + nvec * 16 + (t - head);
        out[i] = in[i];
    }
}

// One buffer written to m buffers (the shape of write_monolithic_kernel_N, kernels.cl:423-560).  A wave does one load
// and one store, like the copy; a block serves one destination.  The source is taken in sections of kBcastSect
// 4 KiB tiles: all tiles of a section go to the first destination, then all of them to the second, and so on, so
// that every destination sees one ascending stream of writes while the section is re-read from the L2 caches (a
// tile is always handled on the same XCD: sections are a multiple of eight tiles, and blocks go to the XCDs
// round-robin).  Sections of 4 to 24 MiB measure 6.4-6.5 TB/s for 1 -> 7 at 1 GiB; 32 MiB no longer fits (4.2), and
// a wave that stores its vector to all seven destinations itself measures 5.5.
constexpr uint32_t kBcastSect = 4096;       // tiles of kBlock vectors per section: 16 MiB

__global__ void __launch_bounds__(kBlock)
broadcast_kernel(const unsigned char* in, DstTable d, int m, uint32_t head, uint64_t nvec, uint32_t tail, uint32_t sect_tiles) {
    const BcastLane l = bcast_lane(blockIdx.x, threadIdx.x, sect_tiles, (uint32_t)m);
    const uint32_t k = l.dst;
    const uint64_t i = l.vec;
    if (i < nvec) {
        const u32x4 v = *((const u32x4_u*)(in + head) + i);         // cached: the other destinations read it again
        st_loose((u32x4_u*)((unsigned char*)d.p[k] + head) + i, v);
    }
    if (blockIdx.x == 0 && threadIdx.x < head + tail) {
        const uint32_t e = threadIdx.x;
        const uint64_t b = (e < head) ? e : (uint64_t)head + nvec * 16 + (e - head);
        const unsigned char x = in[b];
        for (int q = 0; q < m; q++) ((unsigned char*)d.p[q])[b] = x;
    }
}

// Array converters, one tile per block.  The vectors start where the output reaches a 16-byte boundary (`head`
// elements in); the input is read as loose vectors, so the two arrays may sit at any alignment relative to each
// other.  The elements before the first and after the last whole group (at most 14) go to the lanes of block 0.
// fp32 -> bf16: eight elements per lane (two 16-byte loads, one 16-byte store), one step per lane: 6.2 TB/s at 2^28
// elements where two steps measure 6.0-6.2 and, at 2^23, 4.9 against 5.9.

// fp32 -> bf16; elements at or beyond rne_limit are truncated instead of rounded
constexpr int kCvtUnroll = 1;
template <bool RNE>
__global__ void __launch_bounds__(kBlock)
f32_to_bf16_kernel(const uint32_t* in, uint16_t* out, uint32_t head, uint64_t noct, uint32_t tail, uint64_t rne_limit) {
    const u32x4_u* s = (const u32x4_u*)(in + head);
    u32x4_u* d = (u32x4_u*)(out + head);
    const uint64_t base = (uint64_t)blockIdx.x * (kBlock * kCvtUnroll) + threadIdx.x;
    u32x4 x[kCvtUnroll][2];
#pragma unroll
    for (int u = 0; u < kCvtUnroll; u++) {
        const uint64_t o = base + (uint64_t)u * kBlock;
        if (o < noct) {
            x[u][0] = ld_loose(s + 2 * o);
            x[u][1] = ld_loose(s + 2 * o + 1);
        }
    }
#pragma unroll
    for (int u = 0; u < kCvtUnroll; u++) {
        const uint64_t o = base + (uint64_t)u * kBlock;
        if (o < noct) {
            const uint64_t first = head + 8 * o;
            u32x4 r;
            if (RNE && first + 8 <= rne_limit) {
#pragma unroll
                for (int k = 0; k < 4; k++) r[k] = bf16_narrow_rne_pack2(x[u][k >> 1][(2 * k) & 3], x[u][k >> 1][(2 * k + 1) & 3]);
            }
            else {
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    uint32_t h[2];
#pragma unroll
                    for (int e = 0; e < 2; e++) {
                        const uint32_t v = x[u][k >> 1][(2 * k + e) & 3];
                        h[e] = (RNE && first + 2 * k + e < rne_limit) ? bf16_narrow_rne(v) : bf16_narrow_trunc(v);
                    }
                    r[k] = (h[0] & 0xffffu) | (h[1] << 16);
                }
            }
            st_loose(d + o, r);
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < head + tail) {
        const uint32_t t = threadIdx.x;
        const uint64_t i = (t < head) ? t : (uint64_t)head + noct * 8 + (t - head);
        const uint32_t v = in[i];
        out[i] = (uint16_t)((RNE && i < rne_limit) ? bf16_narrow_rne(v) : bf16_narrow_trunc(v));
    }
}

// bf16 -> fp32: a lane widens four elements (8 bytes in, one 16-byte vector out, so that both the loads and the
// stores of a wave are contiguous), one step per lane (6.6 TB/s at 2^28 elements; two steps 6.2, four 6.0).  `nquad`
// groups of four from element `head` on.
constexpr int kWidenUnroll = 1;
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef u32x2 u32x2_u __attribute__((aligned(1)));

__global__ void __launch_bounds__(kBlock)
bf16_to_f32_kernel(const uint16_t* in, uint32_t* out, uint32_t head, uint64_t nquad, uint32_t tail) {
    const u32x2_u* s = (const u32x2_u*)(in + head);
    u32x4_u* d = (u32x4_u*)(out + head);
    const uint64_t base = (uint64_t)blockIdx.x * (kBlock * kWidenUnroll) + threadIdx.x;
    u32x2 x[kWidenUnroll];
#pragma unroll
    for (int u = 0; u < kWidenUnroll; u++) {
        const uint64_t q = base + (uint64_t)u * kBlock;
        if (q < nquad) x[u] = __builtin_nontemporal_load(s + q);
    }
#pragma unroll
    for (int u = 0; u < kWidenUnroll; u++) {
        const uint64_t q = base + (uint64_t)u * kBlock;
        if (q < nquad) {
            const u32x2 h = x[u];
            st_loose(d + q, u32x4{ h[0] << 16, h[0] & 0xffff0000u, h[1] << 16, h[1] & 0xffff0000u });
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < head + tail) {
        const uint32_t t = threadIdx.x;
        const uint64_t i = (t < head) ? t : (uint64_t)head + nquad * 4 + (t - head);
        out[i] = (uint32_t)in[i] << 16;
    }
}

// fp32 <-> fp16 with the same shapes (the reference converts one vector of eight with VCVTPS2PH imm 0 / VCVTPH2PS,
// src/comp/fp16/fp16.cpp:55-61): the hardware conversions round to nearest even, keep subnormals and quiet a
// signalling NaN keeping the top of its payload, as the x86 instructions do.
__global__ void __launch_bounds__(kBlock)
f32_to_f16_kernel(const uint32_t* in, uint16_t* out, uint32_t head, uint64_t noct, uint32_t tail) {
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    const u32x4_u* s = (const u32x4_u*)(in + head);
    u32x4_u* d = (u32x4_u*)(out + head);
    const uint64_t o = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (o < noct) {
        const u32x4 x0 = ld_loose(s + 2 * o), x1 = ld_loose(s + 2 * o + 1);
        u32x4 r;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const u32x4& x = (k < 2) ? x0 : x1;
            const half2_t h = { (_Float16)as_f32(x[(2 * k) & 3]), (_Float16)as_f32(x[(2 * k + 1) & 3]) };
            r[k] = __builtin_bit_cast(uint32_t, h);
        }
        st_loose(d + o, r);
    }
    if (blockIdx.x == 0 && threadIdx.x < head + tail) {
        const uint32_t t = threadIdx.x;
        const uint64_t i = (t < head) ? t : (uint64_t)head + noct * 8 + (t - head);
        out[i] = __builtin_bit_cast(uint16_t, (_Float16)as_f32(in[i]));
    }
}

__global__ void __launch_bounds__(kBlock)
f16_to_f32_kernel(const uint16_t* in, uint32_t* out, uint32_t head, uint64_t nquad, uint32_t tail) {
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    const u32x2_u* s = (const u32x2_u*)(in + head);
    u32x4_u* d = (u32x4_u*)(out + head);
    const uint64_t q = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (q < nquad) {
        const u32x2 x = __builtin_nontemporal_load(s + q);
        const half2_t a = __builtin_bit_cast(half2_t, (uint32_t)x[0]), b = __builtin_bit_cast(half2_t, (uint32_t)x[1]);
        st_loose(d + q, u32x4{ as_u32((float)a[0]), as_u32((float)a[1]), as_u32((float)b[0]), as_u32((float)b[1]) });
    }
    if (blockIdx.x == 0 && threadIdx.x < head + tail) {
        const uint32_t t = threadIdx.x;
        const uint64_t i = (t < head) ? t : (uint64_t)head + nquad * 4 + (t - head);
        out[i] = as_u32((float)__builtin_bit_cast(_Float16, in[i]));
    }
}

// ---------------------------------------------------------------------------------------------------
// Calibration kernels: what the memory system sustains for reads alone and for writes alone, in the access shapes
// the kernels above use.  Measurement aids, not part of any reduce.

// n buffers read as the streaming reduce reads them (a tile of 256 x 4 vectors per block, the inputs one after the
// other, nontemporal loads), nothing written: the xor of what was read decides a store that practically never happens.
__global__ void __launch_bounds__(kBlock)
probe_read_kernel(SrcTable src, int n, uint64_t nvec, u32x4* sink) {
    constexpr int U = 4;
    constexpr uint64_t kTile = (uint64_t)kBlock * U;
    u32x4 acc = { 0, 0, 0, 0 };
    for (uint64_t t = blockIdx.x; t * kTile < nvec; t += gridDim.x) {
        const uint64_t base = t * kTile + threadIdx.x;
        for (int j = 0; j < n; j++) {
            const u32x4* s = (const u32x4*)src.p[j];
            u32x4 x[U];
#pragma unroll
            for (int u = 0; u < U; u++) x[u] = (base + (uint64_t)u * kBlock < nvec) ? __builtin_nontemporal_load(s + base + (uint64_t)u * kBlock) : u32x4{ 0, 0, 0, 0 };
#pragma unroll
            for (int u = 0; u < U; u++) acc ^= x[u];
        }
    }
    if (acc[0] == 0x12345678u && acc[1] == 0x9abcdef0u && acc[2] == 0x0fedcba9u && acc[3] == 0x87654321u) sink[threadIdx.x] = acc;
}

// U vectors per lane stored with nontemporal stores, one tile per block.  U = 1 is the shape of the copy, broadcast
// and converter kernels (a wave issues one store and ends), U = 4 that of the streaming reduce.
template <int U>
__global__ void __launch_bounds__(kBlock)
probe_write_kernel(u32x4* dst, uint64_t nvec) {
    constexpr uint64_t kTile = (uint64_t)kBlock * U;
    const u32x4 v = { 1u, 2u, 3u, blockIdx.x };
    for (uint64_t t = blockIdx.x; t * kTile < nvec; t += gridDim.x) {
        const uint64_t base = t * kTile + threadIdx.x;
#pragma unroll
        for (int u = 0; u < U; u++)
            if (base + (uint64_t)u * kBlock < nvec) __builtin_nontemporal_store(v, dst + base + (uint64_t)u * kBlock);
    }
}

static __device__ u32x4 g_probe_sink[kBlock];
static std::atomic<u32x4*> g_probe_sink_ptr[64];

}  // namespace mi

using namespace mi;

extern "C" {

int mi_ccl_probe_bandwidth(int kind, void* const* bufs, int n, size_t bytes, void* stream) {
    if (!bufs || n < 1 || n > kMaxSrcs || (bytes % 16) != 0 || bytes == 0)
        return MI_CCL_INVALID_ARGUMENTS;
    for (int j = 0; j < n; j++)
        if (!bufs[j] || ((uintptr_t)bufs[j] & 15u))
            return MI_CCL_INVALID_ARGUMENTS;
    const uint64_t nvec = bytes / 16;
    if (kind == MI_CCL_PROBE_READ) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
            return MI_CCL_RUNTIME_ERROR;
        u32x4* sink = g_probe_sink_ptr[dev].load(std::memory_order_acquire);
        if (!sink) {
            void* sym = nullptr;
            const hipError_t e = hipGetSymbolAddress(&sym, HIP_SYMBOL(g_probe_sink));
            if (e != hipSuccess)
                return status_of(e);
            sink = (u32x4*)sym;
            g_probe_sink_ptr[dev].store(sink, std::memory_order_release);
        }
        SrcTable s;
        for (int j = 0; j < n; j++) s.p[j] = bufs[j];
        const uint64_t tiles = (nvec + kBlock * 4 - 1) / (kBlock * 4);
        g_last_kernel = "probe_read_kernel";
        hipLaunchKernelGGL(probe_read_kernel, dim3((unsigned)(tiles < 65536 ? tiles : 65536)), dim3(kBlock), 0,
                           (hipStream_t)stream, s, n, nvec, sink);
        return status_of(hipGetLastError());
    }
    if (kind == MI_CCL_PROBE_WRITE_ONE || kind == MI_CCL_PROBE_WRITE_FOUR) {
        if (n != 1)
            return MI_CCL_INVALID_ARGUMENTS;
        const unsigned u = kind == MI_CCL_PROBE_WRITE_ONE ? 1 : 4;
        const uint64_t tiles = (nvec + kBlock * u - 1) / (kBlock * u);
        const uint64_t cap = kind == MI_CCL_PROBE_WRITE_ONE ? hip_block_limit(kBlock) : 65536;
        const unsigned grid = (unsigned)(tiles < cap ? tiles : cap);
        g_last_kernel = "probe_write_kernel";
        if (u == 1)
            hipLaunchKernelGGL(probe_write_kernel<1>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, (u32x4*)bufs[0], nvec);
        else
            hipLaunchKernelGGL(probe_write_kernel<4>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, (u32x4*)bufs[0], nvec);
        return status_of(hipGetLastError());
    }
    return MI_CCL_INVALID_ARGUMENTS;
}

size_t mi_ccl_datatype_size(int dtype) {
    return (dtype >= 0 && dtype < MI_CCL_DATATYPE_LAST) ? kDtypeSize[dtype] : 0;
}

const char* mi_ccl_datatype_name(int dtype) {
    return (dtype >= 0 && dtype < MI_CCL_DATATYPE_LAST) ? kDtypeName[dtype] : "";
}

const char* mi_ccl_reduction_to_str(int op) {
    switch (op) {
        case MI_CCL_SUM: return "sum";
        case MI_CCL_PROD: return "prod";
        case MI_CCL_MIN: return "min";
        case MI_CCL_MAX: return "max";
        case MI_CCL_CUSTOM: return "custom";
        default: return "unknown";
    }
}

const char* mi_ccl_status_str(int status) {
    switch (status) {
        case MI_CCL_SUCCESS: return "success";
        case MI_CCL_OUT_OF_RESOURCE: return "out_of_resource";
        case MI_CCL_INVALID_ARGUMENTS: return "invalid_arguments";
        case MI_CCL_RUNTIME_ERROR: return "runtime_error";
        default: return "unknown";
    }
}

int mi_ccl_kernel_name(const char* kernel, int dtype, int op, char* buf, size_t buf_len) {
    if (!kernel || !buf || dtype < 0 || dtype >= MI_CCL_DATATYPE_LAST || op < MI_CCL_SUM || op > MI_CCL_MAX)
        return MI_CCL_INVALID_ARGUMENTS;
    int n = snprintf(buf, buf_len, "%s_%s_%s", kernel, kDtypeName[dtype], mi_ccl_reduction_to_str(op));
    if (n < 0 || (size_t)n >= buf_len)
        return MI_CCL_INVALID_ARGUMENTS;
    for (char* c = buf; *c; c++) *c = (char)tolower((unsigned char)*c);
    return MI_CCL_SUCCESS;
}

int mi_ccl_comp_reduce(int dtype, int op, const void* in, size_t count, void* inout, int bf16_impl, int fp16_impl,
                       void* stream) {
    if (count == 0)
        return MI_CCL_SUCCESS;
    const void* srcs[2] = { inout, in };
    return reduce_n_impl(dtype, op, srcs, 2, &inout, 1, count, MI_CCL_LP_PAIRWISE, bf16_impl, fp16_impl, stream);
}

int mi_ccl_bf16_reduce(const void* in, size_t count, void* inout, int op, int bf16_impl, void* stream) {
    return mi_ccl_comp_reduce(MI_CCL_BFLOAT16, op, in, count, inout, bf16_impl, MI_CCL_FP16_DEFAULT, stream);
}

int mi_ccl_fp16_reduce(const void* in, size_t count, void* inout, int op, int fp16_impl, void* stream) {
    return mi_ccl_comp_reduce(MI_CCL_FLOAT16, op, in, count, inout, MI_CCL_BF16_AVX512BF, fp16_impl, stream);
}

int mi_ccl_comp_reduce_n(int dtype, int op, const void* const* srcs, int n, void* dst, size_t count, int lp_mode,
                         int bf16_impl, int fp16_impl, void* stream) {
    return reduce_n_impl(dtype, op, srcs, n, &dst, 1, count, lp_mode, bf16_impl, fp16_impl, stream);
}

int mi_ccl_comp_reduce_write_n(int dtype, int op, const void* const* srcs, int n, void* const* dsts, int m, size_t count,
                               int lp_mode, int bf16_impl, int fp16_impl, void* stream) {
    return reduce_n_impl(dtype, op, srcs, n, dsts, m, count, lp_mode, bf16_impl, fp16_impl, stream);
}

int mi_ccl_comp_reduce_batch(int dtype, int op, const void* const* srcs, int n, void* const* dsts, const size_t* counts,
                             int n_jobs, int lp_mode, int bf16_impl, int fp16_impl, void* stream) {
    if (n_jobs == 0)
        return MI_CCL_SUCCESS;
    if (n_jobs < 0 || !srcs || !dsts || !counts || n < 1 || n > kMaxFixedN)
        return MI_CCL_INVALID_ARGUMENTS;
    if (dtype < 0 || dtype >= MI_CCL_DATATYPE_LAST || op < MI_CCL_SUM || op > MI_CCL_MAX)
        return MI_CCL_INVALID_ARGUMENTS;
    if (bf16_impl < MI_CCL_BF16_SCALAR || bf16_impl > MI_CCL_BF16_AVX512BF || !fp16_impl_ok(fp16_impl))
        return MI_CCL_INVALID_ARGUMENTS;
    const bool keep = (lp_mode & MI_CCL_LP_KEEP_PRECISION) != 0;
    if ((lp_mode & ~MI_CCL_LP_KEEP_PRECISION) != 0 || (keep && dtype != MI_CCL_BFLOAT16))
        return MI_CCL_INVALID_ARGUMENTS;        // the truncated tail (MI_CCL_LP_TAIL_QUIRK) belongs to ccl_comp_batch_reduce
    const size_t esz = kDtypeSize[dtype];
    for (int j = 0; j < n_jobs; j++) {
        if (counts[j] == 0)
            continue;                           // an empty job's pointers are not looked at
        if (!dsts[j] || ((uintptr_t)dsts[j] % esz) != 0)
            return MI_CCL_INVALID_ARGUMENTS;
        for (int k = 0; k < n; k++)
            if (!srcs[(size_t)j * n + k] || ((uintptr_t)srcs[(size_t)j * n + k] % esz) != 0)
                return MI_CCL_INVALID_ARGUMENTS;
    }
    BatchLaunchArgs a;
    a.srcs = srcs;
    a.dsts = dsts;
    a.counts = counts;
    a.n = n;
    a.n_jobs = n_jobs;
    a.op = op;
    a.stream = (hipStream_t)stream;
    a.tune = current_tuning();
    if (fp16_impl != MI_CCL_FP16_DEFAULT)
        a.tune.fp16_impl = fp16_impl;
    // Everything a job can be refused for has been looked at above, for every job, before the first launch.  Nothing is
    // allocated, on the host or on the device: the tables are built on the stack and travel in the kernel arguments.
    // One input per job, rounded after every pair, is a byte copy per job (copy_data): a job of kBatchCopyAlone bytes or
    // more goes to the copy kernel, whose one-store-per-wave shape is about a tenth faster and whose launch is
    // nothing against such a copy; the others share the batch launch.
    if (n == 1 && !keep && a.tune.variant == 0) {
        const size_t from = (kBatchCopyAlone + esz - 1) / esz;
        for (int j = 0; j < n_jobs; j++)
            if (counts[j] >= from && dsts[j] != srcs[j]) {
                const int rc = launch_copy(srcs[j], dsts[j], counts[j] * esz, true, (hipStream_t)stream);
                if (rc != MI_CCL_SUCCESS)
                    return rc;
            }
        a.skip_from_count = from;
    }
    return status_of(dispatch_batch(dtype, keep, bf16_impl, a));
}

int mi_ccl_comp_batch_reduce(const void* in_buf, const size_t* offsets, size_t n_offsets, size_t count, void* inout,
                             int dtype, int op, int bf16_keep_precision_mode, int bf16_impl, int fp16_impl,
                             void* stream) {
    if (dtype < 0 || dtype >= MI_CCL_DATATYPE_LAST)
        return MI_CCL_INVALID_ARGUMENTS;
    if (n_offsets == 0 || n_offsets > (size_t)kMaxSrcs || !offsets)
        return MI_CCL_INVALID_ARGUMENTS;
    if (count == 0)
        return MI_CCL_SUCCESS;
    if (!in_buf || !inout)
        return MI_CCL_INVALID_ARGUMENTS;
    const void* srcs[kMaxSrcs];
    srcs[0] = inout; /* inout_buf => in_buf + offsets[0] (comp.cpp:217) */
    for (size_t i = 1; i < n_offsets; i++) srcs[i] = (const char*)in_buf + kDtypeSize[dtype] * offsets[i];
    int lp = bf16_keep_precision_mode ? (MI_CCL_LP_KEEP_PRECISION | MI_CCL_LP_TAIL_QUIRK) : MI_CCL_LP_PAIRWISE;
    return reduce_n_impl(dtype, op, srcs, (int)n_offsets, &inout, 1, count, lp, bf16_impl, fp16_impl, stream);
}

} /* extern "C" */

namespace mi {
static int launch_copy(const void* in, void* out, size_t bytes, bool nontemporal, hipStream_t stream) {
    // large copies start their vectors on a 128-byte line of the output (a line written in two parts costs more than
    // one read in two parts)
    const uint32_t boundary = bytes >= kLineStartBytes && g_line_start.load(std::memory_order_relaxed) ? kLineBytes : 16u;
    const LaneWork w = lane_work((uintptr_t)out, 1, bytes, 16, boundary);
    const uint64_t limit = block_limit(), n = num_launches(w, kBlock, limit);
    for (uint64_t i = 0; i < n; i++) {
        const LaunchPiece p = launch_piece(w, kBlock, limit, i);
        // a piece other than the first starts at the vector it begins with and has no head
        const uint64_t skip = i ? w.head + p.group0 * 16 : 0;
        const unsigned char* s = (const unsigned char*)in + skip;
        unsigned char* d = (unsigned char*)out + skip;
        g_last_kernel = "copy_kernel";
        if (nontemporal)
            hipLaunchKernelGGL(copy_kernel<true>, dim3(p.grid), dim3(kBlock), 0, stream, s, d, p.head, p.ngroup, p.tail);
        else
            hipLaunchKernelGGL(copy_kernel<false>, dim3(p.grid), dim3(kBlock), 0, stream, s, d, p.head, p.ngroup, p.tail);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess)
            return status_of(e);
    }
    return MI_CCL_SUCCESS;
}

// m >= 2 destinations; the vectors start where the first destination reaches a 16-byte boundary (a 128-byte line when
// the buffer is large)
static int launch_broadcast(const void* in, void* const* dsts, int m, size_t bytes, hipStream_t stream) {
    const uint32_t boundary = bytes >= kLineStartBytes && g_line_start.load(std::memory_order_relaxed) ? kLineBytes : 16u;
    const BcastShape b = bcast_shape((uintptr_t)dsts[0], bytes, kBcastSect, boundary);
    const uint64_t limit = block_limit(), n = bcast_num_launches(b, m, limit);
    for (uint64_t i = 0; i < n; i++) {
        const BcastPiece p = bcast_piece(b, m, limit, i);
        const uint64_t skip = i ? b.head + p.vec0 * 16 : 0;
        DstTable d;
        for (int k = 0; k < kMaxDsts; k++) d.p[k] = (unsigned char*)dsts[k < m ? k : 0] + skip;
        g_last_kernel = "broadcast_kernel";
        hipLaunchKernelGGL(broadcast_kernel, dim3(p.grid), dim3(kBlock), 0, stream, (const unsigned char*)in + skip, d, m,
                           p.head, p.nvec, p.tail, b.sect_tiles);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess)
            return status_of(e);
    }
    return MI_CCL_SUCCESS;
}

// The array converters: `per` elements per lane, vectors from the output's first 16-byte boundary on; launch(p, skip)
// enqueues one piece whose arrays start `skip` elements in.
template <class F>
static int launch_converter(const void* out, uint32_t out_elem_bytes, size_t count, uint32_t per, F&& launch) {
    const LaneWork w = lane_work((uintptr_t)out, out_elem_bytes, count, per);
    const uint64_t limit = block_limit(), n = num_launches(w, kBlock, limit);
    for (uint64_t i = 0; i < n; i++) {
        const LaunchPiece p = launch_piece(w, kBlock, limit, i);
        launch(p, i ? w.head + p.group0 * per : 0);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess)
            return status_of(e);
    }
    return MI_CCL_SUCCESS;
}

}  // namespace mi

extern "C" {

int mi_ccl_comp_copy(const void* in, void* out, size_t bytes, int use_nontemporal, void* stream) {
    if (bytes == 0)
        return MI_CCL_SUCCESS;
    if (!in || !out)
        return MI_CCL_INVALID_ARGUMENTS;
    return launch_copy(in, out, bytes, use_nontemporal != 0, (hipStream_t)stream);
}

int mi_ccl_convert_fp32_to_bf16_arrays(const void* fp32_buf, void* bf16_buf, size_t count, int bf16_impl,
                                       void* stream) {
    if (count == 0)
        return MI_CCL_SUCCESS;
    if (!fp32_buf || !bf16_buf || bf16_impl < MI_CCL_BF16_SCALAR || bf16_impl > MI_CCL_BF16_AVX512BF)
        return MI_CCL_INVALID_ARGUMENTS;
    if (((uintptr_t)fp32_buf & 3u) || ((uintptr_t)bf16_buf & 1u))
        return MI_CCL_INVALID_ARGUMENTS;
    static_assert(kCvtUnroll == 1 && kWidenUnroll == 1, "one group per lane, as the launch geometry assumes");
    const uint64_t rne_limit = bf16_impl == MI_CCL_BF16_AVX512BF ? count - count % 16 : 0;
    return launch_converter(bf16_buf, 2, count, 8, [&](const LaunchPiece& p, uint64_t skip) {
        const uint32_t* s = (const uint32_t*)fp32_buf + skip;
        uint16_t* d = (uint16_t*)bf16_buf + skip;
        const uint64_t lim = rne_limit > skip ? rne_limit - skip : 0;      // first truncated element, as this piece counts
        if (bf16_impl == MI_CCL_BF16_AVX512BF)
            hipLaunchKernelGGL(f32_to_bf16_kernel<true>, dim3(p.grid), dim3(kBlock), 0, (hipStream_t)stream, s, d, p.head,
                               p.ngroup, p.tail, lim);
        else
            hipLaunchKernelGGL(f32_to_bf16_kernel<false>, dim3(p.grid), dim3(kBlock), 0, (hipStream_t)stream, s, d, p.head,
                               p.ngroup, p.tail, (uint64_t)0);
    });
}

int mi_ccl_convert_bf16_to_fp32_arrays(const void* bf16_buf, void* fp32_buf, size_t count, void* stream) {
    if (count == 0)
        return MI_CCL_SUCCESS;
    if (!fp32_buf || !bf16_buf || ((uintptr_t)fp32_buf & 3u) || ((uintptr_t)bf16_buf & 1u))
        return MI_CCL_INVALID_ARGUMENTS;
    return launch_converter(fp32_buf, 4, count, 4, [&](const LaunchPiece& p, uint64_t skip) {
        hipLaunchKernelGGL(bf16_to_f32_kernel, dim3(p.grid), dim3(kBlock), 0, (hipStream_t)stream,
                           (const uint16_t*)bf16_buf + skip, (uint32_t*)fp32_buf + skip, p.head, p.ngroup, p.tail);
    });
}

int mi_ccl_convert_fp32_to_fp16_arrays(const void* fp32_buf, void* fp16_buf, size_t count, void* stream) {
    if (count == 0)
        return MI_CCL_SUCCESS;
    if (!fp32_buf || !fp16_buf || ((uintptr_t)fp32_buf & 3u) || ((uintptr_t)fp16_buf & 1u))
        return MI_CCL_INVALID_ARGUMENTS;
    return launch_converter(fp16_buf, 2, count, 8, [&](const LaunchPiece& p, uint64_t skip) {
        hipLaunchKernelGGL(f32_to_f16_kernel, dim3(p.grid), dim3(kBlock), 0, (hipStream_t)stream,
                           (const uint32_t*)fp32_buf + skip, (uint16_t*)fp16_buf + skip, p.head, p.ngroup, p.tail);
    });
}

int mi_ccl_convert_fp16_to_fp32_arrays(const void* fp16_buf, void* fp32_buf, size_t count, void* stream) {
    if (count == 0)
        return MI_CCL_SUCCESS;
    if (!fp32_buf || !fp16_buf || ((uintptr_t)fp32_buf & 3u) || ((uintptr_t)fp16_buf & 1u))
        return MI_CCL_INVALID_ARGUMENTS;
    return launch_converter(fp32_buf, 4, count, 4, [&](const LaunchPiece& p, uint64_t skip) {
        hipLaunchKernelGGL(f16_to_f32_kernel, dim3(p.grid), dim3(kBlock), 0, (hipStream_t)stream,
                           (const uint16_t*)fp16_buf + skip, (uint32_t*)fp32_buf + skip, p.head, p.ngroup, p.tail);
    });
}

const char* mi_ccl_last_kernel(void) {
    return g_last_kernel;
}

int mi_ccl_set_param(const char* name, long value) {
    if (!name)
        return MI_CCL_INVALID_ARGUMENTS;
    if (!strcmp(name, "waves_per_cu") && value >= 1 && value <= 65536) {
        g_waves_per_cu.store((int)value);
        return MI_CCL_SUCCESS;
    }
    if (!strcmp(name, "max_blocks") && value >= 0 && value <= (1 << 24)) {
        g_max_blocks.store((int)value);
        return MI_CCL_SUCCESS;
    }
    if (!strcmp(name, "xcd_chunked") && (value == 0 || value == 1)) {
        g_xcd_chunked.store((int)value);
        return MI_CCL_SUCCESS;
    }
    if (!strcmp(name, "variant") && (value == 0 || value == 1 || value == 2 || value == 4 || value == 8)) {
        g_variant.store((int)value);
        return MI_CCL_SUCCESS;
    }
    if (!strcmp(name, "phased_min_bytes") && value >= 0) {
        g_phased_min_bytes.store(value);
        return MI_CCL_SUCCESS;
    }
    if (!strcmp(name, "phase_early_loads") && value >= -1 && value <= 4096) {
        g_phase_early_loads.store((int)value);
        return MI_CCL_SUCCESS;
    }
    if (!strcmp(name, "phase_early_stores") && value >= -1 && value <= kPhaseU) {
        g_phase_early_stores.store((int)value);
        return MI_CCL_SUCCESS;
    }
    if (!strcmp(name, "phase_spin_ticks") && value >= 0 && value <= 100000000) {
        g_phase_spin_ticks.store(value);
        return MI_CCL_SUCCESS;
    }
    if (!strcmp(name, "fp16_impl") && value >= MI_CCL_FP16_F16C && value <= MI_CCL_FP16_AVX512FP16) {
        g_fp16_impl.store((int)value);
        return MI_CCL_SUCCESS;
    }
    if (!strcmp(name, "launch_block_limit") && value >= 0) {
        g_launch_block_limit.store(value);
        return MI_CCL_SUCCESS;
    }
    if (!strcmp(name, "realign") && (value == 0 || value == 1)) {
        g_realign.store((int)value);
        return MI_CCL_SUCCESS;
    }
    if (!strcmp(name, "line_start") && (value == 0 || value == 1)) {
        g_line_start.store((int)value);
        return MI_CCL_SUCCESS;
    }
    if (!strcmp(name, "phase_write_pace") && (value == 0 || (value >= 100 && value <= 100000))) {
        g_write_pace.store((int)value);
        return MI_CCL_SUCCESS;
    }
    if (!strcmp(name, "wave_runs") && value >= 0 && value <= 2) {
        g_wave_runs.store((int)value);
        return MI_CCL_SUCCESS;
    }
    return MI_CCL_INVALID_ARGUMENTS;
}

long mi_ccl_get_param(const char* name) {
    if (!name)
        return -1;
    if (!strcmp(name, "waves_per_cu"))
        return g_waves_per_cu.load();
    if (!strcmp(name, "max_blocks"))
        return g_max_blocks.load();
    if (!strcmp(name, "xcd_chunked"))
        return g_xcd_chunked.load();
    if (!strcmp(name, "variant"))
        return g_variant.load();
    if (!strcmp(name, "phased_min_bytes"))
        return g_phased_min_bytes.load();
    if (!strcmp(name, "phase_early_loads"))
        return g_phase_early_loads.load();
    if (!strcmp(name, "phase_early_stores"))
        return g_phase_early_stores.load();
    if (!strcmp(name, "phase_spin_ticks"))
        return g_phase_spin_ticks.load();
    if (!strcmp(name, "fp16_impl"))
        return g_fp16_impl.load();
    if (!strcmp(name, "launch_block_limit"))
        return g_launch_block_limit.load();
    if (!strcmp(name, "num_cus"))
        return num_cus();
    if (!strcmp(name, "realign"))
        return g_realign.load();
    if (!strcmp(name, "realigned_launches"))
        return (long)g_realigned_launches;
    if (!strcmp(name, "wide_phase_launches"))
        return (long)g_wide_phase_launches;
    if (!strcmp(name, "line_start"))
        return g_line_start.load();
    if (!strcmp(name, "wave_runs"))
        return g_wave_runs.load();
    if (!strcmp(name, "phase_write_pace"))
        return g_write_pace.load();
    if (!strcmp(name, "wall_clock_khz"))
        return wall_khz();
    return -1;
}

} /* extern "C" */
