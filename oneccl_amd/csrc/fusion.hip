// Fusion plans and the extern "C" fusion entry points of libmi_ccl_comp.so.
#include <hip/hip_runtime.h>

#include <atomic>
#include <new>
#include <stdexcept>
#include <vector>

#include "../../include/mi_ccl_comp.h"
#include "fusion_kernels.hpp"
#include "launch_geometry.hpp"

namespace mi {

Tuning current_tuning();

#define MI_DECLARE_FUSION(TR) extern template hipError_t launch_fusion_reduce<TR>(const FusionLaunchArgs&)
MI_DECLARE_FUSION(I8Traits);
MI_DECLARE_FUSION(U8Traits);
MI_DECLARE_FUSION(I16Traits);
MI_DECLARE_FUSION(U16Traits);
MI_DECLARE_FUSION(I32Traits);
MI_DECLARE_FUSION(U32Traits);
MI_DECLARE_FUSION(I64Traits);
MI_DECLARE_FUSION(U64Traits);
MI_DECLARE_FUSION(F32Traits);
MI_DECLARE_FUSION(F64Traits);
MI_DECLARE_FUSION(Fp16PairwiseTraits);
MI_DECLARE_FUSION(Fp16NativeTraits);
typedef Bf16PairwiseTraits<false, false> Bf16PairScalar;
typedef Bf16PairwiseTraits<false, true> Bf16PairAvx512f;
typedef Bf16PairwiseTraits<true, true> Bf16PairAvx512bf;
MI_DECLARE_FUSION(Bf16PairScalar);
MI_DECLARE_FUSION(Bf16PairAvx512f);
MI_DECLARE_FUSION(Bf16PairAvx512bf);
MI_DECLARE_FUSION(Bf16KeepTraits<false>);
MI_DECLARE_FUSION(Bf16KeepTraits<true>);

static int fusion_status_of(hipError_t e) {
    if (e == hipSuccess)
        return MI_CCL_SUCCESS;
    if (e == hipErrorOutOfMemory)
        return MI_CCL_OUT_OF_RESOURCE;
    if (e == hipErrorInvalidValue)
        return MI_CCL_INVALID_ARGUMENTS;
    return MI_CCL_RUNTIME_ERROR;
}

static size_t fusion_dtype_size(int dtype) {
    static const size_t sz[MI_CCL_DATATYPE_LAST] = { 1, 1, 2, 2, 4, 4, 8, 8, 2, 4, 8, 2 };
    return (dtype >= 0 && dtype < MI_CCL_DATATYPE_LAST) ? sz[dtype] : 0;
}

// Pack and unpack.  A block copies one 4 KiB quarter of a work item with one vector per lane -- a wave issues one load
// and one store and ends, the shape in which writes run fastest (as in copy_kernel) -- and the four blocks of an item
// read the same descriptor.  Only one pointer table travels with the launch (the tensors; the fusion buffer is one
// pointer), so it holds kFusionCopyGroup tensors: the 256 tensors of a typical bucket are one launch.  Measured on the
// 256-tensor configuration (191 MB of payload): 61.8 us against 68.4 us for 16 KiB per block in two launches, and
// 58.3 us for a plain copy of as many bytes.
//
// The quarters are cut where the DESTINATION crosses a 128-byte line, not at multiples of 4 KiB of the tensor: in a
// tightly packed fusion buffer behind an odd-sized tensor the two differ, and quarters cut by tensor offset would each
// start and end inside a line (and inside a vector: up to 15 single-byte stores at either end) that the neighbouring
// block writes too.  Quarter 0 is short by what the destination lacks to its first line boundary, the tensor's last
// quarter takes the rest (at most 127 bytes more than 4 KiB, so a few lanes copy a second vector).
constexpr int kFusionCopyGroup = 448;
constexpr uint32_t kFusionCopySub = kCopyQuarter;  // bytes per block
static_assert(kFusionChunk % kFusionCopySub == 0 && kFusionCopySub == 16 * kBlock, "an item is a whole number of block-sized quarters");
struct FusionCopyPtrs {
    const void* p[kFusionCopyGroup];
};

// to_fusion != 0: tensors -> fusion buffer (pack); else fusion buffer -> tensors (unpack)
__global__ void __launch_bounds__(kBlock)
fusion_copy_kernel(FusionCopyPtrs tensors, unsigned char* fusion_buf, const uint64_t* off, const uint64_t* bytes,
                   const FusionItem* items, uint32_t t0, int to_fusion) {
    constexpr uint32_t kSubs = kFusionChunk / kFusionCopySub;
    const uint32_t tid = threadIdx.x;
    const FusionItem w = items[blockIdx.x / kSubs];
    unsigned char* tp = (unsigned char*)tensors.p[w.t - t0];
    unsigned char* fp = fusion_buf + off[w.t];
    const CopyQuarter cq = copy_quarter(bytes[w.t], (uint64_t)(uintptr_t)(to_fusion ? fp : tp),
                                        (uint64_t)w.c * kSubs + blockIdx.x % kSubs);
    const uint32_t n = cq.n;                        // at most 4 KiB + 127
    if (n == 0) return;                             // the last item's last quarters may be empty
    const unsigned char* src = (to_fusion ? tp : fp) + cq.lo;
    unsigned char* dst = (to_fusion ? fp : tp) + cq.lo;
    // vectors from the destination's first 16-byte boundary on, whatever the source's alignment is
    uint32_t head = (uint32_t)(-(intptr_t)dst) & 15u;
    if (head > n) head = n;
    const uint32_t nvec = (n - head) >> 4, tail = n - head - (nvec << 4);
    for (uint32_t v = tid; v < nvec; v += kBlock) st_loose((u32x4_u*)(dst + head) + v, ld_loose((const u32x4_u*)(src + head) + v));
    if (tid < head + tail) {
        const uint32_t i = (tid < head) ? tid : head + (nvec << 4) + (tid - head);
        dst[i] = src[i];
    }
}

// One fused reduce of the traits class that (dtype, 16-bit mode, bf16_impl, a.tune.fp16_impl) selects.
static hipError_t dispatch_fusion(int dtype, bool keep, int bf16_impl, const FusionLaunchArgs& a) {
    switch (dtype) {
        case MI_CCL_INT8: return launch_fusion_reduce<I8Traits>(a);
        case MI_CCL_UINT8: return launch_fusion_reduce<U8Traits>(a);
        case MI_CCL_INT16: return launch_fusion_reduce<I16Traits>(a);
        case MI_CCL_UINT16: return launch_fusion_reduce<U16Traits>(a);
        case MI_CCL_INT32: return launch_fusion_reduce<I32Traits>(a);
        case MI_CCL_UINT32: return launch_fusion_reduce<U32Traits>(a);
        case MI_CCL_INT64: return launch_fusion_reduce<I64Traits>(a);
        case MI_CCL_UINT64: return launch_fusion_reduce<U64Traits>(a);
        case MI_CCL_FLOAT16:
            return a.tune.fp16_impl == MI_CCL_FP16_AVX512FP16 ? launch_fusion_reduce<Fp16NativeTraits>(a)
                                                              : launch_fusion_reduce<Fp16PairwiseTraits>(a);
        case MI_CCL_FLOAT32: return launch_fusion_reduce<F32Traits>(a);
        case MI_CCL_FLOAT64: return launch_fusion_reduce<F64Traits>(a);
        case MI_CCL_BFLOAT16:
            if (keep)
                return (bf16_impl == MI_CCL_BF16_AVX512BF) ? launch_fusion_reduce<Bf16KeepTraits<true>>(a)
                                                            : launch_fusion_reduce<Bf16KeepTraits<false>>(a);
            if (bf16_impl == MI_CCL_BF16_SCALAR)
                return launch_fusion_reduce<Bf16PairScalar>(a);
            if (bf16_impl == MI_CCL_BF16_AVX512F)
                return launch_fusion_reduce<Bf16PairAvx512f>(a);
            return launch_fusion_reduce<Bf16PairAvx512bf>(a);
        default: return hipErrorInvalidValue;
    }
}

// ---------------------------------------------------------------------------------------------------
// The fused reduce for callers that cannot allocate: its work table (the per-tensor offset and size tables and the
// item list that a plan keeps in memory of its own) lives in a file-scope device array and is written by a small
// kernel on the caller's stream in front of the reduce kernels.  Every GPU holds its own copy of the array at its own
// address, looked up once per device with that device current; host code only ever uses that looked-up address.

struct StaticFusionTable {
    uint64_t off[MI_CCL_FUSION_STATIC_MAX_TENSORS];
    uint64_t bytes[MI_CCL_FUSION_STATIC_MAX_TENSORS];
    uint32_t tile_end[MI_CCL_FUSION_STATIC_MAX_TENSORS];
    FusionItem items[MI_CCL_FUSION_STATIC_MAX_ITEMS];
};
// kStaticSlots tables per GPU, taken in turn by the calls on that GPU: a call's table is rewritten by the call that
// comes kStaticSlots calls later, so up to that many calls may be in flight on different streams (or sit in graphs
// that replay side by side) before two of them share a table.
constexpr int kStaticSlots = 4;
static __device__ __align__(256) unsigned char scratch[kStaticSlots * sizeof(StaticFusionTable)];
static_assert(sizeof(StaticFusionTable) % 256 == 0, "every table of the array starts on a 256-byte boundary");
static std::atomic<StaticFusionTable*> g_scratch_ptr[64];
static std::atomic<unsigned> g_scratch_next[64];

static hipError_t scratch_table(StaticFusionTable** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return e;
    if (dev < 0 || dev >= 64)
        return hipErrorInvalidDevice;
    StaticFusionTable* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess)
            return e;
        p = (StaticFusionTable*)ptr;
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *out = p + g_scratch_next[dev].fetch_add(1, std::memory_order_relaxed) % kStaticSlots;
    return hipSuccess;
}

struct FusionSizes {                // by-value kernel argument: the sizes of one launch group of tensors, in bytes
    uint64_t bytes[kFusionGroup];
};

// Block b writes the table rows of tensor t0 + b: its byte offset in the fusion buffer (running end rounded up to
// `align`, from `end0`, the end of the tensor before the group), its size, and its work items from item index
// `item0` + (items of the group's tensors before it), and the running count of kFusionTile-byte tiles through it.  Every lane walks the (at most kFusionGroup) sizes before its
// tensor; they are kernel arguments, so the walk is scalar work.
__global__ void __launch_bounds__(kBlock)
fusion_table_kernel(FusionSizes sz, uint32_t t0, uint64_t end0, uint64_t align, uint64_t item0, uint64_t tile0,
                    StaticFusionTable* tab) {
    const uint32_t b = blockIdx.x;
    uint64_t end = end0, item = item0, tile = tile0;
    for (uint32_t u = 0; u < b; u++) {
        end = ((end + align - 1) & ~(align - 1)) + sz.bytes[u];
        item += (sz.bytes[u] + kFusionChunk - 1) / kFusionChunk;
        tile += (sz.bytes[u] + kFusionTile - 1) / kFusionTile;
    }
    const uint64_t off = (end + align - 1) & ~(align - 1);
    const uint64_t nb = sz.bytes[b];
    if (threadIdx.x == 0) {
        tab->off[t0 + b] = off;
        tab->bytes[t0 + b] = nb;
        tab->tile_end[t0 + b] = (uint32_t)(tile + (nb + kFusionTile - 1) / kFusionTile);
    }
    const uint64_t chunks = (nb + kFusionChunk - 1) / kFusionChunk;
    for (uint64_t c = threadIdx.x; c < chunks; c += kBlock) tab->items[item + c] = FusionItem{ t0 + b, (uint32_t)c };
}

}  // namespace mi

using namespace mi;

struct mi_ccl_fusion_plan {
    size_t k = 0;
    int dtype = 0;
    size_t esz = 0;
    size_t align = 1;
    size_t total_bytes = 0;
    std::vector<size_t> counts;
    std::vector<size_t> offsets;           // bytes
    std::vector<uint64_t> item_begin;      // k + 1
    std::vector<uint64_t> tile_begin;      // k + 1: tiles of kFusionTile bytes
    void* d_table = nullptr;               // [off: k x u64][bytes: k x u64][items][tile_end: k x u32]
    const uint64_t* d_off = nullptr;
    const uint64_t* d_bytes = nullptr;
    const FusionItem* d_items = nullptr;
    const uint32_t* d_tile_end = nullptr;
};

extern "C" {

int mi_ccl_fusion_offsets(const size_t* counts, size_t k, size_t dtype_size, size_t align, size_t* byte_offsets,
                          size_t* total_bytes) {
    if (dtype_size == 0 || align == 0 || (align & (align - 1)) != 0 || (k && (!counts || !byte_offsets)))
        return MI_CCL_INVALID_ARGUMENTS;
    size_t end = 0;
    for (size_t i = 0; i < k; i++) {
        size_t off = (end + align - 1) & ~(align - 1);
        byte_offsets[i] = off;
        end = off + counts[i] * dtype_size;
    }
    if (total_bytes)
        *total_bytes = end;
    return MI_CCL_SUCCESS;
}

// The host tables of a plan are std::vectors, so building one may throw; the entry point below turns that into a status.
static int plan_build(mi_ccl_fusion_plan* p, const size_t* counts, size_t k, int dtype, size_t esz, size_t align) {
    p->k = k;
    p->dtype = dtype;
    p->esz = esz;
    p->align = align;
    p->counts.assign(counts, counts + k);
    p->offsets.resize(k);
    mi_ccl_fusion_offsets(counts, k, esz, align, p->offsets.data(), &p->total_bytes);
    p->item_begin.resize(k + 1);
    std::vector<FusionItem> items;
    for (size_t t = 0; t < k; t++) {
        p->item_begin[t] = items.size();
        const uint64_t bytes = (uint64_t)counts[t] * esz;
        const uint64_t chunks = (bytes + kFusionChunk - 1) / kFusionChunk;
        if (chunks > 0xffffffffull || t > 0xffffffffull || items.size() + chunks > 0x7fffffffull)
            return MI_CCL_INVALID_ARGUMENTS;
        for (uint64_t c = 0; c < chunks; c++) items.push_back(FusionItem{ (uint32_t)t, (uint32_t)c });
    }
    p->item_begin[k] = items.size();
    std::vector<uint64_t> host(2 * k);
    std::vector<uint32_t> tile_end(k);
    p->tile_begin.resize(k + 1);
    p->tile_begin[0] = 0;
    for (size_t t = 0; t < k; t++) {
        host[t] = p->offsets[t];
        host[k + t] = (uint64_t)counts[t] * esz;
        p->tile_begin[t + 1] = p->tile_begin[t] + (host[k + t] + kFusionTile - 1) / kFusionTile;
        tile_end[t] = (uint32_t)p->tile_begin[t + 1];       // fits: there are no more tiles than items
    }
    const size_t items_bytes = (items.size() ? items.size() : 1) * sizeof(FusionItem);
    const size_t table_bytes = 2 * k * sizeof(uint64_t) + items_bytes + k * sizeof(uint32_t);
    hipError_t e = hipMalloc(&p->d_table, table_bytes);
    if (e != hipSuccess) {
        p->d_table = nullptr;
        return fusion_status_of(e);
    }
    e = hipMemcpy(p->d_table, host.data(), 2 * k * sizeof(uint64_t), hipMemcpyHostToDevice);
    if (e == hipSuccess && !items.empty())
        e = hipMemcpy((char*)p->d_table + 2 * k * sizeof(uint64_t), items.data(), items.size() * sizeof(FusionItem),
                      hipMemcpyHostToDevice);
    if (e == hipSuccess)
        e = hipMemcpy((char*)p->d_table + 2 * k * sizeof(uint64_t) + items_bytes, tile_end.data(), k * sizeof(uint32_t),
                      hipMemcpyHostToDevice);
    if (e != hipSuccess)
        return fusion_status_of(e);
    p->d_off = (const uint64_t*)p->d_table;
    p->d_bytes = p->d_off + k;
    p->d_items = (const FusionItem*)(p->d_bytes + k);
    p->d_tile_end = (const uint32_t*)((const char*)p->d_items + items_bytes);
    return MI_CCL_SUCCESS;
}

int mi_ccl_fusion_plan_create(const size_t* counts, size_t k, int dtype, size_t align, mi_ccl_fusion_plan** plan) {
    if (!plan)
        return MI_CCL_INVALID_ARGUMENTS;
    *plan = nullptr;
    const size_t esz = fusion_dtype_size(dtype);
    if (esz == 0 || k == 0 || !counts || align == 0 || (align & (align - 1)) != 0)
        return MI_CCL_INVALID_ARGUMENTS;
    mi_ccl_fusion_plan* p = new (std::nothrow) mi_ccl_fusion_plan;
    if (!p)
        return MI_CCL_OUT_OF_RESOURCE;
    int rc;
    try {
        rc = plan_build(p, counts, k, dtype, esz, align);
    }
    catch (const std::exception&) {     // bad_alloc, length_error: out of host memory for the tables
        rc = MI_CCL_OUT_OF_RESOURCE;
    }
    if (rc != MI_CCL_SUCCESS) {
        if (p->d_table)
            (void)hipFree(p->d_table);
        delete p;
        return rc;
    }
    *plan = p;
    return MI_CCL_SUCCESS;
}

int mi_ccl_fusion_plan_destroy(mi_ccl_fusion_plan* plan) {
    if (!plan)
        return MI_CCL_SUCCESS;
    hipError_t e = plan->d_table ? hipFree(plan->d_table) : hipSuccess;
    delete plan;
    return fusion_status_of(e);
}

size_t mi_ccl_fusion_plan_bytes(const mi_ccl_fusion_plan* plan) {
    return plan ? plan->total_bytes : 0;
}

size_t mi_ccl_fusion_plan_offset(const mi_ccl_fusion_plan* plan, size_t i) {
    return (plan && i < plan->k) ? plan->offsets[i] : (size_t)-1;
}

static int fusion_copy(mi_ccl_fusion_plan* plan, const void* const* tensors, void* fusion_buf, void* stream,
                       int to_fusion) {
    if (!plan || !tensors || (!fusion_buf && plan->total_bytes))
        return MI_CCL_INVALID_ARGUMENTS;
    for (size_t t = 0; t < plan->k; t++)
        if (!tensors[t] && plan->counts[t])
            return MI_CCL_INVALID_ARGUMENTS;
    constexpr uint32_t kSubs = kFusionChunk / kFusionCopySub;
    const uint64_t max_items = hip_block_limit(kBlock) / kSubs;       // items one launch may take
    for (size_t t0 = 0; t0 < plan->k; t0 += kFusionCopyGroup) {
        const size_t t1 = (t0 + kFusionCopyGroup < plan->k) ? t0 + kFusionCopyGroup : plan->k;
        FusionCopyPtrs ptrs;
        for (size_t t = t0; t < t1; t++) ptrs.p[t - t0] = tensors[t];
        for (uint64_t i0 = plan->item_begin[t0]; i0 < plan->item_begin[t1]; i0 += max_items) {
            const uint64_t i1 = (i0 + max_items < plan->item_begin[t1]) ? i0 + max_items : plan->item_begin[t1];
            g_last_kernel = "fusion_copy_kernel";
            hipLaunchKernelGGL(fusion_copy_kernel, dim3((unsigned)((i1 - i0) * kSubs)), dim3(kBlock), 0, (hipStream_t)stream,
                               ptrs, (unsigned char*)fusion_buf, plan->d_off, plan->d_bytes, plan->d_items + i0, (uint32_t)t0,
                               to_fusion);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess)
                return fusion_status_of(e);
        }
    }
    return MI_CCL_SUCCESS;
}

int mi_ccl_fusion_pack(mi_ccl_fusion_plan* plan, const void* const* tensors, void* fusion_buf, void* stream) {
    return fusion_copy(plan, tensors, fusion_buf, stream, 1);
}

int mi_ccl_fusion_unpack(mi_ccl_fusion_plan* plan, const void* fusion_buf, void* const* tensors, void* stream) {
    return fusion_copy(plan, (const void* const*)tensors, (void*)fusion_buf, stream, 0);
}

int mi_ccl_fusion_reduce(mi_ccl_fusion_plan* plan, int op, const void* const* own_tensors, const void* const* peers,
                         int n_peers, void* const* out_tensors, int lp_mode, int bf16_impl, int fp16_impl, void* stream) {
    if (!plan || !own_tensors || !out_tensors || n_peers < 0 || n_peers > kFusionMaxPeers || (n_peers && !peers))
        return MI_CCL_INVALID_ARGUMENTS;
    if (op < MI_CCL_SUM || op > MI_CCL_MAX || bf16_impl < MI_CCL_BF16_SCALAR || bf16_impl > MI_CCL_BF16_AVX512BF)
        return MI_CCL_INVALID_ARGUMENTS;
    if (fp16_impl != MI_CCL_FP16_DEFAULT && (fp16_impl < MI_CCL_FP16_F16C || fp16_impl > MI_CCL_FP16_AVX512FP16))
        return MI_CCL_INVALID_ARGUMENTS;
    const bool keep = (lp_mode & MI_CCL_LP_KEEP_PRECISION) != 0;
    // the truncated tail of the array converter belongs to the end of the *fused* buffer; this entry point
    // narrows every element the same way
    if ((lp_mode & ~MI_CCL_LP_KEEP_PRECISION) != 0 || (keep && plan->dtype != MI_CCL_BFLOAT16))
        return MI_CCL_INVALID_ARGUMENTS;
    for (size_t t = 0; t < plan->k; t++) {
        if (plan->counts[t] == 0)
            continue;
        if (!own_tensors[t] || !out_tensors[t] || ((uintptr_t)own_tensors[t] % plan->esz) ||
            ((uintptr_t)out_tensors[t] % plan->esz))
            return MI_CCL_INVALID_ARGUMENTS;
    }
    for (int j = 0; j < n_peers; j++)
        if (!peers[j] || ((uintptr_t)peers[j] % plan->esz))
            return MI_CCL_INVALID_ARGUMENTS;

    FusionLaunchArgs a;
    a.own = own_tensors;
    a.out = out_tensors;
    a.peers = peers;
    a.n_peers = n_peers;
    a.op = op;
    a.k = plan->k;
    a.d_off = plan->d_off;
    a.d_bytes = plan->d_bytes;
    a.d_items = plan->d_items;
    a.d_tile_end = plan->d_tile_end;
    a.item_begin = plan->item_begin.data();
    a.tile_begin = plan->tile_begin.data();
    a.stream = (hipStream_t)stream;
    a.tune = current_tuning();
    if (fp16_impl != MI_CCL_FP16_DEFAULT)
        a.tune.fp16_impl = fp16_impl;
    return fusion_status_of(dispatch_fusion(plan->dtype, keep, bf16_impl, a));
}

int mi_ccl_fusion_reduce_static(const size_t* counts, size_t k, int dtype, size_t align, int op,
                                const void* const* own_tensors, const void* const* peers, int n_peers,
                                void* const* out_tensors, int lp_mode, int bf16_impl, int fp16_impl, void* stream) {
    const size_t esz = fusion_dtype_size(dtype);
    if (esz == 0 || k == 0 || !counts || align == 0 || (align & (align - 1)) != 0)
        return MI_CCL_INVALID_ARGUMENTS;
    if (!own_tensors || !out_tensors || n_peers < 0 || n_peers > kFusionMaxPeers || (n_peers && !peers))
        return MI_CCL_INVALID_ARGUMENTS;
    if (op < MI_CCL_SUM || op > MI_CCL_MAX || bf16_impl < MI_CCL_BF16_SCALAR || bf16_impl > MI_CCL_BF16_AVX512BF)
        return MI_CCL_INVALID_ARGUMENTS;
    if (fp16_impl != MI_CCL_FP16_DEFAULT && (fp16_impl < MI_CCL_FP16_F16C || fp16_impl > MI_CCL_FP16_AVX512FP16))
        return MI_CCL_INVALID_ARGUMENTS;
    const bool keep = (lp_mode & MI_CCL_LP_KEEP_PRECISION) != 0;
    if ((lp_mode & ~MI_CCL_LP_KEEP_PRECISION) != 0 || (keep && dtype != MI_CCL_BFLOAT16))
        return MI_CCL_INVALID_ARGUMENTS;
    if (k > MI_CCL_FUSION_STATIC_MAX_TENSORS)
        return MI_CCL_OUT_OF_RESOURCE;          // more tensors than the table holds
    uint64_t item_begin[MI_CCL_FUSION_STATIC_MAX_TENSORS + 1];      // on the stack: nothing is allocated here
    uint64_t tile_begin[MI_CCL_FUSION_STATIC_MAX_TENSORS + 1];
    uint64_t items = 0, tiles = 0;
    for (size_t t = 0; t < k; t++) {
        item_begin[t] = items;
        tile_begin[t] = tiles;
        if (counts[t] > ((uint64_t)1 << 40) / esz)
            return MI_CCL_OUT_OF_RESOURCE;
        items += ((uint64_t)counts[t] * esz + kFusionChunk - 1) / kFusionChunk;
        tiles += ((uint64_t)counts[t] * esz + kFusionTile - 1) / kFusionTile;
        if (items > MI_CCL_FUSION_STATIC_MAX_ITEMS)
            return MI_CCL_OUT_OF_RESOURCE;      // more payload than the item list holds
        if (counts[t] == 0)
            continue;
        if (!own_tensors[t] || !out_tensors[t] || ((uintptr_t)own_tensors[t] % esz) || ((uintptr_t)out_tensors[t] % esz))
            return MI_CCL_INVALID_ARGUMENTS;
    }
    item_begin[k] = items;
    tile_begin[k] = tiles;
    for (int j = 0; j < n_peers; j++)
        if (!peers[j] || ((uintptr_t)peers[j] % esz))
            return MI_CCL_INVALID_ARGUMENTS;
    if (items == 0)
        return MI_CCL_SUCCESS;

    StaticFusionTable* tab = nullptr;
    hipError_t e = scratch_table(&tab);
    if (e != hipSuccess)
        return fusion_status_of(e);
    // the table first: one small launch per group of kFusionGroup tensors, in stream order before the reduce
    uint64_t end = 0;
    for (size_t t0 = 0; t0 < k; t0 += kFusionGroup) {
        const size_t t1 = (t0 + kFusionGroup < k) ? t0 + kFusionGroup : k;
        FusionSizes sz;
        for (size_t t = t0; t < t1; t++) sz.bytes[t - t0] = (uint64_t)counts[t] * esz;
        hipLaunchKernelGGL(fusion_table_kernel, dim3((unsigned)(t1 - t0)), dim3(kBlock), 0, (hipStream_t)stream, sz,
                           (uint32_t)t0, end, (uint64_t)align, item_begin[t0], tile_begin[t0], tab);
        e = hipGetLastError();
        if (e != hipSuccess)
            return fusion_status_of(e);
        for (size_t t = t0; t < t1; t++) end = ((end + align - 1) & ~((uint64_t)align - 1)) + sz.bytes[t - t0];
    }
    FusionLaunchArgs a;
    a.own = own_tensors;
    a.out = out_tensors;
    a.peers = peers;
    a.n_peers = n_peers;
    a.op = op;
    a.k = k;
    a.d_off = tab->off;             // address arithmetic on the looked-up device address, no host access
    a.d_bytes = tab->bytes;
    a.d_items = tab->items;
    a.d_tile_end = tab->tile_end;
    a.item_begin = item_begin;
    a.tile_begin = tile_begin;
    a.stream = (hipStream_t)stream;
    a.tune = current_tuning();
    if (fp16_impl != MI_CCL_FP16_DEFAULT)
        a.tune.fp16_impl = fp16_impl;
    return fusion_status_of(dispatch_fusion(dtype, keep, bf16_impl, a));
}

} /* extern "C" */
