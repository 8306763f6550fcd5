// extern "C" layer of libmi_ccl_comp.so: argument checks, traits selection and the copy / converter
// kernels.  The reduce kernels themselves are instantiated one traits class per translation unit
// (inst_*.hip) from reduce_kernels.hpp.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <cctype>

#include "../../include/mi_ccl_comp.h"
#include "reduce_kernels.hpp"

namespace mi {

#define MI_DECLARE(TR) extern template hipError_t launch_reduce<TR>(const LaunchArgs&)
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

static std::atomic<int> g_waves_per_cu{ 256 };
static std::atomic<int> g_max_blocks{ 0 };
static std::atomic<int> g_xcd_chunked{ 0 };
static std::atomic<int> g_variant{ 0 };
static std::atomic<long> g_phased_min_bytes{ 160L << 20 };
static std::atomic<int> g_fp16_impl{ MI_CCL_FP16_AVX512F };
static std::atomic<int> g_num_cus[64];

// Barrier words of the phased kernel: one copy per device (each GPU holds its own instance of a
// __device__ variable at its own address), looked up once per device.
static __device__ PhaseSync g_phase_sync;
static std::atomic<PhaseSync*> g_phase_sync_ptr[64];

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
    return p;
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

Tuning current_tuning() {
    Tuning t;
    t.waves_per_cu = g_waves_per_cu.load(std::memory_order_relaxed);
    t.max_blocks = g_max_blocks.load(std::memory_order_relaxed);
    t.xcd_chunked = g_xcd_chunked.load(std::memory_order_relaxed);
    t.variant = g_variant.load(std::memory_order_relaxed);
    t.num_cus = num_cus();
    t.phased_min_bytes = g_phased_min_bytes.load(std::memory_order_relaxed);
    t.sync = phase_sync();
    t.fp16_impl = g_fp16_impl.load(std::memory_order_relaxed);
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

static int reduce_n_impl(int dtype, int op, const void* const* srcs, int n, void* const* dsts, int m, size_t count,
                         int lp_mode, int bf16_impl, void* stream) {
    if (count == 0)
        return MI_CCL_SUCCESS;
    if (m < 1 || m > kMaxDsts || !dsts)
        return MI_CCL_INVALID_ARGUMENTS;
    if (dtype < 0 || dtype >= MI_CCL_DATATYPE_LAST || op < MI_CCL_SUM || op > MI_CCL_MAX)
        return MI_CCL_INVALID_ARGUMENTS;
    if (n < 1 || n > kMaxSrcs || !srcs)
        return MI_CCL_INVALID_ARGUMENTS;
    if (bf16_impl < MI_CCL_BF16_SCALAR || bf16_impl > MI_CCL_BF16_AVX512BF)
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

    LaunchArgs a;
    a.srcs = srcs;
    a.n = n;
    a.dst = dsts[0];
    a.dsts = dsts;
    a.m = m;
    a.count = count;
    a.op = op;
    a.stream = (hipStream_t)stream;
    a.tune = current_tuning();

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

// Vectors from the output's first 16-byte boundary on; the input is read as loose vectors (any alignment).
template <bool NT>
__global__ void __launch_bounds__(kBlock)
copy_kernel(const unsigned char* in, unsigned char* out, uint32_t head, uint64_t nvec, uint32_t tail) {
    constexpr int UNROLL = 4;
    constexpr uint64_t kTile = (uint64_t)kBlock * UNROLL;
    const u32x4_u* s = (const u32x4_u*)(in + head);
    u32x4* d = (u32x4*)(out + head);
    const uint64_t ntiles = (nvec + kTile - 1) / kTile;
    for (uint64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const uint64_t base = tile * kTile + threadIdx.x;
        u32x4 x[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const uint64_t i = base + (uint64_t)u * kBlock;
            if (i < nvec)
                x[u] = NT ? ld_loose(s + i) : *(s + i);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const uint64_t i = base + (uint64_t)u * kBlock;
            if (i < nvec) {
                if (NT)
                    __builtin_nontemporal_store(x[u], d + i);
                else
                    d[i] = x[u];
            }
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < head + tail) {
        uint32_t t = threadIdx.x;
        uint64_t i = (t < head) ? t : (uint64_t)head + nvec * 16 + (t - head);
        out[i] = in[i];
    }
}

// fp32 -> bf16, four elements per lane; elements at or beyond rne_limit are truncated
template <bool RNE>
__global__ void __launch_bounds__(kBlock)
f32_to_bf16_kernel(const uint32_t* in, uint16_t* out, uint64_t count, uint64_t rne_limit, int vec_ok) {
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    const uint64_t nquad = vec_ok ? count / 4 : 0;
    for (uint64_t q = (uint64_t)blockIdx.x * kBlock + threadIdx.x; q < nquad; q += stride) {
        u32x4 x = __builtin_nontemporal_load((const u32x4*)in + q);
        uint32_t r[4];
        // the packed conversion the reduce kernels use (the element form serves the tail below)
        const uint32_t p01 = RNE ? bf16_narrow_rne_pack2(x[0], x[1]) : 0u, p23 = RNE ? bf16_narrow_rne_pack2(x[2], x[3]) : 0u;
        const uint32_t rne[4] = { p01 & 0xffffu, p01 >> 16, p23 & 0xffffu, p23 >> 16 };
#pragma unroll
        for (int k = 0; k < 4; k++) r[k] = (RNE && q * 4 + k < rne_limit) ? rne[k] : bf16_narrow_trunc(x[k]);
        uint2 o = make_uint2(r[0] | (r[1] << 16), r[2] | (r[3] << 16));
        ((uint2*)out)[q] = o;
    }
    for (uint64_t i = nquad * 4 + (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < count; i += stride) {
        uint32_t u = in[i];
        out[i] = (uint16_t)((RNE && i < rne_limit) ? bf16_narrow_rne(u) : bf16_narrow_trunc(u));
    }
}

__global__ void __launch_bounds__(kBlock)
bf16_to_f32_kernel(const uint16_t* in, uint32_t* out, uint64_t count, int vec_ok) {
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    const uint64_t nquad = vec_ok ? count / 4 : 0;
    for (uint64_t q = (uint64_t)blockIdx.x * kBlock + threadIdx.x; q < nquad; q += stride) {
        uint2 h = ((const uint2*)in)[q];
        u32x4 o = { h.x << 16, h.x & 0xffff0000u, h.y << 16, h.y & 0xffff0000u };
        __builtin_nontemporal_store(o, (u32x4*)out + q);
    }
    for (uint64_t i = nquad * 4 + (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < count; i += stride)
        out[i] = (uint32_t)in[i] << 16;
}

}  // namespace mi

using namespace mi;

extern "C" {

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

int mi_ccl_comp_reduce(int dtype, int op, const void* in, size_t count, void* inout, int bf16_impl, void* stream) {
    if (count == 0)
        return MI_CCL_SUCCESS;
    const void* srcs[2] = { inout, in };
    return reduce_n_impl(dtype, op, srcs, 2, &inout, 1, count, MI_CCL_LP_PAIRWISE, bf16_impl, stream);
}

int mi_ccl_bf16_reduce(const void* in, size_t count, void* inout, int op, int bf16_impl, void* stream) {
    return mi_ccl_comp_reduce(MI_CCL_BFLOAT16, op, in, count, inout, bf16_impl, stream);
}

int mi_ccl_fp16_reduce(const void* in, size_t count, void* inout, int op, void* stream) {
    return mi_ccl_comp_reduce(MI_CCL_FLOAT16, op, in, count, inout, MI_CCL_BF16_AVX512BF, stream);
}

int mi_ccl_comp_reduce_n(int dtype, int op, const void* const* srcs, int n, void* dst, size_t count, int lp_mode,
                         int bf16_impl, void* stream) {
    return reduce_n_impl(dtype, op, srcs, n, &dst, 1, count, lp_mode, bf16_impl, stream);
}

int mi_ccl_comp_reduce_write_n(int dtype, int op, const void* const* srcs, int n, void* const* dsts, int m, size_t count,
                               int lp_mode, int bf16_impl, void* stream) {
    return reduce_n_impl(dtype, op, srcs, n, dsts, m, count, lp_mode, bf16_impl, stream);
}

int mi_ccl_comp_batch_reduce(const void* in_buf, const size_t* offsets, size_t n_offsets, size_t count, void* inout,
                             int dtype, int op, int bf16_keep_precision_mode, int bf16_impl, void* stream) {
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
    return reduce_n_impl(dtype, op, srcs, (int)n_offsets, &inout, 1, count, lp, bf16_impl, stream);
}

int mi_ccl_comp_copy(const void* in, void* out, size_t bytes, int use_nontemporal, void* stream) {
    if (bytes == 0)
        return MI_CCL_SUCCESS;
    if (!in || !out)
        return MI_CCL_INVALID_ARGUMENTS;
    Tuning t = current_tuning();
    const uintptr_t mis = (uintptr_t)out & 15u;
    // very large copies go through the one-input reduce (a copy for plain types), whose phased form separates
    // reads from writes; below that the plain copy kernel is as fast
    if (t.sync && t.variant == 0 && 2 * (uint64_t)bytes >= 25 * (uint64_t)t.phased_min_bytes) {
        LaunchArgs a;
        const void* srcs[1] = { in };
        a.srcs = srcs;
        a.n = 1;
        a.dst = out;
        a.count = bytes;
        a.op = OP_SUM;
        a.stream = (hipStream_t)stream;
        a.tune = t;
        return status_of(launch_reduce<U8Traits>(a));
    }
    uint64_t head = mis ? 16u - mis : 0;
    if (head > bytes)
        head = bytes;
    const uint64_t nvec = (bytes - head) / 16;
    const uint32_t tail = (uint32_t)(bytes - head - nvec * 16);
    const uint64_t tile = (uint64_t)kBlock * 4;
    int grid = grid_for((nvec + tile - 1) / tile, t);
    if (use_nontemporal)
        hipLaunchKernelGGL(copy_kernel<true>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream,
                           (const unsigned char*)in, (unsigned char*)out, (uint32_t)head, nvec, tail);
    else
        hipLaunchKernelGGL(copy_kernel<false>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream,
                           (const unsigned char*)in, (unsigned char*)out, (uint32_t)head, nvec, tail);
    return status_of(hipGetLastError());
}

int mi_ccl_convert_fp32_to_bf16_arrays(const void* fp32_buf, void* bf16_buf, size_t count, int bf16_impl,
                                       void* stream) {
    if (count == 0)
        return MI_CCL_SUCCESS;
    if (!fp32_buf || !bf16_buf || bf16_impl < MI_CCL_BF16_SCALAR || bf16_impl > MI_CCL_BF16_AVX512BF)
        return MI_CCL_INVALID_ARGUMENTS;
    if (((uintptr_t)fp32_buf & 3u) || ((uintptr_t)bf16_buf & 1u))
        return MI_CCL_INVALID_ARGUMENTS;
    Tuning t = current_tuning();
    const int vec_ok = (((uintptr_t)fp32_buf & 15u) == 0) && (((uintptr_t)bf16_buf & 7u) == 0);
    int grid = grid_for((count / 4 + kBlock) / kBlock, t);
    if (bf16_impl == MI_CCL_BF16_AVX512BF)
        hipLaunchKernelGGL(f32_to_bf16_kernel<true>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream,
                           (const uint32_t*)fp32_buf, (uint16_t*)bf16_buf, (uint64_t)count,
                           (uint64_t)(count - count % 16), vec_ok);
    else
        hipLaunchKernelGGL(f32_to_bf16_kernel<false>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream,
                           (const uint32_t*)fp32_buf, (uint16_t*)bf16_buf, (uint64_t)count, (uint64_t)0, vec_ok);
    return status_of(hipGetLastError());
}

int mi_ccl_convert_bf16_to_fp32_arrays(const void* bf16_buf, void* fp32_buf, size_t count, void* stream) {
    if (count == 0)
        return MI_CCL_SUCCESS;
    if (!fp32_buf || !bf16_buf || ((uintptr_t)fp32_buf & 3u) || ((uintptr_t)bf16_buf & 1u))
        return MI_CCL_INVALID_ARGUMENTS;
    Tuning t = current_tuning();
    const int vec_ok = (((uintptr_t)fp32_buf & 15u) == 0) && (((uintptr_t)bf16_buf & 7u) == 0);
    int grid = grid_for((count / 4 + kBlock) / kBlock, t);
    hipLaunchKernelGGL(bf16_to_f32_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream,
                       (const uint16_t*)bf16_buf, (uint32_t*)fp32_buf, (uint64_t)count, vec_ok);
    return status_of(hipGetLastError());
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
    if (!strcmp(name, "fp16_impl") && value >= MI_CCL_FP16_F16C && value <= MI_CCL_FP16_AVX512FP16) {
        g_fp16_impl.store((int)value);
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
    if (!strcmp(name, "fp16_impl"))
        return g_fp16_impl.load();
    if (!strcmp(name, "num_cus"))
        return num_cus();
    return -1;
}

} /* extern "C" */
