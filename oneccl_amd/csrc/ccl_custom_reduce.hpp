// ccl::reduction::custom on the device.
//
// The reference's custom reduction is a host callback, ccl::reduction_fn (include/oneapi/ccl/types.hpp:116-124),
// which for device buffers forces a round trip through host memory (src/comp/comp.cpp:163-194; the C++ surface in
// ccl_comp.hpp does the same).  This header is the device form: the user's operation is a functor that is callable
// on the device, compiled into the user's own translation unit by hipcc together with the kernel below --
// the way a functor reaches a HIP kernel without a function-pointer call.
//
//     struct absmax { __device__ float operator()(float in, float inout) const { return fmaxf(fabsf(in), fabsf(inout)); } };
//     ccl_custom_reduce_n<float>(sched, srcs, out, count, absmax{});                              // direct call
//     entry_factory::create<custom_reduce_local_entry<float, absmax>>(sched, in, cnt, inout, absmax{});   // as an entry
//
// Order and roles follow the built-in reductions: acc = srcs[0][i]; acc = f(in = srcs[j][i], inout = acc) for
// j = 1 .. n-1; out[i] = acc.  T is any trivially copyable type of 1, 2, 4, 8 or 16 bytes.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <type_traits>

#include "ccl_sched_entry.hpp"

namespace ccl_custom {

constexpr int kBlock = 256;
constexpr int kMaxSrcs = 16;
template <class T>
struct src_table {
    const T* p[kMaxSrcs];
};
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 u32x4_u __attribute__((aligned(1)));      // a 128-bit access that promises no alignment

// 16 bytes per lane and input per step, two steps in flight, from element `head` on (where dst reaches a 16-byte
// boundary); the sources may sit at any other alignment
template <class T, class F>
__global__ void __launch_bounds__(kBlock) reduce_vec_kernel(src_table<T> src, int n, T* dst, uint64_t head,
                                                            uint64_t nvec, F f) {
    constexpr int VEC = 16 / sizeof(T);
    struct alignas(16) pack {
        T v[VEC];
    };
    static_assert(sizeof(pack) == 16, "element size must divide 16");
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (uint64_t i0 = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i0 < nvec; i0 += 2 * stride) {
        const uint64_t i1 = i0 + stride;
        const bool two = i1 < nvec;
        pack a0 = __builtin_bit_cast(pack, __builtin_nontemporal_load((const u32x4_u*)(src.p[0] + head) + i0)), a1 = a0;
        if (two) a1 = __builtin_bit_cast(pack, __builtin_nontemporal_load((const u32x4_u*)(src.p[0] + head) + i1));
        for (int j = 1; j < n; j++) {
            pack x0 = __builtin_bit_cast(pack, __builtin_nontemporal_load((const u32x4_u*)(src.p[j] + head) + i0)), x1 = x0;
            if (two) x1 = __builtin_bit_cast(pack, __builtin_nontemporal_load((const u32x4_u*)(src.p[j] + head) + i1));
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                a0.v[k] = f(x0.v[k], a0.v[k]);
                a1.v[k] = f(x1.v[k], a1.v[k]);
            }
        }
        __builtin_nontemporal_store(__builtin_bit_cast(u32x4, a0), (u32x4_u*)(dst + head) + i0);
        if (two) __builtin_nontemporal_store(__builtin_bit_cast(u32x4, a1), (u32x4_u*)(dst + head) + i1);
    }
}

// one element per lane: the elements before the first vector and after the last one (elements [0, head) and
// [begin, count))
template <class T, class F>
__global__ void __launch_bounds__(kBlock) reduce_elem_kernel(src_table<T> src, int n, T* dst, uint64_t head,
                                                             uint64_t begin, uint64_t count, F f) {
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (uint64_t t = (uint64_t)blockIdx.x * kBlock + threadIdx.x; t < head + (count - begin); t += stride) {
        const uint64_t i = t < head ? t : begin + (t - head);
        T a = src.p[0][i];
        for (int j = 1; j < n; j++) a = f(src.p[j][i], a);
        dst[i] = a;
    }
}

inline int cu_count() {
    static std::atomic<int> per_device[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = per_device[dev].load(std::memory_order_relaxed);
    if (!n) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        per_device[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

}  // namespace ccl_custom

// out = srcs[0] f srcs[1] f ... in argument order; out may be one of the sources.  Enqueued on the schedule's stream.
template <class T, class F>
ccl::status ccl_custom_reduce_n(ccl_sched* sched, const std::vector<const T*>& srcs, T* out, size_t count, F f) {
    static_assert(std::is_trivially_copyable<T>::value && (16 % sizeof(T)) == 0, "T: trivially copyable, 1..16 bytes");
    using namespace ccl_custom;
    if (count == 0) return ccl::status::success;
    if (srcs.empty() || srcs.size() > (size_t)kMaxSrcs || !out) throw ccl::exception("ccl_custom_reduce_n: bad arguments");
    src_table<T> t{};
    for (size_t j = 0; j < srcs.size(); j++) {
        if (!srcs[j]) throw ccl::exception("ccl_custom_reduce_n: null source");
        t.p[j] = srcs[j];
    }
    hipStream_t stream = (hipStream_t)(sched ? sched->stream : nullptr);
    const int n = (int)srcs.size();
    constexpr uint64_t VEC = 16 / sizeof(T);
    // the vectors start where the output reaches a 16-byte boundary
    const uintptr_t mis = (uintptr_t)out & 15u;
    uint64_t head = (mis % sizeof(T)) == 0 ? ((16u - mis) & 15u) / sizeof(T) : 0;
    if (head > count) head = count;
    const uint64_t nvec = (count - head) / VEC;
    const uint64_t max_grid = (uint64_t)cu_count() * 8;
    if (nvec) {
        uint64_t blocks = (nvec + 2 * kBlock - 1) / (2 * kBlock);
        hipLaunchKernelGGL((reduce_vec_kernel<T, F>), dim3((unsigned)(blocks < max_grid ? blocks : max_grid)), dim3(kBlock),
                           0, stream, t, n, out, head, nvec, f);
    }
    if (head + nvec * VEC < count || head) {
        hipLaunchKernelGGL((reduce_elem_kernel<T, F>), dim3(1), dim3(kBlock), 0, stream, t, n, out, head,
                           head + nvec * VEC, (uint64_t)count, f);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) throw ccl::exception(std::string("ccl_custom_reduce_n: ") + hipGetErrorString(e));
    return ccl::status::success;
}

// REDUCE_LOCAL with a device functor in place of ccl::reduction: inout = f(in, inout)
// (the shape of reduce_local_entry, src/sched/entry/reduce_local_entry.hpp:26-91)
template <class T, class F>
class custom_reduce_local_entry : public sched_entry {
public:
    static constexpr const char* class_name() noexcept { return "REDUCE_LOCAL_CUSTOM"; }
    const char* name() const noexcept override { return class_name(); }
    custom_reduce_local_entry(ccl_sched* sched, const ccl_buffer in_buf, size_t in_cnt, ccl_buffer inout_buf, F f)
            : sched_entry(sched), in_buf(in_buf), in_cnt(in_cnt), inout_buf(inout_buf), f(f) {}
    void start() override {
        const size_t bytes = in_cnt * sizeof(T);
        T* io = (T*)inout_buf.get_ptr(bytes);
        ccl_custom_reduce_n<T, F>(sched, { (const T*)io, (const T*)in_buf.get_ptr(bytes) }, io, in_cnt, f);
        record_started();
    }

private:
    const ccl_buffer in_buf;
    const size_t in_cnt;
    const ccl_buffer inout_buf;
    F f;
};
