/*
 * TEST INFRASTRUCTURE ONLY.  C entry points around the reference's own vector reduce code, compiled
 * from the reference tree where it lies (see oracle/Makefile, target _ref): this file includes
 * src/comp/bf16/bf16_intrisics.hpp and src/comp/fp16/fp16_intrisics.hpp and is linked with
 * src/comp/bf16/bf16_intrisics.cpp and src/comp/fp16/fp16_intrisics.cpp.  Nothing of the reference is
 * copied; the output goes to oracle/_ref/ only.
 *
 * What this reaches: ccl_bf16_reduce_impl_{avx512f,avx512bf} (bf16_intrisics.hpp:106-114),
 * ccl_bf16_load_as_fp32 / ccl_fp32_store_as_bf16_{avx512f,avx512bf} (:62-76), singly and in the loop of the
 * keep-precision batch reduce,
 * ccl_fp16_reduce_impl_{256,512} (fp16_intrisics.hpp:186-196).
 * What it cannot reach: the dispatchers in comp.cpp / bf16.cpp / fp16.cpp need ccl::global_data, the
 * logger and the datatype storage, i.e. the whole library, whose build needs cmake and the prebuilt
 * hwloc/itt archives under deps/ -- treated as unbuildable.
 *
 * The calling CPU must have AVX512F/BW/VL (+AVX512_BF16 for impl 2, F16C for fp16): ref_cpu_support()
 * reports it and every entry point checks it.
 */
#include <cpuid.h>
#include <stddef.h>
#include <stdint.h>

#include "comp/bf16/bf16_intrisics.hpp"
#include "comp/fp16/fp16_intrisics.hpp"

#define REF_TARGET_BF16 __attribute__((target("avx512bw,avx512vl,avx512f,avx512bf16")))
#define REF_TARGET_512  __attribute__((target("avx512bw,avx512vl,avx512f")))
#define REF_TARGET_F16C __attribute__((target("f16c,avx")))

extern "C" {

/* bit 0: avx512f+bw+vl, bit 1: avx512_bf16, bit 2: f16c, bit 3: avx512_fp16 */
int ref_cpu_support(void) {
    unsigned a, b, c, d;
    int r = 0;
    if (__get_cpuid_count(7, 0, &a, &b, &c, &d)) {
        if ((b & (1u << 16)) && (b & (1u << 30)) && (b & (1u << 31)))
            r |= 1;
        if ((b & (1u << 30)) && (d & (1u << 23)))     /* as fp16_utils.hpp:62-70 */
            r |= 8;
    }
    if (__get_cpuid_count(7, 1, &a, &b, &c, &d)) {
        if (a & (1u << 5))
            r |= 2;
    }
    if (__get_cpuid(1, &a, &b, &c, &d)) {
        if (c & (1u << 29))
            r |= 4;
    }
    return r;
}

static ccl_bf16_reduction_func_ptr bf16_op(int op) {
    switch (op) {
        case 0: return &bf16_sum_wrap;
        case 1: return &bf16_prod_wrap;
        case 2: return &bf16_min_wrap;
        case 3: return &bf16_max_wrap;
        default: return nullptr;
    }
}

/* impl: 1 = avx512f (truncate), 2 = avx512bf (VCVTNEPS2BF16).  count < 2^31 (the reference loop index
 * is an int).  Returns 0, or -1 when the op/impl/CPU combination is not available. */
REF_TARGET_BF16 int ref_bf16_reduce(const void* in, size_t count, void* inout, int op, int impl) {
    ccl_bf16_reduction_func_ptr f = bf16_op(op);
    int cpu = ref_cpu_support();
    if (!f || count >= 0x7fffffffu || !(cpu & 1))
        return -1;
    if (impl == 1) {
        ccl_bf16_reduce_impl_avx512f(in, inout, count, f);
        return 0;
    }
    if (impl == 2 && (cpu & 2)) {
        ccl_bf16_reduce_impl_avx512bf(in, inout, count, f);
        return 0;
    }
    return -1;
}

/* 16 elements per call, as the reference helpers work */
REF_TARGET_512 int ref_bf16_load_as_fp32_16(const void* src, void* dst) {
    if (!(ref_cpu_support() & 1))
        return -1;
    ccl_bf16_load_as_fp32(src, dst);
    return 0;
}

REF_TARGET_BF16 int ref_fp32_store_as_bf16_16(const void* src, void* dst, int impl) {
    int cpu = ref_cpu_support();
    if (impl == 1 && (cpu & 1)) {
        ccl_fp32_store_as_bf16_avx512f(src, dst);
        return 0;
    }
    if (impl == 2 && (cpu & 1) && (cpu & 2)) {
        ccl_fp32_store_as_bf16_avx512bf(src, dst);
        return 0;
    }
    return -1;
}

/* The keep-precision batch reduce (sum) with the reference's pass structure (src/comp/comp.cpp:202-249: widen the own
 * slice into acc; per further slice widen into tmp and add tmp into acc in fp32; narrow acc once), its conversions done
 * by the reference's own 16-wide helpers exactly as its array converters call them (src/comp/bf16/bf16.cpp:130-169)
 * and the fp32 add by a plain loop built for the baseline x86-64 target, as the reference's CCL_REDUCE loop is
 * (comp.cpp:31-58).  Slices are in_buf + 2 * offsets[i]; inout is slice 0.  count must be a multiple of 16 (the
 * scalar tail converters live in bf16.cpp, which is not part of this build).  For timing the reference's CPU path. */
__attribute__((noinline)) static void ref_add_f32(const float* in, float* inout, size_t count) {
    for (size_t i = 0; i < count; i++) inout[i] = in[i] + inout[i];
}
REF_TARGET_BF16 __attribute__((noinline)) static void ref_widen(const void* bf16, float* f32, size_t count) {
    for (size_t i = 0; i < count; i += 16) ccl_bf16_load_as_fp32((const char*)bf16 + 2 * i, f32 + i);
}
REF_TARGET_BF16 __attribute__((noinline)) static void ref_narrow(const float* f32, void* bf16, size_t count, int impl) {
    if (impl == 2)
        for (size_t i = 0; i < count; i += 16) ccl_fp32_store_as_bf16_avx512bf(f32 + i, (char*)bf16 + 2 * i);
    else
        for (size_t i = 0; i < count; i += 16) ccl_fp32_store_as_bf16_avx512f(f32 + i, (char*)bf16 + 2 * i);
}
int ref_batch_reduce_keep_sum(const void* in_buf, const size_t* offsets, size_t n, size_t count, void* inout,
                              float* tmp, float* acc, int impl) {
    int cpu = ref_cpu_support();
    if (!(cpu & 1) || (impl == 2 && !(cpu & 2)) || (impl != 1 && impl != 2) || (count % 16) != 0 || n < 1)
        return -1;
    ref_widen(inout, acc, count);
    for (size_t i = 1; i < n; i++) {
        ref_widen((const char*)in_buf + 2 * offsets[i], tmp, count);
        ref_add_f32(tmp, acc, count);
    }
    ref_narrow(acc, inout, count, impl);
    return 0;
}

/* impl: 2 = f16c (8 per iteration, memcpy'd tail), 3 = avx512f (16 per iteration, masked tail),
 * 4 = avx512fp16 (32 per iteration in native fp16, masked tail): only in a build whose compiler knows the
 * AVX512-FP16 intrinsics (the reference's own CCL_FP16_AVX512FP16_COMPILER switch; see oracle/Makefile) */
int ref_fp16_reduce(const void* in, size_t count, void* inout, int op, int impl) {
    int cpu = ref_cpu_support();
    if (count >= 0x7fffffffu || op < 0 || op > 3)
        return -1;
    if (impl == 2 && (cpu & 4)) {
        static const ccl_fp16_reduction_func_ptr_256 f[4] = { &fp16_sum_wrap_256, &fp16_prod_wrap_256,
                                                              &fp16_min_wrap_256, &fp16_max_wrap_256 };
        ccl_fp16_reduce_impl_256(in, inout, count, f[op]);
        return 0;
    }
    if (impl == 3 && (cpu & 1)) {
        static const ccl_fp16_reduction_func_ptr_512 f[4] = { &fp16_sum_wrap_512, &fp16_prod_wrap_512,
                                                              &fp16_min_wrap_512, &fp16_max_wrap_512 };
        ccl_fp16_reduce_impl_512(in, inout, count, f[op]);
        return 0;
    }
#ifdef CCL_FP16_AVX512FP16_COMPILER
    if (impl == 4 && (cpu & 8)) {
        static const ccl_fp16_reduction_func_ptr_512FP16 f[4] = { &fp16_sum_wrap_512FP16, &fp16_prod_wrap_512FP16,
                                                                  &fp16_min_wrap_512FP16, &fp16_max_wrap_512FP16 };
        ccl_fp16_reduce_impl_512FP16(in, inout, count, f[op]);
        return 0;
    }
#endif
    return -1;
}

} /* extern "C" */
