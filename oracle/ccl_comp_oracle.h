/*
 * TEST INFRASTRUCTURE ONLY -- never linked into, imported by or executed from the product.
 *
 * Scalar CPU restatement of the arithmetic of oneCCL's data-parallel reduction path
 * (src/comp, the bf16/fp16 helpers, the N-input chain of src/kernels, the src/fusion layout).
 * Every function cites the reference file:line it follows.  Only tests/, the smoke check and
 * the CPU-baseline leg of the benchmark may load this library, and only as the checker.
 *
 * Pinning status of each function is listed at the top of ccl_comp_oracle.c.
 */
#ifndef CCL_COMP_ORACLE_H
#define CCL_COMP_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ccl::datatype, include/oneapi/ccl/types.hpp:52-69 */
enum {
    ORC_INT8 = 0, ORC_UINT8, ORC_INT16, ORC_UINT16, ORC_INT32, ORC_UINT32, ORC_INT64, ORC_UINT64,
    ORC_FLOAT16 = 8, ORC_FLOAT32, ORC_FLOAT64, ORC_BFLOAT16 = 11, ORC_DTYPE_LAST
};
/* ccl::reduction, include/oneapi/ccl/types.hpp:41-47 */
enum { ORC_SUM = 0, ORC_PROD, ORC_MIN, ORC_MAX, ORC_CUSTOM };
/* ccl_bf16_impl_type, src/comp/bf16/bf16_utils.hpp:26 */
enum { ORC_BF16_SCALAR = 0, ORC_BF16_AVX512F = 1, ORC_BF16_AVX512BF = 2 };
/* ccl_fp16_impl_type, src/comp/fp16/fp16_utils.hpp:26-32 */
enum { ORC_FP16_NO_COMPILER = 0, ORC_FP16_NO_HARDWARE = 1, ORC_FP16_F16C = 2, ORC_FP16_AVX512F = 3,
       ORC_FP16_AVX512FP16 = 4 };
/* ccl::status, src/internal_types.hpp:29-37 */
enum { ORC_OK = 0, ORC_INVALID_ARGUMENTS = 2 };

size_t orc_datatype_size(int dtype);          /* src/common/datatype/datatype.cpp:79-91 */
const char* orc_datatype_name(int dtype);     /* src/common/datatype/datatype.cpp:94-106 */
const char* orc_reduction_to_str(int op);     /* src/comp/comp.cpp:251-260 */

/* element converters */
uint32_t orc_bf16_widen(uint16_t h);          /* bf16.cpp:56-61, bf16_intrisics.hpp:62-65 */
uint16_t orc_bf16_narrow_trunc(uint32_t u);   /* bf16.cpp:50-54, bf16_intrisics.hpp:67-70 */
uint16_t orc_bf16_narrow_rne(uint32_t u);     /* bf16_intrisics.hpp:73-75 (VCVTNEPS2BF16) */
uint32_t orc_fp16_widen(uint16_t h);          /* fp16_intrisics.hpp:100-101 (VCVTPH2PS) */
uint16_t orc_fp16_narrow(uint32_t u);         /* fp16_intrisics.hpp:103 (VCVTPS2PH imm 0) */

/* array converters with the scalar truncating tail, bf16.cpp:130-169 */
void orc_convert_fp32_to_bf16_arrays(const void* fp32_buf, void* bf16_buf, size_t count, int bf16_impl);
void orc_convert_bf16_to_fp32_arrays(const void* bf16_buf, void* fp32_buf, size_t count, int bf16_impl);
void orc_convert_fp32_to_fp16_arrays(const void* fp32_buf, void* fp16_buf, size_t count);   /* fp16.cpp:55-57, per value */
void orc_convert_fp16_to_fp32_arrays(const void* fp16_buf, void* fp32_buf, size_t count);   /* fp16.cpp:59-61 */

/* pairwise in-place primitives */
void orc_bf16_reduce(const void* in, size_t count, void* inout, int op, int bf16_impl); /* bf16.cpp:87-110 */
void orc_fp16_reduce(const void* in, size_t count, void* inout, int op, int fp16_impl); /* fp16.cpp:41-53 */
int orc_comp_reduce(const void* in, size_t count, void* inout, int dtype, int op, int bf16_impl,
                    int fp16_impl);                                                   /* comp.cpp:76-200 */

/* N-input reduce over slices of one buffer, comp.cpp:202-249; offsets in elements, offsets[0] is
 * the slice that inout aliases.  tmp/acc: caller scratch of count floats (keep-precision only). */
int orc_comp_batch_reduce(const void* in_buf, const size_t* offsets, size_t n_offsets, size_t count,
                          void* inout, int dtype, int op, int bf16_keep_precision_mode, float* tmp,
                          float* acc, int bf16_impl, int fp16_impl);

/* N separate buffers, device-kernel argument order (own first, then peers in argument order,
 * kernels.cl:269-421) with the CPU pairwise step: acc = src0; acc = step(in = src_j, inout = acc).
 * lp_keep_precision applies the comp.cpp:214-234 keep-precision recipe to bf16; quirk_tail != 0
 * keeps the truncating tail of bf16.cpp:144-148, 0 rounds every element the same way. */
int orc_reduce_n(const void* const* srcs, int n, void* dst, size_t count, int dtype, int op,
                 int lp_keep_precision, int quirk_tail, int bf16_impl, int fp16_impl);

/* The N-input reduce whose result goes to m buffers: allreduce_kernel (kernels.cl:190-217: one reduce, the result
 * stored to the own and to the peer's output) and, with n == 1, write_monolithic_kernel_N (kernels.cl:423-560: one
 * input copied to N peers).  Same arithmetic as orc_reduce_n; a destination may be one of the sources. */
int orc_reduce_write_n(const void* const* srcs, int n, void* const* dsts, int m, size_t count, int dtype, int op,
                       int lp_keep_precision, int quirk_tail, int bf16_impl, int fp16_impl);

/* comp.cpp:60-74 */
int orc_comp_copy(const void* in, void* out, size_t bytes);

/* fusion layout, fusion.cpp:283-316 (pack) and :323-362 (unpack): running byte offset, tight when
 * align == 1; align > 1 rounds every tensor's start up to a multiple of align bytes.
 * Returns the fused buffer size in bytes (end of the last tensor). */
size_t orc_fusion_offsets(const size_t* counts, size_t k, size_t dtype_size, size_t align,
                          size_t* byte_offsets);
void orc_fusion_pack(const void* const* tensors, const size_t* counts, const size_t* byte_offsets,
                     size_t k, size_t dtype_size, void* fusion_buf);
void orc_fusion_unpack(const void* fusion_buf, const size_t* counts, const size_t* byte_offsets,
                       size_t k, size_t dtype_size, void* const* tensors);

/* Multi-threaded wrappers used only for timing/large checks: split [0,count) in `threads`
 * contiguous partitions as the reference's parallelizer does (parallelizer.cpp:230-241,374-379). */
int orc_reduce_n_mt(const void* const* srcs, int n, void* dst, size_t count, int dtype, int op,
                    int lp_keep_precision, int quirk_tail, int bf16_impl, int fp16_impl, int threads);

#ifdef __cplusplus
}
#endif
#endif
