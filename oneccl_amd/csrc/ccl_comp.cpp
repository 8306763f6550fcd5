// C++ operator surface over the C ABI (see ccl_comp.hpp).
#include "ccl_comp.hpp"

#include <hip/hip_runtime.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/mi_ccl_comp.h"

namespace {

[[noreturn]] void fail(const std::string& what) {
    throw ccl::exception(what);
}

ccl::status to_status(int rc, const char* what) {
    if (rc == MI_CCL_SUCCESS)
        return ccl::status::success;
    fail(std::string(what) + ": " + mi_ccl_status_str(rc));
}

void* stream_of(ccl_sched* sched) {
    return sched ? sched->stream : nullptr;
}

void check_hip(hipError_t e, const char* what) {
    if (e != hipSuccess)
        fail(std::string(what) + ": " + hipGetErrorString(e));
}

// the reference's env_2_enum (src/common/env/env_parser.hpp): the value must be one of the table's names
template <class E>
bool enum_by_name(const std::map<E, std::string>& names, const char* v, E& out) {
    for (const auto& kv : names)
        if (kv.second == v) {
            out = kv.first;
            return true;
        }
    return false;
}

ccl::env_data parse_env() {
    ccl::env_data e;
    if (const char* v = getenv("CCL_BF16")) {      // env.cpp:711-713
        if (!enum_by_name(bf16_impl_names, v, e.bf16_impl_type))
            fail(std::string("unexpected CCL_BF16 value: ") + v);
    }
    if (const char* v = getenv("CCL_FP16")) {      // env.cpp:715-720; f16c and avx512f give the same bits
        if (!enum_by_name(fp16_env_impl_names, v, e.fp16_impl_type))
            fail(std::string("unsupported FP16 impl type: ") + v);
    }
    return e;
}

// float16 follows ccl::global_data::env().fp16_impl_type, which a caller may also set by hand; the value travels
// with every call (nothing process-wide is touched).  fp16_mode returns false when that value names no
// implementation: the reference's dispatch has no branch for it and leaves inout as it was
// (src/comp/fp16/fp16_intrisics.hpp:204-248), and so do the functions below.
int fp16_impl() {
    return (int)ccl::global_data::env().fp16_impl_type;
}
bool fp16_mode(const ccl_datatype& dtype) {
    if (dtype.idx() != ccl::datatype::float16)
        return true;
    return fp16_impl() >= MI_CCL_FP16_F16C && fp16_impl() <= MI_CCL_FP16_AVX512FP16;
}
// the N-input device entry points have no "no implementation" state: such a value falls back to the library's default
int fp16_impl_or_default() {
    return (fp16_impl() >= MI_CCL_FP16_F16C && fp16_impl() <= MI_CCL_FP16_AVX512FP16) ? fp16_impl() : MI_CCL_FP16_DEFAULT;
}

int bf16_impl() {
    return (int)ccl::global_data::env().bf16_impl_type;
}

// ccl::reduction::custom: the callback is host code, so both buffers are staged to the host and the result is
// copied back, blocking, exactly as the reference does for device USM buffers (comp.cpp:163-194).
void custom_on_host(ccl_sched* sched, const void* in_buf, size_t in_count, void* inout_buf, size_t* out_count,
                    const ccl_datatype& dtype, ccl::reduction_fn fn, const ccl::fn_context* context) {
    hipStream_t s = (hipStream_t)stream_of(sched);
    const size_t bytes = in_count * dtype.size();
    std::vector<unsigned char> h_in(bytes), h_io(bytes);
    check_hip(hipMemcpyAsync(h_in.data(), in_buf, bytes, hipMemcpyDeviceToHost, s), "custom reduction: copy in");
    check_hip(hipMemcpyAsync(h_io.data(), inout_buf, bytes, hipMemcpyDeviceToHost, s), "custom reduction: copy in");
    check_hip(hipStreamSynchronize(s), "custom reduction: sync");
    fn(h_in.data(), in_count, h_io.data(), out_count, dtype.idx(), context);
    check_hip(hipMemcpyAsync(inout_buf, h_io.data(), bytes, hipMemcpyHostToDevice, s), "custom reduction: copy out");
    check_hip(hipStreamSynchronize(s), "custom reduction: sync");
}

}  // namespace

ccl::env_data& ccl::global_data::env() {
    static ccl::env_data e = parse_env();
    return e;
}

size_t ccl_datatype::size() const {
    if (m_size == 0)
        fail("non-positive datatype size 0");      // datatype.hpp:46-49
    return m_size;
}

ccl_datatype_storage::ccl_datatype_storage() {
    for (int i = 0; i < 12; i++) {
        table[i] = ccl_datatype((ccl::datatype)i, mi_ccl_datatype_size(i));
        names[i] = mi_ccl_datatype_name(i);
    }
}

ccl_datatype_storage& ccl_datatype_storage::instance() {
    static ccl_datatype_storage s;
    return s;
}

bool ccl_datatype_storage::is_predefined_datatype(ccl::datatype idx) {
    return (int)idx >= (int)ccl::datatype::int8 && (int)idx <= (int)ccl::datatype::last_predefined;
}

const ccl_datatype& ccl_datatype_storage::get(ccl::datatype idx) const {
    if (is_predefined_datatype(idx))
        return table[(int)idx];
    std::lock_guard<std::mutex> lock(guard);
    auto it = custom_table.find((int)idx);
    if (it == custom_table.end())
        fail("unexpected datatype " + std::to_string((int)idx));
    return it->second.first;
}

const std::string& ccl_datatype_storage::name(const ccl_datatype& dtype) const {
    if (is_predefined_datatype(dtype.idx()))
        return names[(int)dtype.idx()];
    std::lock_guard<std::mutex> lock(guard);
    auto it = custom_table.find((int)dtype.idx());
    if (it == custom_table.end())
        fail("unexpected datatype " + std::to_string((int)dtype.idx()));
    return it->second.second;
}

ccl::datatype ccl_datatype_storage::create_by_datatype_size(size_t datatype_size) {
    if (datatype_size == 0)
        fail("non-positive datatype size 0");
    std::lock_guard<std::mutex> lock(guard);
    while (custom_table.count(custom_idx) || is_predefined_datatype((ccl::datatype)custom_idx)) {
        custom_idx++;
        if (custom_idx < (int)ccl::datatype::int8)        // wrapped around
            custom_idx = (int)ccl::datatype::int8;
    }
    const ccl::datatype idx = (ccl::datatype)custom_idx;
    custom_table[custom_idx] = std::make_pair(ccl_datatype(idx, datatype_size), "DTYPE_" + std::to_string(custom_idx));
    return idx;
}

void ccl_datatype_storage::free(ccl::datatype idx) {
    if (is_predefined_datatype(idx))
        fail("attempt to free predefined datatype idx " + std::to_string((int)idx));
    std::lock_guard<std::mutex> lock(guard);
    if (!custom_table.erase((int)idx))
        fail("attempt to free non-existing datatype idx " + std::to_string((int)idx));
}

const char* ccl_reduction_to_str(ccl::reduction type) {
    return mi_ccl_reduction_to_str((int)type);
}

const std::map<ccl_bf16_impl_type, std::string> bf16_impl_names = { { ccl_bf16_scalar, "scalar" },
                                                                   { ccl_bf16_avx512f, "avx512f" },
                                                                   { ccl_bf16_avx512bf, "avx512bf" } };
const std::map<ccl_fp16_impl_type, std::string> fp16_impl_names = { { ccl_fp16_no_compiler_support, "no_compiler_support" },
                                                                   { ccl_fp16_no_hardware_support, "no_hardware_support" },
                                                                   { ccl_fp16_f16c, "f16c" },
                                                                   { ccl_fp16_avx512f, "avx512f" },
                                                                   { ccl_fp16_avx512fp16, "avx512fp16" } };
const std::map<ccl_fp16_impl_type, std::string> fp16_env_impl_names = { { ccl_fp16_f16c, "f16c" },
                                                                       { ccl_fp16_avx512f, "avx512f" },
                                                                       { ccl_fp16_avx512fp16, "avx512fp16" } };

std::set<ccl_bf16_impl_type> ccl_bf16_get_impl_types() {
    return { ccl_bf16_scalar, ccl_bf16_avx512f, ccl_bf16_avx512bf };
}

std::set<ccl_fp16_impl_type> ccl_fp16_get_impl_types() {
    return { ccl_fp16_f16c, ccl_fp16_avx512f, ccl_fp16_avx512fp16 };
}

ccl::status ccl_comp_copy(const void* in_buf, void* out_buf, size_t bytes, bool use_nontemporal, ccl_sched* sched) {
    return to_status(mi_ccl_comp_copy(in_buf, out_buf, bytes, use_nontemporal ? 1 : 0, stream_of(sched)),
                     "ccl_comp_copy");
}

ccl::status ccl_comp_reduce(ccl_sched* sched, const void* in_buf, size_t in_count, void* inout_buf,
                            size_t* out_count, const ccl_datatype& dtype, ccl::reduction reduction,
                            ccl::reduction_fn reduction_fn, const ccl::fn_context* context) {
    if (!in_count)
        return ccl::status::success;                                   // comp.cpp:132-134
    if (reduction == ccl::reduction::custom) {
        if (!reduction_fn)
            fail("custom reduction requires user callback");          // comp.cpp:85
        custom_on_host(sched, in_buf, in_count, inout_buf, out_count, dtype, reduction_fn, context);
        return ccl::status::success;
    }
    // only the 16-bit paths report a count (bf16.cpp:94-96, fp16.cpp:48-50)
    if (out_count && (dtype.idx() == ccl::datatype::bfloat16 || dtype.idx() == ccl::datatype::float16))
        *out_count = in_count;
    if (!fp16_mode(dtype))
        return ccl::status::success;        // float16 without an implementation selected: inout stays as it is
    return to_status(mi_ccl_comp_reduce((int)dtype.idx(), (int)reduction, in_buf, in_count, inout_buf,
                                        bf16_impl(), fp16_impl_or_default(), stream_of(sched)),
                     "ccl_comp_reduce");
}

ccl::status ccl_comp_batch_reduce(const void* in_buf, const std::vector<size_t>& offsets, size_t in_count,
                                  void* inout_buf, size_t* out_count, const ccl_datatype& dtype,
                                  ccl::reduction reduction, ccl::reduction_fn reduction_fn,
                                  const ccl::fn_context* context, int bf16_keep_precision_mode, float* tmp,
                                  float* acc, ccl_sched* sched) {
    (void)tmp;
    (void)acc;
    if (reduction == ccl::reduction::custom) {                         // chain of pairwise calls, comp.cpp:236-245
        for (size_t i = 1; i < offsets.size(); i++)
            ccl_comp_reduce(sched, (const char*)in_buf + dtype.size() * offsets[i], in_count, inout_buf, out_count,
                            dtype, reduction, reduction_fn, context);
        return ccl::status::success;
    }
    if (offsets.empty() || !in_count)
        return ccl::status::success;
    if (out_count && !bf16_keep_precision_mode && offsets.size() > 1 &&
        (dtype.idx() == ccl::datatype::bfloat16 || dtype.idx() == ccl::datatype::float16))
        *out_count = in_count;
    if (!fp16_mode(dtype))
        return ccl::status::success;        // every pairwise call of the chain leaves inout as it is
    return to_status(mi_ccl_comp_batch_reduce(in_buf, offsets.data(), offsets.size(), in_count, inout_buf,
                                              (int)dtype.idx(), (int)reduction, bf16_keep_precision_mode,
                                              bf16_impl(), fp16_impl_or_default(), stream_of(sched)),
                     "ccl_comp_batch_reduce");
}

void ccl_bf16_reduce(const void* in_buf, size_t in_cnt, void* inout_buf, size_t* out_cnt, ccl::reduction reduction_op,
                     ccl_sched* sched) {
    if (out_cnt)
        *out_cnt = in_cnt;                                             // bf16.cpp:94-96
    to_status(mi_ccl_bf16_reduce(in_buf, in_cnt, inout_buf, (int)reduction_op,
                                 (int)ccl::global_data::env().bf16_impl_type, stream_of(sched)),
              "ccl_bf16_reduce");
}

void ccl_fp16_reduce(const void* in_buf, size_t in_cnt, void* inout_buf, size_t* out_cnt, ccl::reduction reduction_op,
                     ccl_sched* sched) {
    if (out_cnt)
        *out_cnt = in_cnt;                                             // fp16.cpp:48-50
    if (!fp16_mode(ccl_datatype_storage::instance().get(ccl::datatype::float16)))
        return;
    to_status(mi_ccl_fp16_reduce(in_buf, in_cnt, inout_buf, (int)reduction_op, fp16_impl(), stream_of(sched)),
              "ccl_fp16_reduce");
}

void ccl_convert_fp32_to_bf16_arrays(void* fp32_buf, void* bf16_buf, size_t count, ccl_sched* sched) {
    to_status(mi_ccl_convert_fp32_to_bf16_arrays(fp32_buf, bf16_buf, count,
                                                 (int)ccl::global_data::env().bf16_impl_type, stream_of(sched)),
              "ccl_convert_fp32_to_bf16_arrays");
}

void ccl_convert_bf16_to_fp32_arrays(void* bf16_buf, float* fp32_buf, size_t count, ccl_sched* sched) {
    to_status(mi_ccl_convert_bf16_to_fp32_arrays(bf16_buf, fp32_buf, count, stream_of(sched)),
              "ccl_convert_bf16_to_fp32_arrays");
}

void ccl_convert_fp32_to_bf16(const void* src, void* dst, ccl_sched* sched) {
    // bf16.cpp:113-123: the avx512bf store when that implementation is selected, the truncating one otherwise
    const int impl = ccl::global_data::env().bf16_impl_type == ccl_bf16_avx512bf ? MI_CCL_BF16_AVX512BF : MI_CCL_BF16_AVX512F;
    to_status(mi_ccl_convert_fp32_to_bf16_arrays(src, dst, 16, impl, stream_of(sched)), "ccl_convert_fp32_to_bf16");
}

void ccl_convert_bf16_to_fp32(const void* src, void* dst, ccl_sched* sched) {
    to_status(mi_ccl_convert_bf16_to_fp32_arrays(src, dst, 16, stream_of(sched)), "ccl_convert_bf16_to_fp32");
}

void ccl_convert_fp32_to_fp16(const void* src, void* dst, ccl_sched* sched) {
    to_status(mi_ccl_convert_fp32_to_fp16_arrays(src, dst, 8, stream_of(sched)), "ccl_convert_fp32_to_fp16");
}

void ccl_convert_fp16_to_fp32(const void* src, void* dst, ccl_sched* sched) {
    to_status(mi_ccl_convert_fp16_to_fp32_arrays(src, dst, 8, stream_of(sched)), "ccl_convert_fp16_to_fp32");
}

void ccl_convert_fp32_to_fp16_arrays(const void* fp32_buf, void* fp16_buf, size_t count, ccl_sched* sched) {
    to_status(mi_ccl_convert_fp32_to_fp16_arrays(fp32_buf, fp16_buf, count, stream_of(sched)),
              "ccl_convert_fp32_to_fp16_arrays");
}

void ccl_convert_fp16_to_fp32_arrays(const void* fp16_buf, float* fp32_buf, size_t count, ccl_sched* sched) {
    to_status(mi_ccl_convert_fp16_to_fp32_arrays(fp16_buf, fp32_buf, count, stream_of(sched)),
              "ccl_convert_fp16_to_fp32_arrays");
}

ccl::status ccl_comp_reduce_n(ccl_sched* sched, const void* own_buf, const std::vector<const void*>& peer_bufs,
                              size_t count, void* out_buf, const ccl_datatype& dtype, ccl::reduction reduction,
                              int bf16_keep_precision_mode) {
    if (!count)
        return ccl::status::success;
    if (reduction == ccl::reduction::custom)
        fail("custom reduction is not available for the N-input device reduce");
    std::vector<const void*> srcs;
    srcs.reserve(peer_bufs.size() + 1);
    srcs.push_back(own_buf);
    srcs.insert(srcs.end(), peer_bufs.begin(), peer_bufs.end());
    int lp = bf16_keep_precision_mode ? MI_CCL_LP_KEEP_PRECISION : MI_CCL_LP_PAIRWISE;
    return to_status(mi_ccl_comp_reduce_n((int)dtype.idx(), (int)reduction, srcs.data(), (int)srcs.size(), out_buf,
                                          count, lp, bf16_impl(), fp16_impl_or_default(), stream_of(sched)),
                     "ccl_comp_reduce_n");
}

ccl::status ccl_comp_reduce_write_n(ccl_sched* sched, const void* own_buf, const std::vector<const void*>& peer_bufs,
                                    size_t count, const std::vector<void*>& out_bufs, const ccl_datatype& dtype,
                                    ccl::reduction reduction, int bf16_keep_precision_mode) {
    if (!count)
        return ccl::status::success;
    if (reduction == ccl::reduction::custom)
        fail("custom reduction is not available for the N-input device reduce");
    std::vector<const void*> srcs;
    srcs.reserve(peer_bufs.size() + 1);
    srcs.push_back(own_buf);
    srcs.insert(srcs.end(), peer_bufs.begin(), peer_bufs.end());
    int lp = bf16_keep_precision_mode ? MI_CCL_LP_KEEP_PRECISION : MI_CCL_LP_PAIRWISE;
    return to_status(mi_ccl_comp_reduce_write_n((int)dtype.idx(), (int)reduction, srcs.data(), (int)srcs.size(),
                                                out_bufs.data(), (int)out_bufs.size(), count, lp,
                                                bf16_impl(), fp16_impl_or_default(), stream_of(sched)),
                     "ccl_comp_reduce_write_n");
}

ccl::status ccl_comp_reduce_batch(ccl_sched* sched, const std::vector<const void*>& srcs, int n_inputs,
                                  const std::vector<void*>& dsts, const std::vector<size_t>& counts,
                                  const ccl_datatype& dtype, ccl::reduction reduction, int bf16_keep_precision_mode) {
    if (dsts.empty())
        return ccl::status::success;
    if (reduction == ccl::reduction::custom)
        fail("custom reduction is not available for the batched device reduce");
    if (n_inputs < 1 || counts.size() != dsts.size() || srcs.size() != dsts.size() * (size_t)n_inputs)
        fail("ccl_comp_reduce_batch: srcs must hold n_inputs pointers per job, dsts and counts one entry per job");
    int lp = bf16_keep_precision_mode ? MI_CCL_LP_KEEP_PRECISION : MI_CCL_LP_PAIRWISE;
    return to_status(mi_ccl_comp_reduce_batch((int)dtype.idx(), (int)reduction, srcs.data(), n_inputs, dsts.data(),
                                              counts.data(), (int)dsts.size(), lp, bf16_impl(), fp16_impl_or_default(),
                                              stream_of(sched)),
                     "ccl_comp_reduce_batch");
}
