// C++ operator surface over the C ABI (see ccl_comp.hpp).
#include "ccl_comp.hpp"

#include <hip/hip_runtime.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>

#include "../../include/mi_ccl_comp.h"
#include "ccl_trace.hpp"

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
    if (const char* v = getenv("MI_CCL_CHECK_POINTERS")) {
        if (strlen(v) != 1 || v[0] < '0' || v[0] > '2')
            fail(std::string("unexpected MI_CCL_CHECK_POINTERS value (0, 1 or 2): ") + v);
        e.check_pointers = v[0] - '0';
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

// ---- which memory a pointer names ----------------------------------------------------------------------------
// The reference looks at both pointers before it picks a path (sycl::get_pointer_type, src/comp/comp.cpp:147-161).
// Here every path is a kernel, and a kernel that is handed pageable host memory takes a GPU memory fault, so the
// functions below refuse such a pointer before anything is enqueued.  Memory the GPU can reach (device, managed,
// pinned host) is accepted.  The answer is remembered per allocation and per thread (hipMemGetAddressRange gives the
// allocation's extent), so a steady-state call costs a search of a short sorted list; env().check_pointers = 2 asks
// the runtime on every call (for callers that free and map memory between calls), 0 switches the check off.
struct known_range {
    uintptr_t lo, hi;
};
thread_local std::vector<known_range> t_known;      // sorted by lo, disjoint
thread_local known_range t_last = { 0, 0 };         // the range of the most recent hit: neighbours in one table mostly share it

bool gpu_can_reach(const void* p, uintptr_t* lo, uintptr_t* hi) {
    hipPointerAttribute_t a;
    memset(&a, 0, sizeof(a));
    if (hipPointerGetAttributes(&a, p) != hipSuccess) {
        (void)hipGetLastError();        // the runtime's answer for memory it has never seen; not an error of this thread's
        return false;
    }
    if (a.type == hipMemoryTypeUnregistered)
        return false;
    *lo = *hi = 0;
    hipDeviceptr_t base = nullptr;
    size_t size = 0;
    if (hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)p) == hipSuccess && size) {
        *lo = (uintptr_t)base;
        *hi = *lo + size;
    }
    else {
        (void)hipGetLastError();
    }
    return true;
}

void require_gpu_memory(const void* p, size_t bytes, const char* fn, const char* arg) {
    const int mode = ccl::global_data::env().check_pointers;
    if (mode == 0 || !p || !bytes)
        return;                         // null pointers are the C ABI's to refuse
    const uintptr_t a = (uintptr_t)p;
    if (mode == 1) {
        if (a >= t_last.lo && a + bytes <= t_last.hi)
            return;
        auto it = std::upper_bound(t_known.begin(), t_known.end(), a,
                                   [](uintptr_t v, const known_range& r) { return v < r.lo; });
        if (it != t_known.begin() && a + bytes <= (it - 1)->hi) {
            t_last = *(it - 1);
            return;
        }
        // not inside anything remembered -- or past the end of a remembered allocation, which may have been freed and
        // replaced by a larger one at the same address: ask the runtime
    }
    uintptr_t lo = 0, hi = 0;
    if (!gpu_can_reach(p, &lo, &hi))
        fail(std::string(fn) + ": " + arg + " is not memory the GPU can reach (pageable host memory?); this build "
             "reduces device buffers only");
    if (hi > lo) {
        if (a + bytes > hi)
            fail(std::string(fn) + ": " + arg + " runs past the end of its allocation");
        if (mode == 1) {
            if (t_known.size() >= 256)
                t_known.clear();
            t_last = known_range{ 0, 0 };
            // a new allocation may cover addresses of remembered ones that have been freed since: drop those
            t_known.erase(std::remove_if(t_known.begin(), t_known.end(),
                                         [&](const known_range& r) { return r.lo < hi && lo < r.hi; }),
                          t_known.end());
            t_known.insert(std::upper_bound(t_known.begin(), t_known.end(), lo,
                                            [](uintptr_t v, const known_range& r) { return v < r.lo; }),
                           known_range{ lo, hi });
        }
    }
}

bool is_gpu_memory(const void* p) {
    uintptr_t lo, hi;
    return gpu_can_reach(p, &lo, &hi);
}

// ccl::reduction::custom: the callback is host code.  With two host buffers it is called on them as they are
// (comp.cpp:84-88, the reference's host path); when either buffer is GPU memory both are staged to the host and the
// result is copied back, blocking, exactly as the reference does for device USM buffers (comp.cpp:163-194).
void custom_on_host(ccl_sched* sched, const void* in_buf, size_t in_count, void* inout_buf, size_t* out_count,
                    const ccl_datatype& dtype, ccl::reduction_fn fn, const ccl::fn_context* context) {
    if (ccl::global_data::env().check_pointers != 0 && !is_gpu_memory(in_buf) && !is_gpu_memory(inout_buf)) {
        fn(in_buf, in_count, inout_buf, out_count, dtype.idx(), context);
        return;
    }
    hipStream_t s = (hipStream_t)stream_of(sched);
    const size_t bytes = in_count * dtype.size();
    std::vector<unsigned char> h_in(bytes), h_io(bytes);
    check_hip(hipMemcpyAsync(h_in.data(), in_buf, bytes, hipMemcpyDefault, s), "custom reduction: copy in");
    check_hip(hipMemcpyAsync(h_io.data(), inout_buf, bytes, hipMemcpyDefault, s), "custom reduction: copy in");
    check_hip(hipStreamSynchronize(s), "custom reduction: sync");
    fn(h_in.data(), in_count, h_io.data(), out_count, dtype.idx(), context);
    check_hip(hipMemcpyAsync(inout_buf, h_io.data(), bytes, hipMemcpyDefault, s), "custom reduction: copy out");
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

void ccl_comp_forget_pointers() {
    t_known.clear();
    t_last = known_range{ 0, 0 };
}

ccl::status ccl_comp_copy(const void* in_buf, void* out_buf, size_t bytes, bool use_nontemporal, ccl_sched* sched) {
    ccl_trace_range tr("ccl_comp_copy");
    require_gpu_memory(in_buf, bytes, "ccl_comp_copy", "in_buf");
    require_gpu_memory(out_buf, bytes, "ccl_comp_copy", "out_buf");
    return to_status(mi_ccl_comp_copy(in_buf, out_buf, bytes, use_nontemporal ? 1 : 0, stream_of(sched)),
                     "ccl_comp_copy");
}

ccl::status ccl_comp_reduce(ccl_sched* sched, const void* in_buf, size_t in_count, void* inout_buf,
                            size_t* out_count, const ccl_datatype& dtype, ccl::reduction reduction,
                            ccl::reduction_fn reduction_fn, const ccl::fn_context* context) {
    ccl_trace_range tr("ccl_comp_reduce");
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
    require_gpu_memory(in_buf, in_count * dtype.size(), "ccl_comp_reduce", "in_buf");
    require_gpu_memory(inout_buf, in_count * dtype.size(), "ccl_comp_reduce", "inout_buf");
    return to_status(mi_ccl_comp_reduce((int)dtype.idx(), (int)reduction, in_buf, in_count, inout_buf,
                                        bf16_impl(), fp16_impl_or_default(), stream_of(sched)),
                     "ccl_comp_reduce");
}

ccl::status ccl_comp_batch_reduce(const void* in_buf, const std::vector<size_t>& offsets, size_t in_count,
                                  void* inout_buf, size_t* out_count, const ccl_datatype& dtype,
                                  ccl::reduction reduction, ccl::reduction_fn reduction_fn,
                                  const ccl::fn_context* context, int bf16_keep_precision_mode, float* tmp,
                                  float* acc, ccl_sched* sched) {
    ccl_trace_range tr("ccl_comp_batch_reduce");
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
    require_gpu_memory(inout_buf, in_count * dtype.size(), "ccl_comp_batch_reduce", "inout_buf");
    for (size_t i = 1; i < offsets.size(); i++)
        require_gpu_memory((const char*)in_buf + dtype.size() * offsets[i], in_count * dtype.size(), "ccl_comp_batch_reduce",
                           "a slice of in_buf");
    return to_status(mi_ccl_comp_batch_reduce(in_buf, offsets.data(), offsets.size(), in_count, inout_buf,
                                              (int)dtype.idx(), (int)reduction, bf16_keep_precision_mode,
                                              bf16_impl(), fp16_impl_or_default(), stream_of(sched)),
                     "ccl_comp_batch_reduce");
}

void ccl_bf16_reduce(const void* in_buf, size_t in_cnt, void* inout_buf, size_t* out_cnt, ccl::reduction reduction_op,
                     ccl_sched* sched) {
    if (out_cnt)
        *out_cnt = in_cnt;                                             // bf16.cpp:94-96
    require_gpu_memory(in_buf, in_cnt * 2, "ccl_bf16_reduce", "in_buf");
    require_gpu_memory(inout_buf, in_cnt * 2, "ccl_bf16_reduce", "inout_buf");
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
    require_gpu_memory(in_buf, in_cnt * 2, "ccl_fp16_reduce", "in_buf");
    require_gpu_memory(inout_buf, in_cnt * 2, "ccl_fp16_reduce", "inout_buf");
    to_status(mi_ccl_fp16_reduce(in_buf, in_cnt, inout_buf, (int)reduction_op, fp16_impl(), stream_of(sched)),
              "ccl_fp16_reduce");
}

void ccl_convert_fp32_to_bf16_arrays(void* fp32_buf, void* bf16_buf, size_t count, ccl_sched* sched) {
    require_gpu_memory(fp32_buf, count * 4, "ccl_convert_fp32_to_bf16_arrays", "fp32_buf");
    require_gpu_memory(bf16_buf, count * 2, "ccl_convert_fp32_to_bf16_arrays", "bf16_buf");
    to_status(mi_ccl_convert_fp32_to_bf16_arrays(fp32_buf, bf16_buf, count,
                                                 (int)ccl::global_data::env().bf16_impl_type, stream_of(sched)),
              "ccl_convert_fp32_to_bf16_arrays");
}

void ccl_convert_bf16_to_fp32_arrays(void* bf16_buf, float* fp32_buf, size_t count, ccl_sched* sched) {
    require_gpu_memory(bf16_buf, count * 2, "ccl_convert_bf16_to_fp32_arrays", "bf16_buf");
    require_gpu_memory(fp32_buf, count * 4, "ccl_convert_bf16_to_fp32_arrays", "fp32_buf");
    to_status(mi_ccl_convert_bf16_to_fp32_arrays(bf16_buf, fp32_buf, count, stream_of(sched)),
              "ccl_convert_bf16_to_fp32_arrays");
}

void ccl_convert_fp32_to_bf16(const void* src, void* dst, ccl_sched* sched) {
    require_gpu_memory(src, 16 * 4, "ccl_convert_fp32_to_bf16", "src");
    require_gpu_memory(dst, 16 * 2, "ccl_convert_fp32_to_bf16", "dst");
    // bf16.cpp:113-123: the avx512bf store when that implementation is selected, the truncating one otherwise
    const int impl = ccl::global_data::env().bf16_impl_type == ccl_bf16_avx512bf ? MI_CCL_BF16_AVX512BF : MI_CCL_BF16_AVX512F;
    to_status(mi_ccl_convert_fp32_to_bf16_arrays(src, dst, 16, impl, stream_of(sched)), "ccl_convert_fp32_to_bf16");
}

void ccl_convert_bf16_to_fp32(const void* src, void* dst, ccl_sched* sched) {
    require_gpu_memory(src, 16 * 2, "ccl_convert_bf16_to_fp32", "src");
    require_gpu_memory(dst, 16 * 4, "ccl_convert_bf16_to_fp32", "dst");
    to_status(mi_ccl_convert_bf16_to_fp32_arrays(src, dst, 16, stream_of(sched)), "ccl_convert_bf16_to_fp32");
}

void ccl_convert_fp32_to_fp16(const void* src, void* dst, ccl_sched* sched) {
    require_gpu_memory(src, 8 * 4, "ccl_convert_fp32_to_fp16", "src");
    require_gpu_memory(dst, 8 * 2, "ccl_convert_fp32_to_fp16", "dst");
    to_status(mi_ccl_convert_fp32_to_fp16_arrays(src, dst, 8, stream_of(sched)), "ccl_convert_fp32_to_fp16");
}

void ccl_convert_fp16_to_fp32(const void* src, void* dst, ccl_sched* sched) {
    require_gpu_memory(src, 8 * 2, "ccl_convert_fp16_to_fp32", "src");
    require_gpu_memory(dst, 8 * 4, "ccl_convert_fp16_to_fp32", "dst");
    to_status(mi_ccl_convert_fp16_to_fp32_arrays(src, dst, 8, stream_of(sched)), "ccl_convert_fp16_to_fp32");
}

void ccl_convert_fp32_to_fp16_arrays(const void* fp32_buf, void* fp16_buf, size_t count, ccl_sched* sched) {
    require_gpu_memory(fp32_buf, count * 4, "ccl_convert_fp32_to_fp16_arrays", "fp32_buf");
    require_gpu_memory(fp16_buf, count * 2, "ccl_convert_fp32_to_fp16_arrays", "fp16_buf");
    to_status(mi_ccl_convert_fp32_to_fp16_arrays(fp32_buf, fp16_buf, count, stream_of(sched)),
              "ccl_convert_fp32_to_fp16_arrays");
}

void ccl_convert_fp16_to_fp32_arrays(const void* fp16_buf, float* fp32_buf, size_t count, ccl_sched* sched) {
    require_gpu_memory(fp16_buf, count * 2, "ccl_convert_fp16_to_fp32_arrays", "fp16_buf");
    require_gpu_memory(fp32_buf, count * 4, "ccl_convert_fp16_to_fp32_arrays", "fp32_buf");
    to_status(mi_ccl_convert_fp16_to_fp32_arrays(fp16_buf, fp32_buf, count, stream_of(sched)),
              "ccl_convert_fp16_to_fp32_arrays");
}

ccl::status ccl_comp_reduce_n(ccl_sched* sched, const void* own_buf, const std::vector<const void*>& peer_bufs,
                              size_t count, void* out_buf, const ccl_datatype& dtype, ccl::reduction reduction,
                              int bf16_keep_precision_mode) {
    ccl_trace_range tr("ccl_comp_reduce_n");
    if (!count)
        return ccl::status::success;
    if (reduction == ccl::reduction::custom)
        fail("custom reduction is not available for the N-input device reduce");
    std::vector<const void*> srcs;
    srcs.reserve(peer_bufs.size() + 1);
    srcs.push_back(own_buf);
    srcs.insert(srcs.end(), peer_bufs.begin(), peer_bufs.end());
    for (const void* p : srcs) require_gpu_memory(p, count * dtype.size(), "ccl_comp_reduce_n", "an input buffer");
    require_gpu_memory(out_buf, count * dtype.size(), "ccl_comp_reduce_n", "out_buf");
    int lp = bf16_keep_precision_mode ? MI_CCL_LP_KEEP_PRECISION : MI_CCL_LP_PAIRWISE;
    return to_status(mi_ccl_comp_reduce_n((int)dtype.idx(), (int)reduction, srcs.data(), (int)srcs.size(), out_buf,
                                          count, lp, bf16_impl(), fp16_impl_or_default(), stream_of(sched)),
                     "ccl_comp_reduce_n");
}

ccl::status ccl_comp_reduce_write_n(ccl_sched* sched, const void* own_buf, const std::vector<const void*>& peer_bufs,
                                    size_t count, const std::vector<void*>& out_bufs, const ccl_datatype& dtype,
                                    ccl::reduction reduction, int bf16_keep_precision_mode) {
    ccl_trace_range tr("ccl_comp_reduce_write_n");
    if (!count)
        return ccl::status::success;
    if (reduction == ccl::reduction::custom)
        fail("custom reduction is not available for the N-input device reduce");
    std::vector<const void*> srcs;
    srcs.reserve(peer_bufs.size() + 1);
    srcs.push_back(own_buf);
    srcs.insert(srcs.end(), peer_bufs.begin(), peer_bufs.end());
    for (const void* p : srcs) require_gpu_memory(p, count * dtype.size(), "ccl_comp_reduce_write_n", "an input buffer");
    for (const void* p : out_bufs) require_gpu_memory(p, count * dtype.size(), "ccl_comp_reduce_write_n", "an output buffer");
    int lp = bf16_keep_precision_mode ? MI_CCL_LP_KEEP_PRECISION : MI_CCL_LP_PAIRWISE;
    return to_status(mi_ccl_comp_reduce_write_n((int)dtype.idx(), (int)reduction, srcs.data(), (int)srcs.size(),
                                                out_bufs.data(), (int)out_bufs.size(), count, lp,
                                                bf16_impl(), fp16_impl_or_default(), stream_of(sched)),
                     "ccl_comp_reduce_write_n");
}

ccl::status ccl_comp_reduce_batch(ccl_sched* sched, const std::vector<const void*>& srcs, int n_inputs,
                                  const std::vector<void*>& dsts, const std::vector<size_t>& counts,
                                  const ccl_datatype& dtype, ccl::reduction reduction, int bf16_keep_precision_mode) {
    ccl_trace_range tr("ccl_comp_reduce_batch");
    if (dsts.empty())
        return ccl::status::success;
    if (reduction == ccl::reduction::custom)
        fail("custom reduction is not available for the batched device reduce");
    if (n_inputs < 1 || counts.size() != dsts.size() || srcs.size() != dsts.size() * (size_t)n_inputs)
        fail("ccl_comp_reduce_batch: srcs must hold n_inputs pointers per job, dsts and counts one entry per job");
    for (size_t j = 0; j < dsts.size(); j++) {
        if (!counts[j])
            continue;                       // an empty job's pointers are not looked at
        for (int k = 0; k < n_inputs; k++)
            require_gpu_memory(srcs[j * n_inputs + k], counts[j] * dtype.size(), "ccl_comp_reduce_batch", "an input buffer");
        require_gpu_memory(dsts[j], counts[j] * dtype.size(), "ccl_comp_reduce_batch", "an output buffer");
    }
    int lp = bf16_keep_precision_mode ? MI_CCL_LP_KEEP_PRECISION : MI_CCL_LP_PAIRWISE;
    return to_status(mi_ccl_comp_reduce_batch((int)dtype.idx(), (int)reduction, srcs.data(), n_inputs, dsts.data(),
                                              counts.data(), (int)dsts.size(), lp, bf16_impl(), fp16_impl_or_default(),
                                              stream_of(sched)),
                     "ccl_comp_reduce_batch");
}
