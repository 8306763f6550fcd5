// C++ operator surface of the MI355X reduction engine: the functions oneCCL's scheduler entries call
// (src/comp/comp.hpp:23-51, src/comp/bf16/bf16.hpp:26-38, src/comp/fp16/fp16.hpp:21-25), with the same
// names, argument order and meaning, running on device buffers through the C ABI of mi_ccl_comp.h.
//
// Differences a caller sees, all of them at the edges:
//   * buffers are HIP device pointers; the work is enqueued on the HIP stream carried by ccl_sched
//     (the reference's sched argument is only used to reach the stream, src/comp/comp.cpp:137-141);
//     a null sched means the default stream.  Calls return once enqueued.
//   * functions that have no sched argument in the reference (batch reduce, copy, the bf16/fp16 entry
//     points, the array converters) take it as a trailing, defaulted argument.
//   * an unknown dtype or reduction throws ccl::exception where the reference calls CCL_FATAL
//     (std::terminate, src/comp/comp.cpp:56,113).
//   * ccl::reduction::custom runs the user's host callback on host copies of the two buffers, as the
//     reference does for device buffers (src/comp/comp.cpp:163-194), and on the buffers themselves when both
//     are host memory (src/comp/comp.cpp:84-88).
//   * a buffer of pageable host memory is refused with ccl::exception before anything is enqueued (the
//     reference reduces it on the host; here every path is a kernel): see env_data::check_pointers.
#pragma once

#include <stddef.h>
#include <stdint.h>

#include <exception>
#include <map>
#include <memory>
#include <mutex>
#include <set>
#include <string>
#include <vector>

namespace ccl {

// include/oneapi/ccl/types.hpp:41-69
enum class reduction : int { sum = 0, prod, min, max, custom };
enum class datatype : int {
    int8 = 0, uint8, int16, uint16, int32, uint32, int64, uint64, float16, float32, float64, bfloat16,
    last_predefined = bfloat16
};

// src/internal_types.hpp:29-37
enum status : int { success = 0, out_of_resource, invalid_arguments, runtime_error, blocked_due_to_resize, last_value };

// include/oneapi/ccl/types.hpp:116-124
typedef struct {
    const char* match_id;
    const size_t offset;
} fn_context;
typedef void (*reduction_fn)(const void* in_buf, size_t in_count, void* inout_buf, size_t* out_count,
                             ccl::datatype dtype, const ccl::fn_context* context);

// include/oneapi/ccl/lp_types.hpp:27-67: 16-bit floats travel as raw bit patterns
struct float16 {
    constexpr float16() : data(0) {}
    constexpr float16(uint16_t v) : data(v) {}
    uint16_t get_data() const { return data; }
    friend bool operator==(const float16& a, const float16& b) { return a.data == b.data; }
    friend bool operator!=(const float16& a, const float16& b) { return a.data != b.data; }

private:
    uint16_t data;
} __attribute__((packed));
struct bfloat16 {
    constexpr bfloat16() : data(0) {}
    constexpr bfloat16(uint16_t v) : data(v) {}
    uint16_t get_data() const { return data; }
    friend bool operator==(const bfloat16& a, const bfloat16& b) { return a.data == b.data; }
    friend bool operator!=(const bfloat16& a, const bfloat16& b) { return a.data != b.data; }

private:
    uint16_t data;
} __attribute__((packed));

// include/oneapi/ccl/exception.hpp:27-51
class exception : public std::exception {
    std::string msg;

public:
    exception(const std::string& info = "") : msg("oneCCL: " + info) {}
    const char* what() const noexcept override { return msg.c_str(); }
};

}  // namespace ccl

// src/comp/bf16/bf16_utils.hpp:26, src/comp/fp16/fp16_utils.hpp:26-32
typedef enum { ccl_bf16_scalar = 0, ccl_bf16_avx512f, ccl_bf16_avx512bf } ccl_bf16_impl_type;
typedef enum {
    ccl_fp16_no_compiler_support = 0, ccl_fp16_no_hardware_support, ccl_fp16_f16c, ccl_fp16_avx512f, ccl_fp16_avx512fp16
} ccl_fp16_impl_type;

// Names as the reference prints and parses them (bf16.cpp:26-30, fp16.cpp:25-37) and the implementations a process
// may choose (bf16_utils.hpp:30-72, fp16_utils.hpp:37-80 ask the CPU; here every implementation's arithmetic is in
// the kernels, so all of them are on offer).
extern const std::map<ccl_bf16_impl_type, std::string> bf16_impl_names;
extern const std::map<ccl_fp16_impl_type, std::string> fp16_impl_names;
extern const std::map<ccl_fp16_impl_type, std::string> fp16_env_impl_names;
std::set<ccl_bf16_impl_type> ccl_bf16_get_impl_types();
std::set<ccl_fp16_impl_type> ccl_fp16_get_impl_types();

namespace ccl {
// The two knobs of the reference's env_data that this path reads (src/common/env/env.cpp:711-720): which
// CPU implementation's results to reproduce.  Defaults: avx512bf (round to nearest even) and avx512f;
// CCL_BF16 = scalar | avx512f | avx512bf and CCL_FP16 = f16c | avx512f | avx512fp16 are read once, like the reference.
// A float16 reduce with fp16_impl_type set to a value that names no implementation leaves inout untouched, as the
// reference's dispatch does (src/comp/fp16/fp16_intrisics.hpp:204-248).
struct env_data {
    ccl_bf16_impl_type bf16_impl_type = ccl_bf16_avx512bf;
    ccl_fp16_impl_type fp16_impl_type = ccl_fp16_avx512f;
    // What the functions below do about a buffer that is not GPU memory (the reference classifies its pointers,
    // src/comp/comp.cpp:147-161, and reduces host buffers on the host; here every path is a kernel, and a kernel
    // handed pageable host memory is a GPU memory fault): 1 = refuse it with ccl::exception before anything is
    // enqueued, remembering per thread which allocations have been seen (the default; MI_CCL_CHECK_POINTERS);
    // 2 = the same, asking the runtime on every call; 0 = no check, for callers that guarantee device memory.
    int check_pointers = 1;
};
struct global_data {
    static env_data& env();
};
}  // namespace ccl

// src/common/datatype/datatype.hpp:31-54 and the predefined table of datatype.cpp:79-106
class ccl_datatype {
public:
    ccl_datatype() = default;
    ccl_datatype(ccl::datatype idx, size_t size) : m_idx(idx), m_size(size) {}
    ccl::datatype idx() const noexcept { return m_idx; }
    size_t size() const;

private:
    ccl::datatype m_idx = ccl::datatype::int8;
    size_t m_size = sizeof(int8_t);
};
class ccl_datatype_storage {
public:
    const ccl_datatype& get(ccl::datatype idx) const;
    const std::string& name(const ccl_datatype& dtype) const;
    static ccl_datatype_storage& instance();
    // user-defined datatypes, for ccl::reduction::custom (datatype.cpp:141-181): an element size and the next free
    // index above the predefined ones; the name is "DTYPE_<index>"
    ccl::datatype create_by_datatype_size(size_t datatype_size);
    void free(ccl::datatype idx);
    static bool is_predefined_datatype(ccl::datatype idx);

private:
    ccl_datatype_storage();
    ccl_datatype table[12];
    std::string names[12];
    mutable std::mutex guard;
    std::map<int, std::pair<ccl_datatype, std::string>> custom_table;
    int custom_idx = (int)ccl::datatype::last_predefined + 1;
};

// What this path needs of a schedule (src/sched/sched.hpp, src/sched/sched_base.hpp): the stream its kernels go to
// (a hipStream_t), the user's reduction callback and match id (ccl_coll_attr, src/coll/coll_param.hpp), and -- for
// callers that drive scheduler entries, ccl_sched_entry.hpp -- the entry list with the reference's progress rule.
struct ccl_coll_attr {
    ccl::reduction_fn reduction_fn = nullptr;
    std::string match_id;
};
class sched_entry;
struct ccl_sched {
    void* stream = nullptr;
    ccl_coll_attr coll_attr;

    // the rest is defined in ccl_sched_entry.cpp and only needed with entries
    std::vector<std::shared_ptr<void>> owned_buffers;      // declared before the entries: destroyed after them
    std::vector<std::shared_ptr<sched_entry>> entries;
    size_t start_idx = 0;
    sched_entry* add_entry(std::shared_ptr<sched_entry> entry);
    void add_barrier();                         // the last entry becomes a barrier (src/sched/sched.cpp:596-605)
    void do_progress();                         // src/sched/sched.cpp:439-490
    bool is_completed() const { return start_idx == entries.size(); }
    void renew();                               // every entry back to not_started, for the next run of the schedule
    void* alloc_buffer(size_t bytes);           // device memory owned by the schedule (sched_base.cpp alloc_buffer)
};

// Drops what this thread remembers about allocations it has seen (env_data::check_pointers = 1): for a caller that
// frees device memory and may get the same addresses back as host memory.
void ccl_comp_forget_pointers();

// src/comp/comp.hpp:23-51
ccl::status ccl_comp_copy(const void* in_buf, void* out_buf, size_t bytes, bool use_nontemporal = false,
                          ccl_sched* sched = nullptr);

ccl::status ccl_comp_reduce(ccl_sched* sched, const void* in_buf, size_t in_count, void* inout_buf,
                            size_t* out_count, const ccl_datatype& dtype, ccl::reduction reduction,
                            ccl::reduction_fn reduction_fn, const ccl::fn_context* context = nullptr);

// tmp and acc (the reference's fp32 scratch arrays) are accepted and ignored: the kernel accumulates in registers.
ccl::status ccl_comp_batch_reduce(const void* in_buf, const std::vector<size_t>& offsets, size_t in_count,
                                  void* inout_buf, size_t* out_count, const ccl_datatype& dtype,
                                  ccl::reduction reduction, ccl::reduction_fn reduction_fn,
                                  const ccl::fn_context* context, int bf16_keep_precision_mode, float* tmp,
                                  float* acc, ccl_sched* sched = nullptr);

const char* ccl_reduction_to_str(ccl::reduction type);

// src/comp/bf16/bf16.hpp:26-38, src/comp/fp16/fp16.hpp:21-25
void ccl_bf16_reduce(const void* in_buf, size_t in_cnt, void* inout_buf, size_t* out_cnt, ccl::reduction reduction_op,
                     ccl_sched* sched = nullptr);
void ccl_fp16_reduce(const void* in_buf, size_t in_cnt, void* inout_buf, size_t* out_cnt, ccl::reduction reduction_op,
                     ccl_sched* sched = nullptr);
void ccl_convert_fp32_to_bf16_arrays(void* fp32_buf, void* bf16_buf, size_t count, ccl_sched* sched = nullptr);
void ccl_convert_bf16_to_fp32_arrays(void* bf16_buf, float* fp32_buf, size_t count, ccl_sched* sched = nullptr);
// One vector of 16 (bf16.cpp:113-127) or 8 (fp16.cpp:55-61) values, as the reference's functions of these names
// convert; the bf16 narrowing follows CCL_BF16 (avx512bf rounds to nearest even, anything else truncates).
void ccl_convert_fp32_to_bf16(const void* src, void* dst, ccl_sched* sched = nullptr);
void ccl_convert_bf16_to_fp32(const void* src, void* dst, ccl_sched* sched = nullptr);
void ccl_convert_fp32_to_fp16(const void* src, void* dst, ccl_sched* sched = nullptr);
void ccl_convert_fp16_to_fp32(const void* src, void* dst, ccl_sched* sched = nullptr);
// count values at a time (no counterpart of these names in the reference; same result per value)
void ccl_convert_fp32_to_fp16_arrays(const void* fp32_buf, void* fp16_buf, size_t count, ccl_sched* sched = nullptr);
void ccl_convert_fp16_to_fp32_arrays(const void* fp16_buf, float* fp32_buf, size_t count, ccl_sched* sched = nullptr);

// The N-input local reduce of the device path (reduce_monolithic_kernel_N and friends, src/kernels/kernels.cl:269-421):
// out = own OP peers[0] OP peers[1] ..., own first, peers in argument order.  keep_precision as in batch reduce.
ccl::status ccl_comp_reduce_n(ccl_sched* sched, const void* own_buf, const std::vector<const void*>& peer_bufs,
                              size_t count, void* out_buf, const ccl_datatype& dtype, ccl::reduction reduction,
                              int bf16_keep_precision_mode = 0);

// The same reduce with the result stored to every buffer of out_bufs in one pass: the reference's allreduce_kernel
// (src/kernels/kernels.cl:190-217: own and peer output) and, with no peers, write_monolithic_kernel_N
// (src/kernels/kernels.cl:423-560: the own buffer copied to N peers).
ccl::status ccl_comp_reduce_write_n(ccl_sched* sched, const void* own_buf, const std::vector<const void*>& peer_bufs,
                                    size_t count, const std::vector<void*>& out_bufs, const ccl_datatype& dtype,
                                    ccl::reduction reduction, int bf16_keep_precision_mode = 0);

// Many independent reduces in ONE launch -- the reference's read_reduce_write (even[i] = pair[i] + local[i] for every
// peer i, src/coll/algorithms/reduce_scatter/sycl/reduce_scatter_large_sycl_impl.hpp:22-66), reduce_read_write_kernel_N
// (src/kernels/kernels.cl:156-177) and, with one input per job, copy_data.  Job j: dsts[j] = srcs[j * n_inputs] OP ... OP
// srcs[j * n_inputs + n_inputs - 1] over counts[j] elements.
ccl::status ccl_comp_reduce_batch(ccl_sched* sched, const std::vector<const void*>& srcs, int n_inputs,
                                  const std::vector<void*>& dsts, const std::vector<size_t>& counts,
                                  const ccl_datatype& dtype, ccl::reduction reduction, int bf16_keep_precision_mode = 0);
