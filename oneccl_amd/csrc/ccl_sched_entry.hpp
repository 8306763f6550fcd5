// Scheduler entries over the MI355X reduction engine, with the shapes oneCCL's schedules are built from
// (src/sched/entry/entry.hpp:31-129, reduce_local_entry.hpp, recv_reduce_entry.hpp, copy/copy_entry.hpp and the
// kernel launch sites of ze/ze_a2a_reduce_scatter_entry.cpp and ze/ze_a2a_allgatherv_entry.cpp): same class names,
// constructor arguments and status machine, so that a schedule written against the reference's entries runs its
// local-reduce, copy and receive-then-reduce steps on device buffers.
//
// An entry's start() enqueues its kernels on the schedule's HIP stream and records an event; update() polls the
// event.  Entries that only enqueue device work (REDUCE_LOCAL, COPY, the monolithic kernels) are ordered by the
// stream they share.  RECV_REDUCE enqueues its reduce only once the receive has completed, so whatever depends on
// it must sit behind a barrier -- ccl_sched::add_barrier() after the step, exactly where the reference's algorithms
// put one (e.g. src/coll/algorithms/allreduce/allreduce.cpp:185-194): a barrier entry holds later entries back
// until it and everything before it have completed (src/sched/sched.cpp:439-490).
#pragma once

#include <sys/types.h>

#include <limits>
#include <sstream>

#include "ccl_comp.hpp"

// src/sched/entry/entry.hpp:35-45
enum ccl_sched_entry_exec_mode { ccl_sched_entry_exec_regular, ccl_sched_entry_exec_once };
enum ccl_sched_entry_status {
    ccl_sched_entry_status_not_started,
    ccl_sched_entry_status_again,
    ccl_sched_entry_status_started,
    ccl_sched_entry_status_complete,
    ccl_sched_entry_status_complete_once,   // higher than 'complete'
    ccl_sched_entry_status_failed,
    ccl_sched_entry_status_invalid
};

// src/common/utils/buffer.hpp:27-230 (direct buffers only): base pointer, size for bounds checks (-1: unknown), offset
class ccl_buffer {
public:
    ccl_buffer() : ccl_buffer(nullptr, -1, 0) {}
    ccl_buffer(void* src, ssize_t size, size_t offset = 0) : src(src), size(size), offset(offset) { check(0); }
    void set(void* s, ssize_t sz = -1, size_t off = 0) { src = s; size = sz; offset = off; check(0); }
    void* get_src() const { return src; }
    ssize_t get_size() const { return size; }
    size_t get_offset() const { return offset; }
    ccl_buffer operator+(size_t val) const { return ccl_buffer(src, size, offset + val); }
    ccl_buffer operator-(size_t val) const;
    ccl_buffer& operator+=(size_t val) { offset += val; check(0); return *this; }
    // throws when [offset, offset + access_size) leaves the buffer
    void* get_ptr(size_t access_size = 0) const { check(access_size); return src ? (char*)src + offset : nullptr; }
    bool operator==(const ccl_buffer& o) const { return get_ptr() == o.get_ptr(); }
    bool operator!=(const ccl_buffer& o) const { return !(*this == o); }
    explicit operator bool() const { return src != nullptr; }

private:
    void check(size_t access_size) const;
    void* src;
    ssize_t size;
    size_t offset;
};

// src/sched/entry/entry.hpp:58-129 without the flow-control credits, timers and ITT hooks
class sched_entry {
public:
    explicit sched_entry(ccl_sched* sched, bool is_barrier = false);
    virtual ~sched_entry();
    sched_entry(const sched_entry&) = delete;
    sched_entry& operator=(const sched_entry&) = delete;

    void do_progress();
    bool is_completed() const;
    virtual void reset(size_t idx);
    virtual bool is_strict_order_satisfied() const { return status >= ccl_sched_entry_status_started; }
    void make_barrier() { barrier = true; }
    bool is_barrier() const { return barrier; }
    ccl_sched_entry_status get_status() const { return status; }
    void set_status(ccl_sched_entry_status s) { status = s; }
    void set_exec_mode(ccl_sched_entry_exec_mode mode) { exec_mode = mode; }
    virtual const char* name() const = 0;
    static const char* status_to_str(ccl_sched_entry_status status);
    void dump(std::stringstream& str, size_t idx) const;
    ccl_sched* get_sched() const { return sched; }

protected:
    virtual void start() = 0;
    virtual void update();                  // default: complete when the recorded event has fired
    virtual void dump_detail(std::stringstream&) const {}
    void record_started();                  // record the event on the schedule's stream, status = started

    ccl_sched* sched;
    bool barrier;
    size_t start_idx = 0;
    ccl_sched_entry_status status = ccl_sched_entry_status_not_started;
    ccl_sched_entry_exec_mode exec_mode = ccl_sched_entry_exec_regular;
    void* event = nullptr;                  // hipEvent_t, created on first use
};

// src/sched/entry/factory/entry_factory.hpp: entry_factory::create<T>(sched, args...) appends a new entry
namespace entry_factory {
template <class EntryType, class... Args>
EntryType* create(ccl_sched* sched, Args&&... args) {
    auto e = std::make_shared<EntryType>(sched, std::forward<Args>(args)...);
    return static_cast<EntryType*>(sched->add_entry(std::move(e)));
}
}  // namespace entry_factory

// ---- REDUCE_LOCAL: inout = inout OP in (src/sched/entry/reduce_local_entry.hpp:26-91, .cpp:68-143) ----
class reduce_local_entry : public sched_entry {
public:
    static constexpr const char* class_name() noexcept { return "REDUCE_LOCAL"; }
    const char* name() const noexcept override { return class_name(); }
    reduce_local_entry(ccl_sched* sched, const ccl_buffer in_buf, size_t in_cnt, ccl_buffer inout_buf, size_t* out_cnt,
                       const ccl_datatype& dtype, ccl::reduction op);
    void start() override;

protected:
    void dump_detail(std::stringstream& str) const override;

private:
    const ccl_buffer in_buf;
    const size_t in_cnt;
    const ccl_buffer inout_buf;
    size_t* out_cnt;
    const ccl_datatype dtype;
    const ccl::reduction op;
    const ccl::reduction_fn fn;
};

// ---- COPY (src/sched/entry/copy/copy_entry.hpp:27-69, copy_helper.hpp:31-71) ----
enum class copy_direction { undefined, h2h, d2h, h2d, d2d };
std::string to_string(copy_direction val);
struct copy_attr {
    copy_direction direction = copy_direction::d2d;
    size_t in_buf_offset = 0;       // in elements, added to the buffers' own offsets
    size_t out_buf_offset = 0;
    bool use_nontemporal = false;
    copy_attr() = default;
    copy_attr(copy_direction direction, size_t in_buf_offset = 0, size_t out_buf_offset = 0)
            : direction(direction), in_buf_offset(in_buf_offset), out_buf_offset(out_buf_offset) {}
};
class copy_entry : public sched_entry {
public:
    static constexpr const char* class_name() noexcept { return "COPY"; }
    const char* name() const noexcept override { return class_name(); }
    copy_entry(ccl_sched* sched, ccl_buffer in_buf, ccl_buffer out_buf, size_t count, const ccl_datatype& dtype,
               copy_attr attr = {});
    void start() override;

protected:
    void dump_detail(std::stringstream& str) const override;

private:
    ccl_buffer in_buf, out_buf;
    const size_t count;
    const ccl_datatype dtype;
    copy_attr attr;
};

// ---- RECV_REDUCE (src/sched/entry/recv_reduce_entry.hpp:26-181) ----
// The transport is what the entry uses of atl_base_comm (src/atl/atl_base_comm.hpp): post a receive into a device
// buffer, poll it, cancel it.  A receive is complete when the data is visible to work enqueued afterwards on any
// stream of this device.
enum atl_status_t { ATL_STATUS_SUCCESS = 0, ATL_STATUS_FAILURE, ATL_STATUS_AGAIN, ATL_STATUS_UNSUPPORTED };
struct atl_req_t {
    int is_completed = 0;
    void* internal = nullptr;
};
class atl_base_comm {
public:
    virtual ~atl_base_comm() {}
    virtual atl_status_t recv(void* buf, size_t bytes, int src, uint64_t tag, atl_req_t& req) = 0;
    virtual atl_status_t check(atl_req_t& req) = 0;
    virtual void cancel(atl_req_t& req) = 0;
};
struct ccl_comm {
    int m_rank = 0, m_size = 1;
    uint16_t comm_id = 0;
    atl_base_comm* atl = nullptr;
    int rank() const { return m_rank; }
    int size() const { return m_size; }
    uint16_t get_comm_id() const { return comm_id; }
    atl_base_comm* get_atl_comm() const { return atl; }
};
enum ccl_recv_reduce_result_buf_type { ccl_recv_reduce_local_buf, ccl_recv_reduce_comm_buf };
class recv_reduce_entry final : public sched_entry {
public:
    static constexpr const char* class_name() noexcept { return "RECV_REDUCE"; }
    const char* name() const override { return class_name(); }
    recv_reduce_entry(ccl_sched* sched, ccl_buffer inout_buf, size_t cnt, const ccl_datatype& dtype,
                      ccl::reduction reduction_op, int src, ccl_comm* comm, ccl_buffer comm_buf = ccl_buffer(),
                      ccl_recv_reduce_result_buf_type result_buf_type = ccl_recv_reduce_local_buf);
    ~recv_reduce_entry() override;
    void start() override;
    void update() override;
    void reset(size_t idx) override;

protected:
    void dump_detail(std::stringstream& str) const override;

private:
    ccl_buffer inout_buf;
    size_t in_cnt;
    ccl_datatype dtype;
    ccl::reduction op;
    int src;
    ccl_comm* comm;
    ccl_buffer comm_buf;
    ccl_recv_reduce_result_buf_type result_buf_type;
    uint64_t atl_tag = 0;
    ccl::reduction_fn fn;
    atl_req_t req{};
    bool reducing = false;      // the receive has completed and the reduce is enqueued
};

// ---- the monolithic kernels of the a2a algorithms ----
// REDUCE_MONOLITHIC: out = own block OP peer blocks, own first, peers in order -- the kernel launch of
// ze_a2a_reduce_scatter_entry::kernel_init (src/sched/entry/ze/ze_a2a_reduce_scatter_entry.cpp:48-136): the own
// block starts rank_buf_offset elements into send_buf, peer p's block (rank_buf_offset + peer_buf_offset)
// elements into peer_send_bufs[p].  The alignment split into two launches that the reference does by hand
// (:78-106) happens inside the kernel here.
class reduce_monolithic_entry : public sched_entry {
public:
    static constexpr const char* class_name() noexcept { return "REDUCE_MONOLITHIC"; }
    const char* name() const noexcept override { return class_name(); }
    reduce_monolithic_entry(ccl_sched* sched, ccl_buffer send_buf, size_t rank_buf_offset, size_t block_count,
                            const std::vector<ccl_buffer>& peer_send_bufs, size_t peer_buf_offset,
                            ccl_buffer output_buf, const ccl_datatype& dtype, ccl::reduction op,
                            int bf16_keep_precision_mode = 0);
    void start() override;

private:
    ccl_buffer send_buf;
    size_t rank_buf_offset, block_count;
    std::vector<ccl_buffer> peer_send_bufs;
    size_t peer_buf_offset;
    ccl_buffer output_buf;
    ccl_datatype dtype;
    ccl::reduction op;
    int keep;
};
// WRITE_MONOLITHIC: the own block copied into every peer's receive buffer -- the kernel launch of
// ze_a2a_allgatherv_op (src/sched/entry/ze/ze_a2a_allgatherv_entry.cpp:526-585).
class write_monolithic_entry : public sched_entry {
public:
    static constexpr const char* class_name() noexcept { return "WRITE_MONOLITHIC"; }
    const char* name() const noexcept override { return class_name(); }
    write_monolithic_entry(ccl_sched* sched, ccl_buffer src_buf, size_t copy_count,
                           const std::vector<ccl_buffer>& peer_dst_bufs, const ccl_datatype& dtype);
    void start() override;

private:
    ccl_buffer src_buf;
    size_t copy_count;
    std::vector<ccl_buffer> peer_dst_bufs;
    ccl_datatype dtype;
};
