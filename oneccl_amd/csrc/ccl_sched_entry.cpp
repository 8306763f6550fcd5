// Scheduler entries over the reduction engine (see ccl_sched_entry.hpp).
#include "ccl_sched_entry.hpp"

#include <hip/hip_runtime.h>


namespace {

[[noreturn]] void fail(const std::string& what) {
    throw ccl::exception(what);
}
void check_hip(hipError_t e, const char* what) {
    if (e != hipSuccess)
        fail(std::string(what) + ": " + hipGetErrorString(e));
}
hipStream_t stream_of(ccl_sched* sched) {
    return (hipStream_t)sched->stream;
}

}  // namespace

// ---- ccl_buffer ----------------------------------------------------------------------------------------

void ccl_buffer::check(size_t access_size) const {        // buffer.hpp:34-58
    if (std::numeric_limits<size_t>::max() - offset < access_size)
        fail("ccl_buffer: offset + access_size overflows");
    if (size != -1 && access_size != 0 && offset + access_size > (size_t)size)
        fail("ccl_buffer: unexpected (offset + access_size): size " + std::to_string(size) + ", offset " +
             std::to_string(offset) + ", access_size " + std::to_string(access_size));
}

ccl_buffer ccl_buffer::operator-(size_t val) const {
    if (offset < val)
        fail("ccl_buffer: unexpected decrement value " + std::to_string(val));
    return ccl_buffer(src, size, offset - val);
}

// ---- ccl_sched -----------------------------------------------------------------------------------------

sched_entry* ccl_sched::add_entry(std::shared_ptr<sched_entry> entry) {
    entries.push_back(std::move(entry));
    entries.back()->reset(entries.size() - 1);      // tells the entry its position in the schedule
    return entries.back().get();
}

void ccl_sched::add_barrier() {
    if (!entries.empty())
        entries.back()->make_barrier();
}

// src/sched/sched.cpp:439-490: progress every entry from the first unfinished one; an entry that asks to be called
// again, or a barrier that has not completed with everything before it, stops the walk.
void ccl_sched::do_progress() {
    for (size_t idx = start_idx; idx < entries.size(); ++idx) {
        sched_entry* entry = entries[idx].get();
        entry->do_progress();
        if (entry->get_status() == ccl_sched_entry_status_again)
            break;
        if (idx == start_idx && entry->is_completed())
            ++start_idx;
        else if (entry->is_barrier() && (!entry->is_completed() || start_idx != idx + 1))
            break;
    }
}

void ccl_sched::renew() {
    start_idx = 0;
    for (size_t idx = 0; idx < entries.size(); ++idx) entries[idx]->reset(idx);
}

void* ccl_sched::alloc_buffer(size_t bytes) {
    void* p = nullptr;
    check_hip(hipMalloc(&p, bytes ? bytes : 1), "ccl_sched::alloc_buffer");
    owned_buffers.emplace_back(p, [](void* q) { (void)hipFree(q); });
    return p;
}

// ---- sched_entry ---------------------------------------------------------------------------------------

sched_entry::sched_entry(ccl_sched* sched, bool is_barrier) : sched(sched), barrier(is_barrier) {
    if (!sched)
        fail("no sched");
}

sched_entry::~sched_entry() {
    if (event)
        (void)hipEventDestroy((hipEvent_t)event);
}

void sched_entry::do_progress() {       // entry.cpp:32-130
    if (is_completed())
        return;
    if (status < ccl_sched_entry_status_started) {
        if (status != ccl_sched_entry_status_not_started && status != ccl_sched_entry_status_again)
            fail(std::string("bad status ") + status_to_str(status));
        start();
        if (status < ccl_sched_entry_status_again)
            fail(std::string("bad status ") + status_to_str(status));
    }
    else if (status == ccl_sched_entry_status_started) {
        update();
        if (status < ccl_sched_entry_status_started)
            fail(std::string("bad status ") + status_to_str(status));
    }
    if (status == ccl_sched_entry_status_complete && exec_mode == ccl_sched_entry_exec_once)
        status = ccl_sched_entry_status_complete_once;
    if (status == ccl_sched_entry_status_failed || status == ccl_sched_entry_status_invalid)
        fail(std::string("bad status ") + status_to_str(status));
}

bool sched_entry::is_completed() const {
    return status == ccl_sched_entry_status_complete || status == ccl_sched_entry_status_complete_once;
}

void sched_entry::reset(size_t idx) {   // entry.cpp:146-160
    if (status == ccl_sched_entry_status_complete_once)
        return;
    start_idx = idx;
    status = ccl_sched_entry_status_not_started;
}

void sched_entry::record_started() {
    if (!event) {
        hipEvent_t ev;
        check_hip(hipEventCreateWithFlags(&ev, hipEventDisableTiming), "sched_entry: event");
        event = ev;
    }
    check_hip(hipEventRecord((hipEvent_t)event, stream_of(sched)), "sched_entry: record");
    status = ccl_sched_entry_status_started;
}

void sched_entry::update() {
    hipError_t e = hipEventQuery((hipEvent_t)event);
    if (e == hipSuccess)
        status = ccl_sched_entry_status_complete;
    else if (e != hipErrorNotReady)
        check_hip(e, name());
}

const char* sched_entry::status_to_str(ccl_sched_entry_status status) {     // entry.cpp:232-245
    switch (status) {
        case ccl_sched_entry_status_not_started: return "NOT_STARTED";
        case ccl_sched_entry_status_again: return "AGAIN";
        case ccl_sched_entry_status_started: return "STARTED";
        case ccl_sched_entry_status_complete: return "COMPLETE";
        case ccl_sched_entry_status_complete_once: return "COMPLETE_ONCE";
        case ccl_sched_entry_status_failed: return "FAILED";
        case ccl_sched_entry_status_invalid: return "INVALID";
        default: return "UNKNOWN";
    }
}

void sched_entry::dump(std::stringstream& str, size_t idx) const {
    str << "[" << idx << "] " << name() << " entry, status " << status_to_str(status) << (barrier ? " barrier " : " ");
    dump_detail(str);
}

// ---- REDUCE_LOCAL --------------------------------------------------------------------------------------

reduce_local_entry::reduce_local_entry(ccl_sched* sched, const ccl_buffer in_buf, size_t in_cnt, ccl_buffer inout_buf,
                                       size_t* out_cnt, const ccl_datatype& dtype, ccl::reduction op)
        : sched_entry(sched), in_buf(in_buf), in_cnt(in_cnt), inout_buf(inout_buf), out_cnt(out_cnt), dtype(dtype),
          op(op), fn(sched->coll_attr.reduction_fn) {
    if (op == ccl::reduction::custom && !fn)       // reduce_local_entry.cpp:83-88
        fail("custom reduction requires user provided callback, op custom, fn null");
}

void reduce_local_entry::start() {                  // reduce_local_entry.cpp:100-117
    const size_t bytes = in_cnt * dtype.size();
    const ccl::fn_context context = { sched->coll_attr.match_id.c_str(), inout_buf.get_offset() };
    ccl_comp_reduce(sched, in_buf.get_ptr(bytes), in_cnt, inout_buf.get_ptr(bytes), out_cnt, dtype, op, fn, &context);
    record_started();
}

void reduce_local_entry::dump_detail(std::stringstream& str) const {
    str << "dt " << ccl_datatype_storage::instance().name(dtype) << ", in_buf " << in_buf.get_ptr() << ", in_cnt "
        << in_cnt << ", inout_buf " << inout_buf.get_ptr() << ", out_cnt " << (void*)out_cnt << ", op "
        << ccl_reduction_to_str(op) << ", red_fn " << (void*)fn << "\n";
}

// ---- COPY ----------------------------------------------------------------------------------------------

std::string to_string(copy_direction val) {         // copy_helper.cpp
    switch (val) {
        case copy_direction::undefined: return "UNDEFINED";
        case copy_direction::h2h: return "H2H";
        case copy_direction::d2h: return "D2H";
        case copy_direction::h2d: return "H2D";
        case copy_direction::d2d: return "D2D";
    }
    return "UNKNOWN";
}

copy_entry::copy_entry(ccl_sched* sched, ccl_buffer in_buf, ccl_buffer out_buf, size_t count, const ccl_datatype& dtype,
                       copy_attr attr)
        : sched_entry(sched), in_buf(in_buf), out_buf(out_buf), count(count), dtype(dtype), attr(attr) {
    if (this->attr.direction == copy_direction::undefined) {       // copy_entry.cpp:55-76: decided from the pointers
        hipPointerAttribute_t ai{}, ao{};
        const bool in_dev = hipPointerGetAttributes(&ai, in_buf.get_ptr()) == hipSuccess && ai.type == hipMemoryTypeDevice;
        const bool out_dev = hipPointerGetAttributes(&ao, out_buf.get_ptr()) == hipSuccess && ao.type == hipMemoryTypeDevice;
        (void)hipGetLastError();    // a plain host pointer is reported as an error by some runtimes
        this->attr.direction = in_dev ? (out_dev ? copy_direction::d2d : copy_direction::d2h)
                                      : (out_dev ? copy_direction::h2d : copy_direction::h2h);
    }
}

void copy_entry::start() {
    const size_t bytes = dtype.size() * count;
    if (bytes == 0) {
        status = ccl_sched_entry_status_complete;
        return;
    }
    const void* in = (const char*)in_buf.get_ptr(bytes + attr.in_buf_offset * dtype.size()) + attr.in_buf_offset * dtype.size();
    void* out = (char*)out_buf.get_ptr(bytes + attr.out_buf_offset * dtype.size()) + attr.out_buf_offset * dtype.size();
    switch (attr.direction) {
        case copy_direction::d2d:       // the reference's do_regular_copy -> ccl_comp_copy (copy_entry.cpp:201-207)
            ccl_comp_copy(in, out, bytes, attr.use_nontemporal, sched);
            break;
        case copy_direction::h2d: check_hip(hipMemcpyAsync(out, in, bytes, hipMemcpyHostToDevice, stream_of(sched)), "COPY h2d"); break;
        case copy_direction::d2h: check_hip(hipMemcpyAsync(out, in, bytes, hipMemcpyDeviceToHost, stream_of(sched)), "COPY d2h"); break;
        case copy_direction::h2h: check_hip(hipMemcpyAsync(out, in, bytes, hipMemcpyHostToHost, stream_of(sched)), "COPY h2h"); break;
        default: fail("unknown copy type");
    }
    record_started();
}

void copy_entry::dump_detail(std::stringstream& str) const {
    str << "dt " << ccl_datatype_storage::instance().name(dtype) << ", count " << count << ", in_buf " << in_buf.get_ptr()
        << ", out_buf " << out_buf.get_ptr() << ", in_buf_offset " << attr.in_buf_offset << ", out_buf_offset "
        << attr.out_buf_offset << ", direction " << to_string(attr.direction) << "\n";
}

// ---- RECV_REDUCE ---------------------------------------------------------------------------------------

recv_reduce_entry::recv_reduce_entry(ccl_sched* sched, ccl_buffer inout_buf, size_t cnt, const ccl_datatype& dtype,
                                     ccl::reduction reduction_op, int src, ccl_comm* comm, ccl_buffer comm_buf,
                                     ccl_recv_reduce_result_buf_type result_buf_type)
        : sched_entry(sched), inout_buf(inout_buf), in_cnt(cnt), dtype(dtype), op(reduction_op), src(src), comm(comm),
          comm_buf(comm_buf), result_buf_type(result_buf_type), fn(sched->coll_attr.reduction_fn) {
    if (op == ccl::reduction::custom && !fn)
        fail("custom reduction requires user provided callback, op custom, fn null");
    if (!comm || !comm->get_atl_comm())
        fail("RECV_REDUCE needs a communicator with a transport");
    if (!((result_buf_type == ccl_recv_reduce_local_buf && inout_buf.get_ptr() != nullptr) ||
          (result_buf_type == ccl_recv_reduce_comm_buf && comm_buf.get_ptr() != nullptr)))
        fail("result buffer should be non null");                          // recv_reduce_entry.hpp:67-71
    if ((comm_buf.get_ptr() == nullptr || comm_buf == inout_buf) && in_cnt) {   // :73-75
        const size_t bytes = in_cnt * dtype.size();
        this->comm_buf = ccl_buffer(sched->alloc_buffer(bytes), (ssize_t)bytes);
    }
}

recv_reduce_entry::~recv_reduce_entry() {
    if (status == ccl_sched_entry_status_started && !reducing)      // :78-85
        comm->get_atl_comm()->cancel(req);
}

void recv_reduce_entry::start() {       // :87-108
    // src/atl/util/pm/... tag_creator: source rank, communicator and position in the schedule identify the message
    atl_tag = ((uint64_t)comm->get_comm_id() << 48) | ((uint64_t)(uint32_t)src << 24) | (uint64_t)(start_idx & 0xffffff);
    const size_t bytes = in_cnt * dtype.size();
    reducing = false;
    req = atl_req_t{};
    atl_status_t st = comm->get_atl_comm()->recv(comm_buf.get_ptr(bytes), bytes, src, atl_tag, req);
    if (st == ATL_STATUS_AGAIN) {        // entry.cpp update_status
        status = ccl_sched_entry_status_again;
        return;
    }
    if (st != ATL_STATUS_SUCCESS)
        fail("RECV_REDUCE entry failed to post the receive");
    status = ccl_sched_entry_status_started;
}

void recv_reduce_entry::update() {      // :110-146
    if (!reducing) {
        if (comm->get_atl_comm()->check(req) != ATL_STATUS_SUCCESS)
            fail("RECV_REDUCE entry failed");
        if (!req.is_completed)
            return;
        const size_t bytes = in_cnt * dtype.size();
        const ccl::fn_context context = { sched->coll_attr.match_id.c_str(), inout_buf.get_offset() };
        const ccl_buffer& reduce_in = (result_buf_type == ccl_recv_reduce_local_buf) ? comm_buf : inout_buf;
        const ccl_buffer& reduce_inout = (result_buf_type == ccl_recv_reduce_local_buf) ? inout_buf : comm_buf;
        ccl_comp_reduce(sched, reduce_in.get_ptr(bytes), in_cnt, reduce_inout.get_ptr(bytes), nullptr, dtype, op, fn, &context);
        reducing = true;
        record_started();
    }
    sched_entry::update();
}

void recv_reduce_entry::reset(size_t idx) {
    sched_entry::reset(idx);
    reducing = false;
}

void recv_reduce_entry::dump_detail(std::stringstream& str) const {
    str << "dt " << ccl_datatype_storage::instance().name(dtype) << ", inout_buf " << inout_buf.get_ptr() << ", in_cnt "
        << in_cnt << ", op " << ccl_reduction_to_str(op) << ", red_fn " << (void*)fn << ", src " << src << ", atl_tag "
        << atl_tag << ", comm_id " << comm->get_comm_id() << ", comm_buf " << comm_buf.get_ptr() << ", result_buf_type "
        << (int)result_buf_type << "\n";
}

// ---- monolithic kernels --------------------------------------------------------------------------------

reduce_monolithic_entry::reduce_monolithic_entry(ccl_sched* sched, ccl_buffer send_buf, size_t rank_buf_offset,
                                                 size_t block_count, const std::vector<ccl_buffer>& peer_send_bufs,
                                                 size_t peer_buf_offset, ccl_buffer output_buf, const ccl_datatype& dtype,
                                                 ccl::reduction op, int bf16_keep_precision_mode)
        : sched_entry(sched), send_buf(send_buf), rank_buf_offset(rank_buf_offset), block_count(block_count),
          peer_send_bufs(peer_send_bufs), peer_buf_offset(peer_buf_offset), output_buf(output_buf), dtype(dtype), op(op),
          keep(bf16_keep_precision_mode) {
    if (op == ccl::reduction::custom)
        fail("custom reduction is not available for the N-input device reduce");
}

void reduce_monolithic_entry::start() {     // ze_a2a_reduce_scatter_entry.cpp:64-106
    const size_t esz = dtype.size(), bytes = block_count * esz;
    const void* own = (const char*)send_buf.get_ptr(rank_buf_offset * esz + bytes) + rank_buf_offset * esz;
    std::vector<const void*> peers;
    for (const ccl_buffer& p : peer_send_bufs) {
        const size_t off = (rank_buf_offset + peer_buf_offset) * esz;
        peers.push_back((const char*)p.get_ptr(off + bytes) + off);
    }
    ccl_comp_reduce_n(sched, own, peers, block_count, output_buf.get_ptr(bytes), dtype, op, keep);
    record_started();
}

write_monolithic_entry::write_monolithic_entry(ccl_sched* sched, ccl_buffer src_buf, size_t copy_count,
                                               const std::vector<ccl_buffer>& peer_dst_bufs, const ccl_datatype& dtype)
        : sched_entry(sched), src_buf(src_buf), copy_count(copy_count), peer_dst_bufs(peer_dst_bufs), dtype(dtype) {
    if (peer_dst_bufs.empty())
        fail("WRITE_MONOLITHIC needs at least one destination");
}

void write_monolithic_entry::start() {      // ze_a2a_allgatherv_entry.cpp:526-585
    const size_t bytes = copy_count * dtype.size();
    if (bytes == 0) {
        status = ccl_sched_entry_status_complete;
        return;
    }
    std::vector<void*> dsts;
    for (const ccl_buffer& p : peer_dst_bufs) dsts.push_back(p.get_ptr(bytes));
    // a copy is the same for every element type: move bytes
    const ccl_datatype& u8 = ccl_datatype_storage::instance().get(ccl::datatype::uint8);
    ccl_comp_reduce_write_n(sched, src_buf.get_ptr(bytes), {}, bytes, dsts, u8, ccl::reduction::sum, 0);
    record_started();
}
