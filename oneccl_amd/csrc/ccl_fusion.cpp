// Fusion manager host logic (see ccl_fusion.hpp).  No device code and no HIP calls in this file.
#include "ccl_fusion.hpp"

#include <stdlib.h>

#include <thread>

namespace {
[[noreturn]] void fusion_fail(const std::string& what) {
    throw ccl::exception(what);
}
}  // namespace

ccl_fusion_config ccl_fusion_config::from_env() {
    ccl_fusion_config c;
    if (const char* v = getenv("CCL_FUSION_BYTES_THRESHOLD"))
        c.bytes_threshold = strtoull(v, nullptr, 10);
    if (const char* v = getenv("CCL_FUSION_COUNT_THRESHOLD"))
        c.count_threshold = strtoull(v, nullptr, 10);
    if (const char* v = getenv("CCL_FUSION_CHECK_URGENT"))
        c.check_urgent = atoi(v) != 0;
    if (const char* v = getenv("CCL_FUSION_CYCLE_MS"))
        c.cycle_ms = atof(v);
    return c;
}

bool ccl_fusion_request::is_completed() {
    int s = state.load(std::memory_order_acquire);
    if (s == 0)
        return true;
    if (s == 1)
        return false;
    if (backend && done_token && !backend->ready(done_token))
        return false;
    done_token.reset();
    state.store(0, std::memory_order_release);
    return true;
}

ccl_fusion_manager::ccl_fusion_manager(ccl_fusion_backend* b, ccl_fused_allreduce_fn fn, const ccl_fusion_config& c)
        : backend(b),
          allreduce(std::move(fn)),
          cfg(c),
          buffer_bytes(c.bytes_threshold * c.count_threshold) {
    if (!backend || !allreduce)
        fusion_fail("fusion manager needs a backend and a collective");
    if (cfg.bytes_threshold < 1)                       // fusion.cpp:48-50
        fusion_fail("unexpected fusion_bytes_threshold " + std::to_string(cfg.bytes_threshold));
    if (cfg.count_threshold < 1)
        fusion_fail("unexpected fusion_count_threshold " + std::to_string(cfg.count_threshold));
    cycle = std::chrono::microseconds((long)(cfg.cycle_ms * 1000.0));
    last_exec_time = std::chrono::steady_clock::now();
}

ccl_fusion_manager::~ccl_fusion_manager() {
    reset();
    for (void* b : free_buffers) backend->release(b);
}

bool ccl_fusion_manager::can_reset() {
    check_tracked(false);
    return tracked.empty();
}

void ccl_fusion_manager::reset() {
    while (!tracked.empty()) check_tracked(true);
}

bool ccl_fusion_manager::can_fuse(const ccl_fusion_request* req) const {
    const size_t bytes = req->count * req->dtype.size();
    if (bytes >= cfg.bytes_threshold)                  // fusion.cpp:108-113
        return false;
    if (req->deps)                                     // :115-118
        return false;
    if (req->reduction_fn || req->reduction == ccl::reduction::custom || req->synchronous)   // :120-123
        return false;
    return true;
}

bool ccl_fusion_manager::add(ccl_fusion_request* req) {
    if (!can_fuse(req))
        return false;
    if (req->state.load(std::memory_order_acquire) != 0)
        fusion_fail("incorrect completion counter");   // fusion.cpp:134
    req->backend = backend;
    req->state.store(1, std::memory_order_release);
    std::lock_guard<std::mutex> lock(guard);
    postponed_queue.push_back(req);
    return true;
}

void ccl_fusion_manager::execute() {
    auto now = std::chrono::steady_clock::now();
    if (last_exec_time + cycle > now) {                // too early, do nothing (fusion.cpp:379-385)
        st.empty_exec_calls++;
        return;
    }
    last_exec_time = now;

    bool flush = false;
    if (cfg.check_urgent) {
        // a request already gathered may have become urgent since the previous call (fusion.cpp:388-398)
        for (ccl_fusion_request* r : exec_queue)
            if (r->urgent.load(std::memory_order_relaxed)) {
                flush = true;
                break;
            }
    }
    {
        std::lock_guard<std::mutex> lock(guard);
        if (!postponed_queue.empty()) {
            ccl_fusion_request* first;
            if (!exec_queue.empty()) {
                first = exec_queue.front();
            }
            else {
                first = postponed_queue.front();
                exec_queue.push_back(first);
                postponed_queue.pop_front();
                exec_queue_sum_bytes = first->count * first->dtype.size();
                if (cfg.check_urgent && first->urgent.load(std::memory_order_relaxed))
                    flush = true;
            }
            for (auto it = postponed_queue.begin(); it != postponed_queue.end();) {
                ccl_fusion_request* s = *it;
                // only requests of one dtype / communicator / reduction / stream share a buffer (fusion.cpp:420-424)
                if (s->dtype.idx() == first->dtype.idx() && s->comm == first->comm &&
                    s->reduction == first->reduction && s->stream == first->stream) {
                    const size_t size = s->count * s->dtype.size();
                    if (exec_queue_sum_bytes + size > buffer_bytes) {      // too many bytes: flush what we have
                        flush = true;
                        break;
                    }
                    exec_queue_sum_bytes += size;
                    if (cfg.check_urgent && s->urgent.load(std::memory_order_relaxed))
                        flush = true;
                    exec_queue.push_back(s);
                    it = postponed_queue.erase(it);
                    if (exec_queue.size() == cfg.count_threshold) {        // too many requests: flush
                        flush = true;
                        break;
                    }
                }
                else {
                    ++it;
                }
            }
        }
    }
    if (flush && !exec_queue.empty())
        build_and_start();
    check_tracked(false);
}

// One fused operation: pack every queued send buffer at its running offset, one collective over the whole buffer,
// unpack to the receive buffers, then every request completes (fusion.cpp:145-376).
void ccl_fusion_manager::build_and_start() {
    ccl_fusion_request* first = exec_queue.front();
    const ccl_datatype dtype = first->dtype;
    std::vector<const void*> sends;
    std::vector<void*> recvs;
    std::vector<size_t> counts;
    size_t sum_count = 0;
    for (ccl_fusion_request* r : exec_queue) {
        sends.push_back(r->send_buf);
        recvs.push_back(r->recv_buf);
        counts.push_back(r->count);
        sum_count += r->count;
    }
    void* buf;
    if (!free_buffers.empty()) {
        buf = free_buffers.back();
        free_buffers.pop_back();
    }
    else {
        buf = backend->alloc(buffer_bytes);
        if (!buf)
            fusion_fail("fusion buffer allocation failed");
    }
    std::shared_ptr<void> token;
    try {
        backend->pack(sends, counts, dtype, buf, first->stream);
        allreduce(buf, sum_count, dtype, first->reduction, first->comm, first->stream);
        backend->unpack(buf, recvs, counts, dtype, first->stream);
        token = backend->record(first->stream);
    }
    catch (...) {
        // the gathered requests stay queued (the next flush tries them again); the buffer may still be in use by
        // whatever was enqueued before the failure, so it is tracked until the stream has drained
        try {
            tracked.push_back(launched_t{ buf, backend->record(first->stream) });
        }
        catch (...) {
            free_buffers.push_back(buf);
        }
        throw;
    }
    for (ccl_fusion_request* r : exec_queue) {
        r->done_token = token;
        r->urgent.store(false, std::memory_order_relaxed);
        r->state.store(2, std::memory_order_release);
    }
    tracked.push_back(launched_t{ buf, token });
    st.fused_ops += exec_queue.size();
    st.fused_bytes += sum_count * dtype.size();
    st.fused_launches++;
    exec_queue.clear();
    exec_queue_sum_bytes = 0;
}

// Fusion buffers go back to the cache when the operation that used them is done (fusion.cpp:468-492).
void ccl_fusion_manager::check_tracked(bool wait) {
    for (auto it = tracked.begin(); it != tracked.end();) {
        if (backend->ready(it->token)) {
            free_buffers.push_back(it->buf);
            it = tracked.erase(it);
        }
        else {
            ++it;
        }
    }
    if (wait && !tracked.empty())
        std::this_thread::yield();
}
