// Host logic of oneCCL's fusion manager (src/fusion/fusion.hpp:24-73, src/fusion/fusion.cpp) in front of the fusion
// kernels: small allreduce requests are postponed, gathered into an execution queue until a threshold or an urgent
// request flushes it, packed into one cached fusion buffer, reduced with ONE collective over the fused buffer, and
// unpacked, after which every request completes.
//
// The manager itself is plain C++ (no HIP): everything that touches a device goes through ccl_fusion_backend, so the
// queueing logic can be exercised on the host with a mock backend.  ccl_fusion_hip_backend (ccl_fusion_hip.cpp) binds
// it to the C ABI of mi_ccl_comp.h.
#pragma once

#include <atomic>
#include <chrono>
#include <deque>
#include <functional>
#include <list>
#include <map>
#include <memory>
#include <mutex>
#include <vector>

#include "ccl_comp.hpp"

// The fields of a postponed allreduce schedule that the manager looks at (coll_param / coll_attr / request of
// src/fusion/fusion.cpp:97-127,420-424 and src/exec/exec.cpp:271-289).
struct ccl_fusion_request {
    const void* send_buf = nullptr;
    void* recv_buf = nullptr;
    size_t count = 0;
    ccl_datatype dtype;
    ccl::reduction reduction = ccl::reduction::sum;
    ccl::reduction_fn reduction_fn = nullptr;   // a custom reduction cannot be fused
    bool synchronous = false;                   // neither can a synchronous call
    size_t deps = 0;                            // nor one with dependencies
    const void* comm = nullptr;                 // requests fuse only within one communicator ...
    void* stream = nullptr;                     // ... and one stream
    std::atomic<bool> urgent{ false };          // set by a waiter: flush the queue this request sits in

    // true once the fused operation that carried it has finished; call it from one thread at a time per request
    bool is_completed();

private:
    friend class ccl_fusion_manager;
    std::shared_ptr<void> done_token;           // backend completion token of the fused operation
    class ccl_fusion_backend* backend = nullptr;
    std::atomic<int> state{ 0 };                // 0 idle/completed, 1 postponed or queued, 2 launched
};

// What the manager needs from a device.  All calls are asynchronous on `stream` except alloc/release.
class ccl_fusion_backend {
public:
    virtual ~ccl_fusion_backend() {}
    virtual void* alloc(size_t bytes) = 0;
    virtual void release(void* buf) = 0;
    // tensors[i] holds counts[i] elements; tensor i sits at a running byte offset in fusion_buf (tight layout,
    // src/fusion/fusion.cpp:314)
    virtual void pack(const std::vector<const void*>& tensors, const std::vector<size_t>& counts,
                      const ccl_datatype& dtype, void* fusion_buf, void* stream) = 0;
    virtual void unpack(const void* fusion_buf, const std::vector<void*>& tensors, const std::vector<size_t>& counts,
                        const ccl_datatype& dtype, void* stream) = 0;
    // a token that becomes ready when everything enqueued on `stream` so far has finished
    virtual std::shared_ptr<void> record(void* stream) = 0;
    virtual bool ready(const std::shared_ptr<void>& token) = 0;
};

// The collective that runs over the fused buffer, in place: buf holds sum_count elements.
typedef std::function<void(void* buf, size_t sum_count, const ccl_datatype& dtype, ccl::reduction reduction,
                           const void* comm, void* stream)>
    ccl_fused_allreduce_fn;

struct ccl_fusion_config {          // CCL_FUSION_* of src/common/env/env.cpp:118-122,432-448
    size_t bytes_threshold = 16384;
    size_t count_threshold = 256;
    bool check_urgent = true;
    double cycle_ms = 0.2;
    static ccl_fusion_config from_env();
};

class ccl_fusion_manager {
public:
    ccl_fusion_manager(ccl_fusion_backend* backend, ccl_fused_allreduce_fn allreduce,
                       const ccl_fusion_config& cfg = ccl_fusion_config::from_env());
    ~ccl_fusion_manager();
    ccl_fusion_manager(const ccl_fusion_manager&) = delete;
    ccl_fusion_manager& operator=(const ccl_fusion_manager&) = delete;

    bool can_fuse(const ccl_fusion_request* req) const;   // fusion.cpp:97-127
    bool add(ccl_fusion_request* req);                     // fusion.cpp:129-143; false: run it unfused
    void execute();                                        // fusion.cpp:378-466; call periodically
    void reset();                                          // wait for everything launched, release buffers
    bool can_reset();

    size_t buffer_size() const { return buffer_bytes; }
    struct stats_t {
        size_t fused_ops = 0, fused_bytes = 0, fused_launches = 0, empty_exec_calls = 0;
    };
    stats_t stats() const { return st; }

private:
    void build_and_start();                                // fusion.cpp:145-376
    void check_tracked(bool wait);

    ccl_fusion_backend* backend;
    ccl_fused_allreduce_fn allreduce;
    const ccl_fusion_config cfg;
    const size_t buffer_bytes;                             // bytes_threshold * count_threshold (fusion.cpp:45-47)

    std::mutex guard;
    std::deque<ccl_fusion_request*> postponed_queue;
    std::deque<ccl_fusion_request*> exec_queue;
    size_t exec_queue_sum_bytes = 0;

    struct launched_t {
        void* buf;
        std::shared_ptr<void> token;
    };
    std::list<launched_t> tracked;                         // fused operations in flight
    std::vector<void*> free_buffers;                       // the buffer cache of fusion.cpp:189

    std::chrono::steady_clock::duration cycle;
    std::chrono::steady_clock::time_point last_exec_time;
    stats_t st;
};

// Backend over libmi_ccl_comp.so: device buffers from hipMalloc, pack/unpack through cached fusion plans
// (mi_ccl_fusion_pack / mi_ccl_fusion_unpack), completion through HIP events.
class ccl_fusion_hip_backend : public ccl_fusion_backend {
public:
    ccl_fusion_hip_backend();
    ~ccl_fusion_hip_backend() override;
    void* alloc(size_t bytes) override;
    void release(void* buf) override;
    void pack(const std::vector<const void*>& tensors, const std::vector<size_t>& counts, const ccl_datatype& dtype,
              void* fusion_buf, void* stream) override;
    void unpack(const void* fusion_buf, const std::vector<void*>& tensors, const std::vector<size_t>& counts,
                const ccl_datatype& dtype, void* stream) override;
    std::shared_ptr<void> record(void* stream) override;
    bool ready(const std::shared_ptr<void>& token) override;

private:
    struct impl;
    impl* p;
};
