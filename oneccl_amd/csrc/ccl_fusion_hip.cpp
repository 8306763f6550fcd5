// ccl_fusion_hip_backend: the fusion manager's device side over the C ABI (see ccl_fusion.hpp).
#include <hip/hip_runtime.h>

#include "../../include/mi_ccl_comp.h"
#include "ccl_fusion.hpp"
#include "ccl_trace.hpp"

struct ccl_fusion_hip_backend::impl {
    // fusion plans cached by (dtype, counts), the way the reference caches the fused schedule by its key
    // (src/fusion/fusion.cpp:206-237)
    std::map<std::pair<int, std::vector<size_t>>, mi_ccl_fusion_plan*> plans;
    std::mutex lock;
    static constexpr size_t kMaxPlans = 256;

    mi_ccl_fusion_plan* plan_for(const std::vector<size_t>& counts, const ccl_datatype& dtype) {
        std::lock_guard<std::mutex> g(lock);
        auto key = std::make_pair((int)dtype.idx(), counts);
        auto it = plans.find(key);
        if (it != plans.end())
            return it->second;
        // a workload whose tensor sets never repeat must not grow the cache without bound: start over when it is
        // full (destroying a plan frees device memory, which waits for the kernels that still read it)
        if (plans.size() >= kMaxPlans) {
            for (auto& kv : plans) mi_ccl_fusion_plan_destroy(kv.second);
            plans.clear();
        }
        mi_ccl_fusion_plan* plan = nullptr;
        int rc = mi_ccl_fusion_plan_create(counts.data(), counts.size(), (int)dtype.idx(), /*align=*/1, &plan);
        if (rc != MI_CCL_SUCCESS)
            throw ccl::exception(std::string("mi_ccl_fusion_plan_create: ") + mi_ccl_status_str(rc));
        plans[key] = plan;
        return plan;
    }
};

ccl_fusion_hip_backend::ccl_fusion_hip_backend() : p(new impl) {}

ccl_fusion_hip_backend::~ccl_fusion_hip_backend() {
    for (auto& kv : p->plans) mi_ccl_fusion_plan_destroy(kv.second);
    delete p;
}

void* ccl_fusion_hip_backend::alloc(size_t bytes) {
    void* buf = nullptr;
    return hipMalloc(&buf, bytes) == hipSuccess ? buf : nullptr;
}

void ccl_fusion_hip_backend::release(void* buf) {
    (void)hipFree(buf);
}

void ccl_fusion_hip_backend::pack(const std::vector<const void*>& tensors, const std::vector<size_t>& counts,
                                  const ccl_datatype& dtype, void* fusion_buf, void* stream) {
    ccl_trace_range tr("ccl_fusion pack");
    int rc = mi_ccl_fusion_pack(p->plan_for(counts, dtype), tensors.data(), fusion_buf, stream);
    if (rc != MI_CCL_SUCCESS)
        throw ccl::exception(std::string("mi_ccl_fusion_pack: ") + mi_ccl_status_str(rc));
}

void ccl_fusion_hip_backend::unpack(const void* fusion_buf, const std::vector<void*>& tensors,
                                    const std::vector<size_t>& counts, const ccl_datatype& dtype, void* stream) {
    ccl_trace_range tr("ccl_fusion unpack");
    int rc = mi_ccl_fusion_unpack(p->plan_for(counts, dtype), fusion_buf, tensors.data(), stream);
    if (rc != MI_CCL_SUCCESS)
        throw ccl::exception(std::string("mi_ccl_fusion_unpack: ") + mi_ccl_status_str(rc));
}

std::shared_ptr<void> ccl_fusion_hip_backend::record(void* stream) {
    hipEvent_t ev = nullptr;
    if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess)
        throw ccl::exception("hipEventCreate failed");
    if (hipEventRecord(ev, (hipStream_t)stream) != hipSuccess) {
        (void)hipEventDestroy(ev);
        throw ccl::exception("hipEventRecord failed");
    }
    return std::shared_ptr<void>((void*)ev, [](void* e) { (void)hipEventDestroy((hipEvent_t)e); });
}

bool ccl_fusion_hip_backend::ready(const std::shared_ptr<void>& token) {
    return !token || hipEventQuery((hipEvent_t)token.get()) == hipSuccess;
}
