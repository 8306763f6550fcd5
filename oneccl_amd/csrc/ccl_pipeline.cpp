// The chunked, double-buffered reduce (see ccl_pipeline.hpp).
#include "ccl_pipeline.hpp"

#include <hip/hip_runtime.h>

#include <string>

namespace {
void check(hipError_t e, const char* what) {
    if (e != hipSuccess)
        throw ccl::exception(std::string(what) + ": " + hipGetErrorString(e));
}
}  // namespace

ccl_chunked_reducer::ccl_chunked_reducer(size_t chunk_bytes, int max_inputs)
        : m_chunk_bytes(chunk_bytes), m_max_inputs(max_inputs) {
    if (chunk_bytes == 0 || (chunk_bytes % 16) != 0 || max_inputs < 1 || max_inputs > 64)
        throw ccl::exception("ccl_chunked_reducer: chunk_bytes must be a positive multiple of 16, 1 <= max_inputs <= 64");
    for (int b = 0; b < 2; b++) {
        check(hipMalloc(&m_work[b], chunk_bytes * (size_t)max_inputs), "ccl_chunked_reducer: work buffer");
        check(hipEventCreateWithFlags((hipEvent_t*)&m_staged[b], hipEventDisableTiming), "ccl_chunked_reducer: event");
        check(hipEventCreateWithFlags((hipEvent_t*)&m_reduced[b], hipEventDisableTiming), "ccl_chunked_reducer: event");
    }
    // default priority, like the caller's stream: streams of different priorities must not wait on each other here
    check(hipStreamCreateWithFlags((hipStream_t*)&m_stage_stream, hipStreamNonBlocking), "ccl_chunked_reducer: stream");
}

ccl_chunked_reducer::~ccl_chunked_reducer() {
    if (m_stage_stream) {
        (void)hipStreamSynchronize((hipStream_t)m_stage_stream);
        (void)hipStreamDestroy((hipStream_t)m_stage_stream);
    }
    for (int b = 0; b < 2; b++) {
        if (m_staged[b]) (void)hipEventDestroy((hipEvent_t)m_staged[b]);
        if (m_reduced[b]) (void)hipEventDestroy((hipEvent_t)m_reduced[b]);
        if (m_work[b]) (void)hipFree(m_work[b]);
    }
}

ccl::status ccl_chunked_reducer::run(ccl_sched* sched, const std::vector<const void*>& local,
                                     const std::vector<const void*>& pair, size_t count, void* out,
                                     const ccl_datatype& dtype, ccl::reduction reduction, int bf16_keep_precision_mode) {
    m_last_chunks = 0;
    if (!count)
        return ccl::status::success;
    const int n = (int)local.size();
    if (n < 1 || n > m_max_inputs || (!pair.empty() && pair.size() != local.size()))
        throw ccl::exception("ccl_chunked_reducer::run: 1 <= inputs <= max_inputs, pair empty or as long as local");
    if (reduction == ccl::reduction::custom)
        throw ccl::exception("ccl_chunked_reducer::run: custom reduction is not available on the device path");
    hipStream_t main = (hipStream_t)(sched ? sched->stream : nullptr);
    hipStream_t stage = (hipStream_t)m_stage_stream;
    const size_t esz = dtype.size();
    const size_t chunk_count = m_chunk_bytes / esz;                         // elements of one input per chunk
    const size_t num_chunks = (count + chunk_count - 1) / chunk_count;      // :129-130
    const bool with_pair = !pair.empty();
    ccl_sched stage_sched;
    stage_sched.stream = m_stage_stream;

    // the inputs must be complete before the staging stream reads them: it starts behind the caller's stream
    hipEvent_t start = nullptr;
    check(hipEventCreateWithFlags(&start, hipEventDisableTiming), "ccl_chunked_reducer::run: event");
    check(hipEventRecord(start, main), "ccl_chunked_reducer::run: record");
    check(hipStreamWaitEvent(stage, start, 0), "ccl_chunked_reducer::run: wait");
    check(hipEventDestroy(start), "ccl_chunked_reducer::run: event");      // released once the wait has been served

    auto stage_chunk = [&](size_t nc) {
        const int b = (int)(nc % 2);
        const size_t off = nc * chunk_count, cnt = (count - off < chunk_count) ? count - off : chunk_count;
        if (nc >= 2)    // work buffer b still holds chunk nc - 2 until its reduce has read it
            check(hipStreamWaitEvent(stage, (hipEvent_t)m_reduced[b], 0), "ccl_chunked_reducer::run: wait");
        std::vector<const void*> srcs;
        std::vector<void*> dsts;
        std::vector<size_t> counts(n, cnt);
        for (int i = 0; i < n; i++) {
            if (with_pair) srcs.push_back((const char*)pair[i] + off * esz);      // pair_val OP local_val, :33-35
            srcs.push_back((const char*)local[i] + off * esz);
            dsts.push_back((char*)m_work[b] + (size_t)i * m_chunk_bytes);
        }
        ccl_comp_reduce_batch(&stage_sched, srcs, with_pair ? 2 : 1, dsts, counts, dtype, reduction, 0);
        check(hipEventRecord((hipEvent_t)m_staged[b], stage), "ccl_chunked_reducer::run: record");
    };

    stage_chunk(0);                                                         // pipeline prologue, :186-205
    for (size_t nc = 0; nc < num_chunks; nc++) {
        const int b = (int)(nc % 2);
        const size_t off = nc * chunk_count, cnt = (count - off < chunk_count) ? count - off : chunk_count;
        if (nc + 1 < num_chunks)
            stage_chunk(nc + 1);                                            // runs beside the reduce below
        check(hipStreamWaitEvent(main, (hipEvent_t)m_staged[b], 0), "ccl_chunked_reducer::run: wait");
        std::vector<const void*> peers;
        for (int i = 1; i < n; i++) peers.push_back((const char*)m_work[b] + (size_t)i * m_chunk_bytes);
        ccl_comp_reduce_n(sched, m_work[b], peers, cnt, (char*)out + off * esz, dtype, reduction, bf16_keep_precision_mode);
        check(hipEventRecord((hipEvent_t)m_reduced[b], main), "ccl_chunked_reducer::run: record");
    }
    m_last_chunks = num_chunks;
    return ccl::status::success;
}
