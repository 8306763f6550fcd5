// One GPU's part of the reference's large-message reduce-scatter pipeline
// (reduce_scatter_large_impl, src/coll/algorithms/reduce_scatter/sycl/reduce_scatter_large_sycl_impl.hpp:98-301).
//
// The reference cuts recv_count into chunks of its tmp-buffer size (:127-130) and keeps two of them in flight
// (pipeline_size = 2, :111): for chunk nc it stages every peer's share into work buffer nc % 2 -- read_reduce_write
// (:22-66: work[i] = pair[i] + local[i], one kernel for all peers i) or, without a pair tile, copy_data -- while the
// same kernel folds the staged buffers of chunk nc - 1 into recv_buf (reduce_sum, :245-257), and an epilogue folds
// the last chunk (:276-299).  Between GPUs the staging step is the transfer; on one GPU, with every contribution
// already in local memory, it is a copy (or a pair-reduce) that stands in for it.
//
// ccl_chunked_reducer keeps that structure: two sets of work buffers (allocated once, like the reference's
// get_tmp_buf), the staging of chunk nc + 1 on a second HIP stream of the same priority as the caller's, the N-input
// reduce of chunk nc on the caller's stream, HIP events in both directions (staged -> reduce, reduced -> buffer free
// for chunk nc + 2).  The staging is ONE launch per chunk for all inputs (mi_ccl_comp_reduce_batch).  Results are
// bit-identical to the unchunked reduce of the staged values, whatever the chunk size.  On one GPU nothing is gained
// in time -- the staging adds memory traffic that a transfer engine would carry -- the point is the call pattern.
#pragma once

#include <vector>

#include "ccl_comp.hpp"

class ccl_chunked_reducer {
public:
    // chunk_bytes: bytes of one input per chunk (the reference's get_tmp_buf_size_per_rank()); max_inputs: the most
    // inputs a run() will bring.  Allocates 2 x max_inputs x chunk_bytes of device memory, a stream and four events.
    ccl_chunked_reducer(size_t chunk_bytes, int max_inputs);
    ~ccl_chunked_reducer();
    ccl_chunked_reducer(const ccl_chunked_reducer&) = delete;
    ccl_chunked_reducer& operator=(const ccl_chunked_reducer&) = delete;

    // out[i] = s_0[i] OP s_1[i] OP ... OP s_{N-1}[i] for i < count, where s_j is local[j] or, when `pair` is not empty
    // (it then has local.size() entries), pair[j] OP local[j] rounded to dtype (the read_reduce_write step).  out may
    // be one of the inputs.  Enqueued on the schedule's stream; the call returns once everything is enqueued.
    ccl::status run(ccl_sched* sched, const std::vector<const void*>& local, const std::vector<const void*>& pair,
                    size_t count, void* out, const ccl_datatype& dtype, ccl::reduction reduction,
                    int bf16_keep_precision_mode = 0);

    size_t chunk_bytes() const { return m_chunk_bytes; }
    size_t chunks_of_last_run() const { return m_last_chunks; }

private:
    size_t m_chunk_bytes;
    int m_max_inputs;
    void* m_work[2] = { nullptr, nullptr };     // pipeline_size = 2
    void* m_stage_stream = nullptr;             // hipStream_t
    void* m_staged[2] = { nullptr, nullptr };   // hipEvent_t: work buffer b holds its chunk
    void* m_reduced[2] = { nullptr, nullptr };  // hipEvent_t: work buffer b has been read
    size_t m_last_chunks = 0;
};
