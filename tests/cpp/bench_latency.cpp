// Per-call time of small 4-input int32 reduces issued from C++ through the C ABI: what a latency-bound caller sees
// (the Python binding used by the other benchmarks adds about 5 us of its own per call).
// Prints one line per size: GPU-clock time per call of 2000 back-to-back calls, host time to enqueue one call, and
// the round trip of one call followed by a stream synchronisation.  Then the case fusion exists for: 1,024 small bf16
// gradient tensors reduced against 7 peers, one call per tensor against the fusion manager (requests queued one by
// one, fused up to 256 per launch: pack, one 8-input reduce over the fusion buffer, unpack).
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <chrono>
#include <memory>
#include <vector>
#include "../../include/mi_ccl_comp.h"
#include "../../oneccl_amd/csrc/ccl_fusion.hpp"
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s line %d\n", hipGetErrorString(e), __LINE__); return 1; } } while (0)
int main() {
    hipStream_t s; CK(hipStreamCreate(&s));
    for (size_t bytes : {1024ul, 65536ul, 1048576ul, 4194304ul, 16777216ul}) {
        void* b[5];
        for (int i = 0; i < 5; i++) { CK(hipMalloc(&b[i], bytes)); CK(hipMemset(b[i], 0, bytes)); }
        const void* srcs[4] = { b[0], b[1], b[2], b[3] };
        for (int i = 0; i < 50; i++) mi_ccl_comp_reduce_n(MI_CCL_INT32, MI_CCL_SUM, srcs, 4, b[4], bytes / 4, 0, 2, 0, s);
        CK(hipStreamSynchronize(s));
        hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
        const int iters = 2000;
        auto t0 = std::chrono::steady_clock::now();
        CK(hipEventRecord(e0, s));
        for (int i = 0; i < iters; i++) mi_ccl_comp_reduce_n(MI_CCL_INT32, MI_CCL_SUM, srcs, 4, b[4], bytes / 4, 0, 2, 0, s);
        CK(hipEventRecord(e1, s));
        auto t1 = std::chrono::steady_clock::now();
        CK(hipStreamSynchronize(s));
        auto t2 = std::chrono::steady_clock::now();
        float ms; CK(hipEventElapsedTime(&ms, e0, e1));
        // single call + sync latency
        auto t3 = std::chrono::steady_clock::now();
        for (int i = 0; i < 200; i++) { mi_ccl_comp_reduce_n(MI_CCL_INT32, MI_CCL_SUM, srcs, 4, b[4], bytes / 4, 0, 2, 0, s); CK(hipStreamSynchronize(s)); }
        auto t4 = std::chrono::steady_clock::now();
        printf("%8zu B x4: back-to-back %.2f us/call on GPU clock, host enqueue %.2f us/call, wall incl. drain %.2f us/call; call+sync %.2f us\n", bytes,
               ms * 1e3 / iters, std::chrono::duration<double, std::micro>(t1 - t0).count() / iters,
               std::chrono::duration<double, std::micro>(t2 - t0).count() / iters,
               std::chrono::duration<double, std::micro>(t4 - t3).count() / 200);
        for (int i = 0; i < 5; i++) CK(hipFree(b[i]));
    }
    {
        const int K = 1024, NPEER = 7;
        const ccl_datatype& bf16 = ccl_datatype_storage::instance().get(ccl::datatype::bfloat16);
        std::vector<size_t> counts(K);
        size_t total = 0;
        for (int t = 0; t < K; t++) { counts[t] = 256 + (size_t)((t * 2654435761u) % 7600); total += counts[t]; }   // 0.5 .. 15.7 KB
        std::vector<void*> send(K), recv(K);
        for (int t = 0; t < K; t++) { CK(hipMalloc(&send[t], counts[t] * 2)); CK(hipMalloc(&recv[t], counts[t] * 2)); CK(hipMemset(send[t], 0, counts[t] * 2)); }
        ccl_fusion_config cfg;
        cfg.cycle_ms = 0;
        std::vector<void*> peers(NPEER);
        for (auto& p : peers) { CK(hipMalloc(&p, cfg.bytes_threshold * cfg.count_threshold)); CK(hipMemset(p, 0, cfg.bytes_threshold * cfg.count_threshold)); }
        ccl_sched sched; sched.stream = s;
        // (i) one 8-input reduce per tensor (peer data taken from the start of the peer buffers)
        std::vector<const void*> pv(peers.begin(), peers.end());
        auto run_unfused = [&]() { for (int t = 0; t < K; t++) ccl_comp_reduce_n(&sched, send[t], pv, counts[t], recv[t], bf16, ccl::reduction::sum, 1); };
        run_unfused(); CK(hipStreamSynchronize(s));
        auto t0 = std::chrono::steady_clock::now();
        for (int r = 0; r < 5; r++) run_unfused();
        CK(hipStreamSynchronize(s));
        auto t1 = std::chrono::steady_clock::now();
        // (ii) the same tensors through the fusion manager
        ccl_fusion_hip_backend backend;
        int launches = 0;
        ccl_fusion_manager mgr(&backend, [&](void* buf, size_t n, const ccl_datatype& dt, ccl::reduction op, const void*, void* st) {
            ccl_sched s2; s2.stream = st;
            ccl_comp_reduce_n(&s2, buf, pv, n, buf, dt, op, 1);
            launches++;
        }, cfg);
        std::vector<std::unique_ptr<ccl_fusion_request>> req(K);
        for (int t = 0; t < K; t++) {
            req[t].reset(new ccl_fusion_request);
            req[t]->send_buf = send[t]; req[t]->recv_buf = recv[t]; req[t]->count = counts[t]; req[t]->dtype = bf16; req[t]->stream = s;
        }
        auto run_fused = [&]() {
            for (int t = 0; t < K; t++) { mgr.add(req[t].get()); if ((t & 63) == 63) mgr.execute(); }
            req[K - 1]->urgent = true;
            bool done = false;
            while (!done) { mgr.execute(); done = true; for (int t = 0; t < K && done; t++) done = req[t]->is_completed(); }
        };
        run_fused();
        launches = 0;
        auto t2 = std::chrono::steady_clock::now();
        for (int r = 0; r < 5; r++) run_fused();
        CK(hipStreamSynchronize(s));
        auto t3 = std::chrono::steady_clock::now();
        printf("%d bf16 tensors (%.1f MB), 8-input sum: one call each %.1f us per round; through the fusion manager %.1f us per round (%d fused launches per round)\n",
               K, total * 2 / 1e6, std::chrono::duration<double, std::micro>(t1 - t0).count() / 5,
               std::chrono::duration<double, std::micro>(t3 - t2).count() / 5, launches / 5);
    }
    return 0;
}
