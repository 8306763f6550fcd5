// Per-call time of small 4-input int32 reduces issued from C++ through the C ABI: what a latency-bound caller sees
// (the Python binding used by the other benchmarks adds about 5 us of its own per call).
// The result of every timed form is checked (all inputs are constant bytes, so the sums are known in closed form).
// Prints one line per size: GPU-clock time per call of 2000 back-to-back calls, host time to enqueue one call, and
// the round trip of one call followed by a stream synchronisation.  Then the case fusion exists for: 1,024 small bf16
// gradient tensors reduced against 7 peers, one call per tensor against the fusion manager (requests queued one by
// one, fused up to 256 per launch: pack, one 8-input reduce over the fusion buffer, unpack).  Also: the same small
// reduces as nodes of a HIP graph (64 per graph, time per node of a replay), and what the C++ layer's check of its
// buffer arguments costs per call (ccl::env_data::check_pointers 0 / 1 / 2).
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <chrono>
#include <memory>
#include <vector>
#include "../../include/mi_ccl_comp.h"
#include "../../oneccl_amd/csrc/ccl_comp.hpp"
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
    // The same small reduces captured into a HIP graph: 64 nodes (rotating over 4 output buffers), replayed 50 times.
    for (size_t bytes : {1024ul, 16384ul, 65536ul, 262144ul, 1048576ul, 4194304ul}) {
        void* b[8];
        for (int i = 0; i < 8; i++) { CK(hipMalloc(&b[i], bytes)); CK(hipMemset(b[i], i < 4 ? i + 1 : 0, bytes)); }
        const void* srcs[4] = { b[0], b[1], b[2], b[3] };
        mi_ccl_comp_reduce_n(MI_CCL_INT32, MI_CCL_SUM, srcs, 4, b[4], bytes / 4, 0, 2, 0, s);   // warm, outside the capture
        CK(hipStreamSynchronize(s));
        const int nodes = 64, replays = 50;
        hipGraph_t g; hipGraphExec_t ge;
        CK(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
        for (int i = 0; i < nodes; i++) mi_ccl_comp_reduce_n(MI_CCL_INT32, MI_CCL_SUM, srcs, 4, b[4 + (i & 3)], bytes / 4, 0, 2, 0, s);
        CK(hipStreamEndCapture(s, &g));
        CK(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0));
        CK(hipGraphLaunch(ge, s)); CK(hipStreamSynchronize(s));
        std::vector<uint32_t> h(bytes / 4);
        CK(hipMemcpy(h.data(), b[7], bytes, hipMemcpyDeviceToHost));
        for (uint32_t v : h) if (v != 0x0a0a0a0au) { printf("WRONG RESULT (graph replay, %zu B)\n", bytes); return 1; }
        hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
        CK(hipEventRecord(e0, s));
        for (int r = 0; r < replays; r++) CK(hipGraphLaunch(ge, s));
        CK(hipEventRecord(e1, s));
        CK(hipStreamSynchronize(s));
        float ms; CK(hipEventElapsedTime(&ms, e0, e1));
        auto t0 = std::chrono::steady_clock::now();
        for (int r = 0; r < 20; r++) { CK(hipGraphLaunch(ge, s)); CK(hipStreamSynchronize(s)); }
        auto t1 = std::chrono::steady_clock::now();
        printf("%8zu B x4 as graph nodes: %.2f us per node (64 nodes per graph, 50 replays back to back); one replay + sync %.1f us\n", bytes,
               ms * 1e3 / replays / nodes, std::chrono::duration<double, std::micro>(t1 - t0).count() / 20);
        CK(hipGraphExecDestroy(ge)); CK(hipGraphDestroy(g));
        for (int i = 0; i < 8; i++) CK(hipFree(b[i]));
    }
    // What the C++ layer's look at its buffer arguments costs: host time to enqueue one 1 KiB ccl_comp_reduce with
    // the check off (0), remembered per allocation (1, the default) and asked of the runtime every time (2); the
    // smallest of five runs of 20,000 calls each.
    {
        void *a, *b;
        CK(hipMalloc(&a, 1024)); CK(hipMalloc(&b, 1024)); CK(hipMemset(a, 0, 1024)); CK(hipMemset(b, 0, 1024));
        ccl_sched sched; sched.stream = s;
        const ccl_datatype& i32 = ccl_datatype_storage::instance().get(ccl::datatype::int32);
        double best[3] = { 1e9, 1e9, 1e9 };
        for (int run = 0; run < 5; run++)
            for (int mode = 0; mode < 3; mode++) {
                ccl::global_data::env().check_pointers = mode;
                for (int i = 0; i < 200; i++) ccl_comp_reduce(&sched, a, 256, b, nullptr, i32, ccl::reduction::sum, nullptr);
                CK(hipStreamSynchronize(s));
                const int iters = 20000;
                auto t0 = std::chrono::steady_clock::now();
                for (int i = 0; i < iters; i++) ccl_comp_reduce(&sched, a, 256, b, nullptr, i32, ccl::reduction::sum, nullptr);
                auto t1 = std::chrono::steady_clock::now();
                CK(hipStreamSynchronize(s));
                const double us = std::chrono::duration<double, std::micro>(t1 - t0).count() / iters;
                if (us < best[mode]) best[mode] = us;
            }
        ccl::global_data::env().check_pointers = 1;
        printf("ccl_comp_reduce, 1 KiB, host enqueue per call: pointer check off %.3f us, remembered (default) %.3f us (+%.3f), runtime query every call %.3f us (+%.3f)\n",
               best[0], best[1], best[1] - best[0], best[2], best[2] - best[0]);
        CK(hipFree(a)); CK(hipFree(b));
    }
    // Many small reduces: 64 independent 4-input int32 sums as 64 calls and as ONE call of mi_ccl_comp_reduce_batch
    // (one launch).  Input k of every job holds the byte k + 1, so every output word must be 0x0a0a0a0a.
    for (size_t bytes : {1024ul, 4096ul, 16384ul, 65536ul, 262144ul, 1048576ul, 4194304ul}) {
        const int J = 64, N = 4;
        std::vector<void*> in(J * N), out(J);
        std::vector<const void*> srcs(J * N);
        std::vector<size_t> counts(J, bytes / 4);
        for (int j = 0; j < J; j++) {
            for (int k = 0; k < N; k++) { CK(hipMalloc(&in[j * N + k], bytes)); CK(hipMemset(in[j * N + k], k + 1, bytes)); srcs[j * N + k] = in[j * N + k]; }
            CK(hipMalloc(&out[j], bytes));
        }
        auto check = [&](const char* what) -> bool {
            std::vector<uint32_t> h(bytes / 4);
            for (int j = 0; j < J; j += 21) {
                if (hipMemcpy(h.data(), out[j], bytes, hipMemcpyDeviceToHost) != hipSuccess) return false;
                for (uint32_t v : h) if (v != 0x0a0a0a0au) { printf("WRONG RESULT (%s, job %d)\n", what, j); return false; }
                (void)hipMemset(out[j], 0, bytes);
            }
            return true;
        };
        hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
        const int rounds = 50;
        auto calls = [&]() { for (int j = 0; j < J; j++) mi_ccl_comp_reduce_n(MI_CCL_INT32, MI_CCL_SUM, &srcs[j * N], N, out[j], bytes / 4, 0, 2, 0, s); };
        auto batch = [&]() { mi_ccl_comp_reduce_batch(MI_CCL_INT32, MI_CCL_SUM, srcs.data(), N, out.data(), counts.data(), J, 0, 2, 0, s); };
        float ms_calls, ms_batch;
        calls(); CK(hipStreamSynchronize(s)); if (!check("64 calls")) return 1;
        CK(hipEventRecord(e0, s)); for (int r = 0; r < rounds; r++) calls(); CK(hipEventRecord(e1, s)); CK(hipStreamSynchronize(s));
        CK(hipEventElapsedTime(&ms_calls, e0, e1));
        batch(); CK(hipStreamSynchronize(s)); if (!check("one batch call")) return 1;
        CK(hipEventRecord(e0, s)); for (int r = 0; r < rounds; r++) batch(); CK(hipEventRecord(e1, s)); CK(hipStreamSynchronize(s));
        CK(hipEventElapsedTime(&ms_batch, e0, e1));
        const double gb = 5.0 * bytes * J / 1e9;
        printf("64 jobs x %8zu B x4: 64 calls %.2f us per job (%.0f GB/s); one batch launch %.2f us per job (%.0f GB/s)\n", bytes,
               ms_calls * 1e3 / rounds / J, gb / (ms_calls * 1e-3 / rounds), ms_batch * 1e3 / rounds / J, gb / (ms_batch * 1e-3 / rounds));
        for (auto p : in) CK(hipFree(p));
        for (auto p : out) CK(hipFree(p));
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
