// Per-call time of small 4-input int32 reduces issued from C++ through the C ABI: what a latency-bound caller sees
// (the Python binding used by the other benchmarks adds about 5 us of its own per call).
// Prints one line per size: GPU-clock time per call of 2000 back-to-back calls, host time to enqueue one call, and
// the round trip of one call followed by a stream synchronisation.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <chrono>
#include "../../include/mi_ccl_comp.h"
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s line %d\n", hipGetErrorString(e), __LINE__); return 1; } } while (0)
int main() {
    hipStream_t s; CK(hipStreamCreate(&s));
    for (size_t bytes : {1024ul, 65536ul, 1048576ul, 4194304ul, 16777216ul}) {
        void* b[5];
        for (int i = 0; i < 5; i++) { CK(hipMalloc(&b[i], bytes)); CK(hipMemset(b[i], 0, bytes)); }
        const void* srcs[4] = { b[0], b[1], b[2], b[3] };
        for (int i = 0; i < 50; i++) mi_ccl_comp_reduce_n(MI_CCL_INT32, MI_CCL_SUM, srcs, 4, b[4], bytes / 4, 0, 2, s);
        CK(hipStreamSynchronize(s));
        hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
        const int iters = 2000;
        auto t0 = std::chrono::steady_clock::now();
        CK(hipEventRecord(e0, s));
        for (int i = 0; i < iters; i++) mi_ccl_comp_reduce_n(MI_CCL_INT32, MI_CCL_SUM, srcs, 4, b[4], bytes / 4, 0, 2, s);
        CK(hipEventRecord(e1, s));
        auto t1 = std::chrono::steady_clock::now();
        CK(hipStreamSynchronize(s));
        auto t2 = std::chrono::steady_clock::now();
        float ms; CK(hipEventElapsedTime(&ms, e0, e1));
        // single call + sync latency
        auto t3 = std::chrono::steady_clock::now();
        for (int i = 0; i < 200; i++) { mi_ccl_comp_reduce_n(MI_CCL_INT32, MI_CCL_SUM, srcs, 4, b[4], bytes / 4, 0, 2, s); CK(hipStreamSynchronize(s)); }
        auto t4 = std::chrono::steady_clock::now();
        printf("%8zu B x4: back-to-back %.2f us/call on GPU clock, host enqueue %.2f us/call, wall incl. drain %.2f us/call; call+sync %.2f us\n", bytes,
               ms * 1e3 / iters, std::chrono::duration<double, std::micro>(t1 - t0).count() / iters,
               std::chrono::duration<double, std::micro>(t2 - t0).count() / iters,
               std::chrono::duration<double, std::micro>(t4 - t3).count() / 200);
        for (int i = 0; i < 5; i++) CK(hipFree(b[i]));
    }
    return 0;
}
