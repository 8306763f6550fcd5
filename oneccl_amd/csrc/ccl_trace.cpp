// See ccl_trace.hpp.  No HIP in this file: it also builds into the host-only test of the knob.
#include "ccl_trace.hpp"

#include <dlfcn.h>
#include <stdlib.h>

#include <atomic>
#include <mutex>

namespace {

typedef int (*push_fn)(const char*);
typedef int (*pop_fn)();

std::atomic<int> g_on{ -1 };                // -1: MI_CCL_TRACE not read yet
std::atomic<unsigned long> g_opened{ 0 };
std::once_flag g_load_once;
push_fn g_push = nullptr;
pop_fn g_pop = nullptr;

void load_roctx() {
    for (const char* name : { "libroctx64.so.4", "libroctx64.so", "librocprofiler-sdk-roctx.so.1", "librocprofiler-sdk-roctx.so" }) {
        void* h = dlopen(name, RTLD_NOW | RTLD_GLOBAL);
        if (!h)
            continue;
        push_fn pu = (push_fn)dlsym(h, "roctxRangePushA");
        pop_fn po = (pop_fn)dlsym(h, "roctxRangePop");
        if (pu && po) {
            g_push = pu;
            g_pop = po;
            return;
        }
    }
}

}  // namespace

bool ccl_trace_enabled() {
    int v = g_on.load(std::memory_order_relaxed);
    if (v < 0) {
        const char* e = getenv("MI_CCL_TRACE");
        v = (e && e[0] == '1' && e[1] == 0) ? 1 : 0;
        g_on.store(v, std::memory_order_relaxed);
    }
    return v == 1;
}

void ccl_trace_enable(bool on) {
    g_on.store(on ? 1 : 0, std::memory_order_relaxed);
}

unsigned long ccl_trace_ranges_opened() {
    return g_opened.load(std::memory_order_relaxed);
}

bool ccl_trace_library_loaded() {
    return g_push != nullptr;
}

ccl_trace_range::ccl_trace_range(const char* name) : open(false) {
    if (!ccl_trace_enabled())
        return;
    std::call_once(g_load_once, load_roctx);
    g_opened.fetch_add(1, std::memory_order_relaxed);
    if (g_push) {
        g_push(name);
        open = true;
    }
}

ccl_trace_range::~ccl_trace_range() {
    if (open)
        g_pop();
}
