// Profiler ranges around the operator-level calls of the C++ layer.  The reference brackets ccl_comp_reduce_regular
// with an ITT event (src/comp/comp.cpp:90-93,116-118) so that a trace shows the operator, not only what it ran; here
// the same calls open a roctx range, which rocprofv3 --marker-trace shows above the kernels they enqueue.  Off unless
// MI_CCL_TRACE=1 is set (or ccl_trace_enable(true) is called): a call then costs one relaxed load and no range is
// opened, no library is looked for.  When on, libroctx64 is loaded on first use; if it cannot be found the ranges are
// counted and otherwise dropped.
#pragma once

void ccl_trace_enable(bool on);
bool ccl_trace_enabled();
unsigned long ccl_trace_ranges_opened();    // ranges opened by this process so far (tests)
bool ccl_trace_library_loaded();            // whether roctxRangePushA / roctxRangePop were found

class ccl_trace_range {
public:
    explicit ccl_trace_range(const char* name);
    ~ccl_trace_range();
    ccl_trace_range(const ccl_trace_range&) = delete;
    ccl_trace_range& operator=(const ccl_trace_range&) = delete;

private:
    bool open;
};
