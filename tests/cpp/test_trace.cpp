// Host-only test of the profiler-range knob of the C++ layer (oneccl_amd/csrc/ccl_trace.{hpp,cpp}): off, a range
// object opens nothing, counts nothing and looks for no library; on, every range is counted, the roctx library is
// looked up once, and ranges nest and close in order.  No HIP, no GPU.
#include <stdio.h>
#include <stdlib.h>

#include "../../oneccl_amd/csrc/ccl_trace.hpp"

static int failed = 0, checks = 0;
#define EXPECT(c) do { checks++; if (!(c)) { failed++; printf("FAIL line %d: %s\n", __LINE__, #c); } } while (0)

int main() {
    unsetenv("MI_CCL_TRACE");
    EXPECT(!ccl_trace_enabled());
    {
        ccl_trace_range a("ccl_comp_reduce");
        ccl_trace_range b("ccl_comp_copy");
    }
    EXPECT(ccl_trace_ranges_opened() == 0);
    EXPECT(!ccl_trace_library_loaded());            // nothing was looked for
    ccl_trace_enable(true);
    EXPECT(ccl_trace_enabled());
    {
        ccl_trace_range a("ccl_comp_reduce");
        { ccl_trace_range b("ccl_fusion pack"); }
        ccl_trace_range c("ccl_comp_batch_reduce");
    }
    EXPECT(ccl_trace_ranges_opened() == 3);
    printf("roctx library %s\n", ccl_trace_library_loaded() ? "found" : "not found (ranges counted, not emitted)");
    ccl_trace_enable(false);
    { ccl_trace_range a("ccl_comp_reduce"); }
    EXPECT(ccl_trace_ranges_opened() == 3);
    printf("%d checks, %d failed\n", checks, failed);
    return failed ? 1 : 0;
}
