// GPU test of the C++ operator surface (oneccl_amd/csrc/ccl_comp.hpp), written the way the reference's own
// functional tests are (tests/functional/test_impl.hpp:242-324): every "rank" r fills its buffer with
// c1*r + c2*buf_idx (+1 for prod), the buffers are reduced, and the result is checked against the closed
// form within the reference's tolerance (test_impl.hpp:160-204) -- and, beyond what the reference checks,
// bit for bit against the CPU oracle.  Exit status 0 = all checks passed.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <memory>
#include <string>
#include <vector>

#include "../../oneccl_amd/csrc/ccl_comp.hpp"
#include "../../oneccl_amd/csrc/ccl_fusion.hpp"
#include "../../oneccl_amd/csrc/ccl_pipeline.hpp"
#include "../../oneccl_amd/csrc/ccl_trace.hpp"
#include "../../include/mi_ccl_comp.h"
#include "../../oracle/ccl_comp_oracle.h"

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); exit(2); } } while (0)
static int g_fail = 0, g_checks = 0;
#define EXPECT(cond, ...) do { g_checks++; if (!(cond)) { g_fail++; printf("FAIL line %d: ", __LINE__); printf(__VA_ARGS__); printf("\n"); } } while (0)

static const ccl_datatype& DT(ccl::datatype d) { return ccl_datatype_storage::instance().get(d); }

template <class T> struct DevBuf {
    T* p = nullptr; size_t n;
    explicit DevBuf(size_t n_) : n(n_) { CK(hipMalloc(&p, (n ? n : 1) * sizeof(T))); }
    explicit DevBuf(const std::vector<T>& h) : n(h.size()) { CK(hipMalloc(&p, (n ? n : 1) * sizeof(T))); CK(hipMemcpy(p, h.data(), n * sizeof(T), hipMemcpyHostToDevice)); }
    ~DevBuf() { (void)hipFree(p); }
    std::vector<T> host() const { std::vector<T> h(n); CK(hipDeviceSynchronize()); CK(hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost)); return h; }
};

static uint16_t to_lp(float v, ccl::datatype d) {
    uint32_t u; memcpy(&u, &v, 4);
    return d == ccl::datatype::bfloat16 ? orc_bf16_narrow_rne(u) : orc_fp16_narrow(u);
}
static float from_lp(uint16_t h, ccl::datatype d) {
    uint32_t u = d == ccl::datatype::bfloat16 ? orc_bf16_widen(h) : orc_fp16_widen(h);
    float f; memcpy(&f, &u, 4); return f;
}

// element of rank r's buffer, as the functional tests fill it (test.hpp:73-86, test_impl.hpp:242-252)
static double fill_value(ccl::datatype d, int r, int buf_idx, ccl::reduction op) {
    double c1 = 1, c2 = 1;
    if (d == ccl::datatype::bfloat16) { c1 = 0.5; c2 = 1; }
    if (d == ccl::datatype::float16) { c1 = 0.01; c2 = 0.01; }
    return c1 * r + c2 * buf_idx + (op == ccl::reduction::prod ? 1 : 0);
}

template <class T>
static void closed_form_case(ccl::datatype d, size_t count, int N, int buf_idx, ccl::reduction op, hipStream_t stream) {
    const bool lp = d == ccl::datatype::bfloat16 || d == ccl::datatype::float16;
    std::vector<std::vector<T>> send(N, std::vector<T>(count));
    std::vector<double> vals(N);
    for (int r = 0; r < N; r++) {
        vals[r] = fill_value(d, r, buf_idx, op);
        T x;
        if (lp) { uint16_t h = to_lp((float)vals[r], d); memcpy(&x, &h, sizeof(T)); vals[r] = from_lp(h, d); }
        else x = (T)vals[r];
        for (size_t i = 0; i < count; i++) send[r][i] = x;
    }
    double expected = vals[0];
    for (int r = 1; r < N; r++) {
        if (op == ccl::reduction::sum) expected += vals[r];
        else if (op == ccl::reduction::prod) expected *= vals[r];
        else if (op == ccl::reduction::min) expected = fmin(expected, vals[r]);
        else expected = fmax(expected, vals[r]);
    }
    // oracle: chain of pairwise calls, recv <- rank 0, then ranks 1..N-1 (reduce_scatter.cpp:111-136)
    std::vector<T> want = send[0];
    for (int r = 1; r < N; r++)
        orc_comp_reduce(send[r].data(), count, want.data(), (int)d, (int)op, ORC_BF16_AVX512BF, ORC_FP16_AVX512F);
    ccl_sched sched; sched.stream = stream;
    // (1) chain of ccl_comp_reduce
    {
        DevBuf<T> recv(send[0]);
        for (int r = 1; r < N; r++) {
            DevBuf<T> in(send[r]);
            size_t out_count = 12345;
            ccl::status st = ccl_comp_reduce(&sched, in.p, count, recv.p, &out_count, DT(d), op, nullptr);
            EXPECT(st == ccl::status::success, "status");
            EXPECT(out_count == (lp ? count : (size_t)12345), "out_count semantics (only 16-bit paths report it)");
            CK(hipStreamSynchronize(stream));
        }
        std::vector<T> got = recv.host();
        EXPECT(memcmp(got.data(), want.data(), count * sizeof(T)) == 0, "chain vs oracle dtype %d op %d count %zu", (int)d, (int)op, count);
        double g = lp ? from_lp(*(uint16_t*)&got[count - 1], d) : (double)got[count - 1];
        double eps = d == ccl::datatype::bfloat16 ? 2 * pow(2, -7) : d == ccl::datatype::float16 ? 2 * pow(2, -10)
                     : d == ccl::datatype::float32 ? pow(2, -23) : 0;
        double le = log2((double)N) * eps, max_err = fabs(expected) * le / (1 - le);
        EXPECT(fabs(g - expected) <= max_err + (lp ? fabs(expected) * eps : 0), "closed form dtype %d op %d: got %g expected %g", (int)d, (int)op, g, expected);
    }
    // (2) ccl_comp_batch_reduce over slices of one buffer (pairwise mode) and the N-input form
    {
        std::vector<T> all;
        std::vector<size_t> offsets;
        for (int r = 0; r < N; r++) { offsets.push_back(all.size()); all.insert(all.end(), send[r].begin(), send[r].end()); }
        DevBuf<T> buf(all);
        ccl_comp_batch_reduce(buf.p, offsets, count, buf.p, nullptr, DT(d), op, nullptr, nullptr, 0, nullptr, nullptr, &sched);
        std::vector<T> got = buf.host();
        EXPECT(memcmp(got.data(), want.data(), count * sizeof(T)) == 0, "batch reduce vs oracle dtype %d op %d", (int)d, (int)op);
        EXPECT(memcmp(got.data() + count, all.data() + count, (all.size() - count) * sizeof(T)) == 0, "batch reduce touched an input slice");
        std::vector<DevBuf<T>*> peers;
        std::vector<const void*> pp;
        DevBuf<T> own(send[0]), out(count);
        for (int r = 1; r < N; r++) { peers.push_back(new DevBuf<T>(send[r])); pp.push_back(peers.back()->p); }
        ccl_comp_reduce_n(&sched, own.p, pp, count, out.p, DT(d), op, 0);
        std::vector<T> got2 = out.host();
        EXPECT(memcmp(got2.data(), want.data(), count * sizeof(T)) == 0, "reduce_n vs oracle dtype %d op %d", (int)d, (int)op);
        for (auto* p : peers) delete p;
    }
}

static void custom_sum_i32(const void* in, size_t n, void* inout, size_t* out_count, ccl::datatype dt, const ccl::fn_context* ctx) {
    const int32_t* a = (const int32_t*)in; int32_t* b = (int32_t*)inout;
    for (size_t i = 0; i < n; i++) b[i] = 2 * b[i] + a[i];
    if (out_count) *out_count = n;
    (void)dt; (void)ctx;
}

static int g_custom_dtype_seen = -1;
static void custom_xyz_max(const void* in, size_t n, void* inout, size_t* out_count, ccl::datatype dt, const ccl::fn_context*) {
    const int32_t* a = (const int32_t*)in; int32_t* b = (int32_t*)inout;
    for (size_t e = 0; e < n; e++)
        if (a[3 * e] > b[3 * e]) { b[3 * e] = a[3 * e]; b[3 * e + 1] = a[3 * e + 1]; b[3 * e + 2] = a[3 * e + 2]; }
    if (out_count) *out_count = n;
    g_custom_dtype_seen = (int)dt;
}

int main() {
    int ndev = 0; CK(hipGetDeviceCount(&ndev));
    if (ndev < 1) { printf("no GPU\n"); return 2; }
    hipStream_t stream; CK(hipStreamCreate(&stream));
    const char* env_bf16 = getenv("CCL_BF16");
    printf("bf16 impl %d (CCL_BF16=%s)\n", (int)ccl::global_data::env().bf16_impl_type, env_bf16 ? env_bf16 : "unset");

    if (!env_bf16) {
        const size_t sizes[] = { 17, 32771, 262144 };   // tests/functional/conf.cpp:51-53
        const ccl::reduction ops[] = { ccl::reduction::sum, ccl::reduction::prod, ccl::reduction::min, ccl::reduction::max };
        for (size_t count : sizes)
            for (ccl::reduction op : ops)
                for (int buf_idx : { 0, 3 }) {
                    closed_form_case<int32_t>(ccl::datatype::int32, count, 4, buf_idx, op, stream);
                    closed_form_case<float>(ccl::datatype::float32, count, 4, buf_idx, op, stream);
                    closed_form_case<uint16_t>(ccl::datatype::float16, count, 4, buf_idx, op, stream);
                    closed_form_case<uint16_t>(ccl::datatype::bfloat16, count, 4, buf_idx, op, stream);
                }
        closed_form_case<int8_t>(ccl::datatype::int8, 1000, 4, 1, ccl::reduction::sum, stream);
        closed_form_case<uint64_t>(ccl::datatype::uint64, 1000, 4, 1, ccl::reduction::prod, stream);
        closed_form_case<double>(ccl::datatype::float64, 1000, 4, 1, ccl::reduction::max, stream);
    }

    ccl_sched sched; sched.stream = stream;
    // keep-precision batch reduce: 1 + 3 * 2^-8 in bf16 -> 3f82 in the body, 3f81 in the truncated tail (count 17)
    {
        const size_t count = 17;
        std::vector<uint16_t> all;
        std::vector<size_t> offsets;
        const uint16_t v[4] = { 0x3f80, 0x3b80, 0x3b80, 0x3b80 };
        for (int r = 0; r < 4; r++) { offsets.push_back(all.size()); all.insert(all.end(), count, v[r]); }
        DevBuf<uint16_t> buf(all);
        std::vector<float> scratch;     // the reference needs tmp/acc; here they may be null
        ccl_comp_batch_reduce(buf.p, offsets, count, buf.p, nullptr, DT(ccl::datatype::bfloat16), ccl::reduction::sum,
                              nullptr, nullptr, 1, nullptr, nullptr, &sched);
        std::vector<uint16_t> got = buf.host();
        std::vector<uint16_t> want(all.begin(), all.begin() + count);
        std::vector<float> tmp(count), acc(count);
        int impl = (int)ccl::global_data::env().bf16_impl_type;
        orc_comp_batch_reduce(all.data(), offsets.data(), 4, count, want.data(), ORC_BFLOAT16, ORC_SUM, 1, tmp.data(), acc.data(), impl, ORC_FP16_AVX512F);
        EXPECT(memcmp(got.data(), want.data(), count * 2) == 0, "keep-precision batch reduce vs oracle");
        if (impl == ccl_bf16_avx512bf) EXPECT(got[0] == 0x3f82 && got[15] == 0x3f82 && got[16] == 0x3f81, "recorded values: body %04x tail %04x", got[0], got[16]);
        else EXPECT(got[0] == 0x3f81 && got[16] == 0x3f81, "truncating impl: %04x %04x", got[0], got[16]);
        // pairwise sum 1 + 1.5 * 2^-8: 3f81 with round-to-nearest-even, 3f80 with truncation
        DevBuf<uint16_t> io(std::vector<uint16_t>(20, 0x3f80)), in(std::vector<uint16_t>(20, 0x3bc0));
        size_t oc = 0;
        ccl_bf16_reduce(in.p, 20, io.p, &oc, ccl::reduction::sum, &sched);
        EXPECT(oc == 20, "ccl_bf16_reduce out_cnt");
        EXPECT(io.host()[7] == (impl == ccl_bf16_avx512bf ? 0x3f81 : 0x3f80), "pairwise rounding per impl: %04x", io.host()[7]);
    }
    // custom reduction: the host callback sees host copies; a missing callback throws
    {
        std::vector<int32_t> a(1000), b(1000);
        for (int i = 0; i < 1000; i++) { a[i] = i; b[i] = 7 - i; }
        DevBuf<int32_t> da(a), db(b);
        size_t oc = 0;
        ccl_comp_reduce(&sched, da.p, 1000, db.p, &oc, DT(ccl::datatype::int32), ccl::reduction::custom, custom_sum_i32);
        std::vector<int32_t> got = db.host();
        bool ok = oc == 1000;
        for (int i = 0; i < 1000; i++) ok = ok && got[i] == 2 * (7 - i) + i;
        EXPECT(ok, "custom reduction result");
        bool threw = false;
        try { ccl_comp_reduce(&sched, da.p, 1000, db.p, &oc, DT(ccl::datatype::int32), ccl::reduction::custom, nullptr); }
        catch (const ccl::exception& e) { threw = strstr(e.what(), "custom reduction requires user callback") != nullptr; }
        EXPECT(threw, "missing callback must throw ccl::exception");
    }
    // a user-defined datatype (datatype.cpp:141-181): 12-byte elements reduced by a callback that sees the datatype's
    // index; create / name / size / free and their errors
    {
        ccl_datatype_storage& st = ccl_datatype_storage::instance();
        const ccl::datatype idx = st.create_by_datatype_size(12);
        const ccl::datatype idx2 = st.create_by_datatype_size(3);
        EXPECT((int)idx == (int)ccl::datatype::last_predefined + 1 && (int)idx2 == (int)idx + 1, "custom datatype indices %d %d", (int)idx, (int)idx2);
        EXPECT(st.get(idx).size() == 12 && st.get(idx2).size() == 3 && st.name(st.get(idx)) == "DTYPE_" + std::to_string((int)idx),
               "custom datatype size and name");
        EXPECT(!ccl_datatype_storage::is_predefined_datatype(idx) && ccl_datatype_storage::is_predefined_datatype(ccl::datatype::bfloat16),
               "is_predefined_datatype");
        g_custom_dtype_seen = -1;
        std::vector<int32_t> a(3 * 500), b(3 * 500);
        for (size_t i = 0; i < a.size(); i++) { a[i] = (int32_t)i; b[i] = (int32_t)(1000 - i); }
        DevBuf<int32_t> da(a), db(b);
        size_t oc = 0;
        ccl_comp_reduce(&sched, da.p, 500, db.p, &oc, st.get(idx), ccl::reduction::custom, custom_xyz_max);
        std::vector<int32_t> got = db.host();
        bool ok = oc == 500 && g_custom_dtype_seen == (int)idx;
        for (size_t e = 0; e < 500; e++)        // the element with the larger first component wins as a whole
            for (int c = 0; c < 3; c++) ok = ok && got[3 * e + c] == (a[3 * e] > b[3 * e] ? a[3 * e + c] : b[3 * e + c]);
        EXPECT(ok, "custom reduction over a 12-byte user datatype");
        st.free(idx2);
        bool threw = false;
        try { st.get(idx2); } catch (const ccl::exception&) { threw = true; }
        EXPECT(threw, "a freed datatype is gone");
        threw = false;
        try { st.free(idx2); } catch (const ccl::exception& e) { threw = strstr(e.what(), "non-existing") != nullptr; }
        EXPECT(threw, "freeing twice throws");
        threw = false;
        try { st.free(ccl::datatype::int32); } catch (const ccl::exception& e) { threw = strstr(e.what(), "predefined") != nullptr; }
        EXPECT(threw, "freeing a predefined datatype throws");
        EXPECT((int)st.create_by_datatype_size(5) == (int)idx + 1, "a freed index is handed out again");
        st.free(idx);
    }
    // in_count == 0 succeeds without looking at anything; an unknown dtype throws
    {
        EXPECT(ccl_comp_reduce(nullptr, nullptr, 0, nullptr, nullptr, ccl_datatype((ccl::datatype)77, 3), ccl::reduction::sum, nullptr) == ccl::status::success, "count 0");
        EXPECT(ccl_comp_copy(nullptr, nullptr, 0) == ccl::status::success, "copy 0 bytes");
        DevBuf<int32_t> x(16);
        bool threw = false;
        try { ccl_comp_reduce(&sched, x.p, 16, x.p, nullptr, ccl_datatype((ccl::datatype)77, 4), ccl::reduction::sum, nullptr); }
        catch (const ccl::exception&) { threw = true; }
        EXPECT(threw, "unknown dtype must throw");
        EXPECT(!strcmp(ccl_reduction_to_str(ccl::reduction::custom), "custom") && !strcmp(ccl_reduction_to_str((ccl::reduction)9), "unknown"), "reduction names");
        EXPECT(DT(ccl::datatype::bfloat16).size() == 2 && ccl_datatype_storage::instance().name(DT(ccl::datatype::uint64)) == "uint64", "datatype table");
    }
    // implementation names and the implementations on offer (bf16.cpp:26-30, fp16.cpp:25-37, *_utils.hpp)
    {
        EXPECT(bf16_impl_names.at(ccl_bf16_scalar) == "scalar" && bf16_impl_names.at(ccl_bf16_avx512f) == "avx512f" &&
               bf16_impl_names.at(ccl_bf16_avx512bf) == "avx512bf" && bf16_impl_names.size() == 3, "bf16 implementation names");
        EXPECT(fp16_impl_names.at(ccl_fp16_no_compiler_support) == "no_compiler_support" && fp16_impl_names.at(ccl_fp16_f16c) == "f16c" &&
               fp16_impl_names.at(ccl_fp16_avx512fp16) == "avx512fp16" && fp16_impl_names.size() == 5 && fp16_env_impl_names.size() == 3 &&
               fp16_env_impl_names.count(ccl_fp16_no_hardware_support) == 0, "fp16 implementation names");
        EXPECT(ccl_bf16_get_impl_types().count(ccl_bf16_avx512bf) == 1 && ccl_bf16_get_impl_types().size() == 3, "bf16 implementations on offer");
        EXPECT(ccl_fp16_get_impl_types().count(ccl_fp16_avx512fp16) == 1 && ccl_fp16_get_impl_types().count(ccl_fp16_no_compiler_support) == 0,
               "fp16 implementations on offer");
    }
    // copy and array converters
    {
        std::vector<uint8_t> src(100003);
        for (size_t i = 0; i < src.size(); i++) src[i] = (uint8_t)(i * 7 + 1);
        DevBuf<uint8_t> a(src), b(src.size());
        ccl_comp_copy(a.p + 1, b.p + 1, src.size() - 1, true, &sched);
        std::vector<uint8_t> got = b.host();
        EXPECT(memcmp(got.data() + 1, src.data() + 1, src.size() - 1) == 0, "copy");
        std::vector<uint32_t> f(22, 0x3f808000u);
        f[1] = 0x007fffffu; f[17] = 0x007fffffu; f[2] = 0x7f800001u; f[18] = 0x7f800001u;
        DevBuf<uint32_t> df(f); DevBuf<uint16_t> dh(22);
        ccl_convert_fp32_to_bf16_arrays(df.p, dh.p, 22, &sched);
        std::vector<uint16_t> h = dh.host(), want(22);
        orc_convert_fp32_to_bf16_arrays(f.data(), want.data(), 22, (int)ccl::global_data::env().bf16_impl_type);
        EXPECT(memcmp(h.data(), want.data(), 44) == 0, "fp32->bf16 arrays (tail truncates): %04x %04x %04x %04x", h[1], h[17], h[2], h[18]);
        DevBuf<uint32_t> back(22);
        ccl_convert_bf16_to_fp32_arrays(dh.p, (float*)back.p, 22, &sched);
        std::vector<uint32_t> w = back.host();
        bool ok = true;
        for (int i = 0; i < 22; i++) ok = ok && w[i] == ((uint32_t)h[i] << 16);
        EXPECT(ok, "bf16->fp32 arrays");
        // the single-vector converters of the reference: 16 values (bf16), 8 values (fp16); the value after the vector
        // stays untouched
        std::vector<uint32_t> v(17, 0x3f808000u);
        v[1] = 0x007fffffu; v[2] = 0x7f800001u; v[3] = 0x477fe000u; v[4] = 0x33000000u; v[5] = 0x38800000u; v[6] = 0xc77ff000u;
        DevBuf<uint32_t> dv(v); DevBuf<uint16_t> d16(std::vector<uint16_t>(17, 0xabcd));
        ccl_convert_fp32_to_bf16(dv.p, d16.p, &sched);
        std::vector<uint16_t> g16 = d16.host(), w16(16);
        const int impl = (int)ccl::global_data::env().bf16_impl_type;
        orc_convert_fp32_to_bf16_arrays(v.data(), w16.data(), 16, impl == ORC_BF16_AVX512BF ? ORC_BF16_AVX512BF : ORC_BF16_AVX512F);
        EXPECT(memcmp(g16.data(), w16.data(), 32) == 0 && g16[16] == 0xabcd, "ccl_convert_fp32_to_bf16 (16 values)");
        DevBuf<uint32_t> d32(std::vector<uint32_t>(17, 0xabcdabcdu));
        ccl_convert_bf16_to_fp32(d16.p, d32.p, &sched);
        std::vector<uint32_t> g32 = d32.host();
        ok = g32[16] == 0xabcdabcdu;
        for (int i = 0; i < 16; i++) ok = ok && g32[i] == ((uint32_t)g16[i] << 16);
        EXPECT(ok, "ccl_convert_bf16_to_fp32 (16 values)");
        DevBuf<uint16_t> dh16(std::vector<uint16_t>(9, 0xabcd));
        ccl_convert_fp32_to_fp16(dv.p, dh16.p, &sched);
        std::vector<uint16_t> gh = dh16.host(), wh(8);
        orc_convert_fp32_to_fp16_arrays(v.data(), wh.data(), 8);
        EXPECT(memcmp(gh.data(), wh.data(), 16) == 0 && gh[8] == 0xabcd, "ccl_convert_fp32_to_fp16 (8 values): %04x %04x %04x %04x %04x %04x %04x",
               gh[0], gh[1], gh[2], gh[3], gh[4], gh[5], gh[6]);
        DevBuf<uint32_t> dback(std::vector<uint32_t>(9, 0xabcdabcdu));
        ccl_convert_fp16_to_fp32(dh16.p, dback.p, &sched);
        std::vector<uint32_t> gb = dback.host(), wb(8);
        orc_convert_fp16_to_fp32_arrays(gh.data(), wb.data(), 8);
        EXPECT(memcmp(gb.data(), wb.data(), 32) == 0 && gb[8] == 0xabcdabcdu, "ccl_convert_fp16_to_fp32 (8 values)");
    }
    // float16 implementation knob (fp16_utils.hpp:26-32): avx512f quiets a signalling NaN that min hands back, avx512fp16
    // keeps it, and a value that names no implementation makes the reduce a no-op, as in the reference (probe values
    // of the reference library: fp16_intrisics.hpp:204-248 has no else branch)
    {
        const ccl_fp16_impl_type saved = ccl::global_data::env().fp16_impl_type;
        std::vector<uint16_t> in = { 0x3c00, 0x3c00, 0x7c01, 0x4000 }, io = { 0x7c01, 0x4000, 0x3c00, 0x3c00 };
        struct { ccl_fp16_impl_type impl; uint16_t want[4]; } cases[] = {
            { ccl_fp16_avx512f, { 0x7e01, 0x3c00, 0x3c00, 0x3c00 } },          // min(in, io): io on NaN, quieted
            { ccl_fp16_avx512fp16, { 0x7c01, 0x3c00, 0x3c00, 0x3c00 } },       // the same operand, untouched
            { ccl_fp16_no_compiler_support, { 0x7c01, 0x4000, 0x3c00, 0x3c00 } },   // inout unchanged
        };
        for (auto& c : cases) {
            ccl::global_data::env().fp16_impl_type = c.impl;
            DevBuf<uint16_t> din(in), dio(io);
            size_t out_count = 0;
            ccl_comp_reduce(&sched, din.p, 4, dio.p, &out_count, DT(ccl::datatype::float16), ccl::reduction::min, nullptr);
            std::vector<uint16_t> got = dio.host();
            EXPECT(memcmp(got.data(), c.want, 8) == 0 && out_count == 4, "fp16 impl %d: %04x %04x %04x %04x", (int)c.impl, got[0], got[1], got[2], got[3]);
            std::vector<uint16_t> exp = io;
            orc_fp16_reduce(in.data(), 4, exp.data(), ORC_MIN, (int)c.impl);
            EXPECT(memcmp(got.data(), exp.data(), 8) == 0, "fp16 impl %d equals the oracle", (int)c.impl);
        }
        ccl::global_data::env().fp16_impl_type = saved;
    }
    // fusion manager over the HIP backend: 700 small bf16 gradient tensors arrive as individual requests, are fused
    // (tight layout, at most 256 per launch), reduced against 7 peer fusion buffers by ONE 8-input reduce per launch,
    // and unpacked.  Peer j holds the constant c_j everywhere, so the expected tensor does not depend on where the
    // manager placed it in the buffer, while a misplaced or mis-sized copy would show.
    {
        ccl_fusion_hip_backend backend;
        ccl_fusion_config cfg;
        cfg.cycle_ms = 0;
        const int NPEER = 7;
        std::vector<DevBuf<uint16_t>*> peer_bufs;
        std::vector<uint16_t> peer_val(NPEER);
        size_t buf_elems = cfg.bytes_threshold * cfg.count_threshold / 2;
        for (int j = 0; j < NPEER; j++) {
            peer_val[j] = to_lp(0.25f * (float)(j + 1), ccl::datatype::bfloat16);
            peer_bufs.push_back(new DevBuf<uint16_t>(std::vector<uint16_t>(buf_elems, peer_val[j])));
        }
        int launches = 0;
        ccl_fused_allreduce_fn allreduce = [&](void* buf, size_t n, const ccl_datatype& dt, ccl::reduction op, const void*, void* st) {
            std::vector<const void*> peers;
            for (auto* p : peer_bufs) peers.push_back(p->p);
            ccl_sched s2; s2.stream = st;
            ccl_comp_reduce_n(&s2, buf, peers, n, buf, dt, op, /*keep precision*/ 1);
            launches++;
        };
        ccl_fusion_manager mgr(&backend, allreduce, cfg);
        const int K = 700;
        std::vector<std::vector<uint16_t>> host(K);
        std::vector<DevBuf<uint16_t>*> send(K), recv(K);
        std::vector<std::unique_ptr<ccl_fusion_request>> reqs(K);
        int refused = 0;
        for (int t = 0; t < K; t++) {
            size_t n = 1 + (size_t)((t * 2654435761u) % 9000);     // up to 18 KB: some exceed the 16 KiB threshold
            host[t].resize(n);
            for (size_t i = 0; i < n; i++) host[t][i] = to_lp(0.001f * (float)((t * 31 + i) % 2001) - 1.0f, ccl::datatype::bfloat16);
            send[t] = new DevBuf<uint16_t>(host[t]);
            recv[t] = new DevBuf<uint16_t>(n + 4);
            CK(hipMemset(recv[t]->p, 0, (n + 4) * 2));
            reqs[t].reset(new ccl_fusion_request);
            reqs[t]->send_buf = send[t]->p; reqs[t]->recv_buf = recv[t]->p; reqs[t]->count = n;
            reqs[t]->dtype = DT(ccl::datatype::bfloat16); reqs[t]->reduction = ccl::reduction::sum; reqs[t]->stream = stream;
            if (!mgr.add(reqs[t].get())) {      // too large to fuse: the caller runs it unfused
                refused++;
                std::vector<const void*> peers;
                for (auto* p : peer_bufs) peers.push_back(p->p);
                ccl_comp_reduce_n(&sched, send[t]->p, peers, n, recv[t]->p, DT(ccl::datatype::bfloat16), ccl::reduction::sum, 1);
            }
            if (t % 50 == 49) mgr.execute();
        }
        reqs[K - 1]->urgent = true;             // a waiter on the last request flushes what is left
        for (int i = 0; i < 20; i++) mgr.execute();
        CK(hipStreamSynchronize(stream));
        bool all_done = true, all_ok = true;
        for (int t = 0; t < K; t++) {
            all_done = all_done && reqs[t]->is_completed();
            std::vector<uint16_t> got = recv[t]->host();
            std::vector<uint16_t> want = host[t];
            std::vector<std::vector<uint16_t>> pv(NPEER);
            std::vector<const void*> srcs = { want.data() };
            for (int j = 0; j < NPEER; j++) { pv[j].assign(want.size(), peer_val[j]); srcs.push_back(pv[j].data()); }
            std::vector<uint16_t> exp(want.size());
            orc_reduce_n(srcs.data(), NPEER + 1, exp.data(), want.size(), ORC_BFLOAT16, ORC_SUM, 1, 0, (int)ccl::global_data::env().bf16_impl_type, ORC_FP16_AVX512F);
            bool ok = memcmp(got.data(), exp.data(), want.size() * 2) == 0;
            for (size_t i = want.size(); i < got.size(); i++) ok = ok && got[i] == 0;
            if (!ok && all_ok) printf("  fused tensor %d (count %zu) differs\n", t, want.size());
            all_ok = all_ok && ok;
        }
        EXPECT(all_done, "every fused request completed");
        EXPECT(all_ok, "every tensor equals the 8-input reduce of its own data with the peers");
        EXPECT(refused > 0 && mgr.stats().fused_ops == (size_t)(K - refused), "fused %zu + unfused %d = %d", mgr.stats().fused_ops, refused, K);
        EXPECT(launches == (int)mgr.stats().fused_launches && launches >= 3 && launches < 40, "%d fused launches for %d requests", launches, K - refused);
        mgr.reset();
        for (auto* p : peer_bufs) delete p;
        for (int t = 0; t < K; t++) { delete send[t]; delete recv[t]; }
    }
    // read_reduce_write shape (reduce_scatter_large_sycl_impl.hpp:22-66): even[i] = pair[i] + local[i] for seven peers in
    // one launch, against seven oracle calls; then copy_data shape (one input per job)
    {
        const int J = 7;
        const size_t cnt[J] = { 1, 17, 4099, 0, 70001, 16, 262144 };
        std::vector<std::vector<uint16_t>> pairv(J), localv(J);
        std::vector<std::unique_ptr<DevBuf<uint16_t>>> dp, dl, de;
        std::vector<const void*> srcs, copy_srcs;
        std::vector<void*> dsts;
        std::vector<size_t> counts;
        uint32_t x = 12345;
        for (int j = 0; j < J; j++) {
            pairv[j].resize(cnt[j]); localv[j].resize(cnt[j]);
            for (size_t i = 0; i < cnt[j]; i++) {
                x = x * 1664525u + 1013904223u; pairv[j][i] = to_lp((float)((int)(x >> 8) % 2001 - 1000) / 256.f, ccl::datatype::bfloat16);
                x = x * 1664525u + 1013904223u; localv[j][i] = to_lp((float)((int)(x >> 8) % 2001 - 1000) / 512.f, ccl::datatype::bfloat16);
            }
            dp.emplace_back(new DevBuf<uint16_t>(pairv[j])); dl.emplace_back(new DevBuf<uint16_t>(localv[j]));
            de.emplace_back(new DevBuf<uint16_t>(cnt[j]));
            srcs.push_back(dp[j]->p); srcs.push_back(dl[j]->p); copy_srcs.push_back(dl[j]->p);
            dsts.push_back(de[j]->p); counts.push_back(cnt[j]);
        }
        ccl_sched sched; sched.stream = stream;
        ccl_comp_reduce_batch(&sched, srcs, 2, dsts, counts, DT(ccl::datatype::bfloat16), ccl::reduction::sum);
        for (int j = 0; j < J; j++) {
            std::vector<uint16_t> want = pairv[j];
            orc_comp_reduce(localv[j].data(), cnt[j], want.data(), ORC_BFLOAT16, ORC_SUM, (int)ccl::global_data::env().bf16_impl_type, ORC_FP16_AVX512F);
            EXPECT(de[j]->host() == want, "read_reduce_write shape: job %d of %zu elements", j, cnt[j]);
        }
        ccl_comp_reduce_batch(&sched, copy_srcs, 1, dsts, counts, DT(ccl::datatype::bfloat16), ccl::reduction::sum);
        for (int j = 0; j < J; j++) EXPECT(de[j]->host() == localv[j], "copy_data shape: job %d", j);
        bool threw = false;
        try { ccl_comp_reduce_batch(&sched, copy_srcs, 2, dsts, counts, DT(ccl::datatype::bfloat16), ccl::reduction::sum); } catch (const ccl::exception&) { threw = true; }
        EXPECT(threw, "a pointer table of the wrong length must throw");
    }
    // The chunked, double-buffered pipeline (reduce_scatter_large_impl, reduce_scatter_large_sycl_impl.hpp:98-301): chunk
    // sizes that do and do not divide the count, with and without the pair-reduce stage, in place -- bit-identical to
    // the unchunked reduce and to the oracle.
    {
        const int N = 5;
        ccl_sched sched; sched.stream = stream;
        for (ccl::datatype d : { ccl::datatype::bfloat16, ccl::datatype::float32 }) {
            const size_t esz = DT(d).size();
            for (size_t count : { (size_t)1000003, (size_t)8 * 65536, (size_t)100 }) {
                for (size_t chunk_bytes : { (size_t)65536 * esz, (size_t)48000 }) {
                    for (int with_pair = 0; with_pair < 2; with_pair++) {
                        for (int keep = 0; keep < (d == ccl::datatype::bfloat16 ? 2 : 1); keep++) {
                            std::vector<std::vector<unsigned char>> hl(N), hp(N);
                            std::vector<std::unique_ptr<DevBuf<unsigned char>>> dl, dp;
                            std::vector<const void*> local, pair;
                            uint32_t x = 777 + (uint32_t)count + with_pair;
                            auto fill = [&](std::vector<unsigned char>& h) {
                                h.resize(count * esz);
                                for (size_t i = 0; i < count; i++) {
                                    x = x * 1664525u + 1013904223u;
                                    const float v = (float)((int)(x >> 8) % 20001 - 10000) / 4096.f;
                                    if (d == ccl::datatype::bfloat16) { uint16_t b = to_lp(v, d); memcpy(&h[i * 2], &b, 2); }
                                    else memcpy(&h[i * 4], &v, 4);
                                }
                            };
                            for (int i = 0; i < N; i++) {
                                fill(hl[i]); dl.emplace_back(new DevBuf<unsigned char>(hl[i])); local.push_back(dl[i]->p);
                                if (with_pair) { fill(hp[i]); dp.emplace_back(new DevBuf<unsigned char>(hp[i])); pair.push_back(dp[i]->p); }
                            }
                            const int impl = (int)ccl::global_data::env().bf16_impl_type;
                            // oracle: staged_i = pair_i OP local_i (rounded to dtype), then the chain over i
                            std::vector<std::vector<unsigned char>> staged = hl;
                            if (with_pair)
                                for (int i = 0; i < N; i++) {
                                    staged[i] = hp[i];
                                    orc_comp_reduce(hl[i].data(), count, staged[i].data(), (int)d, ORC_SUM, impl, ORC_FP16_AVX512F);
                                }
                            std::vector<const void*> sp;
                            for (int i = 0; i < N; i++) sp.push_back(staged[i].data());
                            std::vector<unsigned char> want(count * esz);
                            orc_reduce_n(sp.data(), N, want.data(), count, (int)d, ORC_SUM, keep, 0, impl, ORC_FP16_AVX512F);
                            ccl_chunked_reducer red(chunk_bytes, N);
                            DevBuf<unsigned char> out(count * esz);
                            red.run(&sched, local, pair, count, out.p, DT(d), ccl::reduction::sum, keep);
                            EXPECT(out.host() == want, "chunked reduce: dtype %d count %zu chunk %zu pair %d keep %d", (int)d, count, chunk_bytes, with_pair, keep);
                            EXPECT(red.chunks_of_last_run() == (count * esz + chunk_bytes - 1) / chunk_bytes, "chunk count");
                            if (!with_pair) {       // the same bits as the unchunked call, and in place on input 2
                                DevBuf<unsigned char> whole(count * esz);
                                std::vector<const void*> peers(local.begin() + 1, local.end());
                                ccl_comp_reduce_n(&sched, local[0], peers, count, whole.p, DT(d), ccl::reduction::sum, keep);
                                EXPECT(whole.host() == out.host(), "chunked and unchunked reduce differ");
                                red.run(&sched, local, pair, count, dl[2]->p, DT(d), ccl::reduction::sum, keep);
                                EXPECT(dl[2]->host() == want, "chunked reduce in place");
                            }
                        }
                    }
                }
            }
        }
        // another element type and operation: int32 max with a pair stage, three inputs, a chunk of 4,000 elements
        {
            const size_t count = 100003;
            std::vector<std::vector<int32_t>> hl(3, std::vector<int32_t>(count)), hp(3, std::vector<int32_t>(count));
            uint32_t x = 99;
            for (int i = 0; i < 3; i++)
                for (size_t e = 0; e < count; e++) {
                    x = x * 1664525u + 1013904223u; hl[i][e] = (int32_t)x;
                    x = x * 1664525u + 1013904223u; hp[i][e] = (int32_t)x;
                }
            std::vector<std::unique_ptr<DevBuf<int32_t>>> dl, dp;
            std::vector<const void*> local, pair;
            for (int i = 0; i < 3; i++) {
                dl.emplace_back(new DevBuf<int32_t>(hl[i])); dp.emplace_back(new DevBuf<int32_t>(hp[i]));
                local.push_back(dl[i]->p); pair.push_back(dp[i]->p);
            }
            std::vector<int32_t> want(count);
            for (size_t e = 0; e < count; e++) {
                int32_t m = INT32_MIN;
                for (int i = 0; i < 3; i++) { m = hl[i][e] > m ? hl[i][e] : m; m = hp[i][e] > m ? hp[i][e] : m; }
                want[e] = m;
            }
            ccl_chunked_reducer red(16000, 3);
            DevBuf<int32_t> out(count);
            red.run(&sched, local, pair, count, out.p, DT(ccl::datatype::int32), ccl::reduction::max);
            EXPECT(out.host() == want, "chunked int32 max with a pair stage");
            EXPECT(red.chunks_of_last_run() == 26, "26 chunks of 4,000 elements");
        }
        bool threw = false;
        try { ccl_chunked_reducer bad(1000, 4); } catch (const ccl::exception&) { threw = true; }
        EXPECT(threw, "a chunk size that is not a multiple of 16 bytes must throw");
    }
    // Pageable host memory is refused before anything is enqueued: the reference classifies its pointers and reduces
    // host buffers on the host (comp.cpp:147-161); here a kernel on such a pointer would be a GPU memory fault.  Every
    // call below must throw and must not launch: the thread's last kernel stays the copy that went before.
    {
        const size_t count = 4096;
        std::vector<float> h_a(count, 1.0f), h_b(count, 2.0f);
        DevBuf<float> d_a(std::vector<float>(count, 3.0f)), d_b(std::vector<float>(count, 4.0f)), d_c(count);
        const ccl_datatype& f32 = DT(ccl::datatype::float32);
        const ccl_datatype& b16 = DT(ccl::datatype::bfloat16);
        for (int mode : { 1, 2 }) {
            ccl::global_data::env().check_pointers = mode;
            ccl_comp_copy(d_a.p, d_c.p, count * 4, true, &sched);
            EXPECT(std::string(mi_ccl_last_kernel()) == "copy_kernel", "marker launch");
            int refused = 0, tried = 0;
            auto must_refuse = [&](const char* what, auto&& call) {
                tried++;
                try { call(); printf("FAIL: %s did not throw\n", what); }
                catch (const ccl::exception& e) {
                    if (strstr(e.what(), "not memory the GPU can reach")) refused++;
                    else printf("FAIL: %s threw something else: %s\n", what, e.what());
                }
            };
            const std::vector<size_t> offs = { 0, count / 2 };
            must_refuse("reduce, host in", [&] { ccl_comp_reduce(&sched, h_a.data(), count, d_b.p, nullptr, f32, ccl::reduction::sum, nullptr); });
            must_refuse("reduce, host inout", [&] { ccl_comp_reduce(&sched, d_a.p, count, h_b.data(), nullptr, f32, ccl::reduction::sum, nullptr); });
            must_refuse("reduce, both host", [&] { ccl_comp_reduce(&sched, h_a.data(), count, h_b.data(), nullptr, f32, ccl::reduction::max, nullptr); });
            must_refuse("batch reduce, host buffer", [&] { ccl_comp_batch_reduce(h_a.data(), offs, count / 2, h_a.data(), nullptr, f32, ccl::reduction::sum, nullptr, nullptr, 0, nullptr, nullptr, &sched); });
            must_refuse("batch reduce, host slices", [&] { ccl_comp_batch_reduce(h_a.data(), offs, count / 2, d_b.p, nullptr, f32, ccl::reduction::sum, nullptr, nullptr, 0, nullptr, nullptr, &sched); });
            must_refuse("copy, host in", [&] { ccl_comp_copy(h_a.data(), d_b.p, count * 4, false, &sched); });
            must_refuse("copy, host out", [&] { ccl_comp_copy(d_a.p, h_b.data(), count * 4, true, &sched); });
            must_refuse("reduce_n, host peer", [&] { ccl_comp_reduce_n(&sched, d_a.p, { d_b.p, h_a.data() }, count, d_c.p, f32, ccl::reduction::sum); });
            must_refuse("reduce_n, host out", [&] { ccl_comp_reduce_n(&sched, d_a.p, { d_b.p }, count, h_b.data(), f32, ccl::reduction::sum); });
            must_refuse("reduce_write_n, host out", [&] { ccl_comp_reduce_write_n(&sched, d_a.p, { d_b.p }, count, { d_c.p, h_b.data() }, f32, ccl::reduction::sum); });
            must_refuse("reduce_batch, host input", [&] { ccl_comp_reduce_batch(&sched, { d_a.p, d_b.p, d_a.p, h_a.data() }, 2, { d_c.p, d_c.p }, { 16, 16 }, f32, ccl::reduction::sum); });
            must_refuse("bf16 reduce, host in", [&] { ccl_bf16_reduce(h_a.data(), count, d_b.p, nullptr, ccl::reduction::sum, &sched); });
            must_refuse("fp16 reduce, host inout", [&] { ccl_fp16_reduce(d_a.p, count, h_b.data(), nullptr, ccl::reduction::sum, &sched); });
            must_refuse("fp32 -> bf16, host source", [&] { ccl_convert_fp32_to_bf16_arrays(h_a.data(), d_b.p, count, &sched); });
            must_refuse("bf16 -> fp32, host destination", [&] { ccl_convert_bf16_to_fp32_arrays(d_a.p, h_b.data(), count, &sched); });
            (void)b16;
            EXPECT(refused == tried, "mode %d: %d of %d calls on pageable host memory were refused", mode, refused, tried);
            EXPECT(std::string(mi_ccl_last_kernel()) == "copy_kernel", "mode %d: a refused call launched %s", mode, mi_ccl_last_kernel());
            CK(hipStreamSynchronize(stream));
            bool untouched = true;
            for (size_t i = 0; i < count; i++) untouched = untouched && h_a[i] == 1.0f && h_b[i] == 2.0f;
            std::vector<float> ga = d_a.host(), gb = d_b.host();
            for (size_t i = 0; i < count; i++) untouched = untouched && ga[i] == 3.0f && gb[i] == 4.0f;
            EXPECT(untouched, "mode %d: refused calls left every buffer as it was", mode);
            // a device buffer that is too short for the count is refused too (its allocation's extent is known)
            bool threw = false;
            try { ccl_comp_reduce(&sched, d_a.p, count * 1024, d_b.p, nullptr, f32, ccl::reduction::sum, nullptr); }
            catch (const ccl::exception& e) { threw = strstr(e.what(), "runs past the end") != nullptr; }
            EXPECT(threw, "mode %d: a count beyond the allocation must throw", mode);
            EXPECT(std::string(mi_ccl_last_kernel()) == "copy_kernel", "mode %d: the oversized call launched %s", mode, mi_ccl_last_kernel());
            // pinned host memory is memory the GPU can reach: accepted, and the result is right
            float* pinned = nullptr;
            CK(hipHostMalloc((void**)&pinned, count * 4, hipHostMallocDefault));
            for (size_t i = 0; i < count; i++) pinned[i] = (float)i;
            ccl_comp_reduce(&sched, pinned, count, d_b.p, nullptr, f32, ccl::reduction::sum, nullptr);
            gb = d_b.host();
            bool ok = true;
            for (size_t i = 0; i < count; i++) ok = ok && gb[i] == 4.0f + (float)i;
            EXPECT(ok, "mode %d: pinned host input", mode);
            CK(hipMemcpy(d_b.p, std::vector<float>(count, 4.0f).data(), count * 4, hipMemcpyHostToDevice));
            CK(hipHostFree(pinned));
            ccl_comp_forget_pointers();
        }
        // custom reduction on two host buffers: the callback runs on them as they are (comp.cpp:84-88)
        std::vector<int32_t> ha(100), hb(100);
        for (int i = 0; i < 100; i++) { ha[i] = i; hb[i] = 5; }
        size_t oc = 0;
        ccl_comp_reduce(&sched, ha.data(), 100, hb.data(), &oc, DT(ccl::datatype::int32), ccl::reduction::custom, custom_sum_i32);
        bool ok = oc == 100;
        for (int i = 0; i < 100; i++) ok = ok && hb[i] == 10 + i;
        EXPECT(ok, "custom reduction on host buffers");
        // the check switched off: a good call still works (nothing is ever launched on a bad pointer here)
        ccl::global_data::env().check_pointers = 0;
        ccl_comp_reduce(&sched, d_a.p, count, d_b.p, nullptr, f32, ccl::reduction::sum, nullptr);
        EXPECT(d_b.host()[17] == 7.0f, "check_pointers = 0");
        ccl::global_data::env().check_pointers = 1;
    }
    // profiler ranges around the operator-level calls: none unless switched on (MI_CCL_TRACE=1 or ccl_trace_enable)
    {
        DevBuf<float> a(std::vector<float>(64, 1.0f)), b(std::vector<float>(64, 2.0f));
        const unsigned long before = ccl_trace_ranges_opened();
        if (!getenv("MI_CCL_TRACE")) {
            ccl_comp_reduce(&sched, a.p, 64, b.p, nullptr, DT(ccl::datatype::float32), ccl::reduction::sum, nullptr);
            EXPECT(ccl_trace_ranges_opened() == before, "a range was opened with the knob off");
        }
        ccl_trace_enable(true);
        const unsigned long on0 = ccl_trace_ranges_opened();
        ccl_comp_reduce(&sched, a.p, 64, b.p, nullptr, DT(ccl::datatype::float32), ccl::reduction::sum, nullptr);
        ccl_comp_copy(a.p, b.p, 64 * 4, false, &sched);
        EXPECT(ccl_trace_ranges_opened() == on0 + 2, "two calls, two ranges");
        ccl_trace_enable(false);
        EXPECT(b.host()[5] == 1.0f, "results with ranges on");
    }
    CK(hipStreamDestroy(stream));
    printf("%d checks, %d failed\n", g_checks, g_fail);
    return g_fail ? 1 : 0;
}
