// GPU test of the scheduler entries (oneccl_amd/csrc/ccl_sched_entry.hpp) and of the device form of
// ccl::reduction::custom (ccl_custom_reduce.hpp).  A schedule is built the way the reference's reduce-scatter and
// allreduce schedules are (src/coll/algorithms/reduce_scatter.cpp:111-136: copy the own block, then one RECV_REDUCE
// per peer), run with do_progress() until complete, and checked against the closed forms of the reference's
// functional tests (tests/functional/test_impl.hpp:242-324) and bit for bit against the oracle.  The "network" is a
// loop-back transport: a receive from rank r is an asynchronous device copy of rank r's buffer.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "../../oneccl_amd/csrc/ccl_custom_reduce.hpp"
#include "../../oracle/ccl_comp_oracle.h"

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); exit(2); } } while (0)
static int g_fail = 0, g_checks = 0;
#define EXPECT(cond, ...) do { g_checks++; if (!(cond)) { g_fail++; printf("FAIL line %d: ", __LINE__); printf(__VA_ARGS__); printf("\n"); } } while (0)
#define EXPECT_THROWS(stmt, what) do { bool threw_ = false; try { stmt; } catch (const ccl::exception&) { threw_ = true; } EXPECT(threw_, "%s should throw", what); } while (0)

static const ccl_datatype& DT(ccl::datatype d) { return ccl_datatype_storage::instance().get(d); }

template <class T> struct DevBuf {
    T* p = nullptr; size_t n;
    explicit DevBuf(size_t n_) : n(n_) { CK(hipMalloc(&p, (n ? n : 1) * sizeof(T))); CK(hipMemset(p, 0, (n ? n : 1) * sizeof(T))); }
    explicit DevBuf(const std::vector<T>& h) : n(h.size()) { CK(hipMalloc(&p, (n ? n : 1) * sizeof(T))); CK(hipMemcpy(p, h.data(), n * sizeof(T), hipMemcpyHostToDevice)); }
    ~DevBuf() { (void)hipFree(p); }
    std::vector<T> host() const { std::vector<T> h(n); CK(hipDeviceSynchronize()); CK(hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost)); return h; }
    ccl_buffer buf() const { return ccl_buffer(p, (ssize_t)(n * sizeof(T))); }
};

// rank -> device buffer of that rank; recv = async copy on a private stream, completion = its event.  delay_checks
// makes a receive report "not yet" that many times after the copy has finished; again_first makes the first post
// of every receive return ATL_STATUS_AGAIN.
struct loopback_transport : atl_base_comm {
    std::map<int, const void*> rank_data;
    hipStream_t copy_stream;
    int delay_checks = 0, again_first = 0, posted = 0, cancelled = 0;
    std::map<uint64_t, int> tags_seen;
    struct pending { hipEvent_t ev; int wait; };
    loopback_transport() { CK(hipStreamCreate(&copy_stream)); }
    ~loopback_transport() override { (void)hipStreamDestroy(copy_stream); }
    atl_status_t recv(void* buf, size_t bytes, int src, uint64_t tag, atl_req_t& req) override {
        if (again_first > 0) { again_first--; return ATL_STATUS_AGAIN; }
        if (!rank_data.count(src)) return ATL_STATUS_FAILURE;
        tags_seen[tag]++;
        pending* p = new pending{ nullptr, delay_checks };
        CK(hipEventCreateWithFlags(&p->ev, hipEventDisableTiming));
        CK(hipMemcpyAsync(buf, rank_data[src], bytes, hipMemcpyDeviceToDevice, copy_stream));
        CK(hipEventRecord(p->ev, copy_stream));
        req.internal = p; req.is_completed = 0; posted++;
        return ATL_STATUS_SUCCESS;
    }
    atl_status_t check(atl_req_t& req) override {
        pending* p = (pending*)req.internal;
        if (!p) return ATL_STATUS_FAILURE;
        hipError_t e = hipEventQuery(p->ev);
        if (e == hipErrorNotReady) return ATL_STATUS_SUCCESS;
        if (e != hipSuccess) return ATL_STATUS_FAILURE;
        if (p->wait-- > 0) return ATL_STATUS_SUCCESS;
        (void)hipEventDestroy(p->ev); delete p; req.internal = nullptr; req.is_completed = 1;
        return ATL_STATUS_SUCCESS;
    }
    void cancel(atl_req_t& req) override {
        pending* p = (pending*)req.internal;
        if (p) { CK(hipStreamSynchronize(copy_stream)); (void)hipEventDestroy(p->ev); delete p; req.internal = nullptr; }
        cancelled++;
    }
};

static int run_to_completion(ccl_sched& s, int limit = 2000000) {
    int calls = 0;
    while (!s.is_completed() && calls < limit) { s.do_progress(); calls++; }
    return calls;
}

static uint16_t bf16(float v) { uint32_t u; memcpy(&u, &v, 4); return orc_bf16_narrow_rne(u); }

struct absmax { __device__ float operator()(float in, float inout) const { return fmaxf(fabsf(in), fabsf(inout)); } };
struct val_idx { float v; int32_t i; };
struct argmax { __device__ val_idx operator()(val_idx in, val_idx inout) const { return (in.v > inout.v || (in.v == inout.v && in.i < inout.i)) ? in : inout; } };
struct xor_u16 { __device__ uint16_t operator()(uint16_t in, uint16_t inout) const { return (uint16_t)(in ^ inout); } };
struct sat_add_u8 { __device__ uint8_t operator()(uint8_t in, uint8_t inout) const { unsigned s = (unsigned)in + inout; return (uint8_t)(s > 255 ? 255 : s); } };

static const char* g_match_seen = nullptr; static size_t g_offset_seen = 0;
static void host_fn(const void* in, size_t n, void* inout, size_t* out_count, ccl::datatype, const ccl::fn_context* ctx) {
    const int32_t* a = (const int32_t*)in; int32_t* b = (int32_t*)inout;
    for (size_t i = 0; i < n; i++) b[i] = 3 * b[i] - a[i];
    if (out_count) *out_count = n;
    g_match_seen = ctx->match_id; g_offset_seen = ctx->offset;
}

int main() {
    int ndev = 0; CK(hipGetDeviceCount(&ndev));
    if (ndev < 1) { printf("no GPU\n"); return 2; }
    hipStream_t stream; CK(hipStreamCreate(&stream));

    // ---- ccl_buffer: offsets and bounds (src/common/utils/buffer.hpp) ----
    {
        char base[64];
        ccl_buffer b(base, 64);
        EXPECT((b + 16).get_ptr(48) == base + 16 && (b + 16).get_offset() == 16, "offset arithmetic");
        EXPECT(((b + 16) - 8).get_ptr() == base + 8, "decrement");
        EXPECT_THROWS((b + 16).get_ptr(49), "access past the end");
        EXPECT_THROWS((b + 8) - 9, "decrement below zero");
        ccl_buffer unknown(base, -1);
        EXPECT(unknown.get_ptr(1 << 20) == base, "unknown size is not checked");
        EXPECT(ccl_buffer().get_ptr() == nullptr && !ccl_buffer(), "default buffer is null");
    }

    // ---- reduce-scatter style schedule: COPY own block, RECV_REDUCE from every peer, WRITE_MONOLITHIC ----
    for (ccl::datatype d : { ccl::datatype::float32, ccl::datatype::bfloat16, ccl::datatype::int32 }) {
        for (ccl::reduction op : { ccl::reduction::sum, ccl::reduction::max }) {
            const int N = 8; const size_t count = 32771;    // one of the reference's sizes (tests/functional/conf.cpp:51-53)
            const size_t esz = DT(d).size();
            std::vector<std::vector<unsigned char>> send(N, std::vector<unsigned char>(count * esz));
            for (int r = 0; r < N; r++)
                for (size_t i = 0; i < count; i++) {
                    double v = (d == ccl::datatype::bfloat16 ? 0.5 : 1.0) * r + (double)(i % 7);    // c1*rank + c2*buf_idx
                    if (d == ccl::datatype::float32) { float f = (float)v; memcpy(&send[r][i * 4], &f, 4); }
                    else if (d == ccl::datatype::int32) { int32_t x = (int32_t)v; memcpy(&send[r][i * 4], &x, 4); }
                    else { uint16_t h = bf16((float)v); memcpy(&send[r][i * 2], &h, 2); }
                }
            std::vector<unsigned char> want = send[0];
            for (int r = 1; r < N; r++)
                orc_comp_reduce(send[r].data(), count, want.data(), (int)d, (int)op, ORC_BF16_AVX512BF, ORC_FP16_AVX512F);
            std::vector<DevBuf<unsigned char>*> dev;
            loopback_transport net;
            for (int r = 0; r < N; r++) { dev.push_back(new DevBuf<unsigned char>(send[r])); net.rank_data[r] = dev[r]->p; }
            net.delay_checks = 3; net.again_first = 2;
            ccl_comm comm; comm.m_rank = 0; comm.m_size = N; comm.comm_id = 5; comm.atl = &net;
            DevBuf<unsigned char> recv(count * esz + 64), out1(count * esz), out2(count * esz), out3(count * esz);
            ccl_sched sched; sched.stream = stream;
            entry_factory::create<copy_entry>(&sched, dev[0]->buf(), recv.buf(), count, DT(d), copy_attr(copy_direction::d2d));
            for (int r = 1; r < N; r++) {       // a barrier after every step that the next one depends on
                entry_factory::create<recv_reduce_entry>(&sched, recv.buf(), count, DT(d), op, r, &comm);
                sched.add_barrier();
            }
            auto* w = entry_factory::create<write_monolithic_entry>(&sched, recv.buf(), count,
                                                                    std::vector<ccl_buffer>{ out1.buf(), out2.buf(), out3.buf() }, DT(d));
            EXPECT(std::string(w->name()) == "WRITE_MONOLITHIC" && sched.entries.size() == (size_t)N + 1, "schedule built");
            int calls = run_to_completion(sched);
            EXPECT(sched.is_completed(), "schedule completed after %d progress calls", calls);
            EXPECT(net.posted == N - 1 && net.tags_seen.size() == (size_t)N - 1, "one receive per peer, distinct tags (%d, %zu)", net.posted, net.tags_seen.size());
            for (auto* o : { &out1, &out2, &out3 }) {
                std::vector<unsigned char> got = o->host();
                EXPECT(memcmp(got.data(), want.data(), count * esz) == 0, "schedule result vs oracle chain, dtype %d op %d", (int)d, (int)op);
            }
            std::vector<unsigned char> tail = recv.host();
            bool clean = true; for (size_t i = count * esz; i < tail.size(); i++) clean = clean && tail[i] == 0;
            EXPECT(clean, "nothing written past the block");
            if (d == ccl::datatype::int32 && op == ccl::reduction::sum) {       // closed form: N(N-1)/2 + N*buf_idx
                std::vector<unsigned char> got = out1.host();
                bool ok = true;
                for (size_t i = 0; i < count; i++) { int32_t x; memcpy(&x, &got[i * 4], 4); ok = ok && x == N * (N - 1) / 2 + N * (int)(i % 7); }
                EXPECT(ok, "closed form of the functional tests");
            }
            // the schedule again (a cached schedule is renewed and rerun): same inputs -> same result
            sched.renew();
            EXPECT(!sched.is_completed() && sched.entries[0]->get_status() == ccl_sched_entry_status_not_started, "renew");
            run_to_completion(sched);
            std::vector<unsigned char> again = out2.host();
            EXPECT(sched.is_completed() && memcmp(again.data(), want.data(), count * esz) == 0, "second run of the schedule");
            for (auto* p : dev) delete p;
        }
    }

    // ---- progress rules: barrier entries, complete_once, a receive that is still pending when the schedule dies ----
    {
        std::vector<int32_t> a(1000, 1), b(1000, 10);
        DevBuf<int32_t> in(a), io(b);
        ccl_sched sched; sched.stream = stream;
        auto* e0 = entry_factory::create<reduce_local_entry>(&sched, in.buf(), 1000, io.buf(), nullptr, DT(ccl::datatype::int32), ccl::reduction::sum);
        auto* e1 = entry_factory::create<reduce_local_entry>(&sched, in.buf(), 1000, io.buf(), nullptr, DT(ccl::datatype::int32), ccl::reduction::sum);
        auto* e2 = entry_factory::create<reduce_local_entry>(&sched, in.buf(), 1000, io.buf(), nullptr, DT(ccl::datatype::int32), ccl::reduction::sum);
        e0->set_exec_mode(ccl_sched_entry_exec_once);
        e1->make_barrier();
        // hold the stream so that nothing can complete while the first walk is looked at
        hipEvent_t gate; CK(hipEventCreate(&gate));
        hipStream_t other; CK(hipStreamCreate(&other));
        DevBuf<int32_t> big(64 << 20);
        CK(hipMemsetAsync(big.p, 1, big.n * 4, other));
        CK(hipEventRecord(gate, other));
        CK(hipStreamWaitEvent(stream, gate, 0));
        sched.do_progress();
        bool held = hipEventQuery(gate) == hipErrorNotReady;
        if (held) EXPECT(e0->get_status() == ccl_sched_entry_status_started && e1->get_status() == ccl_sched_entry_status_started &&
                         e2->get_status() == ccl_sched_entry_status_not_started, "a barrier that has not completed holds later entries back");
        run_to_completion(sched);
        EXPECT(e0->get_status() == ccl_sched_entry_status_complete_once && e2->get_status() == ccl_sched_entry_status_complete, "final statuses");
        EXPECT(io.host()[999] == 13, "three reduces ran: %d", io.host()[999]);
        sched.renew();
        run_to_completion(sched);
        EXPECT(io.host()[0] == 15, "an entry marked exec_once does not run again: %d", io.host()[0]);
        std::stringstream ss; e1->dump(ss, 1);
        EXPECT(ss.str().find("REDUCE_LOCAL") != std::string::npos && ss.str().find("int32") != std::string::npos && ss.str().find("barrier") != std::string::npos, "dump: %s", ss.str().c_str());
        CK(hipEventDestroy(gate)); CK(hipStreamDestroy(other));

        loopback_transport net; net.rank_data[1] = in.p; net.delay_checks = 1 << 30;
        ccl_comm comm; comm.atl = &net; comm.m_size = 2;
        {
            ccl_sched s2; s2.stream = stream;
            entry_factory::create<recv_reduce_entry>(&s2, io.buf(), 1000, DT(ccl::datatype::int32), ccl::reduction::sum, 1, &comm);
            for (int i = 0; i < 10; i++) s2.do_progress();
            EXPECT(!s2.is_completed() && net.posted == 1, "receive stays pending");
        }
        EXPECT(net.cancelled == 1, "a started receive is cancelled when its entry is destroyed");
        ccl_sched s3; s3.stream = stream;
        EXPECT_THROWS(entry_factory::create<reduce_local_entry>(&s3, in.buf(), 1000, io.buf(), nullptr, DT(ccl::datatype::int32), ccl::reduction::custom), "custom without a callback");
        EXPECT_THROWS(entry_factory::create<recv_reduce_entry>(&s3, ccl_buffer(), 10, DT(ccl::datatype::int32), ccl::reduction::sum, 1, &comm), "null result buffer");
        auto* eb = entry_factory::create<reduce_local_entry>(&s3, in.buf(), 1001, io.buf(), nullptr, DT(ccl::datatype::int32), ccl::reduction::sum);
        (void)eb;
        EXPECT_THROWS(s3.do_progress(), "count beyond the buffer size");
    }

    // ---- RECV_REDUCE into the communication buffer; host callback with match id and offset ----
    {
        std::vector<int32_t> a(777), b(777);
        for (int i = 0; i < 777; i++) { a[i] = i; b[i] = 1000 - i; }
        DevBuf<int32_t> peer(a), io(b), cb(777);
        loopback_transport net; net.rank_data[3] = peer.p;
        ccl_comm comm; comm.atl = &net; comm.m_size = 4;
        ccl_sched sched; sched.stream = stream;
        entry_factory::create<recv_reduce_entry>(&sched, io.buf(), 777, DT(ccl::datatype::int32), ccl::reduction::min, 3, &comm, cb.buf(), ccl_recv_reduce_comm_buf);
        run_to_completion(sched);
        std::vector<int32_t> got = cb.host(), keep = io.host();
        bool ok = true; for (int i = 0; i < 777; i++) ok = ok && got[i] == std::min(a[i], b[i]) && keep[i] == b[i];
        EXPECT(ok, "result in the communication buffer, inout untouched");

        ccl_sched s2; s2.stream = stream; s2.coll_attr.reduction_fn = host_fn; s2.coll_attr.match_id = "grad.7";
        entry_factory::create<reduce_local_entry>(&s2, peer.buf(), 700, io.buf() + 77 * 4, nullptr, DT(ccl::datatype::int32), ccl::reduction::custom);
        run_to_completion(s2);
        got = io.host();
        ok = true; for (int i = 0; i < 777; i++) ok = ok && got[i] == (i < 77 ? b[i] : 3 * b[i] - a[i - 77]);
        EXPECT(ok && g_match_seen && std::string(g_match_seen) == "grad.7" && g_offset_seen == 77 * 4, "host callback through the entry: match id and byte offset");
    }

    // ---- REDUCE_MONOLITHIC with block offsets (ze_a2a_reduce_scatter_entry.cpp:64-106) vs the oracle ----
    {
        const int P = 7; const size_t total = 40000, rank_off = 12345, peer_off = 100, cnt = 20001;
        std::vector<std::vector<uint16_t>> h(P + 1, std::vector<uint16_t>(total + peer_off));
        for (int r = 0; r <= P; r++) for (size_t i = 0; i < h[r].size(); i++) h[r][i] = bf16(0.001f * (float)((i * 37 + r * 101) % 4001) - 2.0f);
        std::vector<DevBuf<uint16_t>*> dev; std::vector<ccl_buffer> peers;
        for (int r = 0; r <= P; r++) dev.push_back(new DevBuf<uint16_t>(h[r]));
        for (int r = 1; r <= P; r++) peers.push_back(dev[r]->buf());
        DevBuf<uint16_t> out(cnt + 8);
        for (int keep = 0; keep <= 1; keep++) {
            ccl_sched sched; sched.stream = stream;
            entry_factory::create<reduce_monolithic_entry>(&sched, dev[0]->buf(), rank_off, cnt, peers, peer_off, out.buf(), DT(ccl::datatype::bfloat16), ccl::reduction::sum, keep);
            run_to_completion(sched);
            std::vector<const void*> srcs = { h[0].data() + rank_off };
            for (int r = 1; r <= P; r++) srcs.push_back(h[r].data() + rank_off + peer_off);
            std::vector<uint16_t> want(cnt), got = out.host();
            orc_reduce_n(srcs.data(), P + 1, want.data(), cnt, ORC_BFLOAT16, ORC_SUM, keep, 0, ORC_BF16_AVX512BF, ORC_FP16_AVX512F);
            EXPECT(memcmp(got.data(), want.data(), cnt * 2) == 0 && got[cnt] == 0, "monolithic reduce of 1 + 7 blocks, keep precision %d", keep);
        }
        ccl_sched s2; s2.stream = stream;
        entry_factory::create<reduce_monolithic_entry>(&s2, dev[0]->buf(), rank_off, total, peers, peer_off, out.buf(), DT(ccl::datatype::bfloat16), ccl::reduction::sum);
        EXPECT_THROWS(s2.do_progress(), "block beyond the send buffer");
        for (auto* p : dev) delete p;
    }

    // ---- COPY directions and element offsets ----
    {
        std::vector<float> h(5000); for (int i = 0; i < 5000; i++) h[i] = 0.5f * i;
        std::vector<float> back(5000, -1.f);
        DevBuf<float> d1(5000), d2(5000);
        ccl_sched sched; sched.stream = stream;
        const ccl_datatype& f32 = DT(ccl::datatype::float32);
        entry_factory::create<copy_entry>(&sched, ccl_buffer(h.data(), 20000), d1.buf(), 5000, f32, copy_attr(copy_direction::h2d));
        entry_factory::create<copy_entry>(&sched, d1.buf(), d2.buf(), 4000, f32, copy_attr(copy_direction::d2d, 1000, 500));
        entry_factory::create<copy_entry>(&sched, d2.buf(), ccl_buffer(back.data(), 20000), 5000, f32, copy_attr(copy_direction::undefined));
        run_to_completion(sched);
        CK(hipStreamSynchronize(stream));
        bool ok = true;
        for (int i = 0; i < 5000; i++) ok = ok && back[i] == ((i >= 500 && i < 4500) ? h[i + 500] : 0.f);
        EXPECT(ok, "h2d, d2d with element offsets, d2h with the direction found from the pointers");
        ccl_sched s2; s2.stream = stream;
        entry_factory::create<copy_entry>(&s2, d1.buf(), d2.buf(), 4000, f32, copy_attr(copy_direction::d2d, 1000, 1001));
        EXPECT_THROWS(s2.do_progress(), "copy past the end of the output buffer");
    }

    // ---- ccl::reduction::custom as a device functor ----
    {
        const size_t n = 100003;
        std::vector<float> a(n), b(n);
        for (size_t i = 0; i < n; i++) { a[i] = sinf((float)i) * 3.f; b[i] = cosf((float)i * 1.7f) * 3.f; }
        DevBuf<float> da(a), db(b);
        ccl_sched sched; sched.stream = stream;
        entry_factory::create<custom_reduce_local_entry<float, absmax>>(&sched, da.buf(), n, db.buf(), absmax{});
        run_to_completion(sched);
        std::vector<float> got = db.host();
        bool ok = true; for (size_t i = 0; i < n; i++) ok = ok && got[i] == fmaxf(fabsf(a[i]), fabsf(b[i]));
        EXPECT(ok, "absmax through a REDUCE_LOCAL_CUSTOM entry");

        // five inputs of an 8-byte (value, index) pair: arg-max with ties to the lower index; aligned and misaligned
        const int N = 5; const size_t m = 70001;
        std::vector<std::vector<val_idx>> h(N, std::vector<val_idx>(m + 1));
        for (int r = 0; r < N; r++) for (size_t i = 0; i <= m; i++) h[r][i] = { (float)((i * 7919 + r * 104729) % 1000), (int32_t)(r * 1000000 + (int)i) };
        for (int shift = 0; shift <= 1; shift++) {
            std::vector<DevBuf<val_idx>*> dev; std::vector<const val_idx*> srcs;
            for (int r = 0; r < N; r++) { dev.push_back(new DevBuf<val_idx>(h[r])); srcs.push_back(dev[r]->p + shift); }
            DevBuf<val_idx> out(m + 1);
            ccl_custom_reduce_n<val_idx>(&sched, srcs, out.p + shift, m, argmax{});
            std::vector<val_idx> g = out.host();
            ok = true;
            for (size_t i = 0; i < m; i++) {
                val_idx w = h[0][i + shift];
                for (int r = 1; r < N; r++) { val_idx x = h[r][i + shift]; if (x.v > w.v || (x.v == w.v && x.i < w.i)) w = x; }
                ok = ok && g[i + shift].v == w.v && g[i + shift].i == w.i;
            }
            EXPECT(ok, "argmax over 5 inputs of 8-byte pairs, shift %d", shift);
            for (auto* p : dev) delete p;
        }
        std::vector<uint8_t> u(1001, 200), v(1001, 100);
        DevBuf<uint8_t> du(u), dv(v);
        ccl_custom_reduce_n<uint8_t>(&sched, { du.p + 1, dv.p + 1, dv.p + 1 }, du.p + 1, 1000, sat_add_u8{});
        std::vector<uint8_t> gu = du.host();
        EXPECT(gu[0] == 200 && gu[1] == 255 && gu[1000] == 255, "saturating byte add, in place, odd alignment");

        // sources and output at different offsets from a 16-byte boundary (loose vector reads)
        {
            const size_t cnt = 50021;
            std::vector<uint16_t> x(cnt + 16), y(cnt + 16);
            for (size_t i = 0; i < x.size(); i++) { x[i] = (uint16_t)(i * 31 + 7); y[i] = (uint16_t)(i * 17 + 3); }
            DevBuf<uint16_t> dx(x), dy(y), dz(cnt + 16);
            ccl_custom_reduce_n<uint16_t>(&sched, { dx.p + 1, dy.p + 6 }, dz.p + 3, cnt, xor_u16{});
            std::vector<uint16_t> gz = dz.host();
            ok = gz[2] == 0 && gz[3 + cnt] == 0;
            for (size_t i = 0; i < cnt; i++) ok = ok && gz[3 + i] == (uint16_t)(x[1 + i] ^ y[6 + i]);
            EXPECT(ok, "16-bit xor with every buffer at its own alignment");
        }
    }

    CK(hipStreamDestroy(stream));
    printf("%d checks, %d failed\n", g_checks, g_fail);
    return g_fail ? 1 : 0;
}
