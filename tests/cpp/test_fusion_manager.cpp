// Host-only test of the fusion manager's queueing logic (oneccl_amd/csrc/ccl_fusion.{hpp,cpp}) with a mock backend:
// host memory, memcpy pack/unpack at running offsets, an "allreduce" that doubles every int32/float element (two
// ranks holding the same data), completion tokens that become ready a few polls after they are recorded.
// Built with g++ (no HIP); exit status 0 = all checks passed.
#include <stdio.h>
#include <string.h>

#include <thread>

#include "../../oneccl_amd/csrc/ccl_fusion.hpp"

// the two functions of ccl_comp.cpp that the manager's headers need on the host
size_t ccl_datatype::size() const { return m_size; }

static int g_fail = 0, g_checks = 0;
#define EXPECT(cond, ...) do { g_checks++; if (!(cond)) { g_fail++; printf("FAIL line %d: ", __LINE__); printf(__VA_ARGS__); printf("\n"); } } while (0)

struct mock_backend : ccl_fusion_backend {
    int allocs = 0, releases = 0, packs = 0, unpacks = 0, delay = 0;
    std::vector<size_t> pack_sizes;
    void* alloc(size_t bytes) override { allocs++; return malloc(bytes); }
    void release(void* buf) override { releases++; free(buf); }
    void pack(const std::vector<const void*>& t, const std::vector<size_t>& c, const ccl_datatype& d, void* fb, void*) override {
        size_t off = 0;
        for (size_t i = 0; i < t.size(); i++) { memcpy((char*)fb + off, t[i], c[i] * d.size()); off += c[i] * d.size(); }
        packs++; pack_sizes.push_back(t.size());
    }
    void unpack(const void* fb, const std::vector<void*>& t, const std::vector<size_t>& c, const ccl_datatype& d, void*) override {
        size_t off = 0;
        for (size_t i = 0; i < t.size(); i++) { memcpy(t[i], (const char*)fb + off, c[i] * d.size()); off += c[i] * d.size(); }
        unpacks++;
    }
    std::shared_ptr<void> record(void*) override { return std::shared_ptr<void>(new int(delay), [](void* p) { delete (int*)p; }); }
    bool ready(const std::shared_ptr<void>& tok) override { int* n = (int*)tok.get(); if (*n > 0) { (*n)--; return false; } return true; }
};

static void doubling_allreduce(void* buf, size_t n, const ccl_datatype& d, ccl::reduction, const void*, void*) {
    if (d.idx() == ccl::datatype::int32) for (size_t i = 0; i < n; i++) ((int32_t*)buf)[i] *= 2;
    else for (size_t i = 0; i < n; i++) ((float*)buf)[i] *= 2.0f;
}

static const ccl_datatype I32(ccl::datatype::int32, 4), F32(ccl::datatype::float32, 4);

struct req_t {
    ccl_fusion_request r;
    std::vector<int32_t> send, recv;
    req_t(size_t n, int seed, const ccl_datatype& dt = I32) : send(n), recv(n, -1) {
        for (size_t i = 0; i < n; i++) send[i] = seed * 1000 + (int)i;
        r.send_buf = send.data(); r.recv_buf = recv.data(); r.count = n; r.dtype = dt; r.reduction = ccl::reduction::sum;
    }
    bool ok() const { for (size_t i = 0; i < send.size(); i++) if (recv[i] != 2 * send[i]) return false; return true; }
};

int main() {
    ccl_fusion_config cfg;
    cfg.cycle_ms = 0;
    {   // what can be fused (fusion.cpp:97-127)
        mock_backend b;
        ccl_fusion_manager m(&b, doubling_allreduce, cfg);
        req_t small(100, 1), big(4096, 2);           // 16384 bytes is not < bytes_threshold
        EXPECT(m.can_fuse(&small.r), "small request");
        EXPECT(!m.can_fuse(&big.r), "bytes >= threshold");
        req_t c(10, 3); c.r.reduction_fn = (ccl::reduction_fn)1;
        EXPECT(!m.can_fuse(&c.r), "custom reduction");
        req_t s(10, 4); s.r.synchronous = true;
        EXPECT(!m.can_fuse(&s.r), "synchronous");
        req_t d(10, 5); d.r.deps = 1;
        EXPECT(!m.can_fuse(&d.r), "dependencies");
        EXPECT(!m.add(&big.r) && big.r.is_completed(), "add refuses what cannot be fused");
        EXPECT(m.buffer_size() == 16384 * 256, "buffer size = bytes_threshold * count_threshold");
    }
    {   // nothing is flushed until a request is urgent; then everything gathered so far goes in one launch
        mock_backend b; b.delay = 2;
        ccl_fusion_manager m(&b, doubling_allreduce, cfg);
        std::vector<std::unique_ptr<req_t>> rs;
        for (int i = 0; i < 10; i++) { rs.emplace_back(new req_t(17 + i, i)); EXPECT(m.add(&rs.back()->r), "add"); }
        for (int i = 0; i < 5; i++) m.execute();
        EXPECT(b.packs == 0 && !rs[0]->r.is_completed(), "no flush without a reason");
        rs[7]->r.urgent = true;
        m.execute();
        EXPECT(b.packs == 1 && b.pack_sizes[0] == 10 && b.unpacks == 1, "urgent request flushes the whole queue");
        EXPECT(!rs[0]->r.is_completed(), "not complete before the backend says so");
        int polls = 0; while (!rs[0]->r.is_completed() && polls < 10) polls++;
        bool all = true; for (auto& r : rs) all = all && r->r.is_completed() && r->ok();
        EXPECT(all, "all ten requests completed with the reduced values in their own buffers");
        EXPECT(m.stats().fused_ops == 10 && m.stats().fused_launches == 1, "stats");
        EXPECT(!rs[7]->r.urgent, "urgent flag cleared");
        m.reset();
        EXPECT(m.can_reset(), "nothing in flight after reset");
    }
    {   // count threshold (fusion.cpp:441-445)
        mock_backend b;
        ccl_fusion_config c2 = cfg; c2.count_threshold = 4;
        ccl_fusion_manager m(&b, doubling_allreduce, c2);
        std::vector<std::unique_ptr<req_t>> rs;
        for (int i = 0; i < 9; i++) { rs.emplace_back(new req_t(8, i)); m.add(&rs.back()->r); }
        m.execute(); m.execute(); m.execute();
        EXPECT(b.packs == 2 && b.pack_sizes[0] == 4 && b.pack_sizes[1] == 4, "two full groups of four, got %d launches", b.packs);
        EXPECT(rs[7]->r.is_completed() && rs[7]->ok() && !rs[8]->r.is_completed(), "ninth request still queued");
        rs[8]->r.urgent = true;
        m.execute();
        EXPECT(rs[8]->r.is_completed() && rs[8]->ok(), "ninth flushed when urgent");
        EXPECT(b.allocs <= 2, "fusion buffers are reused (allocs %d)", b.allocs);
    }
    {   // buffer full (fusion.cpp:426-431): 64-byte threshold x 4 = 256-byte buffer, 60-byte requests
        mock_backend b;
        ccl_fusion_config c2 = cfg; c2.bytes_threshold = 64; c2.count_threshold = 4;
        ccl_fusion_manager m(&b, doubling_allreduce, c2);
        std::vector<std::unique_ptr<req_t>> rs;
        for (int i = 0; i < 3; i++) { rs.emplace_back(new req_t(15, i)); m.add(&rs.back()->r); }     // 3 x 60 = 180 bytes
        m.execute();
        EXPECT(b.packs == 0, "180 of 256 bytes: keep gathering");
        for (int i = 3; i < 6; i++) { rs.emplace_back(new req_t(15, i)); m.add(&rs.back()->r); }
        m.execute();
        EXPECT(b.packs == 1 && b.pack_sizes[0] == 4, "fourth fills the count threshold (%zu)", b.pack_sizes.empty() ? (size_t)0 : b.pack_sizes[0]);
        req_t odd(10, 9); odd.r.count = 16;            // 64 bytes: not fusable at all
        EXPECT(!m.add(&odd.r), "64 bytes >= 64-byte threshold");
    }
    {   // requests of different dtypes never share a buffer; order inside a dtype is kept
        mock_backend b;
        ccl_fusion_manager m(&b, doubling_allreduce, cfg);
        std::vector<std::unique_ptr<req_t>> rs;
        for (int i = 0; i < 6; i++) { rs.emplace_back(new req_t(9, i, (i % 2) ? F32 : I32)); m.add(&rs.back()->r); }
        for (auto& r : rs) if (r->r.dtype.idx() == ccl::datatype::float32) for (size_t i = 0; i < r->send.size(); i++) { float f = (float)i + 0.5f; memcpy(&r->send[i], &f, 4); }
        rs[0]->r.urgent = true; rs[1]->r.urgent = true;
        m.execute(); m.execute();
        EXPECT(b.packs == 2 && b.pack_sizes[0] == 3 && b.pack_sizes[1] == 3, "one launch per dtype");
        bool ok = true;
        for (auto& r : rs) {
            ok = ok && r->r.is_completed();
            for (size_t i = 0; i < r->send.size(); i++) {
                if (r->r.dtype.idx() == ccl::datatype::float32) { float a, c; memcpy(&a, &r->send[i], 4); memcpy(&c, &r->recv[i], 4); ok = ok && c == 2 * a; }
                else ok = ok && r->recv[i] == 2 * r->send[i];
            }
        }
        EXPECT(ok, "values per dtype");
    }
    {   // the cycle: calls closer together than cycle_ms do nothing (fusion.cpp:379-385)
        mock_backend b;
        ccl_fusion_config c2 = cfg; c2.cycle_ms = 200.0;
        ccl_fusion_manager m(&b, doubling_allreduce, c2);
        req_t r(10, 1); r.r.urgent = true; m.add(&r.r);
        for (int i = 0; i < 100; i++) m.execute();
        EXPECT(m.stats().empty_exec_calls == 100 && b.packs == 0, "too early: %zu empty calls", m.stats().empty_exec_calls);
        std::this_thread::sleep_for(std::chrono::milliseconds(210));
        m.execute();
        EXPECT(b.packs == 1 && r.r.is_completed() && r.ok(), "flushed after the cycle elapsed");
    }
    {   // add() from several threads while one thread executes (fusion.hpp:49-50: the queues are lock-protected)
        mock_backend b;
        ccl_fusion_manager m(&b, doubling_allreduce, cfg);
        const int T = 4, PER = 500;
        std::vector<std::unique_ptr<req_t>> rs(T * PER);
        for (int i = 0; i < T * PER; i++) rs[i].reset(new req_t(1 + i % 50, i));
        std::atomic<int> done{ 0 };
        std::vector<std::thread> th;
        for (int t = 0; t < T; t++)
            th.emplace_back([&, t] { for (int i = 0; i < PER; i++) { rs[t * PER + i]->r.urgent = (i % 37 == 0); m.add(&rs[t * PER + i]->r); } done++; });
        while (done < T) m.execute();
        for (auto& x : th) x.join();
        for (auto& r : rs) r->r.urgent = true;
        for (int i = 0; i < 100; i++) m.execute();
        bool ok = true; for (auto& r : rs) ok = ok && r->r.is_completed() && r->ok();
        EXPECT(ok && m.stats().fused_ops == (size_t)(T * PER), "all %d requests from %d threads completed (fused %zu)", T * PER, T, m.stats().fused_ops);
    }
    {   // bad configuration throws like the reference's constructor checks (fusion.cpp:48-50)
        mock_backend b; bool threw = false;
        ccl_fusion_config c2 = cfg; c2.count_threshold = 0;
        try { ccl_fusion_manager m(&b, doubling_allreduce, c2); } catch (const ccl::exception&) { threw = true; }
        EXPECT(threw, "count_threshold 0");
    }
    printf("%d checks, %d failed\n", g_checks, g_fail);
    return g_fail ? 1 : 0;
}
