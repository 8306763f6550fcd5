"""Launch-context tests: the reduce captured in a HIP graph and replayed, and two large (phased) reduces
overlapping on two streams.  The phased kernel's grid barrier only aligns blocks in time, so neither replay nor
overlap may change a single bit."""
import numpy as np
import pytest

import oracle_lib as O
from gpu_util import to_dev, to_host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def comp():
    import torch
    assert torch.cuda.is_available()
    import oneccl_amd.comp as c
    c.lib()
    return c


@pytest.mark.parametrize("variant", [2, 8])
def test_graph_capture_and_replay(comp, variant):
    import torch
    rng = np.random.default_rng(variant)
    count, n = 3_000_017, 8
    srcs = [O.bf16_from_f32(rng.standard_normal(count).astype(np.float32)) for _ in range(n)]
    want = O.reduce_n(srcs, O.BFLOAT16, O.SUM, keep=1, threads=8)
    d = [to_dev(s) for s in srcs]
    out = torch.zeros_like(d[0])
    comp.set_param("variant", variant)
    try:
        comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, d, out, count, lp_mode=comp.LP_KEEP_PRECISION)   # warm up, eager
        torch.cuda.synchronize()
        assert (to_host(out, np.uint16) == want).all()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, d, out, count, lp_mode=comp.LP_KEEP_PRECISION)
        for rep in range(4):
            out.fill_(0)                     # eager work between the replays
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            assert (to_host(out, np.uint16) == want).all(), f"replay {rep}"
            # an eager launch between replays (it may land on the captured launch's set of barrier words)
            comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, d, out, count, lp_mode=comp.LP_KEEP_PRECISION)
            torch.cuda.synchronize()
            assert (to_host(out, np.uint16) == want).all()
    finally:
        comp.set_param("variant", 0)


def test_graph_of_the_paced_and_the_tiled_phased_kernels(comp):
    """The phased reduce with several destinations (its write phase is let out by the device clock) and the fused
    reduce against six peers (the tiled phased kernel, whose lanes describe the tiles of the next phase while the block
    waits at a barrier), forced on at a few MB, captured together and replayed four times with eager work in between."""
    import torch
    rng = np.random.default_rng(77)
    count, n, m = 2_000_003, 3, 3
    srcs = [O.bf16_from_f32(rng.standard_normal(count).astype(np.float32)) for _ in range(n)]
    want = O.reduce_n(srcs, O.BFLOAT16, O.SUM, keep=1, threads=8)
    d = [to_dev(s) for s in srcs]
    outs = [torch.zeros_like(d[0]) for _ in range(m)]
    counts = [700_001, 5, 1_200_000, 99_997]
    plan = comp.FusionPlan(counts, comp.BFLOAT16, 1)
    tens_h = [O.bf16_from_f32(rng.standard_normal(c).astype(np.float32)) for c in counts]
    peers_h = [O.bf16_from_f32(rng.standard_normal(plan.nbytes // 2).astype(np.float32)) for _ in range(6)]
    tens, peers = [to_dev(t) for t in tens_h], [to_dev(p_) for p_ in peers_h]
    res = [torch.zeros(c, dtype=tens[0].dtype, device="cuda") for c in counts]
    offs, _ = O.fusion_offsets(counts, 2, 1)
    want_res = [O.reduce_n([tens_h[t]] + [p_[offs[t] // 2:offs[t] // 2 + c] for p_ in peers_h], O.BFLOAT16, O.SUM, keep=1)
                for t, c in enumerate(counts)]

    def both():
        comp.comp_reduce_write_n(comp.BFLOAT16, comp.SUM, d, outs, count, lp_mode=comp.LP_KEEP_PRECISION)
        k1 = comp.last_kernel()
        plan.reduce(comp.SUM, tens, peers, res, lp_mode=comp.LP_KEEP_PRECISION)
        return k1, comp.last_kernel()

    def check(tag):
        torch.cuda.synchronize()
        for o_ in outs:
            assert (to_host(o_, np.uint16) == want).all(), tag
        for r_, w_ in zip(res, want_res):
            assert (to_host(r_, np.uint16) == w_).all(), tag

    comp.set_param("variant", 8)
    try:
        assert both() == ("reduce_multi_phased_kernel", "fusion_reduce_tiled_kernel")
        check("eager")
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            both()
        for rep in range(4):
            for t_ in outs + res:
                t_.fill_(0)
            torch.cuda.synchronize()
            g.replay()
            check(f"replay {rep}")
            both()                          # an eager pair between the replays
            check(f"eager after replay {rep}")
    finally:
        comp.set_param("variant", 0)
        plan.close()


def test_graph_of_copy_broadcast_converters_and_fused_reduce(comp):
    """A pipeline of the other kernels in one captured graph -- widen bf16 to fp32, copy, narrow back, broadcast to
    three buffers, fused reduce of two tensors against two peer fusion buffers -- replayed four times with eager work
    in between; every replay equals the eager result and the oracle."""
    import torch
    rng = np.random.default_rng(5)
    count = 1_000_003
    src = O.bf16_from_f32(rng.standard_normal(count).astype(np.float32))
    d_src = to_dev(src)
    f32 = torch.zeros(count, dtype=torch.int32, device="cuda")
    f32b = torch.zeros_like(f32)
    back = torch.zeros_like(d_src)
    outs = [torch.zeros_like(d_src) for _ in range(3)]
    counts = [400_001, count - 400_001]
    plan = comp.FusionPlan(counts, comp.BFLOAT16, 1)
    peers_h = [O.bf16_from_f32(rng.standard_normal(plan.nbytes // 2).astype(np.float32)) for _ in range(2)]
    peers = [to_dev(p_) for p_ in peers_h]
    res = [torch.zeros(c, dtype=d_src.dtype, device="cuda") for c in counts]

    def pipeline():
        comp.convert_bf16_to_fp32_arrays(d_src, f32, count)
        comp.comp_copy(f32, f32b, 4 * count, use_nontemporal=True)
        comp.convert_fp32_to_bf16_arrays(f32b, back, count)
        comp.comp_reduce_write_n(comp.BFLOAT16, comp.SUM, [back], outs, count)
        plan.reduce(comp.SUM, [outs[2][:counts[0]], outs[2][counts[0]:]], peers, res, lp_mode=comp.LP_KEEP_PRECISION)

    offs, _ = O.fusion_offsets(counts, 2, 1)
    want_res = []
    for t, c in enumerate(counts):
        lo = sum(counts[:t])
        o = offs[t] // 2
        want_res.append(O.reduce_n([src[lo:lo + c]] + [p_[o:o + c] for p_ in peers_h], O.BFLOAT16, O.SUM, keep=1))

    def check(tag):
        torch.cuda.synchronize()
        for o_ in outs:
            assert (to_host(o_, np.uint16) == src).all(), tag      # widening and narrowing back is exact
        for r_, w_ in zip(res, want_res):
            assert (to_host(r_, np.uint16) == w_).all(), tag

    pipeline()
    check("eager")
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        pipeline()
    for rep in range(4):
        for t_ in outs + res + [back]:
            t_.fill_(0)
        torch.cuda.synchronize()
        g.replay()
        check(f"replay {rep}")
    plan.close()


def test_two_phased_reduces_overlapping_on_two_streams(comp):
    import torch
    rng = np.random.default_rng(11)
    count, n = 40_000_003, 4              # 4 x 160 MB fp32 per reduce: several phases each
    a = [rng.standard_normal(count).astype(np.float32) for _ in range(n)]
    b = [rng.standard_normal(count).astype(np.float32) for _ in range(n)]
    want_a = O.reduce_n(a, O.FLOAT32, O.SUM, threads=16)
    want_b = O.reduce_n(b, O.FLOAT32, O.MAX, threads=16)
    da, db = [to_dev(x) for x in a], [to_dev(x) for x in b]
    oa, ob = torch.zeros_like(da[0]), torch.zeros_like(db[0])
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    comp.set_param("variant", 8)
    try:
        for _ in range(3):
            comp.comp_reduce_n(comp.FLOAT32, comp.SUM, da, oa, count, stream=s1)
            comp.comp_reduce_n(comp.FLOAT32, comp.MAX, db, ob, count, stream=s2)
        torch.cuda.synchronize()
    finally:
        comp.set_param("variant", 0)
    assert (to_host(oa, np.float32).view(np.uint32) == want_a.view(np.uint32)).all()
    assert (to_host(ob, np.float32).view(np.uint32) == want_b.view(np.uint32)).all()
    # and the barrier words are left consistent: a following launch runs at full speed and is exact
    comp.comp_reduce_n(comp.FLOAT32, comp.SUM, da, oa, count)
    torch.cuda.synchronize()
    assert (to_host(oa, np.float32).view(np.uint32) == want_a.view(np.uint32)).all()


@pytest.mark.parametrize("variant", [0, 8])
def test_worker_threads_on_disjoint_partitions(comp, variant):
    """What CCL_WORKER_COUNT = W does (parallelizer.cpp:230-241,374-379): W host threads, each with a stream of its
    own, reduce disjoint count/W partitions of the same buffers at the same time through the C ABI.  The result is
    the one-call result, bit for bit; variant 8 makes every partition a phased launch, each with its own set of
    barrier words while they overlap."""
    import threading
    import torch
    rng = np.random.default_rng(31 + variant)
    count, n, W = 8_000_011, 4, 4
    srcs = [O.bf16_from_f32(rng.standard_normal(count).astype(np.float32)) for _ in range(n)]
    want = O.reduce_n(srcs, O.BFLOAT16, O.SUM, keep=1, threads=8)
    d = [to_dev(s) for s in srcs]
    out = torch.zeros_like(d[0])
    streams = [torch.cuda.Stream() for _ in range(W)]
    part = count // W
    errors = []

    def worker(w):
        try:
            lo, hi = part * w, (count if w == W - 1 else part * (w + 1))     # the last takes the remainder
            for rep in range(5):
                comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, [t[lo:hi] for t in d], out[lo:hi], hi - lo,
                                   lp_mode=comp.LP_KEEP_PRECISION, stream=streams[w])
            streams[w].synchronize()
        except Exception as e:      # noqa: BLE001 - reported by the main thread
            errors.append(e)

    torch.cuda.synchronize()
    comp.set_param("variant", variant)
    try:
        threads = [threading.Thread(target=worker, args=(w,)) for w in range(W)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
    finally:
        comp.set_param("variant", 0)
    torch.cuda.synchronize()
    assert not errors, errors
    assert (to_host(out, np.uint16) == want).all()


def test_graph_of_batched_reduce_and_allocation_free_fused_reduce(comp):
    """The two entry points meant for callers that hold a graph: mi_ccl_comp_reduce_batch (its job table travels in the
    kernel arguments) and mi_ccl_fusion_reduce_static (its table is rebuilt by a kernel in front of the reduce, no
    allocation, no memset) captured together, replayed four times with eager calls of the same entry points -- which
    share the static table -- in between; every replay equals the oracle."""
    import torch
    rng = np.random.default_rng(11)
    counts = [70_001, 1, 4096, 300_000, 33]
    np_t = np.float32
    jobs_h = [[rng.uniform(-2, 2, c).astype(np_t) for _ in range(3)] for c in counts]
    jobs_d = [[to_dev(x) for x in j] for j in jobs_h]
    jobs_o = [torch.zeros(c, dtype=torch.float32, device="cuda") for c in counts]
    table = comp.BatchJobs([(s, o, c) for s, o, c in zip(jobs_d, jobs_o, counts)])
    want_jobs = [O.reduce_n(j, O.FLOAT32, O.MAX) for j in jobs_h]
    offs, total = O.fusion_offsets(counts, 4, 64)
    nelem = total // 4
    peers_h = [rng.uniform(-2, 2, nelem).astype(np_t) for _ in range(3)]
    peers_d = [to_dev(p_) for p_ in peers_h]
    fused_o = [torch.zeros(c, dtype=torch.float32, device="cuda") for c in counts]
    want_fused = []
    for i, c in enumerate(counts):
        o = int(offs[i]) // 4
        want_fused.append(O.reduce_n([jobs_h[i][0]] + [p_[o:o + c] for p_ in peers_h], O.FLOAT32, O.SUM))
    own = [j[0] for j in jobs_d]

    def both():
        table.reduce(comp.FLOAT32, comp.MAX)
        comp.fusion_reduce_static(counts, comp.FLOAT32, 64, comp.SUM, own, peers_d, fused_o)

    def check(what):
        torch.cuda.synchronize()
        for i in range(len(counts)):
            assert (to_host(jobs_o[i], np.uint32) == want_jobs[i].view(np.uint32)).all(), f"{what}: job {i}"
            assert (to_host(fused_o[i], np.uint32) == want_fused[i].view(np.uint32)).all(), f"{what}: fused tensor {i}"

    both()                                  # eager first: the first call on a device looks the static table up
    check("eager")
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        both()
    other_counts = [5, 100_000]             # an eager call with another layout overwrites the shared table
    other = [to_dev(rng.uniform(-1, 1, c).astype(np_t)) for c in other_counts]
    other_o = [torch.zeros_like(t) for t in other]
    for rep in range(4):
        for t in jobs_o + fused_o:
            t.zero_()
        comp.fusion_reduce_static(other_counts, comp.FLOAT32, 4, comp.SUM, other, [], other_o)
        torch.cuda.synchronize()
        g.replay()
        check(f"replay {rep}")


def test_two_threads_with_different_fp16_implementations(comp):
    """The float16 implementation travels with the call: two host threads, one reducing under avx512f (a signalling
    NaN that min hands back is quieted) and one under avx512fp16 (it stays as it is), each on its own stream, never
    see the other's setting, and the process-wide default is left alone."""
    import threading
    import torch
    snan, one = np.uint16(0x7D01), np.uint16(0x3C00)
    count = 10_007
    a = np.full(count, one, np.uint16)          # in
    b = np.full(count, snan, np.uint16)         # inout: min(in = 1, inout = sNaN) hands inout back
    want = {3: O.comp_reduce(a, b, O.FLOAT16, O.MIN, fp16_impl=3), 4: O.comp_reduce(a, b, O.FLOAT16, O.MIN, fp16_impl=4)}
    assert want[3][0] == 0x7F01 and want[4][0] == 0x7D01
    errors = []

    def worker(impl):
        try:
            stream = torch.cuda.Stream()
            da = to_dev(a)
            for rep in range(200):
                db = to_dev(b)
                comp.comp_reduce(comp.FLOAT16, comp.MIN, da, count, db, fp16_impl=impl, stream=stream)
                stream.synchronize()
                got = to_host(db, np.uint16)
                if not (got == want[impl]).all():
                    errors.append((impl, rep, hex(int(got[0]))))
                    return
        except Exception as e:      # noqa: BLE001
            errors.append((impl, repr(e)))

    default_before = comp.get_param("fp16_impl")
    threads = [threading.Thread(target=worker, args=(impl,)) for impl in (3, 4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert comp.get_param("fp16_impl") == default_before
