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
            # an eager launch between replays shares the barrier words with the captured one
            comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, d, out, count, lp_mode=comp.LP_KEEP_PRECISION)
            torch.cuda.synchronize()
            assert (to_host(out, np.uint16) == want).all()
    finally:
        comp.set_param("variant", 0)


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
    the one-call result, bit for bit; variant 8 makes every partition a phased launch, so the launches share the
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
