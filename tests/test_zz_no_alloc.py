"""mi_ccl_fusion_reduce_static, the fused reduce that allocates nothing (its work table lives in an array inside the
library): called through the C ABI, its output must equal, bit for bit, that of mi_ccl_fusion_reduce on a plan of
the same layout -- on two calls in a row, the second with a smaller input, and on a run of calls long enough that a
table which held a larger layout is used again, so that what an earlier call left in a table cannot leak into a later one.  Also: the limits are refused with out_of_resource, and once the first
call on the device has looked the table's address up, a call makes no device allocation (the free-memory figure of
the device does not move)."""
import numpy as np
import pytest

import oracle_lib as O
from gpu_util import make_inputs, to_dev, to_host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def comp():
    import torch
    assert torch.cuda.is_available(), "needs a GPU"
    import oneccl_amd.comp as c
    c.lib()
    return c


def _case(comp, rng, counts, dtype, op, n_peers, align, lp, variant, check_memory=True):
    """Runs the plan entry point and the static one on the same inputs; returns nothing, asserts equality."""
    import torch
    np_t = O.NP_STORAGE[dtype]
    esz = O.DTYPE_SIZE[dtype]
    offs, total = O.fusion_offsets(counts, esz, align)
    nelem = (total + esz - 1) // esz + 8
    tensors = [make_inputs(rng, dtype, c, op, 1)[0] if c else np.zeros(0, np_t) for c in counts]
    peers = [make_inputs(rng, dtype, nelem, op, 1)[0] for _ in range(n_peers)]
    d_t = [to_dev(t if t.size else np.zeros(1, np_t)) for t in tensors]
    d_p = [to_dev(p) for p in peers]
    plan = comp.FusionPlan(counts, dtype, align)
    comp.set_param("variant", variant)
    try:
        want = [to_dev(np.zeros(c + 5, np_t)) for c in counts]
        plan.reduce(op, d_t, d_p, want, lp_mode=lp)
        torch.cuda.synchronize()
        free0, _ = torch.cuda.mem_get_info()
        got = [to_dev(np.zeros(c + 5, np_t)) for c in counts]
        torch.cuda.synchronize()
        free1, _ = torch.cuda.mem_get_info()
        comp.fusion_reduce_static(counts, dtype, align, op, d_t, d_p, got, lp_mode=lp)
        torch.cuda.synchronize()
        free2, _ = torch.cuda.mem_get_info()
    finally:
        comp.set_param("variant", 0)
        plan.close()
    assert not check_memory or free2 == free1, f"the call changed the device's free memory by {free1 - free2} bytes"
    for i, c in enumerate(counts):
        g, w = to_host(got[i], np_t), to_host(want[i], np_t)
        assert (g.view(np.uint8) == w.view(np.uint8)).all(), f"tensor {i} of {c} elements differs from the plan entry point"
        assert not g[c:].view(np.uint8).any(), f"tensor {i}: wrote past the end"
    # and against the oracle, tensor by tensor
    keep = 1 if lp == comp.LP_KEEP_PRECISION else 0
    for i, c in enumerate(counts):
        if not c:
            continue
        o = int(offs[i]) // esz
        w = O.reduce_n([tensors[i]] + [p[o:o + c] for p in peers], dtype, op, keep=keep)
        assert (to_host(got[i], np_t)[:c].view(np.uint8) == w.view(np.uint8)).all(), f"tensor {i} differs from the oracle"


@pytest.mark.parametrize("variant", [0, 8])
def test_static_entry_point_equals_plan_entry_point_twice_in_a_row(comp, variant):
    """First a larger group (more than one launch group of 256 tensors, odd sizes, an empty tensor), then a smaller
    one with another layout, dtype and peer count; variant 8 forces the phased kernels."""
    rng = np.random.default_rng(2026)
    _case(comp, rng, [3, 70_000], O.INT32, O.SUM, 1, 4, comp.LP_PAIRWISE, variant, check_memory=False)   # first use on this device
    big = [int(c) for c in np.exp(rng.uniform(np.log(3), np.log(300_000), 300))]
    big[7] = 0
    big[100] = 16384 * 3
    _case(comp, rng, big, O.BFLOAT16, O.SUM, 7, 256, comp.LP_KEEP_PRECISION, variant)
    small = [1, 4097, 0, 8192, 33, 70_001]
    _case(comp, rng, small, O.FLOAT32, O.MAX, 2, 1, comp.LP_PAIRWISE, variant)
    _case(comp, rng, [5], O.INT8, O.PROD, 0, 1, comp.LP_PAIRWISE, variant)


def test_static_entry_point_reuses_a_table_that_held_a_larger_layout(comp):
    """The library keeps four tables per GPU and hands them out in turn, so the fifth call gets the table of the first:
    a large layout first, then smaller ones until every table has come round again."""
    rng = np.random.default_rng(77)
    big = [int(c) for c in np.exp(rng.uniform(np.log(3), np.log(200_000), 200))]
    _case(comp, rng, big, O.BFLOAT16, O.SUM, 3, 1, comp.LP_KEEP_PRECISION, 0)
    for r in range(5):
        _case(comp, rng, [17 + r, 4099, 2], O.INT16, O.MIN, 2, 2, comp.LP_PAIRWISE, 0)


def test_static_entry_point_calls_that_overlap_on_two_streams(comp):
    """Two calls with different layouts issued back to back on two streams (they may run side by side): each has a
    table of its own, so each must equal the plan entry point's result on the same inputs."""
    import torch
    rng = np.random.default_rng(78)
    cases = []
    for counts, dtype, n_peers in (([300_001, 5, 1_000_003], O.FLOAT32, 3), ([777, 2_000_001], O.INT32, 2)):
        np_t, esz = O.NP_STORAGE[dtype], O.DTYPE_SIZE[dtype]
        _, total = O.fusion_offsets(counts, esz, 4)
        tens = [to_dev(make_inputs(rng, dtype, c, O.SUM, 1)[0]) for c in counts]
        peers = [to_dev(make_inputs(rng, dtype, total // esz + 8, O.SUM, 1)[0]) for _ in range(n_peers)]
        plan = comp.FusionPlan(counts, dtype, 4)
        want = [torch.zeros_like(t) for t in tens]
        plan.reduce(comp.SUM, tens, peers, want)
        plan.close()
        cases.append((counts, dtype, tens, peers, want, [torch.zeros_like(t) for t in tens]))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for rep in range(3):
        for (counts, dtype, tens, peers, want, got), st in zip(cases, streams):
            comp.fusion_reduce_static(counts, dtype, 4, comp.SUM, tens, peers, got, stream=st)
    torch.cuda.synchronize()
    for counts, dtype, tens, peers, want, got in cases:
        for g, w in zip(got, want):
            assert torch.equal(g, w)


def test_static_entry_point_limits_and_errors(comp):
    import torch
    one = to_dev(np.zeros(16, np.float32))
    k = comp.FUSION_STATIC_MAX_TENSORS + 1
    with pytest.raises(comp.CclError) as e:
        comp.fusion_reduce_static([1] * k, comp.FLOAT32, 4, comp.SUM, [one] * k, [], [one] * k)
    assert e.value.status == comp.OUT_OF_RESOURCE
    too_many = (comp.FUSION_STATIC_MAX_ITEMS + 1) * 16384 // 4        # one tensor with one item too many
    with pytest.raises(comp.CclError) as e:
        comp.fusion_reduce_static([too_many], comp.FLOAT32, 4, comp.SUM, [one], [], [one])
    assert e.value.status == comp.OUT_OF_RESOURCE
    with pytest.raises(comp.CclError) as e:
        comp.fusion_reduce_static([16], comp.FLOAT32, 3, comp.SUM, [one], [], [one])       # alignment not a power of two
    assert e.value.status == comp.INVALID_ARGUMENTS
    with pytest.raises(comp.CclError) as e:
        comp.fusion_reduce_static([16], comp.FLOAT32, 4, comp.SUM, [0], [], [one])         # null tensor
    assert e.value.status == comp.INVALID_ARGUMENTS
    comp.fusion_reduce_static([0, 0], comp.FLOAT32, 4, comp.SUM, [0, 0], [], [0, 0])        # nothing to do
    torch.cuda.synchronize()
    assert not to_host(one, np.float32).any()
