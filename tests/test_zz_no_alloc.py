"""mi_ccl_fusion_reduce_static, the fused reduce that allocates nothing (its work table lives in an array inside the
library): called through the C ABI, its output must equal, bit for bit, that of mi_ccl_fusion_reduce on a plan of
the same layout -- on two calls in a row, the second with a smaller input, so that what the first call left in the
shared table cannot leak into the second.  Also: the limits are refused with out_of_resource, and once the first
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
    """First a larger group (more than one launch group of 192 tensors, odd sizes, an empty tensor), then a smaller
    one with another layout, dtype and peer count; variant 8 forces the phased kernels."""
    rng = np.random.default_rng(2026)
    _case(comp, rng, [3, 70_000], O.INT32, O.SUM, 1, 4, comp.LP_PAIRWISE, variant, check_memory=False)   # first use on this device
    big = [int(c) for c in np.exp(rng.uniform(np.log(3), np.log(300_000), 230))]
    big[7] = 0
    big[100] = 16384 * 3
    _case(comp, rng, big, O.BFLOAT16, O.SUM, 7, 256, comp.LP_KEEP_PRECISION, variant)
    small = [1, 4097, 0, 8192, 33, 70_001]
    _case(comp, rng, small, O.FLOAT32, O.MAX, 2, 1, comp.LP_PAIRWISE, variant)
    _case(comp, rng, [5], O.INT8, O.PROD, 0, 1, comp.LP_PAIRWISE, variant)


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
