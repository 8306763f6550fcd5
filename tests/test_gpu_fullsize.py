"""The benchmark's full-size configurations, bit for bit: 8 x 1,003,782,144 bf16 (fp32 accumulate, RNE once) and
4 x 1,003,782,144 fp32, compared over every element with the 16-thread oracle, plus size-independent properties
(reduce with zeros is the identity on finite values, x + (-x) = +0, in-place equals out-of-place)."""
import numpy as np
import pytest

import oracle_lib as O

pytestmark = pytest.mark.gpu
COUNT = 1_003_782_144


@pytest.fixture(scope="module")
def comp():
    import torch
    assert torch.cuda.is_available()
    import oneccl_amd.comp as c
    c.lib()
    return c


def _host(t, np_t):
    import torch
    v = t.view(torch.int16) if t.dtype == torch.bfloat16 else t
    return v.cpu().numpy().view(np_t)


def test_c5_bf16_8x2GiB_every_element(comp):
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    bufs = [torch.empty(COUNT, dtype=torch.bfloat16, device="cuda").normal_(0, 1e-3, generator=g) for _ in range(8)]
    out = torch.empty_like(bufs[0])
    comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, bufs, out, COUNT, lp_mode=comp.LP_KEEP_PRECISION)
    torch.cuda.synchronize()
    host = [_host(b, np.uint16) for b in bufs]
    want = O.reduce_n(host, O.BFLOAT16, O.SUM, keep=1, threads=16)
    got = _host(out, np.uint16)
    assert (got == want).all(), f"{np.count_nonzero(got != want)} elements differ, first at {np.flatnonzero(got != want)[:5]}"
    del host
    # the streaming kernel gives the same bits as the phased one
    comp.set_param("variant", 2)
    try:
        out2 = torch.empty_like(out)
        comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, bufs, out2, COUNT, lp_mode=comp.LP_KEEP_PRECISION)
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), out2.view(torch.int16))
    finally:
        comp.set_param("variant", 0)
    # reduce with seven zero buffers: identity on finite normal values (N(0,1e-3) has no denormals/NaNs)
    zero = torch.zeros(COUNT, dtype=torch.bfloat16, device="cuda")
    comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, [bufs[3]] + [zero] * 7, out2, COUNT, lp_mode=comp.LP_KEEP_PRECISION)
    torch.cuda.synchronize()
    assert torch.equal(out2.view(torch.int16), bufs[3].view(torch.int16))
    # x + (-x) = +0 everywhere
    neg = (bufs[3].view(torch.int16) ^ torch.tensor(-32768, dtype=torch.int16, device="cuda")).view(torch.bfloat16)
    comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, [bufs[3], neg], out2, COUNT, lp_mode=comp.LP_KEEP_PRECISION)
    torch.cuda.synchronize()
    assert int(out2.view(torch.int16).count_nonzero()) == 0
    # in place on the own buffer (what ccl_comp_batch_reduce does: inout is slice 0)
    comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, bufs, bufs[0], COUNT, lp_mode=comp.LP_KEEP_PRECISION)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), bufs[0].view(torch.int16))


def test_c5_fp32_4x4GiB_every_element(comp):
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(6)
    bufs = [torch.empty(COUNT, dtype=torch.float32, device="cuda").normal_(0, 1e-3, generator=g) for _ in range(4)]
    out = torch.empty_like(bufs[0])
    comp.comp_reduce_n(comp.FLOAT32, comp.SUM, bufs, out, COUNT)
    torch.cuda.synchronize()
    host = [_host(b, np.float32) for b in bufs]
    want = O.reduce_n(host, O.FLOAT32, O.SUM, threads=16)
    got = _host(out, np.float32)
    assert (got.view(np.uint32) == want.view(np.uint32)).all()
    # one IEEE add per pair in input order: same as torch's fp32 adds chained left to right
    ref = ((bufs[0] + bufs[1]) + bufs[2]) + bufs[3]
    assert torch.equal(ref.view(torch.int32), out.view(torch.int32))


@pytest.mark.parametrize("variant", [0, 2])
def test_more_than_2_pow_32_elements(comp, variant):
    """Counts beyond 32 bits (the reference's vector loops stop at 2^31, its scalar loops do not): int8 sum and max
    over 2^32 + 4,099 elements with buffers that start 3 bytes off a 16-byte boundary, in place, through the phased
    (variant 0 at this size) and the streaming kernel; then the same buffers through the copy and the two-destination
    entry points.  Checked against torch's own wrapping int8 arithmetic over every element."""
    import torch
    count = (1 << 32) + 4099
    g = torch.Generator(device="cuda")
    g.manual_seed(17)
    big = [torch.randint(-128, 128, (count + 3,), dtype=torch.int8, device="cuda", generator=g) for _ in range(2)]
    a, b = big[0][3:], big[1][3:]
    head_before = big[0][:3].clone()
    want_sum = a + b                     # int8 addition wraps in torch as in the reference
    want_max = torch.maximum(a, b)
    comp.set_param("variant", variant)
    try:
        out = torch.empty(count + 3, dtype=torch.int8, device="cuda")[3:]
        comp.comp_reduce_n(comp.INT8, comp.MAX, [a, b], out, count)
        torch.cuda.synchronize()
        assert torch.equal(out, want_max)
        del want_max
        o1 = torch.zeros(count + 3, dtype=torch.int8, device="cuda")
        comp.comp_reduce_write_n(comp.INT8, comp.SUM, [a, b], [out, o1[3:]], count)
        torch.cuda.synchronize()
        assert torch.equal(out, want_sum) and torch.equal(o1[3:], want_sum) and int(o1[:3].count_nonzero()) == 0
        del o1
        comp.comp_copy(a, out, count, use_nontemporal=True)
        torch.cuda.synchronize()
        assert torch.equal(out, a)
        comp.comp_reduce(comp.INT8, comp.SUM, b, count, a)      # in place: a += b
        torch.cuda.synchronize()
        assert torch.equal(a, want_sum)
        assert torch.equal(big[0][:3], head_before)             # the bytes in front of the buffer are untouched
    finally:
        comp.set_param("variant", 0)
