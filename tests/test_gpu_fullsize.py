"""The benchmark's full-size configurations, bit for bit: 8 x 1,003,782,144 bf16 (fp32 accumulate, RNE once) and
4 x 1,003,782,144 fp32, compared over every element with the 16-thread oracle, plus size-independent properties
(reduce with zeros is the identity on finite values, x + (-x) = +0, in-place equals out-of-place); the 2-input in-place
fp32 sum at 16,777,216 elements, the 8-input bf16 sum at 33,554,432, and the fusion configuration at its full counts
(256 bf16 tensors, log-uniform over [2,048, 2,097,152], 256-byte aligned offsets, seven peer fusion buffers) through
pack + reduce + unpack and through the fused single pass; and the datatype x op sweep's six (type, operation) pairs with
four inputs at 16 MiB, 64 MiB and 1 GiB per buffer, by the automatic kernel choice, every element."""
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


def test_c1_fp32_two_inputs_in_place_16M(comp):
    """2-input in-place sum, fp32, 16,777,216 elements per buffer, i.i.d. uniform[-1, 1): ccl_comp_reduce's shape."""
    import torch
    n = 16_777_216
    rng = np.random.default_rng(101)
    a = rng.uniform(-1, 1, n).astype(np.float32)
    b = rng.uniform(-1, 1, n).astype(np.float32)
    want = O.comp_reduce(a, b, O.FLOAT32, O.SUM)
    assert (want.view(np.uint32) == (b + a).view(np.uint32)).all()        # one IEEE add per pair (numpy's is one too)
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    comp.comp_reduce(comp.FLOAT32, comp.SUM, da, n, db)
    torch.cuda.synchronize()
    assert comp.last_kernel() == "reduce_vec_kernel"
    assert (db.cpu().numpy().view(np.uint32) == want.view(np.uint32)).all()
    assert torch.equal(da.cpu(), torch.from_numpy(a)), "the in buffer changed"


def test_c2_bf16_eight_inputs_32M(comp):
    """8-input bf16 sum, 33,554,432 elements per buffer, N(0, 1) cast with RNE, fp32 accumulation in input order, one
    RNE narrowing: every element against the oracle, by the default kernel choice and by the streaming kernel."""
    import torch
    n = 33_554_432
    rng = np.random.default_rng(102)
    host = [O.bf16_from_f32(rng.standard_normal(n).astype(np.float32)) for _ in range(8)]
    want = O.reduce_n(host, O.BFLOAT16, O.SUM, keep=1, threads=16)
    dev = [torch.from_numpy(h.view(np.int16)).cuda() for h in host]
    for variant in (0, 4):
        comp.set_param("variant", variant)
        try:
            out = torch.zeros_like(dev[0])
            comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, dev, out, n, lp_mode=comp.LP_KEEP_PRECISION)
            torch.cuda.synchronize()
        finally:
            comp.set_param("variant", 0)
        got = out.cpu().numpy().view(np.uint16)
        assert (got == want).all(), f"variant {variant}: {np.count_nonzero(got != want)} elements differ"


def test_c4_fusion_256_tensors_full_counts(comp):
    """The fusion configuration at its real sizes: pack -> 8-input sum over the fusion buffer -> unpack, and the
    fused single pass in both kernel forms, every tensor against the oracle's pack / reduce / unpack."""
    import math
    import torch
    rng = np.random.default_rng(4)
    counts = [int(round(math.exp(rng.uniform(math.log(2048), math.log(2_097_152))))) for _ in range(256)]
    assert min(counts) >= 2048 and max(counts) <= 2_097_152 and sum(counts) > 50_000_000
    tensors = [O.bf16_from_f32((rng.standard_normal(c) * 0.02).astype(np.float32)) for c in counts]
    offs, total = O.fusion_offsets(counts, 2, 256)
    assert all(int(o) % 256 == 0 for o in offs)
    nelem = total // 2
    peers = [O.bf16_from_f32((rng.standard_normal(nelem) * 0.02).astype(np.float32)) for _ in range(7)]
    fb = O.fusion_pack(tensors, offs, total, 2)
    fused = O.reduce_n([fb.view(np.uint16)] + peers, O.BFLOAT16, O.SUM, keep=1, threads=16)
    want = O.fusion_unpack(fused.view(np.uint8), counts, offs, np.uint16)
    plan = comp.FusionPlan(counts, comp.BFLOAT16, 256)
    assert plan.nbytes == total and [plan.offset(i) for i in (0, 1, 255)] == [int(offs[i]) for i in (0, 1, 255)]
    d_t = [torch.from_numpy(t.view(np.int16)).cuda() for t in tensors]
    d_p = [torch.from_numpy(p.view(np.int16)).cuda() for p in peers]
    # three steps
    d_fb = torch.zeros(nelem, dtype=torch.int16, device="cuda")
    plan.pack(d_t, d_fb)
    comp.comp_reduce_n(comp.BFLOAT16, comp.SUM, [d_fb] + d_p, d_fb, nelem, lp_mode=comp.LP_KEEP_PRECISION)
    outs = [torch.zeros_like(t) for t in d_t]
    plan.unpack(d_fb, outs)
    torch.cuda.synchronize()
    for i in range(256):
        assert (outs[i].cpu().numpy().view(np.uint16) == want[i]).all(), f"pack/reduce/unpack: tensor {i} of {counts[i]} elements"
    # fused single pass: the default choice at this size (phased) and the streaming kernel
    for variant, kernel in ((0, "fusion_reduce_tiled_kernel"), (2, "fusion_reduce_kernel")):
        comp.set_param("variant", variant)
        try:
            outs = [torch.zeros_like(t) for t in d_t]
            plan.reduce(comp.SUM, d_t, d_p, outs, lp_mode=comp.LP_KEEP_PRECISION)
            torch.cuda.synchronize()
            assert comp.last_kernel() == kernel
        finally:
            comp.set_param("variant", 0)
        for i in range(256):
            assert (outs[i].cpu().numpy().view(np.uint16) == want[i]).all(), f"fused ({kernel}): tensor {i}"
    # and without a plan
    outs = [torch.zeros_like(t) for t in d_t]
    comp.fusion_reduce_static(counts, comp.BFLOAT16, 256, comp.SUM, d_t, d_p, outs, lp_mode=comp.LP_KEEP_PRECISION)
    torch.cuda.synchronize()
    for i in range(256):
        assert (outs[i].cpu().numpy().view(np.uint16) == want[i]).all(), f"fused, static table: tensor {i}"
    plan.close()



C3_CASES = [("int8", "SUM"), ("int32", "SUM"), ("int64", "MAX"), ("float16", "SUM"), ("float32", "MIN"), ("float64", "PROD")]


@pytest.mark.parametrize("tname,opname", C3_CASES)
def test_c3_four_inputs_16MiB_64MiB_1GiB_automatic_kernel_every_element(comp, tname, opname):
    """The sweep's (type, operation) pairs at its three largest sizes, kernel form chosen by the library (variant 0):
    the streaming kernel at 16 MiB per buffer, the phased kernel at 64 MiB and 1 GiB.  Integers uniform over the full
    range of the type, floats uniform[-2, 2] (product: uniform[0.9, 1.1]), float16 by a round-to-nearest-even cast;
    every element against the 16-thread oracle."""
    import torch
    tdt = getattr(torch, tname)
    dt = {"int8": O.INT8, "int32": O.INT32, "int64": O.INT64, "float16": O.FLOAT16, "float32": O.FLOAT32, "float64": O.FLOAT64}[tname]
    op = getattr(O, opname)
    esz = O.DTYPE_SIZE[dt]
    np_t = O.NP_STORAGE[dt]
    view = {1: torch.int8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[esz]
    g = torch.Generator(device="cuda")
    g.manual_seed(3000 + dt)
    assert comp.get_param("variant") == 0
    for size, kernel in ((16 << 20, "reduce_vec_kernel"), (64 << 20, "reduce_multi_phased_kernel"), (1 << 30, "reduce_multi_phased_kernel")):
        count = size // esz
        if tdt.is_floating_point:
            lo, hi = (0.9, 1.1) if op == O.PROD else (-2.0, 2.0)
            srcs = [torch.empty(count, dtype=torch.float32 if esz <= 4 else torch.float64, device="cuda").uniform_(lo, hi, generator=g).to(tdt)
                    for _ in range(4)]
        else:
            info = torch.iinfo(tdt)
            srcs = [torch.randint(info.min, info.max, (count,), dtype=tdt, device="cuda", generator=g) for _ in range(4)]
        out = torch.zeros(count, dtype=tdt, device="cuda")
        comp.comp_reduce_n(dt, op, srcs, out, count)
        torch.cuda.synchronize()
        assert comp.last_kernel() == kernel, (size, comp.last_kernel())
        host = [s_.view(view).cpu().numpy().view(np_t) for s_ in srcs]
        want = O.reduce_n(host, dt, op, threads=16)
        got = out.view(view).cpu().numpy()
        u = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[esz]
        bad = got.view(u) != want.view(u)
        assert not bad.any(), f"{tname} {opname} at {size >> 20} MiB: {np.count_nonzero(bad)} elements differ, first at {np.flatnonzero(bad)[:5]}"
        del host, want, got, srcs, out
