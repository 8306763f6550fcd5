"""GPU parity of the fusion-buffer path: pack / N-input reduce / unpack and the fused single-pass form,
against the oracle's pack -> reduce -> unpack (layout of src/fusion/fusion.cpp:283-362)."""
import numpy as np
import pytest

import oracle_lib as O
from gpu_util import assert_same, make_inputs, to_dev, to_host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def comp():
    import torch
    assert torch.cuda.is_available()
    import oneccl_amd.comp as c
    c.lib()
    return c


def log_uniform_counts(rng, k, lo, hi):
    return [int(round(np.exp(rng.uniform(np.log(lo), np.log(hi))))) for _ in range(k)]


def test_fusion_offsets_match_oracle(comp):
    rng = np.random.default_rng(0)
    counts = log_uniform_counts(rng, 300, 1, 100000)
    for align in (1, 2, 16, 256):
        for esz in (1, 2, 4, 8):
            offs, total = comp.fusion_offsets(counts, esz, align)
            o2, t2 = O.fusion_offsets(counts, esz, align)
            assert offs == [int(x) for x in o2] and total == t2
    assert comp.lib().mi_ccl_fusion_offsets(None, 0, 2, 3, None, None) == comp.INVALID_ARGUMENTS


@pytest.mark.parametrize("align", [1, 256])
@pytest.mark.parametrize("dtype", [O.BFLOAT16, O.FLOAT32, O.INT8])
def test_pack_reduce_unpack_and_fused(comp, align, dtype):
    import torch
    rng = np.random.default_rng(42 + align + dtype)
    k = 300                       # more than one launch group of tensors (256 per launch)
    counts = log_uniform_counts(rng, k, 1, 40000)
    counts[5] = 0 if align == 256 else 1
    np_t = O.NP_STORAGE[dtype]
    esz = O.DTYPE_SIZE[dtype]
    n_peers = 3
    tensors = [make_inputs(rng, dtype, c, O.SUM, 1)[0] if c else np.zeros(0, np_t) for c in counts]
    plan = comp.FusionPlan(counts, dtype, align)
    offs, total = O.fusion_offsets(counts, esz, align)
    assert plan.nbytes == total and [plan.offset(i) for i in range(k)] == [int(x) for x in offs]
    nelem = (total + esz - 1) // esz
    peers = [make_inputs(rng, dtype, nelem, O.SUM, 1)[0] for _ in range(n_peers)]
    lp = comp.LP_KEEP_PRECISION if dtype == O.BFLOAT16 else comp.LP_PAIRWISE
    keep = 1 if dtype == O.BFLOAT16 else 0

    # oracle: pack -> N-input reduce over the fused buffer -> unpack
    fb = O.fusion_pack(tensors, offs, nelem * esz, esz)
    fused = O.reduce_n([fb.view(np_t)] + peers, dtype, O.SUM, keep=keep)
    want = O.fusion_unpack(fused.view(np.uint8), counts, offs, np_t)

    # GPU, three steps.  Some tensors sit at odd element offsets inside a larger allocation.
    holders, d_t = [], []
    for i, t in enumerate(tensors):
        sh = (i % 3) if align == 1 else 0
        h = to_dev(np.concatenate([np.zeros(sh, np_t), t, np.zeros(8, np_t)]))
        holders.append(h)
        d_t.append(h.data_ptr() + sh * esz)
    d_fb = to_dev(np.full(nelem, 0, np_t))
    plan.pack(d_t, d_fb)
    torch.cuda.synchronize()
    got_fb = to_host(d_fb, np_t).view(np.uint8)
    for i, c in enumerate(counts):      # payload bytes only; padding is not written
        o = int(offs[i])
        assert (got_fb[o:o + c * esz] == fb[o:o + c * esz]).all(), f"pack tensor {i}"
    d_peers = [to_dev(p) for p in peers]
    comp.comp_reduce_n(dtype, O.SUM, [d_fb] + d_peers, d_fb, nelem, lp_mode=lp)
    outs = [to_dev(np.zeros(c + 4, np_t)) for c in counts]
    plan.unpack(d_fb, outs)
    torch.cuda.synchronize()
    for i, c in enumerate(counts):
        g = to_host(outs[i], np_t)
        assert_same(g[:c], want[i], dtype, f"3-step tensor {i}")
        assert (g[c:] == 0).all(), "unpack wrote past the tensor"
    # unpack into tensors that start at odd element offsets inside larger allocations (the copy is cut where the
    # destination crosses cache lines, which then differs from tensor to tensor): nothing outside the tensor is written
    holders_u, d_u = [], []
    for i, c in enumerate(counts):
        sh = i % 5
        h = to_dev(np.zeros(sh + c + 8, np_t))
        holders_u.append(h)
        d_u.append(h.data_ptr() + sh * esz)
    plan.unpack(d_fb, d_u)
    torch.cuda.synchronize()
    for i, c in enumerate(counts):
        sh = i % 5
        g = to_host(holders_u[i], np_t)
        assert_same(g[sh:sh + c], want[i], dtype, f"unpack to shifted tensor {i}")
        assert (g[:sh] == 0).all() and (g[sh + c:] == 0).all(), "unpack wrote outside the shifted tensor"
    # ... and pack once more into a fusion buffer that itself starts 3 elements into its allocation
    d_fb2 = to_dev(np.zeros(nelem + 3 + 8, np_t))
    plan.pack(d_t, d_fb2.data_ptr() + 3 * esz)
    torch.cuda.synchronize()
    got2 = to_host(d_fb2, np_t)
    assert (got2[:3] == 0).all() and (got2[3 + nelem:] == 0).all(), "pack wrote outside the fusion buffer"
    got2 = got2[3:3 + nelem].view(np.uint8)
    for i, c in enumerate(counts):
        o = int(offs[i])
        assert (got2[o:o + c * esz] == fb[o:o + c * esz]).all(), f"pack into a shifted buffer, tensor {i}"

    # GPU, fused single pass, out of place (streaming kernel, then the phased one forced on) and in place
    for variant in (2, 8):
        comp.set_param("variant", variant)
        try:
            outs2 = [to_dev(np.zeros(c + 4, np_t)) for c in counts]
            plan.reduce(O.SUM, d_t, d_peers, outs2, lp_mode=lp)
            torch.cuda.synchronize()
        finally:
            comp.set_param("variant", 0)
        for i, c in enumerate(counts):
            g = to_host(outs2[i], np_t)
            assert_same(g[:c], want[i], dtype, f"fused tensor {i} variant {variant}")
            assert (g[c:] == 0).all()
    comp.set_param("variant", 8)
    try:
        plan.reduce(O.SUM, d_t, d_peers, d_t, lp_mode=lp)
        torch.cuda.synchronize()
    finally:
        comp.set_param("variant", 0)
    for i, c in enumerate(counts):
        sh = (i % 3) if align == 1 else 0
        g = to_host(holders[i], np_t)
        assert_same(g[sh:sh + c], want[i], dtype, f"fused in-place tensor {i}")
        assert (g[:sh] == 0).all() and (g[sh + c:] == 0).all()
    plan.close()


@pytest.mark.parametrize("dtype,op", [(O.FLOAT16, O.MAX), (O.BFLOAT16, O.SUM), (O.INT32, O.PROD)])
def test_fused_reduce_peer_count_limits_and_errors(comp, dtype, op):
    """No peers at all (every tensor comes back as it is -- or, for bf16 with fp32 accumulate, as widening and
    rounding once leave it), one peer, the maximum of 16, and the argument errors: 17 peers, a null tensor."""
    import torch
    rng = np.random.default_rng(70 + dtype)
    counts = [1, 4095, 4096, 4097, 20_000, 0, 33_333]
    np_t = O.NP_STORAGE[dtype]
    esz = O.DTYPE_SIZE[dtype]
    keep = 1 if dtype == O.BFLOAT16 else 0
    lp = comp.LP_KEEP_PRECISION if keep else comp.LP_PAIRWISE
    plan = comp.FusionPlan(counts, dtype, 1)
    offs, total = O.fusion_offsets(counts, esz, 1)
    nelem = total // esz
    tensors = [make_inputs(rng, dtype, c, op, 1, "bits" if dtype != O.INT32 else "config")[0] if c else np.zeros(0, np_t) for c in counts]
    peers = [make_inputs(rng, dtype, nelem, op, 1)[0] for _ in range(16)]
    d_t = [to_dev(t if t.size else np.zeros(1, np_t)) for t in tensors]
    d_peers = [to_dev(p_) for p_ in peers]
    for n_peers in (0, 1, 16):
        for variant in (0, 8):
            comp.set_param("variant", variant)
            try:
                outs = [to_dev(np.zeros(c + 3, np_t)) for c in counts]
                plan.reduce(op, d_t, d_peers[:n_peers], outs, lp_mode=lp)
                torch.cuda.synchronize()
            finally:
                comp.set_param("variant", 0)
            for i, c in enumerate(counts):
                o = int(offs[i]) // esz
                want = O.reduce_n([tensors[i]] + [p_[o:o + c] for p_ in peers[:n_peers]], dtype, op, keep=keep) if c else tensors[i]
                g = to_host(outs[i], np_t)
                assert_same(g[:c], want, dtype, f"peers={n_peers} variant={variant} tensor {i}")
                assert not g[c:].view(np.uint8).any()
    outs = [to_dev(np.zeros(c + 3, np_t)) for c in counts]
    with pytest.raises(comp.CclError):
        plan.reduce(op, d_t, d_peers + [d_peers[0]], outs, lp_mode=lp)          # 17 peers
    with pytest.raises(comp.CclError):
        plan.reduce(op, [0] + d_t[1:], d_peers[:2], outs, lp_mode=lp)             # a null tensor with a non-zero count
    with pytest.raises(comp.CclError):
        plan.reduce(4, d_t, d_peers[:2], outs, lp_mode=lp)                         # custom has no device form here
    torch.cuda.synchronize()
    assert all(not to_host(o_, np_t).view(np.uint8).any() for o_ in outs), "a rejected call wrote something"
    plan.close()


def test_fusion_config_bf16_256_tensors(comp):
    """The benchmark's fusion configuration at reduced element counts: 256 bf16 gradient tensors, counts
    log-uniform, N(0, 0.02) values, 256-byte aligned offsets, 8-input sum against 7 peer fusion buffers."""
    import torch
    rng = np.random.default_rng(2024)
    counts = log_uniform_counts(rng, 256, 2048, 65536)
    tensors = [O.bf16_from_f32((rng.standard_normal(c) * 0.02).astype(np.float32)) for c in counts]
    plan = comp.FusionPlan(counts, O.BFLOAT16, 256)
    offs, total = O.fusion_offsets(counts, 2, 256)
    nelem = total // 2
    peers = [O.bf16_from_f32((rng.standard_normal(nelem) * 0.02).astype(np.float32)) for _ in range(7)]
    fb = O.fusion_pack(tensors, offs, total, 2)
    fused = O.reduce_n([fb.view(np.uint16)] + peers, O.BFLOAT16, O.SUM, keep=1, threads=8)
    want = O.fusion_unpack(fused.view(np.uint8), counts, offs, np.uint16)
    d_t = [to_dev(t) for t in tensors]
    d_peers = [to_dev(p) for p in peers]
    for variant in (0, 8):
        comp.set_param("variant", variant)
        try:
            outs = [torch.zeros_like(t) for t in d_t]
            plan.reduce(O.SUM, d_t, d_peers, outs, lp_mode=comp.LP_KEEP_PRECISION)
            torch.cuda.synchronize()
        finally:
            comp.set_param("variant", 0)
        for i in range(256):
            assert (to_host(outs[i], np.uint16) == want[i]).all(), (i, variant)
    # per-tensor invariant: fused result == unfused 8-input reduce of the tensor with the peer slices
    i = 17
    lo = int(offs[i]) // 2
    single = torch.empty_like(d_t[i])
    comp.comp_reduce_n(O.BFLOAT16, O.SUM, [d_t[i]] + [p.data_ptr() + lo * 2 for p in d_peers], single, counts[i],
                       lp_mode=comp.LP_KEEP_PRECISION)
    torch.cuda.synchronize()
    assert (to_host(single, np.uint16) == want[i]).all()
    with pytest.raises(comp.CclError):
        plan.reduce(O.SUM, d_t, d_peers, outs, lp_mode=comp.LP_KEEP_PRECISION | comp.LP_TAIL_QUIRK)
    plan.close()


@pytest.mark.parametrize("dtype,op,n_peers,lp,impl,align", [
    (O.BFLOAT16, O.SUM, 7, 1, 2, 256), (O.FLOAT16, O.MAX, 1, 0, 2, 256), (O.INT8, O.MIN, 7, 0, 2, 256),
    (O.FLOAT64, O.PROD, 2, 0, 2, 256), (O.BFLOAT16, O.SUM, 5, 0, 2, 1), (O.INT32, O.SUM, 8, 0, 2, 256),
    (O.FLOAT32, O.MIN, 4, 0, 2, 16), (O.BFLOAT16, O.PROD, 3, 0, 1, 256), (O.UINT8, O.SUM, 6, 0, 2, 1),
    (O.FLOAT16, O.SUM, 16, 0, 2, 2), (O.BFLOAT16, O.SUM, 7, 1, 2, 1)])
def test_fused_reduce_over_several_phases(comp, dtype, op, n_peers, lp, impl, align):
    """The phased fused kernels with enough work that every LDS and register slot of a phase is used and a second
    phase follows (a phase holds 92 MB chip-wide in the item kernel, 101 MB in the tiled one), for several element types, operations and peer counts -- up to four
    peers the item kernel (16 KiB items, all inputs of an item in flight), from five the tiled kernel (32 KiB tiles,
    the inputs one after the other, any number of peers) -- against the oracle tensor by tensor."""
    import torch
    rng = np.random.default_rng(900 + dtype * 8 + n_peers)
    esz = O.DTYPE_SIZE[dtype]
    np_t = O.NP_STORAGE[dtype]
    k = 37
    target = 110 << 20                                   # payload bytes
    w = rng.random(k) ** 3 + 0.01
    counts = [max(1, int(target * x / w.sum()) // esz + int(rng.integers(0, 7))) for x in w]
    counts[3] = 5
    plan = comp.FusionPlan(counts, dtype, align)
    offs, total = O.fusion_offsets(counts, esz, align)
    nelem = (total + esz - 1) // esz
    tensors = [make_inputs(rng, dtype, c, op, 1)[0] for c in counts]
    peers = [make_inputs(rng, dtype, nelem, op, 1)[0] for _ in range(n_peers)]
    d_t = [to_dev(t) for t in tensors]
    d_p = [to_dev(p) for p in peers]
    outs = [to_dev(np.zeros(c + 6, np_t)) for c in counts]
    sh = [i % 3 for i in range(k)]                       # every third output on its holder's boundary, the others 1 and 2 elements off
    views = [o[s_:s_ + c] for o, s_, c in zip(outs, sh, counts)]
    want = []
    for i, c in enumerate(counts):
        o = int(offs[i]) // esz
        want.append(O.reduce_n([tensors[i]] + [p[o:o + c] for p in peers], dtype, op, keep=lp, bf16_impl=impl))
    # the default, then other points at which a block reports its arrival at the barrier and other paces of the write
    # phase (which only few enough inputs for the type take): timing only, same bits
    for loads, stores, pace in ((-1, -1, 7300), (0, 0, 0), (4096, 20, 30000), (40, 3, 400)):
        for o in outs:
            o.zero_()
        comp.set_param("variant", 8)
        comp.set_param("phase_early_loads", loads)
        comp.set_param("phase_early_stores", stores)
        comp.set_param("phase_write_pace", pace)
        try:
            plan.reduce(op, d_t, d_p, views, lp_mode=lp, bf16_impl=impl)
            torch.cuda.synchronize()
            assert comp.last_kernel() == ("fusion_reduce_tiled_kernel" if n_peers >= 5 else "fusion_reduce_phased_kernel")
        finally:
            comp.set_param("variant", 0)
            comp.set_param("phase_early_loads", -1)
            comp.set_param("phase_early_stores", -1)
            comp.set_param("phase_write_pace", 7300)
        for i, c in enumerate(counts):
            g = to_host(outs[i], np_t)
            assert_same(g[sh[i]:sh[i] + c], want[i], dtype, f"tensor {i} of {c} elements, early loads {loads} stores {stores} pace {pace}")
            assert not g[:sh[i]].view(np.uint8).any() and not g[sh[i] + c:].view(np.uint8).any(), "wrote outside the tensor"
    plan.close()



@pytest.mark.parametrize("dtype,op,lp,align", [(O.FLOAT32, O.SUM, 0, 256), (O.BFLOAT16, O.SUM, 1, 1)])
def test_fused_reduce_with_two_peers_takes_the_phased_kernel_when_large(comp, dtype, op, lp, align):
    """Two peers: the streaming kernel below 960 MB of traffic, the phased item kernel (write phase paced by the clock)
    from there; the same bits either way, against the oracle tensor by tensor."""
    import torch
    rng = np.random.default_rng(77 + dtype)
    esz = O.DTYPE_SIZE[dtype]
    np_t = O.NP_STORAGE[dtype]
    for target, kernel in ((300 << 20, "fusion_reduce_phased_kernel"), (100 << 20, "fusion_reduce_kernel")):
        k = 23
        w = rng.random(k) ** 2 + 0.01
        counts = [max(1, int(target * x / w.sum()) // esz + int(rng.integers(0, 5))) for x in w]
        plan = comp.FusionPlan(counts, dtype, align)
        offs, total = O.fusion_offsets(counts, esz, align)
        nelem = (total + esz - 1) // esz
        tensors = [make_inputs(rng, dtype, c, op, 1)[0] for c in counts]
        peers = [make_inputs(rng, dtype, nelem, op, 1)[0] for _ in range(2)]
        d_t = [to_dev(t) for t in tensors]
        d_p = [to_dev(p) for p in peers]
        outs = [to_dev(np.zeros(c, np_t)) for c in counts]
        plan.reduce(op, d_t, d_p, outs, lp_mode=lp)
        torch.cuda.synchronize()
        assert comp.last_kernel() == kernel
        for i, c in enumerate(counts):
            o = int(offs[i]) // esz
            want = O.reduce_n([tensors[i]] + [p[o:o + c] for p in peers], dtype, op, keep=lp)
            assert_same(to_host(outs[i], np_t), want, dtype, f"tensor {i} of {c} elements, {kernel}")
        plan.close()
        del d_t, d_p, outs
