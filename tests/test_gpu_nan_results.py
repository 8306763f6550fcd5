"""NaN results of sum and prod on the GPU, compared on bits: the literal x86 patterns of tests/nan_cases.py, every
pair of special values, and chains with special values sprinkled in -- through the streaming, the phased and the
fused kernels, head/tail lanes included.  Two different NaNs pass only where a step of the chain had two NaN
operands (oracle_lib.same_bits)."""
import numpy as np
import pytest

import nan_cases
import oracle_lib as O
from gpu_util import assert_same, make_inputs, to_dev, to_host

pytestmark = pytest.mark.gpu

# (dtype, lp_mode, bf16_impl, fp16_impl, oracle keep)
MODES = [(O.FLOAT32, 0, 2, 0, 0), (O.FLOAT64, 0, 2, 0, 0),
         (O.BFLOAT16, 0, 0, 0, 0), (O.BFLOAT16, 0, 1, 0, 0), (O.BFLOAT16, 0, 2, 0, 0), (O.BFLOAT16, 1, 2, 0, 1), (O.BFLOAT16, 1, 1, 0, 1),
         (O.FLOAT16, 0, 2, 3, 0), (O.FLOAT16, 0, 2, 4, 0)]


@pytest.fixture(scope="module")
def comp():
    import torch
    assert torch.cuda.is_available(), "needs a GPU"
    import oneccl_amd.comp as c
    c.lib()
    return c


def _okw(impl, f16, keep):
    return dict(keep=keep, bf16_impl=impl, fp16_impl=f16 or O.FP16_AVX512F)


@pytest.mark.parametrize("dtype,lp,impl,f16,keep", MODES)
def test_literal_x86_nan_patterns(comp, dtype, lp, impl, f16, keep):
    """The table of literal patterns, as a pair (ccl_comp_reduce) and as the head of a longer chain; repeated so that
    the cases land in full vectors as well as in the head/tail lanes."""
    import torch
    np_t = O.NP_STORAGE[dtype]
    one = {O.FLOAT32: np.float32(1), O.FLOAT64: np.float64(1), O.BFLOAT16: np.uint16(0x3F80), O.FLOAT16: np.uint16(0x3C00)}[dtype]
    for op in (O.SUM, O.PROD):
        a, b, want = nan_cases.table(dtype, op)
        reps = 37
        a, b, want = np.tile(a, reps), np.tile(b, reps), np.tile(want, reps)
        if not keep:
            da, db = to_dev(a), to_dev(b)
            comp.comp_reduce(dtype, op, da, a.size, db, bf16_impl=impl, fp16_impl=f16)
            torch.cuda.synchronize()
            assert_same(to_host(db, np_t), want, dtype, f"pair op={op}")
        nan = O.nan_mask(want, dtype)
        ones = np.full(a.size, one, np_t)
        for variant in (0, 8):
            comp.set_param("variant", variant)
            try:
                out = to_dev(np.zeros(a.size, np_t))
                comp.comp_reduce_n(dtype, op, [to_dev(b), to_dev(a), to_dev(ones), to_dev(ones)], out, a.size, lp_mode=lp,
                                   bf16_impl=impl, fp16_impl=f16)
                torch.cuda.synchronize()
            finally:
                comp.set_param("variant", 0)
            got = to_host(out, np_t)
            assert_same(got[nan], want[nan], dtype, f"chain op={op} variant={variant}")
            assert_same(got, O.reduce_n([b, a, ones, ones], dtype, op, **_okw(impl, f16, keep)), dtype, f"chain vs oracle op={op}")


@pytest.mark.parametrize("dtype,lp,impl,f16,keep", MODES)
def test_every_pair_of_special_values_and_sprinkled_chains(comp, dtype, lp, impl, f16, keep):
    import torch
    rng = np.random.default_rng(9000 + dtype * 8 + impl + f16)
    np_t = O.NP_STORAGE[dtype]
    esz = O.DTYPE_SIZE[dtype]
    sp = nan_cases.specials(dtype)
    kw = _okw(impl, f16, keep)
    for op in (O.SUM, O.PROD):
        # all pairs, at a shift that puts some of them into the head and tail lanes
        a, b = np.repeat(sp, sp.size), np.tile(sp, sp.size)
        for variant in (0, 2, 8):
            for shift in (0, 1):
                ha, hb = to_dev(np.concatenate([np.zeros(shift, np_t), a])), to_dev(np.concatenate([np.zeros(shift, np_t), b]))
                out = to_dev(np.zeros(a.size + shift, np_t))
                comp.set_param("variant", variant)
                try:
                    comp.comp_reduce_n(dtype, op, [hb.data_ptr() + shift * esz, ha.data_ptr() + shift * esz],
                                       out.data_ptr() + shift * esz, a.size, lp_mode=lp, bf16_impl=impl, fp16_impl=f16)
                    torch.cuda.synchronize()
                finally:
                    comp.set_param("variant", 0)
                want = O.reduce_n([b, a], dtype, op, **kw)
                assert_same(to_host(out, np_t)[shift:], want, dtype, f"pairs op={op} variant={variant} shift={shift}", [b, a], op, **kw)
        # chains of 2..9 inputs of ordinary values with special values at one element in ten
        for n in (2, 3, 5, 8, 9):
            count = 70_001
            srcs = make_inputs(rng, dtype, count, op, n)
            for s in srcs:
                hit = rng.random(count) < 0.1
                s[hit] = rng.choice(sp, int(hit.sum()))
            want = O.reduce_n(srcs, dtype, op, **kw)
            assert O.nan_mask(want, dtype).sum() > 1000
            d = [to_dev(s) for s in srcs]
            for variant in (0, 2, 8):
                comp.set_param("variant", variant)
                try:
                    out = to_dev(np.zeros(count, np_t))
                    comp.comp_reduce_n(dtype, op, d, out, count, lp_mode=lp, bf16_impl=impl, fp16_impl=f16)
                    outs = [to_dev(np.zeros(count, np_t)) for _ in range(2)]
                    comp.comp_reduce_write_n(dtype, op, d, outs, count, lp_mode=lp, bf16_impl=impl, fp16_impl=f16)
                    torch.cuda.synchronize()
                finally:
                    comp.set_param("variant", 0)
                for o in [out] + outs:
                    assert_same(to_host(o, np_t), want, dtype, f"chain n={n} op={op} variant={variant}", srcs, op, **kw)


@pytest.mark.parametrize("dtype,lp,impl,f16,keep", [m for m in MODES if m[0] != O.FLOAT64] + [(O.FLOAT64, 0, 2, 0, 0)])
def test_fused_reduce_nan_results(comp, dtype, lp, impl, f16, keep):
    """The same through the fused (tensors + peer fusion buffers) kernels, streaming and phased, tight layout with
    odd sizes so that tensors start off a 16-byte boundary."""
    import torch
    rng = np.random.default_rng(9500 + dtype * 8 + impl + f16)
    np_t = O.NP_STORAGE[dtype]
    esz = O.DTYPE_SIZE[dtype]
    sp = nan_cases.specials(dtype)
    kw = _okw(impl, f16, keep)
    counts = [401, 8191, 1, 20_003, 4096]
    offs, total = O.fusion_offsets(counts, esz, 1)
    nelem = total // esz
    for op in (O.SUM, O.PROD):
        for n_peers in (1, 3, 7):
            def sprinkle(x):
                hit = rng.random(x.size) < 0.1
                x[hit] = rng.choice(sp, int(hit.sum()))
                return x
            tensors = [sprinkle(make_inputs(rng, dtype, c, op, 1)[0]) for c in counts]
            peers = [sprinkle(make_inputs(rng, dtype, nelem, op, 1)[0]) for _ in range(n_peers)]
            d_t, d_p = [to_dev(t) for t in tensors], [to_dev(p) for p in peers]
            plan = comp.FusionPlan(counts, dtype, 1)
            for variant in (2, 8):
                comp.set_param("variant", variant)
                try:
                    outs = [to_dev(np.zeros(c, np_t)) for c in counts]
                    plan.reduce(op, d_t, d_p, outs, lp_mode=lp, bf16_impl=impl, fp16_impl=f16)
                    torch.cuda.synchronize()
                finally:
                    comp.set_param("variant", 0)
                for i, c in enumerate(counts):
                    o = int(offs[i]) // esz
                    chain = [tensors[i]] + [p[o:o + c] for p in peers]
                    want = O.reduce_n(chain, dtype, op, **kw)
                    assert_same(to_host(outs[i], np_t), want, dtype, f"fused op={op} peers={n_peers} variant={variant} tensor {i}",
                                chain, op, **kw)
            plan.close()
