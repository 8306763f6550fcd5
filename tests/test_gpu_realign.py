"""Inputs of 16- and 8-bit types whose vectors start off a 4-byte boundary (a peer's block behind an odd number of
elements, int8 at an odd offset) are read on that boundary and shifted into place in registers: the next lane's first
dword by a DPP wave shift, lane 63 by one extra dword load, the last whole vector left to the edge lanes.  Every
kernel form that takes the path is compared with the oracle bit for bit, with the knob on (and the library's counter
saying that the path was taken) and off (loose vector loads), at counts around the vector, wave, tile and phase
boundaries, in place and out of place, with one and several destinations, and as jobs of a batch."""
import numpy as np
import pytest

import oracle_lib as O
from gpu_util import assert_same, make_inputs, to_dev, to_host

pytestmark = pytest.mark.gpu

SMALL = [O.INT8, O.UINT8, O.INT16, O.UINT16, O.FLOAT16, O.BFLOAT16]


@pytest.fixture(scope="module")
def comp():
    import torch
    assert torch.cuda.is_available(), "needs a GPU"
    import oneccl_amd.comp as c
    c.lib()
    return c


def _holders(srcs, shifts, pad, np_t):
    out = []
    for s_, sh in zip(srcs, shifts):
        h = np.zeros(s_.size + 2 * pad, np_t)
        h[pad + sh:pad + sh + s_.size] = s_
        out.append(to_dev(h))
    return out


@pytest.mark.parametrize("variant", [0, 8])
@pytest.mark.parametrize("dtype,op,n", [(O.BFLOAT16, O.SUM, 8), (O.BFLOAT16, O.MAX, 3), (O.FLOAT16, O.SUM, 4), (O.INT8, O.SUM, 5),
                                        (O.UINT8, O.MIN, 2), (O.INT16, O.PROD, 9), (O.UINT16, O.MAX, 2)])
def test_inputs_off_a_4_byte_boundary(comp, variant, dtype, op, n):
    import torch
    rng = np.random.default_rng(900 + 16 * dtype + n)
    esz, np_t, per16 = O.DTYPE_SIZE[dtype], O.NP_STORAGE[dtype], 16 // O.DTYPE_SIZE[dtype]
    keep = 1 if dtype == O.BFLOAT16 and op == O.SUM else 0
    pad = 64
    per_wave = 64 * per16
    per_phase = comp.get_param("num_cus") * 512 * 44 * per16
    counts = [per16 - 1, per16, 2 * per16, 2 * per16 + 1, per_wave - 1, per_wave + per16, 4 * 256 * per16 + 3, 70_001, 1_000_003]
    if variant == 8:
        counts += [per_phase + per16 * 2 + 1, 2 * per_phase - 5]
        counts = [c for c in counts if c * esz * (n + 1) <= (4 << 30)]
    odd = [k for k in range(1, per16) if (k * esz) % 4]          # element shifts that leave the 4-byte boundary
    comp.set_param("variant", variant)
    try:
        for count in counts:
            srcs = make_inputs(rng, dtype, count, op, n, "bits" if dtype in (O.FLOAT16, O.BFLOAT16) and count < 100_000 else "config")
            want = O.reduce_n(srcs, dtype, op, keep=keep, threads=16)
            for trial in range(3 if count < 5_000_000 else 1):
                # 0: the first input and the output aligned, the peers at odd shifts; 1: everything at its own shift;
                # 2: in place on input 0 (aligned), the other inputs at one odd shift
                if trial == 0:
                    sh = [0] + [odd[j % len(odd)] for j in range(n - 1)] + [0]
                elif trial == 1:
                    sh = [int(x) for x in rng.integers(0, per16, n + 1)]
                    sh[n - 1] = odd[0]
                else:
                    sh = [0] + [odd[-1]] * (n - 1) + [0]
                for realign in (1, 0):
                    comp.set_param("realign", realign)
                    big = _holders(srcs, sh[:n], pad, np_t)
                    out = big[0] if trial == 2 else to_dev(np.zeros(count + 2 * pad, np_t))
                    sp = [b_.data_ptr() + (pad + k) * esz for b_, k in zip(big, sh[:n])]
                    before = comp.get_param("realigned_launches")
                    comp.comp_reduce_n(dtype, op, sp, out.data_ptr() + (pad + sh[n]) * esz, count, lp_mode=keep)
                    torch.cuda.synchronize()
                    took = comp.get_param("realigned_launches") - before
                    g = to_host(out, np_t)
                    lo = pad + sh[n]
                    what = f"count={count} shifts={sh} realign={realign} trial={trial} kernel={comp.last_kernel()}"
                    assert_same(g[lo:lo + count], want, dtype, what, srcs, op, keep=keep)
                    assert not g[:lo].view(np.uint8).any() and not g[lo + count:].view(np.uint8).any(), "wrote outside: " + what
                    if realign and trial != 1 and count >= 3 * per16:
                        assert took >= 1, "the realigning path was not taken: " + what
                    if not realign:
                        assert took == 0, what
    finally:
        comp.set_param("variant", 0)
        comp.set_param("realign", 1)


def test_output_aliasing_an_input_that_is_realigned(comp):
    """The output is one of the inputs, one element off the boundary the other inputs share.  With few inputs the
    vectors start on the output's boundary (the other inputs are realigned); with twelve they start on the others'
    boundary, and the aliased input is read realigned and overwritten, as loose vectors, in the same launch."""
    import torch
    rng = np.random.default_rng(31)
    for dtype, op, n in ((O.BFLOAT16, O.SUM, 8), (O.INT8, O.SUM, 6), (O.FLOAT16, O.MAX, 5), (O.BFLOAT16, O.SUM, 12)):
        esz, np_t, per16 = O.DTYPE_SIZE[dtype], O.NP_STORAGE[dtype], 16 // O.DTYPE_SIZE[dtype]
        keep = 1 if dtype == O.BFLOAT16 else 0
        for variant in (0, 8):
            comp.set_param("variant", variant)
            try:
                for count in (1000, 300_007, 5_000_011):
                    srcs = make_inputs(rng, dtype, count, op, n)
                    want = O.reduce_n(srcs, dtype, op, keep=keep, threads=16)
                    for alias in (0, n - 1):
                        sh = [0] * n
                        sh[alias] = 1                       # one element off: 2 bytes for the 16-bit types, 1 for int8
                        big = _holders(srcs, sh, 64, np_t)
                        sp = [b_.data_ptr() + (64 + k) * esz for b_, k in zip(big, sh)]
                        comp.comp_reduce_n(dtype, op, sp, sp[alias], count, lp_mode=keep)
                        torch.cuda.synchronize()
                        g = to_host(big[alias], np_t)
                        what = f"dtype={dtype} count={count} alias={alias} variant={variant}"
                        assert_same(g[65:65 + count], want, dtype, what, srcs, op, keep=keep)
                        assert not g[:65].view(np.uint8).any() and not g[65 + count:].view(np.uint8).any(), "wrote outside: " + what
                        for j in range(n):
                            if j != alias:
                                assert (to_host(big[j], np_t)[64:64 + count] == srcs[j]).all(), "an input changed: " + what
            finally:
                comp.set_param("variant", 0)


@pytest.mark.parametrize("dtype", [O.BFLOAT16, O.UINT8])
def test_several_destinations_and_batch_jobs(comp, dtype):
    import torch
    rng = np.random.default_rng(57 + dtype)
    esz, np_t, per16 = O.DTYPE_SIZE[dtype], O.NP_STORAGE[dtype], 16 // O.DTYPE_SIZE[dtype]
    keep = 1 if dtype == O.BFLOAT16 else 0
    pad = 64
    # one reduce stored to three buffers, the second of them off the boundary; inputs at odd shifts
    for variant in (0, 8):
        comp.set_param("variant", variant)
        try:
            for count in (per16 * 3 + 1, 200_003, 4_000_001):
                srcs = make_inputs(rng, dtype, count, O.SUM, 4)
                want = O.reduce_n(srcs, dtype, O.SUM, keep=keep, threads=16)
                sh = [0, 1, 3 % per16, 1]
                big = _holders(srcs, sh, pad, np_t)
                outs = [to_dev(np.zeros(count + 2 * pad, np_t)) for _ in range(3)]
                osh = [0, 1, 0]
                before = comp.get_param("realigned_launches")
                comp.comp_reduce_write_n(dtype, O.SUM, [b_.data_ptr() + (pad + k) * esz for b_, k in zip(big, sh)],
                                         [o_.data_ptr() + (pad + k) * esz for o_, k in zip(outs, osh)], count, lp_mode=keep)
                torch.cuda.synchronize()
                assert comp.get_param("realigned_launches") == before + 1
                for o_, k in zip(outs, osh):
                    g = to_host(o_, np_t)
                    assert_same(g[pad + k:pad + k + count], want, dtype, f"count={count} variant={variant}", srcs, O.SUM, keep=keep)
                    assert not g[:pad + k].view(np.uint8).any() and not g[pad + k + count:].view(np.uint8).any()
        finally:
            comp.set_param("variant", 0)
    # jobs of a batch: every job with its own shifts and count, some in place
    jobs, checks = [], []
    for j, count in enumerate([1, per16, 5 * per16 + 1, 1023, 4096 * per16, 65_537, 300_001, 0, 1_000_003]):
        srcs = make_inputs(rng, dtype, count, O.SUM, 3) if count else [np.zeros(0, np_t)] * 3
        sh = [0, 1, (2 * j + 1) % per16]
        big = _holders(srcs, sh, pad, np_t)
        out = big[0] if j % 2 else to_dev(np.zeros(count + 2 * pad, np_t))
        jobs.append(([b_.data_ptr() + (pad + k) * esz for b_, k in zip(big, sh)], out.data_ptr() + pad * esz, count))
        checks.append((srcs, out, count, big))
    before = comp.get_param("realigned_launches")
    comp.comp_reduce_batch(dtype, O.SUM, jobs, lp_mode=keep)
    torch.cuda.synchronize()
    assert comp.get_param("realigned_launches") > before
    for j, (srcs, out, count, big) in enumerate(checks):
        g = to_host(out, np_t)
        if count:
            assert_same(g[pad:pad + count], O.reduce_n(srcs, dtype, O.SUM, keep=keep), dtype, f"job {j} count={count}", srcs, O.SUM, keep=keep)
        assert not g[:pad].view(np.uint8).any() and not g[pad + count:].view(np.uint8).any(), f"job {j}: wrote outside"
