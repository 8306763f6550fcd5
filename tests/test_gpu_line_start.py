"""Large calls start their vectors on a 128-byte line of the buffers that matter most (the head then reaches up to 127
bytes, handled element by element), and the phased kernels lay a wave's vectors of a group next to each other when a
buffer is off the lines.  Neither changes a result: every combination of the two knobs is compared with the oracle
bit for bit, with buffers at byte offsets that are multiples of the element size but not of 16 or of 128 bytes, in
place and out of place, with one and with several destinations, through the streaming and the phased kernels."""
import numpy as np
import pytest

import oracle_lib as O
from gpu_util import assert_same, make_inputs, to_dev, to_host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def comp():
    import torch
    assert torch.cuda.is_available(), "needs a GPU"
    import oneccl_amd.comp as c
    c.lib()
    return c


CASES = [(O.INT8, O.SUM, 3), (O.BFLOAT16, O.SUM, 8), (O.FLOAT16, O.MAX, 2), (O.INT32, O.PROD, 4), (O.FLOAT32, O.SUM, 2),
         (O.FLOAT64, O.MIN, 5), (O.UINT64, O.SUM, 9)]


@pytest.mark.parametrize("dtype,op,n", CASES)
def test_heads_up_to_a_line(comp, dtype, op, n):
    import torch
    rng = np.random.default_rng(4100 + 16 * dtype + n)
    esz, np_t = O.DTYPE_SIZE[dtype], O.NP_STORAGE[dtype]
    keep = 1 if dtype == O.BFLOAT16 else 0
    pad = 256                                               # elements around every buffer, checked to stay zero
    per_line = 128 // esz
    count = (3 << 20) // esz + 2 * per_line + 5             # past the size from which lines are looked at
    srcs = make_inputs(rng, dtype, count, op, n)
    want = O.reduce_n(srcs, dtype, op, keep=keep, threads=16)
    layouts = [
        [per_line - 1] * (n + 1),                           # everything one element below a line: the longest head
        [1] * (n + 1),                                      # everything one element past a line
        [16 // esz] * (n + 1) if esz < 16 else [1] * (n + 1),   # on the 16-byte boundary, off the line
        [0] * n + [per_line // 2 + (16 // esz if esz <= 8 else 0)],     # the output alone off the line
        [int(x) for x in rng.integers(0, per_line, n + 1)],         # everything at its own place
        [0] + [64 // esz] * (n - 1) + [0],                  # the peers 64 bytes off
    ]
    try:
        for variant in (0, 8, 2):
            comp.set_param("variant", variant)
            for line_start, wave_runs in ((1, 1), (0, 1), (1, 0), (1, 2)):
                if variant == 2 and wave_runs != 1:
                    continue                                # the streaming kernels have one layout
                comp.set_param("line_start", line_start)
                comp.set_param("wave_runs", wave_runs)
                for li, sh in enumerate(layouts):
                    for in_place in (False, True):
                        big = []
                        for s_, k in zip(srcs, sh[:n]):
                            h = np.zeros(count + 2 * pad, np_t)
                            h[pad + k:pad + k + count] = s_
                            big.append(to_dev(h))
                        out = big[0] if in_place else to_dev(np.zeros(count + 2 * pad, np_t))
                        lo = pad + (sh[0] if in_place else sh[n])
                        sp = [b_.data_ptr() + (pad + k) * esz for b_, k in zip(big, sh[:n])]
                        comp.comp_reduce_n(dtype, op, sp, out.data_ptr() + lo * esz, count, lp_mode=keep)
                        torch.cuda.synchronize()
                        g = to_host(out, np_t)
                        what = (f"variant={variant} line_start={line_start} wave_runs={wave_runs} layout={li} shifts={sh} "
                                f"in_place={in_place} kernel={comp.last_kernel()}")
                        assert_same(g[lo:lo + count], want, dtype, what, srcs, op, keep=keep)
                        assert not g[:lo].view(np.uint8).any() and not g[lo + count:].view(np.uint8).any(), "wrote outside: " + what
    finally:
        comp.set_param("variant", 0)
        comp.set_param("line_start", 1)
        comp.set_param("wave_runs", 1)


def test_several_destinations_on_different_lines(comp):
    import torch
    rng = np.random.default_rng(77)
    dtype, op, n = O.BFLOAT16, O.SUM, 4
    esz, np_t, pad = 2, O.NP_STORAGE[dtype], 256
    count = (2 << 20) + 77
    srcs = make_inputs(rng, dtype, count, op, n)
    want = O.reduce_n(srcs, dtype, op, keep=1, threads=16)
    try:
        for variant in (0, 8):
            comp.set_param("variant", variant)
            for wave_runs in (0, 1, 2):
                comp.set_param("wave_runs", wave_runs)
                in_sh, out_sh = [8, 8, 16, 0], [8, 40, 8]
                big = []
                for s_, k in zip(srcs, in_sh):
                    h = np.zeros(count + 2 * pad, np_t)
                    h[pad + k:pad + k + count] = s_
                    big.append(to_dev(h))
                outs = [to_dev(np.zeros(count + 2 * pad, np_t)) for _ in out_sh]
                comp.comp_reduce_write_n(dtype, op, [b_.data_ptr() + (pad + k) * esz for b_, k in zip(big, in_sh)],
                                         [o_.data_ptr() + (pad + k) * esz for o_, k in zip(outs, out_sh)], count, lp_mode=1)
                torch.cuda.synchronize()
                for o_, k in zip(outs, out_sh):
                    g = to_host(o_, np_t)
                    what = f"variant={variant} wave_runs={wave_runs} destination at +{k}"
                    assert_same(g[pad + k:pad + k + count], want, dtype, what, srcs, op, keep=1)
                    assert not g[:pad + k].view(np.uint8).any() and not g[pad + k + count:].view(np.uint8).any(), "wrote outside: " + what
    finally:
        comp.set_param("variant", 0)
        comp.set_param("wave_runs", 1)


def test_knobs_round_trip(comp):
    for name, values in (("line_start", (0, 1)), ("wave_runs", (0, 2, 1))):
        for v in values:
            comp.set_param(name, v)
            assert comp.get_param(name) == v
    with pytest.raises(Exception):
        comp.set_param("wave_runs", 3)
    with pytest.raises(Exception):
        comp.set_param("line_start", 2)
    assert comp.get_param("line_start") == 1 and comp.get_param("wave_runs") == 1
