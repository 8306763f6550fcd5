"""GPU parity of mi_ccl_comp_reduce_write_n (one N-input reduce stored to m buffers; with one input, a copy to m
buffers) against the oracle, through the C ABI.  Bit-exact; two NaNs of a floating type compare equal."""
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


def lp_variants(dtype):
    if dtype == O.BFLOAT16:
        return [(0, 0, 0, 0), (0, 1, 0, 0), (0, 2, 0, 0), (1, 2, 1, 0), (3, 2, 1, 1)]
    return [(0, 2, 0, 0)]


@pytest.mark.parametrize("dtype", range(12))
@pytest.mark.parametrize("op", range(4))
def test_reduce_write_n_all_dtypes_ops(comp, dtype, op):
    import torch
    rng = np.random.default_rng(5000 + dtype * 4 + op)
    for n, m in [(1, 1), (1, 2), (1, 7), (2, 2), (3, 5), (8, 8), (9, 3), (16, 16)]:
        for count in (1, 15, 17, 1000, 4099, 70001):
            if n > 8 and count < 1000:
                continue
            kind = "bits" if dtype in (O.FLOAT16, O.BFLOAT16) and count % 2 else "config"
            srcs = make_inputs(rng, dtype, count, op, n, kind)
            d = [to_dev(s) for s in srcs]
            for lp, impl, keep, quirk in lp_variants(dtype):
                outs = [torch.zeros(count + 8, dtype=d[0].dtype, device="cuda") for _ in range(m)]
                comp.comp_reduce_write_n(dtype, op, d, outs, count, lp_mode=lp, bf16_impl=impl)
                torch.cuda.synchronize()
                want = O.reduce_write_n(srcs, m, dtype, op, keep=keep, quirk_tail=quirk, bf16_impl=impl)
                for k in range(m):
                    got = to_host(outs[k], O.NP_STORAGE[dtype])
                    assert_same(got[:count], want[k], dtype,
                                f"dtype={O.DTYPE_NAMES[dtype]} op={O.OP_NAMES[op]} n={n} m={m} k={k} count={count} "
                                f"lp={lp} impl={impl}", srcs, op, keep=keep, bf16_impl=impl)
                    assert not got[count:].view(np.uint8).any(), "wrote past the end"


def test_one_input_is_a_byte_copy_for_every_dtype(comp):
    """write_monolithic_kernel_N: the input reaches every peer buffer unchanged, whatever bits it holds."""
    import torch
    rng = np.random.default_rng(11)
    for dtype in range(12):
        esz = O.NP_STORAGE[dtype]().itemsize
        src = rng.integers(0, 256, 30011 * esz, dtype=np.uint8)
        d = torch.from_numpy(src.copy()).cuda()
        outs = [torch.zeros_like(d) for _ in range(7)]
        comp.comp_reduce_write_n(dtype, O.SUM, [d], outs, 30011)
        torch.cuda.synchronize()
        for o in outs:
            assert (o.cpu().numpy() == src).all(), O.DTYPE_NAMES[dtype]


def test_broadcast_sections_alignments_and_aliasing(comp):
    """One input to m buffers by the sectioned broadcast kernel (and to one buffer by the copy kernel): sizes below
    one tile, around the 16 MiB section and over several sections, 1 to 16 destinations, the source and every
    destination at its own offset from a 16-byte boundary, one destination being the source itself; nothing outside
    the destinations is written."""
    import torch
    rng = np.random.default_rng(12)
    pad = 64
    sect = 16 << 20
    for nbytes, ms in ((1, (1, 2, 16)), (15, (2,)), (4095, (1, 3)), (100_003, (1, 2, 7)), (sect - 16, (2,)),
                       (sect + 4096 + 5, (1, 3)), (3 * sect + 12_345, (2, 7)), (200_000_001, (5,))):
        src = rng.integers(0, 256, nbytes + 2 * pad, dtype=np.uint8)
        d = torch.from_numpy(src.copy()).cuda()
        for m in ms:
            for trial in range(2):
                sh = [int(x) for x in rng.integers(0, 16, m + 1)] if trial else [0] * (m + 1)
                outs = [torch.zeros(nbytes + 2 * pad, dtype=torch.uint8, device="cuda") for _ in range(m)]
                comp.comp_reduce_write_n(O.UINT8, O.SUM, [d.data_ptr() + pad + sh[0]],
                                         [o.data_ptr() + pad + k for o, k in zip(outs, sh[1:])], nbytes)
                torch.cuda.synchronize()
                want = src[pad + sh[0]:pad + sh[0] + nbytes]
                for o, k in zip(outs, sh[1:]):
                    g = o.cpu().numpy()
                    assert (g[pad + k:pad + k + nbytes] == want).all(), (nbytes, m, sh)
                    assert not g[:pad + k].any() and not g[pad + k + nbytes:].any(), (nbytes, m, sh)
                del outs
        # the source among the destinations, with a wider type
        if nbytes % 4 == 0 or nbytes > 1000:
            cnt = nbytes // 4
            d32 = torch.from_numpy(src[:cnt * 4].copy()).cuda()
            o1, o2 = torch.zeros_like(d32), torch.zeros_like(d32)
            comp.comp_reduce_write_n(O.FLOAT32, O.MAX, [d32], [o1, d32, o2], cnt)
            torch.cuda.synchronize()
            for o in (o1, d32, o2):
                assert (o.cpu().numpy() == src[:cnt * 4]).all(), (nbytes, "aliased")
        del d


@pytest.mark.parametrize("variant", [2, 8])
def test_destination_aliases_a_source_and_misaligned_buffers(comp, variant):
    """In place (destination k is source j, as allreduce_kernel's output may be its input), buffers that share a
    misalignment to 16 bytes (vector path with head and tail) and buffers that do not (loose vector accesses)."""
    import torch
    rng = np.random.default_rng(12)
    comp.set_param("variant", variant)
    try:
        for dtype, op in [(O.BFLOAT16, O.SUM), (O.FLOAT32, O.MIN), (O.INT16, O.PROD), (O.FLOAT64, O.SUM)]:
            np_t = O.NP_STORAGE[dtype]
            count, n, m = 50021, 4, 3
            srcs = make_inputs(rng, dtype, count, op, n)
            keep = 1 if dtype == O.BFLOAT16 else 0
            # in place
            d = [to_dev(s) for s in srcs]
            outs = [d[2], torch.empty_like(d[0]), d[0]]
            comp.comp_reduce_write_n(dtype, op, d, outs, count, lp_mode=keep)
            torch.cuda.synchronize()
            want = O.reduce_n(srcs, dtype, op, keep=keep)
            for o in outs:
                assert_same(to_host(o, np_t), want, dtype, f"in place {O.DTYPE_NAMES[dtype]}")
            # shared and mixed misalignment, in elements
            for offs_s, offs_d in [([3, 3, 3, 3], [3, 3, 3]), ([0, 1, 2, 3], [1, 0, 5])]:
                if np.dtype(np_t).itemsize == 8:
                    offs_s, offs_d = [o % 2 for o in offs_s], [o % 2 for o in offs_d]
                big = [to_dev(np.concatenate([np.zeros(o, np_t), s])) for o, s in zip(offs_s, srcs)]
                dv = [b[o:] for b, o in zip(big, offs_s)]
                obig = [torch.zeros(count + o + 4, dtype=dv[0].dtype, device="cuda") for o in offs_d]
                ov = [b[o:] for b, o in zip(obig, offs_d)]
                comp.comp_reduce_write_n(dtype, op, dv, ov, count, lp_mode=keep)
                torch.cuda.synchronize()
                for b, o in zip(obig, offs_d):
                    got = to_host(b, np_t)
                    assert_same(got[o:o + count], want, dtype, f"misaligned {offs_s} {offs_d}")
                    assert not got[:o].view(np.uint8).any() and not got[o + count:].view(np.uint8).any()
    finally:
        comp.set_param("variant", 0)


def test_phased_form_over_several_phases(comp):
    """The phased kernel forced on (variant 8) from a few elements to several phases of one launch
    (a phase holds gridDim x 512 x 20 vectors = about 42 MB per buffer)."""
    import torch
    rng = np.random.default_rng(13)
    comp.set_param("variant", 8)
    try:
        for dtype, n, m, count in [(O.BFLOAT16, 8, 2, 5), (O.BFLOAT16, 8, 8, 50_000_017), (O.FLOAT32, 2, 2, 23_000_003),
                                   (O.UINT8, 1, 7, 100_000_001), (O.BFLOAT16, 12, 1, 30_000_001), (O.INT32, 9, 1, 11_000_003)]:
            np_t = O.NP_STORAGE[dtype]
            srcs = make_inputs(rng, dtype, count, O.SUM, n)
            d = [to_dev(s) for s in srcs]
            outs = [torch.empty_like(d[0]) for _ in range(m)]
            keep = 1 if dtype == O.BFLOAT16 else 0
            if m == 1:      # more than 8 inputs to one output take the same kernels
                comp.comp_reduce_n(dtype, O.SUM, d, outs[0], count, lp_mode=keep)
            else:
                comp.comp_reduce_write_n(dtype, O.SUM, d, outs, count, lp_mode=keep)
            torch.cuda.synchronize()
            want = O.reduce_n(srcs, dtype, O.SUM, keep=keep, threads=8)
            for o in outs:
                assert_same(to_host(o, np_t), want, dtype, f"phased {O.DTYPE_NAMES[dtype]} n={n} m={m} count={count}")
    finally:
        comp.set_param("variant", 0)


def test_write_phase_paced_by_the_clock(comp):
    """With two or more destinations (and with few enough inputs for their type to one: two for every type, up to
    eight for most) the device clock lets the write phase's stores out at a set rate ("phase_write_pace", GB/s).  Timing only: unpaced, the default, a pace far below what HBM takes (every group of
    stores waits for the clock), one far above (none does) and the largest value all give the oracle's bits, over
    several phases, with the destinations at different alignments, one of them aliasing an input."""
    import torch
    rng = np.random.default_rng(29)
    assert comp.get_param("phase_write_pace") == 7300 and comp.get_param("wall_clock_khz") > 0
    comp.set_param("variant", 8)
    try:
        for dtype, n, m, count in [(O.BFLOAT16, 3, 3, 70_000_003), (O.FLOAT32, 2, 2, 40_000_001), (O.INT8, 4, 5, 1_000_003),
                                   (O.FLOAT32, 2, 1, 50_000_001), (O.BFLOAT16, 2, 1, 100_000_007),      # two inputs to one (in place) are paced too,
                                   (O.INT64, 7, 1, 20_000_003), (O.UINT8, 4, 1, 150_000_001), (O.FLOAT16, 8, 1, 60_000_001)]:   # and up to eight
            np_t, esz = O.NP_STORAGE[dtype], O.DTYPE_SIZE[dtype]
            keep = 1 if dtype == O.BFLOAT16 else 0
            srcs = make_inputs(rng, dtype, count, O.SUM, n)
            want = O.reduce_n(srcs, dtype, O.SUM, keep=keep, threads=16)
            for pace in (0, 7300, 1500, 60_000, 100_000):
                comp.set_param("phase_write_pace", pace)
                d = [to_dev(s) for s in srcs]
                pad = 64
                outs = [torch.zeros(count + 2 * pad, dtype=d[0].dtype, device="cuda") for _ in range(m - 1)]
                shifts = [(k * 8) % pad for k in range(m - 1)]
                ptrs = [d[n - 1].data_ptr()] + [o.data_ptr() + (pad + sh) * esz for o, sh in zip(outs, shifts)]
                comp.comp_reduce_write_n(dtype, O.SUM, [t.data_ptr() for t in d], ptrs, count, lp_mode=keep)
                torch.cuda.synchronize()
                assert comp.last_kernel() == "reduce_multi_phased_kernel"
                what = f"{O.DTYPE_NAMES[dtype]} n={n} m={m} count={count} pace={pace}"
                assert_same(to_host(d[n - 1], np_t), want, dtype, what + " (destination that is an input)", srcs, O.SUM, keep=keep)
                for o, sh in zip(outs, shifts):
                    g = to_host(o, np_t)
                    assert_same(g[pad + sh:pad + sh + count], want, dtype, what, srcs, O.SUM, keep=keep)
                    assert not g[:pad + sh].view(np.uint8).any() and not g[pad + sh + count:].view(np.uint8).any(), "wrote outside: " + what
        for bad in (-1, 1, 99, 100_001):
            with pytest.raises(comp.CclError):
                comp.set_param("phase_write_pace", bad)
    finally:
        comp.set_param("variant", 0)
        comp.set_param("phase_write_pace", 7300)


def test_equals_reduce_n_followed_by_copies_at_a_large_size(comp):
    """Size-independent property at 1 GiB per buffer: every destination equals mi_ccl_comp_reduce_n's output."""
    import torch
    count = 1 << 29
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    srcs = [torch.empty(count, dtype=torch.bfloat16, device="cuda").normal_(0, 1e-3, generator=g) for _ in range(4)]
    ref = torch.empty_like(srcs[0])
    comp.comp_reduce_n(O.BFLOAT16, O.SUM, srcs, ref, count, lp_mode=1)
    outs = [torch.empty_like(ref) for _ in range(4)]
    comp.comp_reduce_write_n(O.BFLOAT16, O.SUM, srcs, outs, count, lp_mode=1)
    torch.cuda.synchronize()
    for o in outs:
        assert torch.equal(o.view(torch.int16), ref.view(torch.int16))


def test_errors(comp):
    import torch
    a = torch.zeros(64, dtype=torch.float32, device="cuda")
    with pytest.raises(comp.CclError):
        comp.comp_reduce_write_n(O.FLOAT32, O.SUM, [a], [a] * 17, 64)
    with pytest.raises(comp.CclError):
        comp.comp_reduce_write_n(O.FLOAT32, 4, [a], [a], 64)
    with pytest.raises(comp.CclError):
        comp.comp_reduce_write_n(O.FLOAT32, O.SUM, [a], [a], 64, lp_mode=1)     # keep precision is for bf16
    comp.comp_reduce_write_n(O.FLOAT32, O.SUM, [a], [a, a], 0)                  # count 0: nothing to do


def test_automatic_kernel_choice_at_mid_and_large_sizes(comp):
    """No knob set: sizes on both sides of the crossovers between the per-N streaming kernel, the run-time-count
    streaming kernel (five and more inputs from 64 MB of traffic) and the phased kernel (from 240 MB with four and
    more inputs), with buffers that share a misalignment, against the oracle."""
    import torch
    rng = np.random.default_rng(77)
    assert comp.get_param("variant") == 0
    for dtype, n, count, shift in [(O.BFLOAT16, 8, 3_000_001, 3), (O.BFLOAT16, 8, 5_000_003, 0), (O.BFLOAT16, 6, 9_000_001, 5),
                                   (O.BFLOAT16, 8, 20_000_003, 1), (O.FLOAT32, 4, 9_000_002, 2), (O.FLOAT32, 4, 16_000_001, 0),
                                   (O.INT8, 5, 30_000_001, 7), (O.INT8, 5, 50_000_017, 0), (O.FLOAT16, 7, 12_000_005, 4)]:
        np_t = O.NP_STORAGE[dtype]
        srcs = make_inputs(rng, dtype, count, O.SUM, n)
        big = [to_dev(np.concatenate([np.zeros(shift, np_t), s])) for s in srcs]
        d = [b[shift:] for b in big]
        obig = torch.zeros(count + shift + 4, dtype=d[0].dtype, device="cuda")
        keep = 1 if dtype == O.BFLOAT16 else 0
        comp.comp_reduce_n(dtype, O.SUM, d, obig[shift:], count, lp_mode=keep)
        torch.cuda.synchronize()
        want = O.reduce_n(srcs, dtype, O.SUM, keep=keep, threads=8)
        got = to_host(obig, np_t)
        assert_same(got[shift:shift + count], want, dtype, f"{O.DTYPE_NAMES[dtype]} n={n} count={count} shift={shift}")
        assert not got[:shift].view(np.uint8).any() and not got[shift + count:].view(np.uint8).any()
