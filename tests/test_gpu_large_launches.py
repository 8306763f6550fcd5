"""Launches beyond what one HIP grid may hold (2^24 - 1 blocks of 256 lanes): the copy, the broadcast and the array
converters cut their work into several launches.  Checked with a small artificial limit (mi_ccl_set_param
"launch_block_limit") at ordinary sizes against the oracle, and at the real limit with a copy of more than 64 GiB and
a broadcast of a source of more than 10 GiB to seven destinations."""
import numpy as np
import pytest

import oracle_lib as O
from gpu_util import to_dev, to_host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def comp():
    import torch
    assert torch.cuda.is_available(), "needs a GPU"
    import oneccl_amd.comp as c
    c.lib()
    return c


@pytest.mark.parametrize("limit", [1, 3, 64])
def test_split_launches_with_a_small_limit(comp, limit):
    import torch
    rng = np.random.default_rng(31 + limit)
    comp.set_param("launch_block_limit", limit)
    try:
        for nbytes in (1, 17, 4096, 70_001, 1_000_003):
            for shift_in, shift_out in ((0, 0), (3, 3), (5, 2)):
                src = rng.integers(0, 256, nbytes + 32, dtype=np.uint8)
                d_src = to_dev(src)
                d_dst = to_dev(np.zeros(nbytes + 32, np.uint8))
                comp.comp_copy(d_src.data_ptr() + shift_in, d_dst.data_ptr() + shift_out, nbytes, use_nontemporal=True)
                outs = [to_dev(np.zeros(nbytes + 32, np.uint8)) for _ in range(3)]
                comp.comp_reduce_write_n(comp.UINT8, comp.SUM, [d_src.data_ptr() + shift_in],
                                         [o.data_ptr() + shift_out for o in outs], nbytes)
                torch.cuda.synchronize()
                for o in [d_dst] + outs:
                    g = to_host(o, np.uint8)
                    assert (g[shift_out:shift_out + nbytes] == src[shift_in:shift_in + nbytes]).all(), (nbytes, shift_in, shift_out)
                    assert not g[:shift_out].any() and not g[shift_out + nbytes:].any(), "wrote outside the destination"
        for count in (1, 15, 16, 17, 4099, 70_001, 1_000_003):
            for shift in (0, 1, 3):
                f = rng.standard_normal(count + 8).astype(np.float32)
                f[::97] = np.float32(1e-40)                    # denormals
                f.view(np.uint32)[5::89] = 0x7F812345          # signalling NaNs
                d_f = to_dev(f)
                for impl in (0, 1, 2):
                    d_h = to_dev(np.zeros(count + 8, np.uint16))
                    comp.convert_fp32_to_bf16_arrays(d_f.data_ptr() + 4 * shift, d_h.data_ptr() + 2 * shift, count, bf16_impl=impl)
                    torch.cuda.synchronize()
                    want = np.empty(count, np.uint16)
                    O.lib().orc_convert_fp32_to_bf16_arrays(f[shift:].ctypes.data, want.ctypes.data, count, impl)
                    g = to_host(d_h, np.uint16)
                    assert (g[shift:shift + count] == want).all(), ("fp32->bf16", count, shift, impl)
                    assert not g[:shift].any() and not g[shift + count:].any()
                d_h = to_dev(np.zeros(count + 8, np.uint16))
                comp.convert_fp32_to_fp16_arrays(d_f.data_ptr() + 4 * shift, d_h.data_ptr() + 2 * shift, count)
                torch.cuda.synchronize()
                want = np.empty(count, np.uint16)
                O.lib().orc_convert_fp32_to_fp16_arrays(f[shift:].ctypes.data, want.ctypes.data, count)
                g = to_host(d_h, np.uint16)
                assert (g[shift:shift + count] == want).all() and not g[:shift].any() and not g[shift + count:].any()
                h = rng.integers(0, 65536, count + 8, dtype=np.uint16)
                d_h = to_dev(h)
                for name, fn, orc in (("bf16", comp.convert_bf16_to_fp32_arrays, "orc_convert_bf16_to_fp32_arrays"),
                                      ("fp16", comp.convert_fp16_to_fp32_arrays, "orc_convert_fp16_to_fp32_arrays")):
                    d_o = to_dev(np.zeros(count + 8, np.uint32))
                    fn(d_h.data_ptr() + 2 * shift, d_o.data_ptr() + 4 * shift, count)
                    torch.cuda.synchronize()
                    want = np.empty(count, np.uint32)
                    if name == "bf16":
                        O.lib().orc_convert_bf16_to_fp32_arrays(h[shift:].ctypes.data, want.ctypes.data, count, 2)
                    else:
                        O.lib().orc_convert_fp16_to_fp32_arrays(h[shift:].ctypes.data, want.ctypes.data, count)
                    g = to_host(d_o, np.uint32)
                    assert (g[shift:shift + count] == want).all(), (name, count, shift)
                    assert not g[:shift].any() and not g[shift + count:].any()
    finally:
        comp.set_param("launch_block_limit", 0)


def test_copy_of_more_than_64_GiB(comp):
    """64 GiB + 4,099 bytes from a source 3 bytes off a 16-byte boundary: two launches at HIP's real limit."""
    import torch
    n = (64 << 30) + 4099
    words = (n + 3 + 7) // 8 + 1
    src = torch.arange(words, dtype=torch.int64, device="cuda").mul_(0x9E3779B97F4A7C15 - (1 << 64)).view(torch.uint8)
    dst = torch.zeros(words * 8, dtype=torch.uint8, device="cuda")
    comp.comp_copy(src.data_ptr() + 3, dst.data_ptr() + 3, n, use_nontemporal=True)
    torch.cuda.synchronize()
    for lo in range(3, 3 + n, 4 << 30):                  # in pieces: a comparison makes a byte per byte compared
        hi = min(3 + n, lo + (4 << 30))
        assert torch.equal(dst[lo:hi], src[lo:hi]), f"copy differs in bytes [{lo}, {hi})"
    assert int(dst[:3].count_nonzero()) == 0 and int(dst[3 + n:].count_nonzero()) == 0
    del dst
    # the widening converter beyond 2^32 values (64-bit indexing): at four values per lane that is 2^22 tiles, still ONE
    # launch -- a converter needs more than 2^34 values to reach HIP's limit of 2^24 - 1 blocks, so the cutting of
    # converter launches is exercised with the artificial launch_block_limit above and by the CPU geometry test only
    cnt = (1 << 32) + 4099
    h = src.view(torch.int16)[:cnt]
    f = torch.empty(cnt, dtype=torch.int32, device="cuda")
    comp.convert_bf16_to_fp32_arrays(h, f, cnt)
    torch.cuda.synchronize()
    for lo in range(0, cnt, 1 << 30):
        hi = min(cnt, lo + (1 << 30))
        assert torch.equal(f[lo:hi], h[lo:hi].to(torch.int32) << 16), f"widening differs in [{lo}, {hi})"


@pytest.mark.parametrize("pace", [7300, 0])
def test_broadcast_of_more_than_10_GiB_to_seven(comp, pace):
    """By the phased kernel with its clock-paced write phase (the default from two phases' worth of bytes), and, with
    the pace switched off, by the sectioned broadcast kernel, whose launches are cut at the block limit."""
    import torch
    n = (10 << 30) + 4099
    words = (n + 7) // 8 + 1
    src = torch.arange(words, dtype=torch.int64, device="cuda").mul_(0x9E3779B97F4A7C15 - (1 << 64)).view(torch.uint8)
    dsts = [torch.zeros(words * 8, dtype=torch.uint8, device="cuda") for _ in range(7)]
    comp.set_param("phase_write_pace", pace)
    try:
        comp.comp_reduce_write_n(comp.UINT8, comp.SUM, [src], dsts, n)
        torch.cuda.synchronize()
        assert comp.last_kernel() == ("reduce_multi_phased_kernel" if pace else "broadcast_kernel")
    finally:
        comp.set_param("phase_write_pace", 7300)
    for d in dsts:
        assert torch.equal(d[:n], src[:n])
        assert int(d[n:].count_nonzero()) == 0
