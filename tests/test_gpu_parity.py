"""GPU parity: the HIP path, called through the C ABI (ctypes binding oneccl_amd.comp), against the CPU oracle
and against the golden vectors made by the reference's own code.  Bit-exact for every type, NaN results of sum and
prod included (one NaN operand comes back quieted, an invalid operation gives the negative default NaN of x86); only
where a step of the chain meets two NaN operands do two NaNs compare equal whatever their payload (which of the two
the reference returns was its compiler's choice)."""
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
    c.lib()     # raises if the HIP library is missing: no fallback
    return c


def lp_variants(dtype):
    """(lp_mode, bf16_impl, oracle keep, oracle quirk) combinations that exist for a dtype."""
    if dtype == O.BFLOAT16:
        return [(0, 0, 0, 0), (0, 1, 0, 0), (0, 2, 0, 0), (1, 2, 1, 0), (1, 1, 1, 0), (3, 2, 1, 1), (3, 0, 1, 1)]
    return [(0, 2, 0, 0)]


COUNTS = [1, 7, 15, 16, 17, 33, 1000, 4099, 70001]


@pytest.mark.parametrize("dtype", range(12))
@pytest.mark.parametrize("op", range(4))
def test_reduce_n_all_dtypes_ops(comp, dtype, op):
    import torch
    rng = np.random.default_rng(1000 + dtype * 4 + op)
    for n in (1, 2, 3, 4, 5, 8, 9, 13):
        for count in COUNTS:
            if n > 8 and count not in (17, 4099, 70001):
                continue
            kinds = ["config", "bits"] if dtype in (O.FLOAT16, O.BFLOAT16) else ["config"]
            for kind in kinds:
                srcs = make_inputs(rng, dtype, count, op, n, kind)
                d = [to_dev(s) for s in srcs]
                for lp, impl, keep, quirk in lp_variants(dtype):
                    out = torch.empty_like(d[0])
                    comp.comp_reduce_n(dtype, op, d, out, count, lp_mode=lp, bf16_impl=impl)
                    torch.cuda.synchronize()
                    want = O.reduce_n(srcs, dtype, op, keep=keep, quirk_tail=quirk, bf16_impl=impl)
                    assert_same(to_host(out, O.NP_STORAGE[dtype]), want, dtype,
                                f"dtype={O.DTYPE_NAMES[dtype]} op={O.OP_NAMES[op]} n={n} count={count} "
                                f"kind={kind} lp={lp} impl={impl}", srcs, op, keep=keep, bf16_impl=impl)


@pytest.mark.parametrize("dtype,op", [(O.BFLOAT16, O.SUM), (O.INT8, O.MIN), (O.FLOAT64, O.PROD), (O.UINT16, O.MAX)])
def test_reduce_n_many_inputs(comp, dtype, op):
    """17 to 64 inputs (the most one call takes): the elements in front of the first and behind the last vector are
    folded eight inputs at a time, so these counts leave one, two and no input over, in the streaming and in the phased
    kernel, with the buffers two elements off their holders' boundary."""
    import torch
    rng = np.random.default_rng(5200 + dtype * 4 + op)
    np_t = O.NP_STORAGE[dtype]
    keep = 1 if dtype == O.BFLOAT16 else 0
    for n in (17, 18, 25, 33, 64):
        for count in (5, 4099, 70001):
            srcs = make_inputs(rng, dtype, count, op, n)
            holders = [to_dev(np.concatenate([np.zeros(2, np_t), s_])) for s_ in srcs]
            want = O.reduce_n(srcs, dtype, op, keep=keep)
            for variant in (0, 8):
                out = to_dev(np.zeros(count + 4, np_t))
                comp.set_param("variant", variant)
                try:
                    comp.comp_reduce_n(dtype, op, [h[2:] for h in holders], out[2:], count, lp_mode=keep)
                    torch.cuda.synchronize()
                finally:
                    comp.set_param("variant", 0)
                g = to_host(out, np_t)
                assert_same(g[2:2 + count], want, dtype, f"n={n} count={count} variant={variant}", srcs, op, keep=keep)
                assert not g[:2].view(np.uint8).any() and not g[2 + count:].view(np.uint8).any(), "wrote outside"
    with pytest.raises(comp.CclError):
        comp.comp_reduce_n(dtype, op, [holders[0]] * 65, out, 5, lp_mode=keep)


@pytest.mark.parametrize("dtype", range(12))
def test_phased_reduce_with_the_wider_phase(comp, dtype):
    """Results of 88 to 96 MiB take one phase when a lane keeps four more vectors in registers (two phases otherwise),
    and the library then launches that form of the phased kernel: every element type and 16-bit mode, two inputs (and
    eight for bfloat16), against the oracle over every element."""
    import torch
    rng = np.random.default_rng(8800 + dtype)
    esz = O.DTYPE_SIZE[dtype]
    assert comp.get_param("num_cus") == 256, "sizes below are for 256 CUs"
    count = (92 << 20) // esz + 3
    op = (O.SUM, O.MAX, O.PROD, O.MIN)[dtype % 4]
    for n in ((2, 8) if dtype == O.BFLOAT16 else (2,)):
        srcs = make_inputs(rng, dtype, count, op, n)
        d = [to_dev(s) for s in srcs]
        for lp, impl, keep, quirk in lp_variants(dtype):
            if quirk:
                continue
            out = torch.empty_like(d[0])
            wide = comp.get_param("wide_phase_launches")
            comp.comp_reduce_n(dtype, op, d, out, count, lp_mode=lp, bf16_impl=impl)
            torch.cuda.synchronize()
            assert comp.last_kernel() == "reduce_multi_phased_kernel" and comp.get_param("wide_phase_launches") == wide + 1
            want = O.reduce_n(srcs, dtype, op, keep=keep, bf16_impl=impl, threads=16)
            assert_same(to_host(out, O.NP_STORAGE[dtype]), want, dtype, f"n={n} lp={lp} impl={impl}", srcs, op, keep=keep, bf16_impl=impl)
        if dtype == O.FLOAT16:      # the avx512fp16 implementation is a kernel family of its own
            out = torch.empty_like(d[0])
            comp.comp_reduce_n(dtype, op, d, out, count, fp16_impl=comp.FP16_AVX512FP16)
            torch.cuda.synchronize()
            want = O.reduce_n(srcs, dtype, op, fp16_impl=O.FP16_AVX512FP16, threads=16)
            assert_same(to_host(out, O.NP_STORAGE[dtype]), want, dtype, f"n={n} native fp16", srcs, op, fp16_impl=O.FP16_AVX512FP16)
        del d
    # 80 MiB is one phase either way, 1 GiB twelve against eleven: the usual form
    wide = comp.get_param("wide_phase_launches")
    small = (80 << 20) // esz
    a, b = to_dev(np.zeros(small, O.NP_STORAGE[dtype])), to_dev(np.zeros(small, O.NP_STORAGE[dtype]))
    comp.comp_reduce_n(dtype, O.MAX, [a, b], a, small)
    torch.cuda.synchronize()
    assert comp.get_param("wide_phase_launches") == wide


@pytest.mark.parametrize("fam,dtype", [("bf16", O.BFLOAT16), ("fp16", O.FLOAT16)])
def test_pairwise_against_reference_made_golden_vectors(comp, golden, fam, dtype):
    """GPU result vs what the reference's ccl_bf16_reduce_impl_* / ccl_fp16_reduce_impl_* produced."""
    import torch
    impls = (1, 2) if fam == "bf16" else (3,)
    checked = 0
    for key in golden.files:
        if not key.startswith(fam + "_") or not key.endswith("_in") or key.startswith("cvt"):
            continue
        stem = key[:-3]
        if "specials" in stem:
            continue
        op = O.OP_NAMES.index(stem.split("_")[1])
        a, b = golden[stem + "_in"], golden[stem + "_inout"]
        for impl in impls:
            da, db = to_dev(a), to_dev(b)
            comp.comp_reduce(dtype, op, da, a.size, db, bf16_impl=impl if fam == "bf16" else 2)
            torch.cuda.synchronize()
            assert_same(to_host(db, np.uint16), golden[stem + f"_impl{impl}"], dtype, f"{stem} impl{impl}", [b, a], op,
                        bf16_impl=impl if fam == "bf16" else 2)
            checked += 1
    assert checked >= 4 * 11 * 2


@pytest.mark.parametrize("fam,dtype", [("bf16", O.BFLOAT16), ("fp16", O.FLOAT16)])
def test_special_value_pairs_against_golden(comp, golden, fam, dtype):
    """Every pair of special values (zeros, denormals, infinities, quiet and signalling NaNs, extremes).
    min/max must return the reference's operand bit for bit, NaN payloads included."""
    import torch
    impls = (1, 2) if fam == "bf16" else (3,)
    a, b = golden[f"{fam}_specials_in"], golden[f"{fam}_specials_inout"]
    for op in range(4):
        for impl in impls:
            da, db = to_dev(a), to_dev(b)
            comp.comp_reduce(dtype, op, da, a.size, db, bf16_impl=impl if fam == "bf16" else 2)
            torch.cuda.synchronize()
            got = to_host(db, np.uint16)
            want = golden[f"{fam}_specials_{O.OP_NAMES[op]}_impl{impl}"]
            if op in (O.MIN, O.MAX):
                assert (got == want).all(), (fam, op, impl, np.flatnonzero(got != want)[:8])
            else:
                assert_same(got, want, dtype, f"{fam} specials op={op} impl={impl}", [b, a], op,
                            bf16_impl=impl if fam == "bf16" else 2)
    if fam == "bf16":   # scalar impl has no golden (not vector code): oracle, pinned by the recorded probes
        for op in range(4):
            da, db = to_dev(a), to_dev(b)
            comp.comp_reduce(dtype, op, da, a.size, db, bf16_impl=0)
            torch.cuda.synchronize()
            want = O.comp_reduce(a, b, dtype, op, bf16_impl=0)
            got = to_host(db, np.uint16)
            if op in (O.MIN, O.MAX):
                assert (got == want).all()
            else:
                assert_same(got, want, dtype, f"bf16 specials op={op} scalar", [b, a], op, bf16_impl=0)


def test_recorded_probe_values_on_gpu(comp, probes):
    """The known answers recorded from the real reference library, reproduced by the GPU path."""
    import torch
    hx = lambda s: np.uint16(int(s, 16))
    p = probes["bf16_pairwise_sum"]
    a = np.array([hx(x) for x in p["in"]], np.uint16)
    for name, impl in (("scalar", 0), ("avx512f", 1), ("avx512bf", 2)):
        db = to_dev(np.full(a.size, hx(p["inout"]), np.uint16))
        comp.bf16_reduce(to_dev(a), a.size, db, O.SUM, bf16_impl=impl)
        torch.cuda.synchronize()
        assert [f"{v:04x}" for v in to_host(db, np.uint16)] == p[name]
    p = probes["batch_reduce_bf16"]
    cnt = p["count"]
    buf = np.concatenate([np.full(cnt, hx(s), np.uint16) for s in p["slices"]])
    offs = [i * cnt for i in range(4)]
    d = to_dev(buf)
    comp.comp_batch_reduce(d, offs, cnt, d, O.BFLOAT16, O.SUM, 1, bf16_impl=2)
    torch.cuda.synchronize()
    r = to_host(d, np.uint16)[:cnt]
    assert all(f"{v:04x}" == p["keep_precision_1_body"] for v in r[:16]) and f"{r[16]:04x}" == p["keep_precision_1_tail"]
    d = to_dev(buf)
    comp.comp_batch_reduce(d, offs, cnt, d, O.BFLOAT16, O.SUM, 0, bf16_impl=2)
    torch.cuda.synchronize()
    assert all(f"{v:04x}" == p["keep_precision_0"] for v in to_host(d, np.uint16)[:cnt])
    p = probes["fp16_pairwise_sum"]
    a = np.array([hx(x) for x in p["in"]], np.uint16)
    db = to_dev(np.array([hx(x) for x in p["inout"]], np.uint16))
    comp.fp16_reduce(to_dev(a), a.size, db, O.SUM)
    torch.cuda.synchronize()
    assert [f"{v:04x}" for v in to_host(db, np.uint16)] == p["avx512f"]
    for c in probes["int_wrap"]["cases"]:
        dt = O.DTYPE_NAMES.index(c["dtype"])
        np_t = O.NP_STORAGE[dt]
        db = to_dev(np.array([c["inout"]] * 5, np_t))
        comp.comp_reduce(dt, O.SUM, to_dev(np.array([c["in"]] * 5, np_t)), 5, db)
        torch.cuda.synchronize()
        assert (to_host(db, np_t) == np_t(c["out"])).all()
    vals = {"nan": np.nan, "1": 1.0, "-0": -0.0, "+0": 0.0}
    for dt, np_t in ((O.FLOAT32, np.float32), (O.FLOAT64, np.float64)):
        for c in probes["fp_minmax_plain"]["cases"]:
            db = to_dev(np.full(67, vals[c["inout"]], np_t))
            comp.comp_reduce(dt, O.OP_NAMES.index(c["op"]), to_dev(np.full(67, vals[c["in"]], np_t)), 67, db)
            torch.cuda.synchronize()
            got = to_host(db, np_t)
            w = np_t(vals[c["out"]])
            assert (np.isnan(got).all() if np.isnan(w) else ((got == w).all() and (np.signbit(got) == np.signbit(w)).all())), c


@pytest.mark.parametrize("dtype", [O.INT8, O.INT16, O.FLOAT32, O.FLOAT64, O.BFLOAT16, O.FLOAT16])
def test_misaligned_and_inplace(comp, dtype):
    """Buffers that share a misalignment modulo 16 bytes (head/tail lanes), buffers that do not (loose vector
    accesses), in-place output, output aliasing a later input."""
    import torch
    rng = np.random.default_rng(77 + dtype)
    esz = O.DTYPE_SIZE[dtype]
    np_t = O.NP_STORAGE[dtype]
    count, n, pad = 5003, 4, 32
    for op in (O.SUM, O.MAX):
        srcs = make_inputs(rng, dtype, count, op, n)
        want = O.reduce_n(srcs, dtype, op)
        for shifts in ([3, 3, 3, 3, 3], [1, 1, 1, 1, 1], [0, 1, 2, 3, 5], [0, 0, 0, 0, 1]):
            # payload j starts shifts[j] elements past a 16-byte boundary (pad elements are a multiple of 16 B)
            big = []
            for s_, sh in zip(srcs, shifts):
                h = np.zeros(count + 2 * pad, np_t)
                h[pad + sh:pad + sh + count] = s_
                big.append(to_dev(h))
            outbig = to_dev(np.zeros(count + 2 * pad, np_t))
            ptrs = [b_.data_ptr() + (pad + sh) * esz for b_, sh in zip(big, shifts)]
            lo = pad + shifts[4]
            comp.comp_reduce_n(dtype, op, ptrs, outbig.data_ptr() + lo * esz, count)
            torch.cuda.synchronize()
            o = to_host(outbig, np_t)
            assert_same(o[lo:lo + count], want, dtype, f"shifts={shifts}", srcs, op)
            assert (o[:lo] == 0).all() and (o[lo + count:] == 0).all(), "wrote outside the destination"
        d = [to_dev(s) for s in srcs]
        comp.comp_reduce_n(dtype, op, d, d[0], count)          # in place on the own buffer
        torch.cuda.synchronize()
        assert_same(to_host(d[0], np_t), want, dtype, "in place", srcs, op)
        d = [to_dev(s) for s in srcs]
        comp.comp_reduce_n(dtype, op, d, d[2], count)          # output aliases a later input
        torch.cuda.synchronize()
        assert_same(to_host(d[2], np_t), want, dtype, "alias", srcs, op)


def test_batch_reduce_slices_keep_precision_tail(comp):
    import torch
    rng = np.random.default_rng(5)
    for count in (1, 15, 16, 17, 31, 100, 1000, 4112 + 9):
        for n in (1, 2, 4, 8):
            for op in range(4):
                slices = make_inputs(rng, O.BFLOAT16, count, op, n)
                gap = 24
                buf = np.zeros(n * (count + gap), np.uint16)
                offs = [i * (count + gap) for i in range(n)]
                for s, o in zip(slices, offs):
                    buf[o:o + count] = s
                for keep in (0, 1):
                    for impl in (0, 1, 2):
                        d = to_dev(buf)
                        comp.comp_batch_reduce(d, offs, count, d, O.BFLOAT16, op, keep, bf16_impl=impl)
                        torch.cuda.synchronize()
                        want = O.batch_reduce(buf, offs, count, O.BFLOAT16, op, keep, bf16_impl=impl)
                        got = to_host(d, np.uint16)
                        what = f"count={count} n={n} op={op} keep={keep} impl={impl}"
                        assert_same(got[:count], want[:count], O.BFLOAT16, what, slices, op, keep=keep, bf16_impl=impl)
                        assert (got[count:] == want[count:]).all(), what + ": the other slices changed"


def test_copy_and_converters(comp):
    import torch
    rng = np.random.default_rng(9)
    for nbytes in (1, 15, 16, 17, 4096, 100003, 1 << 20):
        for sa, sb in ((0, 0), (3, 3), (1, 2), (8, 0)):
            src = rng.integers(0, 256, nbytes + 64, dtype=np.uint8)
            for nt in (False, True):
                ds, dd = to_dev(src), to_dev(np.zeros(nbytes + 64, np.uint8))
                comp.comp_copy(ds.data_ptr() + sa, dd.data_ptr() + sb, nbytes, use_nontemporal=nt)
                torch.cuda.synchronize()
                got = to_host(dd, np.uint8)
                assert (got[sb:sb + nbytes] == src[sa:sa + nbytes]).all()
                assert (got[:sb] == 0).all() and (got[sb + nbytes:] == 0).all()
    # a large copy with head and tail bytes (one 4 KiB tile per block: a few hundred thousand blocks)
    nbytes = (2400 << 20) + 5
    src_d = torch.randint(-128, 127, (nbytes + 32,), dtype=torch.int8, device="cuda")
    dst_d = torch.zeros(nbytes + 32, dtype=torch.int8, device="cuda")
    comp.comp_copy(src_d.data_ptr() + 3, dst_d.data_ptr() + 19, nbytes, use_nontemporal=True)
    torch.cuda.synchronize()
    assert torch.equal(dst_d[19:19 + nbytes], src_d[3:3 + nbytes])
    assert int(dst_d[:19].count_nonzero()) == 0 and int(dst_d[19 + nbytes:].count_nonzero()) == 0
    del dst_d, src_d
    L = O.lib()
    for count in (1, 5, 16, 22, 1000, 65536 + 7):
        f32 = rng.integers(0, 2**32, count, dtype=np.uint32)
        f32[:min(count, 6)] = np.array([1, 0x007FFFFF, 0x7FC00000, 0x7F800001, 0x7F7FFFFF, 0x3F808000], np.uint32)[:min(count, 6)]
        if count >= 22:
            f32[16:22] = f32[:6]
        for impl in (0, 1, 2):
            want = np.empty(count, np.uint16)
            L.orc_convert_fp32_to_bf16_arrays(f32.ctypes.data, want.ctypes.data, count, impl)
            d = to_dev(np.zeros(count, np.uint16))
            comp.convert_fp32_to_bf16_arrays(to_dev(f32), d, count, bf16_impl=impl)
            torch.cuda.synchronize()
            assert (to_host(d, np.uint16) == want).all(), (count, impl)
        h = rng.integers(0, 65536, count, dtype=np.uint16)
        d = to_dev(np.zeros(count, np.uint32))
        comp.convert_bf16_to_fp32_arrays(to_dev(h), d, count)
        torch.cuda.synchronize()
        assert (to_host(d, np.uint32) == (h.astype(np.uint32) << 16)).all()
    # the two arrays at different offsets from a 16-byte boundary (the input is read as loose vectors), sizes from
    # less than one group of eight to many blocks; nothing outside the output is written
    for count in (3, 8, 29, 70_001, 3_000_019):
        for si, so in ((0, 0), (1, 0), (0, 1), (3, 5), (2, 7)):
            f32 = rng.integers(0, 2**32, count + 16, dtype=np.uint32)
            for impl in (1, 2):
                want = np.empty(count, np.uint16)
                L.orc_convert_fp32_to_bf16_arrays(f32[si:].ctypes.data, want.ctypes.data, count, impl)
                d, src_d = to_dev(np.zeros(count + 16, np.uint16)), to_dev(f32)
                comp.convert_fp32_to_bf16_arrays(src_d.data_ptr() + 4 * si, d.data_ptr() + 2 * so, count, bf16_impl=impl)
                torch.cuda.synchronize()
                got = to_host(d, np.uint16)
                assert (got[so:so + count] == want).all(), (count, si, so, impl)
                assert not got[:so].any() and not got[so + count:].any(), (count, si, so, impl)
            h = rng.integers(0, 65536, count + 16, dtype=np.uint16)
            d, src_d = to_dev(np.zeros(count + 16, np.uint32)), to_dev(h)
            comp.convert_bf16_to_fp32_arrays(src_d.data_ptr() + 2 * si, d.data_ptr() + 4 * so, count)
            torch.cuda.synchronize()
            got = to_host(d, np.uint32)
            assert (got[so:so + count] == (h[si:si + count].astype(np.uint32) << 16)).all(), (count, si, so)
            assert not got[:so].any() and not got[so + count:].any(), (count, si, so)


def test_fp16_converters_exhaustive_on_gpu(comp):
    """fp32 -> fp16 for all 2^32 patterns and fp16 -> fp32 for all 2^16, against the oracle (itself exhaustively equal
    to VCVTPS2PH imm 0 / VCVTPH2PS, which the reference's ccl_convert_fp32_to_fp16 / ccl_convert_fp16_to_fp32 are);
    then both directions with the two arrays at different alignments and odd counts."""
    import torch
    L = O.lib()
    chunk = 1 << 27
    d_out = torch.empty(chunk, dtype=torch.int16, device="cuda")
    want = np.empty(chunk, np.uint16)
    for c in range(0, 1 << 32, chunk):
        x = torch.arange(c, c + chunk, dtype=torch.int64, device="cuda")
        src = torch.where(x >= 2**31, x - 2**32, x).to(torch.int32)
        comp.convert_fp32_to_fp16_arrays(src, d_out, chunk)
        torch.cuda.synchronize()
        host = np.arange(c, c + chunk, dtype=np.uint64).astype(np.uint32)
        L.orc_convert_fp32_to_fp16_arrays(host.ctypes.data, want.ctypes.data, chunk)
        got = to_host(d_out, np.uint16)
        assert (got == want).all(), hex(c + int(np.flatnonzero(got != want)[0]))
    h = np.arange(65536, dtype=np.uint16)
    w = np.empty(65536, np.uint32)
    L.orc_convert_fp16_to_fp32_arrays(h.ctypes.data, w.ctypes.data, 65536)
    d = to_dev(np.zeros(65536, np.uint32))
    comp.convert_fp16_to_fp32_arrays(to_dev(h), d, 65536)
    torch.cuda.synchronize()
    assert (to_host(d, np.uint32) == w).all()
    rng = np.random.default_rng(23)
    for count in (1, 7, 8, 29, 70_001):
        for si, so in ((0, 0), (1, 3), (3, 6)):
            f32 = rng.integers(0, 2**32, count + 16, dtype=np.uint32)
            want = np.empty(count, np.uint16)
            L.orc_convert_fp32_to_fp16_arrays(f32[si:].ctypes.data, want.ctypes.data, count)
            d, src_d = to_dev(np.zeros(count + 16, np.uint16)), to_dev(f32)
            comp.convert_fp32_to_fp16_arrays(src_d.data_ptr() + 4 * si, d.data_ptr() + 2 * so, count)
            torch.cuda.synchronize()
            got = to_host(d, np.uint16)
            assert (got[so:so + count] == want).all() and not got[:so].any() and not got[so + count:].any(), (count, si, so)
            h16 = rng.integers(0, 65536, count + 16, dtype=np.uint16)
            want32 = np.empty(count, np.uint32)
            L.orc_convert_fp16_to_fp32_arrays(h16[si:].ctypes.data, want32.ctypes.data, count)
            d, src_d = to_dev(np.zeros(count + 16, np.uint32)), to_dev(h16)
            comp.convert_fp16_to_fp32_arrays(src_d.data_ptr() + 2 * si, d.data_ptr() + 4 * so, count)
            torch.cuda.synchronize()
            got = to_host(d, np.uint32)
            assert (got[so:so + count] == want32).all() and not got[:so].any() and not got[so + count:].any(), (count, si, so)


def test_bf16_narrowing_exhaustive_on_gpu(comp):
    """All 2^32 fp32 patterns through the GPU's round-to-nearest-even narrowing vs the oracle (itself
    exhaustively equal to VCVTNEPS2BF16).  The kernel converts pairs with the packed hardware conversion, so every
    pattern is sent twice: once at an even index (low half of the pair) and once at an odd one (high half)."""
    import torch
    L = O.lib()
    chunk = 1 << 27
    d_out = torch.empty(chunk, dtype=torch.int16, device="cuda")
    want = np.empty(chunk, np.uint16)
    for shift in (0, 1):
        for c in range(0, 1 << 32, chunk):
            x = (torch.arange(c, c + chunk, dtype=torch.int64, device="cuda") + shift) & 0xFFFFFFFF
            src = torch.where(x >= 2**31, x - 2**32, x).to(torch.int32)      # the fp32 bit pattern as int32
            comp.convert_fp32_to_bf16_arrays(src, d_out, chunk, bf16_impl=2)
            torch.cuda.synchronize()
            host = ((np.arange(c, c + chunk, dtype=np.uint64) + shift) & 0xFFFFFFFF).astype(np.uint32)
            L.orc_convert_fp32_to_bf16_arrays(host.ctypes.data, want.ctypes.data, chunk, 2)
            got = to_host(d_out, np.uint16)
            assert (got == want).all(), (shift, hex(c + int(np.flatnonzero(got != want)[0])))


@pytest.mark.parametrize("dtype,impl", [(O.FLOAT16, 3), (O.BFLOAT16, 2)])
def test_all_pairs_of_16bit_values_sum_and_prod(comp, dtype, impl):
    """Every (in, inout) pair of 16-bit patterns -- 2^32 pairs -- through the pairwise GPU kernel."""
    import torch
    allv = np.arange(65536, dtype=np.uint16)
    rows = 512
    a = np.tile(allv, rows)
    da = to_dev(a)
    for op in (O.SUM, O.PROD):
        for r0 in range(0, 65536, rows):
            b = np.repeat(allv[r0:r0 + rows], 65536)
            db = to_dev(b)
            comp.comp_reduce(dtype, op, da, a.size, db, bf16_impl=2)
            torch.cuda.synchronize()
            want = O.reduce_n([b, a], dtype, op, bf16_impl=impl, fp16_impl=3, threads=16)
            assert_same(to_host(db, np.uint16), want, dtype, f"op={op} rows from {r0}", [b, a], op, bf16_impl=impl, fp16_impl=3)


@pytest.mark.parametrize("dtype", [O.INT16, O.UINT16])
def test_all_pairs_of_16bit_integers_sum_and_prod(comp, dtype):
    """Every (in, inout) pair of 16-bit integer patterns -- 2^32 pairs -- through the GPU kernel: the wrapped sum and
    product (65535 x 65535 overflows a signed int, so both sides multiply in unsigned).  Every pair is checked on the
    GPU against the closed form in torch's wrapping 32-bit integer arithmetic, which shares no code with the kernels
    or the oracle; a sample of rows (the extremes among them) also against the oracle."""
    import torch
    np_t = O.NP_STORAGE[dtype]
    rows = 2048
    allv = torch.arange(65536, dtype=torch.int32, device="cuda")
    a32 = allv.repeat(rows)                                     # in: every value, `rows` times over
    da = a32.to(torch.int16)                                    # keeps the low 16 bits
    for op in (O.SUM, O.PROD):
        for r0 in range(0, 65536, rows):
            b32 = allv[r0:r0 + rows].repeat_interleave(65536)   # inout: one value per row
            db = b32.to(torch.int16)
            comp.comp_reduce(dtype, op, da, da.numel(), db)
            torch.cuda.synchronize()
            closed = ((b32 + a32) if op == O.SUM else (b32 * a32)).to(torch.int16)      # modulo 2^32, then modulo 2^16
            assert torch.equal(db, closed), (dtype, op, r0, "closed form")
            if r0 in (0, 32768 - rows, 32768, 65536 - rows):
                for r in (0, rows - 1):
                    b = np.full(65536, r0 + r, np.uint16).view(np_t)
                    a = np.arange(65536, dtype=np.uint16).view(np_t)
                    want = O.reduce_n([b, a], dtype, op)
                    got = db[r * 65536:(r + 1) * 65536].cpu().numpy().view(np.uint16)
                    assert (got == want.view(np.uint16)).all(), (dtype, op, r0 + r, "oracle")


def test_arguments_and_errors(comp):
    import torch
    L = comp.lib()
    assert comp.datatype_size(O.BFLOAT16) == 2 and comp.datatype_size(99) == 0
    assert [comp.datatype_name(i) for i in range(12)] == O.DTYPE_NAMES
    assert [comp.reduction_to_str(i) for i in range(6)] == ["sum", "prod", "min", "max", "custom", "unknown"]
    assert comp.kernel_name("reduce_monolithic_kernel_7", O.BFLOAT16, O.SUM) == "reduce_monolithic_kernel_7_bfloat16_sum"
    # count 0 succeeds without touching pointers (comp.cpp:132-134), even with a bad dtype
    assert L.mi_ccl_comp_reduce(99, 0, None, 0, None, 2, 0, None) == 0
    x = torch.zeros(64, dtype=torch.int32, device="cuda")
    assert L.mi_ccl_comp_reduce(99, 0, x.data_ptr(), 4, x.data_ptr(), 2, 0, None) == comp.INVALID_ARGUMENTS
    assert L.mi_ccl_comp_reduce(O.INT32, 4, x.data_ptr(), 4, x.data_ptr(), 2, 0, None) == comp.INVALID_ARGUMENTS  # custom
    assert L.mi_ccl_comp_reduce(O.INT32, 0, None, 4, x.data_ptr(), 2, 0, None) == comp.INVALID_ARGUMENTS
    assert L.mi_ccl_comp_reduce(O.INT32, 0, x.data_ptr() + 2, 4, x.data_ptr(), 2, 0, None) == comp.INVALID_ARGUMENTS
    with pytest.raises(comp.CclError):
        comp.comp_reduce_n(O.FLOAT32, O.SUM, [x], x, 4, lp_mode=comp.LP_KEEP_PRECISION)   # keep needs bfloat16
    with pytest.raises(comp.CclError):
        comp.comp_reduce_n(O.INT32, O.SUM, [x] * 65, x, 4)
    for bad in (1, 5, -1):          # fp16_impl: 0 (the default), 2, 3 or 4
        assert L.mi_ccl_comp_reduce(O.FLOAT16, 0, x.data_ptr(), 4, x.data_ptr(), 2, bad, None) == comp.INVALID_ARGUMENTS
    torch.cuda.synchronize()
    assert (x == 0).all()


@pytest.mark.parametrize("dtype,op,n", [(O.BFLOAT16, O.SUM, 8), (O.FLOAT32, O.SUM, 4), (O.INT8, O.SUM, 4),
                                        (O.FLOAT16, O.SUM, 4), (O.INT64, O.MAX, 4), (O.FLOAT64, O.PROD, 2),
                                        (O.FLOAT32, O.MIN, 3)])
def test_phased_kernel_parity(comp, dtype, op, n):
    """The large-buffer kernel (read phase into LDS / write phase, blocks aligned by a timing-only barrier)
    forced on at sizes from a few elements to several phases, aligned and with head/tail lanes."""
    import torch
    rng = np.random.default_rng(300 + dtype)
    esz = O.DTYPE_SIZE[dtype]
    per_phase = comp.get_param("num_cus") * 512 * 20 * (16 // esz)      # elements one phase covers
    comp.set_param("variant", 8)
    try:
        for count, shift in ((5, 0), (1000, 1), (per_phase // 3 + 7, 0), (5 * per_phase + 12345, 3)):
            if count * esz * (n + 1) > 6 << 30:
                count = (6 << 30) // (esz * (n + 1))
            srcs = make_inputs(rng, dtype, count + shift, op, n)
            d = [to_dev(s) for s in srcs]
            out = torch.zeros_like(d[0])
            ptrs = [t.data_ptr() + shift * esz for t in d]
            comp.comp_reduce_n(dtype, op, ptrs, out.data_ptr() + shift * esz, count,
                               lp_mode=comp.LP_KEEP_PRECISION if dtype == O.BFLOAT16 else 0)
            torch.cuda.synchronize()
            want = O.reduce_n([s[shift:] for s in srcs], dtype, op, keep=1 if dtype == O.BFLOAT16 else 0, threads=16)
            got = to_host(out, O.NP_STORAGE[dtype])
            assert_same(got[shift:], want, dtype, f"phased count={count} shift={shift}", [s[shift:] for s in srcs], op,
                        keep=1 if dtype == O.BFLOAT16 else 0)
            assert (got[:shift] == 0).all()
    finally:
        comp.set_param("variant", 0)


@pytest.mark.parametrize("dtype,op,n,m", [(O.BFLOAT16, O.SUM, 8, 1), (O.FLOAT32, O.SUM, 2, 1), (O.INT32, O.MAX, 1, 1),
                                          (O.FLOAT16, O.SUM, 3, 2), (O.INT8, O.SUM, 16, 1)])
def test_phased_kernel_early_arrival_settings(comp, dtype, op, n, m):
    """A block of the phased kernel reports its arrival at the chip-wide barrier a few loads / stores before it is done
    ("phase_early_loads", "phase_early_stores").  The barrier aligns the blocks in time only, so every setting, from
    "when done" to "before the first staged load", must give the oracle's bits: three full phases and a partial one."""
    import torch
    rng = np.random.default_rng(900 + dtype + n)
    esz = O.DTYPE_SIZE[dtype]
    keep = 1 if dtype == O.BFLOAT16 else 0
    per_phase = comp.get_param("num_cus") * 512 * 44 * (16 // esz)      # elements one phase covers
    count = 3 * per_phase + per_phase // 5 + 3
    srcs = make_inputs(rng, dtype, count, op, n)
    want = O.reduce_n(srcs, dtype, op, keep=keep, threads=16)
    d = [to_dev(s) for s in srcs]
    assert comp.get_param("phase_early_loads") == -1 and comp.get_param("phase_early_stores") == -1
    comp.set_param("variant", 8)
    try:
        for loads, stores in ((-1, -1), (12, -1), (0, 0), (4, 20), (1000, 1), (4096, 7), (13, 19)):
            comp.set_param("phase_early_loads", loads)
            comp.set_param("phase_early_stores", stores)
            outs = [torch.zeros_like(d[0]) for _ in range(m)]
            comp.comp_reduce_write_n(dtype, op, d, outs, count, lp_mode=comp.LP_KEEP_PRECISION if keep else 0)
            torch.cuda.synchronize()
            assert comp.last_kernel() == "reduce_multi_phased_kernel"
            for o in outs:
                assert_same(to_host(o, O.NP_STORAGE[dtype]), want, dtype, f"early loads {loads} stores {stores}", srcs, op,
                            keep=keep)
        for bad in (("phase_early_loads", -2), ("phase_early_loads", 4097), ("phase_early_stores", -2), ("phase_early_stores", 21)):
            with pytest.raises(comp.CclError):
                comp.set_param(*bad)
    finally:
        comp.set_param("variant", 0)
        comp.set_param("phase_early_loads", -1)
        comp.set_param("phase_early_stores", -1)


def test_grid_cap_keeps_the_streaming_kernels(comp):
    """"max_blocks" caps the grid for callers that want CUs left free; the phased kernels take one block on every CU, so
    while a cap is set a large reduce stays with the (grid-striding) streaming kernels -- same bits either way."""
    import torch
    rng = np.random.default_rng(78)
    count = 40 << 20                 # 8 x 80 MiB of bf16: phased without a cap
    srcs = make_inputs(rng, O.BFLOAT16, count, O.SUM, 8)
    want = O.reduce_n(srcs, O.BFLOAT16, O.SUM, keep=1, threads=16)
    d = [to_dev(s) for s in srcs]
    try:
        for cap, kernel in ((0, "reduce_multi_phased_kernel"), (64, "reduce_multi_kernel"), (1, "reduce_multi_kernel")):
            comp.set_param("max_blocks", cap)
            out = torch.zeros_like(d[0])
            comp.comp_reduce_n(O.BFLOAT16, O.SUM, d, out, count, lp_mode=comp.LP_KEEP_PRECISION)
            torch.cuda.synchronize()
            assert comp.last_kernel() == kernel, (cap, comp.last_kernel())
            assert_same(to_host(out, np.uint16), want, O.BFLOAT16, f"grid cap {cap}", srcs, O.SUM, keep=1)
    finally:
        comp.set_param("max_blocks", 0)


def test_phased_kernel_when_no_block_waits(comp):
    """The bound on a block's wait at the chip-wide barrier set to zero from the host: every block goes on alone after
    its first poll, the phases of different blocks overlap freely, and the result is still the oracle's (the barrier
    carries no data).  Every block still reports all its arrivals, so the launches that follow, with the default
    bound again, find the barrier words consistent and give the same bits."""
    import torch
    rng = np.random.default_rng(77)
    dtype, n = O.BFLOAT16, 8
    per_phase = comp.get_param("num_cus") * 512 * 44 * 8
    count = 4 * per_phase + 12345
    srcs = make_inputs(rng, dtype, count, O.SUM, n)
    want = O.reduce_n(srcs, dtype, O.SUM, keep=1, threads=16)
    d = [to_dev(s) for s in srcs]
    assert comp.get_param("phase_spin_ticks") == 20000
    comp.set_param("variant", 8)
    try:
        for ticks in (0, 0, 20000, 20000):
            comp.set_param("phase_spin_ticks", ticks)
            out = torch.zeros_like(d[0])
            for _ in range(17):         # more calls than there are sets of barrier words: every set is used both ways
                comp.comp_reduce_n(dtype, O.SUM, d, out, count, lp_mode=comp.LP_KEEP_PRECISION)
            torch.cuda.synchronize()
            assert comp.last_kernel() == "reduce_multi_phased_kernel"
            assert_same(to_host(out, np.uint16), want, dtype, f"wait bound {ticks} ticks", srcs, O.SUM, keep=1)
    finally:
        comp.set_param("variant", 0)
        comp.set_param("phase_spin_ticks", 20000)


@pytest.mark.parametrize("variant", [0, 1, 8])
@pytest.mark.parametrize("dtype,op,n,m", [(O.BFLOAT16, O.SUM, 8, 1), (O.INT8, O.MAX, 5, 1), (O.FLOAT16, O.MIN, 3, 2),
                                          (O.FLOAT64, O.SUM, 2, 1), (O.INT32, O.PROD, 11, 3), (O.UINT16, O.SUM, 1, 2)])
def test_buffers_that_disagree_modulo_16_bytes(comp, variant, dtype, op, n, m):
    """Every input and destination at its own offset from a 16-byte boundary, through each kernel form (default
    choice, streaming, phased) and at sizes from less than a vector to several phases: the vectors start on a
    boundary of the most common alignment, every other buffer is accessed as loose vectors, nothing outside the
    destinations is written."""
    import torch
    rng = np.random.default_rng(4000 + 16 * dtype + n)
    esz = O.DTYPE_SIZE[dtype]
    np_t = O.NP_STORAGE[dtype]
    per16 = 16 // esz
    pad = 64
    keep = 1 if dtype == O.BFLOAT16 else 0
    comp.set_param("variant", variant)
    try:
        for count in (1, per16 - 1, per16 + 1, 1000, 70_001, 3_000_017):
            srcs = make_inputs(rng, dtype, count, op, n)
            want = O.reduce_n(srcs, dtype, op, keep=keep, threads=16)
            for trial in range(3):
                # trial 0: all different where possible; 1: inputs agree, destinations do not; 2: random
                if trial == 0:
                    sh = [(j + 1) % per16 for j in range(n + m)]
                elif trial == 1:
                    sh = [3 % per16] * n + [(5 + k) % per16 for k in range(m)]
                else:
                    sh = [int(x) for x in rng.integers(0, per16, n + m)]
                big = []
                for s_, k in zip(srcs, sh[:n]):
                    h = np.zeros(count + 2 * pad, np_t)
                    h[pad + k:pad + k + count] = s_
                    big.append(to_dev(h))
                outs = [to_dev(np.zeros(count + 2 * pad, np_t)) for _ in range(m)]
                sp = [b_.data_ptr() + (pad + k) * esz for b_, k in zip(big, sh[:n])]
                dp = [o_.data_ptr() + (pad + k) * esz for o_, k in zip(outs, sh[n:])]
                if m == 1:
                    comp.comp_reduce_n(dtype, op, sp, dp[0], count, lp_mode=keep)
                else:
                    comp.comp_reduce_write_n(dtype, op, sp, dp, count, lp_mode=keep)
                torch.cuda.synchronize()
                for o_, k in zip(outs, sh[n:]):
                    g = to_host(o_, np_t)
                    assert_same(g[pad + k:pad + k + count], want, dtype, f"count={count} shifts={sh}", srcs, op, keep=keep)
                    assert not g[:pad + k].view(np.uint8).any() and not g[pad + k + count:].view(np.uint8).any(), \
                        f"wrote outside a destination: count={count} shifts={sh}"
    finally:
        comp.set_param("variant", 0)


def test_randomised_calls_against_oracle(comp):
    """400 seeded random calls (MI_CCL_FUZZ_CASES / MI_CCL_FUZZ_SEED change that): dtype, op, input count (1..12),
    1..3 destinations, element count, 16-bit mode, per-buffer element shifts (shared or mixed misalignment), output
    aliasing an input or not, kernel choice forced or automatic, the 128-byte line rule and the wave-run layout on or
    off."""
    import os
    import torch
    rng = np.random.default_rng(int(os.environ.get("MI_CCL_FUZZ_SEED", "20260101")))
    for case in range(int(os.environ.get("MI_CCL_FUZZ_CASES", "400"))):
        dtype = int(rng.integers(0, 12))
        op = int(rng.integers(0, 4))
        n = int(rng.integers(1, 13))
        count = int(rng.choice([1, 2, 3, 15, 16, 17, 255, 1000, 4097, 65535, 200_003, 1_100_003]))     # the last: heads up to a 128-byte line
        esz = O.DTYPE_SIZE[dtype]
        np_t = O.NP_STORAGE[dtype]
        lp, impl, keep, quirk = lp_variants(dtype)[int(rng.integers(0, len(lp_variants(dtype))))]
        kind = "bits" if dtype in (O.FLOAT16, O.BFLOAT16) and rng.random() < 0.5 else "config"
        srcs = make_inputs(rng, dtype, count, op, n, kind)
        same_shift = rng.random() < 0.6
        span = (128 if count > 1_000_000 else 16) // esz
        base_shift = int(rng.integers(0, span + 1))
        shifts = [base_shift if same_shift else int(rng.integers(0, span + 1)) for _ in range(n + 1)]
        pad = 160
        holders, ptrs = [], []
        for s_, sh in zip(srcs, shifts):
            h = np.zeros(count + 2 * pad, np_t)
            h[pad + sh:pad + sh + count] = s_
            holders.append(to_dev(h))
            ptrs.append(holders[-1].data_ptr() + (pad + sh) * esz)
        alias = int(rng.integers(-1, n))            # -1: separate output
        if alias >= 0:
            out_holder, out_lo = holders[alias], pad + shifts[alias]
        else:
            out_holder, out_lo = to_dev(np.zeros(count + 2 * pad, np_t)), pad + shifts[n]
        variant = int(rng.choice([0, 0, 2, 8]))
        m = int(rng.choice([1, 1, 2, 3]))
        extra = []       # further destinations: (holder, first element), with the output's shift or one of their own
        for _ in range(m - 1):
            sh = shifts[alias if alias >= 0 else n] if same_shift else int(rng.integers(0, span + 1))
            extra.append((to_dev(np.zeros(count + 2 * pad, np_t)), pad + sh))
        line_start, wave_runs = int(rng.integers(0, 2)), int(rng.integers(0, 3))
        comp.set_param("variant", variant)
        comp.set_param("line_start", line_start)
        comp.set_param("wave_runs", wave_runs)
        try:
            out_ptr = out_holder.data_ptr() + out_lo * esz
            if m == 1:
                comp.comp_reduce_n(dtype, op, ptrs, out_ptr, count, lp_mode=lp, bf16_impl=impl)
            else:
                comp.comp_reduce_write_n(dtype, op, ptrs, [out_ptr] + [h.data_ptr() + lo * esz for h, lo in extra], count,
                                         lp_mode=lp, bf16_impl=impl)
            torch.cuda.synchronize()
        finally:
            comp.set_param("variant", 0)
            comp.set_param("line_start", 1)
            comp.set_param("wave_runs", 1)
        want = O.reduce_n(srcs, dtype, op, keep=keep, quirk_tail=quirk, bf16_impl=impl)
        got = to_host(out_holder, np_t)
        what = (f"case {case}: dtype={O.DTYPE_NAMES[dtype]} op={O.OP_NAMES[op]} n={n} m={m} count={count} lp={lp} impl={impl} "
                f"shifts={shifts} alias={alias} variant={variant} line_start={line_start} wave_runs={wave_runs} kind={kind}")
        assert_same(got[out_lo:out_lo + count], want, dtype, what, srcs, op, keep=keep, bf16_impl=impl)
        for h, lo in extra:
            g2 = to_host(h, np_t)
            assert_same(g2[lo:lo + count], want, dtype, what + " (further destination)", srcs, op, keep=keep, bf16_impl=impl)
            assert (g2[:lo] == 0).all() and (g2[lo + count:] == 0).all(), what + ": wrote outside a further destination"
        if alias < 0:
            assert (got[:out_lo] == 0).all() and (got[out_lo + count:] == 0).all(), what + ": wrote outside the destination"
        else:
            assert (got[:out_lo] == 0).all() and (got[out_lo + count:] == 0).all(), what + ": wrote outside the aliased input"


def test_fp16_native_mode_against_reference_made_vectors(comp, golden, golden_fp16_native):
    """fp16_impl = avx512fp16 (mi_ccl_set_param): the GPU against what the reference's native-fp16 code produced --
    bits for min/max (a signalling NaN that is handed back stays signalling) and for sum/prod (two NaN operands aside) --
    then the N-input and multi-destination forms against the oracle in the same mode."""
    import torch
    from test_oracle_pins import _fp16_native_cases
    assert comp.get_param("fp16_impl") == 3
    comp.set_param("fp16_impl", 4)
    try:
        n = 0
        for name, op, a, b, want in _fp16_native_cases(golden, golden_fp16_native):
            da, db = to_dev(a), to_dev(b)
            comp.comp_reduce(O.FLOAT16, op, da, a.size, db)
            torch.cuda.synchronize()
            got = to_host(db, np.uint16)
            if op in (O.MIN, O.MAX):
                assert (got == want).all(), (name, np.flatnonzero(got != want)[:8])
            else:
                assert_same(got, want, O.FLOAT16, name, [b, a], op, fp16_impl=O.FP16_AVX512FP16)
            n += 1
        assert n == 96
        rng = np.random.default_rng(123)
        for op in (O.MIN, O.MAX, O.SUM):
            srcs = make_inputs(rng, O.FLOAT16, 70001, op, 5, "bits")
            d = [to_dev(s) for s in srcs]
            outs = [torch.empty_like(d[0]) for _ in range(3)]
            comp.comp_reduce_write_n(O.FLOAT16, op, d, outs, 70001)
            torch.cuda.synchronize()
            want = O.reduce_n(srcs, O.FLOAT16, op, fp16_impl=O.FP16_AVX512FP16)
            for o in outs:
                got = to_host(o, np.uint16)
                if op == O.SUM:
                    assert_same(got, want, O.FLOAT16, "native fp16 sum", srcs, op, fp16_impl=O.FP16_AVX512FP16)
                else:
                    assert (got == want).all()
    finally:
        comp.set_param("fp16_impl", 3)
    with pytest.raises(comp.CclError):
        comp.set_param("fp16_impl", 1)


@pytest.mark.parametrize("dtype", [O.INT8, O.UINT8])
def test_one_byte_integers_every_pair_of_values_through_every_kernel(comp, dtype):
    """All 65,536 (in, inout) pairs of one-byte values for the four operations (wrapping sum and product, signed or
    unsigned min and max), through the streaming kernel, the phased kernel, the run-time-count kernels (nine inputs,
    two outputs) and the fused kernel in both forms: the byte-lane instructions of the vector path against the
    oracle."""
    import torch
    np_t = O.NP_STORAGE[dtype]
    allv = np.arange(256, dtype=np.uint8).view(np_t)
    a = np.tile(np.repeat(allv, 256), 3)         # in
    b = np.tile(np.tile(allv, 256), 3)           # inout
    count = a.size
    rng = np.random.default_rng(8 + dtype)
    extra = [rng.integers(0, 256, count, dtype=np.uint8).view(np_t) for _ in range(7)]
    for op in range(4):
        want2 = O.reduce_n([b, a], dtype, op)
        want9 = O.reduce_n([b, a] + extra, dtype, op)
        for variant in (2, 8):
            comp.set_param("variant", variant)
            try:
                da, db = to_dev(a), to_dev(b)
                comp.comp_reduce(dtype, op, da, count, db)
                torch.cuda.synchronize()
                assert (to_host(db, np_t) == want2).all(), (op, variant, "pair")
                db = to_dev(b)
                de = [to_dev(e) for e in extra]
                outs = [torch.empty_like(db) for _ in range(2)]
                comp.comp_reduce_write_n(dtype, op, [db, da] + de, outs, count)
                torch.cuda.synchronize()
                for o in outs:
                    assert (to_host(o, np_t) == want9).all(), (op, variant, "nine inputs, two outputs")
                h = count // 2 + 5
                plan = comp.FusionPlan([h, count - h], dtype, 1)
                peers = []
                for src in [a] + extra:
                    fb = torch.zeros(plan.nbytes, dtype=db.dtype, device="cuda")
                    d_ = to_dev(src)
                    plan.pack([d_[:h], d_[h:]], fb)
                    peers.append(fb)
                own = [db[:h], db[h:]]
                for npeers, want in ((1, want2), (8, want9)):
                    res = [torch.empty_like(t) for t in own]
                    plan.reduce(op, own, peers[:npeers], res)
                    torch.cuda.synchronize()
                    got = np.concatenate([to_host(r, np_t) for r in res])
                    assert (got == want).all(), (op, variant, "fused", npeers)
            finally:
                comp.set_param("variant", 0)


def test_bf16_pairwise_tiny_and_special_values_through_every_kernel(comp):
    """Round-after-every-pair bf16 under avx512bf where the fp32 sum or product is a denormal: VCVTNEPS2BF16 reads it
    as zero (the result is a signed zero), and a value just under the smallest normal must not round up to it.  Every
    pair of a value set around the bottom of the exponent range (sums) and around the square root of it (products),
    through the streaming and the phased kernel, the run-time-count kernels (nine inputs; two outputs) and the
    fused kernel, in both forms.  min and max hand back one operand, which the same instruction turns into a signed
    zero when it is a denormal and quiets when it is a signalling NaN: the same value set plus infinities and NaNs,
    bit for bit."""
    import torch
    vals = []
    for sign in (0, 0x8000):
        for e in (0, 1, 2, 3, 61, 62, 63, 64, 65, 66):
            for m in (0, 1, 0x3F, 0x40, 0x7E, 0x7F):
                vals.append(sign | (e << 7) | m)
    specials = [0x7F80, 0xFF80, 0x7FC0, 0xFFC0, 0x7F81, 0xFF81, 0x7FBF, 0x7FFF, 0xFFFF, 0x7F7F, 0xFF7F, 0x3F80, 0xBF80]
    for op in (O.SUM, O.PROD, O.MIN, O.MAX):
        v = np.array(vals + (specials if op in (O.MIN, O.MAX) else []), dtype=np.uint16)
        a = np.tile(np.repeat(v, v.size), 25)          # in
        b = np.tile(np.tile(v, v.size), 25)            # inout
        count = a.size
        want2 = O.reduce_n([b, a], O.BFLOAT16, op)
        ident = np.full(count, {O.SUM: 0, O.PROD: 0x3F80, O.MIN: 0x7F80, O.MAX: 0xFF80}[op], np.uint16)
        want9 = O.reduce_n([b, a] + [ident] * 7, O.BFLOAT16, op)
        for variant in (2, 8):
            comp.set_param("variant", variant)
            try:
                da, db = to_dev(a), to_dev(b)
                comp.comp_reduce(O.BFLOAT16, op, da, count, db)
                torch.cuda.synchronize()
                assert (to_host(db, np.uint16) == want2).all(), (op, variant, "pair")
                db = to_dev(b)
                di = to_dev(ident)
                outs = [torch.empty_like(db) for _ in range(2)]
                comp.comp_reduce_write_n(O.BFLOAT16, op, [db, da] + [di] * 7, outs, count)
                torch.cuda.synchronize()
                for o in outs:
                    assert (to_host(o, np.uint16) == want9).all(), (op, variant, "nine inputs, two outputs")
                plan = comp.FusionPlan([count // 2, count - count // 2], O.BFLOAT16, 256)
                fb = torch.zeros(plan.nbytes // 2, dtype=torch.int16, device="cuda")
                own = [db[:count // 2], db[count // 2:]]
                plan.pack([da[:count // 2], da[count // 2:]], fb)
                res = [torch.empty_like(t) for t in own]
                plan.reduce(op, own, [fb], res)
                torch.cuda.synchronize()
                got = np.concatenate([to_host(r, np.uint16) for r in res])
                assert (got == want2).all(), (op, variant, "fused")
            finally:
                comp.set_param("variant", 0)
