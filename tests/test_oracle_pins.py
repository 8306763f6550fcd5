"""Pins the CPU oracle (oracle/ccl_comp_oracle.c) without a GPU: golden vectors produced by the reference's
own vector code, known answers recorded from the real reference library, the CPU's conversion instructions
(exhaustively), numpy closed forms, and -- where it was built -- the reference code itself on fresh inputs."""
import os
import subprocess

import numpy as np
import pytest

import oracle_lib as O

L = O.lib()


def hx(s):
    return np.uint16(int(s, 16))


# ----------------------------------------------------------------------------------------------
# golden vectors from the reference's vector code

@pytest.mark.parametrize("fam,dtype", [("bf16", O.BFLOAT16), ("fp16", O.FLOAT16)])
def test_golden_pairwise(golden, fam, dtype):
    impls = (1, 2) if fam == "bf16" else (2, 3)
    checked = 0
    for key in golden.files:
        if not key.startswith(fam + "_") or not key.endswith("_in") or "specials" in key or key.startswith("cvt"):
            continue
        stem = key[:-3]
        op = O.OP_NAMES.index(stem.split("_")[1])
        a, b = golden[stem + "_in"], golden[stem + "_inout"]
        for impl in impls:
            want = golden[stem + f"_impl{impl}"]
            got = O.comp_reduce(a, b, dtype, op, bf16_impl=impl, fp16_impl=impl)
            ok = O.same_bits(got, want, dtype, [b, a], op, bf16_impl=impl, fp16_impl=impl)
            assert ok.all(), (stem, impl, np.flatnonzero(~ok)[:5], a[~ok][:5], b[~ok][:5], got[~ok][:5], want[~ok][:5])
            checked += 1
    assert checked >= 2 * 4 * 11 * 2


@pytest.mark.parametrize("fam,dtype", [("bf16", O.BFLOAT16), ("fp16", O.FLOAT16)])
def test_golden_special_pairs_exact(golden, fam, dtype):
    """All pairs of special values.  For min/max the result is one of the operands, so NaN payloads are
    pinned too and the comparison is on bits; so is it for sum/prod, except where both operands are NaNs."""
    impls = (1, 2) if fam == "bf16" else (2, 3)
    a, b = golden[f"{fam}_specials_in"], golden[f"{fam}_specials_inout"]
    for op in range(4):
        for impl in impls:
            want = golden[f"{fam}_specials_{O.OP_NAMES[op]}_impl{impl}"]
            got = O.comp_reduce(a, b, dtype, op, bf16_impl=impl, fp16_impl=impl)
            if op in (O.MIN, O.MAX):
                assert (got == want).all(), (fam, op, impl, np.flatnonzero(got != want)[:8])
            else:
                assert O.same_bits(got, want, dtype, [b, a], op, bf16_impl=impl, fp16_impl=impl).all(), (fam, op, impl)


def test_golden_converters(golden):
    f32 = golden["cvt_fp32_in"]
    n = f32.size
    for impl in (1, 2):
        out = np.empty(n, np.uint16)
        L.orc_convert_fp32_to_bf16_arrays(f32.ctypes.data, out.ctypes.data, n, impl)
        assert (out == golden[f"cvt_fp32_to_bf16_impl{impl}"]).all(), impl
    h = golden["cvt_bf16_in"]
    w = np.empty(h.size, np.uint32)
    L.orc_convert_bf16_to_fp32_arrays(h.ctypes.data, w.ctypes.data, h.size, 2)
    assert (w == golden["cvt_bf16_to_fp32"]).all()


# ----------------------------------------------------------------------------------------------
# known answers recorded from the real reference library

def test_probe_bf16_pairwise_sum(probes):
    p = probes["bf16_pairwise_sum"]
    a = np.array([hx(x) for x in p["in"]], np.uint16)
    b = np.full(a.size, hx(p["inout"]), np.uint16)
    for name, impl in (("scalar", 0), ("avx512f", 1), ("avx512bf", 2)):
        got = O.comp_reduce(a, b, O.BFLOAT16, O.SUM, bf16_impl=impl)
        assert [f"{v:04x}" for v in got] == p[name], name


def test_probe_fp32_to_bf16_arrays_tail_truncates(probes):
    p = probes["fp32_to_bf16_arrays"]
    vals = np.array([int(x, 16) for x in p["fp32_in"]], np.uint32)
    src = np.zeros(22, np.uint32)
    src[:6] = vals
    src[16:22] = vals
    for impl, body in ((2, p["avx512bf_body"]), (1, p["scalar_and_avx512f_everywhere"]),
                       (0, p["scalar_and_avx512f_everywhere"])):
        out = np.empty(22, np.uint16)
        L.orc_convert_fp32_to_bf16_arrays(src.ctypes.data, out.ctypes.data, 22, impl)
        assert [f"{v:04x}" for v in out[:6]] == body, impl
        assert [f"{v:04x}" for v in out[16:]] == p["tail_any_impl"], impl


def test_probe_batch_reduce_keep_precision_and_tail(probes):
    p = probes["batch_reduce_bf16"]
    cnt = p["count"]
    buf = np.concatenate([np.full(cnt, hx(s), np.uint16) for s in p["slices"]])
    offs = [i * cnt for i in range(len(p["slices"]))]
    r1 = O.batch_reduce(buf, offs, cnt, O.BFLOAT16, O.SUM, 1, bf16_impl=2)[:cnt]
    assert all(f"{v:04x}" == p["keep_precision_1_body"] for v in r1[:16])
    assert f"{r1[16]:04x}" == p["keep_precision_1_tail"]
    r0 = O.batch_reduce(buf, offs, cnt, O.BFLOAT16, O.SUM, 0, bf16_impl=2)[:cnt]
    assert all(f"{v:04x}" == p["keep_precision_0"] for v in r0)
    # the N-buffer form agrees with the slice form, with and without the tail quirk
    srcs = [buf[o:o + cnt] for o in offs]
    assert (O.reduce_n(srcs, O.BFLOAT16, O.SUM, keep=1, quirk_tail=1) == r1).all()
    nq = O.reduce_n(srcs, O.BFLOAT16, O.SUM, keep=1, quirk_tail=0)
    assert all(f"{v:04x}" == p["keep_precision_1_body"] for v in nq)
    assert (O.reduce_n(srcs, O.BFLOAT16, O.SUM, keep=0) == r0).all()


def _fp(s, np_t):
    return np_t({"nan": np.nan, "1": 1.0, "-0": -0.0, "+0": 0.0}[s])


@pytest.mark.parametrize("dtype,np_t", [(O.FLOAT32, np.float32), (O.FLOAT64, np.float64)])
def test_probe_fp_minmax_returns_in_on_tie_or_nan(probes, dtype, np_t):
    for c in probes["fp_minmax_plain"]["cases"]:
        for n in (4, 67):
            a = np.full(n, _fp(c["in"], np_t), np_t)
            b = np.full(n, _fp(c["inout"], np_t), np_t)
            got = O.comp_reduce(a, b, dtype, O.OP_NAMES.index(c["op"]))
            want = _fp(c["out"], np_t)
            if np.isnan(want):
                assert np.isnan(got).all(), c
            else:
                assert (got == want).all() and (np.signbit(got) == np.signbit(want)).all(), c


def test_probe_bf16_min_operand_order(probes):
    for c in probes["bf16_min"]["cases"]:
        for name, impl in (("scalar", 0), ("avx512f", 1), ("avx512bf", 2)):
            got = O.comp_reduce(np.array([hx(c["in"])] * 20), np.array([hx(c["inout"])] * 20), O.BFLOAT16,
                                O.MIN, bf16_impl=impl)
            assert all(f"{v:04x}" == c[name] for v in got), (c, name)


def test_probe_fp16_pairwise_sum(probes):
    p = probes["fp16_pairwise_sum"]
    a = np.array([hx(x) for x in p["in"]], np.uint16)
    b = np.array([hx(x) for x in p["inout"]], np.uint16)
    for name, impl in (("f16c", 2), ("avx512f", 3)):
        got = O.comp_reduce(a, b, O.FLOAT16, O.SUM, fp16_impl=impl)
        assert [f"{v:04x}" for v in got] == p[name], name
    for impl in (0, 1):
        got = O.comp_reduce(a, b, O.FLOAT16, O.SUM, fp16_impl=impl)
        assert [f"{v:04x}" for v in got] == p["unhandled_impl"]


def test_probe_int_wrap(probes):
    for c in probes["int_wrap"]["cases"]:
        dt = O.DTYPE_NAMES.index(c["dtype"])
        np_t = O.NP_STORAGE[dt]
        got = O.comp_reduce(np.array([c["in"]] * 5, np_t), np.array([c["inout"]] * 5, np_t), dt, O.SUM)
        assert (got == np_t(c["out"])).all(), c


# ----------------------------------------------------------------------------------------------
# the CPU's own conversion instructions, exhaustively (the reference uses exactly these)

def test_selfcheck_exhaustive_vs_cpu_instructions():
    exe = os.path.join(O.ORACLE_DIR, "selfcheck")
    if not os.path.exists(exe):
        O.build_oracle()
    out = subprocess.run([exe, "8", "1"], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "mismatches=0" in out.stdout
    for line in out.stdout.splitlines():
        assert "skipped" in line or line.rstrip().split("mismatches=")[1].split()[0] == "0", line


def test_fp16_converters_vs_numpy_float16():
    """numpy's float16 casts are an independent IEEE binary16 implementation (RNE, subnormals kept)."""
    h = np.arange(65536, dtype=np.uint16)
    w = np.array([L.orc_fp16_widen(int(x)) for x in h], np.uint32)
    want = h.view(np.float16).astype(np.float32).view(np.uint32)
    nan = np.isnan(h.view(np.float16))
    assert (w[~nan] == want[~nan]).all()
    assert np.isnan(w.view(np.float32)[nan]).all()
    rng = np.random.default_rng(7)
    u = np.concatenate([rng.integers(0, 2**32, 200000, dtype=np.uint32),
                        (np.arange(0x38000000, 0x38000000 + 70000, dtype=np.uint32)),
                        (np.arange(0x477FE000 - 3000, 0x477FE000 + 9000, dtype=np.uint32)),
                        (np.arange(0x33000000 - 3000, 0x33000000 + 3000, dtype=np.uint32))])
    f = u.view(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        want16 = f.astype(np.float16).view(np.uint16)
    got16 = np.array([L.orc_fp16_narrow(int(x)) for x in u], np.uint16)
    finite = ~np.isnan(f)
    assert (got16[finite] == want16[finite]).all()


def test_fp16_array_converters_are_the_per_value_converters():
    """orc_convert_fp32_to_fp16_arrays / orc_convert_fp16_to_fp32_arrays loop over the pinned per-value functions;
    checked against them and, for finite values, against numpy's independent float16 casts."""
    rng = np.random.default_rng(17)
    u = np.concatenate([rng.integers(0, 2**32, 50_000, dtype=np.uint32),
                        np.array([0, 0x80000000, 1, 0x33000000, 0x33000001, 0x387FFFFF, 0x38800000, 0x477FEFFF, 0x477FF000,
                                  0x7F800000, 0xFF800000, 0x7F800001, 0x7FC00000, 0xFFFFFFFF], np.uint32)])
    out = np.empty(u.size, np.uint16)
    L.orc_convert_fp32_to_fp16_arrays(u.ctypes.data, out.ctypes.data, u.size)
    assert (out == np.array([L.orc_fp16_narrow(int(x)) for x in u], np.uint16)).all()
    f = u.view(np.float32)
    fin = ~np.isnan(f)
    with np.errstate(over="ignore", invalid="ignore"):
        assert (out[fin] == f.astype(np.float16).view(np.uint16)[fin]).all()
    nan_in = ~fin
    assert ((out[nan_in] & 0x7C00) == 0x7C00).all() and ((out[nan_in] & 0x0200) != 0).all()      # NaN stays NaN, quiet
    h = np.arange(65536, dtype=np.uint16)
    w = np.empty(65536, np.uint32)
    L.orc_convert_fp16_to_fp32_arrays(h.ctypes.data, w.ctypes.data, 65536)
    assert (w == np.array([L.orc_fp16_widen(int(x)) for x in h], np.uint32)).all()


# ----------------------------------------------------------------------------------------------
# closed forms for the plain types

INT_TYPES = [O.INT8, O.UINT8, O.INT16, O.UINT16, O.INT32, O.UINT32, O.INT64, O.UINT64]


@pytest.mark.parametrize("dtype", INT_TYPES)
@pytest.mark.parametrize("op", [O.SUM, O.PROD, O.MIN, O.MAX])
def test_int_ops_vs_python_big_integers(dtype, op):
    np_t = O.NP_STORAGE[dtype]
    info = np.iinfo(np_t)
    rng = np.random.default_rng(dtype * 4 + op)
    n = 257
    a = rng.integers(info.min, info.max, size=n, dtype=np_t, endpoint=True)
    b = rng.integers(info.min, info.max, size=n, dtype=np_t, endpoint=True)
    edge = np.array([info.min, info.max, 0, 1, info.max - 1, info.min + 1] + ([-1] if info.min < 0 else [2]), np_t)
    a[:edge.size] = edge
    b[:edge.size] = edge[::-1]
    got = O.comp_reduce(a, b, dtype, op)
    bits = info.bits
    for i in range(n):
        x, y = int(a[i]), int(b[i])
        if op == O.SUM:
            w = y + x
        elif op == O.PROD:
            w = y * x
        elif op == O.MIN:
            w = min(x, y)
        else:
            w = max(x, y)
        w &= (1 << bits) - 1
        if info.min < 0 and w >= 1 << (bits - 1):
            w -= 1 << bits
        assert int(got[i]) == w, (dtype, op, x, y)


@pytest.mark.parametrize("dtype", [O.INT16, O.UINT16, O.INT8, O.UINT8])
def test_narrow_int_products_wrap_where_a_signed_int_would_overflow(dtype):
    """Every value of the type times a set of rows that includes the largest magnitudes (65535 x 65535 = 0xFFFE0001 does
    not fit a signed int, which is what the operands of a 16-bit multiply are promoted to): the wrapped product on
    32-bit unsigned integers is the expected result."""
    np_t = O.NP_STORAGE[dtype]
    bits = np.iinfo(np_t).bits
    allv = np.arange(1 << bits, dtype=np.uint32)
    rows = np.unique(np.concatenate([np.array([0, 1, 2, 0x7FFF, 0x8000, 0x8001, 0xB504, 0xB505, 0xFFFE, 0xFFFF], np.uint32) & ((1 << bits) - 1),
                                     np.random.default_rng(16).integers(0, 1 << bits, 54, dtype=np.uint32)]))
    a = np.tile(allv, rows.size)
    b = np.repeat(rows, allv.size)
    u_t = np.uint16 if bits == 16 else np.uint8
    got = O.comp_reduce(a.astype(u_t).view(np_t), b.astype(u_t).view(np_t), dtype, O.PROD)
    assert (got.view(u_t) == (a * b).astype(u_t)).all()


@pytest.mark.parametrize("dtype,np_t", [(O.FLOAT32, np.float32), (O.FLOAT64, np.float64)])
def test_fp_sum_prod_are_single_ieee_ops_in_chain_order(dtype, np_t):
    rng = np.random.default_rng(3)
    srcs = [rng.uniform(-2, 2, 1000).astype(np_t) for _ in range(5)]
    srcs[2][:3] = [np.finfo(np_t).tiny / 4, np.finfo(np_t).max, -np.finfo(np_t).max]  # subnormal, overflow
    for op, f in ((O.SUM, np.add), (O.PROD, np.multiply)):
        want = srcs[0].copy()
        with np.errstate(over="ignore"):
            for s in srcs[1:]:
                want = f(want, s)          # numpy elementwise ops are single IEEE operations
        got = O.reduce_n(srcs, dtype, op)
        assert O.same_bits(got, want, dtype).all()
    # exact fractions: ((0.1f + 0.2f) + 0.3f) differs from (0.1f + (0.2f + 0.3f)) -- order matters
    x = [np.full(4, v, np_t) for v in (0.1, 0.2, 0.3)]
    assert (O.reduce_n(x, dtype, O.SUM) == (x[0] + x[1]) + x[2]).all()


def test_bf16_pairwise_vs_exact_rational_rounding():
    """Round-to-nearest-even of the exact sum/product of two bf16 values, computed with Python fractions."""
    from fractions import Fraction
    rng = np.random.default_rng(11)
    a = (rng.integers(0x3000, 0x4F00, 3000) | (rng.integers(0, 2, 3000) << 15)).astype(np.uint16)
    b = (rng.integers(0x3000, 0x4F00, 3000) | (rng.integers(0, 2, 3000) << 15)).astype(np.uint16)
    fa, fb = O.bf16_to_f32(a), O.bf16_to_f32(b)

    def rne_bf16(q):
        if q == 0:
            return None
        s = q < 0
        q = abs(q)
        e = 0
        while q >= 2:
            q /= 2
            e += 1
        while q < 1:
            q *= 2
            e -= 1
        m = q * 128                       # 1.mmmmmmm * 2^7
        fl = m.numerator // m.denominator
        rem = m - fl
        if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl & 1):
            fl += 1
        if fl == 256:
            fl = 128
            e += 1
        return (int(s) << 15) | ((e + 127) << 7) | (fl - 128)

    for op in (O.SUM, O.PROD):
        got = O.comp_reduce(a, b, O.BFLOAT16, op, bf16_impl=2)
        for i in range(a.size):
            x, y = Fraction(float(fa[i])), Fraction(float(fb[i]))
            w = rne_bf16(y + x if op == O.SUM else y * x)
            if w is None:
                assert got[i] & 0x7FFF == 0
            else:
                assert int(got[i]) == w, (hex(a[i]), hex(b[i]), hex(got[i]), hex(w))


def test_functional_test_closed_forms(probes):
    """The reference's own functional tests fill rank r's buffer with c1*r + c2*buf_idx (+1 for prod) and
    expect closed forms (tests/functional/test_impl.hpp:242-324, test.hpp:73-86) within g*expected,
    g = log2(N)*eps / (1 - log2(N)*eps) (test_impl.hpp:160-204)."""
    import math
    N = 4
    for size in probes["closed_form_functional_tests"]["sizes"][:2]:
        for dtype, c1, c2, eps in ((O.INT32, 1, 1, 0.0), (O.FLOAT32, 1.0, 1.0, 2.0**-23),
                                   (O.FLOAT16, 0.01, 0.01, 2 * 2.0**-10), (O.BFLOAT16, 0.5, 1.0, 2 * 2.0**-7)):
            for buf_idx in (0, 3):
                for op in range(4):
                    vals = [c1 * r + c2 * buf_idx + (1 if op == O.PROD else 0) for r in range(N)]
                    if dtype == O.INT32:
                        srcs = [np.full(size, v, np.int32) for v in vals]
                    elif dtype == O.FLOAT32:
                        srcs = [np.full(size, v, np.float32) for v in vals]
                    elif dtype == O.FLOAT16:
                        srcs = [np.full(size, v, np.float16).view(np.uint16) for v in vals]
                    else:
                        srcs = [O.bf16_from_f32(np.full(size, v, np.float32)) for v in vals]
                    got = O.reduce_n(srcs, dtype, op)
                    if dtype == O.FLOAT16:
                        got = got.view(np.float16).astype(np.float64)
                    elif dtype == O.BFLOAT16:
                        got = O.bf16_to_f32(got).astype(np.float64)
                    exp = {O.SUM: sum(vals), O.PROD: math.prod(vals), O.MIN: min(vals), O.MAX: max(vals)}[op]
                    le = math.log2(N) * eps
                    tol = abs(exp) * le / (1 - le) + (abs(exp) * eps if dtype in (O.FLOAT16, O.BFLOAT16) else 0)
                    assert np.all(np.abs(got.astype(np.float64) - exp) <= tol + 1e-300), (dtype, op, buf_idx, exp, got[0])
                    assert (got == got[0]).all()


# ----------------------------------------------------------------------------------------------
# structure: N-way forms agree with chains of the pinned pairwise primitive; fusion layout

@pytest.mark.parametrize("dtype", range(12))
@pytest.mark.parametrize("op", range(4))
def test_reduce_n_equals_chain_of_pairwise(dtype, op):
    rng = np.random.default_rng(100 + dtype * 4 + op)
    n, count = 5, 333
    np_t = O.NP_STORAGE[dtype]
    if dtype in (O.FLOAT32, O.FLOAT64):
        srcs = [rng.uniform(-2, 2, count).astype(np_t) for _ in range(n)]
    elif dtype in (O.FLOAT16, O.BFLOAT16):
        srcs = [rng.integers(0, 65536, count, dtype=np.uint16) for _ in range(n)]
    else:
        info = np.iinfo(np_t)
        srcs = [rng.integers(info.min, info.max, count, dtype=np_t, endpoint=True) for _ in range(n)]
    want = srcs[0].copy()
    for s in srcs[1:]:
        want = O.comp_reduce(s, want, dtype, op)
    got = O.reduce_n(srcs, dtype, op)
    assert O.same_bits(got, want, dtype, srcs, op).all()
    # slice form (ccl_comp_batch_reduce, keep_precision 0) and the partitioned form agree too
    buf = np.concatenate(srcs)
    got2 = O.batch_reduce(buf, [i * count for i in range(n)], count, dtype, op, 0)[:count]
    assert O.same_bits(got2, want, dtype, srcs, op).all()
    got3 = O.reduce_n(srcs, dtype, op, threads=3)
    assert O.same_bits(got3, want, dtype, srcs, op).all()


@pytest.mark.parametrize("impl", [0, 1, 2])
@pytest.mark.parametrize("op", range(4))
def test_keep_precision_is_widen_fp32_chain_narrow(impl, op):
    rng = np.random.default_rng(impl * 4 + op)
    n, count = 8, 100          # 100 = 6*16 + 4: body and tail
    srcs = [(rng.integers(0x3C00, 0x4100, count) | (rng.integers(0, 2, count) << 15)).astype(np.uint16) for _ in range(n)]
    acc = O.bf16_to_f32(srcs[0]).copy()
    for s in srcs[1:]:
        acc = O.comp_reduce(O.bf16_to_f32(s), acc, O.FLOAT32, op)
    want = np.empty(count, np.uint16)
    L.orc_convert_fp32_to_bf16_arrays(acc.ctypes.data, want.ctypes.data, count, impl)
    buf = np.concatenate(srcs)
    got = O.batch_reduce(buf, [i * count for i in range(n)], count, O.BFLOAT16, op, 1, bf16_impl=impl)[:count]
    assert (got == want).all()
    assert (O.reduce_n(srcs, O.BFLOAT16, op, keep=1, quirk_tail=1, bf16_impl=impl) == want).all()


def test_fusion_layout_and_round_trip():
    rng = np.random.default_rng(5)
    counts = [int(c) for c in rng.integers(1, 5000, 37)]
    tensors = [rng.integers(0, 65536, c, dtype=np.uint16) for c in counts]
    for align in (1, 256):
        offs, total = O.fusion_offsets(counts, 2, align)
        end = 0
        for k, c in enumerate(counts):
            assert offs[k] == (end + align - 1) // align * align     # closed form: fusion.cpp:314 when align == 1
            end = int(offs[k]) + 2 * c
        assert total == end
        if align == 1:
            assert total == 2 * sum(counts)
        buf = O.fusion_pack(tensors, offs, total, 2)
        back = O.fusion_unpack(buf, counts, offs, np.uint16)
        assert all((a == b).all() for a, b in zip(tensors, back))
        # reduce over the packed buffer == per-tensor reduce (elementwise invariant)
        peers = [rng.integers(0x3C00, 0x4000, total // 2, dtype=np.uint16) for _ in range(3)]
        fused = O.reduce_n([buf.view(np.uint16)] + peers, O.BFLOAT16, O.SUM, keep=1)
        outs = O.fusion_unpack(fused.view(np.uint8), counts, offs, np.uint16)
        for k, c in enumerate(counts):
            lo = int(offs[k]) // 2
            per = O.reduce_n([tensors[k]] + [p[lo:lo + c] for p in peers], O.BFLOAT16, O.SUM, keep=1)
            assert (outs[k] == per).all()


def test_tables():
    assert [L.orc_datatype_size(i) for i in range(12)] == O.DTYPE_SIZE
    assert [L.orc_datatype_name(i).decode() for i in range(12)] == O.DTYPE_NAMES
    assert [L.orc_reduction_to_str(i).decode() for i in range(6)] == ["sum", "prod", "min", "max", "custom", "unknown"]
    assert L.orc_comp_reduce(None, 0, None, 99, 0, 0, 0) == 0      # count 0 succeeds before any check
    a = np.zeros(1, np.int8)
    assert L.orc_comp_reduce(a.ctypes.data, 1, a.ctypes.data, 99, 0, 0, 0) == 2


# ----------------------------------------------------------------------------------------------
# the reference's vector code on fresh inputs, where oracle/_ref exists

needs_ref = pytest.mark.skipif(O.ref() is None or (O.ref_cpu_support() & 7) != 7,
                               reason="oracle/_ref not built or CPU lacks avx512/bf16/f16c")


@needs_ref
@pytest.mark.parametrize("fam,dtype,impls", [("bf16", O.BFLOAT16, (1, 2)), ("fp16", O.FLOAT16, (2, 3))])
def test_against_reference_code_random(fam, dtype, impls):
    R = O.ref()
    fn = R.ref_bf16_reduce if fam == "bf16" else R.ref_fp16_reduce
    rng = np.random.default_rng(99)
    for count in (5, 64, 100003):
        for op in range(4):
            a = rng.integers(0, 65536, count, dtype=np.uint16)
            b = rng.integers(0, 65536, count, dtype=np.uint16)
            for impl in impls:
                want = b.copy()
                assert fn(a.ctypes.data, count, want.ctypes.data, op, impl) == 0
                got = O.comp_reduce(a, b, dtype, op, bf16_impl=impl, fp16_impl=impl)
                if op in (O.MIN, O.MAX):
                    assert (got == want).all()
                else:
                    assert O.same_bits(got, want, dtype, [b, a], op, bf16_impl=impl, fp16_impl=impl).all()


@needs_ref
@pytest.mark.parametrize("impl", [1, 2])
def test_keep_precision_batch_reduce_against_the_reference_helpers_in_its_pass_structure(impl):
    """orc_comp_batch_reduce (keep-precision sum) against the reference's own 16-wide converters called in the
    reference's pass order (widen own into acc; per slice widen into tmp, fp32 add; narrow once), on random bit
    patterns (NaNs, infinities, denormals included) and on gradient-like values, 1..9 slices."""
    R = O.ref()
    if not hasattr(R, "ref_batch_reduce_keep_sum"):
        pytest.skip("oracle/_ref predates ref_batch_reduce_keep_sum: rebuild it (make -C oracle ref)")
    rng = np.random.default_rng(314 + impl)
    L = O.lib()
    for n in (1, 2, 5, 8, 9):
        for count in (16, 4096, 100_000 - 100_000 % 16):
            for kind in ("bits", "normal"):
                if kind == "bits":
                    buf = rng.integers(0, 65536, n * count, dtype=np.uint16)
                else:
                    buf = (rng.standard_normal(n * count).astype(np.float32) * 1e-3).view(np.uint32)
                    buf = (buf >> 16).astype(np.uint16)
                offs = np.arange(n, dtype=np.uint64) * np.uint64(count)
                tmp, acc = np.empty(count, np.float32), np.empty(count, np.float32)
                want = buf.copy()
                assert R.ref_batch_reduce_keep_sum(want.ctypes.data, offs.ctypes.data, n, count, want.ctypes.data,
                                                   tmp.ctypes.data, acc.ctypes.data, impl) == 0
                got = buf.copy()
                assert L.orc_comp_batch_reduce(got.ctypes.data, offs.ctypes.data, n, count, got.ctypes.data, O.BFLOAT16,
                                               O.SUM, 1, tmp.ctypes.data, acc.ctypes.data, impl, O.FP16_AVX512F) == 0
                slices = [buf[i * count:(i + 1) * count] for i in range(n)]
                assert O.same_bits(got[:count], want[:count], O.BFLOAT16, slices, O.SUM, keep=1, bf16_impl=impl).all(), (n, count, kind)
                assert (got[count:] == buf[count:]).all()


@needs_ref
def test_against_reference_code_every_bf16_pair_sampled():
    """All 65536 bf16 values against 64 partners (sum, RNE): 4M pairs through the reference code."""
    R = O.ref()
    rng = np.random.default_rng(1)
    a = np.tile(np.arange(65536, dtype=np.uint16), 64)
    b = np.repeat(rng.integers(0, 65536, 64, dtype=np.uint16), 65536)
    want = b.copy()
    assert R.ref_bf16_reduce(a.ctypes.data, a.size, want.ctypes.data, O.SUM, 2) == 0
    got = O.comp_reduce(a, b, O.BFLOAT16, O.SUM, bf16_impl=2)
    assert O.same_bits(got, want, O.BFLOAT16, [b, a], O.SUM, bf16_impl=2).all()


def test_reduce_write_n_is_reduce_n_stored_m_times():
    """allreduce_kernel (kernels.cl:190-217) stores one reduce to two outputs, write_monolithic_kernel_N
    (kernels.cl:423-560) copies one input to N: every destination must equal orc_reduce_n's result, also when a
    destination is one of the sources, and one input in pairwise mode must come back byte for byte."""
    rng = np.random.default_rng(77)
    for dtype, op, n, m in [(O.BFLOAT16, O.SUM, 2, 2), (O.FLOAT32, O.MAX, 3, 4), (O.INT8, O.PROD, 8, 7),
                            (O.FLOAT16, O.MIN, 5, 1)]:
        np_t = O.NP_STORAGE[dtype]
        srcs = [rng.integers(0, 256, 1003 * np.dtype(np_t).itemsize, dtype=np.uint8).view(np_t) for _ in range(n)]
        if dtype == O.FLOAT32:
            srcs = [rng.standard_normal(1003).astype(np.float32) for _ in range(n)]
        want = O.reduce_n(srcs, dtype, op)
        for alias in (None, (m - 1, n - 1)):
            outs = O.reduce_write_n(srcs, m, dtype, op, alias=alias)
            for o in outs:
                assert O.same_bits(o, want, dtype).all()
    src = rng.integers(0, 65536, 517, dtype=np.uint16)      # any bf16 bit pattern, NaNs and denormals included
    for o in O.reduce_write_n([src], 7, O.BFLOAT16, O.SUM):
        assert (o == src).all()
    # closed form of the reference's functional tests (test_impl.hpp:242-324): rank r sends r + i
    n, cnt = 8, 64
    srcs = [(np.arange(cnt) % 5 + r).astype(np.float32) for r in range(n)]
    for o in O.reduce_write_n(srcs, 8, O.FLOAT32, O.SUM):
        assert (o == n * (n - 1) / 2 + n * (np.arange(cnt) % 5)).all()


def _fp16_native_cases(golden, native):
    """(name, op, in, inout, want) for every case of the avx512fp16 fixture"""
    for key in native.files:
        if not key.endswith("_impl4"):
            continue
        stem = key[:-len("_impl4")]
        if stem.startswith("fp16_specials_") or stem.startswith("fp16_grid_"):
            fam = "specials" if "specials" in stem else "grid"
            op = O.OP_NAMES.index(stem.split("_")[2])
            src = golden if fam == "specials" else native
            yield stem, op, src[f"fp16_{fam}_in"], src[f"fp16_{fam}_inout"], native[key]
        else:
            op = O.OP_NAMES.index(stem.split("_")[1])
            yield stem, op, golden[stem + "_in"], golden[stem + "_inout"], native[key]


def test_fp16_avx512fp16_against_reference_made_vectors(golden, golden_fp16_native):
    """The native-fp16 implementation (fp16_intrisics.cpp:23-41): min/max return one operand untouched, so bits
    are compared, signalling NaNs included; sum/prod compare on bits too, except where both operands are NaNs."""
    n = 0
    for name, op, a, b, want in _fp16_native_cases(golden, golden_fp16_native):
        got = O.comp_reduce(a, b, O.FLOAT16, op, fp16_impl=O.FP16_AVX512FP16)
        if op in (O.MIN, O.MAX):
            assert (got == want).all(), (name, np.flatnonzero(got != want)[:8])
        else:
            assert O.same_bits(got, want, O.FLOAT16, [b, a], op, fp16_impl=O.FP16_AVX512FP16).all(), name
        n += 1
    assert n == 4 * 11 * 2 + 4 + 4
    # and the point of the mode: a signalling NaN handed back by min/max stays signalling, the other modes quiet it
    a = np.array([0x7C01], np.uint16)
    b = np.array([0x3C00], np.uint16)
    assert O.comp_reduce(b, a, O.FLOAT16, O.MIN, fp16_impl=O.FP16_AVX512FP16)[0] == 0x7C01
    assert O.comp_reduce(b, a, O.FLOAT16, O.MIN, fp16_impl=O.FP16_AVX512F)[0] == 0x7E01


def test_fp16_avx512fp16_against_reference_library_when_built():
    """Direct comparison with the reference's code compiled in place (oracle/_ref, clang build) on a million random
    pairs per op; skipped where that library or the CPU feature is absent (the fixture test above still runs)."""
    import ctypes as C
    so = os.path.join(os.path.dirname(O.REF_SO), "libccl_comp_ref_avx512fp16.so")
    if not os.path.exists(so):
        pytest.skip("oracle/_ref/libccl_comp_ref_avx512fp16.so not built")
    R = C.CDLL(so)
    R.ref_fp16_reduce.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_int, C.c_int]
    if not (R.ref_cpu_support() & 8):
        pytest.skip("CPU without avx512_fp16")
    rng = np.random.default_rng(99)
    for op in range(4):
        a = rng.integers(0, 65536, 1_000_003, dtype=np.uint16)
        b = rng.integers(0, 65536, 1_000_003, dtype=np.uint16)
        want = b.copy()
        assert R.ref_fp16_reduce(a.ctypes.data, a.size, want.ctypes.data, op, 4) == 0
        got = O.comp_reduce(a, b, O.FLOAT16, op, fp16_impl=O.FP16_AVX512FP16)
        if op in (O.MIN, O.MAX):
            assert (got == want).all()
        else:
            assert O.same_bits(got, want, O.FLOAT16, [b, a], op, fp16_impl=O.FP16_AVX512FP16).all()


@pytest.mark.parametrize("dtype", [O.FLOAT32, O.FLOAT64, O.BFLOAT16, O.FLOAT16])
def test_nan_results_of_sum_and_prod_follow_the_x86_rules(dtype):
    """Literal expected patterns (tests/nan_cases.py): a NaN operand comes back quieted, an invalid operation gives
    the negative default NaN -- for every implementation of the 16-bit types, pairwise and keep-precision, and as
    the first NaN of a longer chain."""
    import nan_cases
    impls = {O.BFLOAT16: [dict(bf16_impl=i) for i in (0, 1, 2)], O.FLOAT16: [dict(fp16_impl=i) for i in (2, 3, 4)]}
    for op in (O.SUM, O.PROD):
        a, b, want = nan_cases.table(dtype, op)
        for kw in impls.get(dtype, [{}]):
            got = O.comp_reduce(a, b, dtype, op, **kw)
            assert O.same_bits(got, want, dtype).all(), (op, kw, got, want)
            # the same pair as the first two inputs of a chain: the NaN travels to the end unchanged
            one = np.ones_like(a) if dtype in (O.FLOAT32, O.FLOAT64) else np.full_like(a, 0x3F80 if dtype == O.BFLOAT16 else 0x3C00)
            got3 = O.reduce_n([b, a, one, one], dtype, op, **kw)
            nan = O.nan_mask(want, dtype)
            assert O.same_bits(got3[nan], want[nan], dtype).all(), (op, kw)
            if dtype == O.BFLOAT16:
                gk = O.reduce_n([b, a, one], dtype, op, keep=1, **kw)
                assert O.same_bits(gk[nan], want[nan], dtype).all(), (op, kw, "keep")


@pytest.mark.parametrize("dtype", [O.FLOAT32, O.FLOAT64, O.BFLOAT16, O.FLOAT16])
def test_ambiguity_mask_marks_exactly_the_steps_with_two_nan_operands(dtype):
    """same_bits lets two different NaNs pass only where a chain step had two NaN operands."""
    import nan_cases
    sp = nan_cases.specials(dtype)
    a, b = np.repeat(sp, sp.size), np.tile(sp, sp.size)
    want = O.comp_reduce(a, b, dtype, O.SUM)
    other = want.copy()
    u = other.view({2: np.uint16, 4: np.uint32, 8: np.uint64}[other.dtype.itemsize])
    nan = O.nan_mask(want, dtype)
    u[nan] ^= 1                              # another payload for every NaN result
    ok = O.same_bits(other, want, dtype, [b, a], O.SUM)
    both = O.nan_mask(a, dtype) & O.nan_mask(b, dtype)
    assert (ok == (~nan | both)).all()
    assert both.sum() == 49 and (nan & ~both).sum() > 0

