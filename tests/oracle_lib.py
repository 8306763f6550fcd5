"""ctypes access to the CPU oracle (oracle/libccl_comp_oracle.so) and, where it was built, to the
reference's own vector code (oracle/_ref/libccl_comp_ref.so).  Checker only: tests, the smoke check and
the CPU-baseline leg of the benchmark load this; the product never does."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "libccl_comp_oracle.so")
REF_SO = os.path.join(ORACLE_DIR, "_ref", "libccl_comp_ref.so")

# ccl::datatype (include/oneapi/ccl/types.hpp:52-69)
INT8, UINT8, INT16, UINT16, INT32, UINT32, INT64, UINT64, FLOAT16, FLOAT32, FLOAT64, BFLOAT16 = range(12)
# ccl::reduction (types.hpp:41-47)
SUM, PROD, MIN, MAX, CUSTOM = range(5)
# ccl_bf16_impl_type (src/comp/bf16/bf16_utils.hpp:26), ccl_fp16_impl_type (fp16_utils.hpp:26-32)
BF16_SCALAR, BF16_AVX512F, BF16_AVX512BF = 0, 1, 2
FP16_F16C, FP16_AVX512F, FP16_AVX512FP16 = 2, 3, 4

DTYPE_NAMES = ["int8", "uint8", "int16", "uint16", "int32", "uint32", "int64", "uint64",
               "float16", "float32", "float64", "bfloat16"]
OP_NAMES = ["sum", "prod", "min", "max"]
# storage dtype used on the numpy side (16-bit floats travel as raw uint16, like ccl::bfloat16/float16)
NP_STORAGE = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64,
              np.uint16, np.float32, np.float64, np.uint16]
DTYPE_SIZE = [1, 1, 2, 2, 4, 4, 8, 8, 2, 4, 8, 2]


def build_oracle():
    subprocess.check_call(["make", "-s", "-C", ORACLE_DIR, "all"])


_lib = None
_ref = None


def _vp(a):
    return a.ctypes.data_as(C.c_void_p)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_SO):
            build_oracle()
        L = C.CDLL(ORACLE_SO)
        L.orc_datatype_size.restype = C.c_size_t
        L.orc_datatype_size.argtypes = [C.c_int]
        L.orc_datatype_name.restype = C.c_char_p
        L.orc_datatype_name.argtypes = [C.c_int]
        L.orc_reduction_to_str.restype = C.c_char_p
        L.orc_reduction_to_str.argtypes = [C.c_int]
        for f in ("orc_bf16_widen", "orc_fp16_widen"):
            getattr(L, f).restype = C.c_uint32
            getattr(L, f).argtypes = [C.c_uint16]
        for f in ("orc_bf16_narrow_trunc", "orc_bf16_narrow_rne", "orc_fp16_narrow"):
            getattr(L, f).restype = C.c_uint16
            getattr(L, f).argtypes = [C.c_uint32]
        L.orc_convert_fp32_to_bf16_arrays.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        L.orc_convert_bf16_to_fp32_arrays.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        L.orc_convert_fp32_to_fp16_arrays.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.orc_convert_fp16_to_fp32_arrays.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.orc_bf16_reduce.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_int, C.c_int]
        L.orc_fp16_reduce.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_int, C.c_int]
        L.orc_comp_reduce.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int]
        L.orc_comp_batch_reduce.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p,
                                            C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int]
        L.orc_reduce_n.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int,
                                   C.c_int, C.c_int, C.c_int]
        L.orc_reduce_n_mt.argtypes = L.orc_reduce_n.argtypes + [C.c_int]
        L.orc_reduce_write_n.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_size_t, C.c_int, C.c_int,
                                         C.c_int, C.c_int, C.c_int, C.c_int]
        L.orc_comp_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.orc_fusion_offsets.restype = C.c_size_t
        L.orc_fusion_offsets.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p]
        L.orc_fusion_pack.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p]
        L.orc_fusion_unpack.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p]
        _lib = L
    return _lib


def ref():
    """The reference's own vector code, or None when oracle/_ref was not built or the CPU lacks AVX-512."""
    global _ref
    if _ref is None:
        if not os.path.exists(REF_SO):
            return None
        R = C.CDLL(REF_SO)
        R.ref_bf16_reduce.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_int, C.c_int]
        R.ref_fp16_reduce.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_int, C.c_int]
        R.ref_bf16_load_as_fp32_16.argtypes = [C.c_void_p, C.c_void_p]
        R.ref_fp32_store_as_bf16_16.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        if hasattr(R, "ref_batch_reduce_keep_sum"):
            R.ref_batch_reduce_keep_sum.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p,
                                                    C.c_void_p, C.c_void_p, C.c_int]
        _ref = R
    return _ref


def ref_cpu_support():
    r = ref()
    return r.ref_cpu_support() if r is not None else 0


# ---------------------------------------------------------------------------------------------
# numpy-level wrappers

def comp_reduce(inp, inout, dtype, op, bf16_impl=BF16_AVX512BF, fp16_impl=FP16_AVX512F):
    """inout = inout OP inp, in place on a copy; returns the result array (ccl_comp_reduce)."""
    out = np.ascontiguousarray(inout).copy()
    inp = np.ascontiguousarray(inp)
    assert inp.dtype == out.dtype and inp.size == out.size
    rc = lib().orc_comp_reduce(_vp(inp), inp.size, _vp(out), dtype, op, bf16_impl, fp16_impl)
    assert rc == 0, rc
    return out


def reduce_n(srcs, dtype, op, keep=0, quirk_tail=0, bf16_impl=BF16_AVX512BF, fp16_impl=FP16_AVX512F,
             threads=1):
    """N separate buffers, own first then peers in order; returns a new array."""
    srcs = [np.ascontiguousarray(s) for s in srcs]
    n = len(srcs)
    count = srcs[0].size
    out = np.empty_like(srcs[0])
    ptrs = (C.c_void_p * n)(*[s.ctypes.data for s in srcs])
    if threads > 1:
        rc = lib().orc_reduce_n_mt(ptrs, n, _vp(out), count, dtype, op, keep, quirk_tail, bf16_impl,
                                   fp16_impl, threads)
    else:
        rc = lib().orc_reduce_n(ptrs, n, _vp(out), count, dtype, op, keep, quirk_tail, bf16_impl, fp16_impl)
    assert rc == 0, rc
    return out


def reduce_write_n(srcs, m, dtype, op, keep=0, quirk_tail=0, bf16_impl=BF16_AVX512BF, fp16_impl=FP16_AVX512F,
                   alias=None):
    """The N-input reduce stored to m buffers; returns the m arrays.  alias = (k, j): destination k IS source j
    (a private copy of the sources is reduced, so the caller's arrays stay as they were)."""
    srcs = [np.ascontiguousarray(s).copy() for s in srcs]
    outs = [np.empty_like(srcs[0]) for _ in range(m)]
    if alias is not None:
        outs[alias[0]] = srcs[alias[1]]
    sp = (C.c_void_p * len(srcs))(*[s.ctypes.data for s in srcs])
    dp = (C.c_void_p * m)(*[o.ctypes.data for o in outs])
    rc = lib().orc_reduce_write_n(sp, len(srcs), dp, m, srcs[0].size, dtype, op, keep, quirk_tail, bf16_impl,
                                  fp16_impl)
    assert rc == 0, rc
    return outs


def batch_reduce(buf, offsets, count, dtype, op, keep, bf16_impl=BF16_AVX512BF, fp16_impl=FP16_AVX512F):
    """ccl_comp_batch_reduce over slices of one buffer; slice offsets[0] is inout.  Returns the buffer copy."""
    buf = np.ascontiguousarray(buf).copy()
    offs = np.asarray(offsets, dtype=np.uint64)
    tmp = np.empty(count, np.float32)
    acc = np.empty(count, np.float32)
    esz = DTYPE_SIZE[dtype]
    inout_ptr = C.c_void_p(buf.ctypes.data + int(offs[0]) * esz)
    rc = lib().orc_comp_batch_reduce(_vp(buf), _vp(offs), len(offs), count, inout_ptr, dtype, op, keep,
                                     _vp(tmp), _vp(acc), bf16_impl, fp16_impl)
    assert rc == 0, rc
    return buf


def fusion_offsets(counts, dtype_size, align):
    counts = np.asarray(counts, dtype=np.uint64)
    offs = np.empty(len(counts), dtype=np.uint64)
    total = lib().orc_fusion_offsets(_vp(counts), len(counts), dtype_size, align, _vp(offs))
    return offs, int(total)


def fusion_pack(tensors, byte_offsets, total_bytes, dtype_size):
    k = len(tensors)
    tensors = [np.ascontiguousarray(t) for t in tensors]
    counts = np.asarray([t.size for t in tensors], dtype=np.uint64)
    offs = np.asarray(byte_offsets, dtype=np.uint64)
    buf = np.zeros(total_bytes, dtype=np.uint8)
    ptrs = (C.c_void_p * k)(*[t.ctypes.data for t in tensors])
    lib().orc_fusion_pack(ptrs, _vp(counts), _vp(offs), k, dtype_size, _vp(buf))
    return buf


def fusion_unpack(buf, counts, byte_offsets, np_dtype):
    k = len(counts)
    dtype_size = np.dtype(np_dtype).itemsize
    outs = [np.empty(int(c), dtype=np_dtype) for c in counts]
    cnt = np.asarray(counts, dtype=np.uint64)
    offs = np.asarray(byte_offsets, dtype=np.uint64)
    ptrs = (C.c_void_p * k)(*[t.ctypes.data for t in outs])
    lib().orc_fusion_unpack(_vp(np.ascontiguousarray(buf)), _vp(cnt), _vp(offs), k, dtype_size, ptrs)
    return outs


def bf16_from_f32(x):
    """fp32 array -> raw bf16 bits, round to nearest even.  Input generation only (not a check)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    e = u & 0x7F800000
    m = u & 0x007FFFFF
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF
    r = np.where(e == 0, (u >> 16) & 0x8000, r)
    r = np.where((e == 0x7F800000) & (m != 0), ((u >> 16) | 0x40) & 0xFFFF, r)
    return r.astype(np.uint16).reshape(x.shape)


def bf16_to_f32(h):
    return (np.asarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def nan_mask(a, dtype):
    """Which elements are NaNs (16-bit floats travel as raw uint16)."""
    a = np.asarray(a)
    if dtype == FLOAT32:
        return (a.view(np.uint32) & 0x7FFFFFFF) > 0x7F800000
    if dtype == FLOAT64:
        return (a.view(np.uint64) & 0x7FFFFFFFFFFFFFFF) > 0x7FF0000000000000
    if dtype == BFLOAT16:
        return (a & 0x7FFF) > 0x7F80
    if dtype == FLOAT16:
        return (a & 0x7FFF) > 0x7C00
    return np.zeros(a.shape, bool)


def two_nan_steps(srcs, dtype, op, idx, **kw):
    """Of the elements idx: those at which some step of the chain srcs[0] OP srcs[1] OP ... has two NaN operands.
    Only there is the result's payload not fixed by the reference (which of two NaN operands an x86 add or
    multiply hands back depends on the operand order its compiler chose)."""
    kw = dict(kw)
    kw.pop("quirk_tail", None)      # how the tail is narrowed does not change which values are NaNs
    sub = [np.ascontiguousarray(np.asarray(s)[idx]) for s in srcs]
    amb = np.zeros(len(idx), bool)
    acc_nan = nan_mask(sub[0], dtype)
    for j in range(1, len(sub)):
        amb |= acc_nan & nan_mask(sub[j], dtype)
        acc_nan = nan_mask(reduce_n(sub[:j + 1], dtype, op, **kw), dtype)
    return amb


def same_bits(got, want, dtype, srcs=None, op=None, **kw):
    """Bit equality per element.  The one exception: with srcs (the inputs in chain order, inout first) and op sum or
    prod of a floating type, two NaNs also compare equal at elements where a step of the chain had two NaN
    operands.  A NaN made from one NaN operand (that operand, quieted) or from none (the negative default NaN of
    x86) is compared on bits like any other value.  kw: keep, bf16_impl, fp16_impl as for reduce_n."""
    got = np.asarray(got)
    want = np.asarray(want)
    u = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[got.dtype.itemsize]
    eq = got.view(u) == want.view(u)
    if eq.all() or srcs is None or op not in (SUM, PROD) or dtype not in (FLOAT16, FLOAT32, FLOAT64, BFLOAT16):
        return eq
    bad = np.flatnonzero(~eq.ravel())
    cand = bad[nan_mask(got.ravel()[bad], dtype) & nan_mask(want.ravel()[bad], dtype)]
    if cand.size:
        amb = two_nan_steps([np.asarray(s).ravel() for s in srcs], dtype, op, cand, **kw)
        eq = eq.copy()
        eq.ravel()[cand[amb]] = True
    return eq
