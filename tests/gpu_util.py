"""Helpers shared by the GPU parity tests: seeded inputs per dtype, host<->device moves that keep bits."""
import numpy as np

import oracle_lib as O

SIGNED_VIEW = {np.dtype(np.uint16): np.int16, np.dtype(np.uint32): np.int32, np.dtype(np.uint64): np.int64}


def to_dev(a):
    """numpy array -> cuda tensor with the same bytes (unsigned 16/32/64 travel as the signed twin)."""
    import torch
    a = np.ascontiguousarray(a)
    v = a.view(SIGNED_VIEW[a.dtype]) if a.dtype in SIGNED_VIEW else a
    return torch.from_numpy(v.copy()).cuda()


def to_host(t, np_dtype):
    return t.cpu().numpy().view(np_dtype)


def make_inputs(rng, dtype, count, op, n, kind="config"):
    """n seeded input arrays.  kind "config": the value ranges the benchmark configurations use (ints over
    the full range, floats uniform[-2,2], prod uniform[0.9,1.1], 16-bit floats via RNE casts);
    kind "bits": arbitrary bit patterns (NaNs, infinities, denormals included) for the 16-bit types."""
    np_t = O.NP_STORAGE[dtype]
    out = []
    for _ in range(n):
        if dtype in (O.FLOAT32, O.FLOAT64):
            lo, hi = (0.9, 1.1) if op == O.PROD else (-2.0, 2.0)
            out.append(rng.uniform(lo, hi, count).astype(np_t))
        elif dtype == O.FLOAT16:
            if kind == "bits":
                out.append(rng.integers(0, 65536, count, dtype=np.uint16))
            else:
                lo, hi = (0.9, 1.1) if op == O.PROD else (-2.0, 2.0)
                out.append(rng.uniform(lo, hi, count).astype(np.float16).view(np.uint16))
        elif dtype == O.BFLOAT16:
            if kind == "bits":
                out.append(rng.integers(0, 65536, count, dtype=np.uint16))
            else:
                x = rng.uniform(0.9, 1.1, count) if op == O.PROD else rng.standard_normal(count)
                out.append(O.bf16_from_f32(x.astype(np.float32)))
        else:
            info = np.iinfo(np_t)
            out.append(rng.integers(info.min, info.max, count, dtype=np_t, endpoint=True))
    return out


def assert_same(got, want, dtype, what="", srcs=None, op=None, **kw):
    """Bit equality; with srcs (chain order) and op given, NaN results of sum/prod steps that had two NaN operands
    compare as a class (oracle_lib.same_bits)."""
    ok = O.same_bits(got, want, dtype, srcs, op, **kw)
    if not ok.all():
        bad = np.flatnonzero(~ok)
        raise AssertionError(f"{what}: {bad.size} of {ok.size} elements differ, first at {bad[:5]}: "
                             f"got {got[bad[:5]]} want {want[bad[:5]]}")
