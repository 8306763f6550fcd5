"""Writes tests/golden/ref_vectors.npz from the reference's own vector reduce code.

Run in the build container only (needs oracle/_ref/libccl_comp_ref.so, i.e. `make -C oracle ref` with the
reference tree present, on a CPU with AVX512F/BW/VL, AVX512_BF16 and F16C):

    python tests/golden/make_golden.py

Every case is (in, inout_before) -> inout_after for one call of the reference's
ccl_bf16_reduce_impl_{avx512f,avx512bf} (src/comp/bf16/bf16_intrisics.hpp:106-114) or
ccl_fp16_reduce_impl_{256,512} (src/comp/fp16/fp16_intrisics.hpp:186-196), plus 16-element converter
blocks (bf16_intrisics.hpp:62-76).  Inputs mix seeded random bit patterns with the special values of each
format.  The file holds data only.
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import oracle_lib as O  # noqa: E402

COUNTS = [1, 7, 8, 9, 15, 16, 17, 31, 32, 33, 1000]

BF16_SPECIALS = np.array([0x0000, 0x8000, 0x0001, 0x8001, 0x007F, 0x0080, 0x3F80, 0xBF80, 0x7F7F, 0xFF7F,
                          0x7F80, 0xFF80, 0x7FC0, 0xFFC0, 0x7F81, 0x7FBF, 0x3B80, 0x3BC0, 0x3C40, 0x0040],
                         dtype=np.uint16)
FP16_SPECIALS = np.array([0x0000, 0x8000, 0x0001, 0x8001, 0x03FF, 0x0400, 0x3C00, 0xBC00, 0x7BFF, 0xFBFF,
                          0x7C00, 0xFC00, 0x7E00, 0xFE00, 0x7C01, 0x7DFF, 0x1000, 0x1200, 0x3C01, 0x0200],
                         dtype=np.uint16)


def make_inputs(rng, count, specials, kind):
    """kind 0: any bit pattern; kind 1: moderate finite values; both get specials sprinkled in."""
    if kind == 0:
        a = rng.integers(0, 65536, size=count, dtype=np.uint16)
        b = rng.integers(0, 65536, size=count, dtype=np.uint16)
    else:
        # sign + exponent within a few binades of 1.0 + random mantissa: sums round, products stay finite
        if specials is BF16_SPECIALS:
            a = (rng.integers(0x3E00, 0x4100, size=count) | (rng.integers(0, 2, size=count) << 15)).astype(np.uint16)
            b = (rng.integers(0x3E00, 0x4100, size=count) | (rng.integers(0, 2, size=count) << 15)).astype(np.uint16)
        else:
            a = (rng.integers(0x3000, 0x4400, size=count) | (rng.integers(0, 2, size=count) << 15)).astype(np.uint16)
            b = (rng.integers(0x3000, 0x4400, size=count) | (rng.integers(0, 2, size=count) << 15)).astype(np.uint16)
    k = min(count, len(specials))
    pos = rng.permutation(count)[:k]
    a[pos] = rng.permutation(specials)[:k]
    pos = rng.permutation(count)[:k]
    b[pos] = rng.permutation(specials)[:k]
    return a, b


def main():
    R = O.ref()
    if R is None or (O.ref_cpu_support() & 7) != 7:
        sys.exit("needs oracle/_ref/libccl_comp_ref.so and a CPU with avx512f/bw/vl, avx512_bf16, f16c")
    rng = np.random.default_rng(20211400)
    out = {}
    for fam, impls, specials, fn in (("bf16", (1, 2), BF16_SPECIALS, R.ref_bf16_reduce),
                                     ("fp16", (2, 3), FP16_SPECIALS, R.ref_fp16_reduce)):
        for op in range(4):
            for count in COUNTS:
                for kind in (0, 1):
                    a, b = make_inputs(rng, count, specials, kind)
                    key = f"{fam}_{O.OP_NAMES[op]}_n{count}_k{kind}"
                    out[key + "_in"] = a
                    out[key + "_inout"] = b
                    for impl in impls:
                        r = b.copy()
                        rc = fn(a.ctypes.data, count, r.ctypes.data, op, impl)
                        assert rc == 0
                        out[key + f"_impl{impl}"] = r
    # every (in, inout) pair of special values, all ops, all impls
    for fam, impls, specials, fn in (("bf16", (1, 2), BF16_SPECIALS, R.ref_bf16_reduce),
                                     ("fp16", (2, 3), FP16_SPECIALS, R.ref_fp16_reduce)):
        a = np.repeat(specials, len(specials))
        b = np.tile(specials, len(specials))
        out[f"{fam}_specials_in"] = a
        out[f"{fam}_specials_inout"] = b
        for op in range(4):
            for impl in impls:
                r = b.copy()
                assert fn(a.ctypes.data, a.size, r.ctypes.data, op, impl) == 0
                out[f"{fam}_specials_{O.OP_NAMES[op]}_impl{impl}"] = r
    # converter blocks: 64 blocks of 16 fp32 patterns (random + edge patterns)
    edge = np.array([0x00000000, 0x80000000, 0x00000001, 0x007FFFFF, 0x00800000, 0x3F800000, 0x3F808000,
                     0x3F818000, 0x3F807FFF, 0x3F808001, 0x7F7FFFFF, 0x7F7F8000, 0x7F800000, 0xFF800000,
                     0x7F800001, 0x7FC00000, 0xFFC12345, 0x7FBFFFFF, 0x3F80FFFF, 0x477FE000, 0x477FF000,
                     0x38800000, 0x387FFFFF, 0x33000000, 0x33000001, 0x32FFFFFF, 0x33800000, 0x00000000,
                     0x3B800000, 0x3BC00000, 0x3C400000, 0x80000001], dtype=np.uint32)
    f32 = np.concatenate([edge, rng.integers(0, 2**32, size=64 * 16 - edge.size, dtype=np.uint32)])
    out["cvt_fp32_in"] = f32
    for impl in (1, 2):
        res = np.empty(f32.size, np.uint16)
        for blk in range(0, f32.size, 16):
            assert R.ref_fp32_store_as_bf16_16(f32[blk:].ctypes.data, res[blk:].ctypes.data, impl) == 0
        out[f"cvt_fp32_to_bf16_impl{impl}"] = res
    h = rng.integers(0, 65536, size=64 * 16, dtype=np.uint16)
    h[:BF16_SPECIALS.size] = BF16_SPECIALS
    w = np.empty(h.size, np.uint32)
    for blk in range(0, h.size, 16):
        assert R.ref_bf16_load_as_fp32_16(h[blk:].ctypes.data, w[blk:].ctypes.data) == 0
    out["cvt_bf16_in"] = h
    out["cvt_bf16_to_fp32"] = w
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, len(out), "arrays", os.path.getsize(path), "bytes")


def main_avx512fp16():
    """Second fixture, ref_vectors_avx512fp16.npz: the reference's native-fp16 reduce
    (ccl_fp16_reduce_impl_512FP16, src/comp/fp16/fp16_intrisics.hpp:150-200 with fp16_intrisics.cpp:23-41) on the
    float16 inputs of ref_vectors.npz, on every pair of the special values, and on every pair of 512 patterns that
    cover each exponent with its smallest and largest mantissa, both signs, quiet and signalling NaNs.  Needs
    oracle/_ref/libccl_comp_ref_avx512fp16.so (built by clang, which knows the AVX512-FP16 intrinsics that gcc 11
    lacks) and a CPU with avx512_fp16."""
    import ctypes as C
    here = os.path.dirname(os.path.abspath(__file__))
    so = os.path.join(os.path.dirname(os.path.dirname(here)), "oracle", "_ref", "libccl_comp_ref_avx512fp16.so")
    if not os.path.exists(so):
        sys.exit("needs " + so)
    R = C.CDLL(so)
    R.ref_fp16_reduce.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_int, C.c_int]
    if not (R.ref_cpu_support() & 8):
        sys.exit("needs a CPU with avx512_fp16")
    base = np.load(os.path.join(here, "ref_vectors.npz"))
    out = {}

    def run(a, b, op):
        r = b.copy()
        assert R.ref_fp16_reduce(a.ctypes.data, a.size, r.ctypes.data, op, 4) == 0
        return r

    for key in base.files:
        if key.startswith("fp16_") and key.endswith("_in"):
            stem = key[:-3]
            if "specials" in stem:
                for op in range(4):
                    out[f"fp16_specials_{O.OP_NAMES[op]}_impl4"] = run(base[key], base[stem + "_inout"], op)
            else:
                out[stem + "_impl4"] = run(base[key], base[stem + "_inout"], O.OP_NAMES.index(stem.split("_")[1]))
    pats = []
    for sign in (0, 0x8000):
        for e in range(32):
            for m in (0, 1, 0x1FF, 0x200, 0x201, 0x2AA, 0x3FE, 0x3FF):
                pats.append(sign | (e << 10) | m)
    pats = np.array(pats, dtype=np.uint16)
    a, b = np.repeat(pats, pats.size), np.tile(pats, pats.size)
    out["fp16_grid_in"], out["fp16_grid_inout"] = a, b
    for op in range(4):
        out[f"fp16_grid_{O.OP_NAMES[op]}_impl4"] = run(a, b, op)
    path = os.path.join(here, "ref_vectors_avx512fp16.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, len(out), "arrays", os.path.getsize(path), "bytes")


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "avx512fp16":
        main_avx512fp16()
        sys.exit(0)
    main()
