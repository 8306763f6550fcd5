"""NaN results of sum and prod, written out as literal bit patterns.

The reference computes with SSE/AVX instructions (ADDPS/MULPS, ADDSD/MULSD, VADDPH/VMULPH; src/comp/comp.cpp:37-44,
src/comp/bf16/bf16_intrisics.hpp:80-87, src/comp/fp16/fp16_intrisics.hpp:95-176), whose NaN rules are fixed by the
instruction set: a NaN operand comes back with its quiet bit set (sign and payload kept), and an invalid operation
(Inf + -Inf, 0 x Inf) gives the "real indefinite" quiet NaN, whose sign bit is SET.  The 16-bit types widen first
(bf16: << 16; fp16: VCVTPH2PS, which quiets) and narrow afterwards (truncation or VCVTNEPS2BF16 keep the top of the
payload, VCVTPS2PH likewise).  Each case: (op, in, inout, expected), hex patterns of the storage type.
"""
import numpy as np

import oracle_lib as O

F32 = [
    (O.SUM, 0x7F800000, 0xFF800000, 0xFFC00000),    # Inf + -Inf
    (O.SUM, 0xFF800000, 0x7F800000, 0xFFC00000),
    (O.PROD, 0x00000000, 0x7F800000, 0xFFC00000),   # 0 x Inf
    (O.PROD, 0xFF800000, 0x80000000, 0xFFC00000),   # -Inf x -0
    (O.SUM, 0x7FC12345, 0x3F800000, 0x7FC12345),    # quiet NaN + 1: the NaN, untouched
    (O.SUM, 0x3F800000, 0xFFC00001, 0xFFC00001),    # 1 + negative quiet NaN
    (O.SUM, 0x7F812345, 0x3F800000, 0x7FC12345),    # signalling NaN + 1: quieted, payload kept
    (O.PROD, 0x40000000, 0xFF800001, 0xFFC00001),   # 2 x negative signalling NaN
    (O.PROD, 0x7FA00000, 0x00000000, 0x7FE00000),   # signalling NaN x 0
    (O.SUM, 0x7F800000, 0x7F800000, 0x7F800000),    # Inf + Inf stays Inf
]
F64 = [
    (O.SUM, 0x7FF0000000000000, 0xFFF0000000000000, 0xFFF8000000000000),
    (O.PROD, 0x8000000000000000, 0x7FF0000000000000, 0xFFF8000000000000),
    (O.SUM, 0x7FF8000000012345, 0x3FF0000000000000, 0x7FF8000000012345),
    (O.SUM, 0x3FF0000000000000, 0xFFF0000000000001, 0xFFF8000000000001),
    (O.PROD, 0x7FF4000000000000, 0x4000000000000000, 0x7FFC000000000000),
]
BF16 = [    # the same for every bf16 implementation (scalar, avx512f, avx512bf) and for keep-precision
    (O.SUM, 0x7F80, 0xFF80, 0xFFC0),
    (O.PROD, 0x0000, 0xFF80, 0xFFC0),
    (O.SUM, 0x7FC5, 0x3F80, 0x7FC5),
    (O.SUM, 0x3F80, 0xFF81, 0xFFC1),
    (O.PROD, 0x7FA3, 0x4000, 0x7FE3),
]
FP16 = [    # the same for f16c, avx512f and avx512fp16
    (O.SUM, 0x7C00, 0xFC00, 0xFE00),
    (O.PROD, 0x8000, 0x7C00, 0xFE00),
    (O.SUM, 0x7E05, 0x3C00, 0x7E05),
    (O.SUM, 0x3C00, 0xFC01, 0xFE01),
    (O.PROD, 0x7D03, 0x4000, 0x7F03),
]
TABLES = {O.FLOAT32: (F32, np.uint32), O.FLOAT64: (F64, np.uint64), O.BFLOAT16: (BF16, np.uint16), O.FLOAT16: (FP16, np.uint16)}


def table(dtype, op):
    """(in, inout, expected) arrays in the storage type the oracle wrappers and the device helpers use."""
    rows, u = TABLES[dtype]
    rows = [r for r in rows if r[0] == op]
    np_t = O.NP_STORAGE[dtype]
    cols = [np.array([r[k] for r in rows], dtype=u).view(np_t) for k in (1, 2, 3)]
    return cols


def specials(dtype):
    """Special values of a floating type (storage type): NaNs of both kinds and signs with assorted payloads,
    infinities, zeros, denormals, extremes, a few ordinary values."""
    if dtype == O.FLOAT32:
        v = [0x7FC00000, 0xFFC00000, 0x7FC00001, 0x7F800001, 0xFF812345, 0x7FFFFFFF, 0xFFA00000, 0x7F800000, 0xFF800000,
             0x00000000, 0x80000000, 0x00000001, 0x807FFFFF, 0x7F7FFFFF, 0xFF7FFFFF, 0x3F800000, 0xBF800000, 0x40490FDB,
             0x00800000, 0x7F000000]
        return np.array(v, np.uint32).view(np.float32)
    if dtype == O.FLOAT64:
        v = [0x7FF8000000000000, 0xFFF8000000000000, 0x7FF8000000000001, 0x7FF0000000000001, 0xFFF0000000012345,
             0x7FFFFFFFFFFFFFFF, 0xFFF4000000000000, 0x7FF0000000000000, 0xFFF0000000000000, 0x0000000000000000,
             0x8000000000000000, 0x0000000000000001, 0x800FFFFFFFFFFFFF, 0x7FEFFFFFFFFFFFFF, 0xFFEFFFFFFFFFFFFF,
             0x3FF0000000000000, 0xBFF0000000000000, 0x400921FB54442D18, 0x0010000000000000, 0x7FE0000000000000]
        return np.array(v, np.uint64).view(np.float64)
    if dtype == O.BFLOAT16:
        v = [0x7FC0, 0xFFC0, 0x7FC1, 0x7F81, 0xFF95, 0x7FFF, 0xFFA0, 0x7F80, 0xFF80, 0x0000, 0x8000, 0x0001, 0x807F,
             0x7F7F, 0xFF7F, 0x3F80, 0xBF80, 0x4049, 0x0080, 0x7F00]
        return np.array(v, np.uint16)
    if dtype == O.FLOAT16:
        v = [0x7E00, 0xFE00, 0x7E01, 0x7C01, 0xFD23, 0x7FFF, 0xFD00, 0x7C00, 0xFC00, 0x0000, 0x8000, 0x0001, 0x83FF,
             0x7BFF, 0xFBFF, 0x3C00, 0xBC00, 0x4248, 0x0400, 0x7800]
        return np.array(v, np.uint16)
    raise ValueError(dtype)
