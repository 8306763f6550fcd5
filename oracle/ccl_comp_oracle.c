/*
 * TEST INFRASTRUCTURE ONLY -- never linked into, imported by or executed from the product.
 *
 * CPU restatement of oneCCL's reduction arithmetic (reference paths are relative to the
 * reference tree's root).  Build: see oracle/Makefile (-O2 -ffp-contract=off, no fast-math).
 *
 * Pinning status (what fixes each function's bits independently of this file):
 *   orc_bf16_widen / narrow_trunc   exhaustive vs shifts; vs reference load/store helpers (oracle/_ref)
 *   orc_bf16_narrow_rne             exhaustive 2^32 vs VCVTNEPS2BF16 on an AVX512_BF16 host
 *                                   (oracle/selfcheck.c), vs reference store helper (oracle/_ref), KATs
 *   orc_fp16_widen / orc_fp16_narrow exhaustive 2^16 / 2^32 vs F16C VCVTPH2PS / VCVTPS2PH
 *                                   (oracle/selfcheck.c), numpy float16, KATs
 *   orc_bf16_reduce (avx512f/bf)    reference ccl_bf16_reduce_impl_* compiled in place (oracle/_ref),
 *                                   golden vectors made from it, recorded probe values
 *   orc_bf16_reduce (scalar)        composition of pinned converters + std::min/max truth table
 *                                   (recorded probe values of the reference library)
 *   orc_fp16_reduce (f16c/avx512f)  reference ccl_fp16_reduce_impl_256/_512 compiled in place, golden
 *   orc_fp16_reduce (avx512fp16)    reference ccl_fp16_reduce_impl_512FP16 compiled in place with clang (gcc 11 lacks the
 *                                   AVX512-FP16 intrinsics): all 2^32 (in, inout) pairs of every op compared once
 *                                   (bit-exact for min/max, NaN payloads aside for sum/prod), golden vectors made
 *                                   from it (tests/golden/ref_vectors_avx512fp16.npz)
 *   orc_comp_reduce plain types     IEEE single op per pair / two's-complement wrap: numpy closed forms,
 *                                   min/max truth table recorded from the reference library
 *   orc_convert_*_arrays tail       recorded probe values of the reference library (tail truncation)
 *   orc_convert_fp32_to_fp16_arrays / fp16_to_fp32: loops over orc_fp16_narrow / orc_fp16_widen (pinned above)
 *   orc_comp_batch_reduce           composition; recorded probe values (1+3*2^-8 -> 3f82 body / 3f81 tail); the
 *                                   keep-precision sum against the reference's own 16-wide converters called in
 *                                   the reference's pass order (oracle/_ref, ref_batch_reduce_keep_sum) on random
 *                                   bit patterns and gradient-like values, 1..9 slices
 *   orc_fusion_*                    pack/unpack round trip, offsets closed form
 *   orc_reduce_write_n              composition of orc_reduce_n (pinned above) and memcpy: every destination equals
 *                                   orc_reduce_n's output; closed forms of the reference's functional tests
 *   NaN results of sum/prod         the host's own SSE/AVX add and multiply, as in the reference: a NaN operand comes
 *                                   back quieted, an invalid operation gives the negative default NaN -- literal patterns
 *                                   in tests/nan_cases.py, golden special-value pairs made by oracle/_ref.  Only a step
 *                                   with TWO NaN operands is not pinned (which one comes back follows the operand order
 *                                   the compiler chose, here as in the reference); tests compare those as NaN == NaN.
 */
#define _GNU_SOURCE
#include "ccl_comp_oracle.h"

#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------ */
/* datatype / reduction tables                                                                 */

size_t orc_datatype_size(int dtype) { /* datatype.cpp:79-91 */
    static const size_t sz[ORC_DTYPE_LAST] = { 1, 1, 2, 2, 4, 4, 8, 8, 2, 4, 8, 2 };
    return (dtype >= 0 && dtype < ORC_DTYPE_LAST) ? sz[dtype] : 0;
}

const char* orc_datatype_name(int dtype) { /* datatype.cpp:94-106 */
    static const char* nm[ORC_DTYPE_LAST] = { "int8",  "uint8",  "int16",   "uint16",  "int32",   "uint32",
                                              "int64", "uint64", "float16", "float32", "float64", "bfloat16" };
    return (dtype >= 0 && dtype < ORC_DTYPE_LAST) ? nm[dtype] : "";
}

const char* orc_reduction_to_str(int op) { /* comp.cpp:251-260 */
    switch (op) {
        case ORC_SUM: return "sum";
        case ORC_PROD: return "prod";
        case ORC_MIN: return "min";
        case ORC_MAX: return "max";
        case ORC_CUSTOM: return "custom";
        default: return "unknown";
    }
}

/* ------------------------------------------------------------------------------------------ */
/* bit helpers                                                                                 */

static inline float u2f(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint32_t f2u(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

/* bf16 -> fp32: value << 16, exact.  bf16.cpp:56-61 (scalar), bf16_intrisics.hpp:62-65 (vector). */
uint32_t orc_bf16_widen(uint16_t h) {
    return (uint32_t)h << 16;
}

/* fp32 -> bf16 by dropping the low half.  bf16.cpp:50-54 (scalar), bf16_intrisics.hpp:67-70 (avx512f). */
uint16_t orc_bf16_narrow_trunc(uint32_t u) {
    return (uint16_t)(u >> 16);
}

/* fp32 -> bf16 as _mm512_cvtneps_pbh does it (bf16_intrisics.hpp:73-75): round to nearest even,
 * fp32 denormals read as zero, NaN quieted with its top payload bits kept, overflow rounds to Inf. */
uint16_t orc_bf16_narrow_rne(uint32_t u) {
    uint32_t e = u & 0x7f800000u, m = u & 0x007fffffu;
    if (e == 0)
        return (uint16_t)((u >> 16) & 0x8000u);
    if (e == 0x7f800000u && m != 0)
        return (uint16_t)((u >> 16) | 0x0040u);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

/* fp16 -> fp32 as VCVTPH2PS (fp16_intrisics.hpp:100-101,128-129): exact; subnormals normalised,
 * signalling NaN quieted. */
uint32_t orc_fp16_widen(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    if (e == 0x1f)
        return sign | 0x7f800000u | (m << 13) | (m ? 0x00400000u : 0u);
    if (e == 0) {
        if (m == 0)
            return sign;
        int s = 0;
        while (!(m & 0x400u)) {
            m <<= 1;
            s++;
        }
        return sign | ((uint32_t)(113 - s) << 23) | ((m & 0x3ffu) << 13);
    }
    return sign | ((e + 112u) << 23) | (m << 13);
}

/* fp32 -> fp16 as VCVTPS2PH with imm8 = 0 (fp16_intrisics.hpp:103,132): round to nearest even,
 * results below the normal range become fp16 subnormals (not flushed), overflow -> Inf, NaN quieted. */
uint16_t orc_fp16_narrow(uint32_t u) {
    uint32_t sign = (u >> 16) & 0x8000u, x = u & 0x7fffffffu;
    if (x > 0x7f800000u)
        return (uint16_t)(sign | 0x7e00u | ((x >> 13) & 0x1ffu));
    if (x >= 0x47800000u)
        return (uint16_t)(sign | 0x7c00u);
    if (x < 0x38800000u) {
        volatile float half = 0.5f; /* keep the add at run time, in round-to-nearest-even */
        return (uint16_t)(sign | (f2u(u2f(x) + half) - 0x3f000000u));
    }
    uint32_t odd = (x >> 13) & 1u;
    x += 0xc8000fffu;
    x += odd;
    return (uint16_t)(sign | (x >> 13));
}

/* ------------------------------------------------------------------------------------------ */
/* min/max operand-order semantics                                                             */

/* std::min(in, inout) / std::max(in, inout) as CCL_REDUCE uses them (comp.cpp:46-55) and the scalar
 * bf16 path (bf16.cpp:42-48): ties and unordered operands give `in`. */
#define STD_MIN(in, io) (((io) < (in)) ? (io) : (in))
#define STD_MAX(in, io) (((in) < (io)) ? (io) : (in))
/* _mm512_min_ps(in, inout) / _mm512_max_ps(in, inout) (bf16_intrisics.cpp:28-34,
 * fp16_intrisics.hpp:70-75): ties and unordered operands give the second source, `inout`. */
#define VEC_MIN(in, io) (((in) < (io)) ? (in) : (io))
#define VEC_MAX(in, io) (((in) > (io)) ? (in) : (io))

static inline float f32_step(float in, float io, int op, int vec_sem) {
    switch (op) {
        case ORC_SUM: return io + in;
        case ORC_PROD: return io * in;
        case ORC_MIN: return vec_sem ? VEC_MIN(in, io) : STD_MIN(in, io);
        default: return vec_sem ? VEC_MAX(in, io) : STD_MAX(in, io);
    }
}

/* ------------------------------------------------------------------------------------------ */
/* pairwise in-place primitives                                                                */

/* CCL_REDUCE(type), comp.cpp:31-58.  Sum and product of integers are done on the unsigned type of
 * the same width: the reference's signed `+=`/`*=` wraps in practice and that is the defined result
 * here.  ORC_UWIDE lifts an 8- or 16-bit operand to `unsigned` first (C would promote it to a signed
 * int, and 65535 * 65535 overflows one); wider types stay as they are. */
#define ORC_UWIDE(x) ((x) + 0u)
#define DEFINE_REDUCE_INT(name, T, U)                                                \
    static void name(const void* in_, size_t n, void* io_, int op) {                 \
        const T* in = (const T*)in_;                                                 \
        T* io = (T*)io_;                                                             \
        size_t i;                                                                    \
        switch (op) {                                                                \
            case ORC_SUM:                                                            \
                for (i = 0; i < n; i++) io[i] = (T)(U)(ORC_UWIDE((U)io[i]) + ORC_UWIDE((U)in[i])); \
                break;                                                               \
            case ORC_PROD:                                                           \
                for (i = 0; i < n; i++) io[i] = (T)(U)(ORC_UWIDE((U)io[i]) * ORC_UWIDE((U)in[i])); \
                break;                                                               \
            case ORC_MIN:                                                            \
                for (i = 0; i < n; i++) io[i] = STD_MIN(in[i], io[i]);               \
                break;                                                               \
            default:                                                                 \
                for (i = 0; i < n; i++) io[i] = STD_MAX(in[i], io[i]);               \
                break;                                                               \
        }                                                                            \
    }

#define DEFINE_REDUCE_FP(name, T)                                                    \
    static void name(const void* in_, size_t n, void* io_, int op) {                 \
        const T* in = (const T*)in_;                                                 \
        T* io = (T*)io_;                                                             \
        size_t i;                                                                    \
        switch (op) {                                                                \
            case ORC_SUM:                                                            \
                for (i = 0; i < n; i++) io[i] += in[i];                              \
                break;                                                               \
            case ORC_PROD:                                                           \
                for (i = 0; i < n; i++) io[i] *= in[i];                              \
                break;                                                               \
            case ORC_MIN:                                                            \
                for (i = 0; i < n; i++) io[i] = STD_MIN(in[i], io[i]);               \
                break;                                                               \
            default:                                                                 \
                for (i = 0; i < n; i++) io[i] = STD_MAX(in[i], io[i]);               \
                break;                                                               \
        }                                                                            \
    }

DEFINE_REDUCE_INT(reduce_i8, int8_t, uint8_t)
DEFINE_REDUCE_INT(reduce_u8, uint8_t, uint8_t)
DEFINE_REDUCE_INT(reduce_i16, int16_t, uint16_t)
DEFINE_REDUCE_INT(reduce_u16, uint16_t, uint16_t)
DEFINE_REDUCE_INT(reduce_i32, int32_t, uint32_t)
DEFINE_REDUCE_INT(reduce_u32, uint32_t, uint32_t)
DEFINE_REDUCE_INT(reduce_i64, int64_t, uint64_t)
DEFINE_REDUCE_INT(reduce_u64, uint64_t, uint64_t)
DEFINE_REDUCE_FP(reduce_f32, float)
DEFINE_REDUCE_FP(reduce_f64, double)

/* ccl_bf16_reduce, bf16.cpp:87-110: scalar impl (bf16.cpp:63-85) widens both, applies the fp32 op with
 * std:: semantics and truncates; the vector impls (bf16_intrisics.hpp:80-114) apply _mm512_*_ps(in, inout)
 * and narrow by truncation (avx512f) or VCVTNEPS2BF16 (avx512bf).  The masked tail uses the same
 * converter as the body (bf16_intrisics.hpp:94-104).  Rounds after every pair. */
void orc_bf16_reduce(const void* in_, size_t count, void* io_, int op, int bf16_impl) {
    const uint16_t* in = (const uint16_t*)in_;
    uint16_t* io = (uint16_t*)io_;
    int vec_sem = (bf16_impl != ORC_BF16_SCALAR);
    for (size_t i = 0; i < count; i++) {
        float r = f32_step(u2f(orc_bf16_widen(in[i])), u2f(orc_bf16_widen(io[i])), op, vec_sem);
        io[i] = (bf16_impl == ORC_BF16_AVX512BF) ? orc_bf16_narrow_rne(f2u(r)) : orc_bf16_narrow_trunc(f2u(r));
    }
}

/* ccl_fp16_reduce, fp16.cpp:41-53 -> ccl_fp16_reduce_impl, fp16_intrisics.hpp:204-248.  f16c and avx512f
 * widen, apply _mm*_ps(in, inout), narrow with imm 0; avx512fp16 computes natively in fp16
 * (fp16_intrisics.cpp:24-35), which gives the same bits for + and * and, for min/max, returns the second
 * source unchanged (no NaN quieting).  Any other impl value leaves inout untouched: the dispatch has no
 * else branch (fp16_intrisics.hpp:216-247). */
void orc_fp16_reduce(const void* in_, size_t count, void* io_, int op, int fp16_impl) {
    const uint16_t* in = (const uint16_t*)in_;
    uint16_t* io = (uint16_t*)io_;
    if (fp16_impl != ORC_FP16_F16C && fp16_impl != ORC_FP16_AVX512F && fp16_impl != ORC_FP16_AVX512FP16)
        return;
    for (size_t i = 0; i < count; i++) {
        float a = u2f(orc_fp16_widen(in[i])), b = u2f(orc_fp16_widen(io[i]));
        if (fp16_impl == ORC_FP16_AVX512FP16 && (op == ORC_MIN || op == ORC_MAX)) {
            int take_in = (op == ORC_MIN) ? (a < b) : (a > b);
            io[i] = take_in ? in[i] : io[i];
            continue;
        }
        io[i] = orc_fp16_narrow(f2u(f32_step(a, b, op, 1)));
    }
}

/* ccl_comp_reduce -> ccl_comp_reduce_regular, comp.cpp:76-200 (count == 0 is a successful no-op,
 * comp.cpp:132-134; unknown dtype/op is fatal there and an error code here). */
int orc_comp_reduce(const void* in, size_t count, void* inout, int dtype, int op, int bf16_impl,
                    int fp16_impl) {
    if (count == 0)
        return ORC_OK;
    if (op < ORC_SUM || op > ORC_MAX)
        return ORC_INVALID_ARGUMENTS;
    switch (dtype) {
        case ORC_INT8: reduce_i8(in, count, inout, op); break;
        case ORC_UINT8: reduce_u8(in, count, inout, op); break;
        case ORC_INT16: reduce_i16(in, count, inout, op); break;
        case ORC_UINT16: reduce_u16(in, count, inout, op); break;
        case ORC_INT32: reduce_i32(in, count, inout, op); break;
        case ORC_UINT32: reduce_u32(in, count, inout, op); break;
        case ORC_INT64: reduce_i64(in, count, inout, op); break;
        case ORC_UINT64: reduce_u64(in, count, inout, op); break;
        case ORC_FLOAT16: orc_fp16_reduce(in, count, inout, op, fp16_impl); break;
        case ORC_FLOAT32: reduce_f32(in, count, inout, op); break;
        case ORC_FLOAT64: reduce_f64(in, count, inout, op); break;
        case ORC_BFLOAT16: orc_bf16_reduce(in, count, inout, op, bf16_impl); break;
        default: return ORC_INVALID_ARGUMENTS;
    }
    return ORC_OK;
}

/* ------------------------------------------------------------------------------------------ */
/* array converters                                                                            */

/* ccl_convert_fp32_to_bf16_arrays, bf16.cpp:130-149: the vector impls convert 16*floor(count/16)
 * elements with their own converter; the remaining count % 16 elements always go through the scalar
 * truncating converter (bf16.cpp:144-148). */
void orc_convert_fp32_to_bf16_arrays(const void* fp32_buf, void* bf16_buf, size_t count, int bf16_impl) {
    const uint32_t* src = (const uint32_t*)fp32_buf;
    uint16_t* dst = (uint16_t*)bf16_buf;
    size_t limit = (bf16_impl != ORC_BF16_SCALAR) ? (count / 16) * 16 : 0;
    size_t i;
    if (bf16_impl == ORC_BF16_AVX512BF)
        for (i = 0; i < limit; i++) dst[i] = orc_bf16_narrow_rne(src[i]);
    else
        for (i = 0; i < limit; i++) dst[i] = orc_bf16_narrow_trunc(src[i]);
    for (i = limit; i < count; i++) dst[i] = orc_bf16_narrow_trunc(src[i]);
}

/* ccl_convert_bf16_to_fp32_arrays, bf16.cpp:151-169: exact in body and tail alike. */
void orc_convert_bf16_to_fp32_arrays(const void* bf16_buf, void* fp32_buf, size_t count, int bf16_impl) {
    const uint16_t* src = (const uint16_t*)bf16_buf;
    uint32_t* dst = (uint32_t*)fp32_buf;
    (void)bf16_impl;
    for (size_t i = 0; i < count; i++) dst[i] = orc_bf16_widen(src[i]);
}

/* ccl_convert_fp32_to_fp16 / ccl_convert_fp16_to_fp32, fp16.cpp:55-61: the reference converts one vector of eight
 * values with VCVTPS2PH (imm 0: round to nearest even) / VCVTPH2PS; here for count values. */
void orc_convert_fp32_to_fp16_arrays(const void* fp32_buf, void* fp16_buf, size_t count) {
    const uint32_t* src = (const uint32_t*)fp32_buf;
    uint16_t* dst = (uint16_t*)fp16_buf;
    for (size_t i = 0; i < count; i++) dst[i] = orc_fp16_narrow(src[i]);
}
void orc_convert_fp16_to_fp32_arrays(const void* fp16_buf, void* fp32_buf, size_t count) {
    const uint16_t* src = (const uint16_t*)fp16_buf;
    uint32_t* dst = (uint32_t*)fp32_buf;
    for (size_t i = 0; i < count; i++) dst[i] = orc_fp16_widen(src[i]);
}

/* ------------------------------------------------------------------------------------------ */
/* N-input reduce                                                                              */

/* ccl_comp_batch_reduce, comp.cpp:202-249.  keep-precision: acc = widen(inout); for every further slice
 * tmp = widen(slice), acc = acc OP tmp through the fp32 CCL_REDUCE (std:: min/max); inout = narrow(acc)
 * with the array converter above.  Otherwise a chain of pairwise calls in the buffer's own dtype. */
int orc_comp_batch_reduce(const void* in_buf, const size_t* offsets, size_t n_offsets, size_t count,
                          void* inout, int dtype, int op, int bf16_keep_precision_mode, float* tmp,
                          float* acc, int bf16_impl, int fp16_impl) {
    size_t esz = orc_datatype_size(dtype);
    if (esz == 0 || op < ORC_SUM || op > ORC_MAX)
        return ORC_INVALID_ARGUMENTS;
    if (bf16_keep_precision_mode) {
        orc_convert_bf16_to_fp32_arrays(inout, acc, count, bf16_impl);
        for (size_t i = 1; i < n_offsets; i++) {
            orc_convert_bf16_to_fp32_arrays((const char*)in_buf + esz * offsets[i], tmp, count, bf16_impl);
            reduce_f32(tmp, count, acc, op);
        }
        orc_convert_fp32_to_bf16_arrays(acc, inout, count, bf16_impl);
    }
    else {
        for (size_t i = 1; i < n_offsets; i++) {
            int rc = orc_comp_reduce((const char*)in_buf + esz * offsets[i], count, inout, dtype, op,
                                     bf16_impl, fp16_impl);
            if (rc != ORC_OK)
                return rc;
        }
    }
    return ORC_OK;
}

/* N separate buffers: out = src0, then step(in = src_j, inout = out) for j = 1..n-1 -- the order of the
 * device kernels (own buffer first, peers in argument order, kernels.cl:279-282) driven through the CPU
 * pairwise step (reduce_scatter.cpp:111-136 does exactly this chain on the host).  One fused pass per
 * element; bit-identical to running the multi-pass forms above because every step is elementwise. */
static void reduce_n_range(const void* const* srcs, int n, void* dst, size_t lo, size_t hi, size_t count,
                           int dtype, int op, int keep, int quirk_tail, int bf16_impl, int fp16_impl) {
    size_t esz = orc_datatype_size(dtype);
    if (dtype == ORC_BFLOAT16 && keep) {
        uint16_t* out = (uint16_t*)dst;
        size_t limit = (bf16_impl != ORC_BF16_SCALAR) ? (quirk_tail ? (count / 16) * 16 : count) : 0;
        for (size_t i = lo; i < hi; i++) {
            float a = u2f(orc_bf16_widen(((const uint16_t*)srcs[0])[i]));
            for (int j = 1; j < n; j++)
                a = f32_step(u2f(orc_bf16_widen(((const uint16_t*)srcs[j])[i])), a, op, 0);
            out[i] = (bf16_impl == ORC_BF16_AVX512BF && i < limit) ? orc_bf16_narrow_rne(f2u(a))
                                                                  : orc_bf16_narrow_trunc(f2u(a));
        }
        return;
    }
    /* chain in the buffer's dtype: copy src0 then fold the others in, in chunks that stay in cache */
    const size_t chunk = 4096;
    for (size_t i = lo; i < hi; i += chunk) {
        size_t c = (hi - i < chunk) ? hi - i : chunk;
        char* o = (char*)dst + i * esz;
        if (o != (const char*)srcs[0] + i * esz)
            memmove(o, (const char*)srcs[0] + i * esz, c * esz);
        for (int j = 1; j < n; j++)
            orc_comp_reduce((const char*)srcs[j] + i * esz, c, o, dtype, op, bf16_impl, fp16_impl);
    }
}

int orc_reduce_n(const void* const* srcs, int n, void* dst, size_t count, int dtype, int op,
                 int lp_keep_precision, int quirk_tail, int bf16_impl, int fp16_impl) {
    if (orc_datatype_size(dtype) == 0 || op < ORC_SUM || op > ORC_MAX || n < 1)
        return ORC_INVALID_ARGUMENTS;
    reduce_n_range(srcs, n, dst, 0, count, count, dtype, op, lp_keep_precision, quirk_tail, bf16_impl,
                   fp16_impl);
    return ORC_OK;
}

/* kernels.cl:190-217 and :423-560: every element is read from all inputs before it is stored anywhere, so the
 * result is formed apart and copied out; that also covers a destination that is one of the sources. */
int orc_reduce_write_n(const void* const* srcs, int n, void* const* dsts, int m, size_t count, int dtype, int op,
                       int lp_keep_precision, int quirk_tail, int bf16_impl, int fp16_impl) {
    size_t esz = orc_datatype_size(dtype);
    if (esz == 0 || m < 1)
        return ORC_INVALID_ARGUMENTS;
    if (count == 0)
        return ORC_OK;
    void* res = malloc(count * esz);
    if (!res)
        return ORC_INVALID_ARGUMENTS;
    int rc = orc_reduce_n(srcs, n, res, count, dtype, op, lp_keep_precision, quirk_tail, bf16_impl, fp16_impl);
    if (rc == ORC_OK)
        for (int k = 0; k < m; k++) memcpy(dsts[k], res, count * esz);
    free(res);
    return rc;
}

struct mt_job {
    const void* const* srcs;
    int n;
    void* dst;
    size_t lo, hi, count;
    int dtype, op, keep, quirk, bf16_impl, fp16_impl;
};

static void* mt_worker(void* p) {
    struct mt_job* j = (struct mt_job*)p;
    reduce_n_range(j->srcs, j->n, j->dst, j->lo, j->hi, j->count, j->dtype, j->op, j->keep, j->quirk,
                   j->bf16_impl, j->fp16_impl);
    return NULL;
}

/* Contiguous count/threads partitions, the last one takes the remainder (parallelizer.cpp:230-241). */
int orc_reduce_n_mt(const void* const* srcs, int n, void* dst, size_t count, int dtype, int op,
                    int lp_keep_precision, int quirk_tail, int bf16_impl, int fp16_impl, int threads) {
    if (orc_datatype_size(dtype) == 0 || op < ORC_SUM || op > ORC_MAX || n < 1)
        return ORC_INVALID_ARGUMENTS;
    if (threads < 1)
        threads = 1;
    if (threads > 256)
        threads = 256;
    pthread_t tid[256];
    struct mt_job job[256];
    size_t part = count / (size_t)threads;
    for (int t = 0; t < threads; t++) {
        struct mt_job jb = { srcs, n, dst, part * (size_t)t, (t == threads - 1) ? count : part * (size_t)(t + 1),
                             count, dtype, op, lp_keep_precision, quirk_tail, bf16_impl, fp16_impl };
        job[t] = jb;
        pthread_create(&tid[t], NULL, mt_worker, &job[t]);
    }
    for (int t = 0; t < threads; t++) pthread_join(tid[t], NULL);
    return ORC_OK;
}

/* ------------------------------------------------------------------------------------------ */
/* copy and fusion layout                                                                      */

int orc_comp_copy(const void* in, void* out, size_t bytes) { /* comp.cpp:60-74 */
    if (bytes == 0)
        return ORC_OK;
    memcpy(out, in, bytes);
    return ORC_OK;
}

/* fusion.cpp:283-316: tensor k goes to fusion_buf + offset, offset += count_k * dtype_size.  align > 1
 * is this build's padded layout (start of every tensor rounded up); align == 1 is the reference's. */
size_t orc_fusion_offsets(const size_t* counts, size_t k, size_t dtype_size, size_t align,
                          size_t* byte_offsets) {
    size_t off = 0, end = 0;
    if (align == 0)
        align = 1;
    for (size_t i = 0; i < k; i++) {
        off = (end + align - 1) / align * align;
        byte_offsets[i] = off;
        end = off + counts[i] * dtype_size;
    }
    return end;
}

void orc_fusion_pack(const void* const* tensors, const size_t* counts, const size_t* byte_offsets,
                     size_t k, size_t dtype_size, void* fusion_buf) {
    for (size_t i = 0; i < k; i++)
        orc_comp_copy(tensors[i], (char*)fusion_buf + byte_offsets[i], counts[i] * dtype_size);
}

void orc_fusion_unpack(const void* fusion_buf, const size_t* counts, const size_t* byte_offsets,
                       size_t k, size_t dtype_size, void* const* tensors) { /* fusion.cpp:323-362 */
    for (size_t i = 0; i < k; i++)
        orc_comp_copy((const char*)fusion_buf + byte_offsets[i], tensors[i], counts[i] * dtype_size);
}
