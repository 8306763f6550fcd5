// N-input elementwise reduce kernels for gfx950 (MI355X), templated on an element-traits class.
//
// Every kernel is a pure HBM stream: each lane issues one 128-bit load per input per step (a wave reads 1 KiB
// contiguous per input per instruction), folds the inputs in argument order in registers and writes one 128-bit
// nontemporal store per output.  There is no cross-lane traffic and no MFMA.  Two forms exist: a streaming form
// (reduce_vec_kernel, reduce_multi_kernel), and for large buffers a phased form (reduce_multi_phased_kernel)
// that parks results in LDS and registers so that the whole chip reads for a while and
// then writes for a while -- HBM loses about a quarter of its bandwidth when reads and writes are interleaved.
//
// Arithmetic follows the oneCCL CPU reduction: acc = src0; acc = step(in = src_j, inout = acc), j = 1..N-1
// (src/comp/comp.cpp:31-58 for the step, src/kernels/kernels.cl:279-282 for the order).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "launch_geometry.hpp"

// The inline assembly below (sub-dword byte lanes, MODE-register writes, "sc1 nt" stores with hand-placed wait states)
// is written against the gfx950 instruction set and its hazard rules; no other target is built or tested.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "these kernels are written for gfx950 (MI355X) only"
#endif

namespace mi {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kBlock = 256;     // 4 wavefronts of 64 lanes
constexpr int kMaxFixedN = 8;   // inputs unrolled at compile time
constexpr int kMaxSrcs = 64;    // inputs of the run-time-N kernels
constexpr int kMaxDsts = 16;    // outputs of the multi-destination kernels

enum { OP_SUM = 0, OP_PROD = 1, OP_MIN = 2, OP_MAX = 3 };

struct SrcTable {               // by-value kernel argument
    const void* p[kMaxSrcs];
};
template <int N>
struct SrcFixed {
    const void* p[N];
};
struct DstTable {               // by-value kernel argument
    void* p[kMaxDsts];
};

struct Tuning {
    int waves_per_cu;   // 256-thread blocks per CU the grid is capped at (a block loops over tiles beyond that)
    int max_blocks;     // 0 = no cap
    int xcd_chunked;    // 1: each XCD streams one contiguous eighth of the buffer
    int variant;        // 0 = automatic; 1, 2, 4 = streaming kernel (with that unroll depth where compiled); 8 = phased kernel
    int num_cus;
    long phased_min_bytes;   // automatic choice: no phased kernel below this much traffic per launch
    struct PhaseSync* sync;  // the set of device-resident barrier words this call uses (may be null)
    int early_loads;         // phased kernels: loads per lane still to issue when a block reports the end of its reads (< 0: phase_early_loads chooses)
    int early_stores;        // ... and stores per lane still to issue when it reports the end of its writes (< 0: per type)
    long spin_ticks;         // phased kernels: longest wait at one barrier, in 100 MHz ticks, before a block goes on alone
    int fp16_impl;           // which CPU implementation's float16 results to reproduce: 2, 3 (through fp32) or 4 (native)
    int realign;             // 1: inputs off a 4-byte boundary are read on that boundary and realigned in registers
    int line_start;          // 1: large calls start their vectors on a 128-byte line of the buffers that matter most
    int wave_runs;           // phased kernels: a wave's vectors of a group lie next to each other; 0 never, 1 when a buffer is off the lines, 2 always
    int write_pace;          // phased kernels: the rate, in GB/s, at which the clock lets the write phase's stores out (0: unpaced)
    int wall_khz;            // what wall_clock64() counts, in kHz
};

// Name of the kernel template the calling thread's most recent entry-point call launched (diagnostics and
// measurement: lets a benchmark say which kernel its figures belong to).
extern thread_local const char* g_last_kernel;
// Launches by the calling thread whose inputs off a 4-byte boundary were realigned in registers (tests ask for it).
extern thread_local unsigned long g_realigned_launches;
extern thread_local unsigned long g_wide_phase_launches;    // launches of the phased reduce with one more register group (phase_reg_groups)

struct LaunchArgs {
    const void* const* srcs;    // host array of n device pointers
    int n;
    void* dst;
    size_t count;               // elements
    int op;
    hipStream_t stream;
    Tuning tune;
    void* const* dsts = nullptr;    // m > 1: host array of m device pointers, the result goes to each (dst is unused)
    int m = 1;
};

// How the elements of a call are divided: `head` elements, `nvec` vectors, `tail` elements; beyond = 1: vector nvec
// lies inside every buffer and may be read (see vector_split and load_vectors).
struct VecSplit {
    uint32_t head, tail, beyond;
    uint64_t nvec;
};

// ---------------------------------------------------------------------------------------------------
// bit helpers

__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

// fp32 -> bf16 exactly as VCVTNEPS2BF16 (src/comp/bf16/bf16_intrisics.hpp:73-75): round to nearest even,
// fp32 denormals read as zero, NaN quieted keeping its top payload bits, overflow rounds to Inf.
__device__ __forceinline__ uint32_t bf16_narrow_rne(uint32_t u) {
    uint32_t e = u & 0x7f800000u;
    uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    uint32_t nan = (u >> 16) | 0x40u;
    r = (e == 0x7f800000u && (u & 0x007fffffu) != 0) ? nan : r;
    r = (e == 0) ? ((u >> 16) & 0x8000u) : r;
    return r & 0xffffu;
}
// fp32 -> bf16 by dropping the low half (src/comp/bf16/bf16.cpp:50-54, bf16_intrisics.hpp:67-70)
__device__ __forceinline__ uint32_t bf16_narrow_trunc(uint32_t u) { return u >> 16; }

// Two fp32 values -> two bf16 values packed in one dword (lo in the low half), same results as bf16_narrow_rne.
// gfx950's v_cvt_pk_bf16_f32 rounds to nearest even, quiets NaNs and overflows to Inf exactly like VCVTNEPS2BF16
// (all 2^32 inputs compared on the GPU); the one difference is that it keeps fp32 denormals, which the x86
// instruction reads as zero, so those are replaced by a signed zero first (one v_cmp_class per value).
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t bf16_narrow_rne_pack2(uint32_t lo, uint32_t hi) {
    constexpr int kDenormal = 0x10 | 0x80;      // class mask: negative denormal, positive denormal
    float a = as_f32(lo), b = as_f32(hi);
    a = __builtin_amdgcn_classf(a, kDenormal) ? as_f32(lo & 0x80000000u) : a;
    b = __builtin_amdgcn_classf(b, kDenormal) ? as_f32(hi & 0x80000000u) : b;
    const f32x2 f = { a, b };
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

// compare on the float value, select on the bits: the returned operand's bits are never touched
template <int OP, bool VEC_SEM>
__device__ __forceinline__ uint32_t f32_minmax_bits(uint32_t in, uint32_t io) {
    float a = as_f32(in), b = as_f32(io);
    if (VEC_SEM)   // _mm512_min_ps(in, inout): second source on ties/NaN (bf16_intrisics.cpp:28-34)
        return (OP == OP_MIN) ? ((a < b) ? in : io) : ((a > b) ? in : io);
    // std::min(in, inout) / std::max(in, inout): first argument on ties/NaN (comp.cpp:46-55)
    return (OP == OP_MIN) ? ((b < a) ? io : in) : ((a < b) ? io : in);
}

// Sum and prod are the hardware's own add and multiply, NaN results included: gfx950 returns a single NaN operand with
// its quiet bit set (sign and payload kept) and makes the negative default NaN (0xffc00000, 0xfff8000000000000) from an
// invalid operation (Inf - Inf, 0 x Inf) -- the same bits as the ADDPS / MULPS family of the reference's CPU path.
// Only with two NaN operands does the result depend on the operand order, which the reference leaves to its compiler.
template <int OP, bool VEC_SEM>
__device__ __forceinline__ uint32_t f32_step_bits(uint32_t in, uint32_t io) {
    if (OP == OP_SUM) return as_u32(as_f32(io) + as_f32(in));
    if (OP == OP_PROD) return as_u32(as_f32(io) * as_f32(in));
    return f32_minmax_bits<OP, VEC_SEM>(in, io);
}

// ---------------------------------------------------------------------------------------------------
// element traits: elem_t (storage), acc_t (what is carried between steps), init / step / finish

// Integers and fp32/fp64 (CCL_REDUCE, comp.cpp:31-58).  Integer sum/prod are done on the unsigned type of
// the same width (two's-complement wrap); 8- and 16-bit operands are lifted to `unsigned` first, because the
// language would promote them to a signed int, which 65535 * 65535 overflows.  min/max: ties and unordered
// operands return `in`.
template <class T, class U>
struct PlainTraits {
    typedef T elem_t;
    typedef T acc_t;
    typedef decltype(U() + 0u) W;       // unsigned for the narrow types, U itself from 32 bits up
    static constexpr int VEC = 16 / sizeof(T);
    static __device__ __forceinline__ acc_t init(elem_t x) { return x; }
    template <int OP>
    static __device__ __forceinline__ acc_t step(elem_t in, acc_t io) {
        if (OP == OP_SUM) return (T)(U)((W)(U)io + (W)(U)in);
        if (OP == OP_PROD) return (T)(U)((W)(U)io * (W)(U)in);
        if (OP == OP_MIN) return (io < in) ? io : in;
        return (in < io) ? io : in;
    }
    static __device__ __forceinline__ elem_t finish(acc_t a) { return a; }
};

// float and double go through their bit patterns for min/max so that no floating-point instruction can
// canonicalise the operand that is returned.
struct F32Traits {
    typedef uint32_t elem_t;
    typedef uint32_t acc_t;
    static constexpr int VEC = 4;
    static __device__ __forceinline__ acc_t init(elem_t x) { return x; }
    template <int OP>
    static __device__ __forceinline__ acc_t step(elem_t in, acc_t io) { return f32_step_bits<OP, false>(in, io); }
    static __device__ __forceinline__ elem_t finish(acc_t a) { return a; }
};

struct F64Traits {
    typedef uint64_t elem_t;
    typedef uint64_t acc_t;
    static constexpr int VEC = 2;
    static __device__ __forceinline__ acc_t init(elem_t x) { return x; }
    template <int OP>
    static __device__ __forceinline__ acc_t step(elem_t in, acc_t io) {
        double a = __builtin_bit_cast(double, in), b = __builtin_bit_cast(double, io);
        if (OP == OP_SUM) return __builtin_bit_cast(uint64_t, b + a);
        if (OP == OP_PROD) return __builtin_bit_cast(uint64_t, b * a);
        if (OP == OP_MIN) return (b < a) ? io : in;
        return (a < b) ? io : in;
    }
    static __device__ __forceinline__ elem_t finish(acc_t a) { return a; }
};

// bfloat16, rounded to bf16 after every pair (ccl_bf16_reduce, src/comp/bf16/bf16.cpp:63-110,
// bf16_intrisics.hpp:80-114).  RNE: avx512bf narrowing, else truncation.  VEC_SEM: vector min/max operand
// order (avx512f / avx512bf) instead of std:: (scalar).  The carried value is the raw bf16 pattern, so a
// single input passes through unchanged, as a chain of zero pairwise calls does.
template <bool RNE, bool VEC_SEM>
struct Bf16PairwiseTraits {
    typedef uint16_t elem_t;
    typedef uint32_t acc_t;     // bf16 bits in the low half
    static constexpr int VEC = 8;
    static __device__ __forceinline__ acc_t init(elem_t x) { return x; }
    template <int OP>
    static __device__ __forceinline__ acc_t step(elem_t in, acc_t io) {
        uint32_t r = f32_step_bits<OP, VEC_SEM>((uint32_t)in << 16, io << 16);
        return RNE ? bf16_narrow_rne(r) : bf16_narrow_trunc(r);
    }
    static __device__ __forceinline__ elem_t finish(acc_t a) { return (elem_t)a; }
};

// bfloat16, widened once, accumulated in fp32 with the plain fp32 step (std:: min/max), narrowed once
// (ccl_comp_batch_reduce with bf16_keep_precision_mode, src/comp/comp.cpp:214-234).
template <bool RNE>
struct Bf16KeepTraits {
    typedef uint16_t elem_t;
    typedef uint32_t acc_t;     // fp32 bits
    static constexpr int VEC = 8;
    static __device__ __forceinline__ acc_t init(elem_t x) { return (uint32_t)x << 16; }
    template <int OP>
    static __device__ __forceinline__ acc_t step(elem_t in, acc_t io) {
        return f32_step_bits<OP, false>((uint32_t)in << 16, io);
    }
    static __device__ __forceinline__ elem_t finish(acc_t a) {
        return (elem_t)(RNE ? bf16_narrow_rne(a) : bf16_narrow_trunc(a));
    }
};

// float16, rounded after every pair through fp32 (ccl_fp16_reduce f16c / avx512f implementations,
// src/comp/fp16/fp16_intrisics.hpp:95-148): VCVTPH2PS both, one fp32 op, VCVTPS2PH round-to-nearest-even,
// fp16 subnormals kept.  min/max return `inout` on ties/NaN and quiet a NaN they return (the x86 widening
// conversion quiets it).  NATIVE: the avx512fp16 implementation (fp16_intrisics.cpp:24-35), which works on the
// fp16 values themselves: the same bits for sum and prod (fp32 holds the exact sum or product of two fp16 values
// closely enough that rounding twice equals rounding once), and min/max hand back the chosen operand untouched, a
// signalling NaN included.
template <bool NATIVE>
struct Fp16Traits {
    typedef uint16_t elem_t;
    typedef uint32_t acc_t;     // fp16 bits in the low half
    static constexpr int VEC = 8;
    static __device__ __forceinline__ acc_t init(elem_t x) { return x; }
    static __device__ __forceinline__ float widen(uint32_t h) {
        return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
    }
    template <int OP>
    static __device__ __forceinline__ acc_t step(elem_t in, acc_t io) {
        if (OP == OP_SUM || OP == OP_PROD) {
            float a = widen(in), b = widen(io);
            float r = (OP == OP_SUM) ? (b + a) : (b * a);
            return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)r);
        }
        // ordering and NaN-ness of two fp16 values are the same before and after widening: compare them as they are
        const _Float16 a = __builtin_bit_cast(_Float16, in), b = __builtin_bit_cast(_Float16, (uint16_t)io);
        const bool take_in = (OP == OP_MIN) ? (a < b) : (a > b);
        const uint32_t r = take_in ? (uint32_t)in : io;
        if (NATIVE) return r;
        const _Float16 rf = take_in ? a : b;
        return (rf != rf) ? (r | 0x0200u) : r;
    }
    static __device__ __forceinline__ elem_t finish(acc_t a) { return (elem_t)a; }
};
typedef Fp16Traits<false> Fp16PairwiseTraits;
typedef Fp16Traits<true> Fp16NativeTraits;

typedef PlainTraits<int8_t, uint8_t> I8Traits;
typedef PlainTraits<uint8_t, uint8_t> U8Traits;
typedef PlainTraits<int16_t, uint16_t> I16Traits;
typedef PlainTraits<uint16_t, uint16_t> U16Traits;
typedef PlainTraits<int32_t, uint32_t> I32Traits;
typedef PlainTraits<uint32_t, uint32_t> U32Traits;
typedef PlainTraits<int64_t, uint64_t> I64Traits;
typedef PlainTraits<uint64_t, uint64_t> U64Traits;

// ---------------------------------------------------------------------------------------------------
// 128-bit vector <-> VEC elements

template <class TR>
struct Lanes {
    typename TR::elem_t v[TR::VEC];
};
template <class TR>
struct Accs {
    typename TR::acc_t v[TR::VEC];
};

// Traits/operation pairs whose kernels run with the wave's fp32 denormal mode set to "inputs kept, results flushed
// to a signed zero" (MODE.FP_DENORM[1:0] = 1).  That is what the x86 sequence "fp32 add or multiply, then
// VCVTNEPS2BF16" amounts to: the conversion reads a denormal sum as zero.  With the mode set, the packed conversion
// needs no per-value denormal test.  Every kernel that uses VecOps<TR>::step<OP> calls kernel_prologue<TR, OP>() first.
template <class TR, int OP>
struct FlushF32Results {
    static constexpr bool value = false;
};
template <class TR, int OP>
__device__ __forceinline__ void kernel_prologue() {
    if constexpr (FlushF32Results<TR, OP>::value) {
        // s_setreg hwreg(HW_REG_MODE = 1, offset 4, size 2) <- 1
        __builtin_amdgcn_s_setreg(1 | (4 << 6) | ((2 - 1) << 11), 1);
    }
}

// Vector-level operations on the 128-bit unit a lane moves.  The default walks the VEC elements one by one with
// the traits' init / step / finish; traits with a cheaper packed form specialise VecOps.
template <class TR>
struct VecOps {
    static __device__ __forceinline__ Accs<TR> init(u32x4 x) {
        Lanes<TR> l = __builtin_bit_cast(Lanes<TR>, x);
        Accs<TR> a;
#pragma unroll
        for (int k = 0; k < TR::VEC; k++) a.v[k] = TR::init(l.v[k]);
        return a;
    }
    template <int OP>
    static __device__ __forceinline__ void step(u32x4 x, Accs<TR>& a) {
        Lanes<TR> l = __builtin_bit_cast(Lanes<TR>, x);
#pragma unroll
        for (int k = 0; k < TR::VEC; k++) a.v[k] = TR::template step<OP>(l.v[k], a.v[k]);
    }
    static __device__ __forceinline__ u32x4 finish(const Accs<TR>& a) {
        Lanes<TR> l;
#pragma unroll
        for (int k = 0; k < TR::VEC; k++) l.v[k] = TR::finish(a.v[k]);
        return __builtin_bit_cast(u32x4, l);
    }
};

// every operation of the avx512bf pairwise reduce ends in VCVTNEPS2BF16, which reads a denormal as zero
template <bool VEC_SEM, int OP>
struct FlushF32Results<Bf16PairwiseTraits<true, VEC_SEM>, OP> {
    static constexpr bool value = true;
};

// x as the hardware hands it back from an fp32 operation: with the wave in the mode above a denormal becomes a
// signed zero and a signalling NaN its quiet form, every other value is unchanged -- for a value that is a widened
// bf16, exactly what VCVTNEPS2BF16 followed by widening gives.  (An instruction the compiler cannot fold away: it
// knows nothing of the mode.)
__device__ __forceinline__ uint32_t f32_through_alu(uint32_t x) {
    uint32_t r;
    asm("v_mul_f32 %0, 1.0, %1" : "=v"(r) : "v"(x));
    return r;
}

// bf16 rounded to nearest even after every pair.  The accumulator is carried widened (eight fp32 values whose low
// halves are zero), so a step widens only the new input: sum and prod round the pair of results with the packed
// conversion and widen it again; min and max select on the widened values and pass the selected one through the
// ALU, which is all the rounding step does to a value that already is a bf16.  With one input nothing is touched.
template <bool VEC_SEM>
struct VecOps<Bf16PairwiseTraits<true, VEC_SEM>> {
    typedef Bf16PairwiseTraits<true, VEC_SEM> TR;
    static __device__ __forceinline__ Accs<TR> init(u32x4 x) {
        Accs<TR> a;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            a.v[2 * k] = x[k] << 16;
            a.v[2 * k + 1] = x[k] & 0xffff0000u;
        }
        return a;
    }
    template <int OP>
    static __device__ __forceinline__ void step(u32x4 x, Accs<TR>& a) {
        static_assert(FlushF32Results<TR, OP>::value, "the kernels of this traits class set the wave's denormal mode");
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t lo = f32_step_bits<OP, VEC_SEM>(x[k] << 16, a.v[2 * k]);
            const uint32_t hi = f32_step_bits<OP, VEC_SEM>(x[k] & 0xffff0000u, a.v[2 * k + 1]);
            if (OP == OP_SUM || OP == OP_PROD) {    // a denormal sum or product is already a signed zero
                const f32x2 f = { as_f32(lo), as_f32(hi) };
                const uint32_t r = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
                a.v[2 * k] = r << 16;
                a.v[2 * k + 1] = r & 0xffff0000u;
            }
            else {
                a.v[2 * k] = f32_through_alu(lo);
                a.v[2 * k + 1] = f32_through_alu(hi);
            }
        }
    }
    static __device__ __forceinline__ u32x4 finish(const Accs<TR>& a) {
        u32x4 r;
#pragma unroll
        for (int k = 0; k < 4; k++) r[k] = (a.v[2 * k] >> 16) | (a.v[2 * k + 1] & 0xffff0000u);
        return r;
    }
};

// One-byte integers: the accumulator stays in storage format (four bytes per dword, in a.v[0..3]) and every byte is
// combined by one instruction that reads byte k of both operands and writes byte k of the accumulator, leaving the
// other three alone (the sub-dword addressing of the gfx9 vector ALU).  Sixteen instructions per vector and step
// where extracting, combining and re-inserting bytes takes the compiler about sixty.  The low byte of a 16-bit sum
// or product of sign- or zero-extended bytes is the wrapped 8-bit result; min and max compare the extended bytes.
#define MI_BYTE_OP(INSTR, S0, S1, K)                                                                              \
    asm(INSTR " %0, " S0 ", " S1 " dst_sel:BYTE_" #K " dst_unused:UNUSED_PRESERVE src0_sel:BYTE_" #K              \
              " src1_sel:BYTE_" #K                                                                                 \
        : "+v"(acc)                                                                                                \
        : "v"(in))
#define MI_BYTE_OP4(INSTR, S0, S1) \
    MI_BYTE_OP(INSTR, S0, S1, 0); MI_BYTE_OP(INSTR, S0, S1, 1); MI_BYTE_OP(INSTR, S0, S1, 2); MI_BYTE_OP(INSTR, S0, S1, 3)
template <bool SIGNED, int OP>
__device__ __forceinline__ uint32_t bytes_step(uint32_t in, uint32_t acc) {
    if (OP == OP_SUM) { MI_BYTE_OP4("v_add_u16_sdwa", "%1", "%0"); }
    else if (OP == OP_PROD) { MI_BYTE_OP4("v_mul_lo_u16_sdwa", "%1", "%0"); }
    else if (OP == OP_MIN && SIGNED) { MI_BYTE_OP4("v_min_i16_sdwa", "sext(%1)", "sext(%0)"); }
    else if (OP == OP_MIN) { MI_BYTE_OP4("v_min_u16_sdwa", "%1", "%0"); }
    else if (SIGNED) { MI_BYTE_OP4("v_max_i16_sdwa", "sext(%1)", "sext(%0)"); }
    else { MI_BYTE_OP4("v_max_u16_sdwa", "%1", "%0"); }
    return acc;
}
#undef MI_BYTE_OP4
#undef MI_BYTE_OP
template <class T>
struct VecOps<PlainTraits<T, uint8_t>> {
    typedef PlainTraits<T, uint8_t> TR;
    static_assert(sizeof(Accs<TR>) == 16, "sixteen one-byte accumulators are the vector itself");
    static __device__ __forceinline__ Accs<TR> init(u32x4 x) { return __builtin_bit_cast(Accs<TR>, x); }
    template <int OP>
    static __device__ __forceinline__ void step(u32x4 x, Accs<TR>& a) {
        u32x4 acc = __builtin_bit_cast(u32x4, a);
#pragma unroll
        for (int k = 0; k < 4; k++) acc[k] = bytes_step<((T)-1 < (T)0), OP>(x[k], acc[k]);
        a = __builtin_bit_cast(Accs<TR>, acc);
    }
    static __device__ __forceinline__ u32x4 finish(const Accs<TR>& a) { return __builtin_bit_cast(u32x4, a); }
};

// fp16: the accumulator stays in storage format (two halves per dword, in a.v[0..3]).  sum and prod widen, combine
// and narrow both halves of a dword.  min and max pick each half with one compare and a bit-field insert; the
// quieting of a NaN they hand back (only the first input can bring one: a NaN `in` is never chosen) does not change
// any later compare, so it is done once at the end, for both halves of a dword at a time -- a.v[4] says whether a
// min/max step has happened at all (with one input there is nothing to quiet).
template <bool NATIVE>
struct VecOps<Fp16Traits<NATIVE>> {
    typedef Fp16Traits<NATIVE> TR;
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ Accs<TR> init(u32x4 x) {
        Accs<TR> a;
#pragma unroll
        for (int k = 0; k < 4; k++) a.v[k] = x[k];
        a.v[4] = 0;
        return a;
    }
    template <int OP>
    static __device__ __forceinline__ void step(u32x4 x, Accs<TR>& a) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const half2_t in = __builtin_bit_cast(half2_t, (uint32_t)x[k]), io = __builtin_bit_cast(half2_t, a.v[k]);
            if (OP == OP_SUM || OP == OP_PROD) {
                const float lo = (OP == OP_SUM) ? ((float)io[0] + (float)in[0]) : ((float)io[0] * (float)in[0]);
                const float hi = (OP == OP_SUM) ? ((float)io[1] + (float)in[1]) : ((float)io[1] * (float)in[1]);
                const half2_t r = { (_Float16)lo, (_Float16)hi };
                a.v[k] = __builtin_bit_cast(uint32_t, r);
            }
            else {
                const bool lo = (OP == OP_MIN) ? (in[0] < io[0]) : (in[0] > io[0]);
                const bool hi = (OP == OP_MIN) ? (in[1] < io[1]) : (in[1] > io[1]);
                const uint32_t m = (lo ? 0x0000ffffu : 0u) | (hi ? 0xffff0000u : 0u);
                a.v[k] = (x[k] & m) | (a.v[k] & ~m);
            }
        }
        if (OP == OP_MIN || OP == OP_MAX) a.v[4] = 1;
    }
    static __device__ __forceinline__ u32x4 finish(const Accs<TR>& a) {
        u32x4 r = { a.v[0], a.v[1], a.v[2], a.v[3] };
        if (!NATIVE && a.v[4]) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                // a half h is a NaN iff (h & 0x7fff) > 0x7c00 iff (h & 0x7fff) + 0x03ff has bit 15 set
                const uint32_t nan = ((r[k] & 0x7fff7fffu) + 0x03ff03ffu) & 0x80008000u;
                r[k] |= nan >> 6;      // the quiet bit, 0x0200, of each NaN half
            }
        }
        return r;
    }
};

// bf16 accumulated in fp32 and rounded to nearest even once: element-wise init and step, packed narrowing.
template <>
struct VecOps<Bf16KeepTraits<true>> {
    typedef Bf16KeepTraits<true> TR;
    static __device__ __forceinline__ Accs<TR> init(u32x4 x) {
        Accs<TR> a;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            a.v[2 * k] = x[k] << 16;
            a.v[2 * k + 1] = x[k] & 0xffff0000u;
        }
        return a;
    }
    template <int OP>
    static __device__ __forceinline__ void step(u32x4 x, Accs<TR>& a) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            a.v[2 * k] = f32_step_bits<OP, false>(x[k] << 16, a.v[2 * k]);
            a.v[2 * k + 1] = f32_step_bits<OP, false>(x[k] & 0xffff0000u, a.v[2 * k + 1]);
        }
    }
    static __device__ __forceinline__ u32x4 finish(const Accs<TR>& a) {
        u32x4 r;
#pragma unroll
        for (int k = 0; k < 4; k++) r[k] = bf16_narrow_rne_pack2(a.v[2 * k], a.v[2 * k + 1]);
        return r;
    }
};

template <class TR>
__device__ __forceinline__ Accs<TR> vec_init(u32x4 x) {
    return VecOps<TR>::init(x);
}
template <class TR, int OP>
__device__ __forceinline__ void vec_step(u32x4 x, Accs<TR>& a) {
    VecOps<TR>::template step<OP>(x, a);
}
template <class TR>
__device__ __forceinline__ u32x4 vec_finish(const Accs<TR>& a) {
    return VecOps<TR>::finish(a);
}

// Streaming 128-bit accesses through pointers that promise no alignment (the instruction is the same one).  The
// memory pipeline takes a vector access at any byte address (a wave's 1 KiB then touches one cache line more), so
// buffers that disagree modulo 16 bytes -- tensors behind an odd-sized one in a tightly packed fusion buffer, a
// peer's chunk at an odd offset -- still move as vectors.  The host starts the vectors on the 16-byte boundary of the
// buffer that makes the loose accesses cheapest (vector_head).
typedef u32x4 u32x4_u __attribute__((aligned(1)));
#ifdef MI_EXP_LD_PLAIN
__device__ __forceinline__ u32x4 ld_loose(const u32x4_u* p) { return *p; }
#else
__device__ __forceinline__ u32x4 ld_loose(const u32x4_u* p) { return __builtin_nontemporal_load(p); }
#endif
__device__ __forceinline__ void st_loose(u32x4_u* p, u32x4 v) { __builtin_nontemporal_store(v, p); }
// The same store with device scope on top (sc1 nt).  A 1 : 1 copy gains 2-6 % from it (6.65 against 6.50 TB/s at
// 512 MiB, 6.19 against 5.85 at 64 MiB); the reduce kernels, the converters, pack / unpack and the broadcast measure
// 0-8 % slower with it, so only the copy uses it.  The compiler does not know that this is a store, so what it would
// do for one is done by hand: (1) gfx9 reads the data registers of a vector-memory store of more than 64 bits up to two
// cycles after issue, and a VALU or VMEM write to them in that window is a hazard the compiler's hazard pass covers with
// wait states -- hence the "s_nop 1" (two wait states) inside the same asm statement, which nothing can be scheduled
// into (without it 3 % of a 2-input reduce's elements came back as the NEXT iteration's data); (2) "memory" keeps
// loads and stores from moving across it; (3) the asm is counted by no s_waitcnt the compiler emits, which is harmless
// for a store whose completion nobody waits for (the kernel's end drains it).  Bit-exact copy tests with odd heads and
// tails, across several launches, cover it (tests/test_gpu_parity.py, tests/test_gpu_large_launches.py).
__device__ __forceinline__ void st_loose_device_scope(u32x4_u* p, u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}
template <class E>
struct __attribute__((packed)) LooseElem {
    E v;
};
template <class E>
__device__ __forceinline__ E ld_elem(const void* p, uint64_t i) {
    return ((const LooseElem<E>*)p)[i].v;
}
template <class E>
__device__ __forceinline__ void st_elem(void* p, uint64_t i, E x) {
    ((LooseElem<E>*)p)[i].v = x;
}

// ---- inputs that sit 1-3 bytes off a 4-byte boundary ------------------------------------------------------------------
// A loose vector load is nearly free while its address is a multiple of 4 and dear when it is not (every dword of the
// lane then straddles two: 8 x 1 GiB bf16 with the peers 2 bytes off the vectors' boundary ran at 5.66 against 7.14
// TB/s).  Such an input -- a peer's block behind an odd number of 16-bit elements, the tensors behind an odd-sized one
// in a tightly packed fusion buffer, int8 at any odd offset -- is therefore read from the 4-byte boundary s = 1..3
// bytes below the lane's vector, and the vector is put together in registers: its last s bytes are the first bytes of
// the NEXT lane's load (fetched with a DPP wave shift, no memory or LDS instruction), and every dword is one
// v_alignbyte_b32 of two neighbours.  Lane 63 has no next lane: it alone loads one more dword.  The lane behind the
// last vector that is computed must load too (only its first dword is used), which is why the host, when any input of
// a launch needs this, hands the last whole vector to the element-wise edge lanes: vector `nvec` is then still inside
// every buffer and may be read (nload = nvec + 1).  All of this runs in wave-uniform control flow around the DPP.
__device__ __forceinline__ uint32_t from_next_lane(uint32_t mine, uint32_t for_last_lane) {
    // wave_shl:1 -- lane i reads `mine` of lane i + 1; lane 63, whose source is out of range, keeps `for_last_lane`
    return (uint32_t)__builtin_amdgcn_update_dpp((int)for_last_lane, (int)mine, 0x130, 0xf, 0xf, false);
}
template <int K>
__device__ __forceinline__ uint32_t from_lane_of_quad(uint32_t v) {     // every lane reads lane K of its group of four
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, K * 0x55, 0xf, 0xf, false);
}
__device__ __forceinline__ u32x4 shift_into_place(u32x4 x, uint32_t next0, uint32_t s) {
    u32x4 r;
    r[0] = __builtin_amdgcn_alignbyte(x[1], x[0], s);
    r[1] = __builtin_amdgcn_alignbyte(x[2], x[1], s);
    r[2] = __builtin_amdgcn_alignbyte(x[3], x[2], s);
    r[3] = __builtin_amdgcn_alignbyte(next0, x[3], s);
    return r;
}

// The dwords behind lane 63's G vectors (sa: the input's 4-byte boundary below its first vector), fetched by ONE load
// instruction: lane 64 - G + g fetches the one of vector g.  Zero in the other lanes and where lane 63's vector is not
// computed.  G is 1, 2 or 4, so the fetching lanes are lanes of the wave's last group of four.
template <int G, bool FULL>
__device__ __forceinline__ uint32_t load_behind_last_lane(const u32x4_u* sa, const uint64_t (&idx)[G], uint64_t nvec) {
    static_assert(G == 1 || G == 2 || G == 4, "the fetching lanes must be lanes of one group of four");
    const uint32_t lane = threadIdx.x & 63u;
    uint32_t e = 0;
    if (lane >= 64u - G) {
        // idx[lane - (64 - G)], picked by compare-and-select; the empty asm keeps the compiler from turning the chain
        // into an indexed read of idx[], which it would put in scratch memory
        uint32_t lo = (uint32_t)idx[0], hi = (uint32_t)(idx[0] >> 32);
#pragma unroll
        for (int g = 1; g < G; g++) {
            const bool mine = lane == 64u - G + g;
            lo = mine ? (uint32_t)idx[g] : lo;
            hi = mine ? (uint32_t)(idx[g] >> 32) : hi;
            asm("" : "+v"(lo), "+v"(hi));
        }
        const uint64_t i = (((uint64_t)hi << 32) | lo) + (63u - lane);      // lane 63's vector g
        if (FULL || i < nvec) e = __builtin_nontemporal_load((const uint32_t*)(sa + i + 1));
    }
    return e;
}
// x[g] as loaded from sa -> the vectors that start s bytes further on; e: load_behind_last_lane's result
template <int G>
__device__ __forceinline__ void shift_vectors(u32x4 (&x)[G], uint32_t e, uint32_t s) {
    if constexpr (G == 4) {
        x[0] = shift_into_place(x[0], from_next_lane(x[0][0], from_lane_of_quad<0>(e)), s);
        x[1] = shift_into_place(x[1], from_next_lane(x[1][0], from_lane_of_quad<1>(e)), s);
        x[2] = shift_into_place(x[2], from_next_lane(x[2][0], from_lane_of_quad<2>(e)), s);
        x[3] = shift_into_place(x[3], from_next_lane(x[3][0], from_lane_of_quad<3>(e)), s);
    }
    else if constexpr (G == 2) {
        x[0] = shift_into_place(x[0], from_next_lane(x[0][0], from_lane_of_quad<2>(e)), s);
        x[1] = shift_into_place(x[1], from_next_lane(x[1][0], from_lane_of_quad<3>(e)), s);
    }
    else {
        x[0] = shift_into_place(x[0], from_next_lane(x[0][0], e), s);
    }
}

// Vectors idx[0..G) of one input whose first vector starts at `base` (any alignment): x[g] is the vector for every
// idx[g] < nvec; what the other lanes get is unspecified (they must not store).  ES: element size; FULL: the caller
// knows that every idx[g] of every lane of the wave is below nvec.  nload > nvec switches the in-register
// realignment on for an input that is off a 4-byte boundary (vector nvec must then be readable).  Must be called by
// all lanes of a wave together, with idx[g] of lane i + 1 = idx[g] of lane i + 1.
template <int ES, int G, bool FULL>
__device__ __forceinline__ void load_vectors(const unsigned char* base, const uint64_t (&idx)[G], uint64_t nvec,
                                             uint64_t nload, u32x4 (&x)[G]) {
    if constexpr (ES < 4) {
        const uint32_t s = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)base & 3u);
        if (s != 0 && nload > nvec) {
            const u32x4_u* sa = (const u32x4_u*)(base - s);
#pragma unroll
            for (int g = 0; g < G; g++) x[g] = (FULL || idx[g] < nload) ? ld_loose(sa + idx[g]) : u32x4{ 0, 0, 0, 0 };
            const uint32_t e = load_behind_last_lane<G, FULL>(sa, idx, nvec);
            shift_vectors<G>(x, e, s);
            return;
        }
    }
    const u32x4_u* sp = (const u32x4_u*)base;
#pragma unroll
    for (int g = 0; g < G; g++) x[g] = (FULL || idx[g] < nvec) ? ld_loose(sp + idx[g]) : u32x4{ 0, 0, 0, 0 };
}

// Element i of inputs p[first] .. p[last - 1] folded into r in that order, eight loads in flight together (a plain
// loop waits for every load before the next is issued: one trip to memory per input at the end of a launch).
template <class TR, int OP, class PTR>
__device__ __forceinline__ typename TR::acc_t fold_element(const PTR* p, int first, int last, uint64_t i,
                                                           typename TR::acc_t r) {
    typedef typename TR::elem_t E;
    for (int j0 = first; j0 < last; j0 += 8) {
        E x[8];
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (j0 + u < last) x[u] = ld_elem<E>(p[j0 + u], i);
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (j0 + u < last) r = TR::template step<OP>(x[u], r);
    }
    return r;
}

// The count % VEC elements after the last full vector and the elements before the first aligned one:
// at most 127 + 2 * VEC - 1 <= 158 elements (the head may reach to a 128-byte line), one per lane of block 0.
template <class TR, int OP, class SRC>
__device__ __forceinline__ void reduce_edges(const SRC& src, int n, void* dst, uint32_t head, uint64_t nvec,
                                             uint32_t tail) {
    typedef typename TR::elem_t E;
    uint32_t t = threadIdx.x;
    if (t < head + tail) {
        uint64_t i = (t < head) ? t : (uint64_t)head + nvec * TR::VEC + (t - head);
        const typename TR::acc_t a = fold_element<TR, OP>(src.p, 1, n, i, TR::init(ld_elem<E>(src.p[0], i)));
        st_elem<E>(dst, i, TR::finish(a));
    }
}

// tile index sequence of one block: plain grid stride, or per-XCD contiguous shares (blocks are handed to
// the 8 XCDs round-robin, so blockIdx & 7 names the XCD a block runs on)
struct TileIter {
    uint64_t tile, end, stride;
    __device__ __forceinline__ TileIter(uint64_t ntiles, int xcd_chunked) {
        if (xcd_chunked && (gridDim.x & 7u) == 0) {
            uint64_t per_xcd = (ntiles + 7) >> 3;
            uint64_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3;
            tile = xcd * per_xcd + slot;
            end = (xcd + 1) * per_xcd < ntiles ? (xcd + 1) * per_xcd : ntiles;
            stride = gridDim.x >> 3;
        }
        else {
            tile = blockIdx.x;
            end = ntiles;
            stride = gridDim.x;
        }
    }
};

// Fixed N (1..8): all N*UNROLL loads of a tile are issued before the first use.  `beyond` (0 or 1): vector nvec may be
// read, which lets inputs off a 4-byte boundary be realigned in registers (load_vectors).
template <class TR, int OP, int N, int UNROLL>
__global__ void __launch_bounds__(kBlock)
reduce_vec_kernel(SrcFixed<N> src, void* dst, uint32_t head, uint64_t nvec, uint32_t tail, int xcd_chunked, uint32_t beyond) {
    typedef typename TR::elem_t E;
    kernel_prologue<TR, OP>();
    constexpr uint64_t kTile = (uint64_t)kBlock * UNROLL;
    const unsigned char* s[N];
#pragma unroll
    for (int j = 0; j < N; j++) s[j] = (const unsigned char*)src.p[j] + head * sizeof(E);
    u32x4_u* d = (u32x4_u*)((unsigned char*)dst + head * sizeof(E));
    const uint64_t ntiles = (nvec + kTile - 1) / kTile;
    const uint64_t nload = nvec + beyond;

    for (TileIter it(ntiles, xcd_chunked); it.tile < it.end; it.tile += it.stride) {
        uint64_t idx[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) idx[u] = it.tile * kTile + threadIdx.x + (uint64_t)u * kBlock;
        u32x4 x[N][UNROLL];
        if ((it.tile + 1) * kTile <= nvec) {        // a whole tile (the same answer for every lane of the block)
#pragma unroll
            for (int j = 0; j < N; j++) load_vectors<sizeof(E), UNROLL, true>(s[j], idx, nvec, nload, x[j]);
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                Accs<TR> a = vec_init<TR>(x[0][u]);
#pragma unroll
                for (int j = 1; j < N; j++) vec_step<TR, OP>(x[j][u], a);
                st_loose(d + idx[u], vec_finish<TR>(a));
            }
        }
        else {
#pragma unroll
            for (int j = 0; j < N; j++) load_vectors<sizeof(E), UNROLL, false>(s[j], idx, nvec, nload, x[j]);
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                Accs<TR> a = vec_init<TR>(x[0][u]);
#pragma unroll
                for (int j = 1; j < N; j++) vec_step<TR, OP>(x[j][u], a);
                if (idx[u] < nvec) st_loose(d + idx[u], vec_finish<TR>(a));
            }
        }
    }
    if (blockIdx.x == 0 && (head | tail)) reduce_edges<TR, OP>(src, N, dst, head, nvec, tail);
}

// ---------------------------------------------------------------------------------------------------
// Phased kernel for large buffers.
//
// HBM on this part loses about a quarter of its bandwidth when reads and writes are interleaved (an
// 8-read + 1-write stream sustains ~5.5 TB/s where reads alone reach ~7.1 TB/s and writes alone ~6 TB/s).
// reduce_multi_phased_kernel (further down) keeps the two apart in time, chip-wide: one 512-lane block per CU reduces up to 44 vectors per
// lane into LDS and registers (read phase: HBM sees only reads), all blocks meet at a barrier, then every block
// streams its staged results out (write phase: HBM sees only writes), and they meet again.  Each phase boundary
// costs a few microseconds of idle HBM, so a phase holds as much as the CU can: 160 KiB of LDS plus up to 24
// vectors per lane in registers (8 waves per CU leave 256 registers per lane).
//
// The barrier carries no data between blocks -- it only aligns them in time -- so a block that waits too
// long simply goes on (and stops waiting for the rest of the launch): the result is the same whether the
// barrier holds or not, and no wave can spin forever.

constexpr int kPhaseBlock = 512;                  // 8 wavefronts, one block per CU
constexpr int kPhaseU = 20;                       // vectors per lane per phase staged in LDS: 20 x 16 B x 512 lanes = 160 KiB
constexpr int kPhaseGroups = 16;                  // arrival counters (same-address atomics serialise)
constexpr long kPhaseSpinTicks = 20000;           // default bound on one wait, in 100 MHz ticks: 200 us

struct __attribute__((aligned(256))) PhaseWord {
    unsigned v;
    unsigned pad[63];
};
struct PhaseSync {
    PhaseWord grp[kPhaseGroups];    // arrivals per group of blocks
    PhaseWord top;                  // groups that are complete: kPhaseGroups more with every barrier
};

#define MI_ALOAD(p) __hip_atomic_load((p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define MI_AADD(p, x) __hip_atomic_fetch_add((p), (x), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)

// A barrier in two halves.  One thread of every block reports the block's arrival (phase_arrive), every block does so
// the same number of times per launch (twice per phase, except after the last phase's writes), so the counters stay
// multiples of their group sizes from launch to launch.  A barrier is complete when `top` has counted kPhaseGroups
// complete groups more: the last block of a group bumps `top`, and the waiters poll `top` itself (a third word bumped
// by the last group measured 0.3 % slower: one more dependent atomic between the last arrival and the release; the
// 16 group words polled directly by 16 lanes 1.2 % slower).  gen counts barriers: a block waits for
// top >= gen * kPhaseGroups (phase_wait, called by all its threads).
//
// The halves are apart on purpose.  From the last arrival to the moment the waiting blocks see the release, two
// dependent atomics and a poll go to memory and back, about 2 us in which HBM would idle.  So a block reports its
// arrival a little before it is done: with Tuning::early_loads vector loads per lane of the read phase still to
// issue, and with Tuning::early_stores stores per lane of the write phase still to issue (its first wave, whose
// thread 0 reports, has then seen all its earlier stores acknowledged, because the returning atomic waits for
// them).  The release then reaches the blocks about when the slowest of them finishes.  Measured on 8 x 2 GB bf16:
// 2.619 ms with arrival at the end of each phase, 2.580 with 4 loads, 2.545 with 8, 2.536 with 12 and 2.540 with 16
// early loads (4 early stores each; 8 or 12 early stores measure 0.2-0.5 % slower than 4).
__device__ __forceinline__ unsigned phase_generation(const PhaseSync* ps) {
    return MI_ALOAD(&ps->top.v) / kPhaseGroups;     // at kernel start: the barriers completed so far
}
__device__ __forceinline__ void phase_arrive(PhaseSync* ps) {
    const unsigned per = gridDim.x / kPhaseGroups;
    const unsigned old = MI_AADD(&ps->grp[blockIdx.x % kPhaseGroups].v, 1u);
    if ((old + 1u) % per == 0u) {
        MI_AADD(&ps->top.v, 1u);
    }
}
// No data crosses the barrier (a lane only ever reads back the LDS slots it wrote itself), so the waves of a block
// are held by a bare s_barrier: nothing has to wait for the block's outstanding stores.
__device__ __forceinline__ void phase_wait(PhaseSync* ps, unsigned gen, bool& give_up, long spin_ticks) {
    if (threadIdx.x == 0 && !give_up) {
        const long long t0 = wall_clock64();
        while ((int)(MI_ALOAD(&ps->top.v) - gen * kPhaseGroups) < 0) {
            __builtin_amdgcn_s_sleep(1);
            if (wall_clock64() - t0 >= spin_ticks) {
                give_up = true;
                break;
            }
        }
    }
    __builtin_amdgcn_s_barrier();
}

// G vectors per lane of N inputs (a compile-time count) at once: all N x G loads are issued before the first is
// used, vector 0 of every input, then vector 1 of every input, ...; the inputs that are realigned in registers get
// their one extra load each behind those, and are shifted into place when everything is under way.  base[j]: where
// input j's first vector starts; idx, nvec, nload, FULL as for load_vectors.
template <class TR, int OP, int N, int G, bool FULL>
__device__ __forceinline__ void reduce_group(const unsigned char* const (&base)[N], const uint64_t (&idx)[G], uint64_t nvec,
                                             uint64_t nload, u32x4 (&out)[G]) {
    typedef typename TR::elem_t E;
    u32x4 x[N][G];
    if constexpr (sizeof(E) < 4) {
        uint32_t s[N], e[N];
        const u32x4_u* sa[N];
        uint32_t any = 0;
#pragma unroll
        for (int j = 0; j < N; j++) {
            s[j] = nload > nvec ? __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)base[j] & 3u) : 0u;
            sa[j] = (const u32x4_u*)(base[j] - s[j]);
            any |= s[j];
        }
#pragma unroll
        for (int g = 0; g < G; g++)
#pragma unroll
            for (int j = 0; j < N; j++)
                x[j][g] = (FULL || idx[g] < (s[j] ? nload : nvec)) ? ld_loose(sa[j] + idx[g]) : u32x4{ 0, 0, 0, 0 };
        if (any) {
#pragma unroll
            for (int j = 0; j < N; j++) e[j] = s[j] ? load_behind_last_lane<G, FULL>(sa[j], idx, nvec) : 0u;
#pragma unroll
            for (int j = 0; j < N; j++)
                if (s[j]) shift_vectors<G>(x[j], e[j], s[j]);
        }
    }
    else {
#pragma unroll
        for (int g = 0; g < G; g++)
#pragma unroll
            for (int j = 0; j < N; j++)
                x[j][g] = (FULL || idx[g] < nvec) ? ld_loose((const u32x4_u*)base[j] + idx[g]) : u32x4{ 0, 0, 0, 0 };
    }
#pragma unroll
    for (int g = 0; g < G; g++) {
        Accs<TR> a = vec_init<TR>(x[0][g]);
#pragma unroll
        for (int j = 1; j < N; j++) vec_step<TR, OP>(x[j][g], a);
        out[g] = vec_finish<TR>(a);
    }
}

// ---------------------------------------------------------------------------------------------------
// Run-time counts of inputs (up to 64) and destinations (up to 16): the reduced vector is stored to each of m buffers (the reference's allreduce_kernel stores
// to the own and to the peer's output, kernels.cl:190-217; with one input this is write_monolithic_kernel_N,
// kernels.cl:423-560).  Inputs and outputs are run-time counts.  A lane reads its element from every input before
// it stores it anywhere, so a destination may be one of the inputs.

template <class TR, int OP, int UNROLL>
__device__ __forceinline__ void reduce_rt_tile(const SrcTable& src, int n, uint32_t head, const uint64_t (&idx)[UNROLL],
                                               uint64_t nvec, uint64_t nload, u32x4 (&out)[UNROLL],
                                               PhaseSync* arrive_ps = nullptr, int arrive_j = 0) {
    typedef typename TR::elem_t E;
    Accs<TR> a[UNROLL];
    u32x4 x[UNROLL];
    load_vectors<sizeof(E), UNROLL, false>((const unsigned char*)src.p[0] + head * sizeof(E), idx, nvec, nload, x);
#pragma unroll
    for (int u = 0; u < UNROLL; u++) a[u] = vec_init<TR>(x[u]);
    for (int j = 1; j < n; j++) {
        if (j == arrive_j && threadIdx.x == 0) phase_arrive(arrive_ps);     // arrive_j == 0: never
        load_vectors<sizeof(E), UNROLL, false>((const unsigned char*)src.p[j] + head * sizeof(E), idx, nvec, nload, x);
#pragma unroll
        for (int u = 0; u < UNROLL; u++) vec_step<TR, OP>(x[u], a[u]);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) out[u] = vec_finish<TR>(a[u]);
}

template <class TR, int OP>
__device__ __forceinline__ void reduce_multi_edges(const SrcTable& src, int n, const DstTable& dst, int m, uint32_t head,
                                                   uint64_t nvec, uint32_t tail) {
    typedef typename TR::elem_t E;
    uint32_t t = threadIdx.x;
    if (t < head + tail) {
        uint64_t i = (t < head) ? t : (uint64_t)head + nvec * TR::VEC + (t - head);
        const typename TR::acc_t a = fold_element<TR, OP>(src.p, 1, n, i, TR::init(ld_elem<E>(src.p[0], i)));
        const E r = TR::finish(a);
        for (int k = 0; k < m; k++) st_elem<E>(dst.p[k], i, r);
    }
}

template <class TR, int OP, int UNROLL>
__global__ void __launch_bounds__(kBlock)
reduce_multi_kernel(SrcTable src, int n, DstTable dst, int m, uint32_t head, uint64_t nvec, uint32_t tail,
                    int xcd_chunked, uint32_t beyond) {
    typedef typename TR::elem_t E;
    kernel_prologue<TR, OP>();
    constexpr uint64_t kTile = (uint64_t)kBlock * UNROLL;
    const uint64_t ntiles = (nvec + kTile - 1) / kTile;
    const uint64_t nload = nvec + beyond;
    for (TileIter it(ntiles, xcd_chunked); it.tile < it.end; it.tile += it.stride) {
        uint64_t idx[UNROLL];
        u32x4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) idx[u] = it.tile * kTile + threadIdx.x + (uint64_t)u * kBlock;
        reduce_rt_tile<TR, OP, UNROLL>(src, n, head, idx, nvec, nload, v);
        for (int k = 0; k < m; k++) {
            u32x4_u* d = (u32x4_u*)((unsigned char*)dst.p[k] + head * sizeof(E));
#pragma unroll
            for (int u = 0; u < UNROLL; u++)
                if (idx[u] < nvec) st_loose(d + idx[u], v[u]);
        }
    }
    if (blockIdx.x == 0 && (head | tail)) reduce_multi_edges<TR, OP>(src, n, dst, m, head, nvec, tail);
}

// Groups of four result vectors per lane that the phased form below keeps in registers on top of the kPhaseU vectors
// it keeps in LDS.  A traits class with heavier arithmetic specialises this before its kernels are instantiated; the
// build fails on any scratch use.
template <class TR>
struct MultiPhaseRegs {
    static constexpr int groups = 6;
};

// Stores per lane still to issue when a block reports the end of its write phase (Tuning::early_stores < 0 asks for
// this).  Measured at 2 GB per buffer, 16 against 4: fp32 +1.2 % with 8 inputs, +1.6 % with 4, +2.7 % with 2; the two
// bfloat16 families +0.1-0.3 %, +0.4-0.8 % and +1.5-1.9 %; 20 is within 0.3 % of 16 either way.
constexpr int kPhaseEarlyStores = 16;
// With several destinations the block's waves meet before each of them (see the write phase below), so the report
// that goes out 16 stores before the end of the last destination speaks for the whole block; without that meeting an
// early report with three or more destinations let the next reads start under far too many outstanding writes (8 -> 8
// at 1 GiB: 5.78 TB/s with 4 stores early against 6.25 with a strict report, 6.45 with the meeting and 16 early).  When
// the clock paces the write phase (Tuning::write_pace) the last destination's 20 LDS-staged stores all come after the
// report: 6.98 against 6.94 with 16.
// Element types and operations whose read phase carries a lot of arithmetic per byte: the 8-bit types (byte lanes),
// both bfloat16 families (widen, round) and fp16 min / max (NaN handling).
template <class TR, int OP>
struct PhaseHeavy {
    static constexpr bool value = sizeof(typename TR::elem_t) == 1;
};
template <bool RNE, bool VEC_SEM, int OP>
struct PhaseHeavy<Bf16PairwiseTraits<RNE, VEC_SEM>, OP> {
    static constexpr bool value = true;
};
template <bool RNE, int OP>
struct PhaseHeavy<Bf16KeepTraits<RNE>, OP> {
    static constexpr bool value = true;
};
template <bool NATIVE, int OP>
struct PhaseHeavy<Fp16Traits<NATIVE>, OP> {
    static constexpr bool value = OP == OP_MIN || OP == OP_MAX;
};

// Up to how many inputs a reduce to ONE destination has its write phase paced by the clock (see the kernel), at 1.1 x
// Tuning::write_pace: the blocks of the chip then start the read phase that follows in step, which pays the more the
// shorter that phase is.  Measured at 512 MiB per buffer against the unpaced kernel, each with its best early arrival
// (phase_early_loads below): 2 inputs +1-4 %, 3 inputs +2.0-3.4 %, 4 inputs +1.2-3.0 %, 5 and 6 inputs +1.5-2.3 %,
// 8 inputs +0.6-1.8 % (bfloat16, fp32 accumulation, 8 x 2 GB: 7.15-7.17 against 7.07-7.085 TB/s), 12 inputs
// +0.4-1.1 % (the rounded-every-step bfloat16 family and bfloat16 min / max +-0), 16 inputs +0.5-0.8 % for the light
// types and -0.7..+0.5 % for the heavy ones, which stay unpaced there.
template <class TR, int OP>
struct PhasePacedInputs {
    static constexpr int value = PhaseHeavy<TR, OP>::value ? 12 : 16;
};

// Loads per lane still to issue when a block reports the end of its read phase (Tuning::early_loads < 0 asks for
// this).  Unpaced, 12 hides the barrier's latency best for every type (8 to 16 are within 0.3 %).  Behind a paced write
// phase the blocks reach the end of their reads almost together, and an arrival that early lets the first stores out
// under the last reads: the light types then want 12 with up to four inputs and 8 from five on (+0.3-1 %), the heavy
// ones 8 with two inputs, 5 with three and four, 2 from five on (512 MiB per buffer, 12 against the best: int8 with 4
// inputs 6.92 against 7.09 TB/s, with 8 inputs 7.00 against 7.16; bfloat16 with 8 inputs 7.08 against 7.23, with 3
// inputs 6.76 against 6.91; fp16 max with 4 inputs 6.83 against 7.01).  The same holds with several destinations
// (1 GiB per buffer, bfloat16: 8 -> 8 6.92 against 7.12, 8 -> 2 6.93 against 7.08, 4 -> 4 6.91 against 7.02; one buffer
// copied to 2: 6.80 against 6.88).
constexpr int kPhaseEarlyLoads = 12;
template <class TR, int OP>
inline int phase_early_loads(const Tuning& t, int n, bool paced) {
    if (t.early_loads >= 0) return t.early_loads;
    if (!paced) return kPhaseEarlyLoads;
    if (PhaseHeavy<TR, OP>::value) return n <= 2 ? 8 : n <= 4 ? 5 : 2;
    return n <= 4 ? kPhaseEarlyLoads : 8;
}

template <class TR>
inline int phase_early_stores(const Tuning& t, int n_dsts) {
    const int v = t.early_stores >= 0 ? t.early_stores : n_dsts >= 2 ? (t.write_pace > 0 ? kPhaseU : 16) : kPhaseEarlyStores;
    return v < kPhaseU ? v : kPhaseU;
}

// The phased form of the same: kPhaseU vectors per lane in LDS and 4 x RG in registers (RG = MultiPhaseRegs::groups, or
// one more where that saves a phase: phase_reg_groups) are
// reduced while HBM sees only reads, then stored to every destination while it sees only writes.  The register
// groups are unrolled (a register file has no run-time index); the loop over the inputs inside each stays a loop.
template <class TR, int OP, int RG>
__global__ void __launch_bounds__(kPhaseBlock)
reduce_multi_phased_kernel(SrcTable src, int n, DstTable dst, int m, uint32_t head, uint64_t nvec, uint32_t tail,
                           PhaseSync* ps, int early_loads, int early_stores, long spin_ticks, uint32_t beyond,
                           uint32_t wave_runs, uint32_t write_pace16) {
    typedef typename TR::elem_t E;
    kernel_prologue<TR, OP>();
    const uint64_t nload = nvec + beyond;               // vector nvec may be read when beyond = 1 (load_vectors)
    constexpr int G = 4;                                // vectors per lane and input in flight
    constexpr int LG = kPhaseU / G;                     // groups staged in LDS
    static_assert(kPhaseU % G == 0, "LDS steps must be a multiple of the group size");
    __shared__ u32x4 stage[kPhaseU * kPhaseBlock];
    const uint64_t gthreads = (uint64_t)gridDim.x * kPhaseBlock;
    const uint64_t gtid = (uint64_t)blockIdx.x * kPhaseBlock + threadIdx.x;
    const uint64_t per_phase = gthreads * (uint64_t)(G * (RG + LG));
    // Slot u of this lane.  The G slots of a group lie one slab (gthreads vectors) apart: at every step the chip reads
    // G compact windows.  With wave_runs they lie 64 vectors apart instead, so that a wave covers G KiB in one run and a
    // block 32 KiB: buffers that are off the 128-byte lines then share a line between two waves a quarter as often.
    const uint64_t lane_base = wave_runs ? (gtid & ~(uint64_t)63) * G + (threadIdx.x & 63u) : gtid;
    const uint64_t slot_step = wave_runs ? 64u : gthreads;
    auto pos = [&](uint64_t p0, int u) -> uint64_t {
        return p0 + (uint64_t)(u / G) * (G * gthreads) + lane_base + (uint64_t)(u % G) * slot_step;
    };
    bool give_up = false;
    unsigned gen = 0;
    if (threadIdx.x == 0) gen = phase_generation(ps);
    for (uint64_t p0 = 0; p0 < nvec; p0 += per_phase) {
        u32x4 rs[G * (RG > 0 ? RG : 1)];
#pragma unroll
        for (int q = 0; q < RG; q++) {
            uint64_t idx[G];
            u32x4 v[G];
#pragma unroll
            for (int g = 0; g < G; g++) idx[g] = pos(p0, q * G + g);
            if (idx[0] < nload) {
                reduce_rt_tile<TR, OP, G>(src, n, head, idx, nvec, nload, v);
#pragma unroll
                for (int g = 0; g < G; g++) rs[q * G + g] = v[g];
            }
        }
        bool arrived = false;       // thread 0 has reported this block's arrival at the end of the read phase
        for (int q = 0; q < LG; q++) {
            uint64_t idx[G];
            u32x4 v[G];
#pragma unroll
            for (int g = 0; g < G; g++) idx[g] = pos(p0, (RG + q) * G + g);
            if (idx[0] >= nload) break;     // slabs grow with q: nothing further for this lane in this phase
            // the arrival goes in front of the first load that leaves early_loads or fewer still to issue
            const int rem = (LG - q) * n * G;
            int arrive_j = 0;
            if (!arrived) {
                const int j = rem > early_loads ? (rem - early_loads + G - 1) / G : 0;
                if (j == 0 && threadIdx.x == 0) phase_arrive(ps);
                arrive_j = j < n ? j : 0;
                arrived = j < n;
            }
            reduce_rt_tile<TR, OP, G>(src, n, head, idx, nvec, nload, v, ps, arrive_j);
#pragma unroll
            for (int g = 0; g < G; g++) stage[(q * G + g) * kPhaseBlock + threadIdx.x] = v[g];
        }
        if (early_loads == 0) __syncthreads();      // "when done" means the whole block, and its loads have landed
        if (!arrived && threadIdx.x == 0) phase_arrive(ps);
        phase_wait(ps, ++gen, give_up, spin_ticks);
        const bool more = p0 + per_phase < nvec;
        const int arrive_u = more ? kPhaseU - early_stores : -1;    // kPhaseU: after the last store
        // With several destinations the write phase is hundreds of stores per lane long, the blocks drift apart, and the
        // chip no longer writes one compact window of addresses at a time: HBM then takes the writes at 5.9 TB/s
        // instead of the 6.8 of a write-only stream.  So the clock lets the stores out: group i of four stores (8 MiB
        // over the chip) not before the phase's start + i * write_pace16 / 16 ticks, a little faster than HBM takes them.
        // Every block reads the same clock, so the blocks stay within a fraction of a group of each other without
        // exchanging a word; a block that is behind the schedule is never held.  8 -> 8 at 1 GiB: 6.95 against 6.40
        // TB/s, 4 -> 4: 6.90 against 6.35, 2 -> 2: 6.63 against 6.30.  With one destination (44 stores per lane) a pace
        // a tenth faster keeps the blocks in step for the read phase that follows, which pays while that is short
        // (PhasePacedInputs).
        uint64_t pace_next16 = write_pace16 ? (uint64_t)wall_clock64() << 4 : 0;
        auto paced = [&](int u) {       // u: slot within the phase; groups that lie behind the end of the data take no time
            if (write_pace16 && (u & 3) == 0 && p0 + (uint64_t)u * gthreads < nvec) {
                while (((uint64_t)wall_clock64() << 4) < pace_next16) __builtin_amdgcn_s_sleep(1);
                pace_next16 += write_pace16;
            }
        };
        for (int k = 0; k < m; k++) {
            // The block's waves start every destination together: left alone they drift apart over the several hundred
            // stores per lane of a phase with many destinations, the chip then writes to several destinations at once,
            // and an early report from the first wave says little about the others (8 -> 8 at 1 GiB: 6.45 against 6.25
            // TB/s, 4 -> 4: 6.37 against 6.17, 8 -> 16: 6.2 against 5.95; a further meeting half-way through a destination
            // costs 1 % again).
            if (k > 0) __syncthreads();
            u32x4_u* d = (u32x4_u*)((unsigned char*)dst.p[k] + head * sizeof(E));
#pragma unroll
            for (int u = 0; u < G * RG; u++) {
                const uint64_t i = pos(p0, u);
                paced(u);
                if (i < nvec) st_loose(d + i, rs[u]);
            }
            for (int u = 0; u < kPhaseU; u++) {
                const uint64_t i = pos(p0, G * RG + u);
                paced(G * RG + u);
                if (u == arrive_u && k == m - 1 && threadIdx.x == 0) phase_arrive(ps);
                if (i < nvec) st_loose(d + i, stage[u * kPhaseBlock + threadIdx.x]);
            }
        }
        if (more && arrive_u == kPhaseU) {
            __syncthreads();                        // "when done": every wave's stores have been acknowledged
            if (threadIdx.x == 0) phase_arrive(ps);
        }
        // The elements in front of the first and behind the last vector, once, by block 0: after its report of the
        // first write phase and before its wait, where the round trip to memory costs nothing while other blocks still
        // write (at the end of the launch it would be the last thing the chip does, in front of a report it would hold
        // every block back).
        if (p0 == 0 && blockIdx.x == 0 && (head | tail)) reduce_multi_edges<TR, OP>(src, n, dst, m, head, nvec, tail);
        if (more) phase_wait(ps, ++gen, give_up, spin_ticks);
    }
    if (nvec == 0 && blockIdx.x == 0 && (head | tail)) reduce_multi_edges<TR, OP>(src, n, dst, m, head, nvec, tail);   // no phase at all
}

// ---------------------------------------------------------------------------------------------------
// host-side launch

inline int grid_for(uint64_t ntiles, const Tuning& t) {
    uint64_t g = (uint64_t)t.num_cus * (uint64_t)(t.waves_per_cu > 0 ? t.waves_per_cu : 8);
    if (t.max_blocks > 0 && g > (uint64_t)t.max_blocks) g = (uint64_t)t.max_blocks;
    if (t.xcd_chunked) g = (g + 7) & ~7ull;
    if (g > ntiles) g = ntiles;
    if (t.xcd_chunked && g >= 8) g &= ~7ull;
    return g ? (int)g : 1;
}

template <class TR, int OP, int N, int UNROLL>
inline hipError_t launch_fixed(const LaunchArgs& a, const VecSplit& v) {
    SrcFixed<N> s;
    for (int j = 0; j < N; j++) s.p[j] = a.srcs[j];
    const uint64_t tile = (uint64_t)kBlock * UNROLL;
    int grid = grid_for((v.nvec + tile - 1) / tile, a.tune);
    g_last_kernel = "reduce_vec_kernel";
    g_realigned_launches += v.beyond;
    hipLaunchKernelGGL((reduce_vec_kernel<TR, OP, N, UNROLL>), dim3(grid), dim3(kBlock), 0, a.stream, s, a.dst,
                       v.head, v.nvec, v.tail, a.tune.xcd_chunked, v.beyond);
    return hipGetLastError();
}

// Traits classes whose unroll depth can be switched at run time (Tuning::variant = 1, 2 or 4); for the
// others only the default depth is compiled.
template <class TR>
struct HasUnrollVariants {
    static constexpr bool value = false;
};

// Vectors per lane per tile of the streaming kernel (N x this many 128-bit loads are in flight per lane).  Four
// measures 3-7 % above two for every type at 5-8 inputs; a traits class with heavy per-element arithmetic
// specialises this before its kernels are instantiated.
template <class TR>
struct StreamUnroll {
    static constexpr int get(int) { return 4; }
};

template <class TR, int OP, int N>
inline hipError_t launch_fixed_unroll(const LaunchArgs& a, const VecSplit& v) {
    constexpr int kDefault = StreamUnroll<TR>::get(N);
    if constexpr (HasUnrollVariants<TR>::value) {
        switch (a.tune.variant) {
            case 1: return launch_fixed<TR, OP, N, 1>(a, v);
            case 2: return launch_fixed<TR, OP, N, 2>(a, v);
            case 4: return launch_fixed<TR, OP, N, 4>(a, v);
            default: break;
        }
    }
    return launch_fixed<TR, OP, N, kDefault>(a, v);
}

// One buffer to m >= 2: the sectioned broadcast kernel re-reads every section from the L2s and keeps every destination an
// ascending stream, 6.3-6.5 TB/s at any size; the phased form with the clock pacing its write phase reaches 6.7 (m = 2) to
// 7.0 (m = 7) from 256 MiB per buffer, equals it at 128 MiB and loses below (one partly filled phase: 5.5-5.9 at 64 MiB).
inline bool broadcast_wants_phased(const Tuning& t, uint64_t bytes) {
    if (t.sync == nullptr || t.num_cus < kPhaseGroups || t.max_blocks > 0 || t.variant != 0 || t.write_pace <= 0) return false;
    const uint64_t grid = (uint64_t)(t.num_cus / kPhaseGroups) * kPhaseGroups;
    const uint64_t per_phase = grid * kPhaseBlock * (uint64_t)(4 * MultiPhaseRegs<U8Traits>::groups + kPhaseU) * 16u;
    return bytes >= 2 * per_phase;
}

// When the phased form pays: from Tuning::phased_min_bytes of traffic per launch (default 160 MB), with two or more
// inputs and one destination when its phases are full enough (phases_full_enough: long buffers always are: +8 % with
// 2 inputs, +17 % with 8 at 4 GiB of traffic), with several destinations from twice that traffic.  One input stays with
// the copy and broadcast kernels, except that a buffer of two phases or more going to several destinations takes the
// phased form with its paced write phase (broadcast_wants_phased).  Tuning::variant 8 forces the phased form.
inline uint64_t phase_lanes(const Tuning& t) {       // lanes of a phased launch: one block of kPhaseBlock on every CU
    return (uint64_t)(t.num_cus / kPhaseGroups) * kPhaseGroups * kPhaseBlock;
}
inline bool wants_phased(const LaunchArgs& a, uint64_t nvec, int reg_groups) {
    if (a.tune.sync == nullptr || a.tune.num_cus < kPhaseGroups) return false;
    if (a.tune.variant != 0) return a.tune.variant == 8;
    if (a.tune.max_blocks > 0) return false;        // a caller that caps the grid keeps CUs free: the phased form takes them all
    const uint64_t traffic = (uint64_t)(a.n + a.m) * nvec * 16u;
    if (a.n < 2) return a.m > 1 && broadcast_wants_phased(a.tune, nvec * 16u);    // one input that is not a plain copy (bf16 keep-precision narrows it)
    if (traffic < (uint64_t)a.tune.phased_min_bytes * (a.m > 1 ? 2u : 1u)) return false;
    if (a.m > 1) return true;
    // Five or more inputs meet a stronger streaming kernel (reduce_multi_kernel, which takes the inputs one after the
    // other: 6.15-6.4 TB/s from 64 MB of traffic on): the phased form passes it at about 300 MB of traffic -- 8 inputs of
    // 24 / 28 / 32 / 40 MiB: 5.83 / 5.82 / 6.17 / 6.38 against 6.2; 12 inputs of 16 / 20 / 24 / 32 MiB: 5.79 / 5.76 / 6.25 / 6.47
    // against 6.41 / 6.35 / 6.27 / 6.18; 6 inputs of 32 / 40 / 48 MiB: 5.89 / 6.13 / 6.30 against 6.2.
    if (a.n >= 5 && traffic < (uint64_t)a.tune.phased_min_bytes / 8 * 15) return false;
    const uint64_t grid = (uint64_t)(a.tune.num_cus / kPhaseGroups) * kPhaseGroups;
    return phases_full_enough(nvec, grid * kPhaseBlock * (uint64_t)(4 * reg_groups + kPhaseU), a.n);
}

// Elements before the first vector: the vectors start on the 16-byte boundary that makes the loose accesses of the
// buffers that disagree with it cheapest (vector_grid) and, for large calls, on the 128-byte line that suits the
// buffers on that boundary best (vector_start).  No head when that boundary is not a multiple of the element size.
constexpr size_t kLineStartBytes = 1u << 20;
template <class E>
inline uint64_t vector_head(const LaunchArgs& a) {
    unsigned in_mis[kMaxSrcs], out_mis[kMaxDsts], in_line[kMaxSrcs], out_line[kMaxDsts];
    for (int j = 0; j < a.n; j++) {
        in_line[j] = (unsigned)((uintptr_t)a.srcs[j] & (kLineBytes - 1));
        in_mis[j] = in_line[j] & 15u;
    }
    for (int k = 0; k < a.m; k++) {
        out_line[k] = (unsigned)((uintptr_t)(a.dsts ? a.dsts[k] : a.dst) & (kLineBytes - 1));
        out_mis[k] = out_line[k] & 15u;
    }
    const unsigned mis = vector_grid(in_mis, a.n, out_mis, a.m, sizeof(E) < 4 && a.tune.realign);
    if (mis % sizeof(E)) return 0;
    // below kLineStartBytes per buffer a call is latency-bound and the head stays as short as it can be
    const bool lines = a.tune.line_start && a.count * sizeof(E) >= kLineStartBytes;
    return vector_start(in_line, a.n, out_line, a.m, mis, lines) / sizeof(E);
}

// How the elements of a call are divided: `head` elements, `nvec` vectors, `tail` elements.  When an input's vectors
// start off a 4-byte boundary (16- and 8-bit types only) and Tuning::realign is on, the last whole vector goes to the
// tail (beyond = 1): the kernels may then read vector nvec, which the realignment in registers needs (load_vectors).
template <class E, uint32_t VEC>
inline VecSplit vector_split(const LaunchArgs& a) {
    VecSplit v;
    uint64_t head = vector_head<E>(a);
    if (head > a.count) head = a.count;
    v.head = (uint32_t)head;
    v.nvec = (a.count - head) / VEC;
    v.tail = (uint32_t)(a.count - head - v.nvec * VEC);
    v.beyond = 0;
    if (sizeof(E) < 4 && a.tune.realign && v.nvec > 0) {
        for (int j = 0; j < a.n; j++)
            if (((uintptr_t)a.srcs[j] + head * sizeof(E)) & 3u) v.beyond = 1;
        if (v.beyond) {
            v.nvec -= 1;
            v.tail += VEC;
        }
    }
    return v;
}

template <class TR, int OP>
inline hipError_t launch_multi_op(const LaunchArgs& a) {
    typedef typename TR::elem_t E;
    SrcTable s;
    DstTable d;
    for (int j = 0; j < a.n; j++) s.p[j] = a.srcs[j];
    for (int k = 0; k < a.m; k++) d.p[k] = a.dsts ? a.dsts[k] : a.dst;
    const VecSplit v = vector_split<E, TR::VEC>(a);
    g_realigned_launches += v.beyond;
    const int reg_groups = phase_reg_groups(v.nvec, phase_lanes(a.tune), MultiPhaseRegs<TR>::groups, kPhaseU);
    if (wants_phased(a, v.nvec, reg_groups)) {
        int grid = (a.tune.num_cus / kPhaseGroups) * kPhaseGroups;
        // does any buffer's first vector start off a 128-byte line?
        uint32_t off_lines = 0;
        for (int j = 0; j < a.n; j++) off_lines |= (uint32_t)((uintptr_t)s.p[j] + v.head * sizeof(E)) & (kLineBytes - 1);
        for (int k = 0; k < a.m; k++) off_lines |= (uint32_t)((uintptr_t)d.p[k] + v.head * sizeof(E)) & (kLineBytes - 1);
        // (with several destinations the write phase, which wants the chip's stores in one compact window, loses more
        // to the runs than the reads gain: 8 -> 8 at 1 GiB 6.28 against 6.46 TB/s)
        const uint32_t wave_runs = a.tune.wave_runs == 2 || (a.tune.wave_runs == 1 && off_lines && a.m == 1);
        // the write phase's pace (see the kernel): 1/16 clock ticks per group of four stores of the whole grid
        uint32_t write_pace16 = 0;
        // Several destinations at the pace itself; one destination a tenth faster (its write phase is short) while the
        // inputs are few enough for the type (PhasePacedInputs).
        const double rate = a.m >= 2                              ? (double)a.tune.write_pace
                            : a.n <= PhasePacedInputs<TR, OP>::value ? 1.1 * (double)a.tune.write_pace
                                                                      : 0.0;
        write_pace16 = write_pace_ticks16((uint64_t)grid * kPhaseBlock * 16u * 4u, rate, a.tune.wall_khz);
        g_last_kernel = "reduce_multi_phased_kernel";
        constexpr int kUsual = MultiPhaseRegs<TR>::groups;
        g_wide_phase_launches += reg_groups > kUsual;
        const auto kernel = reg_groups > kUsual ? reduce_multi_phased_kernel<TR, OP, kUsual + 1> : reduce_multi_phased_kernel<TR, OP, kUsual>;
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(kPhaseBlock), 0, a.stream, s, a.n, d,
                           a.m, v.head, v.nvec, v.tail, a.tune.sync, phase_early_loads<TR, OP>(a.tune, a.n, write_pace16 != 0),
                           phase_early_stores<TR>(a.tune, a.m),
                           a.tune.spin_ticks, v.beyond, wave_runs, write_pace16);
        return hipGetLastError();
    }
    constexpr int UNROLL = 4;
    const uint64_t tile = (uint64_t)kBlock * UNROLL;
    int grid = grid_for((v.nvec + tile - 1) / tile, a.tune);
    g_last_kernel = "reduce_multi_kernel";
    hipLaunchKernelGGL((reduce_multi_kernel<TR, OP, UNROLL>), dim3(grid), dim3(kBlock), 0, a.stream, s, a.n, d, a.m,
                       v.head, v.nvec, v.tail, a.tune.xcd_chunked, v.beyond);
    return hipGetLastError();
}

template <class TR, int OP>
inline hipError_t launch_op(const LaunchArgs& a) {
    typedef typename TR::elem_t E;
    if (a.m > 1 || a.n > kMaxFixedN) return launch_multi_op<TR, OP>(a);     // run-time counts of inputs and outputs
    const VecSplit v = vector_split<E, TR::VEC>(a);
    if (wants_phased(a, v.nvec, phase_reg_groups(v.nvec, phase_lanes(a.tune), MultiPhaseRegs<TR>::groups, kPhaseU)))
        return launch_multi_op<TR, OP>(a);          // the phased kernel takes any number of inputs
    // five or more inputs in the range between latency-bound and phased (64 to 315 MB of traffic): taking the inputs
    // one after the other, as the run-time-count streaming kernel does, measures 5-12 % above loading them together
    if (a.n >= 5 && a.tune.variant == 0 && (uint64_t)(a.n + 1) * v.nvec * 16u >= (uint64_t)a.tune.phased_min_bytes / 5 * 2)
        return launch_multi_op<TR, OP>(a);
    switch (a.n) {
        case 1: return launch_fixed_unroll<TR, OP, 1>(a, v);
        case 2: return launch_fixed_unroll<TR, OP, 2>(a, v);
        case 3: return launch_fixed_unroll<TR, OP, 3>(a, v);
        case 4: return launch_fixed_unroll<TR, OP, 4>(a, v);
        case 5: return launch_fixed_unroll<TR, OP, 5>(a, v);
        case 6: return launch_fixed_unroll<TR, OP, 6>(a, v);
        case 7: return launch_fixed_unroll<TR, OP, 7>(a, v);
        case 8: return launch_fixed_unroll<TR, OP, 8>(a, v);
        default: return hipErrorInvalidValue;
    }
}

// One instantiation of this per traits class lives in its own translation unit.
template <class TR>
hipError_t launch_reduce(const LaunchArgs& a) {
    switch (a.op) {
        case OP_SUM: return launch_op<TR, OP_SUM>(a);
        case OP_PROD: return launch_op<TR, OP_PROD>(a);
        case OP_MIN: return launch_op<TR, OP_MIN>(a);
        case OP_MAX: return launch_op<TR, OP_MAX>(a);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace mi
