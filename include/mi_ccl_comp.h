/*
 * mi_ccl_comp.h -- C ABI of the MI355X reduction engine (libmi_ccl_comp.so).
 *
 * Drop-in boundary for oneCCL's data-parallel reduction path.  oneCCL has no public plugin ABI for
 * reductions; its boundary is the internal operator surface of src/comp/comp.hpp:23-51 plus the
 * device-kernel launch sites under src/sched/entry/ze/.  Every entry point below names the reference
 * interface it replaces.
 *
 * Conventions
 *   - All buffer arguments are DEVICE pointers (HIP device memory); the library never dereferences
 *     them on the host, never allocates or frees device memory in a reduce/copy/convert call, and keeps
 *     no pointer after the call returns (fusion plans own one small device table, allocated at plan
 *     creation).  Pointers must be aligned to the element size.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Calls are asynchronous:
 *     they enqueue kernels on `stream` and return.
 *   - dtype / op use the numbering of ccl::datatype / ccl::reduction
 *     (include/oneapi/ccl/types.hpp:41-69).
 *   - Return value: a ccl::status number (src/internal_types.hpp:29-37): 0 success, 1 out_of_resource,
 *     2 invalid_arguments, 3 runtime_error.  Nothing here throws or terminates the process; count == 0
 *     succeeds without touching any pointer (comp.cpp:132-134, :61-63).
 *   - Results are bit-identical to the reference CPU reduction on the same inputs (integers wrap;
 *     one IEEE operation per pair in input order, no FMA; min/max return the same operand as the
 *     reference on ties and NaNs).  NaN results of sum and prod are the x86 ones too: a NaN operand comes back with
 *     its quiet bit set, an invalid operation (Inf - Inf, 0 x Inf) gives the negative default NaN; only when both
 *     operands of a step are NaNs is it unspecified which of the two comes back (in the reference that depends on
 *     the operand order its compiler chose).
 */
#ifndef MI_CCL_COMP_H
#define MI_CCL_COMP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ccl::datatype, include/oneapi/ccl/types.hpp:52-69 */
enum mi_ccl_datatype {
    MI_CCL_INT8 = 0, MI_CCL_UINT8, MI_CCL_INT16, MI_CCL_UINT16, MI_CCL_INT32, MI_CCL_UINT32,
    MI_CCL_INT64, MI_CCL_UINT64, MI_CCL_FLOAT16 = 8, MI_CCL_FLOAT32, MI_CCL_FLOAT64, MI_CCL_BFLOAT16 = 11,
    MI_CCL_DATATYPE_LAST
};

/* ccl::reduction, include/oneapi/ccl/types.hpp:41-47 (custom is handled above this ABI, on the host) */
enum mi_ccl_reduction { MI_CCL_SUM = 0, MI_CCL_PROD, MI_CCL_MIN, MI_CCL_MAX, MI_CCL_CUSTOM };

/* ccl::status, src/internal_types.hpp:29-37 */
enum mi_ccl_status {
    MI_CCL_SUCCESS = 0, MI_CCL_OUT_OF_RESOURCE = 1, MI_CCL_INVALID_ARGUMENTS = 2, MI_CCL_RUNTIME_ERROR = 3
};

/* ccl_bf16_impl_type, src/comp/bf16/bf16_utils.hpp:26 -- which of the reference's three bf16
 * implementations the results must equal (the reference picks one through CCL_BF16, env.cpp:711-713):
 *   scalar   narrow by truncation, min/max with std:: semantics (ties/NaN return `in`)
 *   avx512f  narrow by truncation, min/max return `inout` on ties/NaN
 *   avx512bf narrow with round-to-nearest-even, fp32 denormals to zero, NaN quieted (VCVTNEPS2BF16);
 *            min/max as avx512f */
enum mi_ccl_bf16_impl { MI_CCL_BF16_SCALAR = 0, MI_CCL_BF16_AVX512F = 1, MI_CCL_BF16_AVX512BF = 2 };

/* ccl_fp16_impl_type, src/comp/fp16/fp16_utils.hpp:26-32 (CCL_FP16, env.cpp:715-720).  f16c and avx512f work
 * through fp32 and give the same bits; avx512fp16 works on the fp16 values (fp16_intrisics.cpp:24-35): same bits
 * for sum and prod, and min/max return the chosen operand untouched where the other two quiet a signalling NaN.
 * Every reduce entry point takes the choice as its fp16_impl argument (ignored for other dtypes); MI_CCL_FP16_DEFAULT
 * there means the process-wide default, mi_ccl_set_param("fp16_impl", value), which starts as avx512f. */
enum mi_ccl_fp16_impl { MI_CCL_FP16_DEFAULT = 0, MI_CCL_FP16_F16C = 2, MI_CCL_FP16_AVX512F = 3, MI_CCL_FP16_AVX512FP16 = 4 };

/* How 16-bit floating types are carried through an N-input reduce (flags, OR them):
 *   MI_CCL_LP_PAIRWISE        round to the 16-bit type after every pair: a chain of ccl_comp_reduce calls
 *                             (comp.cpp:236-245; the only mode the reference has for float16)
 *   MI_CCL_LP_KEEP_PRECISION  bfloat16 only: widen, accumulate in fp32 in input order, narrow once
 *                             (ccl_comp_batch_reduce with bf16_keep_precision_mode = 1, comp.cpp:214-234)
 *   MI_CCL_LP_TAIL_QUIRK      with KEEP_PRECISION under avx512f/avx512bf: narrow the last count % 16 elements
 *                             by truncation, as ccl_convert_fp32_to_bf16_arrays does (bf16.cpp:134-148) */
enum mi_ccl_lp_mode { MI_CCL_LP_PAIRWISE = 0, MI_CCL_LP_KEEP_PRECISION = 1, MI_CCL_LP_TAIL_QUIRK = 2 };

/* ---- tables ------------------------------------------------------------------------------------ */

/* Element size in bytes, 0 for an unknown dtype.  Replaces ccl_datatype::size(), datatype.cpp:79-91. */
size_t mi_ccl_datatype_size(int dtype);
/* "int8" ... "bfloat16", "" for an unknown dtype.  Replaces the name table of datatype.cpp:94-106. */
const char* mi_ccl_datatype_name(int dtype);
/* "sum", "prod", "min", "max", "custom", "unknown".  Replaces ccl_reduction_to_str, comp.cpp:251-260. */
const char* mi_ccl_reduction_to_str(int op);
/* Text for a status code. */
const char* mi_ccl_status_str(int status);
/* Name the reference gives the matching device kernel: "<kernel>_<dtype-name>_<op>"
 * (ze_primitives.cpp:152-161); written into buf (NUL terminated), returns the status. */
int mi_ccl_kernel_name(const char* kernel, int dtype, int op, char* buf, size_t buf_len);

/* ---- pairwise, in place ------------------------------------------------------------------------- */

/* inout[i] = inout[i] OP in[i] for i < count.  Replaces ccl_comp_reduce / ccl_comp_reduce_regular
 * (src/comp/comp.cpp:76-200) and reduce_local_inplace_kernel (src/kernels/kernels.cl:236-246,
 * launched from ze_reduce_local_entry.cpp:40-58).  in and inout must be identical or disjoint. */
int mi_ccl_comp_reduce(int dtype, int op, const void* in, size_t count, void* inout, int bf16_impl,
                       int fp16_impl, void* stream);

/* Replaces ccl_bf16_reduce (src/comp/bf16/bf16.cpp:87-110) and ccl_fp16_reduce
 * (src/comp/fp16/fp16.cpp:41-53). */
int mi_ccl_bf16_reduce(const void* in, size_t count, void* inout, int op, int bf16_impl, void* stream);
int mi_ccl_fp16_reduce(const void* in, size_t count, void* inout, int op, int fp16_impl, void* stream);

/* ---- N inputs ----------------------------------------------------------------------------------- */

/* dst[i] = (((srcs[0][i] OP srcs[1][i]) OP srcs[2][i]) ... OP srcs[n-1][i]): own buffer first, peers in
 * argument order, one pass over memory.  srcs is a HOST array of n device pointers (1 <= n <= 64).
 * dst may equal any srcs[j].  Replaces reduce_monolithic_kernel_{1..7}, local_reduce_kernel_{1..7},
 * reduce_single_local_inplace_kernel and reduce_local_outofplace_kernel (src/kernels/kernels.cl:179-421;
 * launch sites ze_a2a_reduce_scatter_entry.cpp:48-136, ze_a2a_pipeline_reduce_scatter_entry.cpp:195-228)
 * and, with slice pointers, ccl_comp_batch_reduce (src/comp/comp.cpp:202-249). */
int mi_ccl_comp_reduce_n(int dtype, int op, const void* const* srcs, int n, void* dst, size_t count,
                         int lp_mode, int bf16_impl, int fp16_impl, void* stream);

/* The same reduce with the result stored to each of m buffers (1 <= m <= 16) in one pass: (n + m) x bytes of
 * memory traffic instead of (n + 1 + 2(m - 1)) x bytes for a reduce followed by m - 1 copies.  dsts is a HOST
 * array of m device pointers; a destination may be one of the sources.  Replaces allreduce_kernel
 * (src/kernels/kernels.cl:190-217, launched from ze_onesided_allreduce_entry.cpp:66-108: n = 2, m = 2) and, with
 * n == 1 and MI_CCL_LP_PAIRWISE (a byte copy for every dtype), write_monolithic_kernel_{1..7}
 * (src/kernels/kernels.cl:423-560, launched from ze_a2a_allgatherv_entry.cpp:526-585: m = peer count). */
int mi_ccl_comp_reduce_write_n(int dtype, int op, const void* const* srcs, int n, void* const* dsts, int m,
                               size_t count, int lp_mode, int bf16_impl, int fp16_impl, void* stream);

/* n_jobs independent reduces of one dtype and operation in ONE launch: for job j and i < counts[j],
 * dsts[j][i] = srcs[j * n + 0][i] OP srcs[j * n + 1][i] OP ... OP srcs[j * n + n - 1][i] (1 <= n <= 8, the same for every
 * job).  srcs (n_jobs x n pointers, job after job), dsts and counts are HOST arrays; a job's output may be one of its
 * own inputs, the jobs must not overlap one another; a job with count 0 is skipped without looking at its pointers.
 * The job table travels in the kernel arguments (96 jobs or 320 pointers (inputs and outputs) per launch, more jobs take
 * more launches): nothing is allocated, on the host or on the device.  Every job's arguments are checked before the
 * first launch, so an argument error leaves every output as it was.  Replaces read_reduce_write (n = 2: even[i] = pair[i]
 * + local[i] for every peer i in one kernel, src/coll/algorithms/reduce_scatter/sycl/reduce_scatter_large_sycl_impl.hpp:22-66),
 * reduce_read_write_kernel_{1..7} (src/kernels/kernels.cl:156-177) and, with n = 1, copy_data (N copies in one kernel,
 * used at :216-224 of the same file); it is also the small-message path: 64 reduces of a few KiB cost one launch, not
 * 64.  The jobs of a launch that together fill whole phases (from "phased_min_bytes" = 160 MB of traffic, two or more
 * inputs: the chunks a large reduce-scatter stages) run in the phased kernel form, all jobs in one launch; with one
 * input per job, a job of 32 MiB or more is a launch of the copy kernel.  lp_mode: MI_CCL_LP_PAIRWISE or
 * MI_CCL_LP_KEEP_PRECISION (bfloat16). */
int mi_ccl_comp_reduce_batch(int dtype, int op, const void* const* srcs, int n, void* const* dsts,
                             const size_t* counts, int n_jobs, int lp_mode, int bf16_impl, int fp16_impl,
                             void* stream);

/* Slice form of the same: slice i starts at in_buf + offsets[i] elements (offsets: HOST array); inout is
 * slice 0 and receives the result.  Replaces ccl_comp_batch_reduce (src/comp/comp.cpp:202-249); the tmp and
 * acc scratch arrays of the reference are not needed.  keep_precision != 0 requires dtype bfloat16 and
 * reproduces the reference bit for bit, including the truncated tail (MI_CCL_LP_TAIL_QUIRK). */
int mi_ccl_comp_batch_reduce(const void* in_buf, const size_t* offsets, size_t n_offsets, size_t count,
                             void* inout, int dtype, int op, int bf16_keep_precision_mode, int bf16_impl,
                             int fp16_impl, void* stream);

/* ---- copies and converters ---------------------------------------------------------------------- */

/* out[0..bytes) = in[0..bytes).  Replaces ccl_comp_copy (src/comp/comp.cpp:60-74) and the copy_entry body
 * (src/sched/entry/copy/copy_entry.cpp:201-207).  use_nontemporal selects streaming stores, as
 * ccl::memcpy_nontemporal does (src/common/utils/memcpy.cpp:49-). */
int mi_ccl_comp_copy(const void* in, void* out, size_t bytes, int use_nontemporal, void* stream);

/* Replace ccl_convert_fp32_to_bf16_arrays / ccl_convert_bf16_to_fp32_arrays (bf16.cpp:130-169), tail
 * truncation included. */
int mi_ccl_convert_fp32_to_bf16_arrays(const void* fp32_buf, void* bf16_buf, size_t count, int bf16_impl,
                                       void* stream);
int mi_ccl_convert_bf16_to_fp32_arrays(const void* bf16_buf, void* fp32_buf, size_t count, void* stream);

/* The reference's fp16 converters, ccl_convert_fp32_to_fp16 / ccl_convert_fp16_to_fp32 (src/comp/fp16/fp16.cpp:55-61),
 * convert one vector of eight values (VCVTPS2PH round-to-nearest-even / VCVTPH2PS); these convert count values with
 * the same result per value (subnormals kept, overflow to infinity, a signalling NaN quieted keeping the top of its
 * payload).  The single-vector ccl_convert_fp32_to_bf16 / ccl_convert_bf16_to_fp32 (bf16.cpp:113-127) are the bf16
 * array converters above with count = 16. */
int mi_ccl_convert_fp32_to_fp16_arrays(const void* fp32_buf, void* fp16_buf, size_t count, void* stream);
int mi_ccl_convert_fp16_to_fp32_arrays(const void* fp16_buf, void* fp32_buf, size_t count, void* stream);

/* ---- fusion buffer ------------------------------------------------------------------------------ */

/* Byte offset of each of k tensors in a fusion buffer: running offset in queue order, every start
 * rounded up to `align` bytes (align = 1 is the reference's tight layout, fusion.cpp:283-316).  Host
 * arithmetic only.  *total_bytes = end of the last tensor. */
int mi_ccl_fusion_offsets(const size_t* counts, size_t k, size_t dtype_size, size_t align,
                          size_t* byte_offsets, size_t* total_bytes);

typedef struct mi_ccl_fusion_plan mi_ccl_fusion_plan;

/* A plan fixes (counts, dtype, alignment) of one fused group -- what ccl_fusion_manager::build_sched
 * derives from its exec_queue (fusion.cpp:145-376) and caches with the fused sched (:206-237).  Creating a
 * plan allocates its device-side work table once; destroy frees it. */
int mi_ccl_fusion_plan_create(const size_t* counts, size_t k, int dtype, size_t align,
                              mi_ccl_fusion_plan** plan);
int mi_ccl_fusion_plan_destroy(mi_ccl_fusion_plan* plan);
size_t mi_ccl_fusion_plan_bytes(const mi_ccl_fusion_plan* plan);            /* fused buffer size */
size_t mi_ccl_fusion_plan_offset(const mi_ccl_fusion_plan* plan, size_t i); /* byte offset of tensor i */

/* tensors: HOST array of k device pointers.  pack copies every tensor to its offset in fusion_buf in one
 * launch (replaces the pack copy_entry list, fusion.cpp:283-316); unpack copies them back (replaces
 * fusion.cpp:323-362).  Padding bytes between tensors are not written by pack. */
int mi_ccl_fusion_pack(mi_ccl_fusion_plan* plan, const void* const* tensors, void* fusion_buf, void* stream);
int mi_ccl_fusion_unpack(mi_ccl_fusion_plan* plan, const void* fusion_buf, void* const* tensors,
                         void* stream);

/* The whole pack -> N-input reduce -> unpack sequence in one pass over memory:
 * out_tensors[t][i] = own_tensors[t][i] OP peers[0][off_t + i] OP ... OP peers[n_peers-1][off_t + i],
 * where every peer is a fusion buffer with this plan's layout.  Same bits as the three-step sequence. */
int mi_ccl_fusion_reduce(mi_ccl_fusion_plan* plan, int op, const void* const* own_tensors,
                         const void* const* peers, int n_peers, void* const* out_tensors, int lp_mode,
                         int bf16_impl, int fp16_impl, void* stream);

/* The same fused reduce for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): no plan, and no hipMalloc, hipFree or other allocating call -- the work
 * table that a plan keeps in memory of its own lives in an array inside the library (four tables of about 1 MiB per
 * GPU, held until the process ends); a call takes the next table in turn and a small kernel on `stream` rewrites it in
 * front of the reduce.  The layout is given directly: counts[k] elements of `dtype`, starts rounded up to `align` bytes
 * (as mi_ccl_fusion_offsets).  Same results as mi_ccl_fusion_reduce on a plan of the same layout.  Limits:
 * k <= MI_CCL_FUSION_STATIC_MAX_TENSORS and at most MI_CCL_FUSION_STATIC_MAX_ITEMS pieces of 16 KiB (a tensor takes
 * ceil(bytes / 16384) of them: 2 GiB of payload when the tensors are multiples of 16 KiB); beyond either the call returns
 * out_of_resource and does nothing.  Calls on the same stream are ordered.  A table comes round again with the fourth
 * call after it on that GPU: up to four calls may overlap on different streams (or sit in graphs that replay side by
 * side); a call that is still running when the fourth call after it starts races with it (results undefined) -- keep
 * at most four in flight per GPU, or order them on one stream; a call captured into a graph keeps, in every replay,
 * the table it took at capture, so order a graph's replays with whatever else may reach that table.  The first call on a GPU looks the array's address up;
 * make that call outside a capture.  This entry point has no counterpart in the reference. */
#define MI_CCL_FUSION_STATIC_MAX_TENSORS 1024
#define MI_CCL_FUSION_STATIC_MAX_ITEMS 131072
int mi_ccl_fusion_reduce_static(const size_t* counts, size_t k, int dtype, size_t align, int op,
                                const void* const* own_tensors, const void* const* peers, int n_peers,
                                void* const* out_tensors, int lp_mode, int bf16_impl, int fp16_impl, void* stream);

/* ---- measurement aid ------------------------------------------------------------------------------ */

/* Read-only and write-only streams in the access shapes of the kernels above, for putting a measured ceiling of the
 * memory system beside a kernel's figure (no counterpart in the reference).  bytes: per buffer, a multiple of 16;
 * buffers 16-byte aligned.  MI_CCL_PROBE_READ reads n buffers and writes nothing; MI_CCL_PROBE_WRITE_ONE /
 * MI_CCL_PROBE_WRITE_FOUR overwrite bufs[0] (n = 1) with one / four 16-byte stores per lane. */
enum mi_ccl_probe_kind { MI_CCL_PROBE_READ = 0, MI_CCL_PROBE_WRITE_ONE = 1, MI_CCL_PROBE_WRITE_FOUR = 2 };
int mi_ccl_probe_bandwidth(int kind, void* const* bufs, int n, size_t bytes, void* stream);

/* Name of the kernel template that the calling thread's most recent reduce / copy / fusion / probe call launched
 * ("reduce_multi_phased_kernel", "reduce_vec_kernel", "copy_kernel", ...; "" before the first call), so that a
 * measurement can say which kernel it belongs to.  No counterpart in the reference. */
const char* mi_ccl_last_kernel(void);

/* ---- launch tuning ------------------------------------------------------------------------------- */

/* Launch-shape knobs, the counterpart of CCL_KERNEL_GROUP_SIZE / CCL_KERNEL_MEM_ALIGN
 * (src/common/env/env.cpp:251-253).  Names: "waves_per_cu" (blocks per CU the streaming kernels' grid is capped
 * at; default 256, i.e. one tile per block up to 65,536 blocks), "max_blocks" (cap on the grid of the streaming kernels, for callers that want CUs left free for other work; 0 = no
 * cap; while a cap is set the phased kernels, which take one block on every CU, are not chosen), "xcd_chunked" (0/1: give each of the 8 XCDs one
 * contiguous share of the buffer), "variant" (kernel form: 0 = chosen by size and shape; 1, 2, 4 = the streaming
 * kernels with that many vectors per lane where a type has them; 8 = the phased kernels at any size; a non-zero value
 * also keeps one-input calls on the general reduce kernels instead of the copy and broadcast kernels -- for tests and
 * measurements),
 * "phased_min_bytes" (scales the sizes from which the phased kernels are used; default 160 MB),
 * "phase_early_loads" / "phase_early_stores" (phased kernels: how many 16-byte loads / stores per lane a block still
 * has to issue when it reports the end of its read / write phase to the chip-wide barrier, which hides the barrier's
 * latency; defaults -1 = 12 loads, or 2 to 8 behind a paced write phase depending on the element type and the number
 * of inputs, and -1 = 16 stores, or 20 with several destinations while the write phase is paced; 0 = report
 * when the whole block is done and its stores are acknowledged; timing only, results do not
 * depend on them), "phase_spin_ticks" (phased kernels: the longest a block waits at one barrier, in 100 MHz ticks,
 * before it goes on alone and stops waiting for the rest of the launch; default 20000 = 200 us; 0 = never wait, which
 * costs speed only and is what the tests of that path use), "num_cus" (read
 * only), "fp16_impl" (what MI_CCL_FP16_DEFAULT stands for: 2, 3 or 4 of enum mi_ccl_fp16_impl above), and
 * "launch_block_limit" (blocks per launch of the copy, broadcast and converter kernels, which cut larger work into
 * several launches; 0 = what HIP allows, 2^24 - 1; smaller values let tests exercise the cutting), "realign" (0/1,
 * default 1: an input of a 16- or 8-bit type whose vectors start off a 4-byte boundary -- a peer's block behind an odd
 * number of elements, a tensor behind an odd-sized one in a tight fusion buffer -- is read on that boundary and shifted
 * into place in registers instead of with misaligned vector loads; same results, about a fifth faster for such
 * layouts), "realigned_launches" (read only: how many launches of the calling thread took that path),
 * "wide_phase_launches" (read only: how many phased reduces of the calling thread kept four more result vectors per
 * lane in registers, 96 instead of 88 MiB of results per phase on 256 CUs, because that took a whole phase off a launch
 * of at most six phases), "line_start"
 * (0/1, default 1: a reduce, copy or broadcast of 1 MiB or more per buffer starts its 16-byte vectors on a 128-byte
 * line of the buffers that matter most -- the outputs before the inputs -- so up to 127 bytes at the front are
 * handled element by element; buffers that share an offset from the lines then run like aligned ones, +6 %) and
 * "phase_write_pace" (phased reduce with two or more destinations, and, a tenth faster, with one destination and up
 * to 16 inputs -- 12 for the 8-bit types, bfloat16 and fp16 min / max -- batched jobs and the phased fused reduces
 * included, where it gains 1-6 %: the rate in GB/s at which the device clock lets
 * the write phase's stores out, which keeps the blocks of the chip in step and the addresses written at any moment in
 * one compact window; default 7300, 0 = unpaced, otherwise 100 to 100000; 8 inputs stored to 8 buffers of 1 GiB run at 6.95 TB/s paced and 6.4
 * unpaced; a block that is behind the schedule is never held, so a rate above what HBM takes only switches the
 * pacing off), "wall_clock_khz" (read only: the rate of that clock),
 * "wave_runs" (phased kernels: a wave's vectors of one step lie next to each other instead of a block apart, which
 * halves to quarters the lines two waves share; 0 never, 1 = default, when a buffer is off the 128-byte lines and
 * there is one destination, 2 always).  Neither changes a result.
 * Returns invalid_arguments for an unknown name or out-of-range value. */
int mi_ccl_set_param(const char* name, long value);
long mi_ccl_get_param(const char* name);

#ifdef __cplusplus
}
#endif
#endif /* MI_CCL_COMP_H */
