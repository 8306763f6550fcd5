"""ctypes binding of libmi_ccl_comp.so (C ABI: include/mi_ccl_comp.h).

Every function takes device tensors (or raw device pointers) and a HIP stream and enqueues the HIP kernels;
there is no CPU fallback: a missing library raises at load time.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("MI_CCL_COMP_LIB") or os.path.join(HERE, "libmi_ccl_comp.so")     # another build, for A/B runs

# ccl::datatype (include/oneapi/ccl/types.hpp:52-69)
INT8, UINT8, INT16, UINT16, INT32, UINT32, INT64, UINT64, FLOAT16, FLOAT32, FLOAT64, BFLOAT16 = range(12)
# ccl::reduction (types.hpp:41-47)
SUM, PROD, MIN, MAX, CUSTOM = range(5)
# ccl::status (src/internal_types.hpp:29-37)
SUCCESS, OUT_OF_RESOURCE, INVALID_ARGUMENTS, RUNTIME_ERROR = range(4)
# ccl_bf16_impl_type (src/comp/bf16/bf16_utils.hpp:26)
BF16_SCALAR, BF16_AVX512F, BF16_AVX512BF = 0, 1, 2
# ccl_fp16_impl_type (src/comp/fp16/fp16_utils.hpp:26-32); 0 = the process-wide default (set_param("fp16_impl"))
FP16_DEFAULT, FP16_F16C, FP16_AVX512F, FP16_AVX512FP16 = 0, 2, 3, 4
LP_PAIRWISE, LP_KEEP_PRECISION, LP_TAIL_QUIRK = 0, 1, 2

DTYPE_SIZE = [1, 1, 2, 2, 4, 4, 8, 8, 2, 4, 8, 2]

EXPORTS = [
    "mi_ccl_datatype_size", "mi_ccl_datatype_name", "mi_ccl_reduction_to_str", "mi_ccl_status_str",
    "mi_ccl_kernel_name", "mi_ccl_comp_reduce", "mi_ccl_bf16_reduce", "mi_ccl_fp16_reduce",
    "mi_ccl_comp_reduce_n", "mi_ccl_comp_reduce_write_n", "mi_ccl_comp_reduce_batch", "mi_ccl_comp_batch_reduce",
    "mi_ccl_comp_copy",
    "mi_ccl_convert_fp32_to_bf16_arrays", "mi_ccl_convert_bf16_to_fp32_arrays",
    "mi_ccl_convert_fp32_to_fp16_arrays", "mi_ccl_convert_fp16_to_fp32_arrays", "mi_ccl_fusion_offsets",
    "mi_ccl_fusion_plan_create", "mi_ccl_fusion_plan_destroy", "mi_ccl_fusion_plan_bytes",
    "mi_ccl_fusion_plan_offset", "mi_ccl_fusion_pack", "mi_ccl_fusion_unpack", "mi_ccl_fusion_reduce",
    "mi_ccl_fusion_reduce_static",
    "mi_ccl_probe_bandwidth", "mi_ccl_last_kernel", "mi_ccl_set_param", "mi_ccl_get_param",
]


class CclError(RuntimeError):
    def __init__(self, status, what):
        self.status = status
        super().__init__(f"{what}: {status_str(status)} ({status})")


_lib = None


def lib():
    """Load the HIP library; raises if it was not built (no fallback of any kind)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: build it with `make -C oneccl_amd/csrc` "
                           "(or __graft_entry__.build()); there is no CPU fallback")
    L = C.CDLL(LIB_PATH)
    vp, sz, i = C.c_void_p, C.c_size_t, C.c_int
    L.mi_ccl_datatype_size.restype = sz
    L.mi_ccl_datatype_size.argtypes = [i]
    for f in ("mi_ccl_datatype_name", "mi_ccl_reduction_to_str", "mi_ccl_status_str"):
        getattr(L, f).restype = C.c_char_p
        getattr(L, f).argtypes = [i]
    L.mi_ccl_kernel_name.argtypes = [C.c_char_p, i, i, C.c_char_p, sz]
    L.mi_ccl_comp_reduce.argtypes = [i, i, vp, sz, vp, i, i, vp]
    L.mi_ccl_bf16_reduce.argtypes = [vp, sz, vp, i, i, vp]
    L.mi_ccl_fp16_reduce.argtypes = [vp, sz, vp, i, i, vp]
    L.mi_ccl_comp_reduce_n.argtypes = [i, i, vp, i, vp, sz, i, i, i, vp]
    L.mi_ccl_comp_reduce_write_n.argtypes = [i, i, vp, i, vp, i, sz, i, i, i, vp]
    L.mi_ccl_comp_reduce_batch.argtypes = [i, i, vp, i, vp, vp, i, i, i, i, vp]
    L.mi_ccl_comp_batch_reduce.argtypes = [vp, vp, sz, sz, vp, i, i, i, i, i, vp]
    L.mi_ccl_comp_copy.argtypes = [vp, vp, sz, i, vp]
    L.mi_ccl_convert_fp32_to_bf16_arrays.argtypes = [vp, vp, sz, i, vp]
    L.mi_ccl_convert_bf16_to_fp32_arrays.argtypes = [vp, vp, sz, vp]
    L.mi_ccl_convert_fp32_to_fp16_arrays.argtypes = [vp, vp, sz, vp]
    L.mi_ccl_convert_fp16_to_fp32_arrays.argtypes = [vp, vp, sz, vp]
    L.mi_ccl_fusion_offsets.argtypes = [vp, sz, sz, sz, vp, vp]
    L.mi_ccl_fusion_plan_create.argtypes = [vp, sz, i, sz, C.POINTER(vp)]
    L.mi_ccl_fusion_plan_destroy.argtypes = [vp]
    L.mi_ccl_fusion_plan_bytes.restype = sz
    L.mi_ccl_fusion_plan_bytes.argtypes = [vp]
    L.mi_ccl_fusion_plan_offset.restype = sz
    L.mi_ccl_fusion_plan_offset.argtypes = [vp, sz]
    L.mi_ccl_fusion_pack.argtypes = [vp, vp, vp, vp]
    L.mi_ccl_fusion_unpack.argtypes = [vp, vp, vp, vp]
    L.mi_ccl_fusion_reduce.argtypes = [vp, i, vp, vp, i, vp, i, i, i, vp]
    L.mi_ccl_fusion_reduce_static.argtypes = [vp, sz, i, sz, i, vp, vp, i, vp, i, i, i, vp]
    L.mi_ccl_probe_bandwidth.argtypes = [i, vp, i, sz, vp]
    L.mi_ccl_last_kernel.restype = C.c_char_p
    L.mi_ccl_last_kernel.argtypes = []
    L.mi_ccl_set_param.argtypes = [C.c_char_p, C.c_long]
    L.mi_ccl_get_param.restype = C.c_long
    L.mi_ccl_get_param.argtypes = [C.c_char_p]
    _lib = L
    return L


def status_str(status):
    return lib().mi_ccl_status_str(int(status)).decode()


def _check(status, what):
    if status != SUCCESS:
        raise CclError(status, what)


def _ptr(x):
    """Device address of a torch tensor, or an int address passed through."""
    if isinstance(x, int):
        return x
    return x.data_ptr()


def _stream(stream):
    if stream is None:
        import torch
        return torch.cuda.current_stream().cuda_stream
    if isinstance(stream, int):
        return stream
    return stream.cuda_stream


def _ptr_array(xs):
    return (C.c_void_p * len(xs))(*[_ptr(x) for x in xs])


def datatype_size(dtype):
    return lib().mi_ccl_datatype_size(dtype)


def datatype_name(dtype):
    return lib().mi_ccl_datatype_name(dtype).decode()


def reduction_to_str(op):
    return lib().mi_ccl_reduction_to_str(op).decode()


def kernel_name(kernel, dtype, op):
    buf = C.create_string_buffer(128)
    _check(lib().mi_ccl_kernel_name(kernel.encode(), dtype, op, buf, 128), "mi_ccl_kernel_name")
    return buf.value.decode()


def comp_reduce(dtype, op, inp, count, inout, bf16_impl=BF16_AVX512BF, fp16_impl=FP16_DEFAULT, stream=None):
    """inout[i] = inout[i] OP inp[i] (ccl_comp_reduce)."""
    _check(lib().mi_ccl_comp_reduce(dtype, op, _ptr(inp), count, _ptr(inout), bf16_impl, fp16_impl, _stream(stream)),
           "mi_ccl_comp_reduce")


def bf16_reduce(inp, count, inout, op, bf16_impl=BF16_AVX512BF, stream=None):
    _check(lib().mi_ccl_bf16_reduce(_ptr(inp), count, _ptr(inout), op, bf16_impl, _stream(stream)),
           "mi_ccl_bf16_reduce")


def fp16_reduce(inp, count, inout, op, fp16_impl=FP16_DEFAULT, stream=None):
    _check(lib().mi_ccl_fp16_reduce(_ptr(inp), count, _ptr(inout), op, fp16_impl, _stream(stream)),
           "mi_ccl_fp16_reduce")


def comp_reduce_n(dtype, op, srcs, dst, count, lp_mode=LP_PAIRWISE, bf16_impl=BF16_AVX512BF, fp16_impl=FP16_DEFAULT,
                  stream=None):
    """dst = srcs[0] OP srcs[1] OP ... in argument order, one pass."""
    arr = _ptr_array(srcs)
    _check(lib().mi_ccl_comp_reduce_n(dtype, op, arr, len(srcs), _ptr(dst), count, lp_mode, bf16_impl, fp16_impl,
                                      _stream(stream)), "mi_ccl_comp_reduce_n")


def comp_reduce_write_n(dtype, op, srcs, dsts, count, lp_mode=LP_PAIRWISE, bf16_impl=BF16_AVX512BF,
                        fp16_impl=FP16_DEFAULT, stream=None):
    """Every dsts[k] = srcs[0] OP srcs[1] OP ... in argument order, one pass; one source and LP_PAIRWISE is a
    copy of one buffer to len(dsts) buffers."""
    s, d = _ptr_array(srcs), _ptr_array(dsts)
    _check(lib().mi_ccl_comp_reduce_write_n(dtype, op, s, len(srcs), d, len(dsts), count, lp_mode, bf16_impl,
                                            fp16_impl, _stream(stream)), "mi_ccl_comp_reduce_write_n")


def comp_reduce_batch(dtype, op, jobs, lp_mode=LP_PAIRWISE, bf16_impl=BF16_AVX512BF, fp16_impl=FP16_DEFAULT, stream=None):
    """Many independent reduces in one launch.  jobs: list of (srcs, dst, count), every job with the same number of
    inputs; dst = srcs[0] OP srcs[1] OP ... over count elements."""
    if not jobs:
        return
    n = len(jobs[0][0])
    assert all(len(j[0]) == n for j in jobs), "every job takes the same number of inputs"
    srcs = _ptr_array([s for j in jobs for s in j[0]])
    dsts = _ptr_array([j[1] for j in jobs])
    counts = (C.c_size_t * len(jobs))(*[int(j[2]) for j in jobs])
    _check(lib().mi_ccl_comp_reduce_batch(dtype, op, srcs, n, dsts, counts, len(jobs), lp_mode, bf16_impl, fp16_impl,
                                          _stream(stream)), "mi_ccl_comp_reduce_batch")


class BatchJobs:
    """The pointer and count tables of a batch, built once: calling it costs one foreign call instead of one
    data_ptr() per buffer (which a timing loop would otherwise measure)."""

    def __init__(self, jobs):
        self.n = len(jobs[0][0])
        assert all(len(j[0]) == self.n for j in jobs), "every job takes the same number of inputs"
        self.keep = jobs                      # the tensors stay alive with the tables
        self.srcs = _ptr_array([s for j in jobs for s in j[0]])
        self.dsts = _ptr_array([j[1] for j in jobs])
        self.counts = (C.c_size_t * len(jobs))(*[int(j[2]) for j in jobs])
        self.n_jobs = len(jobs)

    def reduce(self, dtype, op, lp_mode=LP_PAIRWISE, bf16_impl=BF16_AVX512BF, fp16_impl=FP16_DEFAULT, stream=None):
        _check(lib().mi_ccl_comp_reduce_batch(dtype, op, self.srcs, self.n, self.dsts, self.counts, self.n_jobs, lp_mode,
                                              bf16_impl, fp16_impl, _stream(stream)), "mi_ccl_comp_reduce_batch")


def comp_batch_reduce(in_buf, offsets, count, inout, dtype, op, keep_precision, bf16_impl=BF16_AVX512BF,
                      fp16_impl=FP16_DEFAULT, stream=None):
    offs = (C.c_size_t * len(offsets))(*[int(o) for o in offsets])
    _check(lib().mi_ccl_comp_batch_reduce(_ptr(in_buf), offs, len(offsets), count, _ptr(inout), dtype, op,
                                          int(keep_precision), bf16_impl, fp16_impl, _stream(stream)),
           "mi_ccl_comp_batch_reduce")


def comp_copy(inp, out, nbytes, use_nontemporal=False, stream=None):
    _check(lib().mi_ccl_comp_copy(_ptr(inp), _ptr(out), nbytes, int(use_nontemporal), _stream(stream)),
           "mi_ccl_comp_copy")


def convert_fp32_to_bf16_arrays(fp32_buf, bf16_buf, count, bf16_impl=BF16_AVX512BF, stream=None):
    _check(lib().mi_ccl_convert_fp32_to_bf16_arrays(_ptr(fp32_buf), _ptr(bf16_buf), count, bf16_impl,
                                                    _stream(stream)), "mi_ccl_convert_fp32_to_bf16_arrays")


def convert_fp32_to_fp16_arrays(fp32_buf, fp16_buf, count, stream=None):
    _check(lib().mi_ccl_convert_fp32_to_fp16_arrays(_ptr(fp32_buf), _ptr(fp16_buf), count, _stream(stream)),
           "mi_ccl_convert_fp32_to_fp16_arrays")


def convert_fp16_to_fp32_arrays(fp16_buf, fp32_buf, count, stream=None):
    _check(lib().mi_ccl_convert_fp16_to_fp32_arrays(_ptr(fp16_buf), _ptr(fp32_buf), count, _stream(stream)),
           "mi_ccl_convert_fp16_to_fp32_arrays")


def convert_bf16_to_fp32_arrays(bf16_buf, fp32_buf, count, stream=None):
    _check(lib().mi_ccl_convert_bf16_to_fp32_arrays(_ptr(bf16_buf), _ptr(fp32_buf), count, _stream(stream)),
           "mi_ccl_convert_bf16_to_fp32_arrays")


def fusion_offsets(counts, dtype_size, align):
    k = len(counts)
    cnt = (C.c_size_t * k)(*[int(c) for c in counts])
    offs = (C.c_size_t * k)()
    total = C.c_size_t(0)
    _check(lib().mi_ccl_fusion_offsets(cnt, k, dtype_size, align, offs, C.byref(total)), "mi_ccl_fusion_offsets")
    return list(offs), total.value


class FusionPlan:
    """Layout of one fused group (counts, dtype, alignment) and its device-side work table."""

    def __init__(self, counts, dtype, align=256):
        k = len(counts)
        cnt = (C.c_size_t * k)(*[int(c) for c in counts])
        h = C.c_void_p()
        _check(lib().mi_ccl_fusion_plan_create(cnt, k, dtype, align, C.byref(h)), "mi_ccl_fusion_plan_create")
        self._h = h
        self.k = k
        self.dtype = dtype
        self.counts = [int(c) for c in counts]

    @property
    def nbytes(self):
        return lib().mi_ccl_fusion_plan_bytes(self._h)

    def offset(self, i):
        return lib().mi_ccl_fusion_plan_offset(self._h, i)

    def pack(self, tensors, fusion_buf, stream=None):
        assert len(tensors) == self.k
        _check(lib().mi_ccl_fusion_pack(self._h, _ptr_array(tensors), _ptr(fusion_buf), _stream(stream)),
               "mi_ccl_fusion_pack")

    def unpack(self, fusion_buf, tensors, stream=None):
        assert len(tensors) == self.k
        _check(lib().mi_ccl_fusion_unpack(self._h, _ptr(fusion_buf), _ptr_array(tensors), _stream(stream)),
               "mi_ccl_fusion_unpack")

    def reduce(self, op, own_tensors, peers, out_tensors, lp_mode=LP_PAIRWISE, bf16_impl=BF16_AVX512BF,
               fp16_impl=FP16_DEFAULT, stream=None):
        assert len(own_tensors) == self.k and len(out_tensors) == self.k
        _check(lib().mi_ccl_fusion_reduce(self._h, op, _ptr_array(own_tensors), _ptr_array(peers), len(peers),
                                          _ptr_array(out_tensors), lp_mode, bf16_impl, fp16_impl, _stream(stream)),
               "mi_ccl_fusion_reduce")

    def close(self):
        if self._h:
            lib().mi_ccl_fusion_plan_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


FUSION_STATIC_MAX_TENSORS, FUSION_STATIC_MAX_ITEMS = 1024, 131072


def fusion_reduce_static(counts, dtype, align, op, own_tensors, peers, out_tensors, lp_mode=LP_PAIRWISE,
                         bf16_impl=BF16_AVX512BF, fp16_impl=FP16_DEFAULT, stream=None):
    """FusionPlan.reduce without a plan and without any allocation (mi_ccl_fusion_reduce_static)."""
    k = len(counts)
    cnt = (C.c_size_t * k)(*[int(c) for c in counts])
    _check(lib().mi_ccl_fusion_reduce_static(cnt, k, dtype, align, op, _ptr_array(own_tensors), _ptr_array(peers),
                                             len(peers), _ptr_array(out_tensors), lp_mode, bf16_impl, fp16_impl,
                                             _stream(stream)), "mi_ccl_fusion_reduce_static")


PROBE_READ, PROBE_WRITE_ONE, PROBE_WRITE_FOUR = 0, 1, 2


def probe_bandwidth(kind, bufs, nbytes, stream=None):
    """Read-only (kind PROBE_READ, all of bufs) or write-only (PROBE_WRITE_ONE / PROBE_WRITE_FOUR, bufs[0]) stream."""
    _check(lib().mi_ccl_probe_bandwidth(kind, _ptr_array(bufs), len(bufs), nbytes, _stream(stream)),
           "mi_ccl_probe_bandwidth")


def last_kernel():
    """Kernel template the calling thread's most recent call launched."""
    return lib().mi_ccl_last_kernel().decode()


def set_param(name, value):
    _check(lib().mi_ccl_set_param(name.encode(), int(value)), f"mi_ccl_set_param({name})")


def get_param(name):
    return lib().mi_ccl_get_param(name.encode())
