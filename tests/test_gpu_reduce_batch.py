"""mi_ccl_comp_reduce_batch: many independent reduces in one launch (the shape of the reference's read_reduce_write and
reduce_read_write_kernel_N), against one oracle call per job -- 1, 7, 64 and 200 jobs (the last takes several launches),
counts from 0 and 1 to 2^20 mixed in one call, every buffer at its own alignment, outputs in place, every dtype and
operation, the 16-bit modes, NaN-carrying bit patterns."""
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
    c.lib()
    return c


def _run(comp, rng, dtype, op, n, counts, lp=0, impl=2, f16=0, keep=0, kind="config", in_place_every=3, mixed_align=True, variant=0):
    """Builds the jobs (every buffer inside a zero-padded holder at its own element shift), runs them in one call and
    checks every job against the oracle and every holder for writes outside the payload."""
    import torch
    np_t = O.NP_STORAGE[dtype]
    esz = O.DTYPE_SIZE[dtype]
    per16 = 16 // esz
    pad = 32
    jobs, checks = [], []
    for j, count in enumerate(counts):
        srcs = make_inputs(rng, dtype, count, op, n, kind) if count else [np.zeros(0, np_t) for _ in range(n)]
        shifts = [int(x) for x in rng.integers(0, per16 + 1, n + 1)] if mixed_align else [j % (per16 + 1)] * (n + 1)
        holders = []
        for s_, sh in zip(srcs, shifts):
            h = np.zeros(count + 2 * pad, np_t)
            h[pad + sh:pad + sh + count] = s_
            holders.append(to_dev(h))
        in_place = in_place_every and j % in_place_every == 0
        if in_place:
            k = j % n
            out_h, out_sh = holders[k], shifts[k]
        else:
            out_h, out_sh = to_dev(np.zeros(count + 2 * pad, np_t)), shifts[n]
        ptrs = [h.data_ptr() + (pad + sh) * esz for h, sh in zip(holders, shifts)]
        jobs.append((ptrs, out_h.data_ptr() + (pad + out_sh) * esz, count))
        checks.append((srcs, out_h, pad + out_sh, count, holders))
    comp.set_param("variant", variant)      # 8: the phased form whatever the sizes
    try:
        comp.comp_reduce_batch(dtype, op, jobs, lp_mode=lp, bf16_impl=impl, fp16_impl=f16)
        torch.cuda.synchronize()
    finally:
        comp.set_param("variant", 0)
    kw = dict(keep=keep, bf16_impl=impl, fp16_impl=f16 or O.FP16_AVX512F)
    for j, (srcs, out_h, lo, count, holders) in enumerate(checks):
        g = to_host(out_h, np_t)
        what = f"job {j} of {len(counts)}: dtype={O.DTYPE_NAMES[dtype]} op={O.OP_NAMES[op]} n={n} count={count}"
        if count:
            want = O.reduce_n(srcs, dtype, op, **kw)
            assert_same(g[lo:lo + count], want, dtype, what, srcs, op, **kw)
        assert not g[:lo].view(np.uint8).any() and not g[lo + count:].view(np.uint8).any(), what + ": wrote outside the destination"


@pytest.mark.parametrize("dtype", range(12))
@pytest.mark.parametrize("op", range(4))
def test_every_dtype_and_op_seven_jobs(comp, dtype, op):
    rng = np.random.default_rng(7000 + dtype * 4 + op)
    for n in (1, 2, 3, 8):
        _run(comp, rng, dtype, op, n, [1, 17, 0, 4099, 15, 70_001, 1000])
    for n in (2, 5):
        _run(comp, rng, dtype, op, n, [1, 17, 0, 4099, 15, 70_001, 1000, 9_000], variant=8)
        assert comp.last_kernel() == "reduce_batch_phased_kernel"


@pytest.mark.parametrize("n_jobs", [1, 7, 64, 200])
def test_job_counts_and_mixed_sizes(comp, n_jobs):
    """Counts log-uniform over 1 .. 2^20 (and a few empty jobs) in one call; 200 jobs of two inputs need three launches (96 jobs each at most)."""
    rng = np.random.default_rng(7100 + n_jobs)
    counts = [int(c) for c in np.exp(rng.uniform(0, np.log(1 << 20), n_jobs))]
    counts[0] = 1 << 20
    if n_jobs > 3:
        counts[2] = 0
        counts[3] = 1
    for variant in (0, 8):
        _run(comp, rng, O.FLOAT32, O.SUM, 2, counts, variant=variant)
        _run(comp, rng, O.INT8, O.MAX, 2, counts, variant=variant)
        if n_jobs <= 64:
            _run(comp, rng, O.BFLOAT16, O.SUM, 8, counts, lp=comp.LP_KEEP_PRECISION, keep=1, variant=variant)


def test_more_jobs_than_one_table_holds_with_eight_inputs(comp):
    """Eight inputs per job leave room for 35 jobs per launch (320 pointers): 100 jobs take three launches."""
    rng = np.random.default_rng(7150)
    counts = [int(c) for c in rng.integers(0, 40_000, 100)]
    _run(comp, rng, O.FLOAT16, O.PROD, 8, counts)
    _run(comp, rng, O.INT64, O.MIN, 8, counts, in_place_every=2)


def test_large_jobs_mixed_with_small_ones(comp):
    """The chunks of a large reduce-scatter beside a few stragglers in one call: when the jobs of a launch together fill
    whole phases they run in the phased form (several phases here, job boundaries inside a phase, jobs smaller than
    one block's share), else in the streaming form; every job against the oracle.  One input per job is a copy per
    job: the large ones go to the copy kernel."""
    rng = np.random.default_rng(7170)
    big2 = (340 << 20) // 4           # two fp32 inputs: 3 x 340 MiB of traffic each
    _run(comp, rng, O.FLOAT32, O.SUM, 2, [1000, big2, 0, 77, big2 + 5, 1 << 20, 14 << 20], in_place_every=2)
    assert comp.last_kernel() == "reduce_batch_phased_kernel"
    _run(comp, rng, O.FLOAT32, O.SUM, 2, [14 << 20, 14 << 20 | 1], mixed_align=False)      # 112 MiB of results: 1.3 phases
    assert comp.last_kernel() == "reduce_batch_kernel"
    _run(comp, rng, O.BFLOAT16, O.SUM, 4, [5, 40 << 20, 9], lp=comp.LP_KEEP_PRECISION, keep=1)
    assert comp.last_kernel() == "reduce_batch_phased_kernel"
    _run(comp, rng, O.INT8, O.MAX, 1, [3, 200 << 20, 4099])
    assert comp.last_kernel() == "reduce_batch_kernel"          # the two small jobs; the large one was a copy_kernel launch


def test_chunk_sized_jobs_take_the_phased_form(comp):
    """64 jobs of four inputs of 1 MiB and of 4 MiB each, and seven pair-reduces of 48 MiB (the read_reduce_write shape
    at a tmp-buffer's chunk size): by the automatic choice, all jobs in one launch."""
    rng = np.random.default_rng(7180)
    _run(comp, rng, O.INT32, O.SUM, 4, [(1 << 20) // 4] * 64, in_place_every=0, mixed_align=False)
    assert comp.last_kernel() == "reduce_batch_phased_kernel"
    _run(comp, rng, O.FLOAT16, O.SUM, 4, [(4 << 20) // 2 + (j % 3) for j in range(64)])
    assert comp.last_kernel() == "reduce_batch_phased_kernel"
    _run(comp, rng, O.BFLOAT16, O.SUM, 2, [(48 << 20) // 2] * 7, in_place_every=0)
    assert comp.last_kernel() == "reduce_batch_phased_kernel"
    # jobs of few enough inputs for their type (two for every type, up to eight for the 32-bit ones) have their write
    # phase paced by the device clock: unpaced, a pace no store keeps up with and one that every group of stores waits
    # for give the same bits, with jobs that end inside a tile and in place
    try:
        for pace in (0, 100_000, 2000):
            comp.set_param("phase_write_pace", pace)
            _run(comp, rng, O.FLOAT32, O.SUM, 2, [(6 << 20) // 4 + 5 * j for j in range(40)], in_place_every=3)
            assert comp.last_kernel() == "reduce_batch_phased_kernel"
            _run(comp, rng, O.UINT32, O.MAX, 5, [(3 << 20) // 4 + 3 * j for j in range(40)], in_place_every=4)
            assert comp.last_kernel() == "reduce_batch_phased_kernel"
            _run(comp, rng, O.BFLOAT16, O.SUM, 3, [(5 << 20) // 2 + j for j in range(40)], lp=comp.LP_KEEP_PRECISION, keep=1)
            assert comp.last_kernel() == "reduce_batch_phased_kernel"
    finally:
        comp.set_param("phase_write_pace", 7300)


def test_sixteen_bit_modes_and_nan_patterns(comp):
    rng = np.random.default_rng(7200)
    counts = [33, 8191, 1, 100_003, 16]
    for impl in (0, 1, 2):
        for op in range(4):
            _run(comp, rng, O.BFLOAT16, op, 3, counts, impl=impl, kind="bits")
            _run(comp, rng, O.BFLOAT16, op, 3, counts, lp=comp.LP_KEEP_PRECISION, impl=impl, keep=1, kind="bits")
    for f16 in (2, 3, 4):
        for op in range(4):
            _run(comp, rng, O.FLOAT16, op, 4, counts, f16=f16, kind="bits")


def test_same_as_separate_calls_and_errors(comp):
    """64 jobs in one call give what 64 calls of mi_ccl_comp_reduce_n give; argument errors come back as codes."""
    import torch
    rng = np.random.default_rng(7300)
    counts = [int(c) for c in rng.integers(1, 300_000, 64)]
    srcs = [[to_dev(s) for s in make_inputs(rng, O.FLOAT16, c, O.SUM, 4)] for c in counts]
    one = [torch.empty_like(s[0]) for s in srcs]
    many = [torch.empty_like(s[0]) for s in srcs]
    for s, o, c in zip(srcs, one, counts):
        comp.comp_reduce_n(O.FLOAT16, O.SUM, s, o, c)
    comp.comp_reduce_batch(O.FLOAT16, O.SUM, [(s, o, c) for s, o, c in zip(srcs, many, counts)])
    torch.cuda.synchronize()
    for a, b in zip(one, many):
        assert torch.equal(a, b)
    x = torch.zeros(64, dtype=torch.int32, device="cuda")
    with pytest.raises(comp.CclError):
        comp.comp_reduce_batch(O.INT32, O.SUM, [([x] * 9, x, 4)])                    # more than 8 inputs
    with pytest.raises(comp.CclError):
        comp.comp_reduce_batch(O.INT32, O.SUM, [([x, 0], x, 4)])                     # null input of a non-empty job
    with pytest.raises(comp.CclError):
        comp.comp_reduce_batch(O.INT32, O.SUM, [([x, x.data_ptr() + 2], x, 4)])      # misaligned for the element size
    with pytest.raises(comp.CclError):
        comp.comp_reduce_batch(O.FLOAT32, O.SUM, [([x, x], x, 4)], lp_mode=comp.LP_KEEP_PRECISION)
    comp.comp_reduce_batch(O.INT32, O.SUM, [([0, 0], 0, 0)])                         # an empty job: nothing is looked at
    comp.comp_reduce_batch(O.INT32, O.SUM, [])
    torch.cuda.synchronize()
    assert int(x.count_nonzero()) == 0
