"""Runs the C++ test of the operator surface (tests/cpp/test_ccl_comp.cpp) on the GPU: ccl_comp_reduce,
ccl_comp_batch_reduce, ccl_comp_reduce_n, the custom-reduction callback, the CCL_BF16 knob, copy and converters,
checked against the reference's functional-test closed forms and the oracle."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "cpp", "test_ccl_comp")


def run(env_extra):
    if not os.path.exists(EXE):
        pytest.fail("tests/cpp/test_ccl_comp is not built: run __graft_entry__.build()")
    env = dict(os.environ)
    env.pop("CCL_BF16", None)
    env.update(env_extra)
    p = subprocess.run([EXE], capture_output=True, text=True, timeout=300, env=env)
    assert p.returncode == 0, p.stdout[-4000:] + p.stderr[-2000:]
    assert "0 failed" in p.stdout
    return p.stdout


def test_cpp_surface_default_env():
    out = run({})
    assert "bf16 impl 2" in out          # avx512bf semantics by default


@pytest.mark.parametrize("impl,idx", [("avx512f", 1), ("scalar", 0)])
def test_cpp_surface_ccl_bf16_knob(impl, idx):
    out = run({"CCL_BF16": impl})
    assert f"bf16 impl {idx}" in out


def test_scheduler_entries_and_device_custom_reduction():
    """tests/cpp/test_sched_entries.cpp: COPY / RECV_REDUCE / REDUCE_LOCAL / REDUCE_MONOLITHIC / WRITE_MONOLITHIC
    entries driven by ccl_sched::do_progress over a loop-back transport, and the device-functor custom reduction."""
    exe = os.path.join(HERE, "cpp", "test_sched_entries")
    if not os.path.exists(exe):
        pytest.fail("tests/cpp/test_sched_entries is not built: run __graft_entry__.build()")
    p = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stdout[-4000:] + p.stderr[-2000:]
    assert "0 failed" in p.stdout
