"""Host-only test of the C++ layer's profiler-range knob (oneccl_amd/csrc/ccl_trace.cpp): switched off it opens no
range and looks for no library; switched on every range is counted and the roctx library is looked up once.  Built
with g++ under AddressSanitizer/UBSan; no GPU needed."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))


def test_trace_knob():
    cpp = os.path.join(HERE, "cpp")
    exe = os.path.join(cpp, "test_trace")
    subprocess.check_call(["make", "-s", "-C", cpp, exe])
    env = dict(os.environ)
    env.pop("MI_CCL_TRACE", None)
    p = subprocess.run([exe], capture_output=True, text=True, timeout=120, env=env)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "0 failed" in p.stdout
