"""Host-only test of the fusion manager's queueing logic (oneccl_amd/csrc/ccl_fusion.cpp) against a mock backend:
what can be fused, urgent / count / buffer-size flushes, the cycle timer, per-dtype grouping, buffer reuse, and
add() from several threads while another executes.  Built with g++ under AddressSanitizer/UBSan; no GPU needed."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))


def test_fusion_manager_queue_logic():
    cpp = os.path.join(HERE, "cpp")
    exe = os.path.join(cpp, "test_fusion_manager")
    subprocess.check_call(["make", "-s", "-C", cpp, exe])
    p = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "0 failed" in p.stdout
