"""Host-only test of the launch geometry of the copy, broadcast and converter kernels
(oneccl_amd/csrc/launch_geometry.hpp): sizes from 1 byte to 256 GiB, 1..16 destinations -- every launch below HIP's
2^32 lanes per grid, every group of elements given to exactly one lane.  Built with g++; no GPU needed."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))


def test_launch_geometry():
    cpp = os.path.join(HERE, "cpp")
    exe = os.path.join(cpp, "test_launch_geometry")
    subprocess.check_call(["make", "-s", "-C", cpp, exe])
    p = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stdout[-3000:] + p.stderr[-3000:]
    assert " 0 failed" in p.stdout
