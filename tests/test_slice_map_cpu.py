"""include/util/slice_map.h (which claim counter a workgroup serves, which tiles the counter owns)
checked on the CPU by a small C++ program compiled from the header itself."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_slice_map_partitions_and_bijection(tmp_path):
    exe = str(tmp_path / "slice_map_check")
    subprocess.run(["g++", "-O1", "-std=c++17", "-I" + os.path.join(ROOT, "include"), "-o", exe,
                    os.path.join(ROOT, "tests", "slice_map_check.cpp")], check=True)
    out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout
    assert out.startswith("ok "), out


def test_conv_prologue_arithmetic(tmp_path):
    """include/util/conv_addr.h: the reciprocal division equals the integer division over its domain
    of use, and the window tap mask equals a tap-by-tap loop."""
    exe = str(tmp_path / "conv_addr_check")
    subprocess.run(["g++", "-O2", "-std=c++17", "-I" + os.path.join(ROOT, "include"), "-o", exe,
                    os.path.join(ROOT, "tests", "conv_addr_check.cpp")], check=True)
    out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout
    assert out.startswith("ok "), out
