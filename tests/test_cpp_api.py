"""The C++ host layer (include/libmolgrid/*.h): compiled test program, run as a child process."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "tests", "cpp", "test_api")


def binary():
    if not os.path.exists(BINARY):
        import __graft_entry__
        __graft_entry__.build_cpp_api_test()
    return BINARY


def test_host_side_checks():
    """Views, managed grids, quaternion/transform arithmetic and argument checks: no device."""
    r = subprocess.run([binary(), "check"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr


@pytest.mark.gpu
def test_gridding_through_the_cpp_classes():
    r = subprocess.run([binary(), "gpu"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
