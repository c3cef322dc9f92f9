"""TEST INFRASTRUCTURE: runs the GPU test files of tests/ on the fake device of fake_cuda.py, i.e.
their Python against the emulated kernels (CPU only; what needs real hardware -- timing, graphs,
the C++ API binary -- fails or is deselected).  For the paths that have not met a GPU yet.
    python tests/emu/gpu_tests_on_fake_device.py [pytest arguments, default: the small test files]"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
sys.path.insert(0, HERE)

import fake_cuda  # noqa: E402

fake_cuda.activate()
import pytest  # noqa: E402

args = sys.argv[1:] or [os.path.join(ROOT, "tests"), "-m", "gpu", "-q", "-x",
                        "--deselect", "tests/test_cpp_api.py",
                        "-k", "not full_size and not fullsize and not full_batch and not config3 and not every_example"]
sys.exit(pytest.main(args))
