import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm device (run on the MI355X box)")


# GPU tests whose kernels are re-written sweeps and scans (vector-typed forward with atom lists,
# vector backward, relevance, second order, and the layers on top of them), and tests of behaviour
# that is newer than the last GPU run (radii <= 0 dropped in the sort), run after the tests of
# the paths whose machine code is the one that has already passed on a GPU, or close to it: under
# `pytest -x` a failure among the former then cannot hide the results of the latter.  The two files
# whose names sort last keep their places at the end.
LATER = ("test_vector_gpu.py", "test_second_order_gpu.py", "test_torch_gpu.py", "test_cpp_api.py",
         "test_vector_types_full_size", "test_forward_vector_and_batches_into_double_grids",
         "test_vector_typed_examples", "test_training_", "test_zero_and_negative_radii",
         "test_backward_gpu.py::test_unusual_radius_multiples[gm_args0]")   # the kernel instance for a Gaussian without a tail


def _tier(item):
    name = item.nodeid
    if "test_zz_" in name:
        return 3
    if "test_zx_" in name:
        return 2
    return 1 if any(p in name for p in LATER) else 0


def pytest_collection_modifyitems(config, items):
    items.sort(key=_tier)             # stable: the order inside a tier stays pytest's
    try:
        import torch
        have_gpu = torch.cuda.is_available()
    except Exception:  # pragma: no cover
        have_gpu = False
    if have_gpu:
        return
    skip = pytest.mark.skip(reason="no ROCm device visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
