"""The library's gfx950 kernel sources, compiled for the host against the HIP emulation of
tests/emu (fibers for threads, rendezvous for cross-lane operations and barriers, buffer
descriptors checked against their extent and the allocations behind them, arrays that end at an
inaccessible page), run through the real C ABI and compared with the oracle.  No GPU.

What this checks that the GPU tests cannot: every access stays inside its array (a kernel that
leaves one ends the child process), and the waves of a workgroup meet where they must (a missing or
divergent barrier is reported as a deadlock).  What it cannot check: timing, memory ordering, the
instructions the device compiler picks."""
import os
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
RUNNER = os.path.join(HERE, "emu", "cases.py")


@pytest.fixture(scope="module")
def emulated_library():
    sys.path.insert(0, os.path.join(HERE, "emu"))
    import build_emu
    return build_emu.build()


@pytest.mark.parametrize("group", ["transform", "forward_index", "forward_batch", "forward_paged", "forward_split", "backward_index",
                                   "forward_vector", "backward_vector", "second_order", "interpolate",
                                   "config0"])
def test_group(emulated_library, group):
    p = subprocess.run([sys.executable, RUNNER, group], stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True, timeout=1200)
    assert p.returncode == 0, "emulated %s failed (status %d):\n%s" % (group, p.returncode, p.stdout[-4000:])
    assert "comparisons passed" in p.stdout


def test_hostile_inputs_return(emulated_library):
    """tests/emu/fuzz.py: not-a-number and infinite coordinates, radii, types, centres and
    quaternions, radii <= 0 and far larger than the grid, types at and beyond the channel count,
    grids of 1 to 65 voxels a side, empty examples, 70 examples -- every kernel must return without
    leaving its arrays and without a deadlock (a few rounds here; more by hand)."""
    p = subprocess.run([sys.executable, os.path.join(HERE, "emu", "fuzz.py"), "12", "3"],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=1500)
    assert p.returncode == 0, "fuzz failed (status %d):\n%s" % (p.returncode, p.stdout[-3000:])
    assert "12 rounds returned" in p.stdout
