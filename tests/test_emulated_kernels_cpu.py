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


def test_one_unit_in_the_last_place_of_the_approximate_instructions(emulated_library):
    """The emulation computes v_exp_f32, v_sqrt_f32, v_rsq_f32 and v_rcp_f32 exactly; the hardware
    is off by about one unit in the last place.  EMU_APPROX=hash moves every such result up, down or
    not at all (repeatably, by a hash of the value): culls with a slack must still be supersets,
    indices computed through a reciprocal must come out the same, the bit-exact paths must not
    notice at all, sums stay within twice the tolerance (tests/emu/cases.py)."""
    env = dict(os.environ, EMU_APPROX="hash")
    for args in (["cases.py", "forward_index"], ["cases.py", "backward_index"], ["cases.py", "interpolate"],
                 ["random_parity.py", "10", "9"], ["random_resample.py", "8", "9"]):
        p = subprocess.run([sys.executable, os.path.join(HERE, "emu", args[0])] + args[1:], env=env,
                           stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=1500)
        assert p.returncode == 0 and "passed" in p.stdout, "%s:\n%s" % (" ".join(args), p.stdout[-3000:])


def test_threads_and_workgroups_run_last_to_first(emulated_library):
    """Between two meeting points (a barrier, a cross-lane operation) an emulated thread runs alone,
    and normally thread 0 goes first.  EMU_ORDER=reverse runs threads, hence waves, and workgroups
    last to first: results that depend on who goes first -- a missing barrier, a workgroup that
    relies on another -- change.  (In every mode the emulator fills all LDS with 0xCB before a
    workgroup starts, so neither zeros nor the previous workgroup's leftovers can be relied on.)"""
    env = dict(os.environ, EMU_ORDER="reverse")
    for args in (["cases.py", "forward_batch"], ["cases.py", "forward_vector"], ["cases.py", "second_order"],
                 ["cases.py", "interpolate"], ["random_parity.py", "8", "6"]):
        p = subprocess.run([sys.executable, os.path.join(HERE, "emu", args[0])] + args[1:], env=env,
                           stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=1500)
        assert p.returncode == 0 and "passed" in p.stdout, "%s:\n%s" % (" ".join(args), p.stdout[-3000:])


def test_with_fused_multiply_adds(emulated_library):
    """The device compiler turns a * b + c into one fused operation wherever the source lets it; the
    plain emulated build fuses nothing.  A second build (EMU_CONTRACT=1) fuses like the device
    compiler: the paths that match the reference bit for bit -- binary densities, the transform, the
    exact predicates on cut-offs -- must do so there as well, i.e. say `fp contract(off)` themselves
    wherever it matters."""
    env = dict(os.environ, EMU_CONTRACT="1")
    for args in (["cases.py", "transform"], ["cases.py", "forward_index"], ["cases.py", "backward_index"],
                 ["random_parity.py", "10", "8"]):
        p = subprocess.run([sys.executable, os.path.join(HERE, "emu", args[0])] + args[1:], env=env,
                           stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=1500)
        assert p.returncode == 0 and "passed" in p.stdout, "%s:\n%s" % (" ".join(args), p.stdout[-3000:])


def test_cpp_classes_on_the_emulated_library(emulated_library):
    """tests/cpp/test_api.cpp -- GridMaker, GridInterpolater, Transform, Grid / ManagedGrid and
    CoordinateSet of include/libmolgrid, used the way the reference's own unit tests use its
    classes -- compiled against the emulation's stand-in for the HIP runtime and linked with the
    emulated library: the whole C++ host layer, device paths included, on the CPU."""
    sys.path.insert(0, os.path.join(HERE, "emu"))
    import build_emu
    p = subprocess.run([build_emu.build_cpp_api_test(), "gpu"], stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True, timeout=600)
    assert p.returncode == 0 and "0 failure(s)" in p.stdout, p.stdout[-3000:]


def test_randomised_parity(emulated_library):
    """tests/emu/random_parity.py: the configuration itself is drawn -- grid size, resolution,
    channel count, radius scale, radius multiples (truncated modes too), atoms on voxel centres
    with radii that put voxels ON the cut-off -- and every kernel compared with the oracle under
    the GPU tests' bounds (a few rounds here; thousands by hand, which is how the handling of a
    Gaussian cut off without a tail and of a binary sphere as wide as its index box was found)."""
    p = subprocess.run([sys.executable, os.path.join(HERE, "emu", "random_parity.py"), "20", "5"],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=1500)
    assert p.returncode == 0 and "20 rounds passed" in p.stdout, p.stdout[-3000:]
    # the same for resampling: grid sizes, resolution ratios, centres, shifts beyond the input,
    # axis-aligned and random rotations (tests/emu/random_resample.py; 1,800 rounds by hand)
    p = subprocess.run([sys.executable, os.path.join(HERE, "emu", "random_resample.py"), "20", "5"],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=1500)
    assert p.returncode == 0 and "20 rounds passed" in p.stdout, p.stdout[-3000:]


@pytest.mark.parametrize("checks", ["undefined", "address"])
def test_run_time_checks(emulated_library, checks):
    """The same sources built again with clang's run-time checks, every report fatal, running the
    comparison groups of the kernels, a few random configurations and a few rounds of hostile inputs.  "undefined": fixed-size
    array indices (the register and LDS arrays), shifts, signed overflow, float-to-int conversions
    out of range, alignment -- a conversion of an infinite coordinate is what these found.
    "address": every LDS array (static storage in the emulation) and stack array has poisoned
    neighbours, so an access through a pointer that leaves its array is caught too (the runtime is
    loaded with the library, after the interpreter: hence verify_asan_link_order=0)."""
    env = dict(os.environ, EMU_SANITIZE="1" if checks == "undefined" else "address",
               ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=0")
    groups = [["cases.py", "forward_paged"], ["cases.py", "backward_index"], ["cases.py", "second_order"],
              ["cases.py", "interpolate"], ["random_parity.py", "6", "4"], ["fuzz.py", "6", "5"]]
    if checks == "undefined":
        groups.insert(2, ["cases.py", "forward_vector"])
    for args in groups:
        p = subprocess.run([sys.executable, os.path.join(HERE, "emu", args[0])] + args[1:], env=env,
                           stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=1500)
        assert p.returncode == 0 and "runtime error" not in p.stdout and "AddressSanitizer" not in p.stdout, \
            "%s under the %s checks (status %d):\n%s" % (" ".join(args), checks, p.returncode, p.stdout[-3000:])


def _run(script, *flags, timeout=2400):
    p = subprocess.run([sys.executable, os.path.join(HERE, "emu", script)] + list(flags),
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=timeout)
    assert p.returncode == 0, "%s failed (status %d):\n%s" % (script, p.returncode, p.stdout[-4000:])
    return p.stdout


def test_python_host_layer_on_a_fake_device(emulated_library):
    """tests/emu/python_layer.py: GridMaker / Transform / GridInterpolater / Coords2Grid of the
    package on a stand-in for the ROCm device (CPU tensors that say they are on cuda:0, the emulated
    kernels behind the C ABI) against the oracle: forward overloads, workspaces, the sort and splat
    halves, backward with the fused un-rotation, vector types with atom lists, autograd, resampling."""
    assert "comparisons passed" in _run("python_layer.py")
    # and with the grid maker, the molecule and the way of calling drawn at random (host arrays,
    # float64 grids, ragged batches whose workspaces must grow, radii by type, the autograd layer)
    assert "comparisons passed" in _run("random_python_layer.py", "6", "3")


def test_smoke_and_bench_run_end_to_end_on_a_fake_device(emulated_library):
    """__graft_entry__.smoke() and bench.py (a batch of one example, every step variant, the
    write-out autotune, the JSON line with the fields the driver reads) on the same stand-in: the
    figures mean nothing, the code paths are what is checked.  The other workloads of bench.py are
    left out here (tests/emu/bench_dry_run.py --small-extras by hand runs them too, minutes)."""
    assert "passed" in _run("smoke_dry_run.py")
    assert "JSON line complete" in _run("bench_dry_run.py", "--no-extras", "--no-cpu")
