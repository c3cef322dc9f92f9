"""GPU parity of GridMaker.forward (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle
import synth
from util import assert_close, dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mg():
    import libmolgrid_amd
    return libmolgrid_amd


def gpu_forward(mg, gm_args, center, coords, types, radii, ntypes):
    gm = mg.GridMaker(*gm_args)
    out = torch.full(gm.grid_dimensions(ntypes), 7.0, device="cuda")  # must be overwritten
    gm.forward(center, dev(coords), dev(types), dev(radii), out)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def test_density_profile_closed_form(mg):
    """Same constants as the reference's test_radius_multiples (test/test_gridmaker.py:131-184)."""
    c = np.zeros((1, 3), np.float32)
    t = np.zeros(1, np.float32)
    r = np.ones(1, np.float32)
    g = gpu_forward(mg, (0.1, 6.0), (0, 0, 0), c, t, r, 1)
    assert g[0, 30, 30, 30] == pytest.approx(1.0)
    line = g[0, 30, 30, :]
    x = np.abs(np.arange(-3, 3.1, .1))
    gauss = np.exp(-2 * x ** 2)
    for i in range(20, 41):
        assert line[i] == pytest.approx(gauss[i], abs=1e-6)
    for i in list(range(0, 15)) + list(range(45, 61)):
        assert line[i] == pytest.approx(0, abs=1e-7)
    quad = 4 * np.exp(-2) * x ** 2 - 12 * np.exp(-2) * x + 9 * np.exp(-2)
    for i in list(range(15, 20)) + list(range(41, 45)):
        assert line[i] == pytest.approx(quad[i], abs=1e-5)
    # radius_scale 0.5, gaussian_radius_multiple 3: Gaussian all the way
    g = gpu_forward(mg, (0.1, 6.0, False, False, 0.5, 3.0), (0, 0, 0), c, t, r, 1)
    line = g[0, 30, :, 30]
    gauss = np.exp(-2 * (x * 2.0) ** 2)
    for i in range(0, 61):
        assert line[i] == pytest.approx(gauss[i], abs=1e-5)


@pytest.mark.parametrize("res,dimension,ntypes,natoms", [
    (0.5, 6.0, 3, 20),      # dim 13: partial tiles on every axis
    (0.5, 12.0, 5, 60),     # dim 25
    (0.25, 5.75, 2, 15),    # dim 24
    (1.0, 15.0, 40, 200),   # dim 16, more channels than one LDS pass holds
    (0.5, 23.5, 28, 300),   # dim 48
    (0.5, 29.5, 4, 500),    # dim 60: two slabs in z, the second one partial
    (0.25, 25.25, 3, 400),  # dim 102: three slabs, rows that are not a multiple of four voxels
    (0.5, 31.5, 4, 400),    # dim 64: two slabs of 32 voxels (whole cache lines) instead of 48 + 16
])
@pytest.mark.parametrize("binary", [False, True])
def test_small_random_vs_oracle(mg, res, dimension, ntypes, natoms, binary):
    rng = np.random.default_rng(11 + natoms)
    coords, types, radii = synth.small_index_case(rng, natoms, ntypes, dimension / 2 + 2.0)
    types = types + rng.uniform(0, 0.9, natoms).astype(np.float32) * (types >= 0)  # floor()
    center = rng.uniform(-1, 1, 3).astype(np.float32)
    ref = oracle.GridMaker(res, dimension, binary).forward(center, coords, types, radii, ntypes)
    got = gpu_forward(mg, (res, dimension, binary), center, coords, types, radii, ntypes)
    if binary:
        assert np.array_equal(got, ref)
    else:
        assert_close(got, ref, what="forward")


@pytest.mark.parametrize("gm_args", [
    (0.5, 11.5, False, False, 1.0, -1.5),   # truncated Gaussian, no quadratic tail
    (0.5, 11.5, True, False, 1.0, -0.5),    # binary sphere wider than its index box
    (0.5, 11.5, False, False, 1.3, 0.7),    # radius scale + early quadratic
    (0.5, 11.5, True, False, 0.6, 2.0),
])
def test_unusual_radius_multiples(mg, gm_args):
    rng = np.random.default_rng(5)
    coords, types, radii = synth.small_index_case(rng, 80, 4, 7.0)
    ref = oracle.GridMaker(*gm_args).forward((0, 0, 0), coords, types, radii, 4)
    got = gpu_forward(mg, gm_args, (0, 0, 0), coords, types, radii, 4)
    if gm_args[2]:
        assert np.array_equal(got, ref)
    else:
        assert_close(got, ref, what="forward")


@pytest.mark.parametrize("binary", [False, True])
def test_zero_and_negative_radii_add_nothing(mg, binary):
    """An atom whose radius is zero or negative has an empty index box in the reference
    (src/grid_maker.cu:66-79): it adds nothing, whatever its neighbours are."""
    rng = np.random.default_rng(21)
    coords, types, radii = synth.small_index_case(rng, 120, 3, 6.0)
    radii[::3] = 0.0
    radii[1::3] = -radii[1::3]
    keep = radii > 0
    gm_args = (0.5, 11.5, binary)
    ref = oracle.GridMaker(*gm_args).forward((0, 0, 0), coords, types, radii, 3)
    only = oracle.GridMaker(*gm_args).forward((0, 0, 0), coords[keep], types[keep], radii[keep], 3)
    assert np.array_equal(ref, only)                       # the oracle itself: nothing added
    got = gpu_forward(mg, gm_args, (0, 0, 0), coords, types, radii, 3)
    got_only = gpu_forward(mg, gm_args, (0, 0, 0), coords[keep], types[keep], radii[keep], 3)
    assert np.array_equal(got, got_only)
    if binary:
        assert np.array_equal(got, ref)
    else:
        assert_close(got, ref, what="forward")


def test_many_atoms_on_one_spot(mg):
    """More candidates than one LDS list holds: 3000 atoms inside one tile."""
    rng = np.random.default_rng(3)
    n = 3000
    coords = rng.normal(0, 0.3, (n, 3)).astype(np.float32)
    types = rng.integers(0, 2, n).astype(np.float32)
    radii = rng.uniform(1.0, 1.5, n).astype(np.float32)
    ref = oracle.GridMaker(0.5, 7.5).forward((0, 0, 0), coords, types, radii, 2)
    got = gpu_forward(mg, (0.5, 7.5), (0, 0, 0), coords, types, radii, 2)
    # thousands of terms per voxel, summed by the kernel in record order (x slab of the atom's
    # centre, then atom number) and by the oracle in atom order: equal to rounding
    assert_close(got, ref, what="dense forward")


def test_empty_and_ignored_atoms(mg):
    gm = mg.GridMaker(0.5, 7.5)
    out = torch.full(gm.grid_dimensions(3), 5.0, device="cuda")
    gm.forward((0, 0, 0), torch.zeros((0, 3), device="cuda"), torch.zeros(0, device="cuda"),
               torch.zeros(0, device="cuda"), out)
    assert float(out.abs().max()) == 0.0
    coords = dev(np.zeros((4, 3), np.float32))
    types = dev(np.asarray([-1, -1, 3, 7], np.float32))   # negative and >= ntypes: ignored
    out.fill_(5.0)
    gm.forward((0, 0, 0), coords, types, dev(np.ones(4, np.float32)), out)
    assert float(out.abs().max()) == 0.0


def test_config0_vs_oracle(mg):
    c = synth.config0()
    ref = oracle.GridMaker(0.5, 23.5).forward((0, 0, 0), c["coords"], c["types"], c["radii"], 28)
    got = gpu_forward(mg, (0.5, 23.5), (0, 0, 0), c["coords"], c["types"], c["radii"], 28)
    assert_close(got, ref, what="config 0")
    refb = oracle.GridMaker(0.5, 23.5, True).forward((0, 0, 0), c["coords"], c["types"],
                                                    c["radii"], 28)
    gotb = gpu_forward(mg, (0.5, 23.5, True), (0, 0, 0), c["coords"], c["types"], c["radii"], 28)
    assert np.array_equal(gotb, refb)


@pytest.mark.parametrize("binary", [False, True])
def test_ragged_batch_with_transform_vs_oracle(mg, binary):
    """Configuration 1 at a batch the oracle finishes in seconds."""
    c = synth.config1(nbatch=6)
    B = len(c["offsets"]) - 1
    moved_ref = oracle.transform_forward_batch(c["offsets"], c["quats"], c["centers"],
                                               c["translations"], c["coords"])
    ref = oracle.GridMaker(0.5, 23.5, binary).forward_batch(
        c["offsets"], c["centers"], moved_ref, c["types"], c["radii"], 28, nthreads=6)
    gm = mg.GridMaker(0.5, 23.5, binary)
    coords = dev(c["coords"])
    moved = torch.empty_like(coords)
    mg.transform_batch(c["offsets"], c["quats"], c["centers"], c["translations"], coords, moved)
    out = torch.full((B,) + gm.grid_dimensions(28), 3.0, device="cuda")
    gm.forward_batch(c["offsets"], c["centers"], moved, dev(c["types"]), dev(c["radii"]), out)
    torch.cuda.synchronize()
    assert np.array_equal(moved.cpu().numpy(), moved_ref)   # same float ops, same order
    got = out.cpu().numpy()
    if binary:
        assert np.array_equal(got, ref)
    else:
        assert_close(got, ref, what="config 1")


def test_padded_batch_matches_single_calls(mg):
    rng = np.random.default_rng(9)
    B, N, T = 3, 50, 4
    coords = rng.uniform(-5, 5, (B, N, 3)).astype(np.float32)
    types = rng.integers(-1, T, (B, N)).astype(np.float32)
    radii = rng.uniform(1, 2, (B, N)).astype(np.float32)
    centers = rng.uniform(-1, 1, (B, 3)).astype(np.float32)
    gm = mg.GridMaker(0.5, 9.5)
    out = torch.empty((B,) + gm.grid_dimensions(T), device="cuda")
    gm.forward(dev(centers), dev(coords), dev(types), dev(radii), out)
    for b in range(B):
        one = torch.empty(gm.grid_dimensions(T), device="cuda")
        gm.forward(tuple(centers[b]), dev(coords[b]), dev(types[b]), dev(radii[b]), one)
        assert torch.equal(one, out[b])
        ref = oracle.GridMaker(0.5, 9.5).forward(centers[b], coords[b], types[b], radii[b], T)
        assert_close(one.cpu().numpy(), ref, what="padded batch")


def test_host_arrays_round_trip(mg):
    """numpy in, numpy out: staged through the device, same kernel."""
    rng = np.random.default_rng(2)
    coords, types, radii = synth.small_index_case(rng, 30, 3, 4.0, frac_ignored=0)
    gm = mg.GridMaker(0.5, 7.5)
    out = np.empty(gm.grid_dimensions(3), np.float32)
    gm.forward((0, 0, 0), coords, types, radii, out)
    ref = oracle.GridMaker(0.5, 7.5).forward((0, 0, 0), coords, types, radii, 3)
    assert_close(out, ref, what="host arrays")
    with pytest.raises(IndexError):     # the CPU overload throws for type >= ntypes
        gm.forward((0, 0, 0), coords, types + 5, radii, out)


def test_repeat_runs_are_bit_identical(mg):
    c = synth.config1(nbatch=2)
    gm = mg.GridMaker(0.5, 23.5)
    args = (c["offsets"], c["centers"], dev(c["coords"]), dev(c["types"]), dev(c["radii"]))
    a = torch.empty((2,) + gm.grid_dimensions(28), device="cuda")
    b = torch.empty_like(a)
    gm.forward_batch(*args, a)
    gm.forward_batch(*args, b)
    assert torch.equal(a, b)


def test_more_channels_than_the_channel_sort_handles(mg):
    """70 channels: more than one wave's worth of channels per territory at the default split."""
    rng = np.random.default_rng(70)
    coords, types, radii = synth.small_index_case(rng, 400, 70, 8.0)
    for binary in (False, True):
        ref = oracle.GridMaker(0.5, 11.5, binary).forward((0, 0, 0), coords, types, radii, 70)
        got = gpu_forward(mg, (0.5, 11.5, binary), (0, 0, 0), coords, types, radii, 70)
        if binary:
            assert np.array_equal(got, ref)
        else:
            assert_close(got, ref, what="70 channels")


def test_library_workspace_and_callers_workspace_give_the_same_grid(mg):
    """mg_forward_index (workspace kept by the library, grown on demand) and mg_forward_index_ws
    (workspace passed in) run the same launches: identical grids, dense and binary, for a small
    call followed by a larger one (the library's workspace grows) and a small one again."""
    import ctypes
    from libmolgrid_amd import _capi
    lib = _capi.lib
    rng = np.random.default_rng(5)
    for natoms in (40, 900, 60):
        coords, types, radii = synth.small_index_case(rng, natoms, 28, 14.0)
        dc, dt, dr = dev(coords), dev(types), dev(radii)
        for binary in (False, True):
            gm = mg.GridMaker(0.5, 23.5, binary)
            shape = gm.grid_dimensions(28)
            a = torch.full(shape, 3.0, device="cuda")
            b = torch.full(shape, 5.0, device="cuda")
            center = _capi.f3((0.3, -0.2, 0.1))
            need = lib.mg_forward_index_workspace_size(gm._p, 1, natoms, 28)
            assert need > 0
            ws = torch.empty(need, dtype=torch.uint8, device="cuda")
            stream = torch.cuda.current_stream().cuda_stream
            assert lib.mg_forward_index_ws(gm._p, 1, None, natoms, None, center, dc.data_ptr(),
                                           dt.data_ptr(), dr.data_ptr(), 28, a.data_ptr(),
                                           ws.data_ptr(), need, stream) == 0
            assert lib.mg_forward_index(gm._p, 1, None, natoms, None, center, dc.data_ptr(),
                                        dt.data_ptr(), dr.data_ptr(), 28, b.data_ptr(), stream) == 0
            torch.cuda.synchronize()
            assert torch.equal(a, b)
            ref = oracle.GridMaker(0.5, 23.5, binary).forward((0.3, -0.2, 0.1), coords, types, radii, 28)
            if binary:
                assert np.array_equal(b.cpu().numpy(), ref)
            else:
                assert_close(b.cpu().numpy(), ref, what="library workspace")
            # a workspace that is too small is refused, nothing is launched
            assert lib.mg_forward_index_ws(gm._p, 1, None, natoms, None, center, dc.data_ptr(),
                                           dt.data_ptr(), dr.data_ptr(), 28, a.data_ptr(),
                                           ws.data_ptr(), need - 1, stream) == _capi.MG_ERR_INVALID_ARGUMENT


def test_more_atoms_than_sixteen_bit_indices(mg):
    """70,000 atoms in one example (more than the sort keeps in registers: it then reads the
    atoms once per pass), most of them far from the grid; dense and binary."""
    rng = np.random.default_rng(77)
    coords, types, radii = synth.small_index_case(rng, 70000, 4, 30.0)
    for binary in (False, True):
        ref = oracle.GridMaker(0.5, 11.5, binary).forward((1.0, -2.0, 0.5), coords, types, radii, 4)
        got = gpu_forward(mg, (0.5, 11.5, binary), (1.0, -2.0, 0.5), coords, types, radii, 4)
        if binary:
            assert np.array_equal(got, ref)
        else:
            assert_close(got, ref, what="70,000 atoms")
    assert ref.sum() > 100

