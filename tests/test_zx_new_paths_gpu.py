"""GPU tests of the paths added after the last GPU run of this repository (the paged write-out of
the forward splat, the sort and splat launches as calls of their own, the per-slab atom lists of the
vector forward pass).  They are verified on the CPU under emulation (tests/emu); this file is
collected late so that, should one of them fail on real hardware, the tests of the established
paths have already reported."""
import numpy as np
import pytest
import torch

import oracle
import synth
from test_forward_gpu import gpu_forward
from util import assert_close, dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mg():
    import libmolgrid_amd
    return libmolgrid_amd


@pytest.fixture(scope="module")
def workload():
    c = synth.config1(nbatch=50)
    c["moved"] = oracle.transform_forward_batch(c["offsets"], c["quats"], c["centers"],
                                                c["translations"], c["coords"])
    return c


@pytest.mark.parametrize("binary", [False, True])
def test_sort_and_splat_on_two_streams_equal_forward_batch(mg, binary):
    """mg_forward_index_sort on a side stream, mg_forward_index_splat on the main one after an
    event: the grids of forward_batch, bit for bit."""
    c = synth.config1(nbatch=6)
    gm = mg.GridMaker(0.5, 23.5, binary)
    batch = mg.AtomBatch(c["offsets"])
    coords, types, radii, centers = [dev(c[k]) for k in ("coords", "types", "radii", "centers")]
    whole = torch.full((6,) + gm.grid_dimensions(28), 7.0, device="cuda")
    gm.forward_batch(batch, centers, coords, types, radii, whole)
    split = torch.full_like(whole, 7.0)
    side, main = torch.cuda.Stream(), torch.cuda.current_stream()
    ready, sorted_done = torch.cuda.Event(), torch.cuda.Event()
    ready.record(main)
    side.wait_event(ready)
    with torch.cuda.stream(side):
        sb = gm.sort_batch(batch, centers, coords, types, radii, 28)
        sorted_done.record(side)
    main.wait_event(sorted_done)
    gm.splat_batch(sb, split)
    torch.cuda.synchronize()
    assert torch.equal(split, whole)
    with pytest.raises(ValueError):
        gm.splat_batch(sb, torch.empty((5,) + gm.grid_dimensions(28), device="cuda"))


@pytest.mark.parametrize("binary", [False, True])
@pytest.mark.parametrize("res,dimension,ntypes,natoms", [
    (0.5, 23.5, 28, 300), (1.0, 15.0, 40, 200), (0.25, 5.75, 2, 15), (0.5, 3.5, 3, 12)])
def test_paged_write_out_gives_the_same_grids(mg, res, dimension, ntypes, natoms, binary):
    """The write-out in whole 4 KB pages (mg_forward_index_paged) against the per-wave one, bit for
    bit, and against the oracle."""
    from libmolgrid_amd import _capi
    rng = np.random.default_rng(31 + natoms)
    coords, types, radii = synth.small_index_case(rng, natoms, ntypes, dimension / 2 + 2.0)
    center = rng.uniform(-1, 1, 3).astype(np.float32)
    ref = oracle.GridMaker(res, dimension, binary).forward(center, coords, types, radii, ntypes)
    before = _capi.lib.mg_forward_index_paged(0)
    try:
        plain = gpu_forward(mg, (res, dimension, binary), center, coords, types, radii, ntypes)
        _capi.lib.mg_forward_index_paged(1)
        paged = gpu_forward(mg, (res, dimension, binary), center, coords, types, radii, ntypes)
    finally:
        _capi.lib.mg_forward_index_paged(before)
    assert np.array_equal(paged, plain)
    if binary:
        assert np.array_equal(paged, ref)
    else:
        assert_close(paged, ref, what="paged forward")


@pytest.mark.parametrize("binary", [False, True])
def test_paged_write_out_full_batch(mg, workload, binary):
    """The whole benchmark batch through the write-out in 4 KB pages: the grids of the per-wave
    write-out, bit for bit (which test_forward_every_example holds against the oracle)."""
    from libmolgrid_amd import _capi
    c = workload
    B = len(c["offsets"]) - 1
    gm = mg.GridMaker(0.5, 23.5, binary)
    batch = mg.AtomBatch(c["offsets"])
    moved, types, radii, centers = dev(c["moved"]), dev(c["types"]), dev(c["radii"]), dev(c["centers"])
    plain = torch.full((B,) + gm.grid_dimensions(28), -1.0, device="cuda")
    paged = torch.full_like(plain, -2.0)
    before = _capi.lib.mg_forward_index_paged(0)
    try:
        gm.forward_batch(batch, centers, moved, types, radii, plain)
        _capi.lib.mg_forward_index_paged(1)
        gm.forward_batch(batch, centers, moved, types, radii, paged)
    finally:
        _capi.lib.mg_forward_index_paged(before)
    torch.cuda.synchronize()
    assert torch.equal(paged, plain)


def test_tail_only_blocks_without_the_exponential_give_the_same_grids(mg, workload):
    """mg_forward_index_core_skip(1): the kernel instances whose cull marks the blocks that the
    Gaussian core of an atom can reach and that skip the exponential elsewhere, with either
    write-out, on ten examples of the benchmark batch: the default instance's grids bit for bit."""
    from libmolgrid_amd import _capi
    c = workload
    B = 10
    off = c["offsets"][:B + 1]
    n = int(off[-1])
    gm = mg.GridMaker(0.5, 23.5)
    batch = mg.AtomBatch(off)
    cen, moved, types, radii = dev(c["centers"][:B]), dev(c["moved"][:n]), dev(c["types"][:n]), dev(c["radii"][:n])
    plain = torch.full((B,) + gm.grid_dimensions(28), 7.0, device="cuda")
    gm.forward_batch(batch, cen, moved, types, radii, plain)
    try:
        for paged in (0, 1):
            _capi.lib.mg_forward_index_paged(paged)
            _capi.lib.mg_forward_index_core_skip(1)
            other = torch.full_like(plain, 6.0)
            gm.forward_batch(batch, cen, moved, types, radii, other)
            torch.cuda.synchronize()
            assert torch.equal(other, plain), "paged=%d" % paged
    finally:
        _capi.lib.mg_forward_index_paged(0)
        _capi.lib.mg_forward_index_core_skip(0)


@pytest.mark.parametrize("binary", [False, True])
def test_atom_lists_give_the_same_grids(mg, binary):
    """mg_forward_vector_ws with its workspace (a launch before the splat lists the atoms that can
    reach each slab of four x planes) against mg_forward_vector without: bit for bit, on a ragged
    batch at the benchmark's resolution."""
    import ctypes
    from libmolgrid_amd import _capi
    v = synth.vector_batch(nbatch=3, natoms=1200)
    gm = mg.GridMaker(0.25, 23.75, binary)
    off = torch.as_tensor(v["offsets"].astype(np.int32)).cuda()
    cen, c, t, r = [dev(v[k]) for k in ("centers", "coords", "types", "radii")]
    shape = (3,) + gm.grid_dimensions(28)
    plain = torch.full(shape, 5.0, device="cuda")
    listed = torch.full(shape, 6.0, device="cuda")
    args = [gm._p, 3, off.data_ptr(), 1200, cen.data_ptr(), _capi.f3((0, 0, 0)), c.data_ptr(),
            t.data_ptr(), r.data_ptr(), 28]
    assert _capi.lib.mg_forward_vector(*args, plain.data_ptr(), None) == 0
    need = int(_capi.lib.mg_forward_vector_workspace_size(gm._p, 3, 1200, 28))
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    assert _capi.lib.mg_forward_vector_ws(*args, listed.data_ptr(), ws.data_ptr(), need, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(listed, plain)
    # the Python layer takes the workspace path
    out = torch.full(shape, 7.0, device="cuda")
    gm.forward_batch(v["offsets"], cen, c, t, r, out)
    assert torch.equal(out, plain)


@pytest.mark.parametrize("binary", [False, True])
def test_atom_lists_longer_than_one_scan_window(mg, binary):
    """9,000 atoms crowded into a grid of 8 voxels a side: every slab's list holds nearly all of
    them, more than the splat kernel scans in one window and more than a wave's segment of
    candidates holds, so the list is taken window by window (a quarter of a window per wave).  The
    grids with lists equal those without, bit for bit, and the oracle's."""
    from libmolgrid_amd import _capi
    rng = np.random.default_rng(77)
    n, T = 9000, 3
    coords = rng.uniform(-4.5, 4.5, (n, 3)).astype(np.float32)
    tv = (rng.uniform(0, 1.5, (n, T)) * (rng.random((n, T)) > 0.3)).astype(np.float32)
    radii = rng.uniform(0.6, 2.2, n).astype(np.float32)
    gm_args = (1.0, 7.0, binary)
    gm = mg.GridMaker(*gm_args)
    c, t, r = dev(coords), dev(tv), dev(radii)
    shape = gm.grid_dimensions(T)
    plain, listed = torch.full(shape, 5.0, device="cuda"), torch.full(shape, 6.0, device="cuda")
    args = [gm._p, 1, None, n, None, _capi.f3((0.3, 0, -0.2)), c.data_ptr(), t.data_ptr(), r.data_ptr(), T]
    assert _capi.lib.mg_forward_vector(*args, plain.data_ptr(), None) == 0
    need = int(_capi.lib.mg_forward_vector_workspace_size(gm._p, 1, n, T))
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    assert _capi.lib.mg_forward_vector_ws(*args, listed.data_ptr(), ws.data_ptr(), need, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(listed, plain)
    ref = oracle.GridMaker(*gm_args).forward((0.3, 0, -0.2), coords, tv, radii)
    if binary:
        assert np.array_equal(listed.cpu().numpy(), ref)
    else:
        assert_close(listed.cpu().numpy(), ref, what="9,000 atoms in 8^3 voxels")


def _atoms_on_voxel_centres(res, dim, radius):
    """Atoms on voxel centres of a grid centred at the origin: in the middle, at a face, at a corner."""
    half = (dim - 1) * res / 2
    idx = np.array([[dim // 2, dim // 2, dim // 2], [dim // 2, dim - 1, dim // 2 - 1], [0, 0, dim - 1],
                    [dim // 2 - 3, dim // 2 + 2, 3]], np.float32)
    coords = (idx * res - half).astype(np.float32)
    return coords, np.full(len(coords), radius, np.float32)


def test_truncated_gaussian_with_voxels_on_the_cut_off(mg):
    """A Gaussian cut off without a tail (negative radius multiple) jumps at its cut-off.  With atoms
    on voxel centres and a cut-off of exactly five voxels there are 30 voxels ON it per atom: the
    reference counts those that its index box holds (the one at +5 voxels on an axis is outside,
    src/grid_maker.cu:66-79) by sqrtf(dist^2) > cut.  Forward, backward (index and vector types) and
    relevance must agree with the oracle there, which squares and a symmetric range do not."""
    res, dim, T = 0.5, 32, 3
    gm_args = (res, (dim - 1) * res, False, False, 1.0, -1.0)
    coords, radii = _atoms_on_voxel_centres(res, dim, 2.5)
    types = np.array([0, 1, 2, 1], np.float32)
    og = oracle.GridMaker(*gm_args)
    ref = og.forward((0, 0, 0), coords, types, radii, T)
    got = gpu_forward(mg, gm_args, (0, 0, 0), coords, types, radii, T)
    assert_close(got, ref, what="truncated Gaussian, forward")
    rng = np.random.default_rng(3)
    diff = rng.standard_normal(ref.shape).astype(np.float32)
    gm = mg.GridMaker(*gm_args)
    grads = torch.empty((len(coords), 3), device="cuda")
    gm.backward((0, 0, 0), dev(coords), dev(types), dev(radii), dev(diff), grads)
    ref32 = og.backward((0, 0, 0), coords, types, radii, diff)
    ref64 = og.backward((0, 0, 0), coords, types, radii, diff, f64=True)
    from test_backward_gpu import check_grads, noise_bound
    check_grads(grads.cpu().numpy(), ref32, ref64,
                noise_bound(og, (0, 0, 0), coords, types, radii, diff) + 1.0, "truncated Gaussian, backward")
    # vector types: the same atoms with two-channel weights
    tv = rng.uniform(0.2, 1.0, (len(coords), T)).astype(np.float32)
    vgot = torch.empty(gm.grid_dimensions(T), device="cuda")
    gm.forward((0, 0, 0), dev(coords), dev(tv), dev(radii), vgot)
    assert_close(vgot.cpu().numpy(), og.forward((0, 0, 0), coords, tv, radii), what="truncated, vector forward")
    ag, tg = torch.empty((len(coords), 3), device="cuda"), torch.empty((len(coords), T), device="cuda")
    gm.backward((0, 0, 0), dev(coords), dev(tv), dev(radii), dev(diff), ag, tg)
    ra, rt = og.backward((0, 0, 0), coords, tv, radii, diff, f64=True)
    assert np.allclose(ag.cpu().numpy(), ra, rtol=1e-4, atol=1e-4), np.abs(ag.cpu().numpy() - ra).max()
    assert np.allclose(tg.cpu().numpy(), rt, rtol=1e-4, atol=1e-4), np.abs(tg.cpu().numpy() - rt).max()
    rel = torch.empty(len(coords), device="cuda")
    gm.backward_relevance((0, 0, 0), dev(coords), dev(types), dev(radii), dev(ref), dev(diff), rel)
    rref = og.backward_relevance((0, 0, 0), coords, types, radii, ref, diff)
    assert np.allclose(rel.cpu().numpy(), rref, rtol=1e-4, atol=1e-4), np.abs(rel.cpu().numpy() - rref).max()


@pytest.mark.parametrize("scale", [1.0, 1.3])
def test_binary_sphere_that_coincides_with_its_index_box(mg, scale):
    """Binary density with a final radius multiple of exactly one: the reference's index box has
    the sphere's own radius, and voxels within rounding of the surface are decided by the rounding
    of the box's edges.  Atoms on voxel centres with radii that put voxels on the surface, to the
    last bit and one bit either side; bit-exact against the oracle, index and vector types."""
    res, dim, T = 0.5, 24, 2
    gm_args = (res, (dim - 1) * res, True, False, scale, -1.0)
    coords, _ = _atoms_on_voxel_centres(res, dim, 1.0)
    base = np.float32(2.5 / scale)
    radii = np.array([base, np.nextafter(base, np.float32(9)), np.nextafter(base, np.float32(0)), base], np.float32)
    types = np.array([0, 1, 0, 1], np.float32)
    og = oracle.GridMaker(*gm_args)
    got = gpu_forward(mg, gm_args, (0, 0, 0), coords, types, radii, T)
    assert np.array_equal(got, og.forward((0, 0, 0), coords, types, radii, T))
    tv = np.array([[1, 0.5], [0.25, 1], [1, 1], [0, 2]], np.float32)
    gm = mg.GridMaker(*gm_args)
    vgot = torch.empty(gm.grid_dimensions(T), device="cuda")
    gm.forward((0, 0, 0), dev(coords), dev(tv), dev(radii), vgot)
    assert np.array_equal(vgot.cpu().numpy(), og.forward((0, 0, 0), coords, tv, radii))


def test_relevance_with_voxels_at_the_end_of_the_tail(mg):
    """Relevance divides an atom's density by the grid's.  With atoms on voxel centres, five voxels
    apart, and a final radius of exactly five voxels, the voxel at +5 on an axis sits at the very
    end of the quadratic tail, where the atom's density is next to nothing -- and so is the
    grid's, so the quotient is not small.  The reference's index box leaves that voxel out
    (src/grid_maker.cu:66-79); so must the kernel."""
    res, dim, T, steps = 0.5, 24, 2, 5
    gm_args = (res, (dim - 1) * res, False, False, 1.0, 0.7)
    og = oracle.GridMaker(*gm_args)
    half = (dim - 1) * res / 2
    m = dim // 2
    idx = np.array([[m, m, m], [m - steps, m, m], [m, m + steps, m], [3, 4, 5]], np.float32)
    coords = (idx * res - half).astype(np.float32)
    for nudge in (0, 1):
        r = np.float32(steps * res / float(og.p.final_radius_multiple))
        if nudge:
            r = np.nextafter(r, np.float32(9))
        radii = np.full(4, r, np.float32)
        types = np.array([0, 0, 0, 1], np.float32)
        dens = og.forward((0, 0, 0), coords, types, radii, T)
        diff = np.random.default_rng(9).standard_normal(dens.shape).astype(np.float32)
        gm = mg.GridMaker(*gm_args)
        rel = torch.empty(len(coords), device="cuda")
        gm.backward_relevance((0, 0, 0), dev(coords), dev(types), dev(radii), dev(dens), dev(diff), rel)
        ref = og.backward_relevance((0, 0, 0), coords, types, radii, dens, diff)
        scale = og.backward_relevance((0, 0, 0), coords, types, radii, dens, np.abs(diff))
        eps = float(np.finfo(np.float32).eps)
        assert (np.abs(rel.cpu().numpy() - ref) <= 1e-6 + 1e-5 * np.abs(ref) + 64 * eps * scale).all(), \
            (nudge, rel.cpu().numpy(), ref)
