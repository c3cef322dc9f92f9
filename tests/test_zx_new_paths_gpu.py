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
