"""Double precision arrays at the boundary (the reference's Grid<double, ...> overloads and
torch.[cuda.]DoubleTensor, python/bindings_grids.cpp:108-116; src/grid_maker.cu:293-294, 445-446,
600; src/transform.cu:96): the arithmetic is float as in the reference, so a double array holds the
float result widened -- compared here with the oracle cast to double, and with the float call."""
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


def case(seed=31, natoms=120, ntypes=5):
    rng = np.random.default_rng(seed)
    return synth.small_index_case(rng, natoms, ntypes, 5.0)


@pytest.mark.parametrize("binary", [False, True])
def test_forward_index_into_double_grids(mg, binary):
    coords, types, radii = case()
    gm = mg.GridMaker(0.5, 9.5, binary)
    ref = oracle.GridMaker(0.5, 9.5, binary).forward((0.2, 0, -0.1), coords, types, radii, 5)
    f32 = torch.empty(gm.grid_dimensions(5), device="cuda")
    f64 = torch.full(gm.grid_dimensions(5), 9.0, device="cuda", dtype=torch.float64)
    host64 = np.full(gm.grid_dimensions(5), 9.0, np.float64)
    for out in (f32, f64, host64):
        gm.forward((0.2, 0, -0.1), dev(coords), dev(types), dev(radii), out)
    assert torch.equal(f64, f32.double())
    assert np.array_equal(host64, f64.cpu().numpy())
    if binary:
        assert np.array_equal(f64.cpu().numpy(), ref.astype(np.float64))
    else:
        assert_close(f64.cpu().numpy(), ref.astype(np.float64), what="double grid")


def test_forward_vector_and_batches_into_double_grids(mg):
    rng = np.random.default_rng(32)
    coords, types, radii = case(32)
    tv = rng.uniform(0, 1, (len(coords), 5)).astype(np.float32)
    gm = mg.GridMaker(0.5, 9.5)
    ref = oracle.GridMaker(0.5, 9.5).forward((0, 0, 0), coords, tv, radii)
    out = torch.empty(gm.grid_dimensions(5), device="cuda", dtype=torch.float64)
    gm.forward((0, 0, 0), dev(coords), dev(tv), dev(radii), out)
    assert_close(out.cpu().numpy(), ref.astype(np.float64), what="double grid, vector types")
    # ragged batch and padded batch
    off = np.asarray([0, 50, 120])
    centers = np.asarray([[0, 0, 0], [0.5, -0.5, 0.25]], np.float32)
    b64 = torch.empty((2,) + gm.grid_dimensions(5), device="cuda", dtype=torch.float64)
    b32 = torch.empty((2,) + gm.grid_dimensions(5), device="cuda")
    for o in (b64, b32):
        gm.forward_batch(off, centers, dev(coords), dev(types), dev(radii), o)
    assert torch.equal(b64, b32.double())
    p64 = torch.empty((2,) + gm.grid_dimensions(5), device="cuda", dtype=torch.float64)
    p32 = torch.empty((2,) + gm.grid_dimensions(5), device="cuda")
    pc, pt, pr = dev(coords[:100].reshape(2, 50, 3)), dev(types[:100].reshape(2, 50)), dev(radii[:100].reshape(2, 50))
    for o in (p64, p32):
        gm.forward(dev(centers), pc, pt, pr, o)
    assert torch.equal(p64, p32.double())


def test_backward_with_double_gradients(mg):
    coords, types, radii = case(33)
    gm = mg.GridMaker(0.5, 9.5)
    og = oracle.GridMaker(0.5, 9.5)
    rng = np.random.default_rng(33)
    diff = rng.standard_normal(gm.grid_dimensions(5)).astype(np.float32)
    g32 = torch.empty((len(coords), 3), device="cuda")
    g64 = torch.full((len(coords), 3), 9.0, device="cuda", dtype=torch.float64)
    gm.backward((0, 0, 0), dev(coords), dev(types), dev(radii), dev(diff), g32)
    gm.backward((0, 0, 0), dev(coords), dev(types), dev(radii), dev(diff).double(), g64)
    assert torch.equal(g64, g32.double())
    ref = og.backward((0, 0, 0), coords, types, radii, diff, f64=True)
    np.testing.assert_allclose(g64.cpu().numpy(), ref, rtol=1e-4, atol=1e-4)
    # host float64 arrays
    h64 = np.empty((len(coords), 3), np.float64)
    gm.backward((0, 0, 0), coords, types, radii, diff.astype(np.float64), h64)
    assert np.array_equal(h64, g64.cpu().numpy())
    # vector types: type gradients too
    tv = rng.uniform(0, 1, (len(coords), 5)).astype(np.float32)
    a32, t32 = torch.empty((len(coords), 3), device="cuda"), torch.empty((len(coords), 5), device="cuda")
    a64, t64 = a32.double(), t32.double()
    gm.backward((0, 0, 0), dev(coords), dev(tv), dev(radii), dev(diff), a32, t32)
    gm.backward((0, 0, 0), dev(coords), dev(tv), dev(radii), dev(diff).double(), a64, t64)
    assert torch.equal(a64, a32.double()) and torch.equal(t64, t32.double())


def test_transform_on_double_coordinates(mg):
    rng = np.random.default_rng(34)
    pts = rng.uniform(-5, 5, (40, 3)).astype(np.float32)
    q = rng.normal(size=4)
    q = (q / np.linalg.norm(q)).astype(np.float32)
    T = mg.Transform(mg.Quaternion(*q), (1, 0, -1), (0.5, 2, -3))
    ref = oracle.transform_forward(q, np.asarray([1, 0, -1], np.float32),
                                   np.asarray([0.5, 2, -3], np.float32), pts)
    d64 = dev(pts).double()
    out64 = torch.empty_like(d64)
    T.forward(d64, out64)
    assert np.array_equal(out64.cpu().numpy(), ref.astype(np.float64))
    T.forward(d64, d64)                       # in place
    assert torch.equal(d64, out64)
    T.backward(d64, d64)
    np.testing.assert_allclose(d64.cpu().numpy(), pts, atol=2e-5)


def test_dtypes_that_the_reference_does_not_take_are_refused(mg):
    coords, types, radii = case(35)
    gm = mg.GridMaker(0.5, 9.5)
    with pytest.raises(ValueError):
        gm.forward((0, 0, 0), dev(coords), dev(types), dev(radii),
                   torch.empty(gm.grid_dimensions(5), device="cuda", dtype=torch.float16))
    with pytest.raises(ValueError):      # coordinates of a gridding call are float in the reference
        gm.forward((0, 0, 0), dev(coords).double(), dev(types), dev(radii),
                   torch.empty(gm.grid_dimensions(5), device="cuda"))
