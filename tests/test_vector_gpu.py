"""GPU parity of the vector-typed forward/backward (through the C ABI) against the oracle."""
import numpy as np
import pytest
import torch

import oracle
import synth
from util import ATOL, RTOL, assert_close, dev

pytestmark = pytest.mark.gpu
EPS = float(np.finfo(np.float32).eps)


@pytest.fixture(scope="module")
def mg():
    import libmolgrid_amd
    return libmolgrid_amd


def make_case(rng, natoms, ntypes, extent, sparse=0.5):
    coords = rng.uniform(-extent, extent, (natoms, 3)).astype(np.float32)
    tv = rng.dirichlet(np.full(ntypes, 0.3), natoms) * rng.uniform(0.5, 1.5, (natoms, 1))
    tv = (tv * (rng.random((natoms, ntypes)) > sparse)).astype(np.float32)   # exact zeros too
    radii = rng.uniform(0.8, 2.0, natoms).astype(np.float32)
    return coords, tv, radii


@pytest.mark.parametrize("ntypes", [2, 8, 14, 28, 32, 37])
@pytest.mark.parametrize("binary", [False, True])
def test_forward_small_vs_oracle(mg, ntypes, binary):
    rng = np.random.default_rng(100 + ntypes)
    coords, tv, radii = make_case(rng, 60, ntypes, 7.0)
    ref = oracle.GridMaker(0.5, 11.5, binary).forward((0.2, -0.1, 0), coords, tv, radii)
    gm = mg.GridMaker(0.5, 11.5, binary)
    out = torch.full(gm.grid_dimensions(ntypes), 3.0, device="cuda")
    gm.forward((0.2, -0.1, 0), dev(coords), dev(tv), dev(radii), out)
    if binary:
        assert np.array_equal(out.cpu().numpy(), ref)     # sums of weights in atom order
    else:
        assert_close(out.cpu().numpy(), ref, what="vector forward")


@pytest.mark.parametrize("gm_args", [
    (0.5, 11.5, False, False, 1.0, -1.5),   # truncated Gaussian, no quadratic tail
    (0.5, 11.5, True, False, 1.0, -0.5),    # binary sphere wider than its index box
    (0.5, 11.5, False, False, 1.3, 0.7),    # radius scale + early quadratic
])
def test_forward_unusual_radius_multiples(mg, gm_args):
    """The modes that evaluate the reference's own cut-off predicates, with vector types."""
    rng = np.random.default_rng(11)
    coords, tv, radii = make_case(rng, 70, 5, 7.0)
    ref = oracle.GridMaker(*gm_args).forward((0, 0.1, 0), coords, tv, radii)
    gm = mg.GridMaker(*gm_args)
    out = torch.full(gm.grid_dimensions(5), -1.0, device="cuda")
    gm.forward((0, 0.1, 0), dev(coords), dev(tv), dev(radii), out)
    if gm_args[2]:
        assert np.array_equal(out.cpu().numpy(), ref)
    else:
        assert_close(out.cpu().numpy(), ref, what="vector forward, exact predicates")


@pytest.mark.parametrize("binary", [False, True])
def test_forward_type_indexed_radii(mg, binary):
    rng = np.random.default_rng(7)
    T = 6
    coords, tv, _ = make_case(rng, 50, T, 6.0)
    tradii = rng.uniform(0.8, 2.0, T).astype(np.float32)
    ref = oracle.GridMaker(0.5, 9.5, binary, True).forward((0, 0, 0), coords, tv, tradii)
    gm = mg.GridMaker(0.5, 9.5, binary, True)
    out = torch.empty(gm.grid_dimensions(T), device="cuda")
    gm.forward((0, 0, 0), dev(coords), dev(tv), dev(tradii), out)
    if binary:
        assert np.array_equal(out.cpu().numpy(), ref)
    else:
        assert_close(out.cpu().numpy(), ref, what="type-indexed radii")


def test_one_hot_equals_index_and_half_weight(mg):
    """test/test_gridmaker.py:217-256."""
    gm = mg.GridMaker(0.25, 6.0)
    c = dev(np.asarray([[0, 0, 0], [2, 0, 0]], np.float32))
    r = dev(np.ones(2, np.float32))
    shape = gm.grid_dimensions(2)
    ref, v1, v2 = (torch.empty(shape, device="cuda") for _ in range(3))
    gm.forward((0, 0, 0), c, dev(np.asarray([0, 1], np.float32)), r, ref)
    gm.forward((0, 0, 0), c, dev(np.eye(2, dtype=np.float32)), r, v1)
    gm.forward((0, 0, 0), c, dev(0.5 * np.eye(2, dtype=np.float32)), r, v2)
    np.testing.assert_allclose(ref.cpu().numpy(), v1.cpu().numpy(), atol=1e-6)
    np.testing.assert_allclose(ref.cpu().numpy(), 2 * v2.cpu().numpy(), atol=1e-6)
    assert float(v2.max()) == pytest.approx(0.5)


@pytest.mark.parametrize("binary", [False, True])
def test_config3_shape_vs_oracle(mg, binary):
    """Configuration 3 (96^3, 28 soft types) on fewer atoms/examples than the bench."""
    v = synth.vector_batch(nbatch=2, natoms=1500)
    ref = oracle.GridMaker(0.25, 23.75, binary).forward_batch(
        v["offsets"], v["centers"], v["coords"], v["types"], v["radii"], 28, nthreads=2)
    gm = mg.GridMaker(0.25, 23.75, binary)
    out = torch.empty((2,) + gm.grid_dimensions(28), device="cuda")
    gm.forward_batch(v["offsets"], v["centers"], dev(v["coords"]), dev(v["types"]),
                     dev(v["radii"]), out)
    if binary:
        assert np.array_equal(out.cpu().numpy(), ref)
    else:
        assert_close(out.cpu().numpy(), ref, what="config 3")


def test_matrix_core_kernel_dense_cases(mg):
    """Vector-typed atoms on the matrix cores (four atoms per multiply-accumulate step) against the
    oracle's atom-by-atom sums -- to the stated tolerance for densities, bit for bit for binary
    occupancy: a dense case, more than 32 channels and a grid with partial columns."""
    rng = np.random.default_rng(8)
    for natoms, ntypes, gm_args in ((2500, 28, (0.5, 11.5)), (300, 37, (0.5, 6.0))):
        coords, tv, radii = make_case(rng, natoms, ntypes, gm_args[1] / 2 + 1.0)
        for binary in (False, True):
            gm = mg.GridMaker(gm_args[0], gm_args[1], binary)
            shape = gm.grid_dimensions(ntypes)
            a = torch.full(shape, 7.0, device="cuda")
            gm.forward((0, 0, 0), dev(coords), dev(tv), dev(radii), a)
            ref = oracle.GridMaker(gm_args[0], gm_args[1], binary).forward((0, 0, 0), coords, tv, radii)
            if binary:
                assert np.array_equal(a.cpu().numpy(), ref)
            else:
                assert_close(a.cpu().numpy(), ref, what="matrix-core kernel")
            assert not np.isnan(a.cpu().numpy()).any()


@pytest.mark.parametrize("ntypes,binary,rti", [(3, False, False), (28, False, False),
                                               (37, False, False), (5, True, False),
                                               (6, False, True), (6, True, True)])
def test_backward_vs_oracle(mg, ntypes, binary, rti):
    rng = np.random.default_rng(300 + ntypes)
    coords, tv, radii = make_case(rng, 40, ntypes, 6.0)
    if rti:
        radii = rng.uniform(0.8, 2.0, ntypes).astype(np.float32)
    og = oracle.GridMaker(0.5, 9.5, binary, rti)
    diff = rng.standard_normal(og.grid_shape(ntypes)).astype(np.float32)
    ra32, rt32 = og.backward((0, 0, 0), coords, tv, radii, diff)
    ra64, rt64 = og.backward((0, 0, 0), coords, tv, radii, diff, f64=True)
    ma, mt = og.backward((0, 0, 0), coords, np.abs(tv), radii, np.abs(diff), f64=True)
    ma = np.abs(ma).max(axis=1, keepdims=True) + 1e-30
    gm = mg.GridMaker(0.5, 9.5, binary, rti)
    ag = torch.full((40, 3), 9.0, device="cuda")
    tg = torch.full((40, ntypes), 9.0, device="cuda")
    gm.backward((0, 0, 0), dev(coords), dev(tv), dev(radii), dev(diff), ag, tg)
    ag, tg = ag.cpu().numpy().astype(np.float64), tg.cpu().numpy().astype(np.float64)
    assert (np.abs(ag - ra64) <= ATOL + RTOL * np.abs(ra64) + 16 * EPS * ma).all()
    assert (np.abs(ag - ra32) <= ATOL + RTOL * np.abs(ra32) + 64 * EPS * ma).all()
    assert (np.abs(tg - rt64) <= ATOL + RTOL * np.abs(rt64) + 16 * EPS * mt).all()
    assert (np.abs(tg - rt32) <= ATOL + RTOL * np.abs(rt32) + 64 * EPS * mt).all()


def test_type_gradient_is_density_dot_diff(mg):
    """Brute force: d(sum diff*grid)/d(weight[a,t]) = sum over voxels of density_a * diff_t."""
    rng = np.random.default_rng(12)
    coords, tv, radii = make_case(rng, 10, 3, 3.0, sparse=0.0)
    gm = mg.GridMaker(0.5, 7.5)
    diff = torch.randn(gm.grid_dimensions(3), device="cuda")
    ag = torch.empty((10, 3), device="cuda")
    tg = torch.empty((10, 3), device="cuda")
    gm.backward((0, 0, 0), dev(coords), dev(tv), dev(radii), diff, ag, tg)
    for a in range(10):
        one = torch.empty(gm.grid_dimensions(1), device="cuda")
        gm.forward((0, 0, 0), dev(coords[a:a + 1]), dev(np.zeros(1, np.float32)),
                   dev(radii[a:a + 1]), one)
        want = (one[0][None] * diff).sum(dim=(1, 2, 3)).cpu().numpy()
        np.testing.assert_allclose(tg[a].cpu().numpy(), want, rtol=1e-4, atol=1e-4)

