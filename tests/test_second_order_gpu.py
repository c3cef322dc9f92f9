"""GPU parity of atom relevance and of the gradients of the backward pass (through the C ABI)
against the oracle, plus the closed form the reference's own test asserts."""
import numpy as np
import pytest
import torch

import oracle
from util import dev

pytestmark = pytest.mark.gpu
EPS = float(np.finfo(np.float32).eps)


@pytest.fixture(scope="module")
def mg():
    import libmolgrid_amd
    return libmolgrid_amd


def close_sums(got, ref, scale, what):
    """|got - ref| <= 1e-6 + 1e-5 |ref| + 64 eps * (sum of |terms|): both sides add hundreds of
    float terms of either sign, in different orders."""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    tol = 1e-6 + 1e-5 * np.abs(ref) + 64 * EPS * np.asarray(scale, np.float64)
    bad = np.abs(got - ref) > tol
    assert not bad.any(), "%s: %d values off, worst %g (tol %g)" % (
        what, int(bad.sum()), np.abs(got - ref)[bad].max(), tol[bad].min())


def test_relevance_reference_case(mg):
    """test/test_gridmaker.cpp:313-337"""
    gm = mg.GridMaker(0.1, 6.0)
    d = gm.get_first_dim()
    diff = torch.zeros((1, d, d, d), device="cuda")
    dens = torch.zeros((1, d, d, d), device="cuda")
    diff[0, 31, 30, 30] = 10.0
    dens[0, 31, 30, 30] = 1.0
    rel = torch.full((1,), -7.0, device="cuda")
    gm.backward_relevance((0, 0, 0), dev(np.zeros((1, 3), np.float32)), dev(np.zeros(1, np.float32)),
                          dev(np.full(1, 2.0, np.float32)), dens, diff, rel)
    assert 1.0 < float(rel[0]) < 10.0
    assert float(rel[0]) == pytest.approx(10.0 * np.exp(-2 * 0.01 / 4.0), rel=1e-5)


@pytest.mark.parametrize("binary", [False, True])
def test_relevance_vs_oracle(mg, binary):
    rng = np.random.default_rng(31)
    n, T = 90, 5
    coords = rng.uniform(-6, 6, (n, 3)).astype(np.float32)
    types = rng.integers(0, T, n).astype(np.float32)
    types[::11] = -1
    radii = rng.uniform(0.9, 2.0, n).astype(np.float32)
    og = oracle.GridMaker(0.5, 11.5, binary)
    dens = og.forward((0.3, 0, -0.1), coords, types, radii, T)
    if binary:
        dens = dens * rng.uniform(0.5, 3.0, dens.shape).astype(np.float32)
    dens[1, 4:9] = 0
    diff = rng.standard_normal(dens.shape).astype(np.float32)
    ref = og.backward_relevance((0.3, 0, -0.1), coords, types, radii, dens, diff)
    scale = og.backward_relevance((0.3, 0, -0.1), coords, types, radii, dens, np.abs(diff))
    gm = mg.GridMaker(0.5, 11.5, binary)
    rel = torch.full((n,), 5.0, device="cuda")
    gm.backward_relevance((0.3, 0, -0.1), dev(coords), dev(types), dev(radii), dev(dens), dev(diff),
                          rel)
    close_sums(rel.cpu().numpy(), ref, scale, "relevance")
    assert not rel.cpu().numpy()[::11].any()
    # coordinate-set overload and host arrays
    out = np.full(n, 3.0, np.float32)
    gm.backward_relevance((0.3, 0, -0.1), mg.CoordinateSet(coords, types, radii, T), dens, diff, out)
    close_sums(out, ref, scale, "relevance (host arrays)")


@pytest.mark.parametrize("rti", [False, True])
@pytest.mark.parametrize("grm", [1.0, -1.5])
def test_backward_gradients_vs_oracle(mg, rti, grm):
    rng = np.random.default_rng(32)
    n, T = 40, 4
    coords = rng.uniform(-4, 4, (n, 3)).astype(np.float32)
    tv = rng.uniform(0, 1, (n, T)).astype(np.float32)
    tv[rng.random((n, T)) < 0.4] = 0
    radii = rng.uniform(1.0, 1.9, T if rti else n).astype(np.float32)
    og = oracle.GridMaker(0.5, 9.5, False, rti, 1.0, grm)
    diff = rng.standard_normal(og.grid_shape(T)).astype(np.float32)
    w = rng.standard_normal((n, 3)).astype(np.float32)
    v = rng.standard_normal((n, T)).astype(np.float32)
    dd, add, tdd = og.backward_gradients((0, 0.2, 0), coords, tv, radii, diff, w, v)
    # scales: the same sums over absolute values
    sdd, sadd, _ = og.backward_gradients((0, 0.2, 0), coords, tv, radii, np.abs(diff), np.abs(w),
                                         np.abs(v))
    sdd = np.abs(sdd) + 1.0
    sadd = np.abs(sadd) * 4 + 1.0
    gm = mg.GridMaker(0.5, 9.5, False, rti, 1.0, grm)
    g_dd = torch.full(diff.shape, 9.0, device="cuda")
    g_add = torch.full((n, 3), 9.0, device="cuda")
    g_tdd = torch.full((n, T), 9.0, device="cuda")
    gm.backward_gradients((0, 0.2, 0), dev(coords), dev(tv), dev(radii), dev(diff), dev(w), dev(v),
                          g_dd, g_add, g_tdd)
    assert not g_tdd.cpu().numpy().any()
    close_sums(g_dd.cpu().numpy(), dd, sdd, "diffdiff")
    close_sums(g_add.cpu().numpy(), add, sadd, "atom_diffdiff")
    # a second call overwrites (the scattered sums start from zero again)
    gm.backward_gradients((0, 0.2, 0), dev(coords), dev(tv), dev(radii), dev(diff), dev(w), dev(v),
                          g_dd, g_add, g_tdd)
    close_sums(g_dd.cpu().numpy(), dd, sdd, "diffdiff, second call")


def test_backward_gradients_rejects_binary(mg):
    gm = mg.GridMaker(0.5, 6.0, True)
    z = lambda *s: torch.zeros(s, device="cuda")
    with pytest.raises(ValueError):
        gm.backward_gradients((0, 0, 0), z(2, 3), z(2, 1), z(2), z(1, 13, 13, 13), z(2, 3), z(2, 1),
                              z(1, 13, 13, 13), z(2, 3), z(2, 1))


def test_double_backward_closed_form(mg):
    """test/test_gridmaker.py:439-487: gradient of |d(one voxel)/dcoords|^2 through autograd."""
    from libmolgrid_amd.torch_bindings import Coords2GridFunction
    gmaker = mg.GridMaker(resolution=0.5, dimension=6.0, gaussian_radius_multiple=-2.0)
    types = torch.ones(1, 1, device="cuda")
    radii = torch.ones(1, device="cuda")
    for i in range(3):
        for x in np.arange(-0.9, 3, .1):
            coords = torch.zeros(1, 3, device="cuda")
            coords[0][i] = x
            coords.requires_grad = True
            outgrid = Coords2GridFunction.apply(gmaker, (0, 0, 0), coords, types, radii)
            idx = [0, 6, 6, 6]
            idx[1 + i] = 8
            gp = outgrid[tuple(idx)]
            Lg = torch.autograd.grad(gp, coords, create_graph=True)[0]
            fancyL = torch.sum(Lg ** 2)
            val = float(torch.autograd.grad(fancyL, coords)[0][0][i])
            d = x - 1
            correct = -128 * d ** 3 * np.exp(-4 * d ** 2) + 32 * d * np.exp(-4 * d ** 2)
            assert val == pytest.approx(correct, abs=1e-4)
    # the diagonal is symmetric and decreasing at this range
    coords = torch.zeros(1, 3, device="cuda", requires_grad=True)
    outgrid = Coords2GridFunction.apply(gmaker, (0, 0, 0), coords, types, radii)
    fl = []
    for k in (7, 8):
        Lg = torch.autograd.grad(outgrid[0][k][k][k], coords, create_graph=True)[0]
        fl.append(torch.autograd.grad(torch.sum(Lg ** 2), coords, retain_graph=True)[0][0])
    for f in fl:
        assert float(f[0]) == pytest.approx(float(f[1]), abs=1e-6)
        assert float(f[2]) == pytest.approx(float(f[1]), abs=1e-6)
    assert float(fl[1][0]) < float(fl[0][0])
