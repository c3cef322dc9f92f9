"""Pins the CPU oracle to the reference's behaviour without a reference binary.

Every check is either a constant the reference's own tests assert, a special case
that reduces to a textbook or library routine (rotation matrix, scipy's trilinear
interpolator), an invariant (linearity, forward o backward = identity, finite
difference of the forward pass) or a brute-force evaluation over every voxel that
shares no loop structure with the oracle.
"""
import numpy as np
import pytest
from scipy.interpolate import RegularGridInterpolator

import oracle
from util import rot_matrix

E2 = np.exp(-2.0)


# ------------------------------------------------------------------ set-up ---
def test_initialize_constants():
    g = oracle.GridMaker(0.5, 23.5)
    assert g.dim == 48
    assert g.p.final_radius_multiple == 1.5
    np.testing.assert_allclose([g.p.A, g.p.B, g.p.C, g.p.D, g.p.E],
                               [4 * E2, -12 * E2, 9 * E2, 8 * E2, -12 * E2], rtol=1e-7)
    assert oracle.GridMaker(0.1, 6.0).dim == 61
    assert oracle.GridMaker(0.25, 23.75).dim == 96
    g3 = oracle.GridMaker(0.5, 6.0, gaussian_radius_multiple=3.0)
    assert g3.p.final_radius_multiple == pytest.approx(19.0 / 6.0)
    gt = oracle.GridMaker(0.5, 6.0, gaussian_radius_multiple=-1.5)
    assert gt.p.gaussian_radius_multiple == 1.5 and gt.p.final_radius_multiple == 1.5


def test_quadratic_meets_gaussian_and_zero():
    """Value and slope continuity at r, zero value and slope at 1.5 r (what A..E encode)."""
    g = oracle.GridMaker(0.5, 6.0)
    A, B, C, D, E = g.p.A, g.p.B, g.p.C, g.p.D, g.p.E
    assert A + B + C == pytest.approx(E2, abs=1e-6)
    assert 2 * A + B == pytest.approx(-4 * E2, abs=1e-6)        # d/dx of exp(-2x^2) at 1
    assert A * 2.25 + B * 1.5 + C == pytest.approx(0, abs=1e-6)
    assert 2 * A * 1.5 + B == pytest.approx(0, abs=1e-6)
    assert D == pytest.approx(2 * A, rel=1e-6) and E == pytest.approx(B, rel=1e-6)


def test_bounds_1d_edges():
    g = oracle.GridMaker(0.5, 6.0)   # dim 13, origin at -3 for a centred grid
    # [-1,1]: the upper end is ceil(high/res) exclusive, so a voxel exactly at +R is left out
    assert g.bounds_1d(-3.0, 0.0, 1.0) == (4, 8)
    assert g.bounds_1d(-3.0, 0.1, 1.0) == (4, 9)        # floor(4.2), ceil(8.2)
    assert g.bounds_1d(-3.0, -10.0, 1.0) == (0, 0)      # entirely below the grid
    assert g.bounds_1d(-3.0, -3.5, 1.0) == (0, 1)       # sticks in from below
    assert g.bounds_1d(-3.0, 3.2, 1.0) == (10, 13)      # clamped to dim
    assert g.bounds_1d(-3.0, 10.0, 1.0)[0] >= 13        # above: empty range (lo >= hi)


# ----------------------------------------------------------------- forward ---
def test_density_profile_closed_form():
    """test/test_gridmaker.py:131-184."""
    g = oracle.GridMaker(0.1, 6.0)
    out = g.forward((0, 0, 0), [[0, 0, 0]], [0], [1.0], ntypes=1)
    assert out[0, 30, 30, 30] == pytest.approx(1.0)
    line = out[0, 30, 30, :]
    x = np.abs(np.arange(-3, 3.1, .1))
    for i in range(20, 41):
        assert line[i] == pytest.approx(np.exp(-2 * x[i] ** 2), abs=1e-6)
    for i in list(range(0, 15)) + list(range(45, 61)):
        assert line[i] == pytest.approx(0, abs=1e-7)
    quad = 4 * E2 * x ** 2 - 12 * E2 * x + 9 * E2
    for i in list(range(15, 20)) + list(range(41, 45)):
        assert line[i] == pytest.approx(quad[i], abs=1e-5)
    assert line[35] == pytest.approx(0.6065307, abs=1e-6)      # exp(-0.5)
    assert line[43] == pytest.approx(0.0216535, abs=1e-6)      # quadratic at 1.3
    g2 = oracle.GridMaker(0.1, 6.0, radius_scale=0.5, gaussian_radius_multiple=3.0)
    line = g2.forward((0, 0, 0), [[0, 0, 0]], [0], [1.0], ntypes=1)[0, 30, :, 30]
    for i in range(61):
        assert line[i] == pytest.approx(np.exp(-2 * (2 * x[i]) ** 2), abs=1e-5)


def brute_force_forward(res, dimension, binary, center, coords, types, radii, ntypes,
                        radius_scale=1.0):
    """Every atom against every voxel, no index boxes: float32 arithmetic, ascending atoms."""
    f = np.float32
    dim = int(round(dimension / res)) + 1
    half = f(dimension / 2.0)
    ax = [f(center[d]) - half + np.arange(dim, dtype=f) * f(res) for d in range(3)]
    X, Y, Z = np.meshgrid(*ax, indexing="ij")
    out = np.zeros((ntypes, dim, dim, dim), f)
    for a in range(len(coords)):
        t = int(np.floor(types[a]))
        if t < 0:
            continue
        ar = f(radii[a]) * f(radius_scale)
        dx, dy, dz = X - coords[a, 0], Y - coords[a, 1], Z - coords[a, 2]
        rsq = (dx * dx + dy * dy) + dz * dz
        if binary:
            out[t][rsq < ar * ar] = 1.0
            continue
        d = np.sqrt(rsq)
        gauss = np.exp((-2.0 * d.astype(np.float64) * d / (ar * ar)).astype(f))
        dr = d / ar
        quad = np.maximum((f(4 * E2) * dr + f(-12 * E2)) * dr + f(9 * E2), 0)
        val = np.where(d <= ar, gauss, quad)
        val = np.where(d > ar * f(1.5), f(0), val).astype(f)
        out[t] += val
    return out


@pytest.mark.parametrize("binary", [False, True])
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_forward_against_brute_force(binary, seed):
    rng = np.random.default_rng(seed)
    n, T = 25, 3
    coords = rng.uniform(-5, 5, (n, 3)).astype(np.float32)
    types = rng.integers(-1, T, n).astype(np.float32)
    radii = rng.uniform(0.8, 2.0, n).astype(np.float32)
    center = rng.uniform(-1, 1, 3).astype(np.float32)
    got = oracle.GridMaker(0.5, 7.5, binary).forward(center, coords, types, radii, T)
    want = brute_force_forward(0.5, 7.5, binary, center, coords, types, radii, T)
    if binary:
        assert np.array_equal(got, want)
    else:
        np.testing.assert_allclose(got, want, atol=2e-6, rtol=1e-6)


def test_forward_errors_and_ignored_types():
    g = oracle.GridMaker(0.5, 7.5)
    c, r = np.zeros((2, 3), np.float32), np.ones(2, np.float32)
    with pytest.raises(oracle.OracleError):                      # src/grid_maker.cpp:172
        g.forward((0, 0, 0), c, [0, 3], r, ntypes=3)
    out = g.forward((0, 0, 0), c, [-1, -2.5], r, ntypes=3)
    assert not out.any()
    with pytest.raises(oracle.OracleError):                      # src/grid_maker.cpp:160-162
        oracle.GridMaker(0.5, 7.5, False, True).forward((0, 0, 0), c, [0, 1], r, ntypes=3)
    # floor(), not round(): 1.9 lands in channel 1
    out = oracle.GridMaker(0.5, 8.0).forward((0, 0, 0), c[:1], [1.9], r[:1], ntypes=3)
    assert out[1].max() == pytest.approx(1.0) and not out[2].any() and not out[0].any()


def test_vector_types_linearity_and_equivalences():
    """test/test_gridmaker.py:217-256, test/test_gridmaker.cpp:408-500."""
    rng = np.random.default_rng(3)
    n, T = 12, 4
    coords = rng.uniform(-3, 3, (n, 3)).astype(np.float32)
    idx = rng.integers(0, T, n)
    radii = rng.uniform(1, 2, n).astype(np.float32)
    g = oracle.GridMaker(0.25, 6.0)
    ref = g.forward((0, 0, 0), coords, idx.astype(np.float32), radii, T)
    onehot = np.eye(T, dtype=np.float32)[idx]
    np.testing.assert_allclose(g.forward((0, 0, 0), coords, onehot, radii), ref, atol=1e-6)
    np.testing.assert_allclose(2 * g.forward((0, 0, 0), coords, 0.5 * onehot, radii), ref,
                               atol=1e-6)
    one = g.forward((0, 0, 0), [[0, 0, 0]], np.asarray([[0.5, 0, 0, 0]], np.float32), [1.0])
    assert one.max() == pytest.approx(0.5)                       # test_gridmaker.cpp:453
    # type-indexed radii equal per-atom radii when every atom of a type has that radius
    table = rng.uniform(1, 2, T).astype(np.float32)
    gi = oracle.GridMaker(0.25, 6.0, False, True)
    np.testing.assert_allclose(gi.forward((0, 0, 0), coords, onehot, table),
                               g.forward((0, 0, 0), coords, onehot, table[idx]), atol=1e-6)
    # binary vector mode adds the weight instead of storing 1
    gb = oracle.GridMaker(0.25, 6.0, True)
    two = gb.forward((0, 0, 0), [[0, 0, 0], [0.1, 0, 0]], np.full((2, 1), 0.25, np.float32),
                     [1.0, 1.0])
    assert two.max() == pytest.approx(0.5)
    idxb = gb.forward((0, 0, 0), [[0, 0, 0], [0.1, 0, 0]], [0, 0], [1.0, 1.0], ntypes=1)
    assert idxb.max() == 1.0


# ---------------------------------------------------------------- backward ---
def test_backward_known_answer():
    """test/test_gridmaker.py:186-214 and test/test_torch.py:144-148."""
    g = oracle.GridMaker(0.1, 6.0)
    diff = np.zeros((1, 61, 61, 61), np.float32)
    diff[0, 30, 30, 30] = 1.0
    grad = g.backward((0, 0, 0), [[1.0, 0, 0]], [0], [2.0], diff)
    np.testing.assert_allclose(grad.ravel(), [-0.60653067, 0, 0], atol=1e-6)
    # rotated atom, gradient rotated back (Transform::backward without translation)
    q = np.asarray([0.3, -0.5, 0.7, 0.1], np.float32)
    moved = oracle.transform_forward(q, (0, 0, 0), (0, 0, 0), [[1.0, 0, 0]])
    grad = g.backward((0, 0, 0), moved, [0], [2.0], diff)
    back = oracle.transform_backward(q, (0, 0, 0), (0, 0, 0), grad, dotranslate=False)
    np.testing.assert_allclose(back.ravel(), [-0.60653067, 0, 0], atol=1e-5)


def test_backward_symmetry():
    """test/test_gridmaker.cpp:252-287."""
    g = oracle.GridMaker(0.1, 6.0)
    diff = np.zeros((1, 61, 61, 61), np.float32)
    diff[0, 30, 30, 30] = 1.0
    c = np.asarray([[0, 0, 0], [1, 0, 0], [-1, 0, 0], [0, 0, 2.5]], np.float32)
    grad = g.backward((0, 0, 0), c, [0, 0, 0, 0], [2.0] * 4, diff)
    assert not grad[0].any()
    assert grad[1, 0] == -grad[2, 0] and grad[1, 0] < 0
    assert grad[3, 2] < 0                                        # quadratic tail, still pulls
    # round(), not floor(): 0.6 reads channel 1
    diff2 = np.zeros((2, 61, 61, 61), np.float32)
    diff2[1, 30, 30, 30] = 1.0
    assert g.backward((0, 0, 0), c[1:2], [0.6], [2.0], diff2)[0, 0] < 0
    assert not g.backward((0, 0, 0), c[1:2], [0.4], [2.0], diff2).any()
    assert not g.backward((0, 0, 0), c[1:2], [-1], [2.0], diff2).any()
    with pytest.raises(oracle.OracleError):
        g.backward((0, 0, 0), c[1:2], [2.0], [2.0], diff2)


def test_backward_is_gradient_of_forward():
    """backward = d/dcoords of sum(diff * forward): central differences of the forward pass."""
    rng = np.random.default_rng(5)
    n, T = 6, 2
    coords = rng.uniform(-2, 2, (n, 3)).astype(np.float32)
    types = rng.integers(0, T, n).astype(np.float32)
    radii = rng.uniform(1.2, 2.0, n).astype(np.float32)
    g = oracle.GridMaker(0.25, 8.0)
    d = g.dim
    ax = np.linspace(-1, 1, d)
    X, Y, Z = np.meshgrid(ax, ax, ax, indexing="ij")
    diff = np.stack([np.sin(2 * X) + Y * Z, np.cos(3 * Y) - X]).astype(np.float32)  # smooth
    grad = g.backward((0, 0, 0), coords, types, radii, diff, f64=True)
    h = 5e-3
    for a in range(n):
        for k in range(3):
            cp, cm = coords.copy(), coords.copy()
            cp[a, k] += h
            cm[a, k] -= h
            lp = (diff.astype(np.float64) * g.forward((0, 0, 0), cp, types, radii, T)).sum()
            lm = (diff.astype(np.float64) * g.forward((0, 0, 0), cm, types, radii, T)).sum()
            fd = (lp - lm) / (float(cp[a, k]) - float(cm[a, k]))
            assert grad[a, k] == pytest.approx(fd, rel=2e-2, abs=2e-2)


def test_backward_float_and_double_accumulation_agree():
    rng = np.random.default_rng(6)
    n, T = 40, 3
    coords = rng.uniform(-4, 4, (n, 3)).astype(np.float32)
    types = rng.integers(0, T, n).astype(np.float32)
    radii = rng.uniform(1.2, 2.0, n).astype(np.float32)
    g = oracle.GridMaker(0.5, 9.5)
    diff = rng.standard_normal(g.grid_shape(T)).astype(np.float32)
    a32 = g.backward((0, 0, 0), coords, types, radii, diff)
    a64 = g.backward((0, 0, 0), coords, types, radii, diff, f64=True)
    np.testing.assert_allclose(a32, a64, atol=2e-4, rtol=1e-4)


def test_vector_backward_linearity_and_type_gradient():
    rng = np.random.default_rng(7)
    n, T = 8, 3
    coords = rng.uniform(-2, 2, (n, 3)).astype(np.float32)
    tv = rng.uniform(0, 1, (n, T)).astype(np.float32)
    tv[0, 1] = 0
    radii = rng.uniform(1.2, 2.0, n).astype(np.float32)
    g = oracle.GridMaker(0.5, 7.5)
    diff = rng.standard_normal(g.grid_shape(T)).astype(np.float32)
    ag, tg = g.backward((0, 0, 0), coords, tv, radii, diff, f64=True)
    # atom gradient = sum_t weight_t * (index-typed gradient in channel t)
    want = np.zeros((n, 3))
    for t in range(T):
        want += tv[:, t:t + 1] * g.backward((0, 0, 0), coords, np.full(n, t, np.float32), radii,
                                            diff, f64=True)
    np.testing.assert_allclose(ag, want, atol=1e-6, rtol=1e-6)
    # type gradient = sum over voxels of (density of the atom alone) * diff_t, for every t
    for a in range(n):
        dens = g.forward((0, 0, 0), coords[a:a + 1], [0], radii[a:a + 1], ntypes=1)[0]
        np.testing.assert_allclose(tg[a], (dens[None].astype(np.float64) * diff).sum(axis=(1, 2, 3)),
                                   atol=1e-5, rtol=1e-5)
    # float versions agree with the double ones
    ag32, tg32 = g.backward((0, 0, 0), coords, tv, radii, diff)
    np.testing.assert_allclose(ag32, ag, atol=1e-4, rtol=1e-4)
    np.testing.assert_allclose(tg32, tg, atol=1e-4, rtol=1e-4)
    # type-indexed radii with one radius for all == per-atom radii all equal
    gi = oracle.GridMaker(0.5, 7.5, False, True)
    a1, t1 = gi.backward((0, 0, 0), coords, tv, np.full(T, 1.5, np.float32), diff)
    a2, t2 = g.backward((0, 0, 0), coords, tv, np.full(n, 1.5, np.float32), diff)
    assert np.array_equal(a1, a2) and np.array_equal(t1, t2)


# ------------------------------------------- relevance, second-order pass ---
def test_relevance_known_case_and_brute_force():
    """test/test_gridmaker.cpp:313-337: one atom, one voxel with density 1 and relevance 10."""
    g = oracle.GridMaker(0.1, 6.0)
    d = g.dim
    diff = np.zeros((1, d, d, d), np.float32)
    dens = np.zeros((1, d, d, d), np.float32)
    diff[0, 31, 30, 30] = 10.0
    dens[0, 31, 30, 30] = 1.0
    rel = g.backward_relevance((0, 0, 0), [[0, 0, 0]], [0], [2.0], dens, diff)
    assert 1.0 < rel[0] < 10.0
    assert rel[0] == pytest.approx(10.0 * np.exp(-2 * 0.1 ** 2 / 4.0), rel=1e-6)
    # brute force over every voxel: sum diff * own density / total density where both are positive
    rng = np.random.default_rng(21)
    n, T = 12, 3
    coords = rng.uniform(-3, 3, (n, 3)).astype(np.float32)
    types = rng.integers(0, T, n).astype(np.float32)
    types[3] = -1
    radii = rng.uniform(1.0, 2.0, n).astype(np.float32)
    for binary in (False, True):
        gm = oracle.GridMaker(0.5, 9.5, binary)
        total = gm.forward((0.1, 0, -0.2), coords, types, radii, T)
        if binary:
            total = total * rng.uniform(0.5, 2.0, total.shape).astype(np.float32)
        total[0, 5:8] = 0           # voxels without density hand nothing on
        diff = rng.standard_normal(total.shape).astype(np.float32)
        rel = gm.backward_relevance((0.1, 0, -0.2), coords, types, radii, total, diff)
        for a in range(n):
            if types[a] < 0:
                assert rel[a] == 0
                continue
            t = int(types[a])
            own = gm.forward((0.1, 0, -0.2), coords[a:a + 1], [0], radii[a:a + 1], 1)[0]
            ok = (own > 0) & (total[t] > 0)
            want = (diff[t][ok].astype(np.float64) * own[ok] / total[t][ok]).sum()
            assert rel[a] == pytest.approx(want, rel=1e-4, abs=1e-4)


def test_backward_gradients_closed_form():
    """test/test_gridmaker.py:439-466: d/dx of |d(density at one voxel)/dcoords|^2 for a full
    Gaussian (multiple -2, radius 1) is -128 d^3 exp(-4 d^2) + 32 d exp(-4 d^2), d = x - 1."""
    g = oracle.GridMaker(0.5, 6.0, gaussian_radius_multiple=-2.0)
    types = np.ones((1, 1), np.float32)
    radii = np.ones(1, np.float32)
    for axis in range(3):
        idx = [0, 6, 6, 6]
        idx[1 + axis] = 8                   # the voxel at +1.0 on this axis
        diff = np.zeros(g.grid_shape(1), np.float32)
        diff[tuple(idx)] = 1.0
        for x in np.arange(-0.9, 3, 0.1):
            coords = np.zeros((1, 3), np.float32)
            coords[0, axis] = x
            lg, _ = g.backward((0, 0, 0), coords, types, radii, diff)
            # fancyL = sum(lg^2): its gradient wrt lg is 2 lg, wrt the type gradient 0
            dd, add, tdd = g.backward_gradients((0, 0, 0), coords, types, radii, diff, 2 * lg,
                                                np.zeros((1, 1), np.float32))
            d = float(coords[0, axis]) - 1
            want = -128 * d ** 3 * np.exp(-4 * d ** 2) + 32 * d * np.exp(-4 * d ** 2)
            assert add[0, axis] == pytest.approx(want, abs=1e-4)
            assert not tdd.any()


def test_backward_gradients_are_derivatives_of_backward():
    """F(coords, diff) = <w, atom_gradients> + <v, type_gradients>: diffdiff = dF/ddiff (F is
    linear in diff), type_diffdiff = 0, and, for v = 0, atom_diffdiff = dF/dcoords (central
    differences of the double-accumulating backward pass).  The reference's v term of
    atom_diffdiff is v * sum(diff * d2(density)/da2) (src/grid_maker.cpp:631, the same
    expression as the coordinate term, src/grid_maker.cu:812-855), which is not dF/dcoords; it is
    checked against the analytic second derivative of a pure Gaussian below."""
    rng = np.random.default_rng(22)
    n, T = 5, 2
    coords = rng.uniform(-1.5, 1.5, (n, 3)).astype(np.float32)
    tv = rng.uniform(0.2, 1, (n, T)).astype(np.float32)
    tv[1, 0] = 0
    radii = rng.uniform(1.2, 1.8, n).astype(np.float32)
    g = oracle.GridMaker(0.25, 8.0)
    ax = np.linspace(-1, 1, g.dim)
    X, Y, Z = np.meshgrid(ax, ax, ax, indexing="ij")
    diff = np.stack([np.sin(2 * X) + Y * Z, np.cos(3 * Y) - X * Z]).astype(np.float32)
    w = rng.standard_normal((n, 3)).astype(np.float32)
    v = rng.standard_normal((n, T)).astype(np.float32)

    def F(c, dif):
        ag, tg = g.backward((0, 0, 0), c, tv, radii, dif, f64=True)
        # like the reference, a channel with zero weight takes no part in the second pass
        return float((w * ag).sum() + (v * tg * (tv != 0)).sum())

    dd, add, tdd = g.backward_gradients((0, 0, 0), coords, tv, radii, diff, w, v)
    assert not tdd.any()
    zero = np.zeros_like(v)
    add = g.backward_gradients((0, 0, 0), coords, tv, radii, diff, w, zero)[1]
    v_saved, v = v, zero
    h = 2e-3
    fd = np.zeros((n, 3))
    for a in range(n):
        for k in range(3):
            cp, cm = coords.copy(), coords.copy()
            cp[a, k] += h
            cm[a, k] -= h
            fd[a, k] = (F(cp, diff) - F(cm, diff)) / (float(cp[a, k]) - float(cm[a, k]))
    # every component is a sum of hundreds of terms of either sign: compare on the scale of the sums
    assert np.abs(add - fd).max() < 3e-3 * np.abs(fd).max()
    v = v_saved
    delta = rng.standard_normal(diff.shape).astype(np.float32)
    lin = F(coords, diff + delta) - F(coords, diff)
    assert float((dd.astype(np.float64) * delta).sum()) == pytest.approx(lin, rel=1e-3, abs=1e-3)
    with pytest.raises(oracle.OracleError):
        oracle.GridMaker(0.5, 6.0, True).backward_gradients((0, 0, 0), coords, tv, radii,
                                                            np.zeros((T, 13, 13, 13), np.float32), w, v)
    # the type-gradient term alone, pure Gaussian out to 2 r: v * sum(diff * d2/da2 exp(-2 d^2/r^2))
    gg = oracle.GridMaker(0.25, 8.0, gaussian_radius_multiple=-2.0)
    c1 = np.asarray([[0.3, -0.2, 0.1]], np.float32)
    r1 = np.asarray([1.3], np.float32)
    one = np.ones((1, 1), np.float32)
    d1 = diff[:1]
    got = gg.backward_gradients((0, 0, 0), c1, one, r1, d1, np.zeros((1, 3), np.float32),
                                np.full((1, 1), 0.7, np.float32))[1]
    pos = (-4.0 + 0.25 * np.arange(gg.dim)).astype(np.float64)
    PX, PY, PZ = np.meshgrid(pos, pos, pos, indexing="ij")
    rel = np.stack([PX - 0.3, PY + 0.2, PZ - 0.1])
    d2 = (rel ** 2).sum(axis=0)
    e = np.exp(-2 * d2 / 1.3 ** 2) * (np.sqrt(d2) <= 2 * 1.3)
    for k in range(3):
        second = (16 * rel[k] ** 2 / 1.3 ** 4 - 4 / 1.3 ** 2) * e
        assert got[0, k] == pytest.approx(0.7 * (second * d1[0]).sum(), rel=2e-3, abs=2e-3)


# ------------------------------------------------- quaternion / transform ---
def test_quaternion_hamilton_rules():
    i, j, k = [0, 1, 0, 0], [0, 0, 1, 0], [0, 0, 0, 1]
    assert list(oracle.quat_mul(i, j)) == k
    assert list(oracle.quat_mul(j, k)) == i
    assert list(oracle.quat_mul(k, i)) == j
    assert list(oracle.quat_mul(j, i)) == [0, 0, 0, -1]
    assert list(oracle.quat_mul(i, i)) == [-1, 0, 0, 0]
    q = np.asarray([0.3, -1.2, 0.5, 2.0], np.float32)
    one = oracle.quat_mul(q, oracle.quat_inverse(q))
    np.testing.assert_allclose(one, [1, 0, 0, 0], atol=1e-6)


def test_rotation_matches_matrix_even_unnormalised():
    rng = np.random.default_rng(8)
    for _ in range(5):
        q = rng.normal(size=4).astype(np.float32) * 3
        R = rot_matrix(q)
        for p in rng.uniform(-10, 10, (4, 3)):
            np.testing.assert_allclose(oracle.quat_rotate(q, p), R @ p, atol=2e-5)


def test_transform_known_points():
    """test/test_transform.cpp:55-87: z-90 about (0,1,1), translate (2,0,-3)."""
    s = np.sqrt(0.5)
    pts = np.asarray([[0, 0, 0], [1, 0, 0], [0, 1, 0], [0, 0, 1], [-1, .5, 3], [1, 1, 1],
                      [0, 1, 1], [.333, .75, -9]], np.float32)
    out = oracle.transform_forward([s, 0, 0, s], (0, 1, 1), (2, 0, -3), pts)
    np.testing.assert_allclose(out[6], [2, 1, -2], atol=1e-5)
    np.testing.assert_allclose(out[2], [2, 1, -3], atol=1e-5)
    np.testing.assert_allclose(out[5], [2, 2, -2], atol=1e-5)
    back = oracle.transform_backward([s, 0, 0, s], (0, 1, 1), (2, 0, -3), out)
    np.testing.assert_allclose(back, pts, atol=1e-5)


def test_transform_without_translation_still_rotates_about_center():
    rng = np.random.default_rng(9)
    q = rng.normal(size=4).astype(np.float32)
    c = np.asarray([1.0, -2.0, 0.5], np.float32)
    pts = rng.uniform(-5, 5, (6, 3)).astype(np.float32)
    out = oracle.transform_forward(q, c, (9, 9, 9), pts, dotranslate=False)
    np.testing.assert_allclose(out, (pts - c) @ rot_matrix(q).T + c, atol=2e-5)
    back = oracle.transform_backward(q, c, (9, 9, 9), out, dotranslate=False)
    np.testing.assert_allclose(back, pts, atol=2e-5)


# ----------------------------------------------------------- interpolation ---
def scipy_resample(src, ires, idim, ores, odim, in_c, q, rot_c, tr, out_c):
    """test/test_gridinterp.py:39-65 restated: zero-padded RegularGridInterpolator."""
    n_in = src.shape[1]
    n_out = int(round(odim / ores)) + 1
    axes = [in_c[d] - idim / 2.0 + ires * np.arange(-1, n_in + 1) for d in range(3)]
    oax = [out_c[d] - odim / 2.0 + ores * np.arange(n_out) for d in range(3)]
    P = np.stack(np.meshgrid(*oax, indexing="ij"), -1).reshape(-1, 3)
    back = (P - tr - rot_c) @ rot_matrix(q) + rot_c          # R^T applied = inverse rotation
    out = np.empty((src.shape[0], n_out, n_out, n_out))
    for c in range(src.shape[0]):
        pad = np.zeros((n_in + 2,) * 3)
        pad[1:-1, 1:-1, 1:-1] = src[c]
        f = RegularGridInterpolator(axes, pad, fill_value=0, bounds_error=False)
        out[c] = f(back).reshape(n_out, n_out, n_out)
    return out


@pytest.mark.parametrize("case", [(0.5, 6.0, 0.5, 6.0), (0.5, 6.0, 0.25, 4.0),
                                  (0.25, 4.0, 0.5, 7.0)])
def test_interpolation_against_scipy(case):
    """test/test_gridinterp.py:112-152 (atol 1e-4 there)."""
    rng = np.random.default_rng(10)
    ires, idim, ores, odim = case
    n_in = int(round(idim / ires)) + 1
    src = rng.random((2, n_in, n_in, n_in)).astype(np.float32)
    q = rng.normal(size=4)
    q = (q / np.linalg.norm(q)).astype(np.float32)
    rot_c = rng.uniform(-1, 1, 3).astype(np.float32)
    tr = rng.uniform(-1, 1, 3).astype(np.float32)
    in_c = rng.uniform(-.5, .5, 3).astype(np.float32)
    out_c = rng.uniform(-.5, .5, 3).astype(np.float32)
    got = oracle.interpolate(ires, idim, ores, odim, in_c, src, q, rot_c, tr, out_c)
    want = scipy_resample(src, ires, idim, ores, odim, in_c, q, rot_c, tr, out_c)
    np.testing.assert_allclose(got, want, atol=1e-4)


def test_interpolation_identity_sampling_and_shift():
    """test/test_gridinterp.cpp:13-60, test/test_gridinterp.py:15-108."""
    rng = np.random.default_rng(11)
    src = rng.random((1, 13, 13, 13)).astype(np.float32)
    ident = [1, 0, 0, 0]
    z = (0, 0, 0)
    assert np.array_equal(oracle.interpolate(0.5, 6.0, 0.5, 6.0, z, src, ident, z, z, z), src)
    down = oracle.interpolate(0.5, 6.0, 1.0, 6.0, z, src, ident, z, z, z)
    assert np.array_equal(down, src[:, ::2, ::2, ::2])
    up = oracle.interpolate(0.5, 6.0, 0.25, 6.0, z, src, ident, z, z, z)
    assert np.array_equal(up[:, ::2, ::2, ::2], src)
    np.testing.assert_allclose(up[0, 1, 0, 0], 0.5 * (src[0, 0, 0, 0] + src[0, 1, 0, 0]), atol=1e-6)
    shifted = oracle.interpolate(0.5, 6.0, 0.5, 6.0, z, src, ident, z, (0.5, 0, -1.0), z)
    np.testing.assert_allclose(shifted[:, 1:, :, :-2], src[:, :-1, :, 2:], atol=1e-5)
    assert not shifted[:, 0].any() and not shifted[:, :, :, -2:].any()


# ------------------------------------------------------------ batch drivers ---
def test_batch_drivers_equal_single_calls():
    rng = np.random.default_rng(12)
    off = np.asarray([0, 5, 5, 12])          # one empty example
    n, T = 12, 3
    coords = rng.uniform(-3, 3, (n, 3)).astype(np.float32)
    types = rng.integers(0, T, n).astype(np.float32)
    radii = rng.uniform(1, 2, n).astype(np.float32)
    centers = rng.uniform(-1, 1, (3, 3)).astype(np.float32)
    g = oracle.GridMaker(0.5, 7.5)
    out = g.forward_batch(off, centers, coords, types, radii, T, nthreads=2)
    diff = rng.standard_normal(out.shape).astype(np.float32)
    grads = g.backward_batch(off, centers, coords, types, radii, diff, nthreads=2)
    for b in range(3):
        s = slice(off[b], off[b + 1])
        assert np.array_equal(out[b], g.forward(centers[b], coords[s], types[s], radii[s], T))
        assert np.array_equal(grads[s], g.backward(centers[b], coords[s], types[s], radii[s],
                                                   diff[b]))
    assert not out[1].any()


def test_index_box_is_half_open_at_the_far_side():
    """get_bounds_1d (src/grid_maker.cu:66-79) gives [floor((c - r - o) / res), ceil((c + r - o) / res)),
    and the loops run i < hi: with an atom on a voxel centre and a final radius of exactly five
    voxels, the voxel five steps DOWN an axis is inside the box (floor of an integer) and the one
    five steps UP is not (ceil of an integer, exclusive).  For a Gaussian cut off at its radius
    multiple (no tail) that is visible: exp(-2) on one side, nothing on the other, in the density
    and, with an upstream gradient of one at both voxels, as a net pull in the gradient."""
    res, dim = 0.5, 24
    g = oracle.GridMaker(res, (dim - 1) * res, gaussian_radius_multiple=-1.0)
    assert g.p.final_radius_multiple == 1.0 and g.p.gaussian_radius_multiple == 1.0
    m = dim // 2
    half = (dim - 1) * res / 2
    atom = np.array([[m * res - half] * 3], np.float32)
    types, radii = np.zeros(1, np.float32), np.full(1, 2.5, np.float32)
    lo, hi = g.bounds_1d(-half, float(atom[0, 0]), 2.5)
    assert (lo, hi) == (m - 5, m + 5)                       # half open: m + 5 itself is outside
    d = g.forward((0, 0, 0), atom, types, radii, 1)[0]
    assert d[m, m, m] == 1.0
    for axis in range(3):
        down, up = [m, m, m], [m, m, m]
        down[axis] -= 5
        up[axis] += 5
        assert d[tuple(down)] == pytest.approx(E2, rel=1e-6) and d[tuple(up)] == 0.0
    # every other voxel at distance 2.5 -- (3, 4, 0) steps and permutations -- lies inside the box
    assert d[m + 3, m + 4, m] == pytest.approx(E2, rel=1e-6) and d[m + 4, m, m + 3] == pytest.approx(E2, rel=1e-6)
    diff = np.zeros((1, dim, dim, dim), np.float32)
    diff[0, m - 5, m, m] = diff[0, m + 5, m, m] = 1.0
    grad = g.backward((0, 0, 0), atom, types, radii, diff)[0]
    # only the voxel at -5 counts: -(dx / dist) * (-4 dist / ar^2 exp(-2)) with dx = -2.5, dist = ar = 2.5
    assert grad[0] == pytest.approx(-4.0 / 2.5 * E2, rel=1e-6) and grad[1] == 0 and grad[2] == 0


def test_oracle_is_clean_under_address_and_ub_sanitizers():
    """`make -C oracle asan`: every entry point of the oracle over the edge cases of its loops
    (atoms outside the grid and on its faces, radii <= 0, ignored types, no atoms, a one-voxel
    grid, resampling taps outside the input) in a host build with AddressSanitizer and UBSan."""
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run(["make", "-B", "-C", os.path.join(root, "oracle"), "asan"],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    if p.returncode != 0 and ("cannot find -lasan" in p.stdout or "libasan" in p.stdout
                              and "No such file" in p.stdout):
        pytest.skip("no sanitizer runtime for the host compiler")
    assert p.returncode == 0, p.stdout[-3000:]
    assert "status 0" in p.stdout
