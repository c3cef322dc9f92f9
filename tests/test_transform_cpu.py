"""Transform.forward/backward on host arrays run on the host (the reference's Grid<Dtype, 2, false>
overloads, src/transform.cpp:57-108) and must give the oracle's floats bit for bit.  No GPU."""
import numpy as np
import pytest
import torch

import oracle


@pytest.fixture(scope="module")
def mg():
    import libmolgrid_amd
    return libmolgrid_amd


def _case(seed, n=257):
    rng = np.random.default_rng(seed)
    q = rng.normal(size=4).astype(np.float32)            # deliberately not normalised
    center = rng.uniform(-3, 3, 3).astype(np.float32)
    tr = rng.uniform(-2, 2, 3).astype(np.float32)
    pts = rng.uniform(-20, 20, (n, 3)).astype(np.float32)
    return q, center, tr, pts


@pytest.mark.parametrize("dotranslate", [True, False])
@pytest.mark.parametrize("seed", [6, 7])
def test_numpy_arrays_match_oracle_bit_for_bit(mg, seed, dotranslate):
    q, center, tr, pts = _case(seed)
    T = mg.Transform(mg.Quaternion(*q), tuple(center), tuple(tr))
    out = np.empty_like(pts)
    T.forward(pts, out, dotranslate)
    want = oracle.transform_forward(q, center, tr, pts, dotranslate)
    assert np.array_equal(out, want)
    back = np.empty_like(pts)
    T.backward(out, back, dotranslate)
    assert np.array_equal(back, oracle.transform_backward(q, center, tr, want, dotranslate))
    np.testing.assert_allclose(back, pts, atol=2e-5)


def test_z90_known_points(mg):
    """test/test_transform.cpp:55-103: 90 degrees about z, centre (0,1,0), translate (1,0,-1)."""
    s = float(np.sqrt(0.5))
    T = mg.Transform(mg.Quaternion(s, 0, 0, s), (0, 1, 0), (1, 0, -1))
    pts = np.asarray([[0, 0, -1], [1, 0, -2], [0, 2, -1]], np.float32)
    out = np.empty_like(pts)
    T.forward(pts, out)
    np.testing.assert_allclose(out, [[2, 1, -2], [2, 2, -3], [0, 1, -2]], atol=1e-6)


def test_cpu_tensors_in_place_and_grids(mg):
    q, center, tr, pts = _case(8, n=64)
    T = mg.Transform(mg.Quaternion(*q), tuple(center), tuple(tr))
    want = oracle.transform_forward(q, center, tr, pts, True)
    t = torch.from_numpy(pts.copy())
    T.forward(t, t)                                       # in place
    assert np.array_equal(t.numpy(), want)
    g_in = mg.MGrid2f(64, 3)
    g_in.copyFrom(pts)
    g_out = mg.MGrid2f(64, 3)
    T.forward(g_in, g_out)
    assert np.array_equal(g_out.tonumpy(), want)
    cs = mg.CoordinateSet(pts, np.zeros(64, np.float32), np.ones(64, np.float32), 1)
    cs_out = cs.clone()
    T.forward(cs, cs_out)
    assert np.array_equal(np.asarray(cs_out.coords.tonumpy()), want)


def test_float64_arrays_store_the_float_results(mg):
    """The reference's double overload narrows at the call of Quaternion::transform and stores the
    float results widened (src/transform.cpp:57-79)."""
    q, center, tr, pts = _case(9, n=50)
    T = mg.Transform(mg.Quaternion(*q), tuple(center), tuple(tr))
    out = np.empty((50, 3), np.float64)
    T.forward(pts.astype(np.float64), out)
    assert np.array_equal(out, oracle.transform_forward(q, center, tr, pts, True).astype(np.float64))


def test_argument_errors(mg):
    T = mg.Transform()
    with pytest.raises(ValueError):
        T.forward(np.zeros((4, 3), np.float32), np.zeros((5, 3), np.float32))
    with pytest.raises(ValueError):
        T.forward(np.zeros((4, 2), np.float32), np.zeros((4, 2), np.float32))
    with pytest.raises(ValueError):
        T.backward(np.zeros((4, 3), np.float32), np.zeros((4, 3), np.int32))
