"""GPU parity of Transform.forward/backward (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle
from util import dev, rot_matrix

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mg():
    import libmolgrid_amd
    return libmolgrid_amd


def test_z90_known_points(mg):
    """test/test_transform.cpp:55-103: 90 degrees about z, centre (0,1,0), translate (1,0,-1)."""
    s = float(np.sqrt(0.5))
    T = mg.Transform(mg.Quaternion(s, 0, 0, s), (0, 1, 0), (1, 0, -1))
    pts = dev(np.asarray([[0, 0, -1], [1, 0, -2], [0, 2, -1]], np.float32))   # hand-checked below
    out = torch.empty_like(pts)
    T.forward(pts, out)
    R = rot_matrix((s, 0, 0, s))
    want = (pts.cpu().numpy() - [0, 1, 0]) @ R.T + [0, 1, 0] + [1, 0, -1]
    np.testing.assert_allclose(out.cpu().numpy(), want, atol=1e-6)
    # (0,0,-1): minus centre (0,-1,-1) -> rotated (1,0,-1) -> plus centre, translate = (2,1,-2)
    np.testing.assert_allclose(out.cpu().numpy()[0], [2, 1, -2], atol=1e-6)
    back = torch.empty_like(pts)
    T.backward(out, back)
    np.testing.assert_allclose(back.cpu().numpy(), pts.cpu().numpy(), atol=1e-5)


@pytest.mark.parametrize("dotranslate", [True, False])
def test_random_vs_oracle_bit_exact(mg, dotranslate):
    rng = np.random.default_rng(6)
    q = rng.normal(size=4).astype(np.float32)            # deliberately not normalised
    center = rng.uniform(-3, 3, 3).astype(np.float32)
    tr = rng.uniform(-2, 2, 3).astype(np.float32)
    pts = rng.uniform(-15, 15, (1000, 3)).astype(np.float32)
    T = mg.Transform(mg.Quaternion(*q), center, tr)
    out = torch.empty((1000, 3), device="cuda")
    T.forward(dev(pts), out, dotranslate)
    ref = oracle.transform_forward(q, center, tr, pts, dotranslate)
    assert np.array_equal(out.cpu().numpy(), ref)
    back = torch.empty_like(out)
    T.backward(out, back, dotranslate)
    assert np.array_equal(back.cpu().numpy(), oracle.transform_backward(q, center, tr, ref,
                                                                        dotranslate))
    np.testing.assert_allclose(back.cpu().numpy(), pts, atol=2e-5)
    # in place
    buf = dev(pts)
    T.forward(buf, buf, dotranslate)
    assert np.array_equal(buf.cpu().numpy(), ref)


def test_host_arrays_and_errors(mg):
    T = mg.Transform(mg.Quaternion(1, 0, 0, 0), (0, 0, 0), (1, 2, 3))
    pts = np.zeros((5, 3), np.float32)
    out = np.empty_like(pts)
    T.forward(pts, out)
    assert np.array_equal(out, np.tile([1, 2, 3], (5, 1)).astype(np.float32))
    with pytest.raises(ValueError):
        T.forward(pts, np.empty((4, 3), np.float32))
    with pytest.raises(ValueError):
        T.forward(np.zeros((5, 2), np.float32), np.empty((5, 2), np.float32))


def test_random_constructor_is_uniform_rotation(mg):
    mg.set_random_seed(3)
    T = mg.Transform((1, 2, 3), 2.0, True)
    assert abs(T.get_quaternion().norm() - 1.0) < 1e-5
    assert all(abs(v) <= 2.0 for v in T.get_translation())
    assert tuple(T.get_rotation_center()) == (1.0, 2.0, 3.0)
