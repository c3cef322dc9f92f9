"""Managed grids with the gridding calls, as the reference's own tests use them
(test/test_gridmaker.py:131-214, test/test_grid.py): one MGrid is filled through its host view,
one through its device view; both go through the same HIP kernels and are checked against the
closed forms of the reference's tests and against the CPU oracle."""
import numpy as np
import pytest
import torch
from pytest import approx

import oracle
from util import ATOL, RTOL, assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def molgrid():
    import libmolgrid_amd
    return libmolgrid_amd


def test_mgrid_migration(molgrid):
    """include/libmolgrid/managed_grid.h:373-404: the whole buffer moves; views share it."""
    g = molgrid.MGrid3f(2, 3, 4)
    g[1, 2, 3] = 5.0
    assert g.oncpu()
    d = g.gpu()
    assert g.ongpu() and isinstance(d, molgrid.Grid3fCUDA)
    d[0, 0, 0] = 2.0                       # written on the device
    sub = g[1]                             # shares the buffer, which now lives on the device
    assert sub.ongpu() and sub.shape == (3, 4)
    t = torch.as_tensor(sub.gpu()._t)
    assert float(t[2, 3]) == 5.0
    assert g[0, 0, 0] == 2.0               # element access migrates back to the host
    assert g.oncpu() and sub.oncpu()
    c = g.clone()
    c.gpu()[1, 2, 3] = 7.0
    assert g[1, 2, 3] == 5.0 and c[1, 2, 3] == 7.0
    with pytest.raises(ValueError):
        molgrid.Grid3f(d)                  # a device view is not host memory
    with pytest.raises(ValueError):
        molgrid.Grid3fCUDA(torch.zeros(2, 3, 4))
    m2 = molgrid.MGrid1f(24)
    m2.gpu()
    assert m2.copyFrom(g) == 24            # host -> device, flat order
    assert m2.tonumpy()[23] == 5.0 and m2.ongpu()


def test_radius_multiples(molgrid):
    """test/test_gridmaker.py:131-183"""
    g1 = molgrid.GridMaker(resolution=.1, dimension=6.0)
    c = np.array([[0, 0, 0]], np.float32)
    t = np.array([0], np.float32)
    r = np.array([1.0], np.float32)
    coords = molgrid.CoordinateSet(molgrid.Grid2f(c), molgrid.Grid1f(t), molgrid.Grid1f(r), 1)
    shape = g1.grid_dimensions(1)
    cpugrid = molgrid.MGrid4f(*shape)
    cpugrid2 = molgrid.MGrid4f(*shape)
    gpugrid = molgrid.MGrid4f(*shape)

    g1.forward((0, 0, 0), coords, cpugrid.cpu())
    g1.forward((0, 0, 0), coords, gpugrid.gpu())
    g1.forward((0, 0, 0), c, t, r, cpugrid2.cpu())
    assert cpugrid.oncpu() and gpugrid.ongpu()

    np.testing.assert_array_equal(cpugrid.tonumpy(), gpugrid.tonumpy())
    np.testing.assert_array_equal(cpugrid.tonumpy(), cpugrid2.tonumpy())
    g = cpugrid.tonumpy()
    ref = oracle.GridMaker(0.1, 6.0).forward((0, 0, 0), c, t, r, 1)
    assert_close(g, ref, what="MGrid forward vs oracle")

    assert g[0, 30, 30, 30] == approx(1)
    line = g[0, 30, 30, :]
    xvals = np.abs(np.arange(-3, 3.1, .1))
    gauss = np.exp(-2 * xvals ** 2)
    for i in range(20, 41):
        assert line[i] == approx(gauss[i])
    for i in list(range(0, 15)) + list(range(45, 61)):
        assert line[i] == approx(0)
    quad = 4 * np.exp(-2) * xvals ** 2 - 12 * np.exp(-2) * xvals + 9 * np.exp(-2)
    for i in list(range(15, 20)) + list(range(41, 45)):
        assert line[i] == approx(quad[i], abs=1e-5)

    g2 = molgrid.GridMaker(resolution=.1, dimension=6.0, radius_scale=0.5,
                           gaussian_radius_multiple=3.0)
    gpugrid = molgrid.MGrid4f(*shape)
    g2.forward((0, 0, 0), coords, gpugrid.gpu())
    g = gpugrid.tonumpy()
    assert g[0, 30, 30, 30] == approx(1)
    line = g[0, 30, :, 30]
    gauss = np.exp(-2 * (xvals * 2.0) ** 2)
    for i in range(0, 61):
        assert line[i] == approx(gauss[i], abs=1e-5)


def test_backwards(molgrid):
    """test/test_gridmaker.py:186-214"""
    g1 = molgrid.GridMaker(resolution=.1, dimension=6.0)
    c = np.array([[1.0, 0, 0]], np.float32)
    t = np.array([0], np.float32)
    r = np.array([2.0], np.float32)
    coords = molgrid.CoordinateSet(c, t, r, 1)
    shape = g1.grid_dimensions(1)

    diff = molgrid.MGrid4f(*shape)
    diff[0, 30, 30, 30] = 1.0

    cpuatoms = molgrid.MGrid2f(1, 3)
    gpuatoms = molgrid.MGrid2f(1, 3)

    molgrid.set_random_seed(11)
    T = molgrid.Transform((0, 0, 0), 0, True)
    T.forward(coords, coords)
    assert c[0, 0] == 1.0                  # the set owns a copy of its arrays

    g1.backward((0, 0, 0), coords, diff.cpu(), cpuatoms.cpu())
    g1.backward((0, 0, 0), coords, diff.gpu(), gpuatoms.gpu())

    T.backward(cpuatoms.cpu(), cpuatoms.cpu(), False)
    T.backward(gpuatoms.gpu(), gpuatoms.gpu(), False)

    np.testing.assert_allclose(cpuatoms.tonumpy(), gpuatoms.tonumpy(), atol=1e-6)
    np.testing.assert_allclose(cpuatoms.tonumpy().flatten(), [-0.60653067, 0, 0], atol=1e-5)


def test_interpolater_takes_grids(molgrid):
    """python/bindings.cpp GridInterpolater.forward with managed grids on either side."""
    gi = molgrid.GridInterpolater(0.5, 6.0, 0.5, 6.0)
    src = molgrid.MGrid4f(2, 13, 13, 13)
    src.copyFrom(np.random.default_rng(3).random((2, 13, 13, 13), np.float32))
    dst = molgrid.MGrid4f(2, 13, 13, 13)
    gi.forward(src.gpu(), molgrid.Transform(), dst.gpu())
    assert dst.ongpu()
    assert_close(dst.tonumpy(), src.tonumpy(), rtol=RTOL, atol=ATOL, what="identity resampling")


def test_mgrid_copy_to_and_from_device_tensors(molgrid):
    """test/test_torch.py:39-53, 78-99"""
    mg2 = molgrid.MGrid2f(3, 4)
    mg3 = molgrid.MGrid3d(3, 4, 2)
    for i in range(3):
        for j in range(4):
            mg2[i, j] = i * j + 1
            for k in range(2):
                mg3[i, j, k] = i * j + 1 + k
    t2 = torch.zeros(3, 4, device="cuda")
    t3 = torch.zeros(3, 4, 2, dtype=torch.float64, device="cuda")
    mg2.copyTo(t2)
    mg3.copyTo(t3)
    b2, b3 = molgrid.MGrid2f(3, 4), molgrid.MGrid3d(3, 4, 2)
    b2.copyFrom(t2)
    b3.copyFrom(t3)
    for i in range(3):
        for j in range(4):
            assert t2[i, j] == i * j + 1 and b2[i, j] == i * j + 1
            for k in range(2):
                assert t3[i, j, k] == i * j + 1 + k and b3[i, j, k] == i * j + 1 + k
