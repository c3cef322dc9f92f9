"""Grid views and managed grids on the host: the reference's test/test_grid.py and
test/test_numpy.py, with this package in place of molgrid."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def molgrid():
    try:
        import libmolgrid_amd
    except Exception as e:  # the shared library has not been built
        pytest.skip("libmolgrid_amd not importable: %s" % e)
    return libmolgrid_amd


def test_grid(molgrid):
    """test/test_grid.py:4-19"""
    g = molgrid.MGrid2f(10, 2)
    assert g.size() == 20
    g2 = molgrid.Grid2f(g.cpu())
    g2[5][1] = 3.0
    assert g[5, 1] == g2[5, 1]
    g1 = g2[5]
    g1[1] = 4.0
    assert g[5, 1] == 4.0
    gclone = g.clone()
    gclone[5, 1] = 5.5
    assert g[5, 1] == 4.0
    assert gclone[5][1] == 5.5


def test_numpy(molgrid):
    """test/test_numpy.py:8-35"""
    mg3d = molgrid.MGrid3d(3, 3, 3)
    mg2f = molgrid.MGrid2f(2, 4)
    a2f = np.arange(27).astype(np.float32).reshape(3, -1)
    a3d = np.arange(27).astype(np.float64).reshape(3, 3, -1)
    g2f = molgrid.Grid2f(a2f)
    g3d = molgrid.Grid3d(a3d)
    g2f[0, 0] = 100
    g3d[0, 0, 0] = 101
    assert a2f[0, 0] == 100
    assert a3d[0, 0, 0] == 101
    mg2f.copyFrom(g2f)
    mg3d.copyFrom(g3d)
    assert mg2f[1, 3] == 7
    mg2f[1, 3] = 200
    assert g2f[1, 3] == 12
    assert a2f[1, 3] == 12
    mg2f.copyTo(g2f)
    assert g2f[0, 7] == 200
    assert a2f[0, 7] == 200


def test_numpy_conv(molgrid):
    """test/test_numpy.py:37-55"""
    mg3d = molgrid.MGrid3d(3, 3, 3)
    mg2f = molgrid.MGrid2f(2, 4)
    a2f = np.arange(27).astype(np.float32).reshape(3, -1)
    a3d = np.arange(27).astype(np.float64).reshape(3, 3, -1)
    a2f[0, 0] = 100
    a3d[0, 0, 0] = 101
    mg2f.copyFrom(a2f)
    mg3d.copyFrom(a3d)
    assert mg2f[1, 3] == 7
    mg2f[1, 3] = 200
    assert a2f[1, 3] == 12
    mg2f.copyTo(a2f)
    assert a2f[0, 7] == 200


def test_tonumpy(molgrid):
    """test/test_numpy.py:57-73: tonumpy copies"""
    mg = molgrid.MGrid1d(10)
    for i in range(10):
        mg[i] = i
    a1 = mg.tonumpy()
    mg[0] = 100
    a2 = molgrid.tonumpy(mg)
    for i in range(10):
        mg[i] = 0
    a3 = mg.tonumpy()
    assert a1.sum() == 45
    assert a2.sum() == 145
    assert a3.sum() == 0


def test_clear(molgrid):
    """test/test_numpy.py:75-84"""
    g1 = molgrid.Grid1d(np.random.rand(20))
    mg = molgrid.MGrid3d(4, 5, 6)
    mg.copyFrom(np.random.rand(4, 5, 6))
    mg.fill_zero()
    g1.fill_zero()
    assert np.all(g1.tonumpy() == 0)
    assert np.all(mg.tonumpy() == 0)


def test_conversion_rules(molgrid):
    """python/bindings_grids.cpp:91-193: element type, rank, contiguity and side are checked."""
    a = np.zeros((3, 4), np.float32)
    with pytest.raises(ValueError):
        molgrid.Grid2d(a)                       # wrong element type
    with pytest.raises(ValueError):
        molgrid.Grid3f(a)                       # wrong rank
    with pytest.raises(ValueError):
        molgrid.Grid2f(a.T)                     # not C-contiguous
    with pytest.raises(ValueError):
        molgrid.Grid2fCUDA(a)                   # host memory is not device memory
    t = torch.zeros(3, 4)
    g = molgrid.Grid2f(t)
    g[1, 2] = 7
    assert t[1, 2] == 7 and g.shape == (3, 4) and len(g) == 3 and g.dimension(1) == 4
    assert g.type() == "float32" and molgrid.Grid1d(np.zeros(2)).type() == "float64"
    with pytest.raises(IndexError):
        g[3]
    m = molgrid.MGrid4f(2, 3, 4, 5)
    assert m.shape == (2, 3, 4, 5) and m.oncpu() and not m.ongpu()
    sub = m[1][2]
    sub[3, 4] = 9.0
    assert m[1, 2, 3, 4] == 9.0 and sub.shape == (4, 5)
    assert np.asarray(m).shape == (2, 3, 4, 5)


def _filled_mgrids(molgrid):
    mg2 = molgrid.MGrid2f(3, 4)
    mg3 = molgrid.MGrid3d(3, 4, 2)
    for i in range(3):
        for j in range(4):
            mg2[i, j] = i * j + 1
            for k in range(2):
                mg3[i, j, k] = i * j + 1 + k
    return mg2, mg3


def test_mgrid_copyto_and_copyfrom_tensor(molgrid):
    """test/test_torch.py:9-37, 55-76"""
    import torch
    mg2, mg3 = _filled_mgrids(molgrid)
    t2 = torch.zeros(3, 4)
    t3 = torch.zeros(3, 4, 2, dtype=torch.float64)
    assert mg2.copyTo(t2) == 12 and mg3.copyTo(t3) == 24
    for i in range(3):
        for j in range(4):
            assert t2[i, j] == i * j + 1
            for k in range(2):
                assert t3[i, j, k] == i * j + 1 + k
    b2, b3 = molgrid.MGrid2f(3, 4), molgrid.MGrid3d(3, 4, 2)
    b2.copyFrom(t2)
    b3.copyFrom(t3)
    for i in range(3):
        for j in range(4):
            assert b2[i, j] == i * j + 1
            for k in range(2):
                assert b3[i, j, k] == i * j + 1 + k
