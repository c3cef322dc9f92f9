"""CoordinateSet, Example and ExampleVec on the host: the array-based cases of the reference's
test/test_coordinateset.py and the merge / label semantics of src/example.cpp and
src/coordinateset.cpp (the molecule-file constructors need a chemistry toolkit and are not part
of this package)."""
import numpy as np
import pytest
from pytest import approx

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def molgrid():
    try:
        import libmolgrid_amd
    except Exception as e:  # the shared library has not been built
        pytest.skip("libmolgrid_amd not importable: %s" % e)
    return libmolgrid_amd


def index_set(molgrid, n, ntypes, seed):
    rng = np.random.default_rng(seed)
    return molgrid.CoordinateSet(rng.uniform(-5, 5, (n, 3)).astype(np.float32),
                                 rng.integers(0, ntypes, n).astype(np.float32),
                                 rng.uniform(1, 2, n).astype(np.float32), ntypes)


def test_coordset_from_array(molgrid):
    """test/test_coordinateset.py:69-88 without the transform (which runs on the device)."""
    coords = np.array([[1, 0, -1], [1, 3, -1], [1, 0, -1]], np.float32)
    types = np.array([3, 2, 1], np.float32)
    radii = np.array([1.5, 1.5, 1.0], np.float32)
    c = molgrid.CoordinateSet(coords, types, radii, 4)
    assert c.coords[1, 1] == 3.0 and c.size() == 3 and c.num_types() == 4
    assert c.has_indexed_types() and not c.has_vector_types()
    coords[1, 1] = 7.0                      # the set owns a copy
    assert c.coords[1, 1] == 3.0
    c2 = c.clone()
    c2.coords[1, 1] = 0
    assert c.coords[1, 1] == 3.0
    assert tuple(c.center()) == approx((1.0, 1.0, -1.0))
    assert molgrid.CoordinateSet().size() == 0
    e = molgrid.CoordinateSet()
    assert e.has_indexed_types() and e.has_vector_types()      # empty sets are both
    with pytest.raises(ValueError):
        molgrid.CoordinateSet(coords, types[:2], radii, 4)


def test_coordset_merge(molgrid):
    """test/test_coordinateset.py:90-114 with array-built sets."""
    c = index_set(molgrid, 16, 80, 1)
    c2 = index_set(molgrid, 8, 14, 2)
    c3 = molgrid.CoordinateSet(c, c2)
    c4 = molgrid.CoordinateSet(c, c2, False)
    assert c3.max_type == c.max_type + c2.max_type
    assert c3.coords.dimension(0) == c.coords.dimension(0) + c2.type_index.size()
    assert c4.max_type == max(c.max_type, c2.max_type)
    t = np.concatenate([c.type_index.tonumpy(), c2.type_index.tonumpy() + c.max_type])
    assert np.array_equal(t, c3.type_index.tonumpy())
    assert c4.coords.tonumpy().shape == (24, 3)
    t = np.concatenate([c.type_index.tonumpy(), c2.type_index.tonumpy()])
    assert np.array_equal(t, c4.type_index.tonumpy())
    assert np.array_equal(c3.radii.tonumpy(),
                          np.concatenate([c.radii.tonumpy(), c2.radii.tonumpy()]))


def test_vector_types_and_copyTo(molgrid):
    """test/test_coordinateset.py:55-66 and 117-147: one-hot vectors with a dummy type and typed
    radii; copyTo pads and truncates."""
    c = index_set(molgrid, 8, 14, 3)
    idx = c.type_index.tonumpy().astype(int)
    cv = c.clone()
    cv.make_vector_types(True, [1.0 + 0.1 * i for i in range(14)])
    assert cv.type_vector.dimension(1) == 15 and cv.radii.dimension(0) == 15
    assert cv.has_vector_types() and cv.radii[14] == 0.0 and cv.radii[3] == approx(1.3)
    tv = cv.type_vector.tonumpy()
    assert np.array_equal(tv.argmax(1), idx) and np.all(tv.sum(1) == 1)
    with pytest.raises(ValueError):
        c.clone().make_vector_types(False, [1.0] * 3)

    c.make_vector_types()
    coords = np.zeros([10, 3], np.float32)
    types = np.zeros([10, 15], np.float32)
    radii = np.zeros(10, np.float32)
    assert c.copyTo(coords, types, radii) == 8
    assert np.sum(coords) != 0
    assert types[:, 14].sum() == 0 and coords[8:].sum() == 0 and radii[8:].sum() == 0
    assert np.array_equal(types[:8, :14], c.type_vector.tonumpy())
    coordsm = np.zeros([5, 3], np.float32)
    typesm = np.zeros([5, 8], np.float32)
    radiim = np.zeros(5, np.float32)
    assert c.copyTo(coordsm, typesm, radiim) == 5
    assert np.all(coordsm == coords[:5])
    assert np.all(typesm == types[:5, :8])
    assert np.all(radiim == radii[:5])


def test_sum_types(molgrid):
    c = index_set(molgrid, 50, 6, 4)
    out = np.full(6, 9.0, np.float32)
    c.sum_types(out)
    assert np.array_equal(out, np.bincount(c.type_index.tonumpy().astype(int), minlength=6))
    c.make_vector_types()
    out2 = np.zeros(6, np.float32)
    c.sum_types(molgrid.Grid1f(out2))
    assert np.array_equal(out, out2)
    with pytest.raises(ValueError):
        c.sum_types(np.zeros(5, np.float32))


def test_example_merge(molgrid):
    """src/example.cpp:19-228."""
    rec, lig = index_set(molgrid, 30, 14, 5), index_set(molgrid, 7, 11, 6)
    ex = molgrid.Example()
    ex.coord_sets = [rec, lig]
    ex.labels = [1.0, 6.05]
    assert ex.num_coordinates() == 37
    assert ex.num_types() == 25 and ex.num_types(False) == 14
    assert ex.has_index_types() and not ex.has_vector_types()
    m = ex.merge_coordinates()
    assert m.max_type == 25 and m.size() == 37
    assert np.array_equal(m.type_index.tonumpy()[30:], lig.type_index.tonumpy() + 14)
    assert np.array_equal(m.coords.tonumpy()[:30], rec.coords.tonumpy())
    m2 = ex.merge_coordinates(0, False)
    assert m2.max_type == 14
    assert np.array_equal(m2.type_index.tonumpy()[30:], lig.type_index.tonumpy())
    only_lig = ex.merge_coordinates(1)
    assert only_lig == lig and only_lig is not lig
    assert ex.merge_coordinates(2).size() == 0
    # into caller's arrays
    c = np.zeros((37, 3), np.float32)
    t = np.zeros(37, np.float32)
    r = np.zeros(37, np.float32)
    ex.merge_coordinates(c, t, r)
    assert np.array_equal(c, m.coords.tonumpy()) and np.array_equal(t, m.type_index.tonumpy())
    with pytest.raises(ValueError):
        ex.merge_coordinates(np.zeros((36, 3), np.float32), t, r)
    # an empty set is skipped before its types are added to the offset (src/example.cpp:87),
    # although the merged set still counts them in its number of types
    ex2 = molgrid.Example()
    ex2.coord_sets = [rec, molgrid.CoordinateSet(np.zeros((0, 3), np.float32),
                                                 np.zeros(0, np.float32),
                                                 np.zeros(0, np.float32), 5), lig]
    m3 = ex2.merge_coordinates()
    assert m3.max_type == 30 and m3.size() == 37
    assert np.array_equal(m3.type_index.tonumpy()[30:], lig.type_index.tonumpy() + 14)
    sums = np.zeros(25, np.float32)
    ex.sum_types(sums)
    assert sums.sum() == 37 and sums[:14].sum() == 30


def test_example_merge_vector_types(molgrid):
    def vector_set(n, ntypes, seed):
        rng = np.random.default_rng(seed)
        return molgrid.CoordinateSet(rng.uniform(-5, 5, (n, 3)).astype(np.float32),
                                     rng.random((n, ntypes), dtype=np.float32),
                                     rng.uniform(1, 2, n).astype(np.float32))
    rec, lig = vector_set(12, 4, 7), vector_set(5, 3, 8)
    assert rec.has_vector_types() and not rec.has_indexed_types() and rec.max_type == 4
    ex = molgrid.Example()
    ex.coord_sets = [rec, lig]
    assert ex.has_vector_types() and not ex.has_index_types()
    m = ex.merge_coordinates()
    assert m.max_type == 7 and m.type_vector.shape == (17, 7)
    tv = m.type_vector.tonumpy()
    assert np.array_equal(tv[:12, :4], rec.type_vector.tonumpy()) and tv[:12, 4:].sum() == 0
    assert np.array_equal(tv[12:, 4:], lig.type_vector.tonumpy()) and tv[12:, :4].sum() == 0
    # a set that went through make_vector_types keeps its indices: it merges either way
    both = index_set(molgrid, 6, 3, 9)
    both.make_vector_types()
    assert both.has_vector_types() and both.has_indexed_types()
    mixed = molgrid.Example()
    mixed.coord_sets = [rec, index_set(molgrid, 3, 2, 9)]
    with pytest.raises(ValueError):
        mixed.merge_coordinates()


def test_example_vec_labels(molgrid):
    """src/example.cpp:254-299, used as in test/test_example_provider.py:76-106."""
    batch = molgrid.ExampleVec()
    for i in range(4):
        ex = molgrid.Example()
        ex.labels = [float(i), 0.5 * i, -1.0]
        batch.append(ex)
    labels = molgrid.MGrid2f(4, 3)
    batch.extract_labels(labels.cpu())
    assert labels[2, 1] == 1.0 and labels[3][0] == 3.0
    one = molgrid.MGrid1f(4)
    batch.extract_label(1, one.cpu())
    assert np.array_equal(one.tonumpy(), [0.0, 0.5, 1.0, 1.5])
    a = np.zeros(4, np.float32)
    batch.extract_label(2, a)
    assert np.all(a == -1.0)
    with pytest.raises(IndexError):
        batch.extract_label(3, a)
    with pytest.raises(IndexError):
        batch.extract_labels(np.zeros((3, 3), np.float32))
