"""The data feed on the host, against the values the reference's own tests hold for its test data
(test/test_example_provider.py, test/test_typing.py, test/test_gridio.py): example lists,
pre-typed structure files, the ligand cache, the sampling schemes and the grid files.  The data
files are a subset of the reference's test/data (tests/golden/make_provider_fixtures.py); cases of
the reference's tests that parse molecule files with a chemistry toolkit are not covered."""
import os

import numpy as np
import pytest
from pytest import approx

torch = pytest.importorskip("torch")

datadir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "molgrid_data")


@pytest.fixture(scope="module")
def molgrid():
    try:
        import libmolgrid_amd
    except Exception as e:  # the shared library has not been built
        pytest.skip("libmolgrid_amd not importable: %s" % e)
    return libmolgrid_amd


# ---- typers (test/test_typing.py, through get_int_type) ------------------------------------
def test_default_gnina_typers(molgrid):
    """test/test_typing.py:79-110 and src/atom_typer.cpp:524-559"""
    t = molgrid.defaultGninaLigandTyper
    assert t.num_types() == 14
    names = t.get_type_names()
    assert names[2] == "AromaticCarbonXSHydrophobe"
    g = molgrid.GninaIndexTyper()
    gn = g.get_type_names()
    assert g.num_types() == 28 and gn[27] == "Boron"
    typ, r = t.get_int_type(gn.index("AromaticCarbonXSHydrophobe"))
    assert names[typ] == "AromaticCarbonXSHydrophobe" and r == approx(1.9)
    typ, r = t.get_int_type(gn.index("OxygenXSDonorAcceptor"))
    assert names[typ] == "OxygenXSDonorAcceptor_OxygenXSDonor" and r == approx(1.7)
    typ, r = t.get_int_type(gn.index("Chlorine"))
    assert names[typ] == "Chlorine" and r == approx(1.8)
    assert t.get_int_type(gn.index("Hydrogen"))[0] == -1          # hydrogens have no channel
    rec = molgrid.defaultGninaReceptorTyper
    assert rec.num_types() == 14
    assert rec.get_type_names()[4] == "Bromine_Iodine_Chlorine_Fluorine"
    assert rec.get_type_radii()[4] == approx((2.0 + 2.2 + 1.8 + 1.5) / 4)
    assert g.get_int_type(40) == (26, approx(1.2))                # unknown types: generic metal
    assert molgrid.GninaIndexTyper(True).get_int_type(2)[1] == approx(0.77)


def test_element_null_subset_typers(molgrid):
    """test/test_typing.py:147-262"""
    t = molgrid.ElementIndexTyper(17)
    names = t.get_type_names()
    assert t.num_types() == 17 and names[2] == "Helium" and names[0] == "GenericAtom"
    assert t.get_int_type(6) == (6, approx(0.76))
    assert t.get_int_type(8) == (8, approx(0.66))
    assert t.get_int_type(1) == (1, approx(0.31))
    assert t.get_int_type(17)[0] == 0                              # truncated
    n = molgrid.NullIndexTyper()
    assert n.num_types() == 0 and n.get_int_type(6) == (-1, 0.0)
    s = molgrid.SubsettedElementTyper([1, 6, 7, 8])
    assert s.num_types() == 5 and s.get_type_names()[4] == "GenericAtom"
    assert s.get_type_names()[1] == "Carbon"
    assert s.get_int_type(6)[0] == 1 and s.get_int_type(17)[0] == 4
    s2 = molgrid.SubsettedElementTyper([1, 6, 7, 8], catchall=False)
    assert s2.num_types() == 4 and s2.get_int_type(17)[0] == -1
    sg = molgrid.SubsettedGninaTyper([[2, 3], [4, 5]], catchall=True)
    assert sg.num_types() == 3
    assert sg.get_type_names()[0] == "AliphaticCarbonXSHydrophobe_AliphaticCarbonXSNonHydrophobe"
    with pytest.raises(NotImplementedError):
        t.get_atom_type_index(object())


def test_file_mapped_typers(molgrid):
    """test/test_typing.py:265-330"""
    t = molgrid.FileMappedGninaTyper(os.path.join(datadir, "recmap"))
    names = t.get_type_names()
    assert len(names) == 14 and names[-2] == "Zinc"
    g = molgrid.GninaIndexTyper().get_type_names()
    typ, r = t.get_int_type(g.index("OxygenXSDonor"))
    assert names[typ] == "OxygenXSDonorAcceptor_OxygenXSDonor" and r == approx(1.7)
    typ, r = t.get_int_type(g.index("Chlorine"))
    assert names[typ] == "Bromine_Iodine_Chlorine_Fluorine" and r == approx(1.8)
    assert t.get_int_type(g.index("PolarHydrogen"))[0] == -1
    e = molgrid.FileMappedElementTyper(os.path.join(datadir, "emap"))
    en = e.get_type_names()
    assert len(en) == 4 and en[0] == "Oxygen"
    assert en[e.get_int_type(6)[0]] == "Carbon" and e.get_int_type(6)[1] == approx(0.76)
    assert e.get_int_type(17)[0] == -1
    with pytest.raises(ValueError):
        molgrid.FileMappedGninaTyper(os.path.join(datadir, "no_such_map"))


# ---- providers -------------------------------------------------------------------------------
def test_gnina_example_provider(molgrid):
    """test/test_example_provider.py:74-123"""
    e = molgrid.ExampleProvider(data_root=datadir + "/structs")
    e.populate(datadir + "/small.types")
    batch_size = 100
    batch = e.next_batch(batch_size)
    nlabels = e.num_labels()
    assert nlabels == 3 and e.size() == 1000 and e.num_types() == 28
    labels = molgrid.MGrid2f(batch_size, nlabels)
    batch.extract_labels(labels.cpu())
    label0, label1, label2 = [molgrid.MGrid1f(batch_size) for _ in range(3)]
    batch.extract_label(0, label0.cpu())
    batch.extract_label(1, label1.cpu())
    batch.extract_label(2, label2.cpu())
    assert label0[0] == 1
    assert label1[0] == approx(6.05)
    assert label2[0] == approx(0.162643)
    assert labels[0, 0] == 1 and labels[0][1] == approx(6.05) and labels[0][2] == approx(0.162643)
    for i in range(nlabels):
        assert label0[i] == labels[i][0] and label1[i] == labels[i][1] and label2[i] == labels[i][2]
    ex = batch[0]
    crec = ex.coord_sets[0]
    assert crec.size() == 1781
    assert list(crec.coords.tonumpy()[0]) == approx([45.042, 12.872, 13.001])
    assert crec.radii[0] == approx(1.8)
    assert list(crec.type_index.tonumpy())[:10] == [6.0, 1.0, 1.0, 7.0, 0.0, 6.0, 1.0, 1.0, 7.0, 1.0]
    clig = ex.coord_sets[1]
    assert clig.size() == 10
    assert list(clig.coords.tonumpy()[9]) == approx([27.0536, 3.2453, 32.4511])
    assert clig.radii[9] == approx(1.8)
    assert list(clig.type_index.tonumpy()) == [8.0, 1.0, 1.0, 9.0, 10.0, 0.0, 0.0, 1.0, 9.0, 8.0]
    assert crec.src == "4kqp/4kqp_rec_0.gninatypes"
    names = e.get_type_names()
    assert len(names) == 28 and names[0] == "0_AliphaticCarbonXSHydrophobe"
    assert names[14] == "1_AliphaticCarbonXSHydrophobe"
    a = np.array([0], dtype=np.float32)
    e.next_batch(1).extract_label(1, a)


def test_custom_typer_and_cache(molgrid):
    """test/test_example_provider.py:64-71 and 174-182: the same typer for every molecule; the
    ligand cache (.molcache2) gives what the structure files give."""
    t = molgrid.ElementIndexTyper(80)
    e = molgrid.ExampleProvider(t, data_root=datadir + "/structs")
    e.populate(datadir + "/small.types")
    assert e.next_batch(10)[0].coord_sets[0].max_type == 80
    e = molgrid.ExampleProvider(t, ligmolcache=datadir + "/lig.molcache2")
    e.populate(datadir + "/ligonly.types")
    c = e.next_batch(10)[0].coord_sets[1]
    assert c.max_type == 80 and c.type_index[0] == 7
    cached = molgrid.ExampleProvider(ligmolcache="lig.molcache2", data_root=datadir)
    files = molgrid.ExampleProvider(data_root=datadir + "/structs")
    cached.populate(datadir + "/ligonly.types")
    files.populate(datadir + "/ligonly.types")
    for a, b in zip(cached.next_batch(20), files.next_batch(20)):
        assert a.coord_sets[1] == b.coord_sets[1] and a.coord_sets[0].size() == 0
    with pytest.raises(ValueError):
        molgrid.ExampleProvider(ligmolcache=datadir + "/recmap")    # not a cache file
    bad = molgrid.ExampleProvider(data_root=datadir)
    bad.populate(datadir + "/ligonly.types")
    with pytest.raises(ValueError):
        bad.next()                                                  # structure file not found


def test_grouped_example_provider(molgrid):
    """test/test_example_provider.py:185-233"""
    fname = datadir + "/grouped.types"
    batch_size = 3

    def testprovider(e, gsize):
        for _ in range(10):
            batch = e.next_batch(batch_size)
            firstrecs = [ex.coord_sets[0].src for ex in batch]
            firstligs = [ex.coord_sets[1].src if len(ex.coord_sets) > 1 else None for ex in batch]
            grps = [ex.group for ex in batch]
            assert not any(x.seqcont for x in batch)
            for i in range(gsize - 1):
                batch = e.next_batch(batch_size)
                recs = [ex.coord_sets[0].src for ex in batch]
                ligs = [ex.coord_sets[1].src if len(ex.coord_sets) > 1 else None for ex in batch]
                for x, g in zip(batch, grps):
                    assert x.seqcont and x.group == g
                for r1, r2 in zip(firstrecs, recs):
                    if r2:
                        assert r1 == r2
                for l1, l2 in zip(firstligs, ligs):
                    assert l1 != l2

    e = molgrid.ExampleProvider(data_root=datadir + "/structs", max_group_size=5,
                                group_batch_size=batch_size)
    e.populate(fname)
    testprovider(e, 5)
    with pytest.raises(ValueError):
        e.next_batch(batch_size + 1)
    molgrid.set_random_seed(3)
    e = molgrid.ExampleProvider(data_root=datadir + "/structs", max_group_size=7,
                                group_batch_size=batch_size, shuffle=True, balanced=True)
    e.populate(fname)
    testprovider(e, 7)


def test_make_vector_types_and_sums(molgrid):
    """test/test_example_provider.py:236-301"""
    fname = datadir + "/ligonly.types"
    e = molgrid.ExampleProvider(molgrid.NullIndexTyper(), molgrid.defaultGninaLigandTyper,
                                data_root=datadir + "/structs", make_vector_types=True)
    e.populate(fname)
    b = e.next_batch(10)
    tv = b[0].merge_coordinates().type_vector.tonumpy()
    assert tv.shape == (10, 14) and tv[0].sum() == 1.0 and tv[0][8] == 1.0
    assert b[0].coord_sets[0].has_vector_types() and b[0].coord_sets[1].has_vector_types()
    assert b[0].num_types() == 14
    sums = molgrid.MGrid2f(10, e.num_types())
    b.sum_types(sums)
    np.testing.assert_allclose(sums[0].tonumpy(), [2., 3., 0., 0., 0., 0., 0., 0., 2., 2., 1., 0.,
                                                   0., 0.], atol=1e-5)
    e2 = molgrid.ExampleProvider(data_root=datadir + "/structs", make_vector_types=True)
    e2.populate(fname)
    b2 = e2.next_batch(10)
    assert b2[0].merge_coordinates(unique_index_types=True).type_vector.tonumpy().shape == (10, 28)
    assert e2.num_types() == b2[0].num_types()       # test_type_sizing: an empty set still counts
    sums = molgrid.MGrid2f(10, e2.num_types())
    b2.sum_types(sums)
    sums2 = np.zeros(sums.shape, np.float32)
    b2.sum_types(sums2)
    np.testing.assert_allclose(sums.tonumpy(), sums2, atol=1e-5)
    np.testing.assert_allclose(sums[0].tonumpy(), [0.] * 14 + [2., 3., 0., 0., 0., 0., 0., 0., 2.,
                                                              2., 1., 0., 0., 0.], atol=1e-5)


def test_copied_and_duplicated_examples(molgrid):
    """test/test_example_provider.py:304-332 (without the device transform) and 494-517"""
    fname = datadir + "/ligonly.types"
    e = molgrid.ExampleProvider(data_root=datadir + "/structs")
    e.populate(fname)
    b = e.next_batch(10)
    lig0 = b[0].coord_sets[1].coords.tonumpy()
    for i in range(1, 10):
        assert np.square(lig0 - b[i].coord_sets[1].coords.tonumpy()).sum() > 0
    e = molgrid.ExampleProvider(data_root=datadir + "/structs", num_copies=10)
    e.populate(fname)
    b = e.next_batch(10)
    lig0 = b[0].coord_sets[1].coords.tonumpy()
    for i in range(1, 10):
        assert np.square(lig0 - b[i].coord_sets[1].coords.tonumpy()).sum() == 0
    b[1].coord_sets[1].coords[0, 0] = 1000.0          # copies do not share memory
    assert np.array_equal(b[0].coord_sets[1].coords.tonumpy(), lig0)
    assert e.mem_caches_size() == 2

    fname = datadir + "/multilig.types"
    e = molgrid.ExampleProvider(data_root=datadir + "/structs")
    e.populate(fname)
    for ex in e.next_batch(10)[1:]:
        assert len(ex.coord_sets) == 3
        assert np.square(ex.coord_sets[1].coords.tonumpy()
                         - ex.coord_sets[2].coords.tonumpy()).sum() > 0
    e = molgrid.ExampleProvider(data_root=datadir + "/structs", duplicate_first=True)
    e.populate(fname)
    for ex in e.next_batch(10)[1:]:
        assert len(ex.coord_sets) == 4
        assert np.square(ex.coord_sets[1].coords.tonumpy()
                         - ex.coord_sets[3].coords.tonumpy()).sum() > 0
        assert ex.coord_sets[0] == ex.coord_sets[2]
    assert e.num_types() == 28     # two typers: the count does not grow with the duplicates


class _RefsOnly(object):
    """Stands in for the extractor where only the order of the examples matters: the full list
    names structure files that are not among the fixtures."""

    def extract(self, ref):
        import libmolgrid_amd as molgrid
        ex = molgrid.Example()
        ex.labels = list(ref.labels)
        for f in ref.files:
            c = molgrid.CoordinateSet()
            c.src = f
            ex.coord_sets.append(c)
        return ex


def test_iterator_interface_and_epochs(molgrid):
    """test/test_example_provider.py:335-354 and 520-610: epoch sizes and batch counts of the
    1000-line list under every sampling scheme."""
    fname = datadir + "/small.types"
    S = molgrid.IterationScheme

    def provider(**kw):
        e = molgrid.ExampleProvider(data_root=datadir + "/structs", **kw)
        e.extractor = _RefsOnly()
        e.populate(fname)
        return e

    e, e2 = provider(default_batch_size=25), provider(default_batch_size=25)
    labels, labels2 = molgrid.MGrid2f(25, 3), molgrid.MGrid2f(25, 3)
    for i, b in enumerate(e):
        b.extract_labels(labels.cpu())
        e2.next_batch().extract_labels(labels2.cpu())
        np.testing.assert_allclose(labels.tonumpy(), labels2.tonumpy())
        if i > 10:
            break

    e = provider(default_batch_size=10, iteration_scheme=S.LargeEpoch)
    assert e.small_epoch_size() == 1000 and e.large_epoch_size() == 1000
    assert sum(1 for _ in e) == 100
    e = provider(default_batch_size=10, balanced=True, iteration_scheme=S.LargeEpoch)
    assert e.small_epoch_size() == 326 and e.large_epoch_size() == 1674
    assert sum(1 for _ in e) == 168
    e = provider(default_batch_size=10, balanced=False, stratify_receptor=True,
                 iteration_scheme=S.SmallEpoch)
    assert e.small_epoch_size() == 120 and e.large_epoch_size() == 1260
    assert sum(1 for _ in e) == 12

    def walk(e, unique):
        values, cnt, small, large = set(), 0, 0, 0
        for batch in e:
            for ex in batch:
                key = ex.coord_sets[0].src + ":" + ex.coord_sets[1].src
                if unique:
                    assert key not in values    # a small epoch shows an example at most once
                values.add(key)
            cnt += 1
            s, l = e.get_small_epoch_num(), e.get_large_epoch_num()
            assert small <= s <= small + 1 and large <= l <= large + 1
            small, large = s, l
        return cnt, values

    e = provider(default_batch_size=8, balanced=True, stratify_receptor=True,
                 iteration_scheme=S.SmallEpoch)
    assert e.small_epoch_size() == 112 and e.large_epoch_size() == 2240
    assert walk(e, True)[0] == 14
    e = provider(default_batch_size=10, balanced=True, stratify_receptor=True,
                 iteration_scheme=S.LargeEpoch)
    assert e.small_epoch_size() == 112 and e.large_epoch_size() == 2240
    cnt, values = walk(e, False)
    assert cnt == 224 and len(values) == e.size()    # a large epoch shows everything


def test_shuffle_and_value_stratification(molgrid):
    """Properties of the schemes whose order depends on the random engine (the reference's
    engine is not reproduced: the order itself is not pinned)."""
    fname = datadir + "/small.types"
    molgrid.set_random_seed(5)
    e = molgrid.ExampleProvider(data_root=datadir + "/structs", shuffle=True)
    e.extractor = _RefsOnly()
    e.populate(fname)
    first = [ex.coord_sets[1].src for ex in e.next_batch(1000)]
    assert len(set(first)) == len(set(open(fname).read().split()[4::5]))     # a permutation
    assert first != sorted(first)
    second = [ex.coord_sets[1].src for ex in e.next_batch(1000)]
    assert sorted(first) == sorted(second) and first != second
    molgrid.set_random_seed(5)
    e2 = molgrid.ExampleProvider(data_root=datadir + "/structs", shuffle=True)
    e2.extractor = _RefsOnly()
    e2.populate(fname)
    assert [ex.coord_sets[1].src for ex in e2.next_batch(1000)] == first      # seeded
    # balanced batches alternate actives and decoys
    e = molgrid.ExampleProvider(data_root=datadir + "/structs", balanced=True, shuffle=True)
    e.extractor = _RefsOnly()
    e.populate(fname)
    assert [ex.labels[0] for ex in e.next_batch(20)] == [1.0, 0.0] * 10
    # bins of |label 1| take turns
    e = molgrid.ExampleProvider(data_root=datadir + "/structs", stratify_min=0, stratify_max=10,
                                stratify_step=5, stratify_pos=1)
    e.extractor = _RefsOnly()
    e.populate(fname)
    vals = [abs(ex.labels[1]) for ex in e.next_batch(40)]
    assert all(v < 5 for v in vals[0::2]) and all(v >= 5 for v in vals[1::2])
    with pytest.raises(ValueError):
        molgrid.ExampleProvider(no_such_setting=1)


def test_mem_caches(molgrid, tmp_path):
    """test/test_example_provider.py:41-61 with pre-typed files"""
    e = molgrid.ExampleProvider(data_root=datadir + "/structs")
    e2 = molgrid.ExampleProvider(data_root=datadir + "/structs")
    e.populate(datadir + "/small.types")
    e2.populate(datadir + "/small.types")
    assert e.mem_caches_size() == 0
    e.next()
    assert e.mem_caches_size() == 2
    f = str(tmp_path / "caches")
    e.save_mem_caches(f)
    e.load_mem_caches(f)
    e2.load_mem_caches(f)
    assert e.mem_caches_size() == 2 and e2.mem_caches_size() == 2
    e.next()
    first = e2.next()
    assert e.mem_caches_size() == 3 and e2.mem_caches_size() == 2      # same receptor, new ligand
    assert first.coord_sets[0].size() == 1781


def test_example_ref_parsing(molgrid):
    """src/example.cpp:301-343"""
    r = molgrid.ExampleRef("1 6.05 0.162643 a/rec.gninatypes a/lig.gninatypes # comment x.sdf")
    assert r.labels == [1.0, 6.05, 0.162643] and r.files == ["a/rec.gninatypes", "a/lig.gninatypes"]
    r = molgrid.ExampleRef("3 0 -6.05 rec lig", -1, True)
    assert r.group == 3 and r.labels == [0.0, -6.05] and r.files == ["rec", "lig"]
    r = molgrid.ExampleRef("1 2 3 rec lig", 1)
    assert r.labels == [1.0] and r.files == ["2", "3", "rec", "lig"]
    r = molgrid.ExampleRef("none lig.gninatypes")
    assert r.labels == [] and r.files == ["none", "lig.gninatypes"]
    with pytest.raises(ValueError):
        molgrid.ExampleRef("1 2 # nothing")


# ---- grid files (test/test_gridio.py) --------------------------------------------------------
def test_dx_round_trip(molgrid, tmp_path):
    rng = np.random.default_rng(2)
    g = rng.random((4, 9, 9, 9), dtype=np.float32)
    center = (1.25, -3.5, 10.0)
    f = str(tmp_path / "tmp.dx")
    molgrid.write_dx(f, molgrid.Grid3f(g[0]), center, 0.5)
    text = open(f).read().split("\n")
    assert text[0] == "object 1 class gridpositions counts 9 9  9"
    assert text[1] == "origin -0.75000 -5.50000 8.00000"
    assert text[2] == "delta 0.50000 0 0" and text[4] == "delta 0 0 0.50000"
    assert text[6] == "object 3 class array type double rank 0 items [ 729] data follows"
    assert text[7] == "%.5f %.5f %.5f" % tuple(g[0].reshape(-1)[:3])
    back = molgrid.read_dx(f)
    np.testing.assert_array_almost_equal(back.grid().tonumpy(), g[0], decimal=5)
    assert tuple(back.center()) == approx(center) and back.resolution() == 0.5
    names = ["a", "b", "c", "d"]
    prefix = str(tmp_path / "all")
    molgrid.write_dx_grids(prefix, names, g, center, 0.5, 0.5)
    check = molgrid.MGrid4f(4, 9, 9, 9)
    molgrid.read_dx_grids(prefix, names, check.cpu())
    np.testing.assert_array_almost_equal(g, 2.0 * check.tonumpy(), decimal=5)
    with pytest.raises(ValueError):
        molgrid.write_dx_grids(prefix, names[:3], g, center, 0.5)
    with pytest.raises(ValueError):
        molgrid.read_dx(f, np.zeros((8, 8, 8), np.float32))
    assert tuple(back.grid2cart(0, 0, 0)) == approx((1.25 - 2.25, -3.5 - 2.25, 10.0 - 2.25))


def test_write_map(molgrid, tmp_path):
    g = np.arange(27, dtype=np.float32).reshape(3, 3, 3) / 7
    f = str(tmp_path / "x.map")
    molgrid.write_map(f, g, (0, 1, 2), 0.375)
    lines = open(f).read().split("\n")
    assert lines[:3] == ["GRID_PARAMETER_FILE", "GRID_DATA_FILE", "MACROMOLECULE"]
    assert lines[3] == "SPACING 0.375" and lines[4] == "NELEMENTS 2 2 2" and lines[5] == "CENTER 0 1 2"
    assert lines[6] == "0" and lines[7] == "%.5g" % g[1, 0, 0] and lines[9] == "%.5g" % g[0, 1, 0]
    assert len(lines) == 6 + 27 + 1


# ---- datasets over example lists (test/test_example_provider.py:357-492) --------------------
def test_example_dataset_and_map_dataset(molgrid):
    """test/test_example_provider.py:357-406 on the examples whose structure files are among the
    fixtures (the first 120 lines of the list)."""
    fname = datadir + "/small.types"
    e = molgrid.ExampleProvider(data_root=datadir + "/structs")
    e.populate(fname)
    m = molgrid.MolMapDataset(fname, data_root=datadir + "/structs")
    assert len(m) == 1000
    assert m.examples.num_labels() == 3 and m.examples.num_types() == 28
    ex = e.next()
    coordinates = ex.merge_coordinates()
    length, center, coords, types, radii, labels = m[0]
    assert length == 1791 and list(center.shape) == [3]
    np.testing.assert_allclose(center, list(ex.coord_sets[-1].center()))
    np.testing.assert_allclose(coords, coordinates.coords.tonumpy())
    np.testing.assert_allclose(types, coordinates.type_index.tonumpy())
    np.testing.assert_allclose(radii, coordinates.radii.tonumpy())
    assert len(labels) == 3 and labels[0] == 1
    np.testing.assert_allclose(labels[1], 6.05)
    np.testing.assert_allclose(labels[-1], 0.162643)
    ref = m.examples.provider[len(m) - 1]                         # the last line of the list
    assert ref.labels[0] == 0 and ref.labels[1] == approx(-10.3)
    with pytest.raises(IndexError):
        m.examples[1000]

    loader = torch.utils.data.DataLoader(m, batch_size=8,
                                         collate_fn=molgrid.MolMapDataset.collateMolDataset)
    it = iter(loader)
    next(it)
    lengths, center, coords, types, radii, labels = next(it)
    for t in (lengths, center, coords, types, radii, labels):
        assert t.shape[0] == 8
    mlength, mcenter, mcoords, mtypes, mradii, mlabels = m[10]
    n = int(lengths[2])
    assert n == mlength
    np.testing.assert_allclose(center[2], mcenter)
    np.testing.assert_allclose(coords[2][:n], mcoords)
    np.testing.assert_allclose(types[2][:n], mtypes)
    np.testing.assert_allclose(radii[2][:n], mradii)
    assert float(radii[2][n:].abs().sum()) == 0                    # padded with zeros
    assert labels[2].tolist() == mlabels.tolist()


def test_iterable_dataset_and_pickling(molgrid):
    """test/test_example_provider.py:408-470 (single process) and the datasets' pickling."""
    import pickle
    fname = datadir + "/small.types"
    bsize = 25
    e = molgrid.ExampleProvider(data_root=datadir + "/structs", default_batch_size=bsize)
    e.populate(fname)
    m = molgrid.MolIterDataset(fname, data_root=datadir + "/structs", default_batch_size=bsize)
    it = iter(m)
    coordinates = e.next().merge_coordinates()
    lengths, centers, coords, types, radii, labels = next(it)
    assert list(centers.shape) == [bsize, 3]
    n = int(lengths[0])
    np.testing.assert_allclose(coords[0, :n, :], coordinates.coords.tonumpy())
    np.testing.assert_allclose(types[0, :n], coordinates.type_index.tonumpy())
    np.testing.assert_allclose(radii[0, :n], coordinates.radii.tonumpy())
    assert len(labels) == bsize and len(labels[0]) == 3 and labels[0, 0] == 1
    np.testing.assert_allclose(labels[0, 1], 6.05)
    np.testing.assert_allclose(labels[0, -1], 0.162643)

    m.examples.reset()
    loader = torch.utils.data.DataLoader(m, batch_size=None)
    it = iter(loader)
    next(it)
    lengths, center, coords, types, radii, labels = next(it)
    for t in (lengths, center, coords, types, radii, labels):
        assert t.shape[0] == bsize
    e.reset()
    e.next_batch()
    ex = e.next_batch()
    coordinates = ex[2].merge_coordinates()
    n = int(lengths[2])
    np.testing.assert_allclose(center[2], np.array(list(ex[2].coord_sets[-1].center())))
    np.testing.assert_allclose(coords[2, :n], coordinates.coords.tonumpy())
    np.testing.assert_allclose(types[2, :n], coordinates.type_index.tonumpy())
    np.testing.assert_allclose(radii[2, :n], coordinates.radii.tonumpy())
    assert labels[2].tolist() == [approx(v) for v in ex[2].labels]

    with pytest.raises(NotImplementedError):
        len(m)                                                     # continuous: no length
    small = molgrid.MolIterDataset(fname, data_root=datadir + "/structs", default_batch_size=bsize,
                                   iteration_scheme=molgrid.IterationScheme.SmallEpoch)
    assert len(small) == 1000 // bsize
    large = molgrid.MolIterDataset(fname, data_root=datadir + "/structs", default_batch_size=30,
                                   iteration_scheme=molgrid.IterationScheme.LargeEpoch)
    assert len(large) == 34

    again = pickle.loads(pickle.dumps(small))
    assert len(again) == len(small) and again.examples.settings().default_batch_size == bsize
    a, b = next(iter(again)), next(iter(small))
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    mm = pickle.loads(pickle.dumps(molgrid.MolMapDataset(fname, data_root=datadir + "/structs")))
    assert len(mm) == 1000 and mm[3][0] == mm[3][2].shape[0]
    typed = molgrid.MolMapDataset(fname, data_root=datadir + "/structs",
                                  typers=(molgrid.defaultGninaReceptorTyper,
                                          molgrid.defaultGninaLigandTyper))
    with pytest.raises(NotImplementedError):
        pickle.dumps(typed)


def test_tensor_as_grid_and_make_ndarray(molgrid):
    """python/torch_bindings.py:9-43"""
    t = torch.zeros(3, 4, 5)
    g = molgrid.tensor_as_grid(t)
    assert type(g).__name__ == "Grid3f" and g.shape == (3, 4, 5)
    assert type(molgrid.tensor_as_grid(t.double()[0])).__name__ == "Grid2d"
    with pytest.raises(ValueError):
        molgrid.tensor_as_grid(torch.zeros(3, dtype=torch.int32))
    assert molgrid.GridMaker.make_ndarray is molgrid.make_grid_ndarray
    assert molgrid.GridMaker.make_tensor is molgrid.make_grid_tensor


def test_labels_into_tensors(molgrid):
    """test/test_torch.py:102-126"""
    e = molgrid.ExampleProvider(data_root=datadir + "/structs")
    e.populate(datadir + "/small.types")
    batch = e.next_batch(100)
    assert e.num_labels() == 3
    labels = torch.zeros((100, 3), dtype=torch.float32)
    batch.extract_labels(labels)
    label0 = torch.zeros(100, dtype=torch.float32)
    batch.extract_label(0, label0)
    assert label0[0] == 1 and labels[0, 0] == 1
    assert float(labels[0][1]) == approx(6.05)
    assert float(labels[0][2]) == approx(0.162643)
    for i in range(100):
        assert label0[i] == labels[i][0]
