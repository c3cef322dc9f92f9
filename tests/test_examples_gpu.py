"""Examples through the gridding calls (include/libmolgrid/grid_maker.h:153-201): an example is
merged, transformed and gridded about the transform's centre; a batch of examples draws its
transforms example by example and is gridded with one launch."""
import numpy as np
import pytest
import torch
from pytest import approx

import oracle
from util import assert_close, dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def molgrid():
    import libmolgrid_amd
    return libmolgrid_amd


def make_example(molgrid, seed, nrec=60, nlig=9):
    rng = np.random.default_rng(seed)
    ex = molgrid.Example()
    rec = molgrid.CoordinateSet(rng.uniform(-6, 6, (nrec, 3)).astype(np.float32),
                                rng.integers(0, 5, nrec).astype(np.float32),
                                rng.uniform(1.2, 2.0, nrec).astype(np.float32), 5)
    lig = molgrid.CoordinateSet(rng.uniform(-2, 3, (nlig, 3)).astype(np.float32),
                                rng.integers(0, 3, nlig).astype(np.float32),
                                rng.uniform(1.2, 2.0, nlig).astype(np.float32), 3)
    ex.coord_sets = [rec, lig]
    ex.labels = [float(seed % 2), 0.25 * seed]
    return ex


def test_coordset_transform_on_device(molgrid):
    """test/test_coordinateset.py:69-88"""
    coords = np.array([[1, 0, -1], [1, 3, -1], [1, 0, -1]], np.float32)
    c = molgrid.CoordinateSet(coords, np.array([3, 2, 1], np.float32),
                              np.array([1.5, 1.5, 1.0], np.float32), 4)
    t = molgrid.Transform(molgrid.Quaternion(), (0, 0, 0), (-1, 0, 1))
    t.forward(c, c)
    assert c.coords[1, 1] == 3.0
    assert np.sum(c.coords.tonumpy()) == approx(3.0)
    c.togpu()
    assert c.coords.ongpu() and c.radii.ongpu()
    t.backward(c, c)
    assert np.array_equal(c.coords.tonumpy(), coords)
    cd = molgrid.CoordinateSet(dev(coords), dev(np.array([3, 2, 1], np.float32)),
                               dev(np.array([1.5, 1.5, 1.0], np.float32)), 4)
    assert cd.coords.ongpu() and cd.size() == 3


def test_forward_example_with_transform(molgrid):
    ex = make_example(molgrid, 3)
    gm = molgrid.GridMaker(0.5, 11.5)
    q = np.random.default_rng(1).normal(size=4)
    T = molgrid.Transform(molgrid.Quaternion(*(q / np.linalg.norm(q))), (0.5, -0.25, 1.0),
                          (0.3, 0.2, -0.1))
    out = torch.empty(gm.grid_dimensions(8), device="cuda")
    gm.forward(ex, T, out)
    m = ex.merge_coordinates()
    moved = oracle.transform_forward(q / np.linalg.norm(q), (0.5, -0.25, 1.0), (0.3, 0.2, -0.1),
                                     m.coords.tonumpy())
    ref = oracle.GridMaker(0.5, 11.5).forward((0.5, -0.25, 1.0), moved, m.type_index.tonumpy(),
                                              m.radii.tonumpy(), 8)
    assert_close(out.cpu().numpy(), ref, what="forward(example, transform)")
    assert np.array_equal(ex.coord_sets[0].coords.tonumpy(),
                          make_example(molgrid, 3).coord_sets[0].coords.tonumpy())   # untouched
    host = molgrid.MGrid4f(*gm.grid_dimensions(8))
    gm.forward(ex, T, host.cpu())
    assert np.array_equal(host.tonumpy(), out.cpu().numpy())
    with pytest.raises(IndexError):
        gm.forward(ex, T, torch.empty(gm.grid_dimensions(7), device="cuda"))


def test_forward_example_default_center(molgrid):
    """Without a centre the grid sits on the centre of the last coordinate set."""
    ex = make_example(molgrid, 5)
    gm = molgrid.GridMaker(0.5, 11.5)
    out = torch.empty(gm.grid_dimensions(8), device="cuda")
    gm.forward(ex, out)
    m = ex.merge_coordinates()
    center = tuple(ex.coord_sets[1].center())
    ref = oracle.GridMaker(0.5, 11.5).forward(center, m.coords.tonumpy(), m.type_index.tonumpy(),
                                              m.radii.tonumpy(), 8)
    assert_close(out.cpu().numpy(), ref, what="forward(example)")
    out2 = torch.empty_like(out)
    gm.forward(ex, out2, center=(0, 0, 0))
    ref2 = oracle.GridMaker(0.5, 11.5).forward((0, 0, 0), m.coords.tonumpy(),
                                               m.type_index.tonumpy(), m.radii.tonumpy(), 8)
    assert_close(out2.cpu().numpy(), ref2, what="forward(example, center)")


def test_forward_batch_of_examples(molgrid):
    """One launch for the batch gives what the reference's loop over the examples gives: the same
    random transforms in the same order, the same grids bit for bit."""
    batch = molgrid.ExampleVec([make_example(molgrid, s, nrec=40 + 7 * s) for s in range(6)])
    gm = molgrid.GridMaker(0.5, 11.5)
    out = torch.empty((6,) + gm.grid_dimensions(8), device="cuda")
    molgrid.set_random_seed(17)
    gm.forward(batch, out, random_translation=2.0, random_rotation=True)
    one = torch.empty_like(out)
    molgrid.set_random_seed(17)
    for i, ex in enumerate(batch):
        gm.forward(ex, one[i], random_translation=2.0, random_rotation=True)
    assert torch.equal(out, one)
    assert float(out.sum()) > 0
    # no randomness: each grid is the example about its ligand's centre
    gm.forward(batch, out)
    m = batch[2].merge_coordinates()
    ref = oracle.GridMaker(0.5, 11.5).forward(tuple(batch[2].coord_sets[1].center()),
                                              m.coords.tonumpy(), m.type_index.tonumpy(),
                                              m.radii.tonumpy(), 8)
    assert_close(out[2].cpu().numpy(), ref, what="forward(batch)")
    with pytest.raises(IndexError):
        gm.forward(batch, torch.empty((5,) + gm.grid_dimensions(8), device="cuda"))
    labels = torch.empty((6, 2), device="cuda")
    batch.extract_labels(labels)
    assert labels[3].tolist() == [1.0, 0.75]


def test_backward_with_coordinate_set(molgrid):
    ex = make_example(molgrid, 8)
    m = ex.merge_coordinates()
    gm = molgrid.GridMaker(0.5, 11.5)
    diff = torch.randn(gm.grid_dimensions(8), device="cuda")
    grads = molgrid.MGrid2f(m.size(), 3)
    gm.backward((0, 0, 0), m, diff, grads.gpu())
    direct = torch.empty((m.size(), 3), device="cuda")
    gm.backward((0, 0, 0), dev(m.coords.tonumpy()), dev(m.type_index.tonumpy()),
                dev(m.radii.tonumpy()), diff, direct)
    assert np.array_equal(grads.tonumpy(), direct.cpu().numpy())


def test_training_loop_from_example_provider(molgrid):
    """The loop of the reference's README: a provider over an example list, a batch gridded into a
    device tensor with random rotations and translations, labels extracted to the device
    (test/test_example_provider.py:74-123, test/test_gridmaker.py:86-100)."""
    import os
    datadir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "molgrid_data")
    e = molgrid.ExampleProvider(data_root=datadir + "/structs", balanced=True, shuffle=True)
    molgrid.set_random_seed(0)
    e.populate(datadir + "/small.types")
    for part in (e.provider.actives, e.provider.decoys):      # structure files among the fixtures
        part.all = [r for r in part.all
                    if all(os.path.exists(datadir + "/structs/" + f) for f in r.files)]
        assert len(part.all) >= 12
    gmaker = molgrid.GridMaker()
    dims = gmaker.grid_dimensions(e.num_types())
    assert dims == (28, 48, 48, 48)
    batch_size = 8
    tensor = torch.zeros((batch_size,) + dims, dtype=torch.float32, device="cuda")
    labels = torch.zeros(batch_size, dtype=torch.float32, device="cuda")
    for _ in range(3):
        batch = e.next_batch(batch_size)
        gmaker.forward(batch, tensor, random_translation=2.0, random_rotation=True)
        batch.extract_label(0, labels)
        assert labels.tolist() == [1.0, 0.0] * 4
        per_example = tensor.reshape(batch_size, -1).sum(1)
        assert bool((per_example > 100).all())
    # without randomness the grid is the oracle's grid about the ligand's centre
    ex = batch[0]
    out = torch.empty(dims, device="cuda")
    gmaker.forward(ex, out)
    m = ex.merge_coordinates()
    ref = oracle.GridMaker(0.5, 23.5).forward(tuple(ex.coord_sets[1].center()), m.coords.tonumpy(),
                                              m.type_index.tonumpy(), m.radii.tonumpy(), 28)
    assert_close(out.cpu().numpy(), ref, what="example from the provider")


def test_vector_typed_examples_with_type_radii(molgrid):
    """test/test_example_provider.py:236-265: one-hot type vectors with radii per type."""
    import os
    datadir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "molgrid_data")
    e = molgrid.ExampleProvider(molgrid.NullIndexTyper(), molgrid.defaultGninaLigandTyper,
                                data_root=datadir + "/structs", make_vector_types=True)
    e.populate(datadir + "/ligonly.types")
    b = e.next_batch(10)
    gmaker = molgrid.GridMaker(dimension=23.5, radius_type_indexed=True)
    shape = gmaker.grid_dimensions(molgrid.defaultGninaLigandTyper.num_types())
    mgrid = molgrid.MGrid5f(10, *shape)
    gmaker.forward(b, mgrid.gpu())
    # the same atoms through index types and per-atom radii
    e2 = molgrid.ExampleProvider(molgrid.NullIndexTyper(), molgrid.defaultGninaLigandTyper,
                                 data_root=datadir + "/structs")
    e2.populate(datadir + "/ligonly.types")
    b2 = e2.next_batch(10)
    plain = torch.empty((10,) + shape, device="cuda")
    molgrid.GridMaker(dimension=23.5).forward(b2, plain)
    assert_close(mgrid.tonumpy(), plain.cpu().numpy(), what="type-indexed radii vs per-atom radii")
    assert float(plain.sum()) > 0


def test_datasets_grid_like_the_provider(molgrid):
    """test/test_example_provider.py:357-492: padded batches from the two datasets gridded with the
    tensor overload equal the provider's examples gridded directly; random transforms in a dataset
    are rigid motions about the last coordinate set's centre."""
    import os
    datadir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "molgrid_data")
    fname = datadir + "/small.types"
    bsize = 8
    e = molgrid.ExampleProvider(data_root=datadir + "/structs", default_batch_size=bsize)
    e.populate(fname)
    m = molgrid.MolIterDataset(fname, data_root=datadir + "/structs", default_batch_size=bsize)
    it = iter(m)
    next(it)
    lengths, center, coords, types, radii, labels = next(it)
    e.next_batch()
    ex = e.next_batch()
    gmaker = molgrid.GridMaker()
    shape = gmaker.grid_dimensions(e.num_types())
    mgridg = molgrid.MGrid5f(bsize, *shape)
    gmaker.forward(center.cuda(), coords.cuda(), types.cuda(), radii.cuda(), mgridg.gpu())
    egrid = molgrid.MGrid5f(bsize, *shape)
    gmaker.forward(ex, egrid.gpu())
    np.testing.assert_allclose(mgridg.tonumpy(), egrid.tonumpy(), atol=1e-5)
    assert float(egrid.tonumpy().sum()) > 1000

    mm = molgrid.MolMapDataset(fname, data_root=datadir + "/structs")
    loader = torch.utils.data.DataLoader(mm, batch_size=bsize,
                                         collate_fn=molgrid.MolMapDataset.collateMolDataset)
    it = iter(loader)
    next(it)
    lengths, center, coords, types, radii, labels = next(it)
    mgrid = molgrid.MGrid5f(bsize, *shape)
    gmaker.forward(center.cuda(), coords.cuda(), types.cuda(), radii.cuda(), mgrid.gpu())
    np.testing.assert_allclose(mgrid.tonumpy(), egrid.tonumpy(), atol=1e-5)
    one = gmaker.make_tensor(tuple(ex[2].coord_sets[-1].center()), ex[2].merge_coordinates())
    assert tuple(one.shape) == shape and one.is_cuda
    np.testing.assert_allclose(one.cpu().numpy(), egrid.tonumpy()[2], atol=1e-5)
    arr = gmaker.make_ndarray(tuple(ex[2].coord_sets[-1].center()), ex[2].merge_coordinates())
    np.testing.assert_allclose(arr, egrid.tonumpy()[2], atol=1e-5)

    mlength, mcenter, mcoords, mtypes, mradii, mlabels = mm[10]
    molgrid.set_random_seed(3)
    r = molgrid.MolMapDataset(fname, data_root=datadir + "/structs", random_translation=2.0,
                              random_rotation=True)
    rl, rc, rcoords, rtypes, rradii, rlabels = r[10]
    np.testing.assert_allclose(rc, mcenter)
    assert rtypes.tolist() == mtypes.tolist() and rlabels.tolist() == mlabels.tolist()
    d0 = torch.cdist(mcoords[:20], mcoords[:20])
    d1 = torch.cdist(rcoords[:20], rcoords[:20])
    np.testing.assert_allclose(d0, d1, atol=2e-3)
    assert float((rcoords - mcoords).abs().max()) > 0.5


def test_training_a_small_network_on_gridded_batches(molgrid):
    """The reference's end-to-end training test (test/test_torch_cnn.py) on the examples whose
    structure files are among the fixtures: balanced, shuffled batches gridded straight into a
    device tensor, labels extracted, a small network trained until it separates the classes.
    (Pooling and linear layers instead of the reference's 3-D convolutions keep the test short.)"""
    import os
    import torch.nn as nn
    import torch.nn.functional as F
    datadir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "molgrid_data")
    molgrid.set_random_seed(0)
    torch.manual_seed(0)
    e = molgrid.ExampleProvider(data_root=datadir + "/structs", balanced=True, shuffle=True)
    e.populate(datadir + "/small.types")
    for part in (e.provider.actives, e.provider.decoys):
        part.all = [r for r in part.all
                    if all(os.path.exists(datadir + "/structs/" + f) for f in r.files)][:12]
        assert len(part.all) == 12
    gmaker = molgrid.GridMaker()
    dims = gmaker.grid_dimensions(e.num_types())
    batch_size = 24
    model = nn.Sequential(nn.MaxPool3d(4), nn.Flatten(),
                          nn.Linear(dims[0] * (dims[1] // 4) ** 3, 64), nn.ReLU(),
                          nn.Linear(64, 2)).to("cuda")
    optimizer = torch.optim.SGD(model.parameters(), lr=0.01, momentum=0.9)
    input_tensor = torch.zeros((batch_size,) + dims, dtype=torch.float32, device="cuda")
    float_labels = torch.zeros(batch_size, dtype=torch.float32)
    losses = []
    for _ in range(60):
        batch = e.next_batch(batch_size)
        gmaker.forward(batch, input_tensor, 0, random_rotation=False)
        batch.extract_label(0, float_labels)
        labels = float_labels.long().to("cuda")
        assert int(labels.sum()) == batch_size // 2                # balanced
        optimizer.zero_grad()
        loss = F.cross_entropy(model(input_tensor), labels)
        loss.backward()
        optimizer.step()
        losses.append(loss.item())
    assert np.mean(losses[-5:]) < 0.4 < losses[0]
