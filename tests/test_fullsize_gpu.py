"""The benchmark workload at its full size (batch 50, 28x48^3, 121,231 atoms) through the C ABI:
every example of the forward pass against the oracle, the gradients of a few examples against the
oracle, and properties that need no oracle (a batch equals its single launches, reordering atoms
leaves the binary grid unchanged, the backward pass is linear in the upstream gradient)."""
import numpy as np
import pytest
import torch

import oracle
import synth
from test_backward_gpu import EPS, check_grads, noise_bound
from util import assert_close, dev, parity_stats

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mg():
    import libmolgrid_amd
    return libmolgrid_amd


@pytest.fixture(scope="module")
def workload():
    c = synth.config1(nbatch=50)
    c["moved"] = oracle.transform_forward_batch(c["offsets"], c["quats"], c["centers"],
                                                c["translations"], c["coords"])
    return c


def test_forward_every_example(mg, workload):
    c = workload
    B = len(c["offsets"]) - 1
    threads = min(oracle.max_threads(), 16)
    gm = mg.GridMaker(0.5, 23.5)
    moved, types, radii = dev(c["moved"]), dev(c["types"]), dev(c["radii"])
    out = torch.full((B,) + gm.grid_dimensions(28), -1.0, device="cuda")
    gm.forward_batch(c["offsets"], c["centers"], moved, types, radii, out)
    og = oracle.GridMaker(0.5, 23.5)
    off = c["offsets"]
    for b0 in range(0, B, 10):       # ten examples at a time keeps the host copies small
        ref = og.forward_batch(off[b0:b0 + 11] - off[b0], c["centers"][b0:b0 + 10],
                               c["moved"][off[b0]:off[b0 + 10]], c["types"][off[b0]:off[b0 + 10]],
                               c["radii"][off[b0]:off[b0 + 10]], 28, nthreads=threads)
        got = out[b0:b0 + 10].cpu().numpy()
        for k in range(ref.shape[0]):
            assert_close(got[k], ref[k], what="example %d" % (b0 + k))
    # a batch is its single launches, bit for bit
    for b in (0, 17, 49):
        s = slice(off[b], off[b + 1])
        one = torch.empty(gm.grid_dimensions(28), device="cuda")
        gm.forward(tuple(c["centers"][b]), moved[s], types[s], radii[s], one)
        assert torch.equal(one, out[b])


def test_binary_grid_ignores_atom_order(mg, workload):
    c = workload
    B = len(c["offsets"]) - 1
    gm = mg.GridMaker(0.5, 23.5, True)
    out = torch.empty((B,) + gm.grid_dimensions(28), device="cuda")
    gm.forward_batch(c["offsets"], c["centers"], dev(c["moved"]), dev(c["types"]), dev(c["radii"]),
                     out)
    rng = np.random.default_rng(4)
    perm = np.concatenate([c["offsets"][b] + rng.permutation(c["offsets"][b + 1] - c["offsets"][b])
                           for b in range(B)])
    out2 = torch.empty_like(out)
    gm.forward_batch(c["offsets"], c["centers"], dev(c["moved"][perm]), dev(c["types"][perm]),
                     dev(c["radii"][perm]), out2)
    assert torch.equal(out, out2)
    vals = torch.unique(out)
    assert vals.tolist() == [0.0, 1.0]


def test_backward_full_batch(mg, workload):
    c = workload
    B = len(c["offsets"]) - 1
    off = c["offsets"]
    gm = mg.GridMaker(0.5, 23.5)
    gen = torch.Generator(device="cuda").manual_seed(5)
    diff = torch.randn((B,) + gm.grid_dimensions(28), device="cuda", generator=gen)
    moved, types, radii = dev(c["moved"]), dev(c["types"]), dev(c["radii"])
    grads = torch.empty((off[-1], 3), device="cuda")
    gm.backward_batch(off, c["centers"], moved, types, radii, diff, grads)
    got = grads.cpu().numpy()
    og = oracle.GridMaker(0.5, 23.5)
    d = diff.cpu().numpy()
    ref32 = og.backward_batch(off, c["centers"], c["moved"], c["types"], c["radii"], d, nthreads=8)
    ref64, mag = [], []
    for b in range(B):                          # every example of the batch
        s = slice(off[b], off[b + 1])
        args = (c["centers"][b], c["moved"][s], c["types"][s], c["radii"][s], d[b])
        ref64.append(og.backward(*args, f64=True))
        mag.append(noise_bound(og, *args))
    ref64, mag = np.concatenate(ref64), np.concatenate(mag)
    check_grads(got, ref32, ref64, mag, "batch of 50")
    # what is measured (values quoted are those of this batch on MI355X): against the sums in
    # double, the kernel is off by at most 4.4e-6 and 0.09 % of the 363,693 components lie outside
    # 1e-6 + 1e-5*|ref|; the reference's own float loop is off by up to 1.8e-5 with 0.10 % outside
    gpu64, cpu64 = parity_stats(got, ref64), parity_stats(ref32, ref64)
    gpu32 = parity_stats(got, ref32)
    print("\nbackward parity, %d components: gpu vs f64 sums %s; gpu vs float loop %s; float loop "
          "vs f64 sums %s" % (gpu64["n"], gpu64, gpu32, cpu64))
    assert gpu64["max_abs"] <= 1e-5 and gpu64["outside"] <= 0.002 * gpu64["n"]
    excess = np.maximum(np.abs(got - ref64) - (1e-6 + 1e-5 * np.abs(ref64)), 0) / (EPS * mag)
    assert float(excess.max()) <= 16.0          # measured: 11.9
    # the launch that also un-rotates gives what backward + Transform.backward give, bit for bit
    quats, zeros = dev(c["quats"]), dev(np.zeros_like(c["centers"]))
    two_calls = grads.clone()
    mg.transform_batch(off, quats, dev(c["centers"]), zeros, two_calls, two_calls, dotranslate=False,
                       inverse=True)
    fused = torch.empty_like(grads)
    gm.backward_batch(off, c["centers"], moved, types, radii, diff, fused,
                      unrotate=(quats, dev(c["centers"])))
    assert torch.equal(fused, two_calls)
    # linear in the upstream gradient: a factor of two is exact in floating point
    grads2 = torch.empty_like(grads)
    gm.backward_batch(off, c["centers"], moved, types, radii, diff * 2, grads2)
    assert torch.equal(grads2, grads * 2)


def test_vector_types_full_size_properties(mg):
    """Configuration 3 at its full size (16 x 10,000 atoms into 28x96^3) without the oracle: the
    grid is linear in the type vectors, one example of the batch equals its single launch, and a
    one-hot type vector gives the index-typed grid."""
    v = synth.vector_batch()
    B = len(v["offsets"]) - 1
    gm = mg.GridMaker(0.25, 23.75)
    dims = gm.grid_dimensions(28)
    coords, radii = dev(v["coords"]), dev(v["radii"])
    w = dev(v["types"])
    off = v["offsets"]

    def grid(weights, rows=slice(0, B)):
        n0, n1 = int(off[rows.start]), int(off[rows.stop])
        o = torch.empty((rows.stop - rows.start,) + dims, device="cuda")
        gm.forward_batch(off[rows.start:rows.stop + 1] - off[rows.start],
                         v["centers"][rows], coords[n0:n1], weights[n0:n1], radii[n0:n1], o)
        return o

    full = grid(w)
    assert float(full.min()) >= 0.0 and float(full.max()) > 0.5
    # linear in the weights (scaling by a power of two is exact)
    assert torch.equal(grid(0.5 * w, slice(3, 5)), 0.5 * full[3:5])
    gen = torch.Generator(device="cuda").manual_seed(2)
    w2 = torch.rand(w.shape, device="cuda", generator=gen)
    both = grid(w + w2, slice(6, 8))
    parts = full[6:8] + grid(w2, slice(6, 8))
    assert float((both - parts).abs().max()) <= 1e-6 + 2e-5 * float(parts.abs().max())
    # an example of the batch is its single launch
    s = slice(int(off[9]), int(off[10]))
    one = torch.empty(dims, device="cuda")
    gm.forward(tuple(v["centers"][9]), coords[s], w[s], radii[s], one)
    assert torch.equal(one, full[9])
    # one-hot weights: the index-typed grid
    types = torch.randint(0, 28, (int(off[1]),), device="cuda")
    hot = torch.zeros((int(off[1]), 28), device="cuda")
    hot[torch.arange(int(off[1]), device="cuda"), types] = 1.0
    a = torch.empty(dims, device="cuda")
    b = torch.empty(dims, device="cuda")
    gm.forward(tuple(v["centers"][0]), coords[:int(off[1])], hot, radii[:int(off[1])], a)
    gm.forward(tuple(v["centers"][0]), coords[:int(off[1])], types.float(), radii[:int(off[1])], b)
    err = (a - b).abs()
    assert float((err - 1e-5 * b.abs()).max()) <= 1e-6


@pytest.mark.parametrize("binary", [False, True])
def test_vector_types_full_size_example_vs_oracle(mg, binary):
    """One whole example of configuration 3 (10,000 atoms, 28 soft types, 28x96^3) against the CPU
    loop (src/grid_maker.cpp:214-271): densities within 1e-6 + 1e-5*|ref|, binary occupancy (sums
    of about 35 weights per voxel, added four atoms per matrix-core step) bit for bit."""
    v = synth.vector_batch(nbatch=1, natoms=10000)
    ref = oracle.GridMaker(0.25, 23.75, binary).forward_batch(
        v["offsets"], v["centers"], v["coords"], v["types"], v["radii"], 28, nthreads=8)
    gm = mg.GridMaker(0.25, 23.75, binary)
    out = torch.empty((1,) + gm.grid_dimensions(28), device="cuda")
    gm.forward_batch(v["offsets"], v["centers"], dev(v["coords"]), dev(v["types"]),
                     dev(v["radii"]), out)
    got = out.cpu().numpy()
    if binary:
        assert float(ref.max()) > 1.0
        assert np.array_equal(got, ref)
    else:
        assert_close(got, ref, what="config 3, full example")


def test_interpolation_full_size_properties(mg):
    """Configuration 4 at its full size (50 x 28x48^3) without the oracle: the identity gives the
    input back, a quarter turn about z through the grid centre is a permutation of the voxels,
    resampling is linear in the input, and a batch equals its single launches."""
    B, K, D = 50, 28, 48
    gen = torch.Generator(device="cuda").manual_seed(4)
    src = torch.randn((B, K, D, D, D), device="cuda", generator=gen)
    gi = mg.GridInterpolater(0.5, 23.5, 0.5, 23.5)
    zeros = np.zeros((B, 3), np.float32)
    ident = np.tile(np.asarray([1, 0, 0, 0], np.float32), (B, 1))
    out = torch.empty_like(src)
    gi.forward_batch(src, ident, zeros, zeros, out)
    assert torch.equal(out, src)
    # rotation by 90 degrees about z: (x, y, z) -> (-y, x, z); the grid is symmetric about its
    # centre, so every output voxel is one input voxel (up to rounding of the rotated coordinate)
    s = np.float32(np.sqrt(0.5))
    turn = np.tile(np.asarray([s, 0, 0, s], np.float32), (B, 1))
    gi.forward_batch(src, turn, zeros, zeros, out)
    a = torch.rot90(src, 1, dims=(2, 3))
    b = torch.rot90(src, -1, dims=(2, 3))
    err = min(float((out - a).abs().max()), float((out - b).abs().max()))
    assert err < 2e-4        # weights of 1 - O(1e-6) on values of a few units
    # random transforms: linear in the input, and a batch is its single launches
    rng = np.random.default_rng(40)
    quats = synth.random_quaternions(rng, B)
    trans = rng.uniform(-1.5, 1.5, (B, 3)).astype(np.float32)
    gi.forward_batch(src, quats, zeros, trans, out)
    other = torch.randn((4, K, D, D, D), device="cuda", generator=gen)
    o1 = torch.empty_like(other)
    o2 = torch.empty_like(other)
    gi.forward_batch(other, quats[10:14], zeros[:4], trans[10:14], o1)
    gi.forward_batch(0.5 * src[10:14] + other, quats[10:14], zeros[:4], trans[10:14], o2)
    want = 0.5 * out[10:14] + o1
    assert float((o2 - want).abs().max()) <= 1e-6 + 1e-5 * float(want.abs().max())
    one = torch.empty((K, D, D, D), device="cuda")
    for bidx in (0, 23, 49):
        gi.forward(src[bidx], mg.Transform(mg.Quaternion(*[float(x) for x in quats[bidx]]),
                                           (0, 0, 0), tuple(float(x) for x in trans[bidx])), one)
        assert torch.equal(one, out[bidx])
