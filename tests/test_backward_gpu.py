"""GPU parity of GridMaker.backward (through the C ABI) against the CPU oracle.

The oracle follows the reference and sums each atom's gradient sequentially in a
float; the kernel sums the same terms in a lane-parallel tree.  Both carry
rounding noise of a few float ulps of sum(|term|), so the comparison against the
float oracle allows that noise on top of the stated tolerance, while the
comparison against the double-accumulated oracle is held to the stated tolerance
plus the kernel's own float accumulation noise.
"""
import numpy as np
import pytest
import torch

import oracle
import synth
from util import ATOL, RTOL, assert_close, dev

pytestmark = pytest.mark.gpu

EPS = float(np.finfo(np.float32).eps)


@pytest.fixture(scope="module")
def mg():
    import libmolgrid_amd
    return libmolgrid_amd


def noise_bound(gm, center, coords, types, radii, diff):
    """Per-atom sum of |term| (upper bound of what rounding can touch), from the oracle run
    on |diff| with all signs aligned: an over-estimate is fine for a noise allowance."""
    mag = gm.backward(center, coords, types, radii, np.abs(diff), f64=True)
    if isinstance(mag, tuple):
        mag = mag[0]
    # |dx|/d <= 1 per term, so the magnitude of the aligned sum bounds each component
    return np.abs(mag).max(axis=1, keepdims=True) + 1e-30


def check_grads(got, ref32, ref64, mag, what):
    got = np.asarray(got, np.float64)
    # against the double-accumulated oracle: stated tolerance + float accumulation noise
    bound64 = ATOL + RTOL * np.abs(ref64) + 16 * EPS * mag
    err64 = np.abs(got - ref64)
    assert (err64 <= bound64).all(), "%s vs f64 oracle: worst excess %g" % (
        what, float((err64 - bound64).max()))
    # against the float oracle (reference order): its own sequential noise is allowed too
    bound32 = ATOL + RTOL * np.abs(ref32) + 64 * EPS * mag
    err32 = np.abs(got - ref32.astype(np.float64))
    assert (err32 <= bound32).all(), "%s vs f32 oracle: worst excess %g" % (
        what, float((err32 - bound32).max()))


def test_known_answer_single_atom(mg):
    """test/test_gridmaker.py:186-214: gradient at the grid centre of an atom at x=1, r=2."""
    gm = mg.GridMaker(0.1, 6.0)
    diff = torch.zeros(gm.grid_dimensions(1), device="cuda")
    diff[0, 30, 30, 30] = 1.0
    q = np.random.default_rng(4).normal(size=4)
    T = mg.Transform(mg.Quaternion(*(q / np.linalg.norm(q))))
    coords = dev(np.asarray([[1.0, 0, 0]], np.float32))
    T.forward(coords, coords)
    grads = torch.empty((1, 3), device="cuda")
    gm.backward((0, 0, 0), coords, dev(np.zeros(1, np.float32)), dev(np.full(1, 2.0, np.float32)),
                diff, grads)
    T.backward(grads, grads, False)
    np.testing.assert_allclose(grads.cpu().numpy().ravel(), [-0.60653067, 0, 0], atol=1e-5)


def test_zero_at_centre_and_antisymmetry(mg):
    """test/test_gridmaker.cpp:252-287."""
    gm = mg.GridMaker(0.1, 6.0)
    diff = torch.zeros(gm.grid_dimensions(1), device="cuda")
    diff[0, 30, 30, 30] = 1.0
    coords = dev(np.asarray([[0, 0, 0], [1, 0, 0], [-1, 0, 0], [0, 0.5, 0]], np.float32))
    grads = torch.empty((4, 3), device="cuda")
    gm.backward((0, 0, 0), coords, dev(np.zeros(4, np.float32)), dev(np.full(4, 2.0, np.float32)),
                diff, grads)
    g = grads.cpu().numpy()
    assert np.all(g[0] == 0)
    assert g[1, 0] == pytest.approx(-g[2, 0]) and g[1, 0] < 0
    assert g[3, 1] < 0 and g[3, 0] == 0


@pytest.mark.parametrize("res,dimension,ntypes,natoms", [
    (0.5, 6.0, 3, 20), (0.5, 12.0, 5, 60), (0.25, 5.75, 2, 15), (0.5, 23.5, 28, 200)])
def test_small_random_vs_oracle(mg, res, dimension, ntypes, natoms):
    rng = np.random.default_rng(21 + natoms)
    coords, types, radii = synth.small_index_case(rng, natoms, ntypes, dimension / 2 + 2.0)
    # backward rounds the type index (forward floors it)
    types = types + rng.uniform(-0.4, 0.4, natoms).astype(np.float32) * (types >= 0)
    center = rng.uniform(-1, 1, 3).astype(np.float32)
    og = oracle.GridMaker(res, dimension)
    diff = rng.standard_normal(og.grid_shape(ntypes)).astype(np.float32)
    ref32 = og.backward(center, coords, types, radii, diff)
    ref64 = og.backward(center, coords, types, radii, diff, f64=True)
    mag = noise_bound(og, center, coords, types, radii, diff)
    gm = mg.GridMaker(res, dimension)
    grads = torch.full((natoms, 3), 9.0, device="cuda")
    gm.backward(center, dev(coords), dev(types), dev(radii), dev(diff), grads)
    check_grads(grads.cpu().numpy(), ref32, ref64, mag, "backward")
    assert np.all(grads.cpu().numpy()[types < -0.5] == 0)   # ignored atoms get zeros


@pytest.mark.parametrize("sparse", [False, True])
def test_ragged_batch_vs_oracle(mg, sparse):
    """Configuration 2 at a batch the oracle finishes in seconds."""
    c = synth.config1(nbatch=4)
    B = len(c["offsets"]) - 1
    rng = np.random.default_rng(8)
    og = oracle.GridMaker(0.5, 23.5)
    diff = rng.standard_normal((B,) + og.grid_shape(28)).astype(np.float32)
    if sparse:
        diff *= rng.random(diff.shape) < 0.1
    moved = oracle.transform_forward_batch(c["offsets"], c["quats"], c["centers"],
                                           c["translations"], c["coords"])
    ref32 = og.backward_batch(c["offsets"], c["centers"], moved, c["types"], c["radii"], diff,
                              nthreads=4)
    gm = mg.GridMaker(0.5, 23.5)
    grads = torch.empty((len(moved), 3), device="cuda")
    gm.backward_batch(c["offsets"], c["centers"], dev(moved), dev(c["types"]), dev(c["radii"]),
                      dev(diff), grads)
    got = grads.cpu().numpy()
    off = c["offsets"]
    for b in range(B):
        s = slice(off[b], off[b + 1])
        ref64 = og.backward(c["centers"][b], moved[s], c["types"][s], c["radii"][s], diff[b],
                            f64=True)
        mag = noise_bound(og, c["centers"][b], moved[s], c["types"][s], c["radii"][s], diff[b])
        check_grads(got[s], ref32[s], ref64, mag, "config 2 example %d" % b)
    # un-rotation of the gradients (Transform::backward without translation)
    un_ref = oracle.transform_backward_batch(off, c["quats"], c["centers"], c["translations"],
                                             got, dotranslate=False)
    mg.transform_batch(off, c["quats"], c["centers"], c["translations"], grads, grads,
                       dotranslate=False, inverse=True)
    assert np.array_equal(grads.cpu().numpy(), un_ref)


@pytest.mark.parametrize("gm_args", [
    dict(gaussian_radius_multiple=-1.5),              # truncated Gaussian, no quadratic tail
    dict(gaussian_radius_multiple=2.0),
    dict(radius_scale=0.5, gaussian_radius_multiple=3.0),
    dict(radius_scale=1.7),
    dict(binary=True),                                # the gradient ignores the binary flag
])
def test_unusual_radius_multiples(mg, gm_args):
    """The tail of the gradient scale is cut off by clamping it at zero, which relies on the tail
    reaching zero at the final radius for every choice of the multiples (src/grid_maker.cpp:20-36)."""
    rng = np.random.default_rng(77)
    natoms, ntypes = 40, 4
    coords, types, radii = synth.small_index_case(rng, natoms, ntypes, 7.0)
    og = oracle.GridMaker(0.5, 11.5, **gm_args)
    diff = rng.standard_normal(og.grid_shape(ntypes)).astype(np.float32)
    center = (0.3, -0.2, 0.1)
    ref32 = og.backward(center, coords, types, radii, diff)
    ref64 = og.backward(center, coords, types, radii, diff, f64=True)
    mag = noise_bound(og, center, coords, types, radii, diff)
    gm = mg.GridMaker(0.5, 11.5, **gm_args)
    grads = torch.full((natoms, 3), 9.0, device="cuda")
    gm.backward(center, dev(coords), dev(types), dev(radii), dev(diff), grads)
    check_grads(grads.cpu().numpy(), ref32, ref64, mag, "backward %r" % (gm_args,))


def test_values_out_of_reach_are_never_used(mg):
    """A voxel beyond the final radius is skipped whatever it holds
    (density_grad_dist returns NaN there and the term is dropped, src/grid_maker.cu:884-915)."""
    og = oracle.GridMaker(0.5, 11.5)
    gm = mg.GridMaker(0.5, 11.5)
    coords = np.asarray([[0.1, 0.2, -0.3], [2.0, -1.0, 0.7]], np.float32)
    types = np.asarray([0, 0], np.float32)
    radii = np.asarray([1.5, 1.2], np.float32)
    rng = np.random.default_rng(5)
    diff = rng.standard_normal(og.grid_shape(1)).astype(np.float32)
    ref = og.backward((0, 0, 0), coords, types, radii, diff)
    # poison every voxel farther than the final radius from both atoms
    ax = np.arange(24) * 0.5 - 5.75
    X, Y, Z = np.meshgrid(ax, ax, ax, indexing="ij")
    far = np.ones(X.shape, bool)
    for c, r in zip(coords, radii):
        far &= np.sqrt((X - c[0]) ** 2 + (Y - c[1]) ** 2 + (Z - c[2]) ** 2) > 1.5 * r + 1e-3
    poisoned = diff.copy()
    poisoned[0][far] = np.where(rng.random(int(far.sum())) < 0.5, np.inf, np.nan)
    grads = torch.empty((2, 3), device="cuda")
    gm.backward((0, 0, 0), dev(coords), dev(types), dev(radii), dev(poisoned), grads)
    got = grads.cpu().numpy()
    assert np.isfinite(got).all()
    clean = torch.empty((2, 3), device="cuda")
    gm.backward((0, 0, 0), dev(coords), dev(types), dev(radii), dev(diff), clean)
    assert np.array_equal(got, clean.cpu().numpy())
    assert_close(got, ref, rtol=1e-4, atol=1e-5, what="poisoned grid vs oracle on the clean one")


def test_repeat_runs_are_bit_identical(mg):
    c = synth.config1(nbatch=2)
    gm = mg.GridMaker(0.5, 23.5)
    diff = torch.randn((2,) + gm.grid_dimensions(28), device="cuda")
    args = (c["offsets"], c["centers"], dev(c["coords"]), dev(c["types"]), dev(c["radii"]), diff)
    a = torch.empty((len(c["coords"]), 3), device="cuda")
    b = torch.empty_like(a)
    gm.backward_batch(*args, a)
    gm.backward_batch(*args, b)
    assert torch.equal(a, b)


def test_argument_errors(mg):
    gm = mg.GridMaker(0.5, 7.5)
    z = lambda *s: torch.zeros(s, device="cuda")
    with pytest.raises(ValueError):
        gm.backward((0, 0, 0), z(4, 3), z(4), z(4), z(2, 16, 16, 15), z(4, 3))
    with pytest.raises(ValueError):
        gm.backward((0, 0, 0), z(4, 3), z(4), z(3), z(2, 16, 16, 16), z(4, 3))
    with pytest.raises(ValueError):
        mg.GridMaker(0.5, 7.5, False, True).backward((0, 0, 0), z(4, 3), z(4), z(4),
                                                     z(2, 16, 16, 16), z(4, 3))


def test_padding_atoms_without_radius_get_zero_gradient(mg):
    """The rows that pad a batch (radius 0, coordinates 0) sit exactly on a voxel centre when the
    grid is centred at the origin with an odd number of points: their gradient is 0, as in the
    reference (its distance test fails for every voxel of such an atom), not NaN."""
    rng = np.random.default_rng(21)
    coords, types, radii = synth.small_index_case(rng, 30, 3, 4.0, frac_ignored=0.0)
    coords = np.concatenate([coords, np.zeros((4, 3), np.float32)])
    types = np.concatenate([types, np.zeros(4, np.float32)])
    radii = np.concatenate([radii, np.zeros(4, np.float32)])
    gm = mg.GridMaker(0.5, 8.0)                 # 17 points a side: a voxel centre at the origin
    og = oracle.GridMaker(0.5, 8.0)
    diff = rng.standard_normal(gm.grid_dimensions(3)).astype(np.float32)
    grads = torch.full((34, 3), 7.0, device="cuda")
    gm.backward((0, 0, 0), dev(coords), dev(types), dev(radii), dev(diff), grads)
    got = grads.cpu().numpy()
    assert np.all(got[30:] == 0.0) and np.isfinite(got).all()
    args = ((0, 0, 0), coords, types, radii, diff)
    ref = og.backward(*args)
    assert np.all(ref[30:] == 0.0)
    check_grads(got, ref, og.backward(*args, f64=True), noise_bound(og, *args), "padded")
