"""TEST INFRASTRUCTURE: parity cases of the library's kernels run on the CPU through the HIP
emulation (emu_capi.py), checked against the oracle.  Run as ``python tests/emu/cases.py GROUP``;
a kernel that faults, deadlocks or leaves its arrays ends the process with a non-zero status, which
is why pytest runs each group in a child process (tests/test_emulated_kernels_cpu.py)."""
import ctypes
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)

import emu_capi as E  # noqa: E402
import oracle  # noqa: E402
import synth  # noqa: E402

lib = E.lib
RTOL, ATOL = 1e-5, 1e-6
# With EMU_APPROX (hip_emu.h: the approximate instructions moved by one unit in the last place) the
# float comparisons get this factor of head room: what that mode looks for are voxels and atoms
# that change SIDES -- a cull that loses one, an index that comes out different, a bit-exact path
# that turns out to depend on an approximation --, not the last digit of a sum of tails.
if os.environ.get("EMU_APPROX"):
    RTOL, ATOL = 2e-5, 2e-6
STATIC_BYTES = 16 << 20      # MG_STATIC_SCRATCH_BYTES of include/molgrid_hip.h
_checked = [0]


def close(got, ref, what, exact=False):
    _checked[0] += 1
    if exact:
        ok = np.array_equal(got, ref)
    else:
        ok = bool(np.all(np.abs(got - ref) <= ATOL + RTOL * np.abs(ref)))
    if not ok:
        bad = np.argwhere(~(np.abs(got - ref) <= ATOL + RTOL * np.abs(ref)) if not exact else got != ref)
        raise AssertionError("%s: %d values differ, first at %s: got %r want %r, max abs %g"
                             % (what, len(bad), tuple(bad[0]), got[tuple(bad[0])],
                                ref[tuple(bad[0])], float(np.nanmax(np.abs(got - ref)))))


def forward_index(gm_args, centers, coords, types, radii, ntypes, offsets=None, per_example=None,
                  nbatch=1, variant="ws"):
    """mg_forward_index_* on host arrays; centers (3,) host triple or (B,3) device rows."""
    g = E.gridmaker(*gm_args)
    dim = int(g.dim)
    out = E.array((nbatch, ntypes, dim, dim, dim), fill=7.0)          # must be overwritten
    n = per_example if per_example is not None else len(coords)
    off = E.put(offsets, np.int32) if offsets is not None else None
    centers = np.asarray(centers, np.float32)
    cdev = E.put(centers) if centers.ndim == 2 else None
    chost = E.f3(centers if centers.ndim == 1 else (0, 0, 0))
    c, t, r = E.put(coords), E.put(types), E.put(radii)
    if variant == "ws":
        need = lib.mg_forward_index_workspace_size(ctypes.byref(g), nbatch, n, ntypes)
        ws = E.array(need, np.uint8, tight=False)
        code = lib.mg_forward_index_ws(ctypes.byref(g), nbatch, E.ptr(off), n, E.ptr(cdev), chost,
                                       E.ptr(c), E.ptr(t), E.ptr(r), ntypes, E.ptr(out), E.ptr(ws),
                                       need, None)
    elif variant == "cached":
        code = lib.mg_forward_index(ctypes.byref(g), nbatch, E.ptr(off), n, E.ptr(cdev), chost,
                                    E.ptr(c), E.ptr(t), E.ptr(r), ntypes, E.ptr(out), None)
    else:
        code = lib.mg_forward_index_static(ctypes.byref(g), nbatch, E.ptr(off), n, E.ptr(cdev),
                                           chost, E.ptr(c), E.ptr(t), E.ptr(r), ntypes, E.ptr(out),
                                           None)
    assert code == 0, "mg_forward_index_%s returned %d" % (variant, code)
    return out if nbatch > 1 or offsets is not None else out[0]


# --------------------------------------------------------------------------------------------------
def group_transform():
    for seed, dotranslate in ((6, True), (7, False)):
        rng = np.random.default_rng(seed)
        q = rng.normal(size=4).astype(np.float32)
        c = rng.uniform(-3, 3, 3).astype(np.float32)
        t = rng.uniform(-2, 2, 3).astype(np.float32)
        pts = rng.uniform(-20, 20, (700, 3)).astype(np.float32)
        src, dst = E.put(pts), E.array((700, 3))
        for fn, ref in ((lib.mg_transform_forward, oracle.transform_forward),
                        (lib.mg_transform_backward, oracle.transform_backward)):
            assert fn(1, None, 700, None, E.f4(q), None, E.f3(c), None, E.f3(t), int(dotranslate),
                      E.ptr(src), E.ptr(dst), None) == 0
            close(dst, ref(q, c, t, pts, dotranslate), "transform", exact=True)
    # a ragged batch with device rows of quaternions, centres and translations
    cfg = synth.index_batch(1, 5, (20, 60), (3, 9))
    off = cfg["offsets"]
    n = int(off[-1])
    dst = E.array((n, 3))
    assert lib.mg_transform_forward(5, E.ptr(E.put(off, np.int32)), int(np.diff(off).max()),
                                    E.ptr(E.put(cfg["quats"])), E.f4((1, 0, 0, 0)),
                                    E.ptr(E.put(cfg["centers"])), E.f3((0, 0, 0)),
                                    E.ptr(E.put(cfg["translations"])), E.f3((0, 0, 0)), 1,
                                    E.ptr(E.put(cfg["coords"])), E.ptr(dst), None) == 0
    close(dst, oracle.transform_forward_batch(off, cfg["quats"], cfg["centers"],
                                              cfg["translations"], cfg["coords"]),
          "transform batch", exact=True)


def group_forward_index():
    """The cases of tests/test_forward_gpu.py::test_small_random_vs_oracle and
    test_unusual_radius_multiples, on the CPU."""
    shapes = [(0.5, 6.0, 3, 20), (0.5, 12.0, 5, 60), (0.25, 5.75, 2, 15), (1.0, 15.0, 40, 200),
              (0.5, 23.5, 28, 300), (0.5, 29.5, 4, 500), (0.25, 25.25, 3, 400), (0.5, 31.5, 4, 400)]
    for res, dimension, ntypes, natoms in shapes:
        for binary in (False, True):
            rng = np.random.default_rng(11 + natoms)
            coords, types, radii = synth.small_index_case(rng, natoms, ntypes, dimension / 2 + 2.0)
            types = types + rng.uniform(0, 0.9, natoms).astype(np.float32) * (types >= 0)
            center = rng.uniform(-1, 1, 3).astype(np.float32)
            ref = oracle.GridMaker(res, dimension, binary).forward(center, coords, types, radii, ntypes)
            got = forward_index((res, dimension, binary), center, coords, types, radii, ntypes)
            close(got, ref, "forward %s binary=%s" % ((res, dimension, ntypes, natoms), binary),
                  exact=binary)
    for gm_args in [(0.5, 11.5, False, False, 1.0, -1.5), (0.5, 11.5, True, False, 1.0, -0.5),
                    (0.5, 11.5, False, False, 1.3, 0.7), (0.5, 11.5, True, False, 0.6, 2.0)]:
        rng = np.random.default_rng(5)
        coords, types, radii = synth.small_index_case(rng, 80, 4, 7.0)
        ref = oracle.GridMaker(*gm_args).forward((0, 0, 0), coords, types, radii, 4)
        got = forward_index(gm_args, (0, 0, 0), coords, types, radii, 4)
        close(got, ref, "forward %s" % (gm_args,), exact=gm_args[2])
    # zero and negative radii add nothing; many atoms on one spot; the three workspace variants
    rng = np.random.default_rng(21)
    coords, types, radii = synth.small_index_case(rng, 120, 3, 6.0)
    radii[::3] = 0.0
    radii[1::3] = -radii[1::3]
    for binary in (False, True):
        ref = oracle.GridMaker(0.5, 11.5, binary).forward((0, 0, 0), coords, types, radii, 3)
        results = [forward_index((0.5, 11.5, binary), (0, 0, 0), coords, types, radii, 3, variant=v)
                   for v in ("ws", "cached", "static")]
        close(results[0], ref, "radii <= 0, binary=%s" % binary, exact=binary)
        close(results[1], results[0], "cached workspace", exact=True)
        close(results[2], results[0], "static workspace", exact=True)
    rng = np.random.default_rng(3)
    n = 3000
    coords = rng.normal(0, 0.3, (n, 3)).astype(np.float32)
    types = rng.integers(0, 2, n).astype(np.float32)
    radii = rng.uniform(1.0, 1.5, n).astype(np.float32)
    ref = oracle.GridMaker(0.5, 7.5).forward((0, 0, 0), coords, types, radii, 2)
    close(forward_index((0.5, 7.5), (0, 0, 0), coords, types, radii, 2), ref, "3000 atoms on a spot")


def group_forward_batch():
    """Ragged and padded batches, empty examples, per-example centres."""
    cfg = synth.index_batch(2, 6, (30, 120), (3, 9), ntypes=6)
    off = cfg["offsets"].copy()
    gm = oracle.GridMaker(0.5, 11.5)
    moved = oracle.transform_forward_batch(off, cfg["quats"], cfg["centers"], cfg["translations"],
                                           cfg["coords"])
    ref = gm.forward_batch(off, cfg["centers"], moved, cfg["types"], cfg["radii"], 6)
    got = forward_index((0.5, 11.5), cfg["centers"], moved, cfg["types"], cfg["radii"], 6,
                        offsets=off, per_example=int(np.diff(off).max()), nbatch=6)
    close(got, ref, "ragged batch")
    # the same examples padded to one length (radius 0, type -1 in the padding rows)
    width = int(np.diff(off).max())
    pc = np.zeros((6, width, 3), np.float32)
    pt = np.full((6, width), -1.0, np.float32)
    pr = np.zeros((6, width), np.float32)
    for b in range(6):
        k = off[b + 1] - off[b]
        pc[b, :k], pt[b, :k], pr[b, :k] = moved[off[b]:off[b + 1]], cfg["types"][off[b]:off[b + 1]], \
            cfg["radii"][off[b]:off[b + 1]]
    pt[:, -1] = 2.0          # a padding row with a type but radius 0: adds nothing
    got_p = forward_index((0.5, 11.5), cfg["centers"], pc.reshape(-1, 3), pt.reshape(-1),
                          pr.reshape(-1), 6, per_example=width, nbatch=6)
    close(got_p, got, "padded batch equals ragged batch", exact=True)
    # an example without atoms in the middle, and a batch without any atom
    off2 = np.array([0, 40, 40, 90], np.int64)
    ref2 = gm.forward_batch(off2, cfg["centers"][:3], moved[:90], cfg["types"][:90], cfg["radii"][:90], 6)
    got2 = forward_index((0.5, 11.5), cfg["centers"][:3], moved[:90], cfg["types"][:90],
                         cfg["radii"][:90], 6, offsets=off2, per_example=50, nbatch=3)
    close(got2, ref2, "empty example")
    assert not got2[1].any()
    got3 = forward_index((0.5, 11.5), (0, 0, 0), np.zeros((0, 3), np.float32), np.zeros(0, np.float32),
                         np.zeros(0, np.float32), 3, per_example=0, nbatch=2)
    assert not got3.any()
    _checked[0] += 1


def group_forward_split():
    """mg_forward_index_sort + mg_forward_index_splat give the grids of mg_forward_index_ws."""
    cfg = synth.index_batch(2, 5, (30, 120), (3, 9), ntypes=6)
    off = cfg["offsets"]
    width = int(np.diff(off).max())
    for binary in (False, True):
        g = E.gridmaker(0.5, 11.5, binary)
        dim = int(g.dim)
        whole = forward_index((0.5, 11.5, binary), cfg["centers"], cfg["coords"], cfg["types"],
                              cfg["radii"], 6, offsets=off, per_example=width, nbatch=5)
        need = lib.mg_forward_index_workspace_size(ctypes.byref(g), 5, width, 6)
        ws = E.array(need, np.uint8, tight=False)
        out = E.array((5, 6, dim, dim, dim), fill=7.0)
        assert lib.mg_forward_index_sort(ctypes.byref(g), 5, E.ptr(E.put(off, np.int32)), width,
                                         E.ptr(E.put(cfg["centers"])), E.f3((0, 0, 0)),
                                         E.ptr(E.put(cfg["coords"])), E.ptr(E.put(cfg["types"])),
                                         E.ptr(E.put(cfg["radii"])), 6, E.ptr(ws), need, None) == 0
        assert np.all(out == 7.0)                       # the sort does not touch the grids
        assert lib.mg_forward_index_splat(ctypes.byref(g), 5, width, 6, E.ptr(out), E.ptr(ws), need,
                                          None) == 0
        close(out, whole, "sort + splat, binary=%s" % binary, exact=True)
    # a workspace the sort launch never filled (0xCB bytes, then random bytes): wrong grids are
    # fine, leaving the arrays or looping for ever is not
    junk = E.array(need, np.uint8, tight=False)
    assert lib.mg_forward_index_splat(ctypes.byref(g), 5, width, 6, E.ptr(out), E.ptr(junk), need, None) == 0
    junk[...] = np.random.default_rng(1).integers(0, 256, need, dtype=np.uint8)
    assert lib.mg_forward_index_splat(ctypes.byref(g), 5, width, 6, E.ptr(out), E.ptr(junk), need, None) == 0
    lib.mg_forward_index_paged.argtypes = [ctypes.c_int]
    lib.mg_forward_index_paged(1)
    assert lib.mg_forward_index_splat(ctypes.byref(g), 5, width, 6, E.ptr(out), E.ptr(junk), need, None) == 0
    lib.mg_forward_index_paged(0)
    # argument errors: a workspace that is too small or misaligned, no workspace
    assert lib.mg_forward_index_splat(ctypes.byref(g), 5, width, 6, E.ptr(out), E.ptr(ws), need - 1, None) == -1
    assert lib.mg_forward_index_splat(ctypes.byref(g), 5, width, 6, E.ptr(out), ws[16:].ctypes.data, need, None) == -1
    assert lib.mg_forward_index_splat(ctypes.byref(g), 5, width, 6, E.ptr(out), None, need, None) == -4
    _checked[0] += 1


def group_forward_paged():
    """The paged write-out (workgroups that own a slab and write whole 4 KB pages) gives the grids
    of the per-wave write-out bit for bit: dims 16, 24, 48 and smaller, binary and Gaussian, batches
    with empty examples, output arrays at several alignments inside a 4 KB page."""
    lib.mg_forward_index_paged.argtypes = [ctypes.c_int]
    lib.mg_forward_index_core_skip.argtypes = [ctypes.c_int]
    shapes = [(1.0, 15.0, 40, 200), (0.25, 5.75, 2, 15), (0.5, 23.5, 28, 300), (0.5, 3.5, 3, 12),
              (0.5, 1.5, 2, 5), (0.5, 21.5, 5, 150)]
    for res, dimension, ntypes, natoms in shapes:
        for binary in (False, True):
            rng = np.random.default_rng(31 + natoms)
            coords, types, radii = synth.small_index_case(rng, natoms, ntypes, dimension / 2 + 2.0)
            center = rng.uniform(-1, 1, 3).astype(np.float32)
            ref = oracle.GridMaker(res, dimension, binary).forward(center, coords, types, radii, ntypes)
            assert lib.mg_forward_index_paged(0) in (0, 1)
            plain = forward_index((res, dimension, binary), center, coords, types, radii, ntypes).copy()
            lib.mg_forward_index_paged(1)
            paged = forward_index((res, dimension, binary), center, coords, types, radii, ntypes)
            lib.mg_forward_index_paged(0)
            what = "paged %s binary=%s" % ((res, dimension, ntypes, natoms), binary)
            close(paged, plain, what + " vs per-wave write-out", exact=True)
            close(paged, ref, what + " vs oracle", exact=binary)
            if not binary:
                # the instances that skip the exponential in tail-only blocks, with either write-out
                for paged_on in (0, 1):
                    lib.mg_forward_index_paged(paged_on)
                    lib.mg_forward_index_core_skip(1)
                    skipped = forward_index((res, dimension, binary), center, coords, types, radii, ntypes)
                    lib.mg_forward_index_paged(0)
                    lib.mg_forward_index_core_skip(0)
                    close(skipped, plain, what + ", tail-only blocks without the exponential, paged=%d" % paged_on,
                          exact=True)
    # a ragged batch with an empty example; the output at offsets of 16, 1040 and 4080 bytes from
    # a page boundary (pages are taken by address)
    cfg = synth.index_batch(2, 4, (30, 120), (3, 9), ntypes=6)
    off = np.array([0, 40, 40, 130, 200], np.int64)
    gm = oracle.GridMaker(0.5, 11.5)
    ref = gm.forward_batch(off, cfg["centers"], cfg["coords"][:200], cfg["types"][:200],
                           cfg["radii"][:200], 6)
    g = E.gridmaker(0.5, 11.5)
    dim = int(g.dim)
    nfl = 4 * 6 * dim ** 3
    need = lib.mg_forward_index_workspace_size(ctypes.byref(g), 4, 90, 6)
    ws = E.array(need, np.uint8, tight=False)
    args = [E.ptr(E.put(off, np.int32)), 90, E.ptr(E.put(cfg["centers"])), E.f3((0, 0, 0)),
            E.ptr(E.put(cfg["coords"][:200])), E.ptr(E.put(cfg["types"][:200])),
            E.ptr(E.put(cfg["radii"][:200])), 6]
    lib.mg_forward_index_paged(1)
    for shift in (4, 260, 1020):
        big = E.array(nfl + shift, fill=7.0)
        out = big[shift:]
        assert lib.mg_forward_index_ws(ctypes.byref(g), 4, *args, out.ctypes.data, E.ptr(ws), need, None) == 0
        close(out.reshape(ref.shape), ref, "paged, output %d bytes into its page" % (4 * shift))
        assert np.all(big[:shift] == 7.0)
    lib.mg_forward_index_paged(0)


EPS = float(np.finfo(np.float32).eps)


def check_grads(got, ref32, ref64, mag, what):
    """The bounds of tests/test_backward_gpu.py."""
    _checked[0] += 1
    got = np.asarray(got, np.float64)
    bound64 = ATOL + RTOL * np.abs(ref64) + 16 * EPS * mag
    err64 = np.abs(got - ref64)
    assert (err64 <= bound64).all(), "%s vs f64 oracle: worst excess %g" % (what, float((err64 - bound64).max()))
    bound32 = ATOL + RTOL * np.abs(ref32) + 64 * EPS * mag
    err32 = np.abs(got - ref32.astype(np.float64))
    assert (err32 <= bound32).all(), "%s vs f32 oracle: worst excess %g" % (what, float((err32 - bound32).max()))


def group_backward_index():
    for res, dimension, ntypes, natoms in [(0.5, 6.0, 3, 20), (0.5, 12.0, 5, 60), (0.25, 5.75, 2, 15),
                                           (0.5, 23.5, 28, 200)]:
        rng = np.random.default_rng(21 + natoms)
        coords, types, radii = synth.small_index_case(rng, natoms, ntypes, dimension / 2 + 2.0)
        types = types + rng.uniform(-0.4, 0.4, natoms).astype(np.float32) * (types >= 0)
        radii[0] = 0.0                                   # an atom without extent: zero gradient
        center = rng.uniform(-1, 1, 3).astype(np.float32)
        og = oracle.GridMaker(res, dimension)
        diff = rng.standard_normal(og.grid_shape(ntypes)).astype(np.float32)
        ref32 = og.backward(center, coords, types, radii, diff)
        ref64 = og.backward(center, coords, types, radii, diff, f64=True)
        mag = np.abs(og.backward(center, coords, types, radii, np.abs(diff), f64=True)).max(
            axis=1, keepdims=True) + 1e-30
        g = E.gridmaker(res, dimension)
        grads = E.array((natoms, 3), fill=9.0)
        c, t, r, d = E.put(coords), E.put(types), E.put(radii), E.put(diff)
        assert lib.mg_backward_index(ctypes.byref(g), 1, None, natoms, None, E.f3(center), E.ptr(c),
                                     E.ptr(t), E.ptr(r), ntypes, E.ptr(d), E.ptr(grads), None) == 0
        check_grads(grads, ref32, ref64, mag, "backward %s" % ((res, dimension, ntypes, natoms),))
        assert np.all(grads[np.round(types) < 0] == 0) and np.all(grads[0] == 0)
        # the launch that also un-rotates = backward + Transform.backward(dotranslate=False)
        q = rng.normal(size=4).astype(np.float32)
        rc = rng.uniform(-2, 2, 3).astype(np.float32)
        un = E.array((natoms, 3), fill=9.0)
        assert lib.mg_backward_index_unrotated(ctypes.byref(g), 1, None, natoms, None, E.f3(center),
                                               E.ptr(c), E.ptr(t), E.ptr(r), ntypes, E.ptr(d), None,
                                               E.f4(q), None, E.f3(rc), E.ptr(un), None) == 0
        close(un, oracle.transform_backward(q, rc, np.zeros(3, np.float32), np.array(grads), False),
              "fused un-rotation", exact=True)
    # a ragged batch, 10 % of the upstream gradient non-zero
    cfg = synth.index_batch(2, 4, (60, 200), (5, 20), ntypes=8)
    off = cfg["offsets"]
    rng = np.random.default_rng(8)
    og = oracle.GridMaker(0.5, 15.5)
    diff = rng.standard_normal((4,) + og.grid_shape(8)).astype(np.float32)
    diff *= rng.random(diff.shape) < 0.1
    ref32 = og.backward_batch(off, cfg["centers"], cfg["coords"], cfg["types"], cfg["radii"], diff)
    g = E.gridmaker(0.5, 15.5)
    n = int(off[-1])
    grads = E.array((n, 3), fill=9.0)
    assert lib.mg_backward_index(ctypes.byref(g), 4, E.ptr(E.put(off, np.int32)),
                                 int(np.diff(off).max()), E.ptr(E.put(cfg["centers"])),
                                 E.f3((0, 0, 0)), E.ptr(E.put(cfg["coords"])), E.ptr(E.put(cfg["types"])),
                                 E.ptr(E.put(cfg["radii"])), 8, E.ptr(E.put(diff)), E.ptr(grads), None) == 0
    _checked[0] += 1
    assert np.allclose(grads, ref32, rtol=1e-4, atol=2e-5), float(np.abs(grads - ref32).max())


def vector_case(rng, natoms, ntypes, extent, sparse=0.5):
    coords = rng.uniform(-extent, extent, (natoms, 3)).astype(np.float32)
    tv = rng.dirichlet(np.full(ntypes, 0.3), natoms) * rng.uniform(0.5, 1.5, (natoms, 1))
    tv = (tv * (rng.random((natoms, ntypes)) > sparse)).astype(np.float32)
    radii = rng.uniform(0.8, 2.0, natoms).astype(np.float32)
    return coords, tv, radii


def forward_vector(gm_args, center, coords, tv, radii, lists=False):
    """lists: with the workspace for per-slab atom lists (mg_forward_vector_ws)"""
    g = E.gridmaker(*gm_args)
    dim, ntypes = int(g.dim), tv.shape[1]
    out = E.array((ntypes, dim, dim, dim), fill=3.0)
    args = [ctypes.byref(g), 1, None, len(coords), None, E.f3(center), E.ptr(E.put(coords)),
            E.ptr(E.put(tv)), E.ptr(E.put(radii)), ntypes, E.ptr(out)]
    if lists:
        need = lib.mg_forward_vector_workspace_size(ctypes.byref(g), 1, len(coords), ntypes)
        ws = E.array(need, np.uint8, tight=False) if need else None
        code = lib.mg_forward_vector_ws(*args, E.ptr(ws), need, None)
    else:
        code = lib.mg_forward_vector(*args, None)
    assert code == 0, code
    return out


def group_forward_vector():
    """Matrix-core kernel (per-atom radii) and the tile kernel (exact predicates, radii by type)."""
    for ntypes in (2, 14, 28, 37):
        for binary in (False, True):
            rng = np.random.default_rng(100 + ntypes)
            coords, tv, radii = vector_case(rng, 60, ntypes, 7.0)
            ref = oracle.GridMaker(0.5, 11.5, binary).forward((0.2, -0.1, 0), coords, tv, radii)
            got = forward_vector((0.5, 11.5, binary), (0.2, -0.1, 0), coords, tv, radii)
            close(got, ref, "vector forward T=%d binary=%s" % (ntypes, binary), exact=binary)
    for gm_args in [(0.5, 11.5, False, False, 1.0, -1.5), (0.5, 11.5, True, False, 1.0, -0.5),
                    (0.5, 11.5, False, False, 1.3, 0.7)]:
        rng = np.random.default_rng(11)
        coords, tv, radii = vector_case(rng, 70, 5, 7.0)
        ref = oracle.GridMaker(*gm_args).forward((0, 0.1, 0), coords, tv, radii)
        got = forward_vector(gm_args, (0, 0.1, 0), coords, tv, radii)
        close(got, ref, "vector forward %s" % (gm_args,), exact=gm_args[2])
    # radii by type
    rng = np.random.default_rng(12)
    coords, tv, _ = vector_case(rng, 50, 6, 6.0)
    tr = rng.uniform(0.8, 2.0, 6).astype(np.float32)
    for binary in (False, True):
        ref = oracle.GridMaker(0.5, 9.5, binary, True).forward((0, 0, 0), coords, tv, tr)
        got = forward_vector((0.5, 9.5, binary, True), (0, 0, 0), coords, tv, tr)
        close(got, ref, "vector forward, radii by type, binary=%s" % binary, exact=binary)
    # per-slab atom lists: the same grids bit for bit, also for a batch with an empty example and
    # for more atoms than one scan pass holds per wave (several passes over the list)
    for ntypes, natoms, dimension in ((5, 60, 11.5), (28, 300, 15.5), (3, 6000, 9.5)):
        for binary in (False, True):
            rng = np.random.default_rng(200 + natoms)
            coords, tv, radii = vector_case(rng, natoms, ntypes, dimension / 2 + 1.0)
            plain = forward_vector((0.5, dimension, binary), (0.1, 0, 0), coords, tv, radii).copy()
            listed = forward_vector((0.5, dimension, binary), (0.1, 0, 0), coords, tv, radii, lists=True)
            close(listed, plain, "atom lists T=%d n=%d binary=%s" % (ntypes, natoms, binary), exact=True)
    rng = np.random.default_rng(14)
    coords, tv, radii = vector_case(rng, 130, 4, 6.5)
    off = np.array([0, 50, 50, 130], np.int32)
    g = E.gridmaker(0.5, 11.5)
    dim = int(g.dim)
    cen = E.put(rng.uniform(-1, 1, (3, 3)).astype(np.float32))
    outs = []
    for use in (False, True):
        need = lib.mg_forward_vector_workspace_size(ctypes.byref(g), 3, 80, 4) if use else 0
        ws = E.array(need, np.uint8, tight=False) if need else None
        out = E.array((3, 4, dim, dim, dim), fill=3.0)
        assert lib.mg_forward_vector_ws(ctypes.byref(g), 3, E.ptr(E.put(off, np.int32)), 80, E.ptr(cen),
                                        E.f3((0, 0, 0)), E.ptr(E.put(coords)), E.ptr(E.put(tv)),
                                        E.ptr(E.put(radii)), 4, E.ptr(out), E.ptr(ws), need, None) == 0
        outs.append(np.array(out))
    close(outs[1], outs[0], "atom lists, ragged batch", exact=True)
    ref = oracle.GridMaker(0.5, 11.5).forward_batch(off.astype(np.int64), np.array(cen), coords, tv, radii, 4)
    close(outs[1], ref, "atom lists, ragged batch vs oracle")
    assert not outs[1][1].any()
    # a larger grid (two z slabs in the matrix-core kernel's terms): dim 60
    rng = np.random.default_rng(13)
    coords, tv, radii = vector_case(rng, 150, 4, 16.0)
    ref = oracle.GridMaker(0.5, 29.5).forward((0, 0, 0), coords, tv, radii)
    close(forward_vector((0.5, 29.5), (0, 0, 0), coords, tv, radii), ref, "vector forward dim 60")


def group_backward_vector():
    """The cases and bounds of tests/test_vector_gpu.py::test_backward_vs_oracle, plus a binary
    sphere that is wider than its index box (final radius multiple below one)."""
    cases = [(3, (0.5, 9.5, False, False)), (28, (0.5, 9.5, False, False)), (37, (0.5, 9.5, False, False)),
             (5, (0.5, 9.5, True, False)), (6, (0.5, 9.5, False, True)), (6, (0.5, 9.5, True, True)),
             (4, (0.5, 9.5, True, False, 1.0, -0.5)), (4, (0.5, 9.5, False, False, 1.3, 0.7))]
    for ntypes, gm_args in cases:
        rti = gm_args[3]
        rng = np.random.default_rng(300 + ntypes)
        coords, tv, radii = vector_case(rng, 40, ntypes, 6.0)
        if rti:
            radii = rng.uniform(0.8, 2.0, ntypes).astype(np.float32)
        og = oracle.GridMaker(*gm_args)
        diff = rng.standard_normal(og.grid_shape(ntypes)).astype(np.float32)
        ra32, rt32 = og.backward((0, 0, 0), coords, tv, radii, diff)
        ra64, rt64 = og.backward((0, 0, 0), coords, tv, radii, diff, f64=True)
        ma, mt = og.backward((0, 0, 0), coords, np.abs(tv), radii, np.abs(diff), f64=True)
        ma = np.abs(ma).max(axis=1, keepdims=True) + 1e-30
        g = E.gridmaker(*gm_args)
        ag, tg = E.array((40, 3), fill=9.0), E.array((40, ntypes), fill=9.0)
        assert lib.mg_backward_vector(ctypes.byref(g), 1, None, 40, None, E.f3((0, 0, 0)),
                                      E.ptr(E.put(coords)), E.ptr(E.put(tv)), E.ptr(E.put(radii)),
                                      ntypes, E.ptr(E.put(diff)), E.ptr(ag), E.ptr(tg), None) == 0
        _checked[0] += 1
        a64, t64 = np.asarray(ag, np.float64), np.asarray(tg, np.float64)
        what = "vector backward T=%d %s" % (ntypes, gm_args)
        assert (np.abs(a64 - ra64) <= ATOL + RTOL * np.abs(ra64) + 16 * EPS * ma).all(), what
        assert (np.abs(a64 - ra32) <= ATOL + RTOL * np.abs(ra32) + 64 * EPS * ma).all(), what
        assert (np.abs(t64 - rt64) <= ATOL + RTOL * np.abs(rt64) + 16 * EPS * mt).all(), what
        assert (np.abs(t64 - rt32) <= ATOL + RTOL * np.abs(rt32) + 64 * EPS * mt).all(), what


def close_sums(got, ref, scale, what):
    """|got - ref| <= 1e-6 + 1e-5 |ref| + 64 eps * (sum of |terms|), as tests/test_second_order_gpu.py"""
    _checked[0] += 1
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    tol = 1e-6 + 1e-5 * np.abs(ref) + 64 * EPS * np.asarray(scale, np.float64)
    bad = np.abs(got - ref) > tol
    assert not bad.any(), "%s: %d values off, worst %g" % (what, int(bad.sum()), np.abs(got - ref)[bad].max())


def group_second_order():
    """The cases of tests/test_second_order_gpu.py on the CPU."""
    for gm_args in ((0.5, 11.5, False), (0.5, 11.5, True), (0.5, 11.5, True, False, 1.0, -0.5)):
        binary = gm_args[2]
        rng = np.random.default_rng(31)
        n, T = 90, 5
        coords = rng.uniform(-6, 6, (n, 3)).astype(np.float32)
        types = rng.integers(0, T, n).astype(np.float32)
        types[::11] = -1
        radii = rng.uniform(0.9, 2.0, n).astype(np.float32)
        og = oracle.GridMaker(*gm_args)
        cen = (0.3, 0, -0.1)
        dens = og.forward(cen, coords, types, radii, T)
        if binary:
            dens = dens * rng.uniform(0.5, 3.0, dens.shape).astype(np.float32)
        dens[1, 4:9] = 0
        diff = rng.standard_normal(dens.shape).astype(np.float32)
        ref = og.backward_relevance(cen, coords, types, radii, dens, diff)
        scale = og.backward_relevance(cen, coords, types, radii, dens, np.abs(diff))
        g = E.gridmaker(*gm_args)
        rel = E.array(n, fill=5.0)
        assert lib.mg_backward_relevance(ctypes.byref(g), 1, None, n, None, E.f3(cen),
                                         E.ptr(E.put(coords)), E.ptr(E.put(types)), E.ptr(E.put(radii)),
                                         T, E.ptr(E.put(dens)), E.ptr(E.put(diff)), E.ptr(rel), None) == 0
        close_sums(rel, ref, scale, "relevance %s" % (gm_args,))
        assert not rel[::11].any()
    for rti in (False, True):
        for grm in (1.0, -1.5):
            rng = np.random.default_rng(32)
            n, T = 40, 4
            coords = rng.uniform(-4, 4, (n, 3)).astype(np.float32)
            tv = rng.uniform(0, 1, (n, T)).astype(np.float32)
            tv[rng.random((n, T)) < 0.4] = 0
            radii = rng.uniform(1.0, 1.9, T if rti else n).astype(np.float32)
            og = oracle.GridMaker(0.5, 9.5, False, rti, 1.0, grm)
            diff = rng.standard_normal(og.grid_shape(T)).astype(np.float32)
            w = rng.standard_normal((n, 3)).astype(np.float32)
            v = rng.standard_normal((n, T)).astype(np.float32)
            cen = (0, 0.2, 0)
            dd, add, tdd = og.backward_gradients(cen, coords, tv, radii, diff, w, v)
            sdd, sadd, _ = og.backward_gradients(cen, coords, tv, radii, np.abs(diff), np.abs(w), np.abs(v))
            g = E.gridmaker(0.5, 9.5, False, rti, 1.0, grm)
            g_dd, g_add, g_tdd = E.array(diff.shape, fill=9.0), E.array((n, 3), fill=9.0), E.array((n, T), fill=9.0)
            assert lib.mg_backward_gradients(ctypes.byref(g), 1, None, n, None, E.f3(cen),
                                             E.ptr(E.put(coords)), E.ptr(E.put(tv)), E.ptr(E.put(radii)),
                                             T, E.ptr(E.put(diff)), E.ptr(E.put(w)), E.ptr(E.put(v)),
                                             E.ptr(g_dd), E.ptr(g_add), E.ptr(g_tdd), None) == 0
            assert not g_tdd.any()
            close_sums(g_dd, dd, np.abs(sdd) + 1.0, "diffdiff rti=%s grm=%s" % (rti, grm))
            close_sums(g_add, add, np.abs(sadd) * 4 + 1.0, "atom_diffdiff rti=%s grm=%s" % (rti, grm))


def interpolate(in_res, in_dim_a, out_res, out_dim_a, grids, quats, shifts, centers):
    B, K = grids.shape[:2]
    od = int(round(out_dim_a / out_res)) + 1
    out = E.array((B, K, od, od, od), fill=9.0)
    zeros = E.put(np.zeros((B, 3), np.float32))
    assert lib.mg_interpolate(in_res, in_dim_a, out_res, out_dim_a, B, K, E.ptr(E.put(centers)),
                              E.f3((0, 0, 0)), E.ptr(E.put(grids)), E.ptr(E.put(quats)),
                              E.f4((1, 0, 0, 0)), E.ptr(zeros), E.f3((0, 0, 0)), E.ptr(E.put(shifts)),
                              E.f3((0, 0, 0)), E.ptr(E.put(centers)), E.f3((0, 0, 0)), E.ptr(out),
                              None) == 0
    return out


def group_interpolate():
    lib.mg_interpolate_force_gather.argtypes = [ctypes.c_int]
    rng = np.random.default_rng(60)
    for in_res, in_a, out_res, out_a, K in [(0.5, 11.5, 0.5, 11.5, 3), (0.5, 15.5, 0.5, 15.5, 2),
                                           (0.5, 11.5, 0.25, 5.75, 2), (0.25, 5.75, 0.5, 11.5, 2)]:
        B = 2
        idim = int(round(in_a / in_res)) + 1
        grids = rng.standard_normal((B, K, idim, idim, idim)).astype(np.float32)
        quats = synth.random_quaternions(rng, B)
        quats[0] = (1, 0, 0, 0)
        shifts = rng.uniform(-1.5, 1.5, (B, 3)).astype(np.float32)
        centers = rng.uniform(-1, 1, (B, 3)).astype(np.float32)
        ref = oracle.interpolate_batch(in_res, in_a, out_res, out_a, centers, grids, quats,
                                       np.zeros((B, 3), np.float32), shifts, centers)
        got = interpolate(in_res, in_a, out_res, out_a, grids, quats, shifts, centers).copy()
        close(got, ref, "interpolate %s" % ((in_res, in_a, out_res, out_a),))
        lib.mg_interpolate_force_gather(1)
        gathered = interpolate(in_res, in_a, out_res, out_a, grids, quats, shifts, centers)
        lib.mg_interpolate_force_gather(0)
        # (bit for bit when both kernels round the lerps alike: in the plain build, where nothing is
        # contracted, and on the device, whose compiler contracts them the same way in both -- the
        # GPU test asserts it --; the host compiler of the contracting build does not)
        close(gathered, got, "gather path equals staged path", exact=not os.environ.get("EMU_CONTRACT"))


def group_config0():
    """The benchmark's configuration 0 at full size (1,540 atoms into 28 x 48^3) plus one example of
    configuration 1 (rotated, translated): forward in both write-outs, backward."""
    lib.mg_forward_index_paged.argtypes = [ctypes.c_int]
    c0 = synth.config0()
    c1 = synth.config1(nbatch=2)
    moved = oracle.transform_forward_batch(c1["offsets"], c1["quats"], c1["centers"],
                                           c1["translations"], c1["coords"])
    s1 = slice(int(c1["offsets"][1]), int(c1["offsets"][2]))
    for name, center, coords, types, radii in (
            ("configuration 0", c0["centers"][0], c0["coords"], c0["types"], c0["radii"]),
            ("configuration 1, example 1", c1["centers"][1], moved[s1], c1["types"][s1], c1["radii"][s1])):
        og = oracle.GridMaker(0.5, 23.5)
        ref = og.forward(center, coords, types, radii, 28)
        plain = forward_index((0.5, 23.5), center, coords, types, radii, 28).copy()
        lib.mg_forward_index_paged(1)
        paged = forward_index((0.5, 23.5), center, coords, types, radii, 28)
        lib.mg_forward_index_paged(0)
        close(plain, ref, name + " forward")
        close(paged, plain, name + " paged write-out", exact=True)
        rng = np.random.default_rng(5)
        diff = rng.standard_normal(ref.shape).astype(np.float32)
        ref32 = og.backward(center, coords, types, radii, diff)
        ref64 = og.backward(center, coords, types, radii, diff, f64=True)
        mag = np.abs(og.backward(center, coords, types, radii, np.abs(diff), f64=True)).max(
            axis=1, keepdims=True) + 1e-30
        g = E.gridmaker(0.5, 23.5)
        n = len(coords)
        grads = E.array((n, 3), fill=9.0)
        assert lib.mg_backward_index(ctypes.byref(g), 1, None, n, None, E.f3(center),
                                     E.ptr(E.put(coords)), E.ptr(E.put(types)), E.ptr(E.put(radii)), 28,
                                     E.ptr(E.put(diff)), E.ptr(grads), None) == 0
        check_grads(grads, ref32, ref64, mag, name + " backward")


GROUPS = {k[len("group_"):]: v for k, v in list(globals().items()) if k.startswith("group_")}

if __name__ == "__main__":
    names = sys.argv[1:] or sorted(GROUPS)
    for name in names:
        before = _checked[0]
        GROUPS[name]()
        print("emulated %s: %d comparisons passed" % (name, _checked[0] - before), flush=True)
