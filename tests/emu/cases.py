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


def group_forward_paged():
    """The paged write-out (workgroups that own a slab and write whole 4 KB pages) gives the grids
    of the per-wave write-out bit for bit: dims 16, 24, 48 and smaller, binary and Gaussian, batches
    with empty examples, output arrays at several alignments inside a 4 KB page."""
    lib.mg_forward_index_paged.argtypes = [ctypes.c_int]
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


GROUPS = {k[len("group_"):]: v for k, v in list(globals().items()) if k.startswith("group_")}

if __name__ == "__main__":
    names = sys.argv[1:] or sorted(GROUPS)
    for name in names:
        before = _checked[0]
        GROUPS[name]()
        print("emulated %s: %d comparisons passed" % (name, _checked[0] - before), flush=True)
