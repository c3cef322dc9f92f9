"""TEST INFRASTRUCTURE: hostile inputs against every kernel under the HIP emulation (CPU only).
Not-a-number and infinite coordinates, radii, types, centres and quaternions, radii of zero, below
zero and far larger than the grid, types at and beyond the channel count, grids of 1 to 65 voxels a
side, empty examples, batches of more examples than a wave has lanes.  The only requirement is that
every kernel returns: no access outside an array (the arrays end at an inaccessible page, buffer
descriptors are checked), no deadlock.  Run as ``python tests/emu/fuzz.py [rounds] [seed]``."""
import ctypes
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)

import emu_capi as E  # noqa: E402

lib = E.lib
BAD = np.array([np.nan, np.inf, -np.inf, 1e30, -1e30, 1e-40, 0.0, -0.0], np.float32)


def poison(rng, a, frac):
    """Replaces a fraction of the entries of a by hostile values."""
    a = np.array(a, np.float32)
    m = rng.random(a.shape) < frac
    a[m] = rng.choice(BAD, int(m.sum()))
    return a


def one_round(rng):
    res = float(rng.choice([0.25, 0.5, 1.0, 0.37]))
    dim = int(rng.choice([1, 2, 3, 4, 5, 8, 12, 13, 16, 24, 25, 31, 48, 50, 65]))
    dimension = (dim - 1) * res
    ntypes = int(rng.choice([1, 2, 3, 7, 28, 33, 65]))
    if dim > 31:
        ntypes = min(ntypes, 3)                  # keeps a round short
    nbatch = int(rng.choice([1, 2, 3, 5, 70]))
    if dim > 16 and nbatch > 3:
        nbatch = 3
    sizes = rng.integers(0, 40, nbatch)
    sizes[rng.random(nbatch) < 0.3] = 0
    off = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    n = int(off[-1])
    width = int(max(sizes.max(), 0))
    frac = float(rng.choice([0.0, 0.05, 0.5]))
    half = dimension / 2 + 3
    coords = poison(rng, rng.uniform(-half, half, (n, 3)), frac)
    types = poison(rng, rng.integers(-2, ntypes + 2, n) + rng.uniform(-0.6, 0.6, n), frac)
    radii = poison(rng, rng.choice([0.0, -1.0, 0.3, 1.5, 3.0, 500.0], n), frac)
    tv = poison(rng, rng.uniform(0, 1, (n, ntypes)) * (rng.random((n, ntypes)) > 0.5), frac / 4)
    tr = poison(rng, rng.uniform(0.5, 2.5, (nbatch, ntypes)), frac / 4)
    centers = poison(rng, rng.uniform(-1, 1, (nbatch, 3)), frac / 4)
    binary = bool(rng.integers(0, 2))
    grm = float(rng.choice([1.0, 1.0, 0.7, 2.0, -1.5, -0.5]))
    scale = float(rng.choice([1.0, 1.3]))
    tag = "res %g dim %d T %d B %d n %d binary %d grm %g poison %g" % (res, dim, ntypes, nbatch, n,
                                                                       binary, grm, frac)
    print("fuzz:", tag, flush=True)
    g = E.gridmaker(res, dimension, binary, False, scale, grm)
    grti = E.gridmaker(res, dimension, binary, True, scale, grm)
    assert int(g.dim) == dim, (int(g.dim), dim)
    d_off, d_cen = E.put(off, np.int32), E.put(centers)
    d_c, d_t, d_r, d_tv, d_tr = E.put(coords), E.put(types), E.put(radii), E.put(tv), E.put(tr)
    vox = (nbatch, ntypes, dim, dim, dim)
    out = E.array(vox, fill=7.0)
    diff = E.put(poison(rng, rng.standard_normal(vox), frac / 8))
    common = [nbatch, E.ptr(d_off), width, E.ptr(d_cen), E.f3((0, 0, 0)), E.ptr(d_c)]
    ok = (0, -3)        # MG_OK or MG_ERR_UNSUPPORTED

    for paged, core in ((0, 0), (1, 0), (0, 1), (1, 1)):      # every instance of the splat launch
        lib.mg_forward_index_paged(paged)
        lib.mg_forward_index_core_skip(core)
        need = lib.mg_forward_index_workspace_size(ctypes.byref(g), nbatch, width, ntypes)
        ws = E.array(max(need, 1), np.uint8, tight=False)
        assert lib.mg_forward_index_ws(ctypes.byref(g), *common, E.ptr(d_t), E.ptr(d_r), ntypes,
                                       E.ptr(out), E.ptr(ws), need, None) in ok
    lib.mg_forward_index_paged(0)
    lib.mg_forward_index_core_skip(0)
    for gg, rad in ((g, d_r), (grti, d_tr)):
        need = lib.mg_forward_vector_workspace_size(ctypes.byref(gg), nbatch, width, ntypes)
        ws = E.array(max(need, 1), np.uint8, tight=False)
        assert lib.mg_forward_vector_ws(ctypes.byref(gg), *common, E.ptr(d_tv), E.ptr(rad), ntypes,
                                        E.ptr(out), E.ptr(ws) if need else None, need, None) in ok
    ag, tg, rel = E.array((max(n, 1), 3), fill=9.0), E.array((max(n, 1), ntypes), fill=9.0), \
        E.array(max(n, 1), fill=9.0)
    assert lib.mg_backward_index(ctypes.byref(g), *common, E.ptr(d_t), E.ptr(d_r), ntypes,
                                 E.ptr(diff), E.ptr(ag), None) in ok
    quats = E.put(poison(rng, rng.normal(size=(nbatch, 4)), frac / 4))
    assert lib.mg_backward_index_unrotated(ctypes.byref(g), *common, E.ptr(d_t), E.ptr(d_r), ntypes,
                                           E.ptr(diff), E.ptr(quats), E.f4((1, 0, 0, 0)), E.ptr(d_cen),
                                           E.f3((0, 0, 0)), E.ptr(ag), None) in ok
    for gg, rad in ((g, d_r), (grti, d_tr)):
        assert lib.mg_backward_vector(ctypes.byref(gg), *common, E.ptr(d_tv), E.ptr(rad), ntypes,
                                      E.ptr(diff), E.ptr(ag), E.ptr(tg), None) in ok
    assert lib.mg_backward_relevance(ctypes.byref(g), *common, E.ptr(d_t), E.ptr(d_r), ntypes,
                                     E.ptr(out), E.ptr(diff), E.ptr(rel), None) in ok
    if not binary:
        dd = E.array(vox, fill=9.0)
        add, tdd = E.array((max(n, 1), 3), fill=9.0), E.array((max(n, 1), ntypes), fill=9.0)
        for gg, rad in ((g, d_r), (grti, d_tr)):
            assert lib.mg_backward_gradients(ctypes.byref(gg), *common, E.ptr(d_tv), E.ptr(rad), ntypes,
                                             E.ptr(diff), E.ptr(ag), E.ptr(tg), E.ptr(dd), E.ptr(add),
                                             E.ptr(tdd), None) in ok
    moved = E.array((max(n, 1), 3))
    for fn in (lib.mg_transform_forward, lib.mg_transform_backward):
        assert fn(nbatch, E.ptr(d_off), width, E.ptr(quats), E.f4((1, 0, 0, 0)), E.ptr(d_cen),
                  E.f3((0, 0, 0)), E.ptr(d_cen), E.f3((0, 0, 0)), 1, E.ptr(d_c), E.ptr(moved), None) in ok
    # resampling onto a grid of another size
    odim = int(rng.choice([1, 3, 8, 13, 16, 24]))
    ores = float(rng.choice([res, res * 0.97, res * 2, res / 2]))
    K = min(ntypes, 3)
    src = E.put(poison(rng, rng.standard_normal((nbatch, K, dim, dim, dim)), frac / 8))
    dst = E.array((nbatch, K, odim, odim, odim), fill=9.0)
    for force in (0, 1):
        lib.mg_interpolate_force_gather(force)
        assert lib.mg_interpolate(res, dimension, ores, (odim - 1) * ores, nbatch, K, E.ptr(d_cen),
                                  E.f3((0, 0, 0)), E.ptr(src), E.ptr(quats), E.f4((1, 0, 0, 0)),
                                  E.ptr(d_cen), E.f3((0, 0, 0)), E.ptr(d_cen), E.f3((0, 0, 0)),
                                  E.ptr(d_cen), E.f3((0, 0, 0)), E.ptr(dst), None) in ok
    lib.mg_interpolate_force_gather(0)


def extreme_scalars():
    """Batch sizes, atom counts and channel counts of zero, one, minus one and 2^31 - 1 with no arrays
    at all: the size functions must not overflow and every launching entry point must refuse."""
    big = 2 ** 31 - 1
    z3, q1 = E.f3((0, 0, 0)), E.f4((1, 0, 0, 0))
    for res, dimension in ((0.5, 3.5), (0.001, 65.0), (0.5, 32767.0)):
        g = E.gridmaker(res, dimension)
        for nb in (0, 1, big):
            for per in (0, 1, big):
                for ntypes in (0, 1, big):
                    lib.mg_forward_index_workspace_size(ctypes.byref(g), nb, per, ntypes)
                    lib.mg_forward_vector_workspace_size(ctypes.byref(g), nb, per, ntypes)
        for nb, per, ntypes in ((big, big, big), (-1, 1, 1), (1, -1, 1), (1, 1, -1), (big, 1, 1)):
            codes = [
                lib.mg_forward_index(ctypes.byref(g), nb, None, per, None, z3, None, None, None, ntypes, None, None),
                lib.mg_backward_index(ctypes.byref(g), nb, None, per, None, z3, None, None, None, ntypes, None,
                                      None, None),
                lib.mg_forward_vector(ctypes.byref(g), nb, None, per, None, z3, None, None, None, ntypes, None, None),
                lib.mg_transform_forward(nb, None, per, None, q1, None, z3, None, z3, 1, None, None, None)]
            assert all(c < 0 for c in codes), (nb, per, ntypes, codes)
    print("fuzz: extreme scalar arguments refused", flush=True)


if __name__ == "__main__":
    rounds = int(sys.argv[1]) if len(sys.argv) > 1 else 20
    seed = int(sys.argv[2]) if len(sys.argv) > 2 else 0
    lib.mg_forward_index_paged.argtypes = [ctypes.c_int]
    lib.mg_forward_index_core_skip.argtypes = [ctypes.c_int]
    lib.mg_interpolate_force_gather.argtypes = [ctypes.c_int]
    extreme_scalars()
    rng = np.random.default_rng(seed)
    for _ in range(rounds):
        one_round(rng)
    print("fuzz: %d rounds returned" % rounds)
