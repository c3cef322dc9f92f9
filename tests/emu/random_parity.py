"""TEST INFRASTRUCTURE: randomised parity of the emulated kernels against the oracle (CPU only).
Where cases.py repeats the fixed shapes of the GPU tests, this draws the configuration itself:
grids of 1 to 52 voxels a side at four resolutions, 1 to 40 channels, radius scales and Gaussian
radius multiples (negative ones: the truncated modes), centres off the origin, atoms inside, at the
edge of and outside the grid, fractional type indices, ragged batches with empty examples, sparse
and dense type vectors, radii by atom and by type.  Every draw runs the forward pass for index types
(per-wave and paged write-out, the latter bit-identical to the former), the backward pass for index
types, the forward pass for vector types (with and without per-slab atom lists, bit-identical), the
vector backward pass, relevance and -- on small grids -- resampling, with the bounds of the GPU
tests (binary densities bit-exact).  ``python tests/emu/random_parity.py [rounds] [seed]``."""
import ctypes
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)

import cases as C  # noqa: E402
import emu_capi as E  # noqa: E402
import oracle  # noqa: E402
import synth  # noqa: E402

lib = E.lib
EPS = C.EPS


def draw(rng):
    res = float(rng.choice([0.25, 0.5, 0.75, 1.0]))
    dim = int(rng.choice([1, 2, 3, 5, 7, 8, 12, 13, 16, 20, 24, 31, 32, 33, 40, 48, 52]))
    dimension = (dim - 1) * res
    ntypes = int(rng.choice([1, 2, 3, 4, 5, 8, 14, 28, 40]))
    if dim > 33:
        ntypes = min(ntypes, 4)                   # keeps a round short
    binary = bool(rng.integers(0, 2))
    grm = float(rng.choice([1.0, 1.0, 1.0, 0.7, 1.5, 2.0, -1.5, -0.5, -1.0]))
    scale = float(rng.choice([1.0, 1.0, 0.6, 1.3]))
    natoms = int(rng.choice([1, 2, 7, 30, 64, 65, 150]))
    size = rng.random()
    if size < 0.04:          # a grid of more than one z slab (64: slabs of 32 voxels), few atoms and channels
        dim, ntypes, natoms = int(rng.choice([64, 65, 96])), min(ntypes, 2), min(natoms, 30)
        dimension = (dim - 1) * res
    elif size < 0.10:        # more atoms than the sort keeps in registers, than one chunk of records holds
        dim, ntypes, natoms = min(dim, 24), min(ntypes, 5), int(rng.choice([700, 5000]))
        dimension = (dim - 1) * res
    half = dimension / 2
    spread = half + float(rng.choice([0.0, 1.0, 3.0]))
    center = rng.uniform(-2, 2, 3).astype(np.float32) * float(rng.choice([0, 1, 10]))
    coords = (center + rng.uniform(-spread - 1e-3, spread + 1e-3, (natoms, 3))).astype(np.float32)
    if rng.random() < 0.3:                         # some atoms exactly on voxel centres and grid corners
        k = rng.integers(0, dim, (natoms, 3))
        on = rng.random(natoms) < 0.4
        coords[on] = (center - half + k[on] * res).astype(np.float32)
    radii = rng.uniform(0.3, 2.5, natoms).astype(np.float32)
    if rng.random() < 0.5:
        # radii whose cut-off (final radius) is the distance between two voxel centres, to the
        # last bit or next to it: with atoms on voxel centres, voxels then sit ON the cut-off,
        # where a truncated density and its gradient jump
        frm = -grm if grm < 0 else (1 + 2 * grm * grm) / (2 * grm)
        if binary:
            frm = 1.0
        steps = rng.integers(0, 6, (natoms, 3))
        lattice = res * np.sqrt((steps * steps).sum(1).astype(np.float64))
        pick = (rng.random(natoms) < 0.6) & ((steps * steps).sum(1) > 0)
        exact = (np.maximum(lattice, res) / (scale * frm)).astype(np.float32)
        nudge = rng.integers(-1, 2, natoms)
        exact = np.where(nudge > 0, np.nextafter(exact, np.float32(9)), np.where(nudge < 0, np.nextafter(exact, np.float32(0)), exact))
        radii[pick] = exact[pick].astype(np.float32)
    radii[rng.random(natoms) < 0.05] = 0.0
    return dict(res=res, dim=dim, dimension=dimension, ntypes=ntypes, binary=binary, grm=grm,
                scale=scale, natoms=natoms, center=center, coords=coords, radii=radii)


def tail_allowance(og, center, coords, radii_of, weights, diff, all_channels=False):
    """What rounding inside the quadratic tail can move a sum by, which the noise allowances of the
    GPU tests (a multiple of eps * sum |term|) do not cover because the TERMS themselves are
    differences of nearly equal numbers towards the cut-off: the gradient (D * dist / ar + E) / ar,
    formed with two divisions by the reference (src/grid_maker.cu:881-896) and with the reciprocal
    of ar by the kernels, and the density A q^2 + B q + C (src/grid_maker.cu:95-130).  Returns
    (per atom [n, 1], per atom and channel [n, T]): a few eps * (|D| frm + |E|) / ar, and
    eps * (|A| frm^2 + |B| frm + |C|), for every unit of |upstream value| of a voxel in the tail.
    weights [n, T] (index types: one-hot), radii_of(a, t) the radius of atom a in channel t.  Only
    matters when the rest of the sum is small -- an atom on a voxel centre whose neighbours sit at
    the cut-off, an atom that reaches the grid with the end of its tail only."""
    p = og.p
    dim, res = int(p.dim), float(p.resolution)
    grm, frm = float(p.gaussian_radius_multiple), float(p.final_radius_multiple)
    origin = np.asarray(center, np.float64) - float(p.dimension) / 2
    ax = [origin[d] + np.arange(dim) * res for d in range(3)]
    n, T = weights.shape
    atom, chan = np.zeros((n, 1)), np.zeros((n, T))
    for a in range(n):
        for t in (range(T) if all_channels else np.nonzero(weights[a])[0]):
            ar = float(radii_of(a, t)) * float(p.radius_scale)
            if not ar > 0:
                continue
            reach = ar * frm * 1.001
            sl = [np.nonzero(np.abs(ax[d] - coords[a, d]) <= reach)[0] for d in range(3)]
            if min(len(x) for x in sl) == 0:
                continue
            gx, gy, gz = np.meshgrid(ax[0][sl[0]], ax[1][sl[1]], ax[2][sl[2]], indexing="ij")
            dist = np.sqrt((gx - coords[a, 0]) ** 2 + (gy - coords[a, 1]) ** 2 + (gz - coords[a, 2]) ** 2)
            tail = (dist > ar * grm * 0.999) & (dist <= reach)
            mass = np.abs(diff[t][np.ix_(sl[0], sl[1], sl[2])])[tail].sum()
            atom[a, 0] += abs(float(weights[a, t])) * mass * 4 * EPS * (abs(float(p.D)) * frm + abs(float(p.E))) / ar
            chan[a, t] += mass * 4 * EPS * (abs(float(p.A)) * frm * frm + abs(float(p.B)) * frm + abs(float(p.C)))
    return atom, chan


def one_round(rng):
    d = draw(rng)
    res, dimension, T, binary, grm, scale, n = (d["res"], d["dimension"], d["ntypes"], d["binary"],
                                                d["grm"], d["scale"], d["natoms"])
    center, coords, radii = d["center"], d["coords"], d["radii"]
    gm_args = (res, dimension, binary, False, scale, grm)
    tag = "res %g dim %d T %d n %d binary %d grm %g scale %g" % (res, d["dim"], T, n, binary, grm, scale)
    print("parity:", tag, flush=True)
    og = oracle.GridMaker(*gm_args)

    # ---- index types: forward (both write-outs), backward, relevance --------------------------
    types = rng.integers(-1, T, n).astype(np.float32)
    # (a fraction below one half: the forward pass takes floor(type), the backward pass round(type),
    # src/grid_maker.cpp:436-467, and beyond the last channel the reference throws)
    types = types + rng.uniform(0, 0.45, n).astype(np.float32) * (types >= 0)
    ref = og.forward(center, coords, types, radii, T)
    lib.mg_forward_index_paged(0)
    plain = np.array(C.forward_index(gm_args, center, coords, types, radii, T))
    C.close(plain, ref, "forward " + tag, exact=binary)
    # the library's own workspace, or the entry point that allocates nothing (when the case fits
    # its fixed scratch memory): the same grid bit for bit
    variant = str(rng.choice(["cached", "static"]))
    g0 = E.gridmaker(*gm_args)
    if variant == "cached" or lib.mg_forward_index_workspace_size(ctypes.byref(g0), 1, n, T) <= C.STATIC_BYTES:
        other = C.forward_index(gm_args, center, coords, types, radii, T, variant=variant)
        C.close(other, plain, "forward, %s workspace, " % variant + tag, exact=True)
    # the other instances of the splat launch: paged write-out, tail-only blocks without the
    # exponential, both -- the same grid bit for bit
    for paged_on, core_on in ((1, 0), (0, 1), (1, 1)):
        lib.mg_forward_index_paged(paged_on)
        lib.mg_forward_index_core_skip(core_on)
        other = C.forward_index(gm_args, center, coords, types, radii, T)
        lib.mg_forward_index_paged(0)
        lib.mg_forward_index_core_skip(0)
        C.close(other, plain, "splat instance paged=%d core_skip=%d, " % (paged_on, core_on) + tag, exact=True)

    if True:
        diff = rng.standard_normal(ref.shape).astype(np.float32)
        ref32 = og.backward(center, coords, types, radii, diff)
        ref64 = og.backward(center, coords, types, radii, diff, f64=True)
        mag = np.abs(og.backward(center, coords, types, radii, np.abs(diff), f64=True)).max(
            axis=1, keepdims=True) + 1e-30
        onehot = np.zeros((n, T), np.float32)
        chan = np.round(types).astype(int)
        onehot[np.nonzero(chan >= 0)[0], chan[chan >= 0]] = 1.0
        mag = mag + tail_allowance(og, center, coords, lambda a, t: radii[a], onehot, diff)[0] / (16 * EPS)
        g = E.gridmaker(*gm_args)
        grads = E.array((n, 3), fill=9.0)
        assert lib.mg_backward_index(ctypes.byref(g), 1, None, n, None, E.f3(center),
                                     E.ptr(E.put(coords)), E.ptr(E.put(types)), E.ptr(E.put(radii)), T,
                                     E.ptr(E.put(diff)), E.ptr(grads), None) == 0
        C.check_grads(grads, ref32, ref64, mag, "backward " + tag)

        dens = ref * rng.uniform(0.5, 3.0, ref.shape).astype(np.float32) if binary else ref
        rel_ref = og.backward_relevance(center, coords, types, radii, dens, diff)
        rel_scale = og.backward_relevance(center, coords, types, radii, dens, np.abs(diff))
        rel = E.array(n, fill=5.0)
        assert lib.mg_backward_relevance(ctypes.byref(g), 1, None, n, None, E.f3(center),
                                         E.ptr(E.put(coords)), E.ptr(E.put(types)), E.ptr(E.put(radii)),
                                         T, E.ptr(E.put(dens)), E.ptr(E.put(diff)), E.ptr(rel), None) == 0
        C.close_sums(rel, rel_ref, rel_scale, "relevance " + tag)

    # ---- a ragged batch of the same atoms, with an empty example -----------------------------
    if n >= 7:
        cuts = np.sort(rng.integers(0, n + 1, 3))
        off = np.array([0, cuts[0], cuts[0], cuts[1], cuts[2], n], np.int64)
        B = len(off) - 1
        centers = (center + rng.uniform(-1, 1, (B, 3))).astype(np.float32)
        refb = og.forward_batch(off, centers, coords, types, radii, T)
        gotb = C.forward_index(gm_args, centers, coords, types, radii, T, offsets=off,
                               per_example=max(int(np.diff(off).max()), 1), nbatch=B)
        C.close(gotb, refb, "ragged batch " + tag, exact=binary)

    # ---- the same ragged batch through the transform, the backward pass and the launch that also
    # takes the gradients back through the rotation (bit-identical to the two calls)
    if n >= 7:
        quats = synth.random_quaternions(rng, B)
        rot_c = rng.uniform(-2, 2, (B, 3)).astype(np.float32)
        trans = rng.uniform(-1, 1, (B, 3)).astype(np.float32)
        off32 = E.put(off, np.int32)
        width = max(int(np.diff(off).max()), 1)
        moved = E.array((n, 3), fill=9.0)
        assert lib.mg_transform_forward(B, E.ptr(off32), width, E.ptr(E.put(quats)), E.f4((1, 0, 0, 0)),
                                        E.ptr(E.put(rot_c)), E.f3((0, 0, 0)), E.ptr(E.put(trans)),
                                        E.f3((0, 0, 0)), 1, E.ptr(E.put(coords)), E.ptr(moved), None) == 0
        ref_moved = oracle.transform_forward_batch(off, quats, rot_c, trans, coords)
        C.close(moved, ref_moved, "transform batch " + tag, exact=True)
        bdiff = rng.standard_normal(refb.shape).astype(np.float32)
        bref = og.backward_batch(off, centers, ref_moved, types, radii, bdiff)
        gb = E.gridmaker(*gm_args)
        bgot, bun = E.array((n, 3), fill=9.0), E.array((n, 3), fill=9.0)
        bargs = [ctypes.byref(gb), B, E.ptr(off32), width, E.ptr(E.put(centers)), E.f3((0, 0, 0)),
                 E.ptr(E.put(ref_moved)), E.ptr(E.put(types)), E.ptr(E.put(radii)), T, E.ptr(E.put(bdiff))]
        assert lib.mg_backward_index(*bargs, E.ptr(bgot), None) == 0
        magb = np.concatenate([
            np.abs(og.backward(centers[b], ref_moved[off[b]:off[b + 1]], types[off[b]:off[b + 1]],
                               radii[off[b]:off[b + 1]], np.abs(bdiff[b]), f64=True)).max(axis=1, keepdims=True)
            if off[b + 1] > off[b] else np.zeros((0, 1)) for b in range(B)]) + 1e-30
        allow = np.concatenate([
            tail_allowance(og, centers[b], ref_moved[off[b]:off[b + 1]],
                           (lambda a, t, lo=off[b]: radii[lo + a]),
                           onehot[off[b]:off[b + 1]], bdiff[b])[0] for b in range(B)])
        err = np.abs(np.asarray(bgot, np.float64) - bref)
        assert (err <= C.ATOL + C.RTOL * np.abs(bref) + 64 * EPS * magb + 4 * allow).all(), \
            "backward batch %s: worst %g" % (tag, float(err.max()))
        assert lib.mg_backward_index_unrotated(*bargs, E.ptr(E.put(quats)), E.f4((1, 0, 0, 0)), E.ptr(E.put(rot_c)),
                                               E.f3((0, 0, 0)), E.ptr(bun), None) == 0
        C.close(bun, oracle.transform_backward_batch(off, quats, rot_c, trans, np.array(bgot), dotranslate=False),
                "fused un-rotation " + tag, exact=True)

    # ---- vector types: forward (atom lists or not), backward -----------------------------------
    rti = bool(rng.random() < 0.25)
    sparse = float(rng.choice([0.0, 0.5, 0.9]))
    tv = (rng.uniform(0, 1.5, (n, T)) * (rng.random((n, T)) >= sparse)).astype(np.float32)
    vr = rng.uniform(0.4, 2.2, T).astype(np.float32) if rti else radii
    vargs = (res, dimension, binary, rti, scale, grm)
    ogv = oracle.GridMaker(*vargs)
    vref = ogv.forward(center, coords, tv, vr)
    plainv = np.array(C.forward_vector(vargs, center, coords, tv, vr))
    C.close(plainv, vref, "vector forward rti=%d " % rti + tag, exact=binary)
    listed = C.forward_vector(vargs, center, coords, tv, vr, lists=True)
    C.close(listed, plainv, "atom lists " + tag, exact=True)
    vdiff = rng.standard_normal(vref.shape).astype(np.float32)
    ra32, rt32 = ogv.backward(center, coords, tv, vr, vdiff)
    ra64, rt64 = ogv.backward(center, coords, tv, vr, vdiff, f64=True)
    ma, mt = ogv.backward(center, coords, np.abs(tv), vr, np.abs(vdiff), f64=True)
    ma = np.abs(ma).max(axis=1, keepdims=True) + 1e-30
    extra_a, extra_t = tail_allowance(ogv, center, coords, (lambda a, t: vr[t]) if rti else (lambda a, t: vr[a]),
                                      tv, vdiff, all_channels=True)
    ma, mt = ma + extra_a / (16 * EPS), mt + extra_t / (16 * EPS)
    gv = E.gridmaker(*vargs)
    ag, tg = E.array((n, 3), fill=9.0), E.array((n, T), fill=9.0)
    assert lib.mg_backward_vector(ctypes.byref(gv), 1, None, n, None, E.f3(center), E.ptr(E.put(coords)),
                                  E.ptr(E.put(tv)), E.ptr(E.put(vr)), T, E.ptr(E.put(vdiff)),
                                  E.ptr(ag), E.ptr(tg), None) == 0
    a64, t64 = np.asarray(ag, np.float64), np.asarray(tg, np.float64)
    what = "vector backward rti=%d " % rti + tag
    for got, r64, r32, m, name in ((a64, ra64, ra32, ma, "atom"), (t64, rt64, rt32, mt, "type")):
        for ref_, k in ((r64, 16), (r32, 64)):
            bound = C.ATOL + C.RTOL * np.abs(ref_) + k * EPS * m
            bad = np.argwhere(np.abs(got - ref_) > bound)
            if len(bad):
                i = tuple(bad[0])
                raise AssertionError("%s: %s gradient %s got %r f64 %r f32 %r bound %g scale %g; atom at voxel %s "
                                     "radius %r weights %s" % (what, name, i, got[i], r64[i], r32[i], bound[i],
                                                               np.broadcast_to(m, got.shape)[i],
                                                               (coords[i[0]] - (center - dimension / 2)) / res,
                                                               vr if rti else vr[i[0]], tv[i[0]]))

    # ---- a padded batch of vector-typed examples (every example `width` rows, the rows past its
    # atoms with zero weights and radius): forward and backward equal the single launches
    if 2 <= n <= 65 and not rti and d["dim"] <= 33:
        PB = 3
        width = n + int(rng.integers(0, 5))
        counts = [n, int(rng.integers(0, n + 1)), int(rng.integers(1, n + 1))]
        pc = np.zeros((PB, width, 3), np.float32)
        pw = np.zeros((PB, width, T), np.float32)
        pr = np.zeros((PB, width), np.float32)
        pcen = (center + rng.uniform(-1, 1, (PB, 3))).astype(np.float32)
        for b, k in enumerate(counts):
            pc[b, :k], pw[b, :k], pr[b, :k] = coords[:k], tv[:k], vr[:k]
        pout = E.array((PB, T) + vref.shape[1:], fill=3.0)
        flat = [E.ptr(E.put(pc.reshape(-1, 3))), E.ptr(E.put(pw.reshape(-1, T))), E.ptr(E.put(pr.reshape(-1)))]
        assert lib.mg_forward_vector(ctypes.byref(gv), PB, None, width, E.ptr(E.put(pcen)), E.f3((0, 0, 0)),
                                     flat[0], flat[1], flat[2], T, E.ptr(pout), None) == 0
        pdiff = rng.standard_normal(pout.shape).astype(np.float32)
        pag, ptg = E.array((PB * width, 3), fill=9.0), E.array((PB * width, T), fill=9.0)
        assert lib.mg_backward_vector(ctypes.byref(gv), PB, None, width, E.ptr(E.put(pcen)), E.f3((0, 0, 0)),
                                      flat[0], flat[1], flat[2], T, E.ptr(E.put(pdiff)), E.ptr(pag),
                                      E.ptr(ptg), None) == 0
        for b, k in enumerate(counts):
            one = np.array(C.forward_vector(vargs, pcen[b], coords[:k], tv[:k], vr[:k])) if k else np.zeros_like(vref)
            C.close(pout[b], one, "padded vector batch, example %d, " % b + tag, exact=True)
            if k:
                a1, t1 = E.array((k, 3), fill=9.0), E.array((k, T), fill=9.0)
                assert lib.mg_backward_vector(ctypes.byref(gv), 1, None, k, None, E.f3(pcen[b]),
                                              E.ptr(E.put(coords[:k])), E.ptr(E.put(tv[:k])), E.ptr(E.put(vr[:k])),
                                              T, E.ptr(E.put(pdiff[b])), E.ptr(a1), E.ptr(t1), None) == 0
                C.close(pag[b * width:b * width + k], a1, "padded vector backward, atoms, " + tag, exact=True)
                C.close(ptg[b * width:b * width + k], t1, "padded vector backward, types, " + tag, exact=True)
            assert not np.asarray(pag[b * width + k:(b + 1) * width]).any(), "gradient of a padding row"

    # ---- second order (Gaussian densities only, src/grid_maker.cpp:559), few atoms: the oracle is slow
    if not binary and n <= 65 and d["dim"] <= 33:
        w = rng.standard_normal((n, 3)).astype(np.float32)
        v = rng.standard_normal((n, T)).astype(np.float32)
        dd, add, _ = ogv.backward_gradients(center, coords, tv, vr, vdiff, w, v)
        sdd, sadd, _ = ogv.backward_gradients(center, coords, np.abs(tv), vr, np.abs(vdiff), np.abs(w), np.abs(v))
        g_dd, g_add, g_tdd = E.array(vdiff.shape, fill=9.0), E.array((n, 3), fill=9.0), E.array((n, T), fill=9.0)
        assert lib.mg_backward_gradients(ctypes.byref(gv), 1, None, n, None, E.f3(center), E.ptr(E.put(coords)),
                                         E.ptr(E.put(tv)), E.ptr(E.put(vr)), T, E.ptr(E.put(vdiff)),
                                         E.ptr(E.put(w)), E.ptr(E.put(v)), E.ptr(g_dd), E.ptr(g_add),
                                         E.ptr(g_tdd), None) == 0
        # (the oracle sums up to a million terms per atom in a float, in another order than the
        # kernel: four times the allowance of the GPU tests' cases, which have 4 channels)
        C.close_sums(g_dd, dd, 4 * (np.abs(sdd) + 1.0), "diffdiff rti=%d " % rti + tag)
        C.close_sums(g_add, add, 4 * (np.abs(sadd) * 4 + 1.0), "atom_diffdiff rti=%d " % rti + tag)

    # ---- resampling of the density under a random rotation (small grids: the oracle is a loop) --
    if 2 <= d["dim"] <= 24 and T <= 8:
        B = 2
        grids = np.stack([ref, ref[:, ::-1].copy()]).astype(np.float32)
        quats = synth.random_quaternions(rng, B)
        shifts = rng.uniform(-1.5, 1.5, (B, 3)).astype(np.float32)
        centers = np.stack([center, center]).astype(np.float32)
        out_res = float(rng.choice([res, res, res * 0.5, res * 1.25]))
        out_dim = int(rng.choice([d["dim"], max(d["dim"] - 3, 1), d["dim"] + 2]))
        out_a = (out_dim - 1) * out_res
        iref = oracle.interpolate_batch(res, dimension, out_res, out_a, centers, grids, quats,
                                        np.zeros((B, 3), np.float32), shifts, centers)
        igot = C.interpolate(res, dimension, out_res, out_a, grids, quats, shifts, centers)
        C.close(igot, iref, "interpolate to res %g dim %d, " % (out_res, out_dim) + tag)


def main():
    """random_parity.py [rounds] [seed] [first round]: every round has a generator of its own, seeded
    by (seed, round), so that a failing round can be run alone."""
    rounds = int(sys.argv[1]) if len(sys.argv) > 1 else 10
    seed = int(sys.argv[2]) if len(sys.argv) > 2 else 1
    first = int(sys.argv[3]) if len(sys.argv) > 3 else 0
    lib.mg_forward_index_paged.argtypes = [ctypes.c_int]
    lib.mg_forward_index_core_skip.argtypes = [ctypes.c_int]
    for r in range(first, first + rounds):
        print("round %d of seed %d:" % (r, seed), end=" ")
        # (the arrays of this round start 0 to 12 bytes past a 16-byte boundary)
        E.MISALIGN = int(np.random.default_rng([seed, r, 1]).choice([0, 0, 1, 2, 3]))
        one_round(np.random.default_rng([seed, r]))
        E.release_all()
    print("random parity: %d rounds passed" % rounds)


if __name__ == "__main__":
    main()
