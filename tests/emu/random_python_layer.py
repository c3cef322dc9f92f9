"""TEST INFRASTRUCTURE: randomised calls of the Python host layer on the fake device of fake_cuda.py
(emulated kernels behind it) against the oracle.  Each round draws a grid maker (resolution, size,
binary, radius scale, radius multiple), a molecule, and the way the call is made: device tensors,
host arrays or float64 grids; a single example, a padded batch or a ragged batch whose AtomBatch is
reused with a larger batch afterwards (its cached workspaces must grow); index or vector types,
radii by atom or by type; backward with and without the fused un-rotation; the autograd layer with
one example and with a padded batch; the overloads of GridInterpolater; Transform on device and
host arrays.  ``python tests/emu/random_python_layer.py [rounds] [seed]``."""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, HERE)

import python_layer as P  # noqa: E402  (activates the fake device)
import libmolgrid_amd as mg  # noqa: E402
import oracle  # noqa: E402
import synth  # noqa: E402

dev, close = P.dev, P.close


def as_input(rng, a):
    """The array as a device tensor or as a host array (which the layer stages itself)."""
    return dev(a) if rng.random() < 0.7 else np.ascontiguousarray(a)


def one_round(rng):
    res = float(rng.choice([0.25, 0.5, 1.0]))
    dim = int(rng.choice([4, 7, 12, 16, 24]))
    dimension = (dim - 1) * res
    binary = bool(rng.integers(0, 2))
    grm = float(rng.choice([1.0, 1.0, 0.7, 2.0, -1.5]))
    scale = float(rng.choice([1.0, 1.3]))
    T = int(rng.choice([1, 3, 8, 30]))
    n = int(rng.choice([1, 9, 40, 70]))
    tag = "res %g dim %d T %d n %d binary %d grm %g scale %g" % (res, dim, T, n, binary, grm, scale)
    print("python layer:", tag, flush=True)
    gm = mg.GridMaker(res, dimension, binary, False, scale, grm)
    og = oracle.GridMaker(res, dimension, binary, False, scale, grm)
    center = tuple(float(v) for v in rng.uniform(-1, 1, 3))
    half = dimension / 2 + 1.0
    coords = (np.asarray(center) + rng.uniform(-half, half, (n, 3))).astype(np.float32)
    types = rng.integers(-1, T, n).astype(np.float32)
    radii = rng.uniform(0.4, 2.2, n).astype(np.float32)

    # ---- one example, index types: float32 device grid, host grid or float64 device grid ----------
    ref = og.forward(center, coords, types, radii, T)
    kind = rng.integers(0, 3)
    if kind == 0:
        out = torch.full(gm.grid_dimensions(T), 7.0, device="cuda")
    elif kind == 1:
        out = np.full(ref.shape, 7.0, np.float32)
    else:
        out = torch.full(gm.grid_dimensions(T), 7.0, device="cuda", dtype=torch.float64)
    gm.forward(center, as_input(rng, coords), as_input(rng, types), as_input(rng, radii), out)
    close(out, ref.astype(np.float64) if kind == 2 else ref, "forward (grid kind %d) " % kind + tag, exact=binary)
    diff = rng.standard_normal(ref.shape).astype(np.float32)
    grads = torch.full((n, 3), 9.0, device="cuda")
    gm.backward(center, as_input(rng, coords), as_input(rng, types), as_input(rng, radii), as_input(rng, diff), grads)
    close(grads, og.backward(center, coords, types, radii, diff), "backward " + tag, rtol=1e-4, atol=5e-5)

    # ---- ragged batch; then the SAME AtomBatch object is not reusable for another layout, but a second
    # one with more and larger examples on the same grid maker must get workspaces of its own size
    if n >= 9:
        for copies in (1, 3):
            cuts = np.sort(rng.integers(0, n + 1, 2))
            off1 = np.array([0, cuts[0], cuts[1], n], np.int64)
            off = np.concatenate([off1] + [off1[1:] + n * (k + 1) for k in range(copies - 1)])
            B = len(off) - 1
            bc, bt, br = np.tile(coords, (copies, 1)), np.tile(types, copies), np.tile(radii, copies)
            cen = (np.asarray(center) + rng.uniform(-0.5, 0.5, (B, 3))).astype(np.float32)
            batch = mg.AtomBatch(off)
            grid = torch.full((B,) + gm.grid_dimensions(T), 7.0, device="cuda")
            args = [dev(cen), dev(bc), dev(bt), dev(br)]
            for _ in range(2):                             # the second call finds the cached workspace
                gm.forward_batch(batch, *args, grid)
                close(grid, og.forward_batch(off, cen, bc, bt, br, T), "forward_batch x%d " % copies + tag, exact=binary)
            bdiff = rng.standard_normal(tuple(grid.shape)).astype(np.float32)
            bg = torch.full((len(bc), 3), 9.0, device="cuda")
            gm.backward_batch(batch, *args, dev(bdiff), bg)
            close(bg, og.backward_batch(off, cen, bc, bt, br, bdiff), "backward_batch x%d " % copies + tag,
                  rtol=1e-4, atol=5e-5)
            quats = synth.random_quaternions(rng, B)
            un = torch.full_like(bg, 9.0)
            gm.backward_batch(batch, *args, dev(bdiff), un, unrotate=(dev(quats), dev(cen)))
            close(un, oracle.transform_backward_batch(off, quats, cen, np.zeros_like(cen), bg.numpy(), dotranslate=False),
                  "backward_batch with un-rotation " + tag, exact=True)

    # ---- vector types, radii by atom or by type; the autograd layer -------------------------------
    rti = bool(rng.random() < 0.3)
    gv = mg.GridMaker(res, dimension, binary, rti, scale, grm)
    ov = oracle.GridMaker(res, dimension, binary, rti, scale, grm)
    tv = (rng.uniform(0, 1.5, (n, T)) * (rng.random((n, T)) > 0.5)).astype(np.float32)
    vr = rng.uniform(0.5, 2.0, T).astype(np.float32) if rti else radii
    vref = ov.forward(center, coords, tv, vr)
    vout = torch.full(gv.grid_dimensions(T), 3.0, device="cuda")
    gv.forward(center, as_input(rng, coords), as_input(rng, tv), as_input(rng, vr), vout)
    close(vout, vref, "vector forward rti=%d " % rti + tag, exact=binary)
    vdiff = rng.standard_normal(vref.shape).astype(np.float32)
    ra, rt = ov.backward(center, coords, tv, vr, vdiff)
    ag, tg = torch.full((n, 3), 9.0, device="cuda"), torch.full((n, T), 9.0, device="cuda")
    gv.backward(center, dev(coords), dev(tv), dev(vr), dev(vdiff), ag, tg)
    close(ag, ra, "vector backward, atoms, " + tag, rtol=1e-4, atol=5e-5)
    close(tg, rt, "vector backward, types, " + tag, rtol=1e-4, atol=5e-5)
    if not rti:
        from libmolgrid_amd.torch_bindings import Coords2Grid
        layer = Coords2Grid(gv, center=center)
        x = dev(coords)
        x.requires_grad_(True)
        g1 = layer(x, dev(tv), dev(vr))
        close(g1.detach(), vref, "Coords2Grid forward " + tag, exact=binary)
        g1.backward(dev(vdiff))
        close(x.grad, ra, "Coords2Grid backward " + tag, rtol=1e-4, atol=5e-5)
        xb = dev(np.stack([coords, coords]))
        xb.requires_grad_(True)
        g2 = layer(xb, dev(np.stack([tv, 0.5 * tv])), dev(np.stack([vr, vr])))
        close(g2.detach()[0], vref, "batched Coords2Grid forward " + tag, exact=binary)
        g2.backward(dev(np.stack([vdiff, vdiff])))
        close(xb.grad[0], ra, "batched Coords2Grid backward " + tag, rtol=1e-4, atol=5e-5)
        close(xb.grad[1], 0.5 * xb.grad[0].numpy(), "batched Coords2Grid backward, half weights, " + tag,
              rtol=1e-5, atol=1e-5)

    # ---- resampling: the three overloads of one grid, and a batch; Transform on device and on host --
    if dim <= 16 and T <= 8:
        q = synth.random_quaternions(rng, 1)[0]
        rc = rng.uniform(-1, 1, 3).astype(np.float32)
        tr = rng.uniform(-1.5, 1.5, 3).astype(np.float32)
        t = mg.Transform(mg.Quaternion(*q), tuple(rc), tuple(tr))
        out_res = float(rng.choice([res, res * 0.5, res * 1.5]))
        out_dim = int(rng.choice([dim, dim + 3, max(dim - 2, 1)]))
        gi = mg.GridInterpolater(res, dimension, out_res, (out_dim - 1) * out_res)
        src = ref if not binary else rng.standard_normal(ref.shape).astype(np.float32)
        dst = torch.full((T, out_dim, out_dim, out_dim), 9.0, device="cuda")
        gi.forward(as_input(rng, src), t, dst)
        one = oracle.interpolate_batch(res, dimension, out_res, (out_dim - 1) * out_res, rc[None], src[None],
                                       q[None], rc[None], tr[None], rc[None])[0]
        close(dst, one, "GridInterpolater.forward(in, transform, out) " + tag)
        ic, oc = rng.uniform(-1, 1, 3).astype(np.float32), rng.uniform(-1, 1, 3).astype(np.float32)
        gi.forward(tuple(ic), dev(src), t, tuple(oc), dst)
        close(dst, oracle.interpolate_batch(res, dimension, out_res, (out_dim - 1) * out_res, ic[None], src[None],
                                            q[None], rc[None], tr[None], oc[None])[0],
              "GridInterpolater.forward with centres " + tag)
        B = 3
        qs = synth.random_quaternions(rng, B)
        cs, ts = rng.uniform(-1, 1, (B, 3)).astype(np.float32), rng.uniform(-2, 2, (B, 3)).astype(np.float32)
        srcs = np.stack([src, src[:, ::-1].copy(), 2 * src]).astype(np.float32)
        dsts = torch.full((B, T, out_dim, out_dim, out_dim), 9.0, device="cuda")
        gi.forward_batch(dev(srcs), as_input(rng, qs), as_input(rng, cs), as_input(rng, ts), dsts)
        close(dsts, oracle.interpolate_batch(res, dimension, out_res, (out_dim - 1) * out_res, cs, srcs, qs, cs, ts, cs),
              "GridInterpolater.forward_batch " + tag)
        a, b = torch.empty((n, 3), device="cuda"), np.empty((n, 3), np.float32)
        t.forward(dev(coords), a)
        t.forward(coords, b)
        close(a, b, "Transform.forward on the device and on the host " + tag, exact=True)
        close(b, oracle.transform_forward(q, rc, tr, coords), "Transform.forward against the oracle " + tag, exact=True)
        t.backward(dev(b), a)
        t.backward(b.copy(), b)
        close(a, b, "Transform.backward on the device and on the host " + tag, exact=True)


def main():
    rounds = int(sys.argv[1]) if len(sys.argv) > 1 else 10
    seed = int(sys.argv[2]) if len(sys.argv) > 2 else 1
    first = int(sys.argv[3]) if len(sys.argv) > 3 else 0
    for r in range(first, first + rounds):
        print("round %d of seed %d:" % (r, seed), end=" ")
        one_round(np.random.default_rng([seed, r]))
    print("random python layer: %d rounds, %d comparisons passed" % (rounds, P.checked[0]))


if __name__ == "__main__":
    main()
