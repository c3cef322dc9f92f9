"""TEST INFRASTRUCTURE: the Python host layer (GridMaker / Transform / GridInterpolater /
Coords2Grid of libmolgrid_amd) on the fake device of fake_cuda.py, against the emulated kernels and
the oracle.  Exercises the argument plumbing of the host layer -- workspaces, overloads, the sort
and splat halves, autograd -- without a GPU.  Run as ``python tests/emu/python_layer.py``."""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, HERE)

import fake_cuda  # noqa: E402

fake_cuda.activate()

import libmolgrid_amd as mg  # noqa: E402
import oracle  # noqa: E402
import synth  # noqa: E402

RTOL, ATOL = 1e-5, 1e-6
checked = [0]


def dev(a):
    return fake_cuda.on_device(torch.as_tensor(np.ascontiguousarray(a)))


def close(got, ref, what, exact=False, rtol=RTOL, atol=ATOL):
    checked[0] += 1
    got = got.numpy() if isinstance(got, torch.Tensor) else np.asarray(got)
    ok = np.array_equal(got, ref) if exact else bool(np.all(np.abs(got - ref) <= atol + rtol * np.abs(ref)))
    assert ok, "%s: max abs difference %g" % (what, float(np.abs(got - ref).max()))


def main():
    rng = np.random.default_rng(7)
    # ---- one example, index types: device tensors, host arrays, float64 grid --------------------
    coords, types, radii = synth.small_index_case(rng, 60, 4, 7.0)
    gm, og = mg.GridMaker(0.5, 11.5), oracle.GridMaker(0.5, 11.5)
    ref = og.forward((0.1, 0, 0), coords, types, radii, 4)
    out = torch.full(gm.grid_dimensions(4), 7.0, device="cuda")
    gm.forward((0.1, 0, 0), dev(coords), dev(types), dev(radii), out)
    close(out, ref, "forward, device tensors")
    host = np.full(ref.shape, 7.0, np.float32)
    gm.forward((0.1, 0, 0), coords, types, radii, host)
    close(host, ref, "forward, host arrays")
    wide = torch.full(gm.grid_dimensions(4), 7.0, device="cuda", dtype=torch.float64)
    gm.forward((0.1, 0, 0), dev(coords), dev(types), dev(radii), wide)
    close(wide, out.numpy().astype(np.float64), "forward, float64 grid", exact=True)
    # ---- ragged batch: forward_batch, sort_batch + splat_batch, AtomBatch workspace reuse ---------
    cfg = synth.index_batch(2, 4, (30, 100), (3, 9), ntypes=6)
    refb = og.forward_batch(cfg["offsets"], cfg["centers"], cfg["coords"], cfg["types"], cfg["radii"], 6)
    batch = mg.AtomBatch(cfg["offsets"])
    c, t, r, cen = dev(cfg["coords"]), dev(cfg["types"]), dev(cfg["radii"]), dev(cfg["centers"])
    grid = torch.full((4,) + gm.grid_dimensions(6), 7.0, device="cuda")
    for _ in range(2):                                   # the second call reuses the workspace
        gm.forward_batch(batch, cen, c, t, r, grid)
        close(grid, refb, "forward_batch")
    split = torch.full_like(grid, 7.0)
    sb = gm.sort_batch(batch, cen, c, t, r, 6)
    gm.splat_batch(sb, split)
    close(split, grid.numpy(), "sort_batch + splat_batch", exact=True)
    try:
        gm.splat_batch(sb, torch.empty((3,) + gm.grid_dimensions(6), device="cuda"))
        raise AssertionError("a grid of another batch size was accepted")
    except ValueError:
        checked[0] += 1
    # ---- backward, index types, with the fused un-rotation ---------------------------------------
    diff = rng.standard_normal(refb.shape).astype(np.float32)
    rg = og.backward_batch(cfg["offsets"], cfg["centers"], cfg["coords"], cfg["types"], cfg["radii"], diff)
    grads = torch.full((len(cfg["coords"]), 3), 9.0, device="cuda")
    gm.backward_batch(batch, cen, c, t, r, dev(diff), grads)
    close(grads, rg, "backward_batch", rtol=1e-4, atol=2e-5)
    un = torch.full_like(grads, 9.0)
    q = dev(cfg["quats"])
    gm.backward_batch(batch, cen, c, t, r, dev(diff), un, unrotate=(q, cen))
    want = oracle.transform_backward_batch(cfg["offsets"], cfg["quats"], cfg["centers"],
                                           np.zeros_like(cfg["centers"]), grads.numpy(), dotranslate=False)
    close(un, want, "backward_batch with un-rotation", exact=True)
    # ---- transform on device tensors (kernel) and on host arrays (host path): the same floats ------
    moved = torch.empty_like(c)
    mg.transform_batch(batch, q, cen, dev(cfg["translations"]), c, moved)
    close(moved, oracle.transform_forward_batch(cfg["offsets"], cfg["quats"], cfg["centers"],
                                                cfg["translations"], cfg["coords"]), "transform_batch", exact=True)
    T = mg.Transform(mg.Quaternion(*cfg["quats"][0]), (0.5, 0, -1), (1, 2, 3))
    a = torch.empty((50, 3), device="cuda")
    T.forward(dev(cfg["coords"][:50]), a)
    b = np.empty((50, 3), np.float32)
    T.forward(cfg["coords"][:50], b)
    close(a, b, "Transform.forward: kernel and host path", exact=True)
    # ---- vector types: single, padded batch, ragged batch (atom lists), backward --------------------
    n, K = 50, 5
    vc = rng.uniform(-6, 6, (n, 3)).astype(np.float32)
    tv = (rng.dirichlet(np.full(K, 0.3), n) * (rng.random((n, K)) > 0.4)).astype(np.float32)
    vr = rng.uniform(0.8, 2.0, n).astype(np.float32)
    vref = og.forward((0, 0, 0), vc, tv, vr)
    vout = torch.full(gm.grid_dimensions(K), 3.0, device="cuda")
    gm.forward((0, 0, 0), dev(vc), dev(tv), dev(vr), vout)
    close(vout, vref, "vector forward")
    pad = torch.full((2,) + gm.grid_dimensions(K), 3.0, device="cuda")
    gm.forward(dev(np.zeros((2, 3), np.float32)), dev(np.stack([vc, vc])), dev(np.stack([tv, tv])),
               dev(np.stack([vr, vr])), pad)
    close(pad[1], vout.numpy(), "vector forward, padded batch", exact=True)
    vb = mg.AtomBatch(np.array([0, 20, 20, 50]))
    rag = torch.full((3,) + gm.grid_dimensions(K), 3.0, device="cuda")
    gm.forward_batch(vb, dev(np.zeros((3, 3), np.float32)), dev(vc), dev(tv), dev(vr), rag)
    close(rag, og.forward_batch(np.array([0, 20, 20, 50]), np.zeros((3, 3), np.float32), vc, tv, vr, K),
          "vector forward_batch")
    vdiff = rng.standard_normal(vref.shape).astype(np.float32)
    ra, rt = og.backward((0, 0, 0), vc, tv, vr, vdiff)
    ag, tg = torch.full((n, 3), 9.0, device="cuda"), torch.full((n, K), 9.0, device="cuda")
    gm.backward((0, 0, 0), dev(vc), dev(tv), dev(vr), dev(vdiff), ag, tg)
    close(ag, ra, "vector backward, atoms", rtol=1e-4, atol=3e-5)
    close(tg, rt, "vector backward, types", rtol=1e-4, atol=3e-5)
    # ---- the autograd layer: one example and a padded batch --------------------------------------
    from libmolgrid_amd.torch_bindings import Coords2Grid
    layer = Coords2Grid(gm)
    x = dev(vc)
    x.requires_grad_(True)
    g1 = layer(x, dev(tv), dev(vr))
    close(g1.detach(), vref, "Coords2Grid forward")
    g1.backward(dev(vdiff))
    close(x.grad, ra, "Coords2Grid backward", rtol=1e-4, atol=3e-5)
    xb = dev(np.stack([vc, vc]))
    xb.requires_grad_(True)
    g2 = layer(xb, dev(np.stack([tv, tv])), dev(np.stack([vr, vr])))
    g2.backward(dev(np.stack([vdiff, 2 * vdiff])))
    close(xb.grad[0], ra, "batched Coords2Grid backward", rtol=1e-4, atol=3e-5)
    close(xb.grad[1], 2 * xb.grad[0].numpy(), "batched Coords2Grid backward is linear", rtol=1e-5, atol=1e-5)
    # ---- resampling ----------------------------------------------------------------------------------
    gi = mg.GridInterpolater(0.5, 11.5, 0.5, 11.5)
    src = rng.standard_normal((2, 3, 24, 24, 24)).astype(np.float32)
    qs = synth.random_quaternions(rng, 2)
    sh = rng.uniform(-1.5, 1.5, (2, 3)).astype(np.float32)
    z3 = np.zeros((2, 3), np.float32)
    dst = torch.full((2, 3, 24, 24, 24), 9.0, device="cuda")
    gi.forward_batch(dev(src), dev(qs), dev(z3), dev(sh), dst)
    close(dst, oracle.interpolate_batch(0.5, 11.5, 0.5, 11.5, z3, src, qs, z3, sh, z3), "interpolate batch")
    print("python layer on the fake device: %d comparisons passed" % checked[0])


if __name__ == "__main__":
    main()
