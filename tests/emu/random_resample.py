"""TEST INFRASTRUCTURE: randomised parity of the resampling kernels (mg_interpolate) under the HIP
emulation against the oracle: input and output grids of 1 to 50 voxels a side at resolution ratios
from 0.4 to 2.5 (the staged kernel, its gather path and the down-sampling kernel), 1 to 9 channels,
batches of 1 to 10 examples (more than one XCD's worth of example slots), separate input, output
and rotation centres, shifts from nothing to several grid widths (outputs that fall partly or
wholly outside the input and must read zeros), identity and axis-aligned rotations next to random
ones, integral source coordinates (weights of exactly zero).  1e-6 + 1e-5 |ref| everywhere, and
the gather path equal to the staged one bit for bit.
``python tests/emu/random_resample.py [rounds] [seed] [first round]``."""
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


def resample(in_res, in_a, out_res, out_a, in_c, grids, quats, rot_c, shifts, out_c):
    B, K = grids.shape[:2]
    od = int(round(out_a / out_res)) + 1
    out = E.array((B, K, od, od, od), fill=9.0)
    z3, q1 = E.f3((0, 0, 0)), E.f4((1, 0, 0, 0))
    code = lib.mg_interpolate(in_res, in_a, out_res, out_a, B, K, E.ptr(E.put(in_c)), z3,
                              E.ptr(E.put(grids)), E.ptr(E.put(quats)), q1, E.ptr(E.put(rot_c)), z3,
                              E.ptr(E.put(shifts)), z3, E.ptr(E.put(out_c)), z3, E.ptr(out), None)
    assert code == 0, code
    return out


def one_round(rng):
    in_dim = int(rng.choice([1, 2, 3, 5, 8, 12, 16, 17, 24, 31, 32, 33, 48, 50]))
    in_res = float(rng.choice([0.25, 0.5, 0.75, 1.0]))
    ratio = float(rng.choice([1.0, 1.0, 1.0, 0.4, 0.5, 0.8, 0.97, 1.03, 1.25, 2.0, 2.5]))
    out_res = in_res * ratio
    out_dim = int(rng.choice([1, 2, 4, 7, 8, 15, 16, 17, 24, 33, 48, 50]))
    if in_dim * out_dim > 1200:
        out_dim = min(out_dim, 24)
    K = int(rng.choice([1, 2, 3, 9]))
    B = int(rng.choice([1, 2, 3, 10])) if max(in_dim, out_dim) <= 24 else int(rng.choice([1, 2]))
    in_a, out_a = (in_dim - 1) * in_res, (out_dim - 1) * out_res
    grids = rng.standard_normal((B, K, in_dim, in_dim, in_dim)).astype(np.float32)
    kind = rng.integers(0, 4)
    quats = synth.random_quaternions(rng, B)
    s = np.float32(np.sqrt(0.5))
    if kind == 0:
        quats[:] = (1, 0, 0, 0)
    elif kind == 1:
        quats[:] = [(s, s, 0, 0), (s, 0, s, 0), (s, 0, 0, s), (0, 1, 0, 0)][int(rng.integers(0, 4))]
    in_c = (rng.uniform(-3, 3, (B, 3)) * rng.choice([0, 1])).astype(np.float32)
    out_c = in_c.copy() if rng.random() < 0.5 else (in_c + rng.uniform(-2, 2, (B, 3))).astype(np.float32)
    rot_c = (rng.uniform(-3, 3, (B, 3)) * rng.choice([0, 1])).astype(np.float32)
    span = float(rng.choice([0.0, 0.0, 1.5, in_a + 1.0, 3 * in_a + 5.0]))
    shifts = rng.uniform(-span - 1e-6, span + 1e-6, (B, 3)).astype(np.float32)
    if rng.random() < 0.3:                         # whole voxels: source coordinates on the lattice
        shifts = (np.round(shifts / in_res) * in_res).astype(np.float32)
    tag = "in %d @ %g -> out %d @ %g, K %d B %d rotation kind %d shift up to %g" % (
        in_dim, in_res, out_dim, out_res, K, B, kind, span)
    print("resample:", tag, flush=True)
    ref = oracle.interpolate_batch(in_res, in_a, out_res, out_a, in_c, grids, quats, rot_c, shifts, out_c)
    got = np.array(resample(in_res, in_a, out_res, out_a, in_c, grids, quats, rot_c, shifts, out_c))
    C.close(got, ref, tag)
    lib.mg_interpolate_force_gather(1)
    gathered = resample(in_res, in_a, out_res, out_a, in_c, grids, quats, rot_c, shifts, out_c)
    lib.mg_interpolate_force_gather(0)
    C.close(gathered, got, "gather path equals staged path, " + tag, exact=not os.environ.get("EMU_CONTRACT"))


def main():
    rounds = int(sys.argv[1]) if len(sys.argv) > 1 else 10
    seed = int(sys.argv[2]) if len(sys.argv) > 2 else 1
    first = int(sys.argv[3]) if len(sys.argv) > 3 else 0
    lib.mg_interpolate_force_gather.argtypes = [ctypes.c_int]
    for r in range(first, first + rounds):
        print("round %d of seed %d:" % (r, seed), end=" ")
        # (the arrays of this round start 0 to 12 bytes past a 16-byte boundary)
        E.MISALIGN = int(np.random.default_rng([seed, r, 1]).choice([0, 0, 1, 2, 3]))
        one_round(np.random.default_rng([seed, r]))
        E.release_all()
    print("random resampling: %d rounds passed" % rounds)


if __name__ == "__main__":
    main()
