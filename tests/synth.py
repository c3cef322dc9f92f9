"""Seeded synthetic workloads shaped like the benchmark configurations.

Coordinates are uniform in a cube with a minimum pairwise separation enforced by
rejection, index types are uniform over the receptor/ligand channel halves, and
radii come from a seeded per-type table, as the configuration text prescribes.
"""
import numpy as np
from scipy.spatial import cKDTree

SEED = 0xC0FFEE


def sample_coords(rng, n, half=13.0, min_sep=0.9):
    """n points uniform in [-half, half]^3 with pairwise distance >= min_sep (rejection)."""
    pts = np.empty((0, 3), np.float64)
    while len(pts) < n:
        need = n - len(pts)
        cand = rng.uniform(-half, half, (int(need * 1.5) + 16, 3))
        allp = np.vstack([pts, cand])
        pairs = cKDTree(allp).query_pairs(min_sep, output_type="ndarray")
        bad = np.zeros(len(allp), bool)
        if len(pairs):
            pairs = pairs[np.argsort(pairs.max(axis=1), kind="stable")]
            for i, j in pairs:
                lo, hi = (i, j) if i < j else (j, i)
                if hi >= len(pts) and not bad[lo]:
                    bad[hi] = True
        keep = cand[~bad[len(pts):]]
        pts = np.vstack([pts, keep[:need]])
    return pts.astype(np.float32)


def random_quaternions(rng, n):
    q = rng.normal(size=(n, 4))
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    return q.astype(np.float32)


def radius_table(rng, ntypes=28):
    return rng.uniform(1.2, 2.0, ntypes).astype(np.float32)


def index_batch(config_id, nbatch, nrec_range, nlig_range, ntypes=28, rot=True, trans=2.0,
                seed=SEED):
    """Packed ragged batch of index-typed complexes (configurations 0-2)."""
    rng = np.random.default_rng(seed + config_id)
    table = radius_table(rng, ntypes)
    half = ntypes // 2
    coords, types, offsets = [], [], [0]
    for b in range(nbatch):
        erng = np.random.default_rng(seed + config_id + 1000 * (b + 1))
        nrec = int(erng.integers(nrec_range[0], nrec_range[1] + 1))
        nlig = int(erng.integers(nlig_range[0], nlig_range[1] + 1))
        c = sample_coords(erng, nrec + nlig)
        t = np.concatenate([erng.integers(0, half, nrec), erng.integers(half, ntypes, nlig)])
        coords.append(c)
        types.append(t.astype(np.float32))
        offsets.append(offsets[-1] + nrec + nlig)
    coords = np.concatenate(coords)
    types = np.concatenate(types)
    radii = table[types.astype(np.int64)]
    out = dict(offsets=np.asarray(offsets, np.int64), coords=coords, types=types, radii=radii,
               ntypes=ntypes, centers=np.zeros((nbatch, 3), np.float32))
    if rot:
        out["quats"] = random_quaternions(rng, nbatch)
    else:
        out["quats"] = np.tile(np.asarray([[1, 0, 0, 0]], np.float32), (nbatch, 1))
    out["translations"] = rng.uniform(-trans, trans, (nbatch, 3)).astype(np.float32) if trans \
        else np.zeros((nbatch, 3), np.float32)
    return out


def config0(seed=SEED):
    return index_batch(0, 1, (1500, 1500), (40, 40), rot=False, trans=0.0, seed=seed)


def config1(nbatch=50, seed=SEED):
    return index_batch(1, nbatch, (1000, 4000), (15, 80), seed=seed)


def vector_batch(nbatch=16, natoms=10000, ntypes=28, seed=SEED):
    """Configuration 3: soft-typed atoms, Dirichlet(0.3) type vectors scaled by U[0.5,1.5]."""
    rng = np.random.default_rng(seed + 3)
    coords, offsets = [], [0]
    for b in range(nbatch):
        erng = np.random.default_rng(seed + 3 + 1000 * (b + 1))
        coords.append(sample_coords(erng, natoms))
        offsets.append(offsets[-1] + natoms)
    n = offsets[-1]
    tv = rng.dirichlet(np.full(ntypes, 0.3), n) * rng.uniform(0.5, 1.5, (n, 1))
    return dict(offsets=np.asarray(offsets, np.int64), coords=np.concatenate(coords),
                types=tv.astype(np.float32), radii=rng.uniform(1.2, 2.0, n).astype(np.float32),
                ntypes=ntypes, centers=np.zeros((nbatch, 3), np.float32))


def small_index_case(rng, natoms, ntypes, extent, rmin=0.8, rmax=2.0, frac_ignored=0.1):
    """A small random molecule for exhaustive comparisons."""
    coords = rng.uniform(-extent, extent, (natoms, 3)).astype(np.float32)
    types = rng.integers(0, ntypes, natoms).astype(np.float32)
    types[rng.random(natoms) < frac_ignored] = -1.0
    radii = rng.uniform(rmin, rmax, natoms).astype(np.float32)
    return coords, types, radii
