"""Helpers shared by the GPU parity tests."""
import numpy as np

# tolerance of the comparison against the CPU oracle for float32 densities,
# atom gradients and interpolated values: |gpu - ref| <= ATOL + RTOL * |ref|
RTOL = 1e-5
ATOL = 1e-6


def assert_close(got, ref, rtol=RTOL, atol=ATOL, what=""):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    err = np.abs(got - ref)
    bound = atol + rtol * np.abs(ref)
    bad = err > bound
    if bad.any():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(
            "%s: %d of %d values outside %g + %g*|ref|; worst at %s: got %r ref %r (abs err %g)"
            % (what, int(bad.sum()), err.size, atol, rtol, i, got[i], ref[i], err[i]))


def dev(a, dtype=None):
    import torch
    t = torch.as_tensor(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def rot_matrix(q):
    """3x3 rotation matrix of a (possibly unnormalised) quaternion (a,b,c,d)."""
    a, b, c, d = [float(v) for v in q]
    n = a * a + b * b + c * c + d * d
    return np.array([
        [a * a + b * b - c * c - d * d, 2 * (b * c - a * d), 2 * (b * d + a * c)],
        [2 * (b * c + a * d), a * a - b * b + c * c - d * d, 2 * (c * d - a * b)],
        [2 * (b * d - a * c), 2 * (c * d + a * b), a * a - b * b - c * c + d * d]]) / n


def parity_stats(got, ref, rtol=RTOL, atol=ATOL):
    """Measured distance of `got` from `ref`: largest absolute error, largest relative error
    (over |ref| > 1e-3), and how many values lie outside atol + rtol*|ref|."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    err = np.abs(got - ref)
    big = np.abs(ref) > 1e-3
    return {
        "n": int(err.size),
        "max_abs": float(err.max()) if err.size else 0.0,
        "max_rel": float((err[big] / np.abs(ref[big])).max()) if big.any() else 0.0,
        "outside": int((err > atol + rtol * np.abs(ref)).sum()),
    }
