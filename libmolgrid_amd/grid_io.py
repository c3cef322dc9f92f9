"""Reading and writing density grids as OpenDX files and AutoDock maps, byte for byte in the
reference's formats (src/grid_io.cpp, include/libmolgrid/cartesian_grid.h)."""
import numpy as np

from . import gridding as _g
from . import grids as _grids


def _host(grid, ndim):
    """numpy copy of a grid / managed grid / tensor / array with `ndim` dimensions."""
    g = _g._unwrap(grid)
    a = g.detach().cpu().numpy() if hasattr(g, "detach") else np.asarray(g)
    if a.ndim != ndim:
        raise ValueError("expected a %d-dimensional grid, got %d dimensions" % (ndim, a.ndim))
    return a


class CartesianGrid(object):
    """A cubic grid with its centre and resolution (include/libmolgrid/cartesian_grid.h)."""

    def __init__(self, grid, center, resolution):
        self._grid, self._center, self._resolution = grid, _g._to_float3(center), float(resolution)
        dims = tuple(grid.shape)[-3:]
        c = self._center
        self._origin = _g.float3(c.x - dims[0] * self._resolution / 2.0,
                                 c.y - dims[1] * self._resolution / 2.0,
                                 c.z - dims[2] * self._resolution / 2.0)

    def center(self):
        return self._center

    def resolution(self):
        return self._resolution

    def grid(self):
        return self._grid

    def cart2grid(self, x, y, z):
        o, r = self._origin, self._resolution
        return _g.float3((x - o.x) / r, (y - o.y) / r, (z - o.z) / r)

    def grid2cart(self, i, j, k):
        o, r = self._origin, self._resolution
        return _g.float3(o.x + i * r, o.y + j * r, o.z + k * r)


CartesianMGrid = CartesianGrid


def _dx_text(a, center, resolution, scale):
    n = a.shape[0]
    c = _g._to_float3(center)
    res = float(np.float32(resolution))
    half = res * (n - 1) / 2.0
    head = ["object 1 class gridpositions counts %d %d  %d" % (n, n, n),
            "origin %.5f %.5f %.5f" % (c.x - half, c.y - half, c.z - half),
            "delta %.5f 0 0" % res, "delta 0 %.5f 0" % res, "delta 0 0 %.5f" % res,
            "object 2 class gridconnections counts %d %d  %d" % (n, n, n),
            "object 3 class array type double rank 0 items [ %d] data follows" % (n * n * n)]
    vals = ["%.5f" % v for v in (a.reshape(-1).astype(a.dtype) * a.dtype.type(scale)).tolist()]
    body = []
    for i in range(0, len(vals), 3):
        chunk = vals[i:i + 3]
        body.append(" ".join(chunk) + ("\n" if len(chunk) == 3 else " "))
    return "\n".join(head) + "\n" + "".join(body)


def write_dx(file_name, grid, center, resolution, scale=1.0):
    """One cubic grid as an OpenDX file: fixed notation with five decimals, three values a line."""
    a = _host(grid, 3)
    try:
        f = open(file_name, "w")
    except OSError:
        raise ValueError("Could not open file " + file_name)
    with f:
        f.write(_dx_text(a, center, resolution, scale))


def _read_dx(file_name):
    try:
        f = open(file_name)
    except OSError:
        raise ValueError("Could not read file " + file_name)
    with f:
        tok = f.readline().split()
        if len(tok) != 8:
            raise ValueError("Could not read dx file: tokens != 8")
        n = int(tok[7])
        if int(tok[6]) != n or int(tok[5]) != n:
            raise ValueError("Could not read dx file: grid is not cubic")
        tok = f.readline().split()
        if len(tok) != 4:
            raise ValueError("Could not read dx file: tokens != 4")
        x, y, z = float(tok[1]), float(tok[2]), float(tok[3])
        res = None
        for axis in range(3):
            tok = f.readline().split()
            if len(tok) != 4:
                raise ValueError("Could not read dx file: tokens != 4 (%d)" % (axis + 2))
            r = float(np.float32(tok[1 + axis]))
            if res is not None and r != res:
                raise ValueError("Could not read dx file: mismatch")
            res = r
        f.readline()   # grid connections
        f.readline()   # object 3
        data = np.array(f.read().split(), dtype=np.float64)
    if data.size != n * n * n:
        raise ValueError("Could not read dx file: incorrect number of data points (%d vs %d"
                         % (data.size, n * n * n))
    half = res * (n - 1) / 2.0
    return data.reshape(n, n, n), _g.float3(x + half, y + half, z + half), res


def read_dx(file_name, grid=None):
    """read_dx(file_name) -> CartesianGrid holding an MGrid3f; read_dx(file_name, grid) fills a
    grid of the right size."""
    data, center, res = _read_dx(file_name)
    if grid is None:
        m = _grids.MGrid3f(*data.shape)
        m.copyFrom(data.astype(np.float32))
        return CartesianGrid(m, center, res)
    g = _g._unwrap(grid)
    if tuple(g.shape) != data.shape:
        raise ValueError("Grid incorrect size in read_dx: %d != %d" % (data.shape[0], tuple(g.shape)[0]))
    if hasattr(g, "copy_"):
        import torch
        g.copy_(torch.from_numpy(data).to(g.dtype))
    else:
        g[...] = data


def _dx_name(prefix, name):
    fname = "%s_%s.dx" % (prefix, name)
    if len(fname) > 255:
        fname = fname[:250] + ".dx"
    return fname


def write_dx_grids(prefix, type_names, grid, center, resolution, scale=1.0):
    """One file ``<prefix>_<name>.dx`` per channel."""
    a = _host(grid, 4)
    if len(type_names) != a.shape[0]:
        raise ValueError("Number of names and number of grids doesn't match in write_dx_grids: "
                         "%d != %d" % (len(type_names), a.shape[0]))
    for name, channel in zip(type_names, a):
        write_dx(_dx_name(prefix, name), channel, center, resolution, scale)


def read_dx_grids(prefix, type_names, grid):
    g = _g._unwrap(grid)
    if len(type_names) != tuple(g.shape)[0]:
        raise ValueError("Number of names and number of grids doesn't match in read_dx_grids: "
                         "%d != %d" % (len(type_names), tuple(g.shape)[0]))
    for i, name in enumerate(type_names):
        read_dx("%s_%s.dx" % (prefix, name), g[i])


def write_map(file_name, grid, center, resolution, scale=1.0):
    """AutoDock map: x runs fastest, values with five significant digits."""
    a = _host(grid, 3)
    c = _g._to_float3(center)
    n = a.shape[0]
    try:
        f = open(file_name, "w")
    except OSError:
        raise ValueError("Could not open file " + file_name)
    with f:
        f.write("GRID_PARAMETER_FILE\nGRID_DATA_FILE\nMACROMOLECULE\n")
        f.write("SPACING %.5g\n" % float(np.float32(resolution)))
        f.write("NELEMENTS %d %d %d\n" % (n - 1, n - 1, n - 1))
        f.write("CENTER %.5g %.5g %.5g\n" % (c.x, c.y, c.z))
        vals = (a.transpose(2, 1, 0).reshape(-1) * a.dtype.type(scale)).tolist()
        f.write("".join("%.5g\n" % v for v in vals))


__all__ = ["CartesianGrid", "CartesianMGrid", "write_dx", "read_dx", "write_dx_grids",
           "read_dx_grids", "write_map"]
