"""MI355X-native gridding hot path with libmolgrid's interface.

``GridMaker.forward/backward``, ``Transform.forward/backward`` and
``GridInterpolater.forward`` run as hand-written HIP kernels (gfx950) behind the
C ABI of ``include/molgrid_hip.h``; this package is the Python host side that
mirrors the reference's ``molgrid`` module for that path.
"""
from ._capi import LIB_PATH, lib as _lib  # noqa: F401  (fails loudly if the .so is missing)
from .gridding import (AtomBatch, CoordinateSet, Example, ExampleVec, GridInterpolater, GridMaker,  # noqa: F401
                       Quaternion, Transform, float3, set_random_seed, transform_batch)

from .grids import *  # noqa: F401,F403,E402  (Grid1f .. Grid8dCUDA, MGrid1f .. MGrid8d, tonumpy)
from .typers import *  # noqa: F401,F403,E402
from .providers import *  # noqa: F401,F403,E402
from .grid_io import *  # noqa: F401,F403,E402
from .torch_bindings import (BatchedCoords2GridFunction, Coords2Grid, Coords2GridFunction,  # noqa: F401,E402
                             Grid2CoordsGradientFunction, MolIterDataset, MolMapDataset,
                             make_grid_ndarray, make_grid_tensor, tensor_as_grid)

GridMaker.make_tensor = make_grid_tensor
GridMaker.make_ndarray = make_grid_ndarray

__version__ = "0.1.0"


def get_gpu_device():
    import torch
    return torch.cuda.current_device()


def set_gpu_device(index):
    import torch
    torch.cuda.set_device(int(index))
