"""torch.autograd wrappers around GridMaker, with the names and call shapes of the reference's
python/torch_bindings.py:44-163 (``Coords2GridFunction``, ``BatchedCoords2GridFunction``,
``Grid2CoordsGradientFunction``, ``Coords2Grid``).

A batch is gridded (and back-propagated) with ONE kernel launch instead of the reference's Python
loop over examples.  ``Coords2GridFunction`` supports a second backward pass through
``GridMaker.backward_gradients``, like the reference; the batched function does not.
"""
import torch

from .gridding import GridMaker  # noqa: F401


class Grid2CoordsGradientFunction(torch.autograd.Function):
    """Grid gradient -> (coordinate gradient, type gradient)."""

    @staticmethod
    def forward(ctx, gmaker, center, coords, types, radii, grid_gradient):
        grid_gradient = grid_gradient.contiguous()
        ctx.save_for_backward(coords, types, radii, grid_gradient)
        ctx.gmaker, ctx.center = gmaker, center
        grad_coords = torch.empty_like(coords)
        grad_types = torch.empty_like(types)
        gmaker.backward(center, coords, types, radii, grid_gradient, grad_coords, grad_types)
        return grad_coords, grad_types

    @staticmethod
    def backward(ctx, grad_coords, grad_types):
        """Second-order pass (python/torch_bindings.py:59-72)."""
        coords, types, radii, grid_gradient = ctx.saved_tensors
        ddcoords = torch.empty_like(coords)
        ddtypes = torch.empty_like(types)
        ddG = torch.empty_like(grid_gradient)
        ctx.gmaker.backward_gradients(ctx.center, coords, types, radii, grid_gradient,
                                      grad_coords.contiguous(), grad_types.contiguous(), ddG,
                                      ddcoords, ddtypes)
        return None, None, ddcoords, ddtypes, None, ddG


class Coords2GridFunction(torch.autograd.Function):
    """coords (N,3), type vectors (N,T), radii (N) -> grid (T,D,D,D)."""

    @staticmethod
    def forward(ctx, gmaker, center, coords, types, radii):
        if types.dim() != 2:
            raise ValueError("Vector types required in Coords2Grid.")
        ctx.save_for_backward(coords, types, radii)
        ctx.gmaker, ctx.center = gmaker, center
        out = torch.empty(gmaker.grid_dimensions(types.shape[1]), dtype=coords.dtype,
                          device=coords.device)
        gmaker.forward(center, coords, types, radii, out)
        return out

    @staticmethod
    def backward(ctx, grid_gradient):
        coords, types, radii = ctx.saved_tensors
        grad_coords, grad_types = Grid2CoordsGradientFunction.apply(
            ctx.gmaker, ctx.center, coords, types, radii, grid_gradient)
        return None, None, grad_coords, grad_types, None


class BatchedCoords2GridFunction(torch.autograd.Function):
    """coords (B,N,3), type vectors (B,N,T), radii (B,N) -> grids (B,T,D,D,D), one launch."""

    @staticmethod
    def forward(ctx, gmaker, center, coords, types, radii):
        if coords.shape[0] != types.shape[0] or coords.shape[0] != radii.shape[0]:
            raise RuntimeError("Inconsistent batch sizes in Coords2Grid inputs")
        if types.dim() != 3:
            raise ValueError("Vector types required in BatchedCoords2Grid.")
        ctx.save_for_backward(coords, types, radii)
        ctx.gmaker, ctx.center = gmaker, center
        out = torch.empty((coords.shape[0],) + gmaker.grid_dimensions(types.shape[2]),
                          dtype=coords.dtype, device=coords.device)
        gmaker.forward(center, coords, types, radii, out)
        return out

    @staticmethod
    def backward(ctx, grid_gradient):
        coords, types, radii = ctx.saved_tensors
        grad_coords = torch.empty_like(coords)
        grad_types = torch.empty_like(types)
        ctx.gmaker.backward(ctx.center, coords, types, radii, grid_gradient.contiguous(),
                            grad_coords, grad_types)
        return None, None, grad_coords, grad_types, None


class Coords2Grid(torch.nn.Module):
    """Layer turning coordinates / type vectors / radii into a grid with a fixed GridMaker and
    grid centre; accepts one example or a padded batch."""

    def __init__(self, gmaker, center=(0, 0, 0)):
        super().__init__()
        self.gmaker = gmaker
        self.center = center

    def forward(self, coords, types, radii):
        coords, types, radii = coords.contiguous(), types.contiguous(), radii.contiguous()
        if coords.dim() == 3 and types.dim() == 3 and radii.dim() == 2:
            return BatchedCoords2GridFunction.apply(self.gmaker, self.center, coords, types, radii)
        if coords.dim() == 2 and types.dim() == 2 and radii.dim() == 1:
            return Coords2GridFunction.apply(self.gmaker, self.center, coords, types, radii)
        raise RuntimeError("Invalid input dimensions in forward of Coords2Grid")

    def extra_repr(self):
        return "resolution {:.2f}, dimension {}, center {:.3f},{:.3f},{:.3f}".format(
            self.gmaker.get_resolution(), self.gmaker.get_dimension(), *self.center)


# --------------------------------------------------------------------------------------------
# datasets over example lists (python/torch_bindings.py:165-372)
# --------------------------------------------------------------------------------------------
def _example_tensors(ex, random_translation, random_rotation):
    """(atom count, centre, coords, types, radii, labels) of one example as CPU tensors; the
    centre is that of the last coordinate set, which is also the centre of the random transform."""
    from . import gridding as _gr
    center = torch.tensor(list(ex.coord_sets[-1].center()))
    merged = ex.merge_coordinates()
    if random_translation > 0 or random_rotation:
        _gr.Transform(ex.coord_sets[-1].center(), random_translation, random_rotation).forward(
            merged, merged)
    if merged.has_vector_types() and merged.size() > 0:
        types = torch.tensor(merged.type_vector.tonumpy(), dtype=torch.long).float()
    else:
        types = torch.tensor(merged.type_index.tonumpy(), dtype=torch.long).float()
    coords = torch.tensor(merged.coords.tonumpy())
    return (len(coords), center, coords, types, torch.tensor(merged.radii.tonumpy()),
            torch.tensor(ex.labels))


def _padded(parts):
    lengths, centers, coords, types, radii, labels = zip(*parts)
    pad = torch.nn.utils.rnn.pad_sequence
    return (torch.tensor(lengths), torch.stack(centers, dim=0), pad(coords, batch_first=True),
            pad(types, batch_first=True), pad(radii, batch_first=True), torch.stack(labels, dim=0))


class _ListDatasetState(object):
    """Construction and pickling shared by the two datasets: keyword settings, optional typers,
    the example list files."""
    _source = None

    def _open(self, files, random_translation, random_rotation, kwargs):
        self._random_translation, self._random_rotation = random_translation, random_rotation
        self.typers = kwargs.pop("typers", None)
        self.examples = self._source(*(self.typers or ()), **kwargs)
        self.types_files = list(files)
        self.examples.populate(self.types_files)

    def __getstate__(self):
        from .providers import _SETTINGS
        if self.typers is not None:
            raise NotImplementedError("%s does not support pickling when not using the default "
                                      "gnina atom typers" % type(self).__name__)
        settings = self.examples.settings()
        state = {name: getattr(settings, name) for name, _ in _SETTINGS}
        state["random_translation"] = self._random_translation
        state["random_rotation"] = self._random_rotation
        return state, self.types_files

    def __setstate__(self, state):
        kwargs = dict(state[0])
        rt, rr = kwargs.pop("random_translation"), kwargs.pop("random_rotation")
        self._open(state[1], rt, rr, kwargs)


class MolMapDataset(_ListDatasetState, torch.utils.data.Dataset):
    """Map-style dataset over example lists: item i is (atom count, centre, coords, types, radii,
    labels) of example i; ``collateMolDataset`` pads a batch to its longest example."""

    def __init__(self, *args, random_translation=0.0, random_rotation=False, **kwargs):
        from .providers import ExampleDataset
        self._source = ExampleDataset
        self._open(args, random_translation, random_rotation, kwargs)

    def __setstate__(self, state):
        from .providers import ExampleDataset
        self._source = ExampleDataset
        super().__setstate__(state)

    def __len__(self):
        return len(self.examples)

    def __getitem__(self, idx):
        return _example_tensors(self.examples[idx], self._random_translation,
                                self._random_rotation)

    @staticmethod
    def collateMolDataset(batch):
        return _padded(batch)


class MolIterDataset(_ListDatasetState, torch.utils.data.IterableDataset):
    """Iterable dataset: every item is a padded batch of ``default_batch_size`` examples in the
    provider's order; workers and ranks take every n-th batch.  Use DataLoader(batch_size=None)."""

    def __init__(self, *args, random_translation=0.0, random_rotation=False, **kwargs):
        from .providers import ExampleProvider
        self._source = ExampleProvider
        self._open(args, random_translation, random_rotation, kwargs)
        self._num_labels = self.examples.num_labels()

    def __setstate__(self, state):
        from .providers import ExampleProvider
        self._source = ExampleProvider
        super().__setstate__(state)
        self._num_labels = self.examples.num_labels()

    def example_to_tensor(self, ex):
        return _example_tensors(ex, self._random_translation, self._random_rotation)

    def batch_to_tensors(self, batch):
        return _padded([self.example_to_tensor(ex) for ex in batch])

    def generate(self):
        for batch in self.examples:
            yield self.batch_to_tensors(batch)

    def __iter__(self):
        from itertools import islice
        info = torch.utils.data.get_worker_info()
        worker, workers = (info.id, info.num_workers) if info is not None else (0, 1)
        dist = torch.distributed
        if dist.is_available() and dist.is_initialized() and dist.get_world_size() > 1:
            return islice(self.generate(), dist.get_rank() * workers + worker, None,
                          workers * dist.get_world_size())
        return islice(self.generate(), worker, None, workers)

    def __len__(self):
        from .providers import IterationScheme
        settings = self.examples.settings()
        batch = int(settings.default_batch_size)
        if settings.iteration_scheme == IterationScheme.SmallEpoch:
            return self.examples.small_epoch_size() // batch
        if settings.iteration_scheme == IterationScheme.LargeEpoch:
            return -(-self.examples.large_epoch_size() // batch)
        raise NotImplementedError("a continuous iteration has no length")


def make_grid_tensor(gridmaker, center, c):
    """A device tensor of the right size holding the densities of coordinate set c."""
    t = torch.zeros(gridmaker.grid_dimensions(c.max_type), dtype=torch.float32, device="cuda")
    gridmaker.forward(center, c, t)
    return t


def make_grid_ndarray(gridmaker, center, c):
    """A numpy array of the right size holding the densities of coordinate set c."""
    import numpy as np
    a = np.zeros(gridmaker.grid_dimensions(c.max_type), dtype=np.float32)
    gridmaker.forward(center, c, a)
    return a


def tensor_as_grid(t):
    """Grid view of tensor t (python/torch_bindings.py:9-29)."""
    from . import grids
    if t.dtype not in (torch.float32, torch.float64):
        raise ValueError("Tensor base type %s not supported as grid type." % str(t.dtype))
    name = "Grid%d%s%s" % (t.dim(), "f" if t.dtype == torch.float32 else "d",
                           "CUDA" if t.is_cuda else "")
    return getattr(grids, name)(t)
