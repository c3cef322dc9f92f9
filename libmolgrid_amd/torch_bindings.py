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
