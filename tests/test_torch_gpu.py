"""Autograd layer (Coords2Grid) on the GPU: the constants of the reference's test/test_torch.py."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mg():
    import libmolgrid_amd
    return libmolgrid_amd


def test_function(mg):
    """test/test_torch.py:128-148."""
    from libmolgrid_amd.torch_bindings import Coords2GridFunction
    for dev in ("cuda", "cpu"):
        gmaker = mg.GridMaker(resolution=.1, dimension=6.0)
        c = torch.tensor([[1.0, 0, 0], [1, 0, 0]], device=dev, requires_grad=True)
        vt = torch.tensor([[0, 1.0, 0], [1.0, 0, 0]], device=dev, requires_grad=True)
        r = torch.tensor([2.0, 2.0], device=dev)
        grid = Coords2GridFunction.apply(gmaker, (0, 0, 0), c, vt, r)
        diff = torch.zeros(gmaker.grid_dimensions(3), device=dev)
        diff[0, 30, 30, 30] = 1.0
        diff[1, 30, 30, 30] = -1.0
        grid.backward(diff)
        assert c.grad[0].cpu().numpy() == pytest.approx([0.60653, 0, 0], abs=1e-4)
        assert c.grad[1].cpu().numpy() == pytest.approx([-0.60653, 0, 0], abs=1e-4)
        assert vt.grad[0].cpu().numpy() == pytest.approx([0.60653, -0.60653, 0], abs=1e-4)
        assert vt.grad[1].cpu().numpy() == pytest.approx([0.60653, -0.60653, 0], abs=1e-4)


def test_batched_function(mg):
    """test/test_torch.py:150-177."""
    from libmolgrid_amd.torch_bindings import BatchedCoords2GridFunction
    gmaker = mg.GridMaker(resolution=.1, dimension=6.0)
    c = torch.tensor([[[1.0, 0, 0], [1, 0, 0]], [[0, 1, 0], [0, 1, 0]]], device="cuda",
                     requires_grad=True)
    vt = torch.tensor([[[0, 1.0, 0], [1.0, 0, 0]], [[0, 1.0, 0], [1.0, 0, 0]]], device="cuda",
                      requires_grad=True)
    r = torch.full((2, 2), 2.0, device="cuda")
    grid = BatchedCoords2GridFunction.apply(gmaker, (0, 0, 0), c, vt, r)
    diff = torch.zeros((2,) + gmaker.grid_dimensions(3), device="cuda")
    diff[:, 0, 30, 30, 30] = 1.0
    diff[:, 1, 30, 30, 30] = -1.0
    grid.backward(diff)
    g = c.grad.cpu().numpy()
    assert g[0][0] == pytest.approx([0.60653, 0, 0], abs=1e-4)
    assert g[0][1] == pytest.approx([-0.60653, 0, 0], abs=1e-4)
    assert g[1][0] == pytest.approx([0, 0.60653, 0], abs=1e-4)
    assert g[1][1] == pytest.approx([0, -0.60653, 0], abs=1e-4)
    t = vt.grad.cpu().numpy()
    for b in range(2):
        for a in range(2):
            assert t[b][a] == pytest.approx([0.60653, -0.60653, 0], abs=1e-4)


def test_module_optimises_coordinates(mg):
    """Gradient descent through the layer pulls an atom onto a target density."""
    from libmolgrid_amd.torch_bindings import Coords2Grid
    gmaker = mg.GridMaker(resolution=0.5, dimension=11.5)
    layer = Coords2Grid(gmaker, center=(0, 0, 0))
    types = torch.ones((1, 1), device="cuda")
    radii = torch.full((1,), 1.5, device="cuda")
    target = layer(torch.tensor([[1.0, 0.5, -0.5]], device="cuda"), types, radii).detach()
    coords = torch.zeros((1, 3), device="cuda", requires_grad=True)
    opt = torch.optim.SGD([coords], lr=0.05)
    first = None
    for _ in range(60):
        opt.zero_grad()
        loss = ((layer(coords, types, radii) - target) ** 2).sum()
        loss.backward()
        opt.step()
        first = first if first is not None else float(loss.detach())
    assert float(loss.detach()) < 0.05 * first
    assert np.allclose(coords.detach().cpu().numpy(), [[1.0, 0.5, -0.5]], atol=0.1)
    assert "resolution 0.50" in repr(layer)
