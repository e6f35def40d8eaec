"""GRNet's gridding operator: point clouds to occupancy grids (API of the reference's
torch_points_kernels/gridding.py: GriddingFunction, gridding)."""
import torch

from ._native import native, require_gpu


class GriddingFunction(torch.autograd.Function):
    """Trilinear deposit of points given in grid units into a grid spanning [-scale, scale - 1] on
    every axis; returns the grid flattened to (B, (2 * scale) ** 3).  Differentiable in the points
    (reference gridding.py:7-31)."""

    @staticmethod
    def forward(ctx, ptcloud, scale):
        require_gpu(ptcloud, "gridding")
        lo, hi = -scale, scale - 1
        grid, weights, vertices = native().gridding(lo, hi, lo, hi, lo, hi, ptcloud.contiguous())
        ctx.save_for_backward(weights, vertices)  # (B, n, 8, 3) factors and (B, n, 8) vertex numbers per point
        return grid

    @staticmethod
    def backward(ctx, grad_grid):
        weights, vertices = ctx.saved_tensors
        return native().gridding_grad(weights, vertices, grad_grid.contiguous()), None


def gridding(ptcloud, scale):
    """Grids of resolution 2 * scale per axis from clouds with coordinates in [-1, 1).

    ptcloud: (B, n_pts, 3) floating point tensor on the GPU; scale: int.
    Returns (B, (2 * scale) ** 3).  As in the reference (gridding.py:34-60) the coordinates are
    multiplied by `scale`, and each cloud is gridded on its own after dropping the points whose
    three coordinates sum to zero (padding).
    """
    if ptcloud.dim() != 3 or ptcloud.size(2) != 3:
        raise ValueError("The input point cloud should be of size (B, n_pts, 3)")
    scaled = ptcloud * scale
    grids = []
    for cloud in scaled.unbind(0):
        kept = cloud[cloud.sum(dim=1) != 0]
        grids.append(GriddingFunction.apply(kept.unsqueeze(0), scale))
    return torch.cat(grids, dim=0).contiguous()
