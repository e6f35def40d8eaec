"""GRNet's cubic feature sampling: the features of the grid vertices around every point (API of
the reference's torch_points_kernels/cubic_feature_sampling.py)."""
import torch

from ._native import native, require_gpu


class CubicFeatureSamplingFunction(torch.autograd.Function):
    """ptcloud (B, n, 3) in grid units, cubic_features (B, c, m, m, m) -> (B, n, (2 * ns) ** 3, c).
    The gradient flows to the feature maps only: the coordinates merely choose vertices
    (reference cubic_feature_sampling.py:7-31)."""

    @staticmethod
    def forward(ctx, ptcloud, cubic_features, neighborhood_size=1):
        require_gpu(ptcloud, "cubic_feature_sampling")
        require_gpu(cubic_features, "cubic_feature_sampling")
        ctx.scale = cubic_features.size(2)
        ctx.neighborhood_size = neighborhood_size
        sampled, vertices = native().cubic_feature_sampling(
            ctx.scale, neighborhood_size, ptcloud.contiguous(), cubic_features.contiguous()
        )
        ctx.save_for_backward(vertices)
        return sampled

    @staticmethod
    def backward(ctx, grad_sampled):
        (vertices,) = ctx.saved_tensors
        grad_points, grad_maps = native().cubic_feature_sampling_grad(
            ctx.scale, ctx.neighborhood_size, grad_sampled.contiguous(), vertices
        )
        return grad_points, grad_maps, None


def cubic_feature_sampling(ptcloud, cubic_features, neighborhood_size=1):
    """Features of the vertices of the cube a point lies in (neighborhood_size = 1) or of that cube and
    neighborhood_size - 1 rings of cubes around it.

    ptcloud: (B, n_pts, 3) with coordinates in [-1, 1); cubic_features: (B, c, m, m, m).
    Returns (B, n_pts, (2 * neighborhood_size) ** 3, c); vertices outside the map give zeros.
    As in the reference (cubic_feature_sampling.py:34-59) the coordinates are mapped to grid units by
    x * m / 2 + m / 2 first.
    """
    if ptcloud.dim() != 3 or ptcloud.shape[2] != 3:
        raise ValueError("The input point cloud should be of size (B, n_pts, 3).")
    half = cubic_features.size(2) / 2
    return CubicFeatureSamplingFunction.apply(ptcloud * half + half, cubic_features, neighborhood_size)
