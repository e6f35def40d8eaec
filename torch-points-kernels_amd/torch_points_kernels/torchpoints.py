"""Point-cloud operators with the names, argument order and error behaviour of
torch-points-kernels' ``torchpoints.py`` (reference: torch_points_kernels/torchpoints.py),
backed by the HIP kernels of this package for tensors on an AMD GPU.
"""
from typing import Optional

import torch
from torch.autograd import Function

from ._native import native, require_gpu


def furthest_point_sample(xyz, npoint):
    r"""Iterative furthest point sampling (reference: torchpoints.py:14-37).

    xyz (B, N, 3) float32 on the GPU, npoint <= N.  Returns int32 (B, npoint); sampling starts
    at point 0 of each cloud.
    """
    if npoint > xyz.shape[1]:
        raise ValueError("caanot sample %i points from an input set of %i points" % (npoint, xyz.shape[1]))
    require_gpu(xyz, "furthest_point_sample")
    return native().furthest_point_sampling(xyz, npoint)


def three_nn(unknown, known):
    r"""Three nearest neighbours of `unknown` (B, n, 3) in `known` (B, m, 3)
    (reference: torchpoints.py:40-64).  Returns (dist (B, n, 3) euclidean, idx (B, n, 3) int32).
    """
    if unknown.shape[1] < 3:
        raise ValueError("Not enough points. unknown should ahve at least 3 points.")
    require_gpu(unknown, "three_nn")
    dist2, idx = native().three_nn(unknown, known)
    return torch.sqrt(dist2), idx


class ThreeInterpolate(Function):
    """Weighted interpolation from three neighbours (reference: torchpoints.py:67-106)."""

    @staticmethod
    def forward(ctx, features, idx, weight):
        B, c, m = features.size()
        ctx.three_interpolate_for_backward = (idx, weight, m)
        require_gpu(features, "three_interpolate")
        return native().three_interpolate(features, idx, weight)

    @staticmethod
    def backward(ctx, grad_out):
        idx, weight, m = ctx.three_interpolate_for_backward
        require_gpu(grad_out, "three_interpolate (backward)")
        grad_features = native().three_interpolate_grad(grad_out.contiguous(), idx, weight, m)
        return grad_features, None, None


def three_interpolate(features, idx, weight):
    r"""features (B, c, m), idx (B, n, 3) int32, weight (B, n, 3) -> (B, c, n)
    (reference: torchpoints.py:109-126)."""
    return ThreeInterpolate.apply(features, idx, weight)


class GroupingOperation(Function):
    """Gather of feature columns with a native backward.  The reference expresses the same
    function with ``torch.gather`` on an index repeated over channels (torchpoints.py:129-146);
    the result and its gradient are the same."""

    @staticmethod
    def forward(ctx, features, idx):
        require_gpu(features, "grouping_operation")
        ctx.grouping_for_backward = (idx, features.size(2))
        return native().grouping_operation(features.contiguous(), idx.contiguous())

    @staticmethod
    def backward(ctx, grad_out):
        idx, n = ctx.grouping_for_backward
        return native().grouping_operation_grad(grad_out.contiguous(), idx.contiguous(), n), None


def grouping_operation(features, idx):
    r"""features (B, C, N), idx (B, npoint, nsample) int64 -> (B, C, npoint, nsample)
    (reference: torchpoints.py:129-146)."""
    return GroupingOperation.apply(features, idx)


def ball_query_dense(radius, nsample, xyz, new_xyz, batch_xyz=None, batch_new_xyz=None, sort=False):
    """Reference: torchpoints.py:149-157.  Returns (idx int64 (B, M, nsample), dist2 float32)."""
    require_gpu(new_xyz, "ball_query_dense")
    # sort=True: the nsample nearest neighbours within the radius, nearest first - what the reference
    # computes for CPU tensors (torchpoints.py:154-155); its CUDA path raises NotImplementedError.
    ind, dist = native().ball_query_dense(new_xyz, xyz, radius, nsample, bool(sort))
    return ind, dist


def ball_query_partial_dense(radius, nsample, x, y, batch_x, batch_y, sort=False):
    """Reference: torchpoints.py:160-168.  Returns (idx int64 (|y|, nsample), dist2 float32)."""
    require_gpu(x, "ball_query_partial_dense")
    # sort=True: as for the dense layout (reference, CPU tensors only: torchpoints.py:165-166)
    ind, dist = native().ball_query_partial_dense(x, y, batch_x, batch_y, radius, nsample, bool(sort))
    return ind, dist


def ball_query(
    radius: float,
    nsample: int,
    x: torch.Tensor,
    y: torch.Tensor,
    mode: Optional[str] = "dense",
    batch_x: Optional[torch.Tensor] = None,
    batch_y: Optional[torch.Tensor] = None,
    sort: Optional[bool] = False,
):
    """Radius search (reference: torchpoints.py:171-218).

    x: support points, (M, 3) [partial_dense] or (B, M, 3) [dense]; y: ball centres,
    (npoint, 3) or (B, npoint, 3); mode: "dense" or "partial_dense" (any case); batch_x,
    batch_y: sorted cloud ids, partial_dense only.  Returns (idx, dist2); unused slots are
    padded as the reference's GPU path pads them.
    """
    if mode is None:
        raise Exception('The mode should be defined within ["partial_dense | dense"]')

    if mode.lower() == "partial_dense":
        if (batch_x is None) or (batch_y is None):
            raise Exception("batch_x and batch_y should be provided")
        assert x.size(0) == batch_x.size(0)
        assert y.size(0) == batch_y.size(0)
        assert x.dim() == 2
        return ball_query_partial_dense(radius, nsample, x, y, batch_x, batch_y, sort=sort)

    elif mode.lower() == "dense":
        if (batch_x is not None) or (batch_y is not None):
            raise Exception("batch_x and batch_y should not be provided")
        assert x.dim() == 3
        return ball_query_dense(radius, nsample, x, y, sort=sort)
    else:
        raise Exception("unrecognized mode {}".format(mode))
