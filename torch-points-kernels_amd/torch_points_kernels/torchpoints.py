"""Point-cloud operators with the names, argument order and error behaviour of
torch-points-kernels' ``torchpoints.py`` (reference: torch_points_kernels/torchpoints.py),
backed by the HIP kernels of this package for tensors on an AMD GPU and by the package's host module
(points_cpu) for tensors in host memory.  As in the reference the two follow different conventions
where its CUDA and CPU paths do (index types, start point of the sampling, order and padding of the
ball query); each docstring says which.
"""
from typing import Optional

import torch
from torch.autograd import Function

from ._native import host, native
from .knn import knn


def furthest_point_sample(xyz, npoint):
    r"""Iterative furthest point sampling (reference: torchpoints.py:14-37).

    xyz (B, N, 3), npoint <= N.  GPU tensors (float32): int32 (B, npoint), sampling starts at point 0
    of each cloud.  CPU tensors: int64, sampling starts at a point drawn from torch's default generator
    (the reference passes random=True, torchpoints.py:37).
    """
    if npoint > xyz.shape[1]:
        raise ValueError("caanot sample %i points from an input set of %i points" % (npoint, xyz.shape[1]))
    if xyz.is_cuda:
        return native().furthest_point_sampling(xyz, npoint)
    return host().fps(xyz, npoint, True)


def three_nn(unknown, known):
    r"""Three nearest neighbours of `unknown` (B, n, 3) in `known` (B, m, 3)
    (reference: torchpoints.py:40-64).  Returns (dist (B, n, 3) euclidean, idx (B, n, 3): int32 for GPU
    tensors, int64 for CPU tensors).
    """
    if unknown.shape[1] < 3:
        raise ValueError("Not enough points. unknown should ahve at least 3 points.")
    if unknown.is_cuda:
        dist2, idx = native().three_nn(unknown, known)
    else:
        idx, dist2 = knn(known, unknown, 3)
    return torch.sqrt(dist2), idx


class ThreeInterpolate(Function):
    """Weighted interpolation from three neighbours (reference: torchpoints.py:67-106)."""

    @staticmethod
    def forward(ctx, features, idx, weight):
        B, c, m = features.size()
        ctx.three_interpolate_for_backward = (idx, weight, m)
        ctx.three_interpolate_lists = None
        if features.is_cuda:
            if ctx.needs_input_grad[0]:
                # a backward pass will follow: what it needs of (idx, weight) - the index inverted into lists per
                # target - is built now, and the backward pass only walks it (and any further backward pass shares it)
                out, lists = native().three_interpolate_recording(features.contiguous(), idx.contiguous(), weight.contiguous())
                ctx.three_interpolate_lists = lists if lists.numel() else None
                return out
            return native().three_interpolate(features, idx, weight)
        return host().knn_interpolate(features, idx, weight)

    @staticmethod
    def backward(ctx, grad_out):
        idx, weight, m = ctx.three_interpolate_for_backward
        if grad_out.is_cuda and ctx.three_interpolate_lists is not None:
            grad_features = native().three_interpolate_grad_lists(grad_out.contiguous(), ctx.three_interpolate_lists, m)
        elif grad_out.is_cuda:
            grad_features = native().three_interpolate_grad(grad_out.contiguous(), idx, weight, m)
        else:
            grad_features = host().knn_interpolate_grad(grad_out.contiguous(), idx, weight, m)
        return grad_features, None, None


def three_interpolate(features, idx, weight):
    r"""features (B, c, m), idx (B, n, 3) (int32 on the GPU, int64 on the CPU: what three_nn returns there),
    weight (B, n, 3) -> (B, c, n) (reference: torchpoints.py:109-126)."""
    return ThreeInterpolate.apply(features, idx, weight)


class GroupingOperation(Function):
    """Gather of feature columns with a native backward.  The reference expresses the same
    function with ``torch.gather`` on an index repeated over channels (torchpoints.py:129-146);
    the result and its gradient are the same."""

    @staticmethod
    def forward(ctx, features, idx):
        ctx.grouping_for_backward = (idx, features.size(2))
        ctx.grouping_lists = None
        if ctx.needs_input_grad[0]:
            # (as in ThreeInterpolate: the lists the backward pass walks are built with the forward pass)
            out, lists = native().grouping_operation_recording(features.contiguous(), idx.contiguous())
            ctx.grouping_lists = lists if lists.numel() else None
            return out
        return native().grouping_operation(features.contiguous(), idx.contiguous())

    @staticmethod
    def backward(ctx, grad_out):
        idx, n = ctx.grouping_for_backward
        if ctx.grouping_lists is not None:
            return native().grouping_operation_grad_lists(grad_out.contiguous(), ctx.grouping_lists, n), None
        return native().grouping_operation_grad(grad_out.contiguous(), idx.contiguous(), n), None


def grouping_operation(features, idx):
    r"""features (B, C, N), idx (B, npoint, nsample) int64 -> (B, C, npoint, nsample)
    (reference: torchpoints.py:129-146).  float32 tensors on the GPU take the native kernels; every other
    device and dtype is served, as in the reference, by torch's own gather (and its autograd)."""
    if features.is_cuda and features.dtype == torch.float32 and idx.dtype == torch.int64:
        return GroupingOperation.apply(features, idx)
    b, c = features.shape[0], features.shape[1]
    columns = idx.reshape(b, 1, -1).expand(b, c, -1)
    return torch.gather(features, 2, columns).reshape(b, c, idx.shape[1], idx.shape[2])


def ball_query_dense(radius, nsample, xyz, new_xyz, batch_xyz=None, batch_new_xyz=None, sort=False):
    """Reference: torchpoints.py:149-157.  Returns (idx int64 (B, M, nsample), dist2 float32)."""
    if new_xyz.is_cuda:
        # sort=True: the nsample nearest neighbours within the radius, nearest first - what the reference
        # computes for CPU tensors (torchpoints.py:154-155); its CUDA path raises NotImplementedError.
        ind, dist = native().ball_query_dense(new_xyz, xyz, radius, nsample, bool(sort))
    else:
        # CPU tensors, as in the reference: sort=False returns a random choice of nsample hits in random order
        ind, dist = host().dense_ball_query(new_xyz, xyz, radius, nsample, mode=0, sorted=bool(sort))
    return ind, dist


def ball_query_partial_dense(radius, nsample, x, y, batch_x, batch_y, sort=False):
    """Reference: torchpoints.py:160-168.  Returns (idx int64 (|y|, nsample), dist2 float32)."""
    if x.is_cuda:
        # sort=True: as for the dense layout (reference, CPU tensors only: torchpoints.py:165-166)
        ind, dist = native().ball_query_partial_dense(x, y, batch_x, batch_y, radius, nsample, bool(sort))
    else:
        ind, dist = host().batch_ball_query(x, y, batch_x, batch_y, radius, nsample, mode=0, sorted=bool(sort))
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
    padded as the reference pads them on the device the tensors live on.
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
