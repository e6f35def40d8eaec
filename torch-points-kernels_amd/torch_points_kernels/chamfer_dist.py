"""Chamfer distance between point clouds (API of the reference's torch_points_kernels/chamfer_dist.py)."""
import torch

from ._native import native


def _is_cloud_batch(t):
    return t.dim() == 3 and t.size(2) == 3


class ChamferFunction(torch.autograd.Function):
    """(xyz1 (B, n, 3), xyz2 (B, m, 3)) -> (dist1 (B, n), dist2 (B, m)): squared distance of every point
    to the nearest point of the other cloud (reference chamfer_dist.py:7-22).  float32 and float64."""

    @staticmethod
    def forward(ctx, xyz1, xyz2):
        if not xyz1.is_cuda:
            raise NotImplementedError("CPU version is not available for Chamfer Distance")
        dist1, dist2, nearest1, nearest2 = native().chamfer_dist(xyz1, xyz2)
        ctx.save_for_backward(xyz1, xyz2, nearest1, nearest2)
        return dist1, dist2

    @staticmethod
    def backward(ctx, grad_dist1, grad_dist2):
        xyz1, xyz2, nearest1, nearest2 = ctx.saved_tensors
        grad_xyz1, grad_xyz2 = native().chamfer_dist_grad(xyz1, xyz2, nearest1, nearest2, grad_dist1.contiguous(),
                                                          grad_dist2.contiguous())
        return grad_xyz1, grad_xyz2


def chamfer_dist(xyz1, xyz2, ignore_zeros=False):
    """mean(dist1) + mean(dist2) of ChamferFunction over the whole batch (reference chamfer_dist.py:25-54).

    ignore_zeros applies to a batch of one pair only: points whose coordinates sum to zero (padding) are
    removed from both clouds first.
    """
    if not (_is_cloud_batch(xyz1) and _is_cloud_batch(xyz2)):
        raise ValueError("The input point cloud should be of size (B, n_pts, 3)")
    if ignore_zeros and xyz1.size(0) == 1:
        xyz1 = xyz1[:, xyz1[0].sum(dim=1) != 0]
        xyz2 = xyz2[:, xyz2[0].sum(dim=1) != 0]
    dist1, dist2 = ChamferFunction.apply(xyz1, xyz2)
    return dist1.mean() + dist2.mean()
