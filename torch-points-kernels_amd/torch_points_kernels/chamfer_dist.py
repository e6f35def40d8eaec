"""Chamfer distance (reference: torch_points_kernels/chamfer_dist.py)."""
import torch

from ._native import native


class ChamferFunction(torch.autograd.Function):
    """dist1, dist2 = squared distance of every point to its nearest point of the other cloud
    (reference: chamfer_dist.py:7-22).  float32 and float64."""

    @staticmethod
    def forward(ctx, xyz1, xyz2):
        if not xyz1.is_cuda:
            raise NotImplementedError("CPU version is not available for Chamfer Distance")
        dist1, dist2, idx1, idx2 = native().chamfer_dist(xyz1, xyz2)
        ctx.save_for_backward(xyz1, xyz2, idx1, idx2)
        return dist1, dist2

    @staticmethod
    def backward(ctx, grad_dist1, grad_dist2):
        xyz1, xyz2, idx1, idx2 = ctx.saved_tensors
        grad_xyz1, grad_xyz2 = native().chamfer_dist_grad(
            xyz1, xyz2, idx1, idx2, grad_dist1.contiguous(), grad_dist2.contiguous()
        )
        return grad_xyz1, grad_xyz2


def chamfer_dist(xyz1, xyz2, ignore_zeros=False):
    r"""mean(dist1) + mean(dist2) over B pairs of clouds (reference: chamfer_dist.py:25-54).

    xyz1 (B, n1, 3), xyz2 (B, n2, 3).  With ignore_zeros and B == 1, points whose coordinates
    sum to zero are dropped first.
    """
    if len(xyz1.shape) != 3 or xyz1.size(2) != 3 or len(xyz2.shape) != 3 or xyz2.size(2) != 3:
        raise ValueError("The input point cloud should be of size (B, n_pts, 3)")

    batch_size = xyz1.size(0)
    if batch_size == 1 and ignore_zeros:
        non_zeros1 = torch.sum(xyz1, dim=2).ne(0)
        non_zeros2 = torch.sum(xyz2, dim=2).ne(0)
        xyz1 = xyz1[non_zeros1].unsqueeze(dim=0)
        xyz2 = xyz2[non_zeros2].unsqueeze(dim=0)

    dist1, dist2 = ChamferFunction.apply(xyz1, xyz2)
    return torch.mean(dist1) + torch.mean(dist2)
