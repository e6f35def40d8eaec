"""Dense k nearest neighbours (API of the reference's torch_points_kernels/knn.py)."""
from ._native import host, native


def knn(pos_support, pos, k):
    """For every query point the k nearest support points of the same cloud.

    pos_support (B, N, 3): points searched; pos (B, M, 3): query points; k <= N.
    Returns (idx (B, M, k) int64, dist2 (B, M, k) squared distances), nearest first; equal distances
    keep the lower index first.

    The reference (knn.py:4-18) serves CPU tensors only and raises for CUDA tensors; here CPU tensors go
    to the host module and GPU tensors to the HIP kernels.
    """
    assert pos_support.dim() == 3 and pos.dim() == 3
    if pos_support.is_cuda != pos.is_cuda:
        raise ValueError("pos_support and pos must live on the same device")
    if pos_support.is_cuda:
        return native().dense_knn(pos_support, pos, k)
    return host().dense_knn(pos_support, pos, k)
