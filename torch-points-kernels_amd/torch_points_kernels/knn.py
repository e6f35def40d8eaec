"""Dense k nearest neighbours (reference: torch_points_kernels/knn.py:4-18)."""
from ._native import native, require_gpu


def knn(pos_support, pos, k):
    """Dense knn search

    Arguments:
        pos_support - [B,N,3] support points
        pos - [B,M,3] centre of queries
        k - number of neighbours, needs to be <= N

    Returns:
        idx - [B,M,k]
        dist2 - [B,M,k] squared distances

    The reference serves CPU tensors only and raises for CUDA tensors; this build serves GPU
    tensors only.  Neighbours ascend by (squared distance, index).
    """
    assert pos_support.dim() == 3 and pos.dim() == 3
    require_gpu(pos_support, "knn")
    require_gpu(pos, "knn")
    return native().dense_knn(pos_support, pos, k)
