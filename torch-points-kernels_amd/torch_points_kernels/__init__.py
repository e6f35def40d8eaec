"""torch_points_kernels for AMD MI355X: the spatial-search operators of
torch-points3d/torch-points-kernels (furthest point sampling, ball query, three_nn /
three_interpolate, grouping, Chamfer distance, dense knn, region growing, instance IoU, GRNet's gridding and cubic feature sampling) on hand-written HIP kernels.

Same names and call signatures as the reference package (torch_points_kernels/__init__.py).  GPU
tensors run on the HIP kernels (points_cuda); CPU tensors are served by the host module (points_cpu)
for the operators the reference serves on the CPU.
"""
from .torchpoints import (
    ThreeInterpolate,
    GroupingOperation,
    ball_query,
    ball_query_dense,
    ball_query_partial_dense,
    furthest_point_sample,
    grouping_operation,
    three_interpolate,
    three_nn,
)
from .knn import knn
from .cluster import grow_proximity, region_grow
from .metrics import instance_iou
from .cubic_feature_sampling import cubic_feature_sampling
from .gridding import gridding
from .chamfer_dist import ChamferFunction
from . import chamfer_dist  # the reference exports the submodule under this name

# the names the reference package exports (torch_points_kernels/__init__.py), plus ChamferFunction
__all__ = (
    "ball_query furthest_point_sample grouping_operation three_interpolate three_nn knn region_grow "
    "instance_iou chamfer_dist cubic_feature_sampling gridding ChamferFunction"
).split()
