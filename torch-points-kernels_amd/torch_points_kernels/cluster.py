"""Region growing over ball-query neighbourhoods (reference: torch_points_kernels/cluster.py).

The reference searches the neighbours on the device, copies the matrix to the host and grows the
clusters there with a numba routine; here both steps run on the device the tensors live on (the HIP
kernels for GPU tensors, the host module for CPU tensors).
"""
from typing import List

import torch

from ._native import host, native
from .torchpoints import ball_query_partial_dense


def _grow(pos, batch, nsample, radius, min_cluster_size, member_order):
    if member_order not in ("reference", "index"):
        raise ValueError("member_order must be 'reference' or 'index'")
    assert pos.shape[0] == batch.shape[0]
    if pos.is_cuda != batch.is_cuda:
        raise ValueError("pos and batch must live on the same device")
    neighbours = ball_query_partial_dense(radius, nsample, pos, pos, batch, batch)[0]
    if pos.is_cuda:
        members, starts = native().grow_proximity(neighbours, int(min_cluster_size), member_order == "reference")
    else:
        # the host walk is the reference's walk: members come in its order whatever member_order says
        members, starts = host().grow_proximity(neighbours, int(min_cluster_size))
    return members, starts


def grow_proximity(pos, batch, nsample=16, radius=0.02, min_cluster_size=32, member_order="reference"):
    """Grow based on proximity only (reference cluster.py:40-45).

    Returns the clusters as a list of lists of point indices, ordered by their first point.
    member_order (GPU tensors): "reference" lists the members of a cluster in the order the reference
    does (the order in which its walk over the neighbour matrix meets them); that walk is serial inside a
    cluster, and on the GPU it is slower than one host core once a cluster holds tens of thousands of
    points.  "index" lists the members in ascending order, everything data-parallel - about 100 times
    faster on such clusters: use it whenever the order inside a cluster does not matter (it does not for
    instance segmentation, the use region_grow was written for).  The clusters themselves are the same.
    """
    members, starts = _grow(pos, batch, nsample, radius, min_cluster_size, member_order)
    members = members.tolist()
    starts = starts.tolist()
    return [members[a:b] for a, b in zip(starts[:-1], starts[1:])]


def region_grow(
    pos, labels, batch, ignore_labels=[], nsample=16, radius=0.02, min_cluster_size=32, member_order="reference"
) -> List[torch.Tensor]:
    """PointGroup's region growing (https://arxiv.org/pdf/2004.01658.pdf): clusters of points of equal label
    that are chained by neighbourhoods of the given radius, label by label.

    pos (N, 3), labels (N,), batch (N,) sorted sample ids; labels in ignore_labels are skipped; a row of the
    neighbour search holds at most nsample points; clusters below min_cluster_size are dropped.
    Returns a list of index tensors into pos (on pos.device), label after label, ordered by first point
    inside a label.  member_order: see grow_proximity; pass "index" unless the reference's order inside a
    cluster is needed.

    Reference: cluster.py:48-109.
    """
    assert labels.dim() == 1
    assert pos.dim() == 2
    assert pos.shape[0] == labels.shape[0]

    clusters = []
    ind = torch.arange(0, pos.shape[0], device=pos.device)
    for l in torch.unique(labels).tolist():
        if l in ignore_labels:
            continue

        # points of this label only, their clouds renumbered to 0, 1, 2, ...
        label_mask = labels == l
        local_ind = ind[label_mask]
        remaped_batch = torch.unique(batch[label_mask], return_inverse=True)[1]

        members, starts = _grow(
            pos[label_mask, :].contiguous(), remaped_batch, nsample, radius, min_cluster_size, member_order
        )
        members = local_ind[members]
        starts = starts.tolist()
        for a, b in zip(starts[:-1], starts[1:]):
            clusters.append(members[a:b])

    return clusters
