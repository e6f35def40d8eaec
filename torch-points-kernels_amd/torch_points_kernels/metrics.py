"""IoU between proposed and ground-truth instances (reference: torch_points_kernels/metrics.py)."""
from typing import List, Optional

import torch

from ._native import host, native


def instance_iou(
    instance_idx: List[torch.Tensor],
    gt_instances: torch.Tensor,
    batch: Optional[torch.Tensor] = None,
):
    """IoU of every proposed instance with every ground-truth instance.

    instance_idx: list of index tensors, one per proposal (the points it holds);
    gt_instances: (N,) ground-truth instance of every point, numbered from 1 inside each sample, 0 (or a
    negative value) for points of no instance; batch: (N,) sample of every point, sorted (default: one sample).
    Returns float32 (number of proposals, ground-truth instances of all samples); a proposal is compared
    with the instances of the sample its first point belongs to, the other columns are 0.

    Reference: metrics.py:37-104.  As there, the GPU kernel adds 1e-5 to the union and the host routine
    does not.
    """
    if batch is None:
        batch = torch.zeros_like(gt_instances)

    # Number of ground-truth instances per sample and their sizes (one bincount per sample in place of the
    # reference's loop over instance ids)
    gt_instance_sizes = []
    num_gt_instances = []
    batch_size = int(batch[-1]) + 1
    for s in range(batch_size):
        sample_gt_instances = gt_instances[batch == s]
        sample_num_gt_instances = int(torch.max(sample_gt_instances).item())
        num_gt_instances.append(sample_num_gt_instances)
        if sample_num_gt_instances > 0:
            counts = torch.bincount(sample_gt_instances[sample_gt_instances > 0], minlength=sample_num_gt_instances + 1)
            gt_instance_sizes.append(counts[1 : sample_num_gt_instances + 1])
    device = gt_instances.device
    gt_instance_sizes = torch.cat(gt_instance_sizes) if gt_instance_sizes else torch.zeros(0, dtype=torch.long, device=device)
    num_gt_instances = torch.tensor(num_gt_instances, dtype=torch.long, device=device)

    # Instance offset when flatten
    instance_offsets = [0]
    cum_offset = 0
    for instance in instance_idx:
        cum_offset += instance.shape[0]
        instance_offsets.append(cum_offset)

    instance_idx = torch.cat(instance_idx) if len(instance_idx) else torch.zeros(0, dtype=torch.long, device=device)
    if not gt_instances.is_cuda:
        return host().instance_iou(
            instance_idx.long().contiguous(),
            torch.tensor(instance_offsets, dtype=torch.long),
            gt_instances.long().contiguous(),
            gt_instance_sizes.long().contiguous(),
            num_gt_instances,
            batch.long().contiguous(),
        )
    return native().instance_iou_cuda(
        instance_idx.to(device).long().contiguous(),
        torch.tensor(instance_offsets, dtype=torch.long, device=device),
        gt_instances.long().contiguous(),
        gt_instance_sizes.long().contiguous(),
        num_gt_instances,
        batch.long().contiguous(),
    )
