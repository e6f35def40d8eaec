// IoU between proposed instances and ground-truth instances (PointGroup's scoring step).
// Reference: cuda/src/metrics_gpu.cu:9-61 - one block per proposal, one thread per ground-truth
// instance, each thread walking the whole proposal: |proposal| x instances label look-ups.
// Here a workgroup owns a proposal and counts its points per ground-truth instance once, in an
// LDS histogram (integer LDS atomics); the quotients are then formed from the counts:
// |proposal| + instances steps.  Samples with more instances than the histogram holds fall back
// to the reference's walk.  Every element of the output row is written (zeros outside the columns
// of the proposal's sample; the reference pre-zeroes the tensor, cuda/src/metrics.cpp:37-39).
#include "tpk_device.h"

namespace {

constexpr int IOU_THREADS = 256;
constexpr int IOU_BINS = 8192; // ground-truth instances of one sample counted in LDS (32 KiB)

// The kernel's expression, with its types: float operands, the 1e-5 a double, stored as float.
__device__ __forceinline__ float iou_value(int intersection, int proposal_total, int instance_total)
{
    return static_cast<float>(static_cast<float>(intersection) /
                              (static_cast<float>(proposal_total + instance_total - intersection) + 1e-5));
}

__global__ __launch_bounds__(IOU_THREADS) void instance_iou_kernel(
    int64_t total_instances, int64_t n_proposals, int64_t n_points, int64_t n_samples,
    const int64_t* __restrict__ n_instances, const int64_t* __restrict__ proposals_idx,
    const int64_t* __restrict__ proposals_offset, const int64_t* __restrict__ labels,
    const int64_t* __restrict__ instance_offset, const int64_t* __restrict__ batch,
    const int64_t* __restrict__ instance_pointnum, float* __restrict__ iou)
{
    __shared__ int bins[IOU_BINS];
    const int tid = threadIdx.x;
    for (int64_t p = blockIdx.x; p < n_proposals; p += gridDim.x)
    {
        float* row = iou + p * total_instances;
        const int64_t start = proposals_offset[p], end = proposals_offset[p + 1];
        int64_t first = 0, count = 0;
        if (end > start)
        {
            const int64_t point = proposals_idx[start];
            const int64_t sample = point >= 0 && point < n_points ? batch[point] : -1;
            if (sample >= 0 && sample < n_samples)
            {
                first = instance_offset[sample];
                count = n_instances[sample];
            }
        }
        if (first < 0 || count < 0 || first + count > total_instances)
            count = 0; // inconsistent description: the row stays zero
        for (int64_t c = tid; c < total_instances; c += IOU_THREADS)
            if (c < first || c >= first + count)
                row[c] = 0.0f;
        const int proposal_total = static_cast<int>(end - start);
        if (count <= IOU_BINS)
        {
            for (int k = tid; k < count; k += IOU_THREADS)
                bins[k] = 0;
            __syncthreads();
            for (int64_t i = start + tid; i < end; i += IOU_THREADS)
            {
                const int64_t point = proposals_idx[i];
                if (point < 0 || point >= n_points)
                    continue;
                const int label = static_cast<int>(labels[point]); // label k + 1 = instance k; 0: none
                if (label >= 1 && label <= count)
                    atomicAdd(&bins[label - 1], 1);
            }
            __syncthreads();
            for (int k = tid; k < count; k += IOU_THREADS)
                row[first + k] = iou_value(bins[k], proposal_total, static_cast<int>(instance_pointnum[first + k]));
            __syncthreads(); // the histogram is reused by the next proposal
        }
        else
        {
            for (int64_t k = tid; k < count; k += IOU_THREADS)
            {
                int intersection = 0;
                for (int64_t i = start; i < end; ++i)
                {
                    const int64_t point = proposals_idx[i];
                    if (point >= 0 && point < n_points && static_cast<int>(labels[point]) == k + 1)
                        ++intersection;
                }
                row[first + k] = iou_value(intersection, proposal_total, static_cast<int>(instance_pointnum[first + k]));
            }
        }
    }
}

} // namespace

extern "C" int tpk_instance_iou(int64_t total_gt_instances, int64_t n_proposals, int64_t n_points, int64_t n_samples,
                                const int64_t* num_gt_instances, const int64_t* proposals_idx,
                                const int64_t* proposals_offset, const int64_t* instance_labels,
                                const int64_t* offset_num_gt_instances, const int64_t* batch,
                                const int64_t* instance_pointnum, float* proposals_iou, void* stream)
{
    if (total_gt_instances < 0 || n_proposals < 0 || n_points < 0 || n_samples < 0)
        return TPK_ERR_INVALID_ARG;
    if (n_proposals == 0 || total_gt_instances == 0)
        return TPK_OK;
    if (!proposals_offset || !proposals_iou || !num_gt_instances || !offset_num_gt_instances || !instance_pointnum ||
        (n_points > 0 && (!instance_labels || !batch)))
        return TPK_ERR_INVALID_ARG;
    const int64_t blocks = n_proposals < 262144 ? n_proposals : 262144;
    hipLaunchKernelGGL(instance_iou_kernel, dim3(static_cast<unsigned>(blocks)), dim3(IOU_THREADS), 0,
                       tpk_stream(stream), total_gt_instances, n_proposals, n_points, n_samples, num_gt_instances,
                       proposals_idx, proposals_offset, instance_labels, offset_num_gt_instances, batch,
                       instance_pointnum, proposals_iou);
    return tpk_launch_status();
}
