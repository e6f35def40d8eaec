// Inverted index ("lists"): for every target position of a cloud, the entries that refer to
// it.  Shared by the backward passes that would otherwise scatter with float atomics
// (three_interpolate, grouping, Chamfer): they gather along these lists instead.
#pragma once

#include "tpk_device.h"

namespace {

constexpr int G_THREADS = 1024;

template <typename Kernel>
int allow_lds(Kernel kernel, size_t bytes)
{
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       static_cast<int>(bytes));
    return e == hipSuccess ? TPK_OK : static_cast<int>(e);
}

// One entry of a target's list: the column that references it and the weight it carries.
template <bool WEIGHTED>
struct ListEntry;
template <>
struct ListEntry<true>
{
    int j;
    float w;
};
template <>
struct ListEntry<false>
{
    int j;
};

constexpr int L_MAX_TARGETS = 30720; // target positions whose counters fit in LDS (120 KiB)

// Inverts the index of one cloud.  grid: (clouds * splits); a workgroup builds the lists of
// the targets [split * span, (split + 1) * span) of its cloud: it reads every index entry of
// the cloud, counts those inside its span (LDS integer atomics) and those below it (their
// number is where its lists start), prefix-sums the counts and fills the lists in a second
// pass.  Workgroups never wait for each other.  dynamic LDS: (span + 1 + G_THREADS) ints.
//   offsets[cloud][0..m]  start of each target's list (exclusive prefix sum of the counts)
//   entries[cloud][...]   the lists, back to back
// Index values outside [0, m) are dropped.
template <int K, bool WEIGHTED, typename IdxT>
__global__ __launch_bounds__(G_THREADS) void build_lists_kernel(
    int m, int total, int splits, int span, const IdxT* __restrict__ idx,
    const float* __restrict__ weight, int* __restrict__ offsets,
    ListEntry<WEIGHTED>* __restrict__ entries)
{
    extern __shared__ int counters[];
    int* scan = counters + span + 1;
    const int tid = threadIdx.x;
    const int cloud = blockIdx.x / splits;
    const int split = blockIdx.x - cloud * splits;
    const int i0 = split * span;
    const int i1 = min(i0 + span, m);
    const int width = i1 - i0;
    idx += static_cast<int64_t>(cloud) * total;
    if (WEIGHTED)
        weight += static_cast<int64_t>(cloud) * total;
    offsets += static_cast<int64_t>(cloud) * (m + 1);
    entries += static_cast<int64_t>(cloud) * total;

    for (int t = tid; t < width; t += G_THREADS)
        counters[t] = 0;
    __syncthreads();
    int below = 0; // valid entries whose target lies before this span
    constexpr int BATCH = 8; // index loads in flight per thread
    for (int e0 = tid; e0 < total; e0 += BATCH * G_THREADS)
    {
        int64_t iv[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
        {
            const int e = e0 + u * G_THREADS;
            const int64_t v = static_cast<int64_t>(idx[min(e, total - 1)]);
            iv[u] = e < total ? v : -1;
        }
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
        {
            below += (iv[u] >= 0 && iv[u] < i0) ? 1 : 0;
            if (iv[u] >= i0 && iv[u] < i1)
                atomicAdd(&counters[static_cast<int>(iv[u]) - i0], 1);
        }
    }
    __syncthreads();

    // prefix sums over the threads: of `below` (gives the start of the span's lists) and of
    // the counters (every thread owns a run of `per` consecutive counters)
    const int per = (width + G_THREADS - 1) / G_THREADS;
    const int lo = min(tid * per, width), hi = min(lo + per, width);
    int sum = 0;
    for (int t = lo; t < hi; ++t)
        sum += counters[t];
    __shared__ int below_total;
    if (tid == 0)
        below_total = 0;
    scan[tid] = sum;
    __syncthreads();
    atomicAdd(&below_total, below);
    for (int step = 1; step < G_THREADS; step <<= 1)
    {
        const int add = tid >= step ? scan[tid - step] : 0;
        __syncthreads();
        scan[tid] += add;
        __syncthreads();
    }
    int run = below_total + scan[tid] - sum;
    for (int t = lo; t < hi; ++t)
    {
        const int c = counters[t];
        counters[t] = run; // becomes the fill cursor of target i0 + t
        offsets[i0 + t] = run;
        run += c;
    }
    if (split == splits - 1 && tid == G_THREADS - 1)
        offsets[m] = below_total + scan[tid];
    __syncthreads();

    // Second pass: all loads of a batch are issued unconditionally (clamped index) before
    // the entries inside the span take their list positions.
    for (int e0 = tid; e0 < total; e0 += BATCH * G_THREADS)
    {
        int64_t iv[BATCH];
        float wv[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
        {
            const int e = min(e0 + u * G_THREADS, total - 1);
            iv[u] = static_cast<int64_t>(idx[e]);
            if constexpr (WEIGHTED)
                wv[u] = weight[e];
        }
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
        {
            const bool mine = iv[u] >= i0 && iv[u] < i1 && e0 + u * G_THREADS < total;
            if (mine)
            {
                const int pos = atomicAdd(&counters[static_cast<int>(iv[u]) - i0], 1);
                ListEntry<WEIGHTED> entry;
                entry.j = (e0 + u * G_THREADS) / K;
                if constexpr (WEIGHTED)
                    entry.w = wv[u];
                entries[pos] = entry;
            }
        }
    }
}


// Launches build_lists_kernel for `clouds` clouds of `m` targets and `total` index entries
// each.  Returns TPK_ERR_UNSUPPORTED when a span of targets would not fit in LDS.
template <int K, bool WEIGHTED, typename IdxT>
int launch_build_lists(int clouds, int m, int64_t total, const IdxT* idx, const float* weight,
                       int* offsets, ListEntry<WEIGHTED>* entries, hipStream_t s)
{
    if (clouds <= 0 || m <= 0 || total <= 0)
        return TPK_OK;
    if (total > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    // Enough workgroups to occupy a good part of the chip; spans of a multiple of 64 targets.
    int splits = static_cast<int>(tpk_ceil_div(128, clouds));
    if (splits > 16)
        splits = 16;
    if (splits < tpk_ceil_div(m, L_MAX_TARGETS))
        splits = static_cast<int>(tpk_ceil_div(m, L_MAX_TARGETS));
    const int span = static_cast<int>(tpk_ceil_div(tpk_ceil_div(m, splits), 64) * 64);
    splits = static_cast<int>(tpk_ceil_div(m, span));
    if (span > L_MAX_TARGETS || static_cast<int64_t>(clouds) * splits > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const size_t lds = (static_cast<size_t>(span) + 1 + G_THREADS) * sizeof(int);
    auto build = build_lists_kernel<K, WEIGHTED, IdxT>;
    int st = allow_lds(build, lds);
    if (st != TPK_OK)
        return st;
    hipLaunchKernelGGL(build, dim3(static_cast<unsigned>(clouds) * splits), dim3(G_THREADS), lds, s, m,
                       static_cast<int>(total), splits, span, idx, weight, offsets, entries);
    return tpk_launch_status();
}

} // namespace
