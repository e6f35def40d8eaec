// Inverted index ("lists"): for every target position of a cloud, the entries that refer to
// it.  Shared by the backward passes that would otherwise scatter with float atomics
// (three_interpolate, grouping): they gather along these lists instead.
#pragma once

#include "tpk_device.h"

namespace {

constexpr int G_THREADS = 1024;

template <typename Kernel>
int allow_lds(Kernel kernel, size_t bytes)
{
    return tpk_allow_lds(reinterpret_cast<const void*>(kernel), bytes);
}

// One entry of a target's list: the column that references it and the weight it carries.  The
// column is stored the way the walker uses it: as the byte offset of that column's value in a
// staged row that starts with four zeros, (column + 4) * 4 - so an all-zero entry, which is what
// a lane without entry is given, points at a zero.
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

constexpr int L_MAX_TARGETS = 15360; // targets whose bookkeeping fits in LDS (2 ints each)
constexpr int L_BLOCK = TPK_WAVE;    // targets per block of lists: one per lane
constexpr int L_SLACK = 832;         // entry slots a block owns beyond three per entry
constexpr int L_WIDTH_STEP = 8;      // widths of the slot-major parts are multiples of this
constexpr int L_COUNT_BITS = 20;     // bits of a meta word that hold a list length
constexpr int L_COUNT_MASK = (1 << L_COUNT_BITS) - 1;

// Layout of the lists of one cloud ("sliced": made to be walked by one lane per target).
// Targets are taken in blocks of 64.  Inside a block the lanes serve the targets in order of
// descending list length, so that in step i of a walk the lanes that still have an entry are
// the first ones: a step requests one contiguous run of entries and nothing for the others.
// `meta` holds one word per position p of a block:
//   bits  0..19  length of the list served by LANE p
//   bits 20..25  the target (position inside the block) that lane p serves
//   bits 26..31  the lane that serves TARGET p
// Block b owns the entry slots from
//   start_b = 3 * (entries of all earlier targets) + L_SLACK * b
// and stores slot i of lane L at start_b + i * 64 + L for i < width_b (only the slots a list
// really has are written; the others are never read).  width_b = min(longest list of the
// block, 2 * ceil(entries of the block / 64) + 4), rounded up to a multiple of 8.  The entries
// of a list beyond width_b follow that part, list after list in lane order.  Slot-major part
// <= 2 * entries + 830 slots, the rest <= entries: a block never leaves its own slots, whatever
// the index looks like.
//   meta[cloud][64 * blocks]
//   blocks[cloud][b]         (start_b, width_b; bit 31 of the width: some list is longer)
//   entries[cloud][capacity]
template <bool WEIGHTED>
struct Lists
{
    int* meta;
    int2* blocks;
    ListEntry<WEIGHTED>* entries;
    int64_t capacity; // entry slots per cloud
};

inline int64_t list_blocks(int m)
{
    return (static_cast<int64_t>(m) + L_BLOCK - 1) / L_BLOCK;
}
inline int64_t list_capacity(int m, int64_t total)
{
    return 3 * total + L_SLACK * list_blocks(m);
}
inline size_t list_align(size_t v)
{
    return (v + 255) & ~static_cast<size_t>(255);
}
// Workspace bytes of the lists of `clouds` clouds with m targets and `total` index entries each.
template <bool WEIGHTED>
size_t lists_bytes(int clouds, int m, int64_t total)
{
    const size_t c = static_cast<size_t>(clouds);
    const size_t positions = static_cast<size_t>(list_blocks(m)) * L_BLOCK;
    return list_align(c * positions * sizeof(int)) +
           list_align(c * static_cast<size_t>(list_blocks(m)) * sizeof(int2)) +
           list_align(c * static_cast<size_t>(list_capacity(m, total)) * sizeof(ListEntry<WEIGHTED>));
}
template <bool WEIGHTED>
Lists<WEIGHTED> lists_at(void* workspace, int clouds, int m, int64_t total)
{
    const size_t c = static_cast<size_t>(clouds);
    const size_t positions = static_cast<size_t>(list_blocks(m)) * L_BLOCK;
    char* p = static_cast<char*>(workspace);
    Lists<WEIGHTED> l;
    l.meta = reinterpret_cast<int*>(p);
    p += list_align(c * positions * sizeof(int));
    l.blocks = reinterpret_cast<int2*>(p);
    p += list_align(c * static_cast<size_t>(list_blocks(m)) * sizeof(int2));
    l.entries = reinterpret_cast<ListEntry<WEIGHTED>*>(p);
    l.capacity = list_capacity(m, total);
    return l;
}

// What a wavefront needs to walk the lists of block `block` of a cloud: start and width of the
// slot-major part, and whether longer lists exist.
struct ListBlock
{
    int start;
    int width;
    bool longer;
};
__device__ __forceinline__ ListBlock list_block(const int2* __restrict__ cloud_blocks, int block)
{
    const int2 d = cloud_blocks[__builtin_amdgcn_readfirstlane(block)];
    return ListBlock{d.x, d.y & 0x7fffffff, d.y < 0};
}
// For a block with longer lists: how many entries of this lane's list lie beyond the slot-major
// part (`extra`), and where they start relative to its end (`extra_at`).  Every lane of the
// wavefront calls it; `count` is the length of the lane's list.
__device__ __forceinline__ void list_extra(int count, int width, int& extra, int& extra_at)
{
    extra = max(count - width, 0);
    extra_at = wave_exclusive_sum(extra);
}

// Inverts the index of one part of one cloud: the cloud's `cloud_total` index entries are cut
// into `parts` runs of `part_total` (a multiple of K; the last may be shorter), and every
// (cloud, part) gets lists of its own, stored as cloud number cloud * parts + part; the columns
// in its entries count from the first column of the part.  grid: (clouds * parts * splits); a
// workgroup builds the lists of the targets [split * span, (split + 1) * span) (span is a
// multiple of 64): it reads every index entry of its part, counts those inside its span (LDS
// integer atomics) and those below it (their number fixes where its blocks start), prefix-sums
// the lengths, orders the lanes of its blocks and fills the lists in a second pass.  Workgroups
// never wait for each other.  dynamic LDS: (2 * span + span / 32 + G_THREADS) ints.  Index values
// outside [0, m) are dropped.
template <bool WEIGHTED, typename IdxT>
struct ListJob
{
    int m, cloud_total, parts, part_total, splits, span, workgroups;
    const IdxT* idx;
    const float* weight;
    Lists<WEIGHTED> lists;
};

template <int K, bool WEIGHTED, typename IdxT>
__global__ __launch_bounds__(G_THREADS) void build_lists_kernel(ListJob<WEIGHTED, IdxT> job)
{
    const int workgroup = blockIdx.x;
    const int m = job.m, cloud_total = job.cloud_total, parts = job.parts, part_total = job.part_total;
    const int splits = job.splits, span = job.span;
    const IdxT* __restrict__ idx = job.idx;
    const float* __restrict__ weight = job.weight;
    const Lists<WEIGHTED>& lists = job.lists;

    extern __shared__ int counters[];            // [span] list lengths, later fill cursors
    int* const aux = counters + span;            // [span] list starts, later (start of the long part | lane << 26)
    int* const block_start = aux + span;         // [span / 64]
    int* const block_width = block_start + span / L_BLOCK;
    int* const scan = block_width + span / L_BLOCK; // [G_THREADS]
    __shared__ int below_total;
    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int wave = tid / TPK_WAVE;
    const int cloud_part = workgroup / splits;
    const int split = workgroup - cloud_part * splits;
    const int part = cloud_part % parts;
    const int total = min(part_total, cloud_total - part * part_total);
    const int i0 = split * span;
    const int i1 = min(i0 + span, m);
    const int width = i1 - i0;
    const int64_t first_entry = static_cast<int64_t>(cloud_part / parts) * cloud_total + static_cast<int64_t>(part) * part_total;
    idx += first_entry;
    if (WEIGHTED)
        weight += first_entry;
    const int64_t cloud_blocks = (m + L_BLOCK - 1) / L_BLOCK;
    int* __restrict__ meta = lists.meta + cloud_part * cloud_blocks * L_BLOCK;
    int2* __restrict__ blocks = lists.blocks + cloud_part * cloud_blocks;
    ListEntry<WEIGHTED>* __restrict__ entries = lists.entries + static_cast<int64_t>(cloud_part) * lists.capacity;

    for (int t = tid; t < span; t += G_THREADS)
        counters[t] = 0;
    if (tid == 0)
        below_total = 0;
    __syncthreads();
    int below = 0; // valid entries whose target lies before this span
    constexpr int BATCH = 16; // index loads in flight per thread
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

    // Prefix sum of the list lengths (every thread owns a run of `per` consecutive targets; sums
    // inside a wavefront by DPP, across wavefronts through LDS): where the entries of every
    // target would start.
    {
        const int below_before = wave_exclusive_sum(below);
        if (lane == TPK_WAVE - 1)
            atomicAdd(&below_total, below_before + below);
    }
    const int per = (width + G_THREADS - 1) / G_THREADS;
    const int lo = min(tid * per, width), hi = min(lo + per, width);
    int sum = 0;
    for (int t = lo; t < hi; ++t)
        sum += counters[t];
    const int before_in_wave = wave_exclusive_sum(sum);
    if (lane == TPK_WAVE - 1)
        scan[wave] = before_in_wave + sum;
    __syncthreads();
    int run = below_total + before_in_wave;
    for (int w = 0; w < wave; ++w)
        run += scan[w];
    for (int t = lo; t < hi; ++t)
    {
        aux[t] = run;
        run += counters[t];
    }
    __syncthreads();

    // Layout of the blocks, one wavefront per block at a time.
    const int nblocks = (width + L_BLOCK - 1) / L_BLOCK;
    for (int blk = wave; blk < nblocks; blk += G_THREADS / TPK_WAVE)
    {
        const int t = blk * L_BLOCK + lane;
        const int count = t < width ? min(counters[t], L_COUNT_MASK) : 0;
        const int first = aux[blk * L_BLOCK];
        const int before = wave_exclusive_sum(count);
        const int block_entries = __builtin_amdgcn_readlane(before + count, TPK_WAVE - 1);
        const int longest = wave_max_i32(count);
        const int w = (min(longest, 2 * ((block_entries + L_BLOCK - 1) / L_BLOCK) + 4) + L_WIDTH_STEP - 1) &
                      ~(L_WIDTH_STEP - 1);
        const int start = 3 * first + L_SLACK * (i0 / L_BLOCK + blk);
        // the lane that serves this target: its rank by descending length (equal lengths in order)
        int serving = 0;
        for (int other = 0; other < TPK_WAVE; ++other)
        {
            const int oc = __builtin_amdgcn_readlane(count, other);
            serving += (oc > count || (oc == count && other < lane)) ? 1 : 0;
        }
        // what lane `lane` serves: the target and the length sent to it by that target's position
        const int served = __builtin_amdgcn_ds_permute(serving * 4, lane);
        const int served_count = __builtin_amdgcn_ds_permute(serving * 4, count);
        int extra, extra_at;
        list_extra(served_count, w, extra, extra_at);
        const int my_extra_at = __builtin_amdgcn_ds_bpermute(serving * 4, extra_at); // of the lane that serves this target
        if (t < width)
        {
            aux[t] = my_extra_at | (serving << 26);
            counters[t] = 0;
        }
        meta[i0 + t] = served_count | (served << L_COUNT_BITS) | (serving << 26);
        if (lane == 0)
        {
            block_start[blk] = start;
            block_width[blk] = w;
            blocks[i0 / L_BLOCK + blk] = make_int2(start, longest > w ? w | static_cast<int>(0x80000000u) : w);
        }
    }
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
        // (the cursor updates of a batch are all issued before their results are used)
        int slot[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
        {
            const bool mine = iv[u] >= i0 && iv[u] < i1 && e0 + u * G_THREADS < total;
            slot[u] = mine ? atomicAdd(&counters[static_cast<int>(iv[u]) - i0], 1) : -1;
        }
        // (and so are the look-ups of where the entries go)
        int at[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
        {
            const int t = slot[u] >= 0 ? static_cast<int>(iv[u]) - i0 : 0;
            const int blk = t / L_BLOCK;
            const int w = block_width[blk];
            const int a = aux[t];
            const int serving = static_cast<int>(static_cast<unsigned>(a) >> 26);
            at[u] = block_start[blk] +
                    (slot[u] < w ? slot[u] * L_BLOCK + serving : w * L_BLOCK + (a & 0x3FFFFFF) + (slot[u] - w));
            if (slot[u] >= L_COUNT_MASK) // (a list longer than a meta word can say is cut there)
                slot[u] = -1;
        }
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
            if (slot[u] >= 0)
            {
                ListEntry<WEIGHTED> entry;
                entry.j = ((e0 + u * G_THREADS) / K + 4) * 4;
                if constexpr (WEIGHTED)
                    entry.w = wv[u];
                entries[at[u]] = entry;
            }
    }
}

// Describes the job of building the lists of `clouds` clouds of `m` targets and `cloud_total`
// index entries each, in parts of `part_total` entries (`lists` sized for clouds * parts clouds
// of part_total entries).  Returns TPK_ERR_UNSUPPORTED when a span of targets would not fit in
// LDS or entry positions would not fit their fields.
template <int K, bool WEIGHTED, typename IdxT>
int make_list_job(int clouds, int m, int64_t cloud_total, int64_t part_total, const IdxT* idx, const float* weight,
                  const Lists<WEIGHTED>& lists, ListJob<WEIGHTED, IdxT>* job)
{
    *job = ListJob<WEIGHTED, IdxT>{};
    if (clouds <= 0 || m <= 0 || cloud_total <= 0)
        return TPK_OK; // nothing to build: no workgroups
    if (part_total <= 0 || part_total % K != 0)
        return TPK_ERR_INVALID_ARG;
    const int64_t parts = tpk_ceil_div(cloud_total, part_total);
    // (a list holds at most part_total entries: lengths must fit a meta word, positions in the
    // long part 26 bits, byte offsets of entries 32 bits)
    if (part_total >= L_COUNT_MASK || list_capacity(m, part_total) * 8 > 0xffffffffLL || cloud_total > 0x7fffffffLL ||
        clouds * parts > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    // Enough workgroups to occupy the chip; spans of a multiple of 64 targets.
    int splits = static_cast<int>(tpk_ceil_div(256, clouds * parts));
    if (splits > 16)
        splits = 16;
    if (splits < tpk_ceil_div(m, L_MAX_TARGETS))
        splits = static_cast<int>(tpk_ceil_div(m, L_MAX_TARGETS));
    const int span = static_cast<int>(tpk_ceil_div(tpk_ceil_div(m, splits), L_BLOCK) * L_BLOCK);
    splits = static_cast<int>(tpk_ceil_div(m, span));
    if (span > L_MAX_TARGETS || clouds * parts * splits > 0x3fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    job->m = m;
    job->cloud_total = static_cast<int>(cloud_total);
    job->parts = static_cast<int>(parts);
    job->part_total = static_cast<int>(part_total);
    job->splits = splits;
    job->span = span;
    job->workgroups = static_cast<int>(clouds * parts * splits);
    job->idx = idx;
    job->weight = weight;
    job->lists = lists;
    return TPK_OK;
}

template <int K, bool WEIGHTED, typename IdxT>
int launch_build_lists(int clouds, int m, int64_t cloud_total, int64_t part_total, const IdxT* idx,
                       const float* weight, const Lists<WEIGHTED>& lists, hipStream_t s)
{
    ListJob<WEIGHTED, IdxT> job;
    const int st = make_list_job<K, WEIGHTED, IdxT>(clouds, m, cloud_total, part_total, idx, weight, lists, &job);
    if (st != TPK_OK || job.workgroups == 0)
        return st;
    const size_t lds = (2 * static_cast<size_t>(job.span) + 2 * (job.span / L_BLOCK) + G_THREADS) * sizeof(int);
    auto build = build_lists_kernel<K, WEIGHTED, IdxT>;
    const int allowed = allow_lds(build, lds);
    if (allowed != TPK_OK)
        return allowed;
    hipLaunchKernelGGL(build, dim3(static_cast<unsigned>(job.workgroups)), dim3(G_THREADS), lds, s, job);
    return tpk_launch_status();
}

} // namespace
