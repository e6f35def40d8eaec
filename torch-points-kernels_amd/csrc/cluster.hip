// Clusters grown over a neighbour matrix: the device side of grow_proximity / region_grow
// (reference: torch_points_kernels/cluster.py:9-45, where the matrix is copied to the host and a
// numba routine walks it).
//
// The reference takes the points in index order; an unseen point i starts a cluster that
// receives every unseen point reachable from i along rows of the matrix (a row lists the
// neighbours of its point and ends at the first -1).  Rows cut at nsample entries make the
// relation one-directional, so these are not connected components.  What decides the cluster of
// a point v is the smallest index among the points that reach v (v included): that point is
// reached by no smaller one, so it is unseen at its turn and starts a cluster, and every other
// point that reaches v comes later.  The labels are therefore the fixed point of
//     label[v] = min(v, label[u] for every row u that lists v),
// which is found here in two steps.  Points that list each other (all of them, where no row was
// cut) are first merged into groups by union-find: they reach and are reached by the same points.
// Then repeated sweeps hand labels from group to group with atomicMin, shortened by following
// the label of a label (valid because reaching is transitive).  Without the merging a label
// would cross a cluster one row per sweep.  Clusters are numbered by their first point, as in
// the reference, and those below min_cluster_size are dropped.
//
// Members inside a cluster, two orders:
//   TPK_MEMBERS_AS_REFERENCE  the order in which the reference's stack walk appends them.  The walk
//       of a cluster never leaves it (anything a member reaches outside was seen by an earlier
//       cluster), so the clusters are walked independently, one wavefront each; inside a cluster
//       the walk is the reference's, serial, one expanded point per step.
//   TPK_MEMBERS_BY_INDEX      ascending index: a stable radix sort (rocPRIM) of the point numbers by
//       cluster number.  Everything is data-parallel.
//
// The entry point blocks the host: the number of sweeps and the sizes of the outputs depend on
// the data.
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>

#include "tpk_device.h"

namespace
{

constexpr int CL_THREADS = 256;
constexpr int CL_ROW_LANES = 16; // lanes that share one row of the matrix in a sweep
constexpr int CL_SWEEPS = 8;     // sweeps enqueued between two looks at the `changed` flags
constexpr int CL_FOLLOW = 16;    // labels followed per point and sweep
constexpr int64_t CL_MAX_POINTS = (int64_t)1 << 30;

using u64 = unsigned long long;

__global__ void __launch_bounds__(CL_THREADS)
    cluster_init_kernel(int n, int words, int* parent, int* label, int* size, int* handed, unsigned* mutual, int* changed)
{
    const int v = blockIdx.x * CL_THREADS + threadIdx.x;
    if (v < n)
    {
        parent[v] = v;
        label[v] = v;
        size[v] = 0;
        handed[v] = n; // nothing handed over yet
        for (int w = 0; w < words; ++w)
            mutual[(int64_t)v * words + w] = 0;
    }
    if (v < CL_SWEEPS)
        changed[v] = 0;
}

__global__ void __launch_bounds__(CL_THREADS) cluster_clear_kernel(int* changed)
{
    if (threadIdx.x < CL_SWEEPS)
        changed[threadIdx.x] = 0;
}

// The part of a row that counts: lanes of a group of CL_ROW_LANES hold consecutive entries (-1
// beyond the row's width); returns how many of them come before the row's end and whether the
// row ends in this chunk.
__device__ __forceinline__ int entries_before_end(int64_t nei, int shift, bool* row_ends)
{
    const unsigned ends = (unsigned)(__ballot(nei == -1) >> shift) & 0xffffu;
    *row_ends = ends != 0;
    return ends ? __builtin_ctz(ends) : CL_ROW_LANES;
}

// Bit j of a point's mask: entry j of its row is a point whose own row lists this point back.
// The smallest such point below u becomes u's first parent (a plain store: only u's lanes
// write parent[u] in this kernel), which leaves far fewer trees for the merge sweeps to hang.
__global__ void __launch_bounds__(CL_THREADS)
    cluster_mutual_kernel(int n, int nsample, int words, const int64_t* __restrict__ neighbours, unsigned* mutual,
                          int* parent)
{
    const int64_t t = (int64_t)blockIdx.x * CL_THREADS + threadIdx.x;
    const int64_t point = t / CL_ROW_LANES;
    const int g = (int)(t % CL_ROW_LANES);
    if (point >= n)
        return; // the whole group of lanes leaves together
    const int u = (int)point;
    const int shift = (int)(tpk_lane_id() & (TPK_WAVE - CL_ROW_LANES)); // first lane of this row's group
    int lowest = u;
    for (int first = 0; first < nsample; first += CL_ROW_LANES)
    {
        const int j = first + g;
        const int64_t nei = j < nsample ? neighbours[(int64_t)u * nsample + j] : -1;
        bool row_ends;
        const int valid = entries_before_end(nei, shift, &row_ends);
        bool back = false;
        if (g < valid && nei >= 0 && nei < n && nei != u)
        {
            const int64_t* other = neighbours + nei * nsample;
            for (int i = 0; i < nsample; ++i)
            {
                const int64_t e = other[i];
                if (e == -1)
                    break;
                if (e == u)
                {
                    back = true;
                    break;
                }
            }
        }
        const unsigned bits = (unsigned)(__ballot(back) >> shift) & 0xffffu;
        if (g == 0 && bits)
            atomicOr(&mutual[(int64_t)u * words + (first >> 5)], bits << (first & 31));
        if (back && (int)nei < lowest)
            lowest = (int)nei;
        if (row_ends)
            break;
    }
    // minimum over the group's lanes (the lanes of a group are together again here)
    for (int step = 1; step < CL_ROW_LANES; step <<= 1)
        lowest = min(lowest, __shfl_xor(lowest, step, CL_ROW_LANES));
    if (g == 0 && lowest < u)
        parent[u] = lowest;
}

__device__ __forceinline__ int find_root(const int* parent, int v)
{
    for (int up = parent[v]; up < v; up = parent[v])
        v = up;
    return v;
}

// Points that list each other reach the same points and are reached by the same points, so they
// can be merged outright: union-find over the mutual entries (the tree of the larger root is hung
// under the smaller root), repeated until no tree is hung any more.  Each mutual pair is handled
// from its smaller point.
__global__ void __launch_bounds__(CL_THREADS)
    cluster_merge_kernel(int n, int nsample, int words, const int64_t* __restrict__ neighbours,
                         const unsigned* __restrict__ mutual, int* parent, int* changed, int sweep)
{
    if (sweep > 0 && changed[sweep - 1] == 0)
        return;
    const int64_t t = (int64_t)blockIdx.x * CL_THREADS + threadIdx.x;
    const int64_t point = t / CL_ROW_LANES;
    const int g = (int)(t % CL_ROW_LANES);
    if (point >= n)
        return;
    const int u = (int)point;
    const int mine = find_root(parent, u);
    bool hung = false;
    for (int j = g; j < nsample; j += CL_ROW_LANES)
    {
        if (((mutual[(int64_t)u * words + (j >> 5)] >> (j & 31)) & 1u) == 0)
            continue;
        const int nei = (int)neighbours[(int64_t)u * nsample + j];
        if (nei < u)
            continue;
        const int theirs = find_root(parent, nei);
        if (theirs != mine)
        {
            // Many entries join the same two trees; only while the higher root still is a root
            // is it worth an atomic on that one address.  Otherwise another entry has hung it
            // meanwhile and this pair is looked at again in the next sweep.
            const int low = min(mine, theirs), high = max(mine, theirs);
            if (__hip_atomic_load(&parent[high], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == high)
                hung |= atomicMin(&parent[high], low) > low;
            else
                hung = true;
        }
    }
    if (g == 0 && mine < parent[u])
        atomicMin(&parent[u], mine);
    if (hung)
        changed[sweep] = 1;
}

// Shortens the trees before a merge sweep: every point moves its parent a few steps up (only
// the point's own thread writes its entry in this kernel).
__global__ void __launch_bounds__(CL_THREADS) cluster_jump_kernel(int n, int* parent, const int* changed, int sweep)
{
    if (sweep > 0 && changed[sweep - 1] == 0)
        return;
    const int v = blockIdx.x * CL_THREADS + threadIdx.x;
    if (v >= n)
        return;
    const int first = parent[v];
    int p = first;
    for (int step = 0; step < CL_FOLLOW; ++step)
    {
        const int up = parent[p];
        if (up >= p)
            break;
        p = up;
    }
    if (p < first)
        parent[v] = p;
}

// parent[v] becomes the smallest point of v's merged group.
__global__ void __launch_bounds__(CL_THREADS) cluster_flatten_kernel(int n, int* parent)
{
    const int v = blockIdx.x * CL_THREADS + threadIdx.x;
    if (v < n)
    {
        const int root = find_root(parent, v);
        if (root < parent[v])
            atomicMin(&parent[v], root);
    }
}

// One sweep over all entries.  Labels live at the first point of every merged group (`group`):
// label[group[v]] is a point that reaches v.  Every point hands the smallest label it can find by
// following its own (label of the group of the label ...) to the groups of the points its row
// lists - unless that is what it handed over last time (`handed`): labels only fall, so those
// groups still hold it or less.  Sweep `sweep` of a batch does nothing when the one before
// changed nothing, so a batch can be enqueued without looking at the flags in between.
__global__ void __launch_bounds__(CL_THREADS)
    cluster_sweep_kernel(int n, int nsample, const int64_t* __restrict__ neighbours, const int* __restrict__ group,
                         int* label, int* handed, int* changed, int sweep)
{
    if (sweep > 0 && changed[sweep - 1] == 0)
        return;
    const int64_t t = (int64_t)blockIdx.x * CL_THREADS + threadIdx.x;
    const int64_t point = t / CL_ROW_LANES;
    const int g = (int)(t % CL_ROW_LANES);
    if (point >= n)
        return; // the whole group of lanes leaves together
    const int u = (int)point;
    const int shift = (int)(tpk_lane_id() & (TPK_WAVE - CL_ROW_LANES)); // first lane of this row's group
    const int home = group[u];
    const int mine = label[home];
    const int before = handed[u];
    // A few steps upstream: any point found this way reaches u, and storing it makes the next
    // sweep's steps that much longer, so chains shorten geometrically.
    int root = mine;
    for (int step = 0; step < CL_FOLLOW; ++step)
    {
        const int up = label[group[root]];
        if (up >= root)
            break;
        root = up;
    }
    if (root == before)
        return;
    bool lowered = false;
    if (g == 0)
    {
        handed[u] = root;
        if (root < mine)
            lowered = atomicMin(&label[home], root) > root;
    }
    for (int first = 0; first < nsample; first += CL_ROW_LANES)
    {
        const int j = first + g;
        const int64_t nei = j < nsample ? neighbours[(int64_t)u * nsample + j] : -1;
        bool row_ends;
        const int valid = entries_before_end(nei, shift, &row_ends);
        if (g < valid && nei >= 0 && nei < n)
        {
            const int there = group[nei];
            if (there != home && label[there] > root)
                lowered |= atomicMin(&label[there], root) > root;
        }
        if (row_ends)
            break;
    }
    if (lowered)
        changed[sweep] = 1;
}

// Every point takes the label of its group.  Labels of other points than the first of a group
// are read by nobody, so this can be done in place.
__global__ void __launch_bounds__(CL_THREADS) cluster_spread_kernel(int n, const int* __restrict__ group, int* label)
{
    const int v = blockIdx.x * CL_THREADS + threadIdx.x;
    if (v < n && group[v] != v)
        label[v] = label[group[v]];
}

// Members per cluster, counted at the cluster's first point.  Lanes with the same label add once.
__global__ void __launch_bounds__(CL_THREADS) cluster_count_kernel(int n, const int* __restrict__ label, int* size)
{
    const int v = blockIdx.x * CL_THREADS + threadIdx.x;
    const int l = v < n ? label[v] : -1;
    u64 left = __ballot(l >= 0);
    while (left)
    {
        const int leader = __builtin_ctzll(left);
        const int which = __builtin_amdgcn_readlane(l, leader);
        const u64 same = __ballot(l == which);
        if ((int)tpk_lane_id() == leader)
            atomicAdd(&size[which], __builtin_popcountll(same));
        left &= ~same;
    }
}

// Scan input: for the first point of a kept cluster (1 << 32 | members), else 0; one more zero
// at the end so that the exclusive scan also gives the totals.
__global__ void __launch_bounds__(CL_THREADS)
    cluster_kept_kernel(int n, int min_size, const int* __restrict__ label, const int* __restrict__ size, u64* packed)
{
    const int v = blockIdx.x * CL_THREADS + threadIdx.x;
    if (v > n)
        return;
    u64 p = 0;
    if (v < n && label[v] == v && size[v] >= min_size)
        p = ((u64)1 << 32) | (unsigned)size[v];
    packed[v] = p;
}

// From the scan: number and first output position of every kept cluster.
__global__ void __launch_bounds__(CL_THREADS)
    cluster_describe_kernel(int n, const u64* __restrict__ packed, const u64* __restrict__ scanned, int* number,
                            int* seeds, int64_t* starts)
{
    const int v = blockIdx.x * CL_THREADS + threadIdx.x;
    if (v > n)
        return;
    const u64 s = scanned[v];
    const int c = (int)(s >> 32);
    const int64_t at = (int64_t)(s & 0xffffffffu);
    if (v == n)
    {
        starts[c] = at; // totals: one past the last cluster
        return;
    }
    if (packed[v] != 0)
    {
        number[v] = c;
        seeds[c] = v;
        starts[c] = at;
    }
    else
        number[v] = -1;
}

// Sort keys: the number of the point's cluster, `clusters` for points of dropped clusters.
__global__ void __launch_bounds__(CL_THREADS)
    cluster_keys_kernel(int n, int clusters, const int* __restrict__ label, const int* __restrict__ number,
                        unsigned* keys, unsigned* values)
{
    const int v = blockIdx.x * CL_THREADS + threadIdx.x;
    if (v >= n)
        return;
    const int c = number[label[v]];
    keys[v] = c < 0 ? (unsigned)clusters : (unsigned)c;
    values[v] = (unsigned)v;
}

__global__ void __launch_bounds__(CL_THREADS) cluster_widen_kernel(int count, const unsigned* __restrict__ values, int64_t* members)
{
    const int i = blockIdx.x * CL_THREADS + threadIdx.x;
    if (i < count)
        members[i] = values[i];
}

// The reference's walk (cluster.py:15-33), one wavefront per kept cluster: the point taken off
// the stack has its row read by the lanes; the unseen members of the cluster among the entries
// are marked, and appended to the stack and to the cluster in row order.  A member is unseen
// while its label still is the cluster's first point; one compare-and-swap tests and marks it
// (the label becomes the complement), so a point enters once even if a row repeats it, and the
// labels are used up by this kernel.  The stack of a cluster occupies the cluster's own range of
// `stack` (it never holds more than the cluster has members).
__global__ void __launch_bounds__(CL_THREADS)
    cluster_walk_kernel(int n, int nsample, int clusters, const int64_t* __restrict__ neighbours, int* label,
                        const int* __restrict__ seeds, const int64_t* __restrict__ starts, int* stack, int64_t* members)
{
    const int c = blockIdx.x * (CL_THREADS / TPK_WAVE) + threadIdx.x / TPK_WAVE;
    if (c >= clusters)
        return;
    const int lane = (int)tpk_lane_id();
    const int seed = seeds[c];
    const int64_t base = starts[c];
    const int capacity = (int)(starts[c + 1] - base);
    int* my_stack = stack + base;
    int64_t* mine = members + base;
    if (lane == 0)
    {
        label[seed] = ~seed;
        mine[0] = seed;
    }
    int filled = 1, top = 0;
    int k = seed;
    while (true)
    {
        int pushed_last = -1;
        for (int first = 0; first < nsample; first += TPK_WAVE)
        {
            const int j = first + lane;
            const int64_t nei = j < nsample ? neighbours[(int64_t)k * nsample + j] : -1;
            const u64 ends = __ballot(nei == -1);
            const int valid = ends ? __builtin_ctzll(ends) : TPK_WAVE;
            bool take = false;
            if (lane < valid && nei >= 0 && nei < n)
                take = atomicCAS(&label[nei], seed, ~seed) == seed;
            const u64 taken = __ballot(take);
            const int count = __builtin_popcountll(taken);
            if (count > 0 && filled + count <= capacity)
            {
                const int at = (int)tpk_prefix_count(taken);
                if (take)
                {
                    my_stack[top + at] = (int)nei;
                    mine[filled + at] = nei;
                }
                pushed_last = __builtin_amdgcn_readlane((int)nei, 63 - __builtin_clzll(taken));
                top += count;
                filled += count;
            }
            if (ends)
                break;
        }
        if (top == 0)
            break;
        --top;
        if (pushed_last >= 0)
            k = pushed_last;
        else
        {
            __threadfence_block(); // entries written by other lanes in earlier steps
            k = __builtin_amdgcn_readfirstlane(__hip_atomic_load(&my_stack[top], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
        }
    }
}

struct Layout
{
    size_t parent, mutual, label, size, number, seeds, stack, keys_in, keys_out, values_in, values_out, packed, scanned, changed,
        temp, temp_bytes, total;
};

// 32-bit words of a point's mask of mutual entries.
int mask_words(int nsample)
{
    return nsample > 0 ? (nsample + 31) / 32 : 1;
}

size_t aligned(size_t v)
{
    return (v + 255) / 256 * 256;
}

// Temporary storage rocPRIM asks for (the larger of the scan's and the sort's); false when it
// cannot say (no device).
bool temp_bytes(int64_t n, size_t* bytes)
{
    size_t scan = 0, sort = 0;
    u64* p64 = nullptr;
    unsigned* p32 = nullptr;
    if (rocprim::exclusive_scan(nullptr, scan, p64, p64, (u64)0, (size_t)n + 1, rocprim::plus<u64>()) != hipSuccess)
        return false;
    if (rocprim::radix_sort_pairs(nullptr, sort, p32, p32, p32, p32, (size_t)n, 0u, 32u) != hipSuccess)
        return false;
    *bytes = scan > sort ? scan : sort;
    return true;
}

bool layout(int64_t n, int nsample, Layout* l)
{
    size_t temp = 0;
    if (!temp_bytes(n, &temp))
        return false;
    size_t at = 0;
    auto take = [&](size_t bytes) {
        const size_t here = at;
        at += aligned(bytes);
        return here;
    };
    const size_t ints = (size_t)n * 4;
    l->parent = take(ints);
    l->mutual = take(ints * (size_t)mask_words(nsample));
    l->label = take(ints);
    l->size = take(ints);
    l->number = take(ints);
    l->seeds = take(ints);
    l->stack = take(ints);
    l->keys_in = take(ints);
    l->keys_out = take(ints);
    l->values_in = take(ints);
    l->values_out = take(ints);
    l->packed = take(((size_t)n + 1) * 8);
    l->scanned = take(((size_t)n + 1) * 8);
    l->changed = take(CL_SWEEPS * 4);
    l->temp = take(temp);
    l->temp_bytes = temp;
    l->total = at;
    return true;
}

} // namespace

extern "C" size_t tpk_grow_proximity_workspace_bytes(int64_t n, int nsample)
{
    Layout l;
    if (n <= 0 || n > CL_MAX_POINTS || nsample < 0 || !layout(n, nsample, &l))
        return 0;
    return l.total;
}

extern "C" int tpk_grow_proximity(int64_t n, int nsample, const int64_t* neighbours, int64_t min_cluster_size,
                                  int member_order, int64_t* members, int64_t* starts, int64_t* found,
                                  void* workspace, size_t workspace_bytes, void* stream)
{
    if (n < 0 || nsample < 0 || !found || (member_order != TPK_MEMBERS_AS_REFERENCE && member_order != TPK_MEMBERS_BY_INDEX))
        return TPK_ERR_INVALID_ARG;
    found[0] = found[1] = 0;
    if (n == 0)
        return TPK_OK;
    if (!members || !starts || (nsample > 0 && !neighbours))
        return TPK_ERR_INVALID_ARG;
    if (n > CL_MAX_POINTS)
        return TPK_ERR_UNSUPPORTED;
    Layout l;
    if (!layout(n, nsample, &l))
        return TPK_ERR_UNSUPPORTED;
    if (!workspace || workspace_bytes < l.total || (reinterpret_cast<uintptr_t>(workspace) & 255) != 0)
        return TPK_ERR_WORKSPACE;
    hipStream_t s = tpk_stream(stream);
    char* ws = static_cast<char*>(workspace);
    int* parent = reinterpret_cast<int*>(ws + l.parent);
    unsigned* mutual = reinterpret_cast<unsigned*>(ws + l.mutual);
    int* label = reinterpret_cast<int*>(ws + l.label);
    int* size = reinterpret_cast<int*>(ws + l.size);
    int* number = reinterpret_cast<int*>(ws + l.number);
    int* seeds = reinterpret_cast<int*>(ws + l.seeds);
    int* stack = reinterpret_cast<int*>(ws + l.stack);
    unsigned* keys_in = reinterpret_cast<unsigned*>(ws + l.keys_in);
    unsigned* keys_out = reinterpret_cast<unsigned*>(ws + l.keys_out);
    unsigned* values_in = reinterpret_cast<unsigned*>(ws + l.values_in);
    unsigned* values_out = reinterpret_cast<unsigned*>(ws + l.values_out);
    u64* packed = reinterpret_cast<u64*>(ws + l.packed);
    u64* scanned = reinterpret_cast<u64*>(ws + l.scanned);
    int* changed = reinterpret_cast<int*>(ws + l.changed);
    void* temp = ws + l.temp;
    size_t temp_size = l.temp_bytes;

    const int ni = (int)n;
    const unsigned blocks = (unsigned)tpk_ceil_div(n, CL_THREADS);
    const unsigned blocks1 = (unsigned)tpk_ceil_div(n + 1, CL_THREADS);
    const unsigned sweep_blocks = (unsigned)tpk_ceil_div(n * CL_ROW_LANES, CL_THREADS);
    const int min_size = (int)(min_cluster_size > n ? n + 1 : (min_cluster_size < 0 ? 0 : min_cluster_size));

    const int words = mask_words(nsample);
    // `stack` serves the sweeps as `handed` first
    cluster_init_kernel<<<blocks, CL_THREADS, 0, s>>>(ni, words, parent, label, size, stack, mutual, changed);
    if (nsample > 0)
    {
        // Enqueues batches of sweeps until the last sweep of a batch reports no change.
        auto until_stable = [&](auto&& launch) -> hipError_t {
            while (true)
            {
                for (int sweep = 0; sweep < CL_SWEEPS; ++sweep)
                    launch(sweep);
                int last = 0;
                const hipError_t e = static_cast<hipError_t>(tpk_read_back(&last, changed + CL_SWEEPS - 1, sizeof(int), s));
                cluster_clear_kernel<<<1, CL_THREADS, 0, s>>>(changed);
                if (e != hipSuccess || last == 0)
                    return e;
            }
        };
        cluster_mutual_kernel<<<sweep_blocks, CL_THREADS, 0, s>>>(ni, nsample, words, neighbours, mutual, parent);
        hipError_t e = until_stable([&](int sweep) {
            cluster_jump_kernel<<<blocks, CL_THREADS, 0, s>>>(ni, parent, changed, sweep);
            cluster_merge_kernel<<<sweep_blocks, CL_THREADS, 0, s>>>(ni, nsample, words, neighbours, mutual, parent, changed, sweep);
        });
        if (e != hipSuccess)
            return (int)e;
        cluster_flatten_kernel<<<blocks, CL_THREADS, 0, s>>>(ni, parent);
        e = until_stable([&](int sweep) {
            cluster_sweep_kernel<<<sweep_blocks, CL_THREADS, 0, s>>>(ni, nsample, neighbours, parent, label, stack, changed, sweep);
        });
        if (e != hipSuccess)
            return (int)e;
        cluster_spread_kernel<<<blocks, CL_THREADS, 0, s>>>(ni, parent, label);
    }
    cluster_count_kernel<<<blocks, CL_THREADS, 0, s>>>(ni, label, size);
    cluster_kept_kernel<<<blocks1, CL_THREADS, 0, s>>>(ni, min_size, label, size, packed);
    hipError_t e = rocprim::exclusive_scan(temp, temp_size, packed, scanned, (u64)0, (size_t)n + 1, rocprim::plus<u64>(), s);
    if (e != hipSuccess)
        return (int)e;
    cluster_describe_kernel<<<blocks1, CL_THREADS, 0, s>>>(ni, packed, scanned, number, seeds, starts);
    u64 totals = 0;
    e = static_cast<hipError_t>(tpk_read_back(&totals, scanned + n, sizeof(u64), s));
    if (e != hipSuccess)
        return (int)e;
    const int clusters = (int)(totals >> 32);
    const int kept_points = (int)(totals & 0xffffffffu);
    found[0] = clusters;
    found[1] = kept_points;
    if (clusters == 0)
        return tpk_launch_status();
    if (member_order == TPK_MEMBERS_BY_INDEX)
    {
        cluster_keys_kernel<<<blocks, CL_THREADS, 0, s>>>(ni, clusters, label, number, keys_in, values_in);
        const unsigned bits = 32u - (unsigned)__builtin_clz((unsigned)clusters);
        temp_size = l.temp_bytes;
        e = rocprim::radix_sort_pairs(temp, temp_size, keys_in, keys_out, values_in, values_out, (size_t)n, 0u, bits, s);
        if (e != hipSuccess)
            return (int)e;
        cluster_widen_kernel<<<(unsigned)tpk_ceil_div(kept_points, CL_THREADS), CL_THREADS, 0, s>>>(kept_points, values_out, members);
    }
    else
    {
        const int per_block = CL_THREADS / TPK_WAVE;
        cluster_walk_kernel<<<(unsigned)tpk_ceil_div(clusters, per_block), CL_THREADS, 0, s>>>(
            ni, nsample, clusters, neighbours, label, seeds, starts, stack, members);
    }
    return tpk_launch_status();
}
