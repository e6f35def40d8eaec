// k nearest neighbours, dense layout: for every query point the k nearest support points of the
// same cloud, ascending by (squared distance, index).
//
// The reference offers this operator on the CPU only (torch_points_kernels/knn.py:4-18 raises for
// CUDA tensors; cpu/src/knn.cpp:8-59 runs nanoflann per cloud).  Semantics here: squared fp32
// distances evaluated like three_nn's; equal distances keep the lower index first, as the
// reference's three_nn kernel does (cuda/src/interpolate_gpu.cu:9-65) - nanoflann's order among
// exactly equal distances is unspecified.  k must not exceed the number of support points
// (cpu/src/knn.cpp:12-14 raises).
//
// With a workspace, clouds of 512..163840 points are searched over curve-ordered cells
// (nn_grid.hip).  Otherwise all pairs are tested: one lane owns one query and keeps its list in
// registers (topk.h); the support points of the cloud stream through LDS in tiles of float4, read
// by all lanes at the same address.  k above 32 is served in rounds of 32 entries.
#include "ball_cells.h"
#include "nn_grid.h"
#include "topk.h"

namespace {

constexpr int KNN_THREADS = 256;
constexpr int KNN_TILE = 1024; // support points per LDS tile (16 KiB)

constexpr int KNN_GROUP = 8;   // candidates whose distances are formed together

// The `cnt` candidates of an LDS tile (indices base, base + 1, ...) offered to the lane's list.
// Distances are formed KNN_GROUP at a time, so that the LDS reads overlap; the list is only
// touched when the nearest of a group can enter it.
template <int K>
__device__ __forceinline__ void scan_tile(const float4* tile, int cnt, int base, float qx, float qy, float qz,
                                          NearestK<K>& s)
{
    float worst = s.worst();
    int c = 0;
    for (; c + KNN_GROUP <= cnt; c += KNN_GROUP)
    {
        float d[KNN_GROUP];
        float nearest = 0.f;
#pragma unroll
        for (int i = 0; i < KNN_GROUP; ++i)
        {
            const float4 p = tile[c + i];
            d[i] = tpk_dist2(qx, qy, qz, p.x, p.y, p.z);
            nearest = i == 0 ? d[i] : fminf(nearest, d[i]);
        }
        if (nearest <= worst)
        {
#pragma unroll
            for (int i = 0; i < KNN_GROUP; ++i)
            {
                const unsigned long long cand = knn_key(d[i], base + c + i);
                if (s.admits(cand))
                    s.insert(cand);
            }
            worst = s.worst();
        }
    }
    for (; c < cnt; ++c)
    {
        const float4 p = tile[c];
        const unsigned long long cand = knn_key(tpk_dist2(qx, qy, qz, p.x, p.y, p.z), base + c);
        if (s.admits(cand))
            s.insert(cand);
    }
}

// first: number of entries found by earlier rounds; count: entries this round finds (<= K).
template <int K>
__global__ __launch_bounds__(KNN_THREADS) void knn_kernel(
    int n, int m, int k, int first, int count, float limit, int blocks_per_cloud, const float* __restrict__ query,
    const float* __restrict__ support, float* __restrict__ dist2, int64_t* __restrict__ idx)
{
    __shared__ float4 tile[KNN_TILE];

    const int cloud = blockIdx.x / blocks_per_cloud;
    const int blk = blockIdx.x - cloud * blocks_per_cloud;
    query += static_cast<int64_t>(cloud) * n * 3;
    support += static_cast<int64_t>(cloud) * m * 3;
    dist2 += static_cast<int64_t>(cloud) * n * k;
    idx += static_cast<int64_t>(cloud) * n * k;

    const int tid = threadIdx.x;
    const int j = blk * KNN_THREADS + tid;
    const bool real = j < n;
    const int jj = real ? j : n - 1; // lanes past the end shadow the last query and store nothing
    const float qx = query[jj * 3 + 0], qy = query[jj * 3 + 1], qz = query[jj * 3 + 2];
    NearestK<K> s;
    {
        // the last pair of the round before (rounds of one call run one after the other)
        const int64_t at = static_cast<int64_t>(jj) * k + first - 1;
        s.reset(first > 0, first > 0 ? dist2[at] : 0.f, first > 0 ? static_cast<int>(idx[at]) : 0, !real, limit);
    }

    for (int base = 0; base < m; base += KNN_TILE)
    {
        const int cnt = min(KNN_TILE, m - base);
        __syncthreads(); // the previous tile has been consumed by every wave
        for (int t = tid; t < KNN_TILE; t += KNN_THREADS)
        {
            float4 p;
            if (t < cnt)
            {
                const float* src = support + static_cast<int64_t>(base + t) * 3;
                p = make_float4(src[0], src[1], src[2], 0.f);
            }
            else
            {
                // Padding: infinitely far away, with an index no list admits.
                p = make_float4(__builtin_inff(), __builtin_inff(), __builtin_inff(), 0.f);
            }
            tile[t] = p;
        }
        __syncthreads();

        scan_tile<K>(tile, cnt, base, qx, qy, qz, s);
    }

    if (real)
    {
#pragma unroll
        for (int e = 0; e < K; ++e)
            if (e < count)
            {
                dist2[static_cast<int64_t>(j) * k + first + e] = s.dist(e);
                idx[static_cast<int64_t>(j) * k + first + e] = s.index(e);
            }
    }
}

template <int K>
int launch_knn(int b, int n, int m, int k, float limit, const float* query, const float* support, float* dist2,
               int64_t* idx, hipStream_t stream)
{
    const int64_t blocks_per_cloud = tpk_ceil_div(n, KNN_THREADS);
    const int64_t blocks = blocks_per_cloud * b;
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    for (int first = 0; first < k; first += K)
    {
        hipLaunchKernelGGL(knn_kernel<K>, dim3(static_cast<unsigned>(blocks)), dim3(KNN_THREADS), 0, stream, n, m,
                           k, first, k - first < K ? k - first : K, limit, static_cast<int>(blocks_per_cloud), query,
                           support, dist2, idx);
        const int st = tpk_launch_status();
        if (st != TPK_OK)
            return st;
    }
    return TPK_OK;
}

// The k nearest support points closer than `limit` (squared), for every query: search over
// curve-ordered cells where it applies and a workspace is given, otherwise all pairs.
int nearest_within(int b, int n_support, int m_query, int k, float limit, const float* support, const float* query,
                   int64_t* idx, float* dist2, void* workspace, size_t workspace_bytes, hipStream_t s)
{
    if (workspace)
    {
        const int st = tpk_grid_knn(b, m_query, n_support, k, limit, query, support, dist2, idx, workspace,
                                    workspace_bytes, s);
        if (st != TPK_ERR_UNSUPPORTED)
            return st;
    }
    if (k <= 4)
        return launch_knn<4>(b, m_query, n_support, k, limit, query, support, dist2, idx, s);
    if (k <= 8)
        return launch_knn<8>(b, m_query, n_support, k, limit, query, support, dist2, idx, s);
    if (k <= 16)
        return launch_knn<16>(b, m_query, n_support, k, limit, query, support, dist2, idx, s);
    return launch_knn<KNN_MAX_K>(b, m_query, n_support, k, limit, query, support, dist2, idx, s);
}

} // namespace

extern "C" size_t tpk_knn_workspace_bytes(int b, int n_support, int m_query)
{
    return tpk_grid_knn_workspace_bytes(b, m_query, n_support);
}

extern "C" int tpk_knn_f32(int b, int n_support, int m_query, int k, const float* support,
                           const float* query, int64_t* idx, float* dist2, void* workspace,
                           size_t workspace_bytes, void* stream)
{
    if (b < 0 || n_support < 0 || m_query < 0 || k < 0 || k > n_support)
        return TPK_ERR_INVALID_ARG; // (fewer support points than neighbours asked for)
    if (b == 0 || m_query == 0 || k == 0)
        return TPK_OK;
    if (!support || !query || !idx || !dist2)
        return TPK_ERR_INVALID_ARG;
    if (static_cast<int64_t>(n_support) * 3 > 0x7fffffffLL || static_cast<int64_t>(m_query) * 3 > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    return nearest_within(b, n_support, m_query, k, __builtin_inff(), support, query, idx, dist2, workspace,
                          workspace_bytes, tpk_stream(stream));
}

// ---------------------------------------------------------------------------------------------
// Ball query with sorted neighbours: the nsample nearest support points closer than the radius,
// nearest first.  This is what the reference computes for CPU tensors with sort=True
// (cpu/src/neighbors.cpp:8-136 dense, :139-310 packed: nanoflann's radius search, which keeps
// a point when its squared distance is < radius * radius, sorted by distance and cut at max_num)
// and refuses for CUDA tensors (torch_points_kernels/torchpoints.py:152-153, :163-164).  Equal
// distances keep the lower index first (nanoflann sorts by distance only and leaves that open).
// Unused slots: dense - index of the nearest neighbour, or 0 when there is none, distance -1
// (neighbors.cpp:60-61, :88-105); packed - index -1, distance -1 (:248-275).
// ---------------------------------------------------------------------------------------------
namespace {

// Slots the search left empty read (limit, 0); they become the padding of the layout.
// Indices of found neighbours are raised by `add` (packed layout searched cloud by cloud: the
// position of the cloud's first support point).
__global__ __launch_bounds__(KNN_THREADS) void pad_sorted_kernel(int64_t slots, int nsample, float limit, bool packed,
                                                                 int64_t add, int64_t* __restrict__ idx,
                                                                 float* __restrict__ dist)
{
    const int64_t o = static_cast<int64_t>(blockIdx.x) * KNN_THREADS + threadIdx.x;
    if (o >= slots)
        return;
    const float d = dist[o];
    if (d < limit)
    {
        if (add != 0)
            idx[o] += add;
        return;
    }
    // The first slot of the row: the nearest neighbour, or the empty entry's 0 (also after this
    // kernel has padded it, in the dense layout).
    const int64_t token = packed ? -1 : idx[o - o % nsample];
    if (packed || o % nsample != 0)
        idx[o] = token;
    dist[o] = -1.0f;
}

int pad_sorted(int64_t rows, int nsample, float limit, bool packed, int64_t add, int64_t* idx, float* dist,
               hipStream_t s)
{
    const int64_t slots = rows * nsample;
    const int64_t blocks = tpk_ceil_div(slots, KNN_THREADS);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(pad_sorted_kernel, dim3(static_cast<unsigned>(blocks)), dim3(KNN_THREADS), 0, s, slots, nsample,
                       limit, packed, add, idx, dist);
    return tpk_launch_status();
}

__device__ __forceinline__ int64_t first_not_below(const int64_t* __restrict__ a, int64_t n, int64_t v)
{
    int64_t lo = 0, hi = n;
    while (lo < hi)
    {
        const int64_t mid = (lo + hi) >> 1;
        if (a[mid] < v)
            lo = mid + 1;
        else
            hi = mid;
    }
    return lo;
}

// Packed layout, all pairs: one lane owns one query.  The queries of a workgroup are consecutive,
// so they belong to a few clouds (the cloud ids are sorted); for each of those clouds its support
// points stream through LDS and the lanes of that cloud's queries scan them.
template <int K>
__global__ __launch_bounds__(KNN_THREADS) void nearest_packed_kernel(
    int64_t size_x, int64_t size_y, int nsample, int first, int count, float limit, const float* __restrict__ x,
    const float* __restrict__ y, const int64_t* __restrict__ batch_x, const int64_t* __restrict__ batch_y,
    int64_t* __restrict__ idx, float* __restrict__ dist)
{
    __shared__ float4 tile[KNN_TILE];

    const int tid = threadIdx.x;
    const int64_t q0 = static_cast<int64_t>(blockIdx.x) * KNN_THREADS;
    const int64_t q1 = tpk_min64(q0 + KNN_THREADS, size_y);
    const int64_t j = q0 + tid;
    const bool real = j < size_y;
    const int64_t jj = real ? j : size_y - 1;
    const float qx = y[jj * 3 + 0], qy = y[jj * 3 + 1], qz = y[jj * 3 + 2];
    const int64_t mine = batch_y[jj];
    NearestK<K> s;
    {
        const int64_t at = jj * nsample + first - 1;
        s.reset(first > 0, first > 0 ? dist[at] : 0.f, first > 0 ? static_cast<int>(idx[at]) : 0, !real, limit);
    }

    int64_t run_start = q0;
    while (run_start < q1) // the same runs for every lane of the workgroup
    {
        const int64_t c = batch_y[run_start];
        const int64_t run_end = tpk_min64(q1, q0 + first_not_below(batch_y + q0, q1 - q0, c + 1));
        const int64_t s0 = first_not_below(batch_x, size_x, c);
        const int64_t s1 = s0 + first_not_below(batch_x + s0, size_x - s0, c + 1);
        const bool in_run = real && mine == c;
        for (int64_t base = s0; base < s1; base += KNN_TILE)
        {
            const int cnt = static_cast<int>(tpk_min64(KNN_TILE, s1 - base));
            __syncthreads(); // the previous tile has been consumed by every wave
            for (int t = tid; t < cnt; t += KNN_THREADS)
            {
                const float* src = x + (base + t) * 3;
                tile[t] = make_float4(src[0], src[1], src[2], 0.f);
            }
            __syncthreads();
            if (in_run)
                scan_tile<K>(tile, cnt, static_cast<int>(base), qx, qy, qz, s);
        }
        run_start = run_end > run_start ? run_end : run_start + 1;
    }

    if (real)
    {
#pragma unroll
        for (int e = 0; e < K; ++e)
            if (e < count)
            {
                dist[j * nsample + first + e] = s.dist(e);
                idx[j * nsample + first + e] = s.index(e);
            }
    }
}

template <int K>
int launch_nearest_packed(int64_t size_x, int64_t size_y, int nsample, float limit, const float* x, const float* y,
                          const int64_t* batch_x, const int64_t* batch_y, int64_t* idx, float* dist, hipStream_t s)
{
    const int64_t blocks = tpk_ceil_div(size_y, KNN_THREADS);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    for (int first = 0; first < nsample; first += K)
    {
        hipLaunchKernelGGL(nearest_packed_kernel<K>, dim3(static_cast<unsigned>(blocks)), dim3(KNN_THREADS), 0, s, size_x,
                           size_y, nsample, first, nsample - first < K ? nsample - first : K, limit, x, y, batch_x,
                           batch_y, idx, dist);
        const int st = tpk_launch_status();
        if (st != TPK_OK)
            return st;
    }
    return TPK_OK;
}

} // namespace

extern "C" size_t tpk_ball_query_sorted_dense_workspace_bytes(int b, int n, int m)
{
    // up to 64 neighbours: one wavefront per query over the ordered support points; more: the lists
    // of the k-nearest search, which orders both sets
    const size_t waves = tpk_grid_ball_sorted_workspace_bytes(b, n), lists = tpk_grid_knn_workspace_bytes(b, m, n);
    return waves > lists ? waves : lists;
}

extern "C" int tpk_ball_query_sorted_dense_f32(int b, int n, int m, float radius, int nsample, const float* new_xyz,
                                               const float* xyz, int64_t* idx, float* dist, void* workspace,
                                               size_t workspace_bytes, void* stream)
{
    if (b < 0 || n < 0 || m < 0 || nsample < 0)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || m == 0 || nsample == 0)
        return TPK_OK;
    if (!new_xyz || !idx || !dist || (n > 0 && !xyz))
        return TPK_ERR_INVALID_ARG;
    if (static_cast<int64_t>(n) * 3 > 0x7fffffffLL || static_cast<int64_t>(m) * 3 > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipStream_t s = tpk_stream(stream);
    const float limit = radius * radius; // fp32 product (cpu/src/neighbors.cpp:19)
    {
        // clouds that fit in LDS, up to 64 neighbours: buckets of cells built by every workgroup, no workspace
        const int cells = tpk_cells_ball_query_dense(b, n, m, radius, limit, nsample, true, new_xyz, xyz, idx, dist, s);
        if (cells != TPK_ERR_UNSUPPORTED)
            return cells; // (padding included)
    }
    if (workspace)
    {
        const int direct = tpk_grid_ball_sorted(b, m, n, nsample, limit, false, 0, new_xyz, xyz, dist, idx, workspace,
                                                workspace_bytes, s);
        if (direct != TPK_ERR_UNSUPPORTED)
            return direct; // (padding included)
    }
    const int st = nearest_within(b, n, m, nsample, limit, xyz, new_xyz, idx, dist, workspace, workspace_bytes, s);
    if (st != TPK_OK)
        return st;
    return pad_sorted(static_cast<int64_t>(b) * m, nsample, limit, false, 0, idx, dist, s);
}

namespace {

constexpr int NP_MAX_CLOUDS = 1024; // cloud ids served cloud by cloud; larger ids: all pairs in one launch

// ranges[c] / ranges[NP_MAX_CLOUDS + 1 + c]: position of the first support point / query with
// cloud id >= c, for c = 0 .. NP_MAX_CLOUDS.
__global__ __launch_bounds__(KNN_THREADS) void cloud_ranges_kernel(int64_t size_x, int64_t size_y,
                                                                   const int64_t* __restrict__ batch_x,
                                                                   const int64_t* __restrict__ batch_y,
                                                                   int64_t* __restrict__ ranges)
{
    const int c = blockIdx.x * KNN_THREADS + threadIdx.x;
    if (c > NP_MAX_CLOUDS)
        return;
    ranges[c] = first_not_below(batch_x, size_x, c);
    ranges[NP_MAX_CLOUDS + 1 + c] = first_not_below(batch_y, size_y, c);
}

int nearest_packed(int64_t size_x, int64_t size_y, int nsample, float limit, const float* x, const float* y,
                   const int64_t* batch_x, const int64_t* batch_y, int64_t* idx, float* dist, hipStream_t s)
{
    if (nsample <= 4)
        return launch_nearest_packed<4>(size_x, size_y, nsample, limit, x, y, batch_x, batch_y, idx, dist, s);
    if (nsample <= 8)
        return launch_nearest_packed<8>(size_x, size_y, nsample, limit, x, y, batch_x, batch_y, idx, dist, s);
    if (nsample <= 16)
        return launch_nearest_packed<16>(size_x, size_y, nsample, limit, x, y, batch_x, batch_y, idx, dist, s);
    return launch_nearest_packed<KNN_MAX_K>(size_x, size_y, nsample, limit, x, y, batch_x, batch_y, idx, dist, s);
}

constexpr size_t NP_RANGES_BYTES = (2 * (NP_MAX_CLOUDS + 1) * sizeof(int64_t) + 255) / 256 * 256;
constexpr int64_t NP_GRID_POINTS = 163840; // largest cloud the search over cells takes

} // namespace

// The workspace lets clouds of 512..163840 support points be searched over curve-ordered cells, one
// cloud after the other (up to 64 neighbours: one wavefront per query; more: the k-nearest lists,
// which also want 512 queries or more); the call then waits for the stream once, to read the
// clouds' ranges.
extern "C" size_t tpk_ball_query_sorted_partial_workspace_bytes(int64_t size_x, int64_t size_y)
{
    if (size_x < 512 || size_y < 1)
        return 0;
    const int most_x = static_cast<int>(tpk_min64(size_x, NP_GRID_POINTS));
    const size_t lists = tpk_grid_knn_workspace_bytes(1, static_cast<int>(tpk_min64(size_y, NP_GRID_POINTS)), most_x);
    const size_t waves = tpk_grid_ball_sorted_workspace_bytes(1, most_x);
    const size_t grid = waves > lists ? waves : lists;
    // (up to 64 neighbours the packed array is searched as a whole, bins of windows of consecutive rows: no wait)
    const size_t bins = tpk_grid_ball_query_workspace_bytes(size_x, size_y, TPK_WAVE);
    const size_t cloudwise = grid ? NP_RANGES_BYTES + grid : 0;
    return bins > cloudwise ? bins : cloudwise;
}

extern "C" int tpk_ball_query_sorted_partial_f32(int64_t size_x, int64_t size_y, float radius, int nsample,
                                                 const float* x, const float* y, const int64_t* batch_x,
                                                 const int64_t* batch_y, int64_t* idx, float* dist, void* workspace,
                                                 size_t workspace_bytes, void* stream)
{
    if (size_x < 0 || size_y < 0 || nsample < 0)
        return TPK_ERR_INVALID_ARG;
    if (size_y == 0 || nsample == 0)
        return TPK_OK;
    if (!y || !batch_y || !idx || !dist || (size_x > 0 && (!x || !batch_x)))
        return TPK_ERR_INVALID_ARG;
    if (size_x > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipStream_t s = tpk_stream(stream);
    const float limit = radius * radius; // fp32 product (cpu/src/neighbors.cpp:153)
    const size_t wanted = tpk_ball_query_sorted_partial_workspace_bytes(size_x, size_y);
    if (!workspace || wanted == 0)
    {
        const int st = nearest_packed(size_x, size_y, nsample, limit, x, y, batch_x, batch_y, idx, dist, s);
        return st != TPK_OK ? st : pad_sorted(size_y, nsample, limit, true, 0, idx, dist, s);
    }
    if (workspace_bytes < wanted || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return TPK_ERR_WORKSPACE;
    if (nsample <= TPK_WAVE)
    {
        // One launch over the whole packed array (windows of consecutive rows, bins of a 16^3 grid per window,
        // the rows of every query's cloud found on the device): no wait for the stream.
        const int st = tpk_grid_ball_query_partial(size_x, size_y, radius, limit, nsample, true, x, y, batch_x, batch_y,
                                                   idx, dist, workspace, workspace_bytes, s);
        if (st != TPK_ERR_UNSUPPORTED)
            return st;
    }

    // Where every cloud starts in both arrays.
    static_assert(NP_MAX_CLOUDS + 1 <= 5 * KNN_THREADS, "one thread per cloud id");
    int64_t* ranges_dev = static_cast<int64_t*>(workspace);
    hipLaunchKernelGGL(cloud_ranges_kernel, dim3(5), dim3(KNN_THREADS), 0, s, size_x, size_y, batch_x, batch_y, ranges_dev);
    int64_t ranges[2 * (NP_MAX_CLOUDS + 1)];
    static_assert(sizeof(ranges) <= TPK_READ_BACK_BYTES, "the cloud ranges fit the pinned buffer");
    const int read = tpk_read_back(ranges, ranges_dev, sizeof(ranges), s);
    if (read != TPK_OK)
        return read;
    const int64_t* rx = ranges;
    const int64_t* ry = ranges + NP_MAX_CLOUDS + 1;
    void* grid_ws = static_cast<char*>(workspace) + NP_RANGES_BYTES;
    const size_t grid_bytes = workspace_bytes - NP_RANGES_BYTES;

    // Queries q0..q1 (one cloud when `points` >= 0: its support points are s0 .. s0 + points).
    auto segment = [&](int64_t q0, int64_t q1, int64_t s0, int64_t points) -> int {
        if (q1 <= q0)
            return TPK_OK;
        const int64_t queries = q1 - q0;
        int64_t* idx_c = idx + q0 * nsample;
        float* dist_c = dist + q0 * nsample;
        int st = TPK_ERR_UNSUPPORTED;
        int64_t add = 0;
        if (points >= 0 && points <= NP_GRID_POINTS && queries <= 0x7fffffffLL)
        {
            // up to 64 neighbours: one wavefront per query over the cloud's ordered support points
            st = tpk_grid_ball_sorted(1, static_cast<int>(queries), static_cast<int>(points), nsample, limit, true, s0,
                                      y + q0 * 3, x + s0 * 3, dist_c, idx_c, grid_ws, grid_bytes, s);
            if (st != TPK_ERR_UNSUPPORTED)
                return st; // (padding included)
        }
        if (points >= 0 && queries <= NP_GRID_POINTS && points <= NP_GRID_POINTS &&
            tpk_grid_knn_workspace_bytes(1, static_cast<int>(queries), static_cast<int>(points)) != 0)
        {
            // search over cells; it numbers the support points from the cloud's first one
            st = tpk_grid_knn(1, static_cast<int>(queries), static_cast<int>(points), nsample, limit, y + q0 * 3,
                              x + s0 * 3, dist_c, idx_c, grid_ws, grid_bytes, s);
            add = s0;
        }
        if (st == TPK_ERR_UNSUPPORTED)
        {
            st = nearest_packed(size_x, queries, nsample, limit, x, y + q0 * 3, batch_x, batch_y + q0, idx_c, dist_c, s);
            add = 0;
        }
        return st != TPK_OK ? st : pad_sorted(queries, nsample, limit, true, add, idx_c, dist_c, s);
    };
    int st = segment(0, ry[0], 0, -1); // negative cloud ids, if any: all pairs
    for (int c = 0; c < NP_MAX_CLOUDS && st == TPK_OK; ++c)
        st = segment(ry[c], ry[c + 1], rx[c], rx[c + 1] - rx[c]);
    if (st == TPK_OK)
        st = segment(ry[NP_MAX_CLOUDS], size_y, 0, -1); // cloud ids of NP_MAX_CLOUDS and more: all pairs
    return st;
}
