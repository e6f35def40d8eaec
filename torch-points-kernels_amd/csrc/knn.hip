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
#include "nn_grid.h"
#include "topk.h"

namespace {

constexpr int KNN_THREADS = 256;
constexpr int KNN_TILE = 1024; // support points per LDS tile (16 KiB)

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

        for (int c = 0; c < cnt; ++c)
        {
            const float4 p = tile[c];
            const unsigned long long cand = knn_key(tpk_dist2(qx, qy, qz, p.x, p.y, p.z), base + c);
            if (s.admits(cand))
                s.insert(cand);
        }
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
__global__ __launch_bounds__(KNN_THREADS) void pad_sorted_kernel(int64_t slots, int nsample, float limit, bool packed,
                                                                 int64_t* __restrict__ idx, float* __restrict__ dist)
{
    const int64_t o = static_cast<int64_t>(blockIdx.x) * KNN_THREADS + threadIdx.x;
    if (o >= slots)
        return;
    const float d = dist[o];
    if (d < limit)
        return;
    // The first slot of the row: the nearest neighbour, or the empty entry's 0 (also after this
    // kernel has padded it, in the dense layout).
    const int64_t token = packed ? -1 : idx[o - o % nsample];
    if (packed || o % nsample != 0)
        idx[o] = token;
    dist[o] = -1.0f;
}

int pad_sorted(int64_t rows, int nsample, float limit, bool packed, int64_t* idx, float* dist, hipStream_t s)
{
    const int64_t slots = rows * nsample;
    const int64_t blocks = tpk_ceil_div(slots, KNN_THREADS);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(pad_sorted_kernel, dim3(static_cast<unsigned>(blocks)), dim3(KNN_THREADS), 0, s, slots, nsample,
                       limit, packed, idx, dist);
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
                for (int p = 0; p < cnt; ++p)
                {
                    const float4 v = tile[p];
                    const unsigned long long cand =
                        knn_key(tpk_dist2(qx, qy, qz, v.x, v.y, v.z), static_cast<int>(base + p));
                    if (s.admits(cand))
                        s.insert(cand);
                }
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
    return tpk_grid_knn_workspace_bytes(b, m, n);
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
    const int st = nearest_within(b, n, m, nsample, limit, xyz, new_xyz, idx, dist, workspace, workspace_bytes, s);
    if (st != TPK_OK)
        return st;
    return pad_sorted(static_cast<int64_t>(b) * m, nsample, limit, false, idx, dist, s);
}

extern "C" int tpk_ball_query_sorted_partial_f32(int64_t size_x, int64_t size_y, float radius, int nsample,
                                                 const float* x, const float* y, const int64_t* batch_x,
                                                 const int64_t* batch_y, int64_t* idx, float* dist, void* stream)
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
    int st;
    if (nsample <= 4)
        st = launch_nearest_packed<4>(size_x, size_y, nsample, limit, x, y, batch_x, batch_y, idx, dist, s);
    else if (nsample <= 8)
        st = launch_nearest_packed<8>(size_x, size_y, nsample, limit, x, y, batch_x, batch_y, idx, dist, s);
    else if (nsample <= 16)
        st = launch_nearest_packed<16>(size_x, size_y, nsample, limit, x, y, batch_x, batch_y, idx, dist, s);
    else
        st = launch_nearest_packed<KNN_MAX_K>(size_x, size_y, nsample, limit, x, y, batch_x, batch_y, idx, dist, s);
    if (st != TPK_OK)
        return st;
    return pad_sorted(size_y, nsample, limit, true, idx, dist, s);
}
