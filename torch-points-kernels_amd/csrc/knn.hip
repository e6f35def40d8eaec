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
    int n, int m, int k, int first, int count, int blocks_per_cloud, const float* __restrict__ query,
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
        s.reset(first > 0, first > 0 ? dist2[at] : 0.f, first > 0 ? static_cast<int>(idx[at]) : 0, !real);
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
int launch_knn(int b, int n, int m, int k, const float* query, const float* support, float* dist2,
               int64_t* idx, hipStream_t stream)
{
    const int64_t blocks_per_cloud = tpk_ceil_div(n, KNN_THREADS);
    const int64_t blocks = blocks_per_cloud * b;
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    for (int first = 0; first < k; first += K)
    {
        hipLaunchKernelGGL(knn_kernel<K>, dim3(static_cast<unsigned>(blocks)), dim3(KNN_THREADS), 0, stream, n, m,
                           k, first, k - first < K ? k - first : K, static_cast<int>(blocks_per_cloud), query,
                           support, dist2, idx);
        const int st = tpk_launch_status();
        if (st != TPK_OK)
            return st;
    }
    return TPK_OK;
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
    hipStream_t s = tpk_stream(stream);
    if (workspace)
    {
        // Search over curve-ordered cells where it applies; otherwise all pairs.
        const int st = tpk_grid_knn(b, m_query, n_support, k, query, support, dist2, idx, workspace,
                                    workspace_bytes, s);
        if (st != TPK_ERR_UNSUPPORTED)
            return st;
    }
    if (k <= 4)
        return launch_knn<4>(b, m_query, n_support, k, query, support, dist2, idx, s);
    if (k <= 8)
        return launch_knn<8>(b, m_query, n_support, k, query, support, dist2, idx, s);
    if (k <= 16)
        return launch_knn<16>(b, m_query, n_support, k, query, support, dist2, idx, s);
    return launch_knn<KNN_MAX_K>(b, m_query, n_support, k, query, support, dist2, idx, s);
}
