// Ball query (radius search), dense and packed variable-length ("partial dense") layouts.
//
// Semantics (reference kernels cuda/src/ball_query_gpu.cu:9-52 and :54-95): for every
// query centre the support points of its cloud are visited in index order; the first
// `nsample` whose squared distance passes the radius test are kept, in that order.
//   dense:   test d2 <  r2; unused idx slots repeat the first hit (0 if none), dist -1
//   partial: test d2 <= r2; idx are positions in the packed support array; unused slots -1
//
// Work split: the LANES of a wavefront hold 64 consecutive support points, and the
// wavefront tests them against BQ_Q query centres it keeps in registers as wave-uniform
// values.  A ballot of the radius test gives the hits of one query among the 64 points;
// the hit in lane L lands in output slot (hits so far) + (hits in lanes below L), which is
// exactly the order of a serial scan, and the wavefront stops testing a query once it has
// nsample hits.  A finished query is switched off by setting its radius to -1.  Support
// points stream through LDS in structure-of-arrays tiles shared by the workgroup's
// wavefronts (conflict-free: lane i reads word i).
//
// Packed layout: the per-point cloud ids are sorted, so the support range of cloud c is
// the equal range of c in batch_x, found by binary search on the device.  A workgroup
// owns a block of consecutive queries; where the block straddles clouds it processes one
// run of equal cloud id at a time.  Nothing is copied to the host.
#include "nn_grid.h"

namespace {

constexpr int BQ_WAVES = 4;
constexpr int BQ_THREADS = BQ_WAVES * TPK_WAVE;
constexpr int BQ_Q = 8;                    // queries per wavefront
constexpr int BQ_BLOCK_Q = BQ_WAVES * BQ_Q; // queries per workgroup
constexpr int BQ_Q_FEW = 2;                // queries per wavefront when the whole call has few queries
constexpr int BQ_TILE = 2048;              // support points per LDS tile (24 KiB)

struct Tile
{
    float x[BQ_TILE];
    float y[BQ_TILE];
    float z[BQ_TILE];
};

// First position in sorted `a[0..len)` whose value is >= v.
__device__ __forceinline__ int64_t lower_bound_i64(const int64_t* __restrict__ a, int64_t len,
                                                   int64_t v)
{
    int64_t lo = 0, hi = len;
    while (lo < hi)
    {
        const int64_t mid = lo + ((hi - lo) >> 1);
        if (a[mid] < v)
            lo = mid + 1;
        else
            hi = mid;
    }
    return lo;
}

// Scan support[s0, s1) for the wavefront's queries.  in_run_mask: bit q set when query q
// of this wavefront takes part.  row0: output row of the wavefront's query 0.
template <bool PARTIAL, int BQ_Q>
__device__ __forceinline__ void scan_run(Tile& tile, const float* __restrict__ support,
                                         int64_t s0, int64_t s1, unsigned in_run_mask,
                                         const float (&qx)[BQ_Q], const float (&qy)[BQ_Q],
                                         const float (&qz)[BQ_Q], float radius2, int nsample,
                                         int64_t row0, int64_t* __restrict__ idx,
                                         float* __restrict__ dist)
{
    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    TPK_WORK_DECL

    float r2q[BQ_Q];   // radius of a live query, -1 once it is finished / not in this run
    int cnt[BQ_Q];     // hits so far
    int64_t first[BQ_Q]; // support index of the first hit (dense padding value)
    int live = 0;
#pragma unroll
    for (int q = 0; q < BQ_Q; ++q)
    {
        const bool on = (in_run_mask >> q) & 1u;
        r2q[q] = on ? radius2 : -1.0f;
        cnt[q] = 0;
        first[q] = 0;
        live += on ? 1 : 0;
    }

    for (int64_t base = s0; base < s1; base += BQ_TILE)
    {
        // Barrier + vote: the previous tile is consumed, and the workgroup stops streaming
        // once every one of its queries is finished.
        if (!__syncthreads_or(live > 0))
            break;
        const int tcnt = static_cast<int>(tpk_min64(BQ_TILE, s1 - base));
        const int tpad = (tcnt + TPK_WAVE - 1) & ~(TPK_WAVE - 1);
        // (the loads of a whole tile are issued before the first LDS write: one memory latency per
        // tile, not one per 256 points)
        constexpr int PER_THREAD = BQ_TILE / BQ_THREADS;
        float px[PER_THREAD], py[PER_THREAD], pz[PER_THREAD];
#pragma unroll
        for (int u = 0; u < PER_THREAD; ++u)
        {
            const int t = min(tid + u * BQ_THREADS, tcnt - 1);
            const float* src = support + (base + t) * 3;
            px[u] = src[0];
            py[u] = src[1];
            pz[u] = src[2];
        }
#pragma unroll
        for (int u = 0; u < PER_THREAD; ++u)
        {
            const int t = tid + u * BQ_THREADS;
            if (t < tpad)
            {
                // Padding: infinitely far away, fails both radius tests.
                const bool real = t < tcnt;
                tile.x[t] = real ? px[u] : __builtin_inff();
                tile.y[t] = real ? py[u] : __builtin_inff();
                tile.z[t] = real ? pz[u] : __builtin_inff();
            }
        }
        __syncthreads();

        if (live > 0)
        {
            for (int k0 = 0; k0 < tpad; k0 += TPK_WAVE)
            {
                const float cx = tile.x[k0 + lane];
                const float cy = tile.y[k0 + lane];
                const float cz = tile.z[k0 + lane];
                const int64_t pos = base + k0 + lane;
                TPK_WORK_ADD(BQ_Q);
#pragma unroll
                for (int q = 0; q < BQ_Q; ++q)
                {
                    const float d = tpk_dist2(qx[q], qy[q], qz[q], cx, cy, cz);
                    const bool hit = PARTIAL ? (d <= r2q[q]) : (d < r2q[q]);
                    const unsigned long long mask = __ballot(hit);
                    if (mask != 0ull)
                    {
                        const int slot = cnt[q] + static_cast<int>(tpk_prefix_count(mask));
                        if (hit && slot < nsample)
                        {
                            const int64_t o = (row0 + q) * nsample + slot;
                            idx[o] = pos;
                            dist[o] = d;
                        }
                        if (cnt[q] == 0)
                            first[q] = base + k0 + __builtin_ctzll(mask);
                        cnt[q] += __builtin_popcountll(mask);
                        if (cnt[q] >= nsample)
                        {
                            cnt[q] = nsample;
                            r2q[q] = -1.0f;
                            --live;
                        }
                    }
                }
                if (live == 0)
                    break;
            }
        }
    }

    TPK_WORK_FLUSH
    // Unused slots.
#pragma unroll
    for (int q = 0; q < BQ_Q; ++q)
    {
        if (!((in_run_mask >> q) & 1u))
            continue;
        const int64_t pad_idx = PARTIAL ? -1 : (cnt[q] > 0 ? first[q] : 0);
        for (int s = cnt[q] + lane; s < nsample; s += TPK_WAVE)
        {
            const int64_t o = (row0 + q) * nsample + s;
            idx[o] = pad_idx;
            dist[o] = -1.0f;
        }
    }
}

// BQ_Q queries per wavefront: 8 amortise the reads of the candidates best; a call with few queries (the usual
// case: a few thousand ball centres) takes 2, so that it still spreads over four wavefronts per SIMD - one
// wavefront per SIMD issues at half the rate.
template <int BQ_Q>
__global__ __launch_bounds__(BQ_THREADS) void ball_query_dense_kernel(
    int n, int m, int blocks_per_cloud, float radius2, int nsample,
    const float* __restrict__ new_xyz, const float* __restrict__ xyz, int64_t* __restrict__ idx,
    float* __restrict__ dist)
{
    __shared__ Tile tile;
    const int cloud = blockIdx.x / blocks_per_cloud;
    const int blk = blockIdx.x - cloud * blocks_per_cloud;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TPK_WAVE);
    const int jq0 = (blk * BQ_WAVES + wave) * BQ_Q; // first query of this wavefront

    new_xyz += static_cast<int64_t>(cloud) * m * 3;
    xyz += static_cast<int64_t>(cloud) * n * 3;

    float qx[BQ_Q], qy[BQ_Q], qz[BQ_Q];
    unsigned in_run = 0;
#pragma unroll
    for (int q = 0; q < BQ_Q; ++q)
    {
        const int j = jq0 + q;
        const bool ok = j < m;
        const int jj = ok ? j : m - 1;
        // wave-uniform values, kept in vector registers (double-rate fp32 arithmetic)
        qx[q] = to_vector_register(new_xyz[jj * 3 + 0]);
        qy[q] = to_vector_register(new_xyz[jj * 3 + 1]);
        qz[q] = to_vector_register(new_xyz[jj * 3 + 2]);
        in_run |= ok ? (1u << q) : 0u;
    }
    scan_run<false, BQ_Q>(tile, xyz, 0, n, in_run, qx, qy, qz, radius2, nsample,
                          static_cast<int64_t>(cloud) * m + jq0, idx, dist);
}

__global__ __launch_bounds__(BQ_THREADS) void ball_query_partial_kernel(
    int64_t size_x, int64_t size_y, float radius2, int nsample, const float* __restrict__ x,
    const float* __restrict__ y, const int64_t* __restrict__ batch_x,
    const int64_t* __restrict__ batch_y, int64_t* __restrict__ idx, float* __restrict__ dist)
{
    __shared__ Tile tile;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TPK_WAVE);
    const int64_t block_q0 = static_cast<int64_t>(blockIdx.x) * BQ_BLOCK_Q;
    const int64_t block_q1 = tpk_min64(block_q0 + BQ_BLOCK_Q, size_y);
    const int64_t jq0 = block_q0 + wave * BQ_Q;

    float qx[BQ_Q], qy[BQ_Q], qz[BQ_Q];
    int64_t qc[BQ_Q]; // cloud id of each query of this wavefront
#pragma unroll
    for (int q = 0; q < BQ_Q; ++q)
    {
        const int64_t j = jq0 + q;
        const int64_t jj = j < size_y ? j : size_y - 1;
        qx[q] = to_vector_register(y[jj * 3 + 0]);
        qy[q] = to_vector_register(y[jj * 3 + 1]);
        qz[q] = to_vector_register(y[jj * 3 + 2]);
        qc[q] = batch_y[jj];
    }

    // Runs of equal cloud id inside the block (ids are sorted, so runs are contiguous).
    int64_t run_start = block_q0;
    while (run_start < block_q1)
    {
        const int64_t c = batch_y[run_start];
        int64_t run_end = run_start + 1;
        while (run_end < block_q1 && batch_y[run_end] == c)
            ++run_end;

        const int64_t s0 = lower_bound_i64(batch_x, size_x, c);
        const int64_t s1 = lower_bound_i64(batch_x + s0, size_x - s0, c + 1) + s0;

        unsigned in_run = 0;
#pragma unroll
        for (int q = 0; q < BQ_Q; ++q)
        {
            const int64_t j = jq0 + q;
            in_run |= (j >= run_start && j < run_end && qc[q] == c) ? (1u << q) : 0u;
        }
        scan_run<true, BQ_Q>(tile, x, s0, s1, in_run, qx, qy, qz, radius2, nsample, jq0, idx, dist);
        run_start = run_end;
    }
}

} // namespace

extern "C" int tpk_ball_query_dense_f32(int b, int n, int m, float radius, int nsample,
                                        const float* new_xyz, const float* xyz, int64_t* idx,
                                        float* dist, void* stream)
{
    if (b < 0 || n < 0 || m < 0 || nsample < 0)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || m == 0 || nsample == 0)
        return TPK_OK;
    if (!new_xyz || !idx || !dist || (n > 0 && !xyz))
        return TPK_ERR_INVALID_ARG;
    if (static_cast<int64_t>(n) * 3 > 0x7fffffffLL || static_cast<int64_t>(m) * 3 > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    // fewer than four workgroups per compute unit with 8 queries per wavefront: 2 per wavefront
    const bool few = tpk_ceil_div(m, BQ_BLOCK_Q) * b < 1024;
    const int64_t bpc = tpk_ceil_div(m, few ? BQ_WAVES * BQ_Q_FEW : BQ_BLOCK_Q);
    const int64_t blocks = bpc * b;
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const float radius2 = radius * radius; // fp32 product, as the reference kernel forms it
    if (few)
        hipLaunchKernelGGL(ball_query_dense_kernel<BQ_Q_FEW>, dim3(static_cast<unsigned>(blocks)), dim3(BQ_THREADS), 0,
                           tpk_stream(stream), n, m, static_cast<int>(bpc), radius2, nsample, new_xyz, xyz, idx, dist);
    else
        hipLaunchKernelGGL(ball_query_dense_kernel<BQ_Q>, dim3(static_cast<unsigned>(blocks)), dim3(BQ_THREADS), 0,
                           tpk_stream(stream), n, m, static_cast<int>(bpc), radius2, nsample, new_xyz, xyz, idx, dist);
    return tpk_launch_status();
}

extern "C" size_t tpk_ball_query_partial_workspace_bytes(int64_t size_x, int64_t size_y, int nsample)
{
    return tpk_grid_ball_query_workspace_bytes(size_x, size_y, nsample);
}

extern "C" int tpk_ball_query_partial_f32(int64_t size_x, int64_t size_y, float radius,
                                          int nsample, const float* x, const float* y,
                                          const int64_t* batch_x, const int64_t* batch_y,
                                          int64_t* idx, float* dist, void* workspace,
                                          size_t workspace_bytes, void* stream)
{
    if (size_x < 0 || size_y < 0 || nsample < 0)
        return TPK_ERR_INVALID_ARG;
    if (size_y == 0 || nsample == 0)
        return TPK_OK;
    if (!y || !batch_y || !idx || !dist || (size_x > 0 && (!x || !batch_x)))
        return TPK_ERR_INVALID_ARG;
    const int64_t blocks = tpk_ceil_div(size_y, BQ_BLOCK_Q);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const float radius2 = radius * radius;
    if (workspace)
    {
        // Search over curve-ordered cells where it applies; otherwise all pairs.
        const int st = tpk_grid_ball_query_partial(size_x, size_y, radius, radius2, nsample, false, x, y, batch_x, batch_y, idx,
                                                   dist, workspace, workspace_bytes, tpk_stream(stream));
        if (st != TPK_ERR_UNSUPPORTED)
            return st;
    }
    hipLaunchKernelGGL(ball_query_partial_kernel, dim3(static_cast<unsigned>(blocks)),
                       dim3(BQ_THREADS), 0, tpk_stream(stream), size_x, size_y, radius2, nsample,
                       x, y, batch_x, batch_y, idx, dist);
    return tpk_launch_status();
}
