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
#include "ball_cells.h"
#include "nn_grid.h"
#include "topk.h"

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

// ---------------------------------------------------------------------------------------
// Dense layout over cells: clouds of BQC_MIN_POINTS .. BQC_MAX_POINTS support points.
//
// Testing every support point costs n / 64 steps per query whatever the radius.  Here a workgroup
// of 16 wavefronts first hangs its cloud into 4096 buckets in LDS: space is cut into cells 0.7
// radii wide, cell (i, j, k) belongs to bucket (i mod 16, j mod 16, k mod 16), and every point
// is pushed onto its bucket's chain (one LDS exchange per point; the points stay in index order
// in LDS and carry the link to the next one).  No bounding box, no counting, no sorting: two
// barriers, and a far outlier or a tiny radius costs nothing.  All workgroups of a cloud repeat
// this (the cloud comes from the L2), which is cheaper than a launch that does it once.  Then
// every wavefront answers queries, one at a time: [q - r, q + r] touches at most four cells per
// axis (five when an end of the interval falls within rounding of a cell's edge), lane c takes
// cell c and walks its bucket's chain, all lanes in step.  Points of other cells that share
// the bucket fail the distance test like any other; no two cells of one query share a bucket.
// A candidate with d2 < radius^2 is a hit; the hits (at most 64) are ranked by index and written
// in ascending index order, which is what the scan in index order produces
// (cuda/src/ball_query_gpu.cu:9-52).  A query with more than 64 hits, with chains longer than
// BQC_MAX_CHAIN in all, or whose interval is wider than five cells (coordinates so large that
// rounding dwarfs the radius) is answered by that scan itself, 64 points per step from global
// memory with early exit: with so many hits it ends soon.
// SORTED (the nsample <= 64 NEAREST points inside the radius, nearest first; cpu/src/neighbors.cpp:8-136):
// the same walk, the hits ranked by (distance, index) instead.  A query with more than 64 hits walks its
// chains once more and keeps the 64 best (distance, index) keys sorted across the lanes, merging the hits
// of every step into them; with an interval wider than five cells it does so over all points.
// ---------------------------------------------------------------------------------------
constexpr int BQC_THREADS = 1024;
constexpr int BQC_WAVES = BQC_THREADS / TPK_WAVE;
constexpr int BQC_MIN_POINTS = 1024;
constexpr int BQC_MAX_POINTS = 8192;
constexpr int BQC_PER_THREAD = BQC_MAX_POINTS / BQC_THREADS;
constexpr int BQC_BUCKETS = 4096;    // 16 x 16 x 16
constexpr float BQC_CELL = 0.7f;     // cell width in radii (measured: 0.55 / 0.85 / 1.0 are 28 / 8 / 18 % slower)
constexpr int BQC_SPAN = 5;          // cells per axis a query may touch
constexpr int BQC_HITS = TPK_WAVE;
constexpr int BQC_MAX_CHAIN = 48;    // steps of the chain walk per query

struct CellWave
{
    int rows[BQC_HITS];
    float dists[BQC_HITS];
};

size_t bqc_lds_bytes(int n)
{
    return static_cast<size_t>(n) * sizeof(float4) + BQC_BUCKETS * sizeof(int) + BQC_WAVES * sizeof(CellWave);
}

// Cell along one axis: monotone in v, so the cells of [v - r, v + r] enclose the cell of every point in
// that interval (the conversion saturates; NaN goes to cell 0).
__device__ __forceinline__ int bqc_cell(float v, float inv)
{
    return static_cast<int>(floorf(v * inv));
}
__device__ __forceinline__ int bqc_bucket(int i, int j, int k)
{
    return (i & 15) | ((j & 15) << 4) | ((k & 15) << 8);
}

template <bool SORTED>
__global__ __launch_bounds__(BQC_THREADS) void ball_query_dense_cells_kernel(
    int n, int m, int blocks_per_cloud, int queries_per_block, float radius, float radius2, int nsample,
    const float* __restrict__ new_xyz, const float* __restrict__ xyz, int64_t* __restrict__ idx,
    float* __restrict__ dist)
{
    extern __shared__ __align__(16) unsigned char bqc_lds[];
    float4* const points = reinterpret_cast<float4*>(bqc_lds); // [n] x, y, z, next point of the bucket's chain
    int* const heads = reinterpret_cast<int*>(points + n);     // [BQC_BUCKETS] first point of the chain, -1: none
    CellWave* const waves = reinterpret_cast<CellWave*>(heads + BQC_BUCKETS);
    __shared__ int occupied; // buckets with a chain

    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / TPK_WAVE);
    const int cloud = blockIdx.x / blocks_per_cloud;
    const int blk = blockIdx.x - cloud * blocks_per_cloud;
    new_xyz += static_cast<int64_t>(cloud) * m * 3;
    xyz += static_cast<int64_t>(cloud) * n * 3;
    TPK_WORK_DECL

    // ---- the cloud's points onto the chains of their buckets ----
    float px[BQC_PER_THREAD], py[BQC_PER_THREAD], pz[BQC_PER_THREAD];
#pragma unroll
    for (int u = 0; u < BQC_PER_THREAD; ++u)
    {
        const int t = min(tid + u * BQC_THREADS, n - 1);
        px[u] = xyz[t * 3 + 0];
        py[u] = xyz[t * 3 + 1];
        pz[u] = xyz[t * 3 + 2];
    }
    static_assert(BQC_BUCKETS == 4 * BQC_THREADS, "one int4 of heads per thread");
    reinterpret_cast<int4*>(heads)[tid] = make_int4(-1, -1, -1, -1);
    if (tid == 0)
        occupied = 0;
    const float reach = fabsf(radius); // (the test itself uses radius * radius)
    const float inv = reach > 0.0f ? 1.0f / (BQC_CELL * reach) : 0.0f;
    lds_barrier();
    int fresh = 0; // chains this wavefront started
#pragma unroll
    for (int u = 0; u < BQC_PER_THREAD; ++u)
    {
        const int t = tid + u * BQC_THREADS;
        int next = 0;
        if (t < n)
        {
            const int bucket = bqc_bucket(bqc_cell(px[u], inv), bqc_cell(py[u], inv), bqc_cell(pz[u], inv));
            next = atomicExch(&heads[bucket], t);
            points[t] = make_float4(px[u], py[u], pz[u], __int_as_float(next));
        }
        fresh += __builtin_popcountll(__ballot(next < 0));
    }
    if (lane == 0 && fresh > 0)
        atomicAdd(&occupied, fresh);
    __syncthreads();

    // Chains or the scan in index order for this cloud?  n / occupied points per cell stand for about 12 times
    // as many in a ball (volumes 4.19 against 0.34 radii cubed).  A chain walk takes a step for every five
    // points in the ball and is lost work when the ball holds more than 64.  The scan stops after nsample hits,
    // 64 points a step, two queries a step; balls at the rim of a cloud hold a fraction of the points and scan
    // far longer, hence the 4.  Both costs in units fitted to measurements on clouds of 1024 .. 8192 points and
    // 2 .. 1100 points per ball.  (A query whose surroundings are denser than the cloud's average still falls
    // back on its own.)
    const float in_ball = 12.2f * static_cast<float>(n) / static_cast<float>(max(occupied, 1));
    const float scan_steps = fminf(static_cast<float>(n), 4.0f * static_cast<float>(nsample) * static_cast<float>(n) / in_ball) * (1.0f / TPK_WAVE);
    const bool scan_all = 1.6f + 0.24f * scan_steps < 2.0f + 0.2f * in_ball;

    // ---- queries: one wavefront each, no workgroup barrier from here on ----
    const int q_end = min(m, (blk + 1) * queries_per_block);
    if (!SORTED && scan_all)
    {
        // The scan in index order over the points in LDS, for two of the wavefront's queries at a time: lanes
        // hold 64 consecutive points; a ballot of the radius test and a prefix count give the hits their slots;
        // a query is switched off (radius -1) once it has nsample hits.
        constexpr int QS = 2;
        for (int j0 = blk * queries_per_block + wave; j0 < q_end; j0 += QS * BQC_WAVES)
        {
            float qx[QS], qy[QS], qz[QS], r2q[QS];
            int cnt[QS], lowest[QS], live = 0;
#pragma unroll
            for (int t = 0; t < QS; ++t)
            {
                const bool on = j0 + t * BQC_WAVES < q_end;
                const int j = on ? j0 + t * BQC_WAVES : j0;
                qx[t] = to_vector_register(new_xyz[j * 3 + 0]);
                qy[t] = to_vector_register(new_xyz[j * 3 + 1]);
                qz[t] = to_vector_register(new_xyz[j * 3 + 2]);
                r2q[t] = on ? radius2 : -1.0f;
                cnt[t] = lowest[t] = 0;
                live += on ? 1 : 0;
            }
            for (int base = 0; base < n && live > 0; base += TPK_WAVE)
            {
                const int pos = base + lane;
                const float4 p = points[min(pos, n - 1)];
                TPK_WORK_ADD(QS);
#pragma unroll
                for (int t = 0; t < QS; ++t)
                {
                    const float d = tpk_dist2(qx[t], qy[t], qz[t], p.x, p.y, p.z);
                    const bool hit = pos < n && d < r2q[t];
                    const unsigned long long mask = __ballot(hit);
                    if (mask != 0ull)
                    {
                        const int slot = cnt[t] + static_cast<int>(tpk_prefix_count(mask));
                        if (hit && slot < nsample)
                        {
                            const int64_t o = (static_cast<int64_t>(cloud) * m + j0 + t * BQC_WAVES) * nsample + slot;
                            idx[o] = pos;
                            dist[o] = d;
                        }
                        if (cnt[t] == 0)
                            lowest[t] = base + __builtin_ctzll(mask);
                        cnt[t] += __builtin_popcountll(mask);
                        if (cnt[t] >= nsample)
                        {
                            cnt[t] = nsample;
                            r2q[t] = -1.0f;
                            --live;
                        }
                    }
                }
            }
#pragma unroll
            for (int t = 0; t < QS; ++t)
                if (j0 + t * BQC_WAVES < q_end)
                    for (int s = cnt[t] + lane; s < nsample; s += TPK_WAVE)
                    {
                        const int64_t o = (static_cast<int64_t>(cloud) * m + j0 + t * BQC_WAVES) * nsample + s;
                        idx[o] = lowest[t];
                        dist[o] = -1.0f;
                    }
        }
        TPK_WORK_FLUSH
        return;
    }
    int* const rows = waves[wave].rows;
    float* const dists = waves[wave].dists;
    for (int j = blk * queries_per_block + wave; j < q_end; j += BQC_WAVES)
    {
        const float ux = new_xyz[j * 3 + 0], uy = new_xyz[j * 3 + 1], uz = new_xyz[j * 3 + 2];
        const float qx = to_vector_register(ux), qy = to_vector_register(uy), qz = to_vector_register(uz);
        const int64_t out = (static_cast<int64_t>(cloud) * m + j) * nsample;
        const float u[3] = {ux, uy, uz};
        int first[3], count[3];
#pragma unroll
        for (int a = 0; a < 3; ++a)
        {
            // (the interval is widened by a few ulps of its ends: a point that the fp32 radius test accepts
            // is never left out)
            const float slack = (fabsf(u[a]) + reach) * 1e-6f + 1e-30f;
            first[a] = bqc_cell((u[a] - reach) - slack, inv);
            // (as a difference of 64-bit values: the ends may lie at the two ends of the int range)
            const long long span = static_cast<long long>(bqc_cell((u[a] + reach) + slack, inv)) - first[a] + 1;
            count[a] = static_cast<int>(span < BQC_SPAN + 1 ? span : BQC_SPAN + 1);
        }
        int cnt = 0;
        const bool wide = count[0] > BQC_SPAN || count[1] > BQC_SPAN || count[2] > BQC_SPAN;
        bool serial = wide;
        const int cells = count[0] * count[1] * count[2];
        const int plane = count[0] * count[1];
        // (lane -> cell by float division: exact for these small numbers)
        const float inv_plane = 1.0f / static_cast<float>(plane), inv_line = 1.0f / static_cast<float>(count[0]);
        // first point of the chain of cell c (-1 past the last cell)
        auto chain_of = [&](int c) __attribute__((always_inline)) {
            const int k = static_cast<int>((static_cast<float>(c) + 0.5f) * inv_plane);
            const int rest = c - k * plane;
            const int jj = static_cast<int>((static_cast<float>(rest) + 0.5f) * inv_line);
            const int i = rest - jj * count[0];
            return c < cells ? heads[bqc_bucket(first[0] + i, first[1] + jj, first[2] + k)] : -1;
        };
        if (!serial)
        {
            int steps = 0;
            for (int c0 = 0; c0 < cells && !serial; c0 += TPK_WAVE)
            {
                int cur = chain_of(c0 + lane);
                // all lanes walk their chains in step
                while (__ballot(cur >= 0) != 0ull)
                {
                    if (++steps > BQC_MAX_CHAIN)
                    {
                        serial = true;
                        break;
                    }
                    const float4 p = points[max(cur, 0)];
                    const float d = tpk_dist2(qx, qy, qz, p.x, p.y, p.z);
                    TPK_WORK_ADD(1);
                    const bool hit = cur >= 0 && d < radius2;
                    const unsigned long long mask = __ballot(hit);
                    if (mask != 0ull)
                    {
                        const int slot = cnt + static_cast<int>(tpk_prefix_count(mask));
                        if (hit && slot < BQC_HITS)
                        {
                            rows[slot] = cur;
                            dists[slot] = d;
                        }
                        cnt += __builtin_popcountll(mask);
                        if (cnt > BQC_HITS)
                        {
                            serial = true;
                            break;
                        }
                    }
                    cur = cur >= 0 ? __float_as_int(p.w) : -1;
                }
            }
        }
        if (!serial)
        {
            // rank of every hit among the hits - by index, SORTED: by (distance, index); the keys are distinct -,
            // hits in that order, then the padding
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            const int my_row = lane < cnt ? rows[lane] : 0x7fffffff;
            const float my_dist = dists[lane < cnt ? lane : 0];
            int rank = 0, lowest = cnt > 0 ? 0x7fffffff : 0;
            // (four hits per turn; the lanes past the last hit hold the largest key, which counts for nothing)
            if constexpr (SORTED)
            {
                const u64 my_key = lane < cnt ? knn_key(my_dist, my_row) : ~0ull;
                u64 nearest = ~0ull;
                for (int h = 0; h < cnt; h += 4)
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                    {
                        const u64 other = read_lane_key(my_key, h + g);
                        rank += other < my_key ? 1 : 0;
                        nearest = other < nearest ? other : nearest;
                    }
                lowest = cnt > 0 ? static_cast<int>(nearest & 0xFFFFFFFFu) : 0;
            }
            else
            {
                for (int h = 0; h < cnt; h += 4)
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                    {
                        const int other = __builtin_amdgcn_readlane(my_row, h + g);
                        rank += other < my_row ? 1 : 0;
                        lowest = min(lowest, other);
                    }
            }
            if (lane < cnt && rank < nsample)
            {
                idx[out + rank] = my_row;
                dist[out + rank] = my_dist;
            }
            for (int s = cnt + lane; s < nsample; s += TPK_WAVE)
            {
                idx[out + s] = lowest;
                dist[out + s] = -1.0f;
            }
            // (the next query's hits overwrite rows / dists: all lanes have read theirs above)
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            continue;
        }

        if constexpr (SORTED)
        {
            // More hits than the buffer holds: lane i keeps the i-th smallest (distance, index) key so far; the
            // hits of a step that beat the nsample-th are sorted the other way round and merged in.
            constexpr u64 NONE = ~0ull;
            u64 best = NONE, admit = NONE;
            auto offer = [&](bool hit, float d, int row) __attribute__((always_inline)) {
                u64 cand = hit ? knn_key(d, row) : NONE;
                cand = cand < admit ? cand : NONE;
                if (__ballot(cand != NONE) == 0ull)
                    return;
                cand = wave_sort_keys(cand, lane, true);
                best = wave_merge_ascending(best < cand ? best : cand, lane);
                admit = read_lane_key(best, nsample - 1);
            };
            if (wide)
                for (int base = 0; base < n; base += TPK_WAVE)
                {
                    const int pos = base + lane;
                    const float4 p = points[min(pos, n - 1)];
                    const float d = tpk_dist2(qx, qy, qz, p.x, p.y, p.z);
                    TPK_WORK_ADD(1);
                    offer(pos < n && d < radius2, d, pos);
                }
            else
                for (int c0 = 0; c0 < cells; c0 += TPK_WAVE)
                {
                    int cur = chain_of(c0 + lane);
                    while (__ballot(cur >= 0) != 0ull)
                    {
                        const float4 p = points[max(cur, 0)];
                        const float d = tpk_dist2(qx, qy, qz, p.x, p.y, p.z);
                        TPK_WORK_ADD(1);
                        offer(cur >= 0 && d < radius2, d, cur);
                        cur = cur >= 0 ? __float_as_int(p.w) : -1;
                    }
                }
            const u64 nearest = read_lane_key(best, 0);
            if (lane < nsample)
            {
                const bool found = best != NONE;
                idx[out + lane] = found ? static_cast<int64_t>(best & 0xFFFFFFFFu)
                                        : (nearest != NONE ? static_cast<int64_t>(nearest & 0xFFFFFFFFu) : 0);
                dist[out + lane] = found ? __int_as_float(static_cast<int>(best >> 32)) : -1.0f;
            }
            continue;
        }

        // The scan in index order itself, over the points in LDS: lanes hold 64 consecutive points; ballot +
        // prefix count give the hits their slots; stop after nsample hits.
        cnt = 0;
        int lowest = 0;
        for (int base = 0; base < n && cnt < nsample; base += TPK_WAVE)
        {
            const int pos = base + lane;
            const float4 p = points[min(pos, n - 1)];
            const float d = tpk_dist2(qx, qy, qz, p.x, p.y, p.z);
            TPK_WORK_ADD(1);
            const bool hit = pos < n && d < radius2;
            const unsigned long long mask = __ballot(hit);
            if (mask == 0ull)
                continue;
            const int slot = cnt + static_cast<int>(tpk_prefix_count(mask));
            if (hit && slot < nsample)
            {
                idx[out + slot] = pos;
                dist[out + slot] = d;
            }
            if (cnt == 0)
                lowest = base + __builtin_ctzll(mask);
            cnt += __builtin_popcountll(mask);
        }
        for (int s = cnt + lane; s < nsample; s += TPK_WAVE)
        {
            idx[out + s] = lowest;
            dist[out + s] = -1.0f;
        }
    }
    TPK_WORK_FLUSH
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

int tpk_cells_ball_query_dense(int b, int n, int m, float radius, float radius2, int nsample, bool sorted,
                               const float* new_xyz, const float* xyz, int64_t* idx, float* dist, hipStream_t s)
{
    if (n < BQC_MIN_POINTS || n > BQC_MAX_POINTS || (sorted && nsample > BQC_HITS))
        return TPK_ERR_UNSUPPORTED;
    // one workgroup per compute unit where the queries allow it (every workgroup hangs up its cloud)
    const int64_t per_cloud = std::max<int64_t>(1, std::min<int64_t>(tpk_ceil_div(m, BQC_WAVES), TPK_COMPUTE_UNITS / b));
    const int per_block = static_cast<int>(tpk_ceil_div(m, per_cloud));
    const int64_t bpc = tpk_ceil_div(m, per_block);
    if (bpc * b > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const size_t lds = bqc_lds_bytes(n);
    const void* kernel = sorted ? reinterpret_cast<const void*>(&ball_query_dense_cells_kernel<true>)
                                : reinterpret_cast<const void*>(&ball_query_dense_cells_kernel<false>);
    const int st = tpk_allow_lds(kernel, lds);
    if (st != TPK_OK)
        return st;
    if (sorted)
        hipLaunchKernelGGL(ball_query_dense_cells_kernel<true>, dim3(static_cast<unsigned>(bpc * b)), dim3(BQC_THREADS), lds, s,
                           n, m, static_cast<int>(bpc), per_block, radius, radius2, nsample, new_xyz, xyz, idx, dist);
    else
        hipLaunchKernelGGL(ball_query_dense_cells_kernel<false>, dim3(static_cast<unsigned>(bpc * b)), dim3(BQC_THREADS), lds, s,
                           n, m, static_cast<int>(bpc), per_block, radius, radius2, nsample, new_xyz, xyz, idx, dist);
    return tpk_launch_status();
}

extern "C" size_t tpk_ball_query_dense_workspace_bytes(int b, int n, int m, int nsample)
{
    return tpk_grid_ball_query_dense_workspace_bytes(b, n, m, nsample);
}

extern "C" int tpk_ball_query_dense_ws_f32(int b, int n, int m, float radius, int nsample,
                                           const float* new_xyz, const float* xyz, int64_t* idx,
                                           float* dist, void* workspace, size_t workspace_bytes, void* stream)
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
    {
        // clouds of 1024 .. 8192 points: buckets of cells in LDS
        const int st = tpk_cells_ball_query_dense(b, n, m, radius, radius2, nsample, false, new_xyz, xyz, idx, dist, tpk_stream(stream));
        if (st != TPK_ERR_UNSUPPORTED)
            return st;
    }
    if (workspace)
    {
        // larger clouds: ordered in windows, a walk over the bins the ball touches
        const int st = tpk_grid_ball_query_dense(b, n, m, radius, radius2, nsample, new_xyz, xyz, idx, dist, workspace,
                                                 workspace_bytes, tpk_stream(stream));
        if (st != TPK_ERR_UNSUPPORTED)
            return st;
    }
    if (few)
        hipLaunchKernelGGL(ball_query_dense_kernel<BQ_Q_FEW>, dim3(static_cast<unsigned>(blocks)), dim3(BQ_THREADS), 0,
                           tpk_stream(stream), n, m, static_cast<int>(bpc), radius2, nsample, new_xyz, xyz, idx, dist);
    else
        hipLaunchKernelGGL(ball_query_dense_kernel<BQ_Q>, dim3(static_cast<unsigned>(blocks)), dim3(BQ_THREADS), 0,
                           tpk_stream(stream), n, m, static_cast<int>(bpc), radius2, nsample, new_xyz, xyz, idx, dist);
    return tpk_launch_status();
}

extern "C" int tpk_ball_query_dense_f32(int b, int n, int m, float radius, int nsample,
                                        const float* new_xyz, const float* xyz, int64_t* idx,
                                        float* dist, void* stream)
{
    return tpk_ball_query_dense_ws_f32(b, n, m, radius, nsample, new_xyz, xyz, idx, dist, nullptr, 0, stream);
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
