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

// ---------------------------------------------------------------------------------------
// Dense layout over cells: clouds of BQC_MIN_POINTS .. BQC_MAX_POINTS support points.
//
// Testing every support point costs n / 64 steps per query whatever the radius.  Here a workgroup
// of 16 wavefronts first bins its cloud in LDS: bounding box, a grid of up to 16 cells per axis
// whose cells are at least one radius wide, a count per cell (LDS atomics that also hand every
// point its place inside its cell), a prefix sum, and the points (x, y, z, index) written cell by
// cell.  All workgroups of a cloud repeat this (a few microseconds; the cloud comes from the L2),
// which is cheaper than a launch that does it once.  Then every wavefront answers queries, one at
// a time: the cells that the cube around the ball touches form, for every (y, z), one run of
// consecutive places - cells are numbered x first - so lane r takes row r's run, and the
// candidates of all runs are dealt to the lanes 64 at a time.  A candidate with d2 < radius^2 is
// a hit; the hits (at most 64) are ranked by index and written in ascending index order, which
// is what the scan in index order produces (cuda/src/ball_query_gpu.cu:9-52).  A query with more
// than 64 hits, or whose cube holds more than BQC_MAX_CANDIDATES points (a ball that covers much
// of its cloud), is answered by that scan itself, 64 points per step from global memory with
// early exit: with so many hits it ends soon.
// ---------------------------------------------------------------------------------------
constexpr int BQC_THREADS = 1024;
constexpr int BQC_WAVES = BQC_THREADS / TPK_WAVE;
constexpr int BQC_MIN_POINTS = 512;
constexpr int BQC_MAX_POINTS = 8192;
constexpr int BQC_PER_THREAD = BQC_MAX_POINTS / BQC_THREADS;
constexpr int BQC_GRID = 16;
constexpr int BQC_CELLS = BQC_GRID * BQC_GRID * BQC_GRID;
constexpr int BQC_STARTS = BQC_CELLS + TPK_WAVE; // the cells' first places, one more for the end, padded
constexpr int BQC_HITS = TPK_WAVE;
constexpr int BQC_MAX_CANDIDATES = 8 * TPK_WAVE;

struct CellWave
{
    int rows[BQC_HITS];
    float dists[BQC_HITS];
    int marks[TPK_WAVE];
};

size_t bqc_lds_bytes(int n)
{
    return static_cast<size_t>(n) * sizeof(float4) + BQC_STARTS * sizeof(int) + BQC_WAVES * sizeof(CellWave);
}

// Smallest / largest v of every 16-lane row, in all lanes of the row.
__device__ __forceinline__ float row_all_min_f32(float v)
{
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true)));
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true)));
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xF, 0xF, true)));
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, true)));
    return v;
}
__device__ __forceinline__ float wave_min_f32(float v)
{
    v = row_all_min_f32(v);
    return fminf(fminf(tpk_read_lane(v, 0), tpk_read_lane(v, 16)), fminf(tpk_read_lane(v, 32), tpk_read_lane(v, 48)));
}

// Cell along one axis: monotone in v (so the cells of [v - r, v + r] enclose the cell of every point in
// that interval), clamped to the grid; NaN goes to cell 0.
__device__ __forceinline__ int bqc_cell(float v, float lo, float inv, int cells)
{
    return min(cells - 1, max(0, static_cast<int>((v - lo) * inv)));
}

__global__ __launch_bounds__(BQC_THREADS) void ball_query_dense_cells_kernel(
    int n, int m, int blocks_per_cloud, int queries_per_block, float radius, float radius2, int nsample,
    const float* __restrict__ new_xyz, const float* __restrict__ xyz, int64_t* __restrict__ idx,
    float* __restrict__ dist)
{
    extern __shared__ __align__(16) unsigned char bqc_lds[];
    float4* const sorted = reinterpret_cast<float4*>(bqc_lds); // [n] x, y, z, index; cell by cell
    int* const starts = reinterpret_cast<int*>(sorted + n);    // [BQC_STARTS] counts, then first places
    CellWave* const waves = reinterpret_cast<CellWave*>(starts + BQC_STARTS);
    __shared__ float box_parts[6][BQC_WAVES]; // per wavefront: -min x, y, z then max x, y, z
    __shared__ float box[6];
    __shared__ int wave_totals[BQC_WAVES];

    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / TPK_WAVE);
    const int cloud = blockIdx.x / blocks_per_cloud;
    const int blk = blockIdx.x - cloud * blocks_per_cloud;
    new_xyz += static_cast<int64_t>(cloud) * m * 3;
    xyz += static_cast<int64_t>(cloud) * n * 3;
    TPK_WORK_DECL

    // ---- the cloud's points and bounding box (finite coordinates only) ----
    float px[BQC_PER_THREAD], py[BQC_PER_THREAD], pz[BQC_PER_THREAD];
#pragma unroll
    for (int u = 0; u < BQC_PER_THREAD; ++u)
    {
        const int t = min(tid + u * BQC_THREADS, n - 1);
        px[u] = xyz[t * 3 + 0];
        py[u] = xyz[t * 3 + 1];
        pz[u] = xyz[t * 3 + 2];
    }
    for (int c = tid; c < BQC_STARTS; c += BQC_THREADS)
        starts[c] = 0;
    {
        const float inf = __builtin_inff();
        float ends[6] = {inf, inf, inf, inf, inf, inf}; // (minima of -max: one kind of reduction)
#pragma unroll
        for (int u = 0; u < BQC_PER_THREAD; ++u)
        {
            // (rows past the end repeat the last point: no effect on the box)
            const float v[3] = {px[u], py[u], pz[u]};
#pragma unroll
            for (int a = 0; a < 3; ++a)
                if (fabsf(v[a]) < inf)
                {
                    ends[a] = fminf(ends[a], v[a]);
                    ends[3 + a] = fminf(ends[3 + a], -v[a]);
                }
        }
#pragma unroll
        for (int a = 0; a < 6; ++a)
        {
            const float e = wave_min_f32(ends[a]);
            if (lane == 0)
                box_parts[a][wave] = e;
        }
    }
    __syncthreads();
    if (wave == 0)
    {
#pragma unroll
        for (int a = 0; a < 6; ++a)
        {
            const float e = row_all_min_f32(box_parts[a][lane & (BQC_WAVES - 1)]);
            if (lane == 0)
                box[a] = e;
        }
    }
    __syncthreads();

    // ---- the grid: per axis as many cells (16 at most) as are at least one radius wide ----
    const float reach = fabsf(radius); // (the test itself uses radius * radius)
    float lo[3], inv[3];
    int cells[3];
#pragma unroll
    for (int a = 0; a < 3; ++a)
    {
        lo[a] = box[a];
        const float extent = -box[3 + a] - lo[a]; // (NaN or -inf for a cloud without finite coordinates)
        const float fit = fminf(extent / reach, static_cast<float>(BQC_GRID));
        cells[a] = fit >= 1.0f ? static_cast<int>(fit) : 1;
        inv[a] = extent > 0.0f ? static_cast<float>(cells[a]) / extent : 0.0f;
        lo[a] = extent > 0.0f ? lo[a] : 0.0f;
    }

    // ---- count per cell; the count before a point's own increment is its place inside the cell ----
    int placed[BQC_PER_THREAD];
#pragma unroll
    for (int u = 0; u < BQC_PER_THREAD; ++u)
        if (tid + u * BQC_THREADS < n)
        {
            const int c = bqc_cell(px[u], lo[0], inv[0], cells[0]) +
                          cells[0] * (bqc_cell(py[u], lo[1], inv[1], cells[1]) + cells[1] * bqc_cell(pz[u], lo[2], inv[2], cells[2]));
            placed[u] = (c << 16) | atomicAdd(&starts[c], 1);
        }
    __syncthreads();
    {
        // exclusive prefix sum over the cells, four per thread
        int4 c4 = reinterpret_cast<int4*>(starts)[tid];
        const int own = c4.x + c4.y + c4.z + c4.w;
        const int before = wave_exclusive_sum(own);
        if (lane == TPK_WAVE - 1)
            wave_totals[wave] = before + own;
        __syncthreads();
        const int total = lane < BQC_WAVES ? wave_totals[lane] : 0;
        int at = __builtin_amdgcn_readlane(wave_exclusive_sum(total), wave) + before;
        int4 s4;
        s4.x = at;
        s4.y = at += c4.x;
        s4.z = at += c4.y;
        s4.w = at += c4.z;
        reinterpret_cast<int4*>(starts)[tid] = s4;
        if (tid == BQC_THREADS - 1)
            starts[BQC_CELLS] = at + c4.w;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < BQC_PER_THREAD; ++u)
        if (tid + u * BQC_THREADS < n)
            sorted[starts[placed[u] >> 16] + (placed[u] & 0xFFFF)] =
                make_float4(px[u], py[u], pz[u], __int_as_float(tid + u * BQC_THREADS));
    __syncthreads();

    // ---- queries: one wavefront each, no workgroup barrier from here on ----
    int* const rows = waves[wave].rows;
    float* const dists = waves[wave].dists;
    volatile int* const marks = waves[wave].marks; // (volatile: a lane reads what other lanes wrote)
    const int q_end = min(m, (blk + 1) * queries_per_block);
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
            first[a] = bqc_cell((u[a] - reach) - slack, lo[a], inv[a], cells[a]);
            count[a] = bqc_cell((u[a] + reach) + slack, lo[a], inv[a], cells[a]) - first[a] + 1;
        }
        const int runs = count[1] * count[2];
        int cnt = 0;
        bool serial = runs > TPK_WAVE;
        if (!serial)
        {
            // lane r: the places of run r (the cells first[0] .. first[0] + count[0] - 1 of one (y, z))
            int start = 0, size = 0;
            if (lane < runs)
            {
                const int c = first[0] + cells[0] * ((first[1] + lane % count[1]) + cells[1] * (first[2] + lane / count[1]));
                start = starts[c];
                size = starts[c + count[0]] - start;
            }
            const int before = wave_exclusive_sum(size);
            const int total = __builtin_amdgcn_readlane(before + size, TPK_WAVE - 1);
            const int origin = start - before; // candidate c lies at origin + c, for the c of this lane's run
            serial = total > BQC_MAX_CANDIDATES;
            for (int c0 = 0; c0 < total && !serial; c0 += TPK_WAVE)
            {
                // Which run does candidate c0 + lane belong to?  Every run's lane marks the slot of its first
                // candidate in this step with its own number; a running maximum carries it to the others.
                marks[lane] = 0;
                if (size > 0 && before < c0 + TPK_WAVE && before + size > c0)
                    marks[max(before - c0, 0)] = lane;
                const int mark = marks[lane];
                const bool has = c0 + lane < total;
                const int at = __shfl(origin, wave_inclusive_max_i32(mark)) + c0 + lane;
                const float4 p = sorted[has ? at : 0];
                const float d = tpk_dist2(qx, qy, qz, p.x, p.y, p.z);
                TPK_WORK_ADD(1);
                const bool hit = has && d < radius2;
                const unsigned long long mask = __ballot(hit);
                if (mask == 0ull)
                    continue;
                const int slot = cnt + static_cast<int>(tpk_prefix_count(mask));
                if (hit && slot < BQC_HITS)
                {
                    rows[slot] = __float_as_int(p.w);
                    dists[slot] = d;
                }
                cnt += __builtin_popcountll(mask);
                serial = cnt > BQC_HITS;
            }
        }
        if (!serial)
        {
            // rank of every hit among the hits (indices are distinct), hits in that order, then the padding
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            const int my_row = rows[lane < cnt ? lane : 0];
            const float my_dist = dists[lane < cnt ? lane : 0];
            int rank = 0, lowest = cnt > 0 ? 0x7fffffff : 0;
            for (int h = 0; h < cnt; ++h)
            {
                const int other = rows[h];
                rank += other < my_row ? 1 : 0;
                lowest = min(lowest, other);
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

        // The scan in index order itself: lanes hold 64 consecutive points; ballot + prefix count give the
        // hits their slots; stop after nsample hits.
        cnt = 0;
        int64_t lowest = 0;
        constexpr int BATCH = 4; // loads of four steps in flight
        for (int base = 0; base < n && cnt < nsample; base += BATCH * TPK_WAVE)
        {
            float sx[BATCH], sy[BATCH], sz[BATCH];
#pragma unroll
            for (int b = 0; b < BATCH; ++b)
            {
                const int pos = min(base + b * TPK_WAVE + lane, n - 1);
                sx[b] = xyz[pos * 3 + 0];
                sy[b] = xyz[pos * 3 + 1];
                sz[b] = xyz[pos * 3 + 2];
            }
#pragma unroll
            for (int b = 0; b < BATCH; ++b)
            {
                const int pos = base + b * TPK_WAVE + lane;
                const float d = tpk_dist2(qx, qy, qz, sx[b], sy[b], sz[b]);
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
                    lowest = base + b * TPK_WAVE + __builtin_ctzll(mask);
                cnt += __builtin_popcountll(mask);
            }
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
    if (n >= BQC_MIN_POINTS && n <= BQC_MAX_POINTS)
    {
        // over cells; one workgroup per compute unit where the queries allow it (every workgroup bins its cloud)
        const int64_t per_cloud = std::max<int64_t>(1, std::min<int64_t>(tpk_ceil_div(m, BQC_WAVES), TPK_COMPUTE_UNITS / b));
        const int per_block = static_cast<int>(tpk_ceil_div(m, per_cloud));
        const int64_t cell_bpc = tpk_ceil_div(m, per_block);
        const size_t lds = bqc_lds_bytes(n);
        const int st = tpk_allow_lds(reinterpret_cast<const void*>(&ball_query_dense_cells_kernel), lds);
        if (st != TPK_OK)
            return st;
        hipLaunchKernelGGL(ball_query_dense_cells_kernel, dim3(static_cast<unsigned>(cell_bpc * b)), dim3(BQC_THREADS), lds,
                           tpk_stream(stream), n, m, static_cast<int>(cell_bpc), per_block, radius, radius2, nsample, new_xyz,
                           xyz, idx, dist);
        return tpk_launch_status();
    }
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
