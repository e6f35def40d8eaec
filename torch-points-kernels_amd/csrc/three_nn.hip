// three_nn: for every "unknown" point the three nearest "known" points of the same cloud.
//
// Work split: one lane owns Q query points and keeps their running best three (distance,
// index) in registers; the known points of the cloud stream through LDS in tiles of
// float4 (x, y, z, pad), so every lane of a wavefront reads the same LDS address at the
// same time (a broadcast read, no bank conflicts) and one LDS read feeds Q distance
// evaluations.  Insertion into the sorted triple happens only in lanes whose distance
// beats their current third best, which after the first few hundred candidates is rare.
//
// Semantics follow the reference kernel (cuda/src/interpolate_gpu.cu:9-65): candidates are
// visited in index order and replace an entry only when strictly smaller, so equal
// distances keep the lower index first.  The reference holds its running bests as doubles
// initialised to 1e40; every distance is an fp32 value, so fp32 running bests initialised
// to +inf select identically and store identical values.
#include "nn_grid.h"

#include <algorithm>
#include <mutex>

namespace {

constexpr int NN_THREADS = 256;
constexpr int NN_TILE = 1024; // known points per LDS tile (16 KiB)

template <int Q>
__global__ __launch_bounds__(NN_THREADS) void three_nn_kernel(
    int n, int m, int blocks_per_cloud, const float* __restrict__ unknown,
    const float* __restrict__ known, float* __restrict__ dist2, int32_t* __restrict__ idx)
{
    __shared__ float4 tile[NN_TILE];

    const int cloud = blockIdx.x / blocks_per_cloud;
    const int blk = blockIdx.x - cloud * blocks_per_cloud;
    unknown += static_cast<int64_t>(cloud) * n * 3;
    known += static_cast<int64_t>(cloud) * m * 3;
    dist2 += static_cast<int64_t>(cloud) * n * 3;
    idx += static_cast<int64_t>(cloud) * n * 3;

    const int tid = threadIdx.x;
    const int j0 = blk * (NN_THREADS * Q) + tid;

    float ux[Q], uy[Q], uz[Q];
    float b1[Q], b2[Q], b3[Q];
    int i1[Q], i2[Q], i3[Q];
#pragma unroll
    for (int q = 0; q < Q; ++q)
    {
        int j = j0 + q * NN_THREADS;
        j = j < n ? j : n - 1; // lanes past the end shadow the last query and store nothing
        ux[q] = unknown[j * 3 + 0];
        uy[q] = unknown[j * 3 + 1];
        uz[q] = unknown[j * 3 + 2];
        b1[q] = b2[q] = b3[q] = __builtin_inff();
        i1[q] = i2[q] = i3[q] = 0;
    }
    TPK_WORK_DECL

    for (int base = 0; base < m; base += NN_TILE)
    {
        const int cnt = min(NN_TILE, m - base);
        __syncthreads(); // the previous tile has been consumed by every wave
        for (int t = tid; t < NN_TILE; t += NN_THREADS)
        {
            float4 p;
            if (t < cnt)
            {
                const float* src = known + static_cast<int64_t>(base + t) * 3;
                p = make_float4(src[0], src[1], src[2], 0.f);
            }
            else
            {
                // Padding: an infinitely distant point never beats a running best.
                p = make_float4(__builtin_inff(), __builtin_inff(), __builtin_inff(), 0.f);
            }
            tile[t] = p;
        }
        __syncthreads();

        const int cnt4 = (cnt + 3) & ~3;
        TPK_WORK_ADD(cnt4 * Q);
#pragma unroll 4
        for (int k = 0; k < cnt4; ++k)
        {
            const float4 c = tile[k];
            const int kk = base + k;
#pragma unroll
            for (int q = 0; q < Q; ++q)
            {
                const float d = tpk_dist2(ux[q], uy[q], uz[q], c.x, c.y, c.z);
                if (d < b3[q])
                {
                    // Sorted insert written as selects: one short block, no nested divergence.
                    const bool lt1 = d < b1[q];
                    const bool lt2 = d < b2[q];
                    b3[q] = lt2 ? b2[q] : d;
                    i3[q] = lt2 ? i2[q] : kk;
                    b2[q] = lt1 ? b1[q] : (lt2 ? d : b2[q]);
                    i2[q] = lt1 ? i1[q] : (lt2 ? kk : i2[q]);
                    b1[q] = lt1 ? d : b1[q];
                    i1[q] = lt1 ? kk : i1[q];
                }
            }
        }
    }

    TPK_WORK_FLUSH
#pragma unroll
    for (int q = 0; q < Q; ++q)
    {
        const int j = j0 + q * NN_THREADS;
        if (j < n)
        {
            dist2[j * 3 + 0] = b1[q];
            dist2[j * 3 + 1] = b2[q];
            dist2[j * 3 + 2] = b3[q];
            idx[j * 3 + 0] = i1[q];
            idx[j * 3 + 1] = i2[q];
            idx[j * 3 + 2] = i3[q];
        }
    }
}

template <int Q>
int launch_three_nn(int b, int n, int m, const float* unknown, const float* known, float* dist2,
                    int32_t* idx, hipStream_t stream)
{
    const int64_t blocks_per_cloud = tpk_ceil_div(n, NN_THREADS * Q);
    const int64_t blocks = blocks_per_cloud * b;
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(three_nn_kernel<Q>, dim3(static_cast<unsigned>(blocks)), dim3(NN_THREADS),
                       0, stream, n, m, static_cast<int>(blocks_per_cloud), unknown, known, dist2,
                       idx);
    return tpk_launch_status();
}

// ---------------------------------------------------------------------------------------------
// Known clouds of TNC_MIN_KNOWN .. TNC_MAX_KNOWN points: a grid in LDS, one lane per query.
//
// Every workgroup (16 wavefronts) sorts its cloud's known points into the cells of a grid over their
// bounding box - up to 16 cells per axis, about two points per cell - in LDS: box, a count per cell (LDS
// atomics that also hand every point its place inside its cell), a prefix sum, the points written cell by
// cell as four arrays (x, y, z, index).  All workgroups of a cloud repeat this (a few microseconds; the
// cloud comes from the L2); no launch in front, no workspace, and the queries need no order.  Then every
// lane takes a query: the cells within one ring of the query's cell form, for every (y, z), one run of
// consecutive places - cells are numbered x first -, and the lane walks its runs point by point, keeping
// its best three (distance, index).  The answer is final when the third best distance is smaller than the
// distance to every face of the examined block that has cells behind it; otherwise the lane widens the
// block by a ring and walks it again (entries it already holds are recognised by their index).  Lanes of
// a wavefront walk different cells: LDS serves their scattered 4-byte reads at a third of the rate of
// consecutive ones, which is what this kernel is bound by together with the issue of the distance
// arithmetic.  Selection by (distance, index) gives what the reference's scan in index order with
// strictly-smaller replacement gives (cuda/src/interpolate_gpu.cu:9-65) whatever the visiting order.
// A cloud whose points crowd into few cells (sum of squared counts / m above m / 40) is scanned whole
// by every lane instead: broadcast reads, the cost of the all-pairs kernel.
// ---------------------------------------------------------------------------------------------
constexpr int TNC_THREADS = 1024;
constexpr int TNC_WAVES = TNC_THREADS / TPK_WAVE;
constexpr int TNC_MIN_KNOWN = 1024;
constexpr int TNC_MAX_KNOWN = 8192;
constexpr int TNC_PER_THREAD = TNC_MAX_KNOWN / TNC_THREADS;
constexpr int TNC_AXIS = 64;    // cells per axis at most
constexpr int TNC_CELLS = 4096; // cells in all at most
constexpr int TNC_STARTS = TNC_CELLS + TPK_WAVE; // the cells' first places, one more for the end, padded
constexpr float TNC_CROWDED = 12.0f; // points per cell, as a point sees them, from which the grid is given up
constexpr float TNC_PER_CELL = 2.0f;             // points per cell aimed at (1 / 1.5 / 3: 9 / 6 / 1 % slower)

size_t tnc_lds_bytes(int m)
{
    return static_cast<size_t>(m) * 16 + TNC_STARTS * sizeof(int);
}

// Smallest v of every 16-lane row, in all lanes of the row; of the wavefront.
__device__ __forceinline__ float tnc_row_min(float v)
{
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true)));
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true)));
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xF, 0xF, true)));
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, true)));
    return v;
}
__device__ __forceinline__ float tnc_wave_min(float v)
{
    v = tnc_row_min(v);
    return fminf(fminf(tpk_read_lane(v, 0), tpk_read_lane(v, 16)), fminf(tpk_read_lane(v, 32), tpk_read_lane(v, 48)));
}

// Cell along one axis, clamped to the grid (NaN goes to cell 0).
__device__ __forceinline__ int tnc_cell(float t, int cells)
{
    return min(cells - 1, max(0, static_cast<int>(t)));
}

// The best three (squared distance, index) of a lane, ascending, each as one integer: distances are >= 0, so
// their bit patterns order like unsigned integers and one 64-bit comparison orders by distance, then index.
// Unused entries are (inf, 0): no candidate at infinite distance, or with a NaN, is smaller.
struct Best3
{
    unsigned long long k1, k2, k3;
    __device__ __forceinline__ static unsigned long long key(float d, int i)
    {
        return (static_cast<unsigned long long>(static_cast<unsigned>(__float_as_int(d))) << 32) | static_cast<unsigned>(i);
    }
    __device__ __forceinline__ void clear() { k1 = k2 = k3 = key(__builtin_inff(), 0); }
    __device__ __forceinline__ float third() const { return __int_as_float(static_cast<int>(k3 >> 32)); }
    __device__ __forceinline__ void offer(unsigned long long k)
    {
        if (k < k3)
        {
            const bool lt1 = k < k1, lt2 = k < k2;
            k3 = lt2 ? k2 : k;
            k2 = lt1 ? k1 : (lt2 ? k : k2);
            k1 = lt1 ? k : k1;
        }
    }
};

__global__ __launch_bounds__(TNC_THREADS) void three_nn_cells_kernel(
    int n, int m, int blocks_per_cloud, int queries_per_block, const float* __restrict__ unknown,
    const float* __restrict__ known, float* __restrict__ dist2, int32_t* __restrict__ idx, int* __restrict__ general)
{
    extern __shared__ __align__(16) unsigned char tnc_lds[];
    float* const sx = reinterpret_cast<float*>(tnc_lds); // [m] each: the known points cell by cell
    float* const sy = sx + m;
    float* const sz = sy + m;
    int* const si = reinterpret_cast<int*>(sz + m);      // [m] their indices
    int* const starts = si + m;                          // [TNC_STARTS] counts, then first places
    __shared__ float box_parts[6][TNC_WAVES]; // per wavefront: min x, y, z then -max x, y, z
    __shared__ float box[6];
    __shared__ int wave_totals[TNC_WAVES];
    __shared__ int crowding; // sum over the cells of count^2

    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / TPK_WAVE);
    const int cloud = blockIdx.x / blocks_per_cloud;
    const int blk = blockIdx.x - cloud * blocks_per_cloud;
    unknown += static_cast<int64_t>(cloud) * n * 3;
    known += static_cast<int64_t>(cloud) * m * 3;
    dist2 += static_cast<int64_t>(cloud) * n * 3;
    idx += static_cast<int64_t>(cloud) * n * 3;
    TPK_WORK_DECL

    // ---- the cloud's points and bounding box (finite coordinates only) ----
    float px[TNC_PER_THREAD], py[TNC_PER_THREAD], pz[TNC_PER_THREAD];
#pragma unroll
    for (int u = 0; u < TNC_PER_THREAD; ++u)
    {
        const int t = min(tid + u * TNC_THREADS, m - 1);
        px[u] = known[t * 3 + 0];
        py[u] = known[t * 3 + 1];
        pz[u] = known[t * 3 + 2];
    }
    for (int c = tid; c < TNC_STARTS; c += TNC_THREADS)
        starts[c] = 0;
    if (tid == 0)
        crowding = 0;
    {
        const float inf = __builtin_inff();
        float ends[6] = {inf, inf, inf, inf, inf, inf}; // (minima of -max: one kind of reduction)
#pragma unroll
        for (int u = 0; u < TNC_PER_THREAD; ++u)
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
            const float e = tnc_wave_min(ends[a]);
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
            const float e = tnc_row_min(box_parts[a][lane & (TNC_WAVES - 1)]);
            if (lane == 0)
                box[a] = e;
        }
    }
    __syncthreads();

    // ---- the grid: about TNC_PER_CELL points per cell, cells as cubic as TNC_AXIS per axis and TNC_CELLS in
    // all allow (a flat cloud gets a flat grid of up to 64 x 64 cells) ----
    float lo[3], inv[3], width[3];
    int cells[3];
    {
        float extent[3], longest = 0.0f;
#pragma unroll
        for (int a = 0; a < 3; ++a)
        {
            lo[a] = box[a];
            extent[a] = -box[3 + a] - lo[a]; // (NaN or -inf for a cloud without finite coordinates)
            extent[a] = extent[a] > 0.0f ? extent[a] : 0.0f;
            longest = fmaxf(longest, extent[a]);
        }
        // cells per axis for `along` cells along the longest axis, and their product
        auto fit = [&](float along, int (&count)[3]) __attribute__((always_inline)) {
            int all = 1;
#pragma unroll
            for (int a = 0; a < 3; ++a)
            {
                const float f = longest > 0.0f ? fminf(extent[a] / longest * along + 0.5f, static_cast<float>(TNC_AXIS)) : 1.0f;
                count[a] = f >= 1.0f ? static_cast<int>(f) : 1;
                all *= count[a];
            }
            return all;
        };
        // (the product grows with `along`: the largest value that stays within the cells wanted, by bisection)
        const int wanted = static_cast<int>(fminf(static_cast<float>(TNC_CELLS), fmaxf(static_cast<float>(m) / TNC_PER_CELL, 1.0f)));
        float few = 0.0f, many = 2.0f * TNC_AXIS;
        for (int step = 0; step < 12; ++step)
        {
            const float mid = 0.5f * (few + many);
            int count[3];
            if (fit(mid, count) > wanted)
                many = mid;
            else
                few = mid;
        }
        fit(few, cells);
#pragma unroll
        for (int a = 0; a < 3; ++a)
        {
            inv[a] = extent[a] > 0.0f ? static_cast<float>(cells[a]) / extent[a] : 0.0f;
            width[a] = extent[a] / static_cast<float>(cells[a]);
            lo[a] = extent[a] > 0.0f ? lo[a] : 0.0f;
        }
    }

    // ---- count per cell; the count before a point's own increment is its place inside the cell ----
    int placed[TNC_PER_THREAD];
#pragma unroll
    for (int u = 0; u < TNC_PER_THREAD; ++u)
        if (tid + u * TNC_THREADS < m)
        {
            const int c = tnc_cell((px[u] - lo[0]) * inv[0], cells[0]) +
                          cells[0] * (tnc_cell((py[u] - lo[1]) * inv[1], cells[1]) + cells[1] * tnc_cell((pz[u] - lo[2]) * inv[2], cells[2]));
            placed[u] = (c << 16) | atomicAdd(&starts[c], 1);
        }
    __syncthreads();
    {
        // exclusive prefix sum over the cells, four per thread
        static_assert(TNC_CELLS == 4 * TNC_THREADS, "four cells per thread");
        int4 c4 = reinterpret_cast<int4*>(starts)[tid];
        const int own = c4.x + c4.y + c4.z + c4.w;
        const int before = wave_exclusive_sum(own);
        const int squares = wave_exclusive_sum(c4.x * c4.x + c4.y * c4.y + c4.z * c4.z + c4.w * c4.w);
        if (lane == TPK_WAVE - 1)
        {
            wave_totals[wave] = before + own;
            atomicAdd(&crowding, squares + c4.x * c4.x + c4.y * c4.y + c4.z * c4.z + c4.w * c4.w);
        }
        __syncthreads();
        const int total = lane < TNC_WAVES ? wave_totals[lane] : 0;
        int at = __builtin_amdgcn_readlane(wave_exclusive_sum(total), wave) + before;
        int4 s4;
        s4.x = at;
        s4.y = at += c4.x;
        s4.z = at += c4.y;
        s4.w = at += c4.z;
        reinterpret_cast<int4*>(starts)[tid] = s4;
        if (tid == TNC_THREADS - 1)
            starts[TNC_CELLS] = at + c4.w;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < TNC_PER_THREAD; ++u)
        if (tid + u * TNC_THREADS < m)
        {
            const int at = starts[placed[u] >> 16] + (placed[u] & 0xFFFF);
            sx[at] = px[u];
            sy[at] = py[u];
            sz[at] = pz[u];
            si[at] = tid + u * TNC_THREADS;
        }
    __syncthreads();
    // Points per cell as a point sees them (3 in a cloud of even density): above TNC_CROWDED the grid is a poor
    // fit - dense cells cost their queries many candidates, empty ones many steps of widening - and, where the
    // caller enqueues it behind this kernel, the search over curve-ordered cells answers the cloud instead.
    // Without it: on with the grid; when 40 points cost a lane what the whole cloud costs by broadcast reads,
    // every lane scans the cloud.
    const float crowd = static_cast<float>(crowding) / static_cast<float>(m);
    if (general)
    {
        const bool hand_over = crowd > TNC_CROWDED;
        if (blk == 0 && tid == 0)
            general[cloud] = hand_over ? 1 : 0;
        if (hand_over)
            return;
    }
    const bool crowded = crowd * 40.0f > static_cast<float>(m);

    // ---- queries: one lane each, no workgroup barrier from here on ----
    const int q_end = min(n, (blk + 1) * queries_per_block);
    for (int j = blk * queries_per_block + tid; j < q_end; j += TNC_THREADS)
    {
        const float qx = unknown[j * 3 + 0], qy = unknown[j * 3 + 1], qz = unknown[j * 3 + 2];
        Best3 best;
        best.clear();
        if (crowded)
        {
            for (int k = 0; k < m; ++k)
            {
                TPK_WORK_ADD(1);
                best.offer(Best3::key(tpk_dist2(qx, qy, qz, sx[k], sy[k], sz[k]), si[k]));
            }
        }
        else
        {
            const float q[3] = {qx, qy, qz};
            float t[3], slack[3];
            int c[3];
#pragma unroll
            for (int a = 0; a < 3; ++a)
            {
                t[a] = (q[a] - lo[a]) * inv[a];
                c[a] = tnc_cell(t[a], cells[a]);
                // (what rounding may have moved a point's cell by, in cell widths)
                slack[a] = 1e-5f * (fabsf(t[a]) + static_cast<float>(TNC_AXIS));
            }
            // Distance along axis a, in cell widths, from the query to cell k (0 for its own cell), a lower bound.
            auto to_cell = [&](int a, int k) __attribute__((always_inline)) {
                const float gap = k > c[a] ? static_cast<float>(k) - t[a] : t[a] - static_cast<float>(k + 1);
                return k == c[a] ? 0.0f : fmaxf(gap - slack[a], 0.0f) * width[a];
            };
            // The runs of a box of cells, one per (y, z), point by point.  A run no point of which can beat the
            // third best so far is passed over.  (The index is read only when the distance does not rule it out.)
            auto examine = [&](int x0, int x1, int y0, int y1, int z0, int z1) __attribute__((always_inline)) {
                const int run = x1 - x0 + 1;
                int y = y0, z = z0, pos = 0, end = 0;
                for (;;)
                {
                    if (pos >= end)
                    {
                        if (z > z1)
                            break;
                        const float dy = to_cell(1, y), dz = to_cell(2, z);
                        if (dy * dy + dz * dz < best.third() * 1.00001f || best.third() == __builtin_inff())
                        {
                            const int c0 = x0 + cells[0] * (y + cells[1] * z);
                            pos = starts[c0];
                            end = starts[c0 + run];
                        }
                        if (++y > y1)
                        {
                            y = y0;
                            ++z;
                        }
                        continue;
                    }
                    TPK_WORK_ADD(1);
                    const float d = tpk_dist2(qx, qy, qz, sx[pos], sy[pos], sz[pos]);
                    if (d <= best.third())
                        best.offer(Best3::key(d, si[pos]));
                    ++pos;
                }
            };
            // the block of cells examined so far: at first the cells within one ring of the query's, its own row first
            int xl = max(c[0] - 1, 0), xh = min(c[0] + 1, cells[0] - 1);
            int yl = max(c[1] - 1, 0), yh = min(c[1] + 1, cells[1] - 1);
            int zl = max(c[2] - 1, 0), zh = min(c[2] + 1, cells[2] - 1);
            examine(xl, xh, c[1], c[1], c[2], c[2]);
            if (yl < c[1])
                examine(xl, xh, yl, c[1] - 1, c[2], c[2]);
            if (yh > c[1])
                examine(xl, xh, c[1] + 1, yh, c[2], c[2]);
            if (zl < c[2])
                examine(xl, xh, yl, yh, zl, c[2] - 1);
            if (zh > c[2])
                examine(xl, xh, yl, yh, c[2] + 1, zh);
            for (;;)
            {
                // Final?  Every point not examined lies behind a face of the block that has cells behind it: the
                // faces nearer than the third best so far are pushed out by one layer of cells each, and only
                // the new layers are examined - first along x, then along y over the widened x, then along z.
                const float limit = best.third() * 1.00001f;
                unsigned push = 0;
                {
                    const int bl[3] = {xl, yl, zl}, bh[3] = {xh, yh, zh};
#pragma unroll
                    for (int a = 0; a < 3; ++a)
                    {
                        const float below = fmaxf((t[a] - static_cast<float>(bl[a])) - slack[a], 0.0f) * width[a];
                        const float above = fmaxf((static_cast<float>(bh[a] + 1) - t[a]) - slack[a], 0.0f) * width[a];
                        push |= (bl[a] > 0 && !(limit < below * below)) ? 1u << (2 * a) : 0u;
                        push |= (bh[a] < cells[a] - 1 && !(limit < above * above)) ? 2u << (2 * a) : 0u;
                    }
                }
                if (push == 0)
                    break;
                if (push & 1u)
                {
                    --xl;
                    examine(xl, xl, yl, yh, zl, zh);
                }
                if (push & 2u)
                {
                    ++xh;
                    examine(xh, xh, yl, yh, zl, zh);
                }
                if (push & 4u)
                {
                    --yl;
                    examine(xl, xh, yl, yl, zl, zh);
                }
                if (push & 8u)
                {
                    ++yh;
                    examine(xl, xh, yh, yh, zl, zh);
                }
                if (push & 16u)
                {
                    --zl;
                    examine(xl, xh, yl, yh, zl, zl);
                }
                if (push & 32u)
                {
                    ++zh;
                    examine(xl, xh, yl, yh, zh, zh);
                }
            }
        }
        dist2[j * 3 + 0] = __int_as_float(static_cast<int>(best.k1 >> 32));
        dist2[j * 3 + 1] = __int_as_float(static_cast<int>(best.k2 >> 32));
        dist2[j * 3 + 2] = best.third();
        idx[j * 3 + 0] = static_cast<int>(best.k1 & 0xFFFFFFFFu);
        idx[j * 3 + 1] = static_cast<int>(best.k2 & 0xFFFFFFFFu);
        idx[j * 3 + 2] = static_cast<int>(best.k3 & 0xFFFFFFFFu);
    }
    TPK_WORK_FLUSH
}

int launch_three_nn_cells(int b, int n, int m, const float* unknown, const float* known, float* dist2, int32_t* idx,
                          int* general, hipStream_t stream)
{
    // one workgroup per compute unit where the queries allow it (every workgroup sorts its cloud)
    const int64_t per_cloud = std::max<int64_t>(1, std::min<int64_t>(tpk_ceil_div(n, TNC_THREADS), TPK_COMPUTE_UNITS / b));
    const int per_block = static_cast<int>(tpk_ceil_div(n, per_cloud));
    const int64_t bpc = tpk_ceil_div(n, per_block);
    if (bpc * b > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const size_t lds = tnc_lds_bytes(m);
    const int st = tpk_allow_lds(reinterpret_cast<const void*>(&three_nn_cells_kernel), lds);
    if (st != TPK_OK)
        return st;
    hipLaunchKernelGGL(three_nn_cells_kernel, dim3(static_cast<unsigned>(bpc * b)), dim3(TNC_THREADS), lds, stream, n, m,
                       static_cast<int>(bpc), per_block, unknown, known, dist2, idx, general);
    return tpk_launch_status();
}

} // namespace

extern "C" size_t tpk_three_nn_workspace_bytes(int b, int n, int m)
{
    return tpk_grid_three_nn_workspace_bytes(b, n, m);
}

extern "C" int tpk_three_nn_f32(int b, int n, int m, const float* unknown, const float* known,
                                float* dist2, int32_t* idx, void* workspace, size_t workspace_bytes,
                                void* stream)
{
    if (b < 0 || n < 0 || m < 0)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || n == 0)
        return TPK_OK;
    if (!unknown || !dist2 || !idx || (m > 0 && !known))
        return TPK_ERR_INVALID_ARG;
    if (static_cast<int64_t>(n) * 3 > 0x7fffffffLL || static_cast<int64_t>(m) * 3 > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipStream_t s = tpk_stream(stream);
    if (m >= TNC_MIN_KNOWN && m <= TNC_MAX_KNOWN)
    {
        // The known cloud fits in LDS: a grid there, one lane per query.  It notes the clouds it gives up (uneven
        // density) in the workspace, and the search over curve-ordered cells, enqueued behind it, answers those.
        int* const general = tpk_grid_three_nn_flags(b, n, m, workspace, workspace_bytes);
        const int st = launch_three_nn_cells(b, n, m, unknown, known, dist2, idx, general, s);
        if (st != TPK_OK || !general)
            return st;
        return tpk_grid_three_nn(b, n, m, unknown, known, dist2, idx, workspace, workspace_bytes, true, s);
    }
    if (workspace)
    {
        // Search over curve-ordered cells where it applies; otherwise all pairs.
        const int st = tpk_grid_three_nn(b, n, m, unknown, known, dist2, idx, workspace, workspace_bytes, false, s);
        if (st != TPK_ERR_UNSUPPORTED)
            return st;
    }
    return tpk_three_nn_all_pairs_f32(b, n, m, unknown, known, dist2, idx, stream);
}

extern "C" int tpk_three_nn_all_pairs_f32(int b, int n, int m, const float* unknown, const float* known,
                                          float* dist2, int32_t* idx, void* stream)
{
    if (b < 0 || n < 0 || m < 0)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || n == 0)
        return TPK_OK;
    if (!unknown || !dist2 || !idx || (m > 0 && !known))
        return TPK_ERR_INVALID_ARG;
    if (static_cast<int64_t>(n) * 3 > 0x7fffffffLL || static_cast<int64_t>(m) * 3 > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipStream_t s = tpk_stream(stream);
    // Queries per lane: as many as still leave a few workgroups per compute unit.
    const int64_t queries = static_cast<int64_t>(b) * n;
    if (queries >= 4LL * NN_THREADS * 2048)
        return launch_three_nn<4>(b, n, m, unknown, known, dist2, idx, s);
    if (queries >= 2LL * NN_THREADS * 2048)
        return launch_three_nn<2>(b, n, m, unknown, known, dist2, idx, s);
    return launch_three_nn<1>(b, n, m, unknown, known, dist2, idx, s);
}

// ---------------------------------------------------------------------------------------------
// three_nn for callers that may not allocate device memory (code under graph capture, serving
// loops, harnesses that forbid it).  The curve-ordered copy of both clouds and the cell boxes,
// which tpk_three_nn_f32 takes as a caller-provided workspace, live in a fixed array in device
// memory instead.  Every GPU the library runs on holds its own copy of the array at its own
// address until the process ends; that address is looked up once per device, with that device
// current, and host code uses the looked-up pointer only (the array's name is not a device
// address on the host).  The search overwrites whatever an earlier call left there (nothing has
// to start at zero), so calls that overlap on one GPU - on different streams or from different
// threads - race on it.
// ---------------------------------------------------------------------------------------------
namespace {

constexpr size_t THREE_NN_STATIC_BYTES = TPK_THREE_NN_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[THREE_NN_STATIC_BYTES];

constexpr int SCRATCH_MAX_DEVICES = 64;
std::mutex scratch_lock;
void* scratch_address[SCRATCH_MAX_DEVICES]; // per device, filled at the first call on that device

// Device address of `scratch` on the current device (looked up once per device).
int static_scratch(void** out)
{
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess)
        return static_cast<int>(e);
    if (device < 0 || device >= SCRATCH_MAX_DEVICES)
        return TPK_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (!scratch_address[device])
    {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess)
            return static_cast<int>(e);
        if (!p || (reinterpret_cast<uintptr_t>(p) & 255u))
            return TPK_ERR_WORKSPACE;
        scratch_address[device] = p;
    }
    *out = scratch_address[device];
    return TPK_OK;
}

} // namespace

extern "C" size_t tpk_three_nn_static_scratch_bytes(void)
{
    return THREE_NN_STATIC_BYTES;
}

extern "C" int tpk_three_nn_static_f32(int b, int n, int m, const float* unknown, const float* known,
                                       float* dist2, int32_t* idx, void* stream)
{
    if (b < 0 || n < 0 || m < 0)
        return TPK_ERR_INVALID_ARG;
    const size_t need = tpk_grid_three_nn_workspace_bytes(b, n, m);
    if (need > THREE_NN_STATIC_BYTES)
        return TPK_ERR_TOO_LARGE;
    if (need == 0) // shapes the cell search does not serve use no scratch memory at all
        return tpk_three_nn_f32(b, n, m, unknown, known, dist2, idx, nullptr, 0, stream);
    void* ptr = nullptr;
    const int st = static_scratch(&ptr);
    if (st != TPK_OK)
        return st;
    return tpk_three_nn_f32(b, n, m, unknown, known, dist2, idx, ptr, THREE_NN_STATIC_BYTES, stream);
}
