// A grid over a cloud of up to LG_MAX_POINTS points, built in LDS by a workgroup of LG_THREADS lanes, and the
// search for a query's nearest points in it, one lane per query (three_nn.hip).
//
// Build: bounding box of the finite coordinates, up to LG_AXIS cells per axis and LG_CELLS in all sized for
// about LG_PER_CELL points per cell (a flat cloud gets a flat grid), a count per cell (LDS atomics that also
// hand every point its place inside its cell), a prefix sum, the points written cell by cell as records
// (x, y, z, index) of 16 bytes.  Search: cells are numbered x first, so the (up to) three cells of a row (y, z)
// are one run of consecutive places; a lane walks the runs around its query point by point - its own cell first, a row is
// passed over when its distance in (y, z) already exceeds the bound the lane's best entries set - and the answer
// is final when that bound is smaller than the distance to every face of the examined block that has cells
// behind it; otherwise the faces that are too near are pushed out by one layer of cells each and only the new
// layers are examined.  The lanes of a wavefront examine their runs together - a run takes the wavefront as many
// steps as the longest of its 64 runs has points, about twice the average - and what bounds the search is the issue
// of its instructions (four wavefronts share a SIMD): 17 for a candidate, 45 to set up a run.  The build is
// bound the same way - every instruction of it costs the workgroup 16 clocks - hence the grid's shape comes
// from the first wavefront alone, and a point is one 16-byte record: one LDS write when it is placed, one read
// per candidate (four arrays x, y, z, index: 2.5 us more per call on 16 clouds of 4096 points, 16384 queries each).
#pragma once

#include "tpk_device.h"

namespace {

constexpr int LG_THREADS = 1024;
constexpr int LG_WAVES = LG_THREADS / TPK_WAVE;
constexpr int LG_MAX_POINTS = 8192;
constexpr int LG_PER_THREAD = LG_MAX_POINTS / LG_THREADS;
constexpr int LG_AXIS = 64;    // cells per axis at most
constexpr int LG_CELLS = 4096; // cells in all at most
constexpr int LG_STARTS = LG_CELLS + TPK_WAVE; // the cells' first places, one more for the end, padded
constexpr float LG_PER_CELL = 2.0f;            // points per cell aimed at (1 / 1.5 / 3: 9 / 6 / 1 % slower on three_nn)

// Dynamic LDS a grid over m points takes.
inline size_t lg_lds_bytes(int m)
{
    return static_cast<size_t>(m) * 16 + LG_STARTS * sizeof(int);
}

// Smallest v of every 16-lane row, in all lanes of the row; of the wavefront.
__device__ __forceinline__ float lg_row_min(float v)
{
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true)));
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true)));
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xF, 0xF, true)));
    v = fminf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, true)));
    return v;
}
__device__ __forceinline__ float lg_wave_min(float v)
{
    v = lg_row_min(v);
    return fminf(fminf(tpk_read_lane(v, 0), tpk_read_lane(v, 16)), fminf(tpk_read_lane(v, 32), tpk_read_lane(v, 48)));
}

// Minimum / maximum of two numbers that are not NaN, in one instruction (fminf / fmaxf first turn a signalling
// NaN that cannot occur here into a quiet one, an instruction per operand).
__device__ __forceinline__ float lg_min(float a, float b)
{
    float r;
    asm("v_min_f32_e32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ float lg_max(float a, float b)
{
    float r;
    asm("v_max_f32_e32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
// A float as an integer that orders the same way, and back.
__device__ __forceinline__ int lg_ordered(float f)
{
    const int b = __float_as_int(f);
    return b >= 0 ? b : b ^ 0x7FFFFFFF;
}
__device__ __forceinline__ float lg_unordered(int b)
{
    return __int_as_float(b >= 0 ? b : b ^ 0x7FFFFFFF);
}

// Cell along one axis, clamped to the grid (NaN goes to cell 0).
__device__ __forceinline__ int lg_cell(float t, int cells)
{
    return min(cells - 1, max(0, static_cast<int>(t)));
}

// A (squared distance, index) pair as one integer: distances are >= 0, so their bit patterns order like unsigned
// integers and one 64-bit comparison orders by distance, then index.
__device__ __forceinline__ unsigned long long lg_key(float d, int i)
{
    return (static_cast<unsigned long long>(static_cast<unsigned>(__float_as_int(d))) << 32) | static_cast<unsigned>(i);
}

struct LdsGrid
{
    float4* points;      // [m] the points cell by cell: x, y, z, index
    int* starts;         // [LG_STARTS] first place of every cell, then the number of points
    float lo[3], inv[3], width[3];
    int cells[3];
    float crowd;         // points per cell as a point sees them (3 in a cloud of even density, LG_PER_CELL + 1)
};

// Builds the grid over known[0 .. m) (m <= LG_MAX_POINTS) in `lds` (lg_lds_bytes(m) bytes, 16-byte aligned); the
// points are recorded under index_base + their number.  Every lane of the workgroup calls it; it starts and ends
// with a barrier, so it may follow searches in an earlier grid at the same place.
__device__ __forceinline__ void lds_grid_build(LdsGrid& g, unsigned char* lds, const float* __restrict__ known, int m,
                                               int index_base)
{
    float4* const points = g.points = reinterpret_cast<float4*>(lds);
    int* const starts = g.starts = reinterpret_cast<int*>(points + m);
    __shared__ int box[6];      // ordered ints: min x, y, z then max x, y, z of the finite coordinates
    __shared__ float shape[12]; // lo, inv, width, cells of the grid, from the first wavefront
    __shared__ int wave_totals[LG_WAVES];
    __shared__ int crowding; // sum over the cells of count^2
    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / TPK_WAVE);
    if (tid < 6)
        box[tid] = tid < 3 ? 0x7FFFFFFF : INT_MIN;
    __syncthreads();

    // ---- the cloud's points and bounding box (finite coordinates only) ----
    float px[LG_PER_THREAD], py[LG_PER_THREAD], pz[LG_PER_THREAD];
#pragma unroll
    for (int u = 0; u < LG_PER_THREAD; ++u)
    {
        const int t = min(tid + u * LG_THREADS, m - 1);
        px[u] = known[t * 3 + 0];
        py[u] = known[t * 3 + 1];
        pz[u] = known[t * 3 + 2];
    }
    for (int c = tid; c < LG_STARTS; c += LG_THREADS)
        starts[c] = 0;
    if (tid == 0)
        crowding = 0;
    {
        // (rows past the end repeat the last point: no effect on the box)
        const float inf = __builtin_inff();
        float lows[3] = {inf, inf, inf}, highs[3] = {-inf, -inf, -inf};
#pragma unroll
        for (int u = 0; u < LG_PER_THREAD; ++u)
        {
            const float v[3] = {px[u], py[u], pz[u]};
#pragma unroll
            for (int a = 0; a < 3; ++a)
            {
                const bool finite = fabsf(v[a]) < inf;
                lows[a] = lg_min(lows[a], finite ? v[a] : inf);
                highs[a] = lg_max(highs[a], finite ? v[a] : -inf);
            }
        }
#pragma unroll
        for (int a = 0; a < 3; ++a)
        {
            const int low = ~wave_max_i32(~lg_ordered(lows[a])), high = wave_max_i32(lg_ordered(highs[a]));
            if (lane == 0)
            {
                atomicMin(&box[a], low);
                atomicMax(&box[3 + a], high);
            }
        }
    }
    __syncthreads();

    // ---- the grid: about LG_PER_CELL points per cell, cells as cubic as LG_AXIS per axis and LG_CELLS in
    // all allow (a flat cloud gets a flat grid of up to 64 x 64 cells).  The first wavefront works it out, its
    // lanes trying 64 sizes at a time. ----
    if (wave == 0)
    {
        float low[3], extent[3], longest = 0.0f;
#pragma unroll
        for (int a = 0; a < 3; ++a)
        {
            low[a] = lg_unordered(box[a]);
            extent[a] = lg_unordered(box[3 + a]) - low[a]; // (NaN or -inf for a cloud without finite coordinates)
            extent[a] = extent[a] > 0.0f ? extent[a] : 0.0f;
            longest = fmaxf(longest, extent[a]);
        }
        float share[3]; // of the longest axis
#pragma unroll
        for (int a = 0; a < 3; ++a)
            share[a] = longest > 0.0f ? extent[a] / longest : 0.0f;
        // cells per axis for `along` cells along the longest axis, and their product
        auto fit = [&](float along, int (&count)[3]) __attribute__((always_inline)) {
            int all = 1;
#pragma unroll
            for (int a = 0; a < 3; ++a)
            {
                const float f = longest > 0.0f ? fminf(share[a] * along + 0.5f, static_cast<float>(LG_AXIS)) : 1.0f;
                count[a] = f >= 1.0f ? static_cast<int>(f) : 1;
                all *= count[a];
            }
            return all;
        };
        // (the product grows with `along`: the largest of the sizes tried that stays within the cells wanted, in
        // steps of 2 up to 2 * LG_AXIS, then in steps of 1 / 32 inside the step found)
        const int wanted = static_cast<int>(fminf(static_cast<float>(LG_CELLS), fmaxf(static_cast<float>(m) / LG_PER_CELL, 1.0f)));
        int count[3];
        const int coarse = __builtin_popcountll(__ballot(fit(2.0f * static_cast<float>(lane + 1), count) <= wanted));
        const int fine = __builtin_popcountll(__ballot(fit(2.0f * static_cast<float>(coarse) + static_cast<float>(lane + 1) * (1.0f / 32.0f), count) <= wanted));
        fit(2.0f * static_cast<float>(coarse) + static_cast<float>(fine) * (1.0f / 32.0f), count);
        if (lane < 3)
        {
            const float e = lane == 0 ? extent[0] : lane == 1 ? extent[1] : extent[2];
            const float l = lane == 0 ? low[0] : lane == 1 ? low[1] : low[2];
            const int k = lane == 0 ? count[0] : lane == 1 ? count[1] : count[2];
            shape[lane] = e > 0.0f ? l : 0.0f;
            shape[3 + lane] = e > 0.0f ? static_cast<float>(k) / e : 0.0f;
            shape[6 + lane] = e / static_cast<float>(k);
            shape[9 + lane] = __int_as_float(k);
        }
    }
    __syncthreads();
    float lo[3], inv[3], width[3];
    int cells[3];
#pragma unroll
    for (int a = 0; a < 3; ++a)
    {
        lo[a] = shape[a];
        inv[a] = shape[3 + a];
        width[a] = shape[6 + a];
        cells[a] = __float_as_int(shape[9 + a]);
    }

    // ---- count per cell; the count before a point's own increment is its place inside the cell ----
    int placed[LG_PER_THREAD];
#pragma unroll
    for (int u = 0; u < LG_PER_THREAD; ++u)
        if (tid + u * LG_THREADS < m)
        {
            const int c = lg_cell((px[u] - lo[0]) * inv[0], cells[0]) +
                          cells[0] * (lg_cell((py[u] - lo[1]) * inv[1], cells[1]) + cells[1] * lg_cell((pz[u] - lo[2]) * inv[2], cells[2]));
            placed[u] = (c << 16) | atomicAdd(&starts[c], 1);
        }
    __syncthreads();
    {
        // exclusive prefix sum over the cells, four per thread
        static_assert(LG_CELLS == 4 * LG_THREADS, "four cells per thread");
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
        const int total = lane < LG_WAVES ? wave_totals[lane] : 0;
        int at = __builtin_amdgcn_readlane(wave_exclusive_sum(total), wave) + before;
        int4 s4;
        s4.x = at;
        s4.y = at += c4.x;
        s4.z = at += c4.y;
        s4.w = at += c4.z;
        reinterpret_cast<int4*>(starts)[tid] = s4;
        if (tid == LG_THREADS - 1)
            starts[LG_CELLS] = at + c4.w;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < LG_PER_THREAD; ++u)
        if (tid + u * LG_THREADS < m)
        {
            const int at = starts[placed[u] >> 16] + (placed[u] & 0xFFFF);
            points[at] = make_float4(px[u], py[u], pz[u], __int_as_float(index_base + tid + u * LG_THREADS));
        }
    __syncthreads();
    g.crowd = static_cast<float>(crowding) / static_cast<float>(m);
#pragma unroll
    for (int a = 0; a < 3; ++a)
    {
        g.lo[a] = lo[a];
        g.inv[a] = inv[a];
        g.width[a] = width[a];
        g.cells[a] = cells[a];
    }
}

// The nearest points of (qx, qy, qz) in the grid, offered to `best`: Best has bound() - the squared distance a
// candidate must not exceed to matter, +inf while entries are missing - and offer(key) for a lg_key that may enter.
template <typename Best>
__device__ __forceinline__ void lds_grid_search(const LdsGrid& g, float qx, float qy, float qz, Best& best TPK_WORK_PARAM)
{
    const float4* const points = g.points;
    const int* const starts = g.starts;
    const float(&lo)[3] = g.lo;
    const float(&inv)[3] = g.inv;
    const float(&width)[3] = g.width;
    const int(&cells)[3] = g.cells;
    const float q[3] = {qx, qy, qz};
    float t[3], slack[3];
    int c[3];
#pragma unroll
    for (int a = 0; a < 3; ++a)
    {
        t[a] = (q[a] - lo[a]) * inv[a];
        c[a] = lg_cell(t[a], cells[a]);
        // (what rounding may have moved a point's cell by, in cell widths)
        slack[a] = 1e-5f * (fabsf(t[a]) + static_cast<float>(LG_AXIS));
    }
    // Distance along axis a, in cell widths, from the query to cell k (0 for its own cell), a lower bound.
    auto to_cell = [&](int a, int k) __attribute__((always_inline)) {
        const float gap = k > c[a] ? static_cast<float>(k) - t[a] : t[a] - static_cast<float>(k + 1);
        return k == c[a] ? 0.0f : fmaxf(gap - slack[a], 0.0f) * width[a];
    };
    // The runs of a box of cells, one per (y, z), point by point.  A run no point of which can beat the
    // bound so far is passed over.
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
                if (dy * dy + dz * dz < best.bound() * 1.00001f || best.bound() == __builtin_inff())
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
            const float4 p = points[pos];
            const float d = tpk_dist2(qx, qy, qz, p.x, p.y, p.z);
            if (d <= best.bound())
                best.offer(lg_key(d, __float_as_int(p.w)));
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
        // faces nearer than the bound so far are pushed out by one layer of cells each, and only
        // the new layers are examined - first along x, then along y over the widened x, then along z.
        const float limit = best.bound() * 1.00001f;
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

// The same by a scan of all m points (broadcast reads): for clouds that crowd into few cells.
template <typename Best>
__device__ __forceinline__ void lds_grid_scan_all(const LdsGrid& g, int m, float qx, float qy, float qz, Best& best TPK_WORK_PARAM)
{
    for (int k = 0; k < m; ++k)
    {
        TPK_WORK_ADD(1);
        const float4 p = g.points[k];
        const float d = tpk_dist2(qx, qy, qz, p.x, p.y, p.z);
        if (d <= best.bound())
            best.offer(lg_key(d, __float_as_int(p.w)));
    }
}

} // namespace
