// A coarse spatial order for clouds of more than one window.
//
// The ordering kernel (curve_cells.h) orders windows of at most CURVE_MAX_POINTS consecutive points.  A cloud of
// several windows, taken as it comes, gives windows that each span the whole cloud, and cells of 64 points as wide
// as if the cloud had 16384 points.  Here the rows of every cloud of a batch - clouds of the same size, more than
// one chunk each - are first brought into the order of the 4096 cells of a 16^3 grid over the cloud's bounding
// box, along the same curve as inside a window, so that consecutive windows of the result are compact
// neighbourhoods; the ordering kernel then reads the result instead of the caller's array.  The result is an array
// of records (x, y, z, number the row had inside its cloud); a cloud's rows are permuted among its own places.
//
// A counting sort over chunks of CO_CHUNK rows of the batch, four launches: (1) every chunk finds the bounding box
// of its rows of either of the (at most two) clouds it holds rows of - the cloud of its first row and the cloud of
// its last row; (2) every chunk forms the boxes of its clouds from the chunks' boxes, counts its rows per cell and
// gives every row its rank among the chunk's rows of the same cell; (3) one workgroup per cloud turns the counts of
// the cloud's chunks into first places, cell after cell and inside a cell chunk after chunk; (4) every row goes to
// its place.
#pragma once

#include "curve_cells.h"

namespace {

constexpr int CO_THREADS = NG_SORT_THREADS;
constexpr int CO_CHUNK = CURVE_MAX_POINTS;
constexpr int CO_PER = CO_CHUNK / CO_THREADS;
constexpr int CO_SHIFT = 14;
static_assert((1 << CO_SHIFT) == CO_CHUNK, "a place is (cell << CO_SHIFT) | rank");
constexpr int CO_MIN_ROWS = CO_CHUNK + 1; // rows of a cloud at least: a chunk then holds rows of two clouds at most

struct CoarseOrder
{
    const float* xyz;     // [rows][3]
    int rows;             // of the batch: clouds of cloud_rows consecutive rows
    int cloud_rows;
    float4* records;      // out [rows]
    unsigned* places;     // [rows] (cell << CO_SHIFT) | rank among the chunk's rows of the cell
    int4* spans;          // [chunks] rows [x, y) of the cloud the chunk's first row lies in, [z, w) of the cloud that
                          // begins inside the chunk; (0, 0): none
    int* boxes;           // [chunks][2][6] ordered ints: box of the chunk's rows of either cloud
    int* counts;          // [chunks][2][CURVE_BINS] rows per cell, then first places inside the cloud
};

inline int co_chunks(int64_t rows)
{
    return static_cast<int>((rows + CO_CHUNK - 1) / CO_CHUNK);
}

// Bytes of the scratch arrays behind the records (places, spans, boxes, counts), 256-byte aligned each.
struct CoarseLayout
{
    size_t records, places, spans, boxes, counts, total;
};
inline CoarseLayout coarse_layout(int64_t rows)
{
    auto up = [](size_t v) { return (v + 255) & ~static_cast<size_t>(255); };
    const size_t chunks = static_cast<size_t>(co_chunks(rows));
    CoarseLayout l;
    size_t pos = 0;
    l.records = pos;
    pos = up(pos + static_cast<size_t>(rows) * sizeof(float4));
    l.places = pos;
    pos = up(pos + static_cast<size_t>(rows) * sizeof(unsigned));
    l.spans = pos;
    pos = up(pos + chunks * sizeof(int4));
    l.boxes = pos;
    pos = up(pos + chunks * 12 * sizeof(int));
    l.counts = pos;
    pos = up(pos + chunks * 2 * CURVE_BINS * sizeof(int));
    l.total = pos;
    return l;
}

// Which of a chunk's two clouds a cloud that begins at row `begin` is in chunk `chunk`: the second where it
// begins inside the chunk, the first where it holds the chunk's first row.
__device__ __forceinline__ int co_slot(int begin, int chunk)
{
    return begin > chunk * CO_CHUNK ? 1 : 0;
}

// (1) spans and boxes of a chunk.
__global__ __launch_bounds__(CO_THREADS) void coarse_spans_kernel(CoarseOrder job)
{
    __shared__ int4 span;
    __shared__ int box[12];
    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int chunk = blockIdx.x;
    const int first = chunk * CO_CHUNK;
    const int n = min(CO_CHUNK, job.rows - first);
    const float* __restrict__ xyz = job.xyz + static_cast<int64_t>(first) * 3;

    // the rows of this thread: tid, tid + 1024, ... (all requested before the first is used)
    float p[CO_PER][3];
#pragma unroll
    for (int u = 0; u < CO_PER; ++u)
    {
        const int k = min(tid + u * CO_THREADS, n - 1);
#pragma unroll
        for (int a = 0; a < 3; ++a)
            p[u][a] = xyz[k * 3 + a];
    }
    if (tid < 12)
        box[tid] = tid % 6 < 3 ? 0x7FFFFFFF : INT_MIN;
    if (tid < TPK_WAVE)
    {
        const int last = first + n - 1;
        const int a0 = first / job.cloud_rows * job.cloud_rows, a1 = a0 + job.cloud_rows;
        int b0 = 0, b1 = 0;
        if (last >= a1)
        {
            b0 = a1;
            b1 = b0 + job.cloud_rows;
        }
        if (tid == 0)
        {
            span = make_int4(a0, a1, b0, b1);
            job.spans[chunk] = span;
        }
    }
    __syncthreads();
    const int4 s = span;
#pragma unroll
    for (int slot = 0; slot < 2; ++slot)
    {
        const int begin = slot ? s.z : s.x, end = slot ? s.w : s.y;
        if (end == 0)
            continue;
        int lo[3] = {0x7FFFFFFF, 0x7FFFFFFF, 0x7FFFFFFF}, hi[3] = {INT_MIN, INT_MIN, INT_MIN};
#pragma unroll
        for (int u = 0; u < CO_PER; ++u)
        {
            const int row = first + tid + u * CO_THREADS;
            const bool in = tid + u * CO_THREADS < n && row >= begin && row < end;
#pragma unroll
            for (int a = 0; a < 3; ++a)
            {
                // (finite coordinates only: the others fall into the first or last cell of their axis)
                const int o = float_to_ordered_int(p[u][a]);
                const bool takes_part = in && fabsf(p[u][a]) < __builtin_inff();
                lo[a] = takes_part ? min(lo[a], o) : lo[a];
                hi[a] = takes_part ? max(hi[a], o) : hi[a];
            }
        }
#pragma unroll
        for (int a = 0; a < 3; ++a)
        {
            const int wave_lo = wave_min_i32(lo[a]), wave_hi = wave_max_i32(hi[a]);
            if (lane == 0)
            {
                atomicMin(&box[slot * 6 + a], wave_lo);
                atomicMax(&box[slot * 6 + 3 + a], wave_hi);
            }
        }
    }
    __syncthreads();
    if (tid < 12)
        job.boxes[chunk * 12 + tid] = box[tid];
}

// (2) cells, counts and ranks of a chunk's rows.
__global__ __launch_bounds__(CO_THREADS) void coarse_count_kernel(CoarseOrder job)
{
    __shared__ int counts[2][CURVE_BINS];
    __shared__ int box[12];
    const int tid = threadIdx.x;
    const int chunk = blockIdx.x;
    const int first = chunk * CO_CHUNK;
    const int n = min(CO_CHUNK, job.rows - first);
    const int4 s = job.spans[chunk];
    const float* __restrict__ xyz = job.xyz + static_cast<int64_t>(first) * 3;
    float p[CO_PER][3];
#pragma unroll
    for (int u = 0; u < CO_PER; ++u)
    {
        const int k = min(tid + u * CO_THREADS, n - 1);
#pragma unroll
        for (int a = 0; a < 3; ++a)
            p[u][a] = xyz[k * 3 + a];
    }
    if (tid < 12)
        box[tid] = tid % 6 < 3 ? 0x7FFFFFFF : INT_MIN;
    for (int i = tid; i < 2 * CURVE_BINS; i += CO_THREADS)
        (&counts[0][0])[i] = 0;
    __syncthreads();
    // the boxes of the two clouds: over all chunks that hold rows of them
#pragma unroll
    for (int slot = 0; slot < 2; ++slot)
    {
        const int begin = slot ? s.z : s.x, end = slot ? s.w : s.y;
        if (end == 0)
            continue;
        const int c0 = begin >> CO_SHIFT, c1 = (end - 1) >> CO_SHIFT;
        for (int i = tid; i < (c1 - c0 + 1) * 6; i += CO_THREADS)
        {
            const int c = c0 + i / 6, a = i % 6;
            const int v = job.boxes[c * 12 + co_slot(begin, c) * 6 + a];
            if (a < 3)
                atomicMin(&box[slot * 6 + a], v);
            else
                atomicMax(&box[slot * 6 + a], v);
        }
    }
    __syncthreads();
    const CurveGrid grid_a = curve_grid(box), grid_b = curve_grid(box + 6);
    unsigned place[CO_PER];
#pragma unroll
    for (int u = 0; u < CO_PER; ++u)
    {
        const int row = first + tid + u * CO_THREADS;
        place[u] = 0;
        if (tid + u * CO_THREADS >= n)
            continue;
        const bool in_a = row < s.y; // (else in the second cloud)
        const CurveGrid& grid = in_a ? grid_a : grid_b;
        unsigned cell[3];
#pragma unroll
        for (int a = 0; a < 3; ++a)
            cell[a] = curve_grid_cell(p[u][a], grid.lo[a], grid.scale[a]);
        const unsigned bin = curve_bin_table.bin[(cell[0] >> 2) | ((cell[1] >> 2) << 4) | ((cell[2] >> 2) << 8)];
        place[u] = (bin << CO_SHIFT) | static_cast<unsigned>(atomicAdd(&counts[in_a ? 0 : 1][bin], 1));
    }
#pragma unroll
    for (int u = 0; u < CO_PER; ++u)
        if (tid + u * CO_THREADS < n)
            job.places[first + tid + u * CO_THREADS] = place[u];
    __syncthreads();
    for (int i = tid; i < 2 * CURVE_BINS; i += CO_THREADS)
        if ((i < CURVE_BINS ? s.y : s.w) != 0)
            job.counts[static_cast<int64_t>(chunk) * 2 * CURVE_BINS + i] = (&counts[0][0])[i];
}

// (3) first places: workgroup 2 * chunk + slot serves the cloud that begins in that chunk as that slot.
__global__ __launch_bounds__(CO_THREADS) void coarse_scan_kernel(CoarseOrder job)
{
    __shared__ int wave_totals[CO_THREADS / TPK_WAVE];
    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / TPK_WAVE);
    const int chunk = blockIdx.x >> 1, slot = blockIdx.x & 1;
    const int4 s = job.spans[chunk];
    const int begin = slot ? s.z : s.x, end = slot ? s.w : s.y;
    if (end == 0 || (begin >> CO_SHIFT) != chunk || co_slot(begin, chunk) != slot)
        return;
    static_assert(CURVE_BINS == 4 * CO_THREADS, "four cells per thread");
    const int c0 = chunk, c1 = (end - 1) >> CO_SHIFT;
    int4* __restrict__ counts = reinterpret_cast<int4*>(job.counts);
    auto at = [&](int c) { return (static_cast<int64_t>(c) * 2 + co_slot(begin, c)) * (CURVE_BINS / 4) + tid; };
    int4 total = make_int4(0, 0, 0, 0);
    for (int c = c0; c <= c1; ++c)
    {
        const int4 v = counts[at(c)];
        total.x += v.x;
        total.y += v.y;
        total.z += v.z;
        total.w += v.w;
    }
    const int own = total.x + total.y + total.z + total.w;
    const int before = wave_exclusive_sum(own);
    if (lane == TPK_WAVE - 1)
        wave_totals[wave] = before + own;
    __syncthreads();
    const int waves_sum = lane < CO_THREADS / TPK_WAVE ? wave_totals[lane] : 0;
    int4 run;
    run.x = __builtin_amdgcn_readlane(wave_exclusive_sum(waves_sum), wave) + before;
    run.y = run.x + total.x;
    run.z = run.y + total.y;
    run.w = run.z + total.z;
    for (int c = c0; c <= c1; ++c)
    {
        const int4 v = counts[at(c)];
        counts[at(c)] = run;
        run.x += v.x;
        run.y += v.y;
        run.z += v.z;
        run.w += v.w;
    }
}

// (4) every row to its place.
__global__ __launch_bounds__(CO_THREADS) void coarse_place_kernel(CoarseOrder job)
{
    const int tid = threadIdx.x;
    const int chunk = blockIdx.x;
    const int first = chunk * CO_CHUNK;
    const int n = min(CO_CHUNK, job.rows - first);
    const int4 s = job.spans[chunk];
    const float* __restrict__ xyz = job.xyz + static_cast<int64_t>(first) * 3;
    const int* __restrict__ counts = job.counts + static_cast<int64_t>(chunk) * 2 * CURVE_BINS;
#pragma unroll 4
    for (int k = tid; k < n; k += CO_THREADS)
    {
        const int row = first + k;
        const unsigned place = job.places[row];
        const float x = xyz[k * 3 + 0], y = xyz[k * 3 + 1], z = xyz[k * 3 + 2];
        const bool in_a = row < s.y;
        const int begin = in_a ? s.x : s.z;
        const int to = begin + counts[(in_a ? 0 : CURVE_BINS) + (place >> CO_SHIFT)] + static_cast<int>(place & (CO_CHUNK - 1));
        job.records[to] = make_float4(x, y, z, __int_as_float(row - begin));
    }
}

// Enqueues the four kernels.  `scratch`: coarse_layout(rows).total bytes, 256-byte aligned; the records lie at its
// start.
inline int launch_coarse_order(const float* xyz, int64_t rows, int64_t cloud_rows, void* scratch, hipStream_t s)
{
    if (rows <= 0 || rows >= (1LL << 30) || cloud_rows < CO_MIN_ROWS || cloud_rows > rows)
        return TPK_ERR_UNSUPPORTED;
    const CoarseLayout l = coarse_layout(rows);
    char* const w = static_cast<char*>(scratch);
    CoarseOrder job{xyz, static_cast<int>(rows), static_cast<int>(cloud_rows), reinterpret_cast<float4*>(w + l.records), reinterpret_cast<unsigned*>(w + l.places),
                    reinterpret_cast<int4*>(w + l.spans), reinterpret_cast<int*>(w + l.boxes),
                    reinterpret_cast<int*>(w + l.counts)};
    const unsigned chunks = static_cast<unsigned>(co_chunks(rows));
    hipLaunchKernelGGL(coarse_spans_kernel, dim3(chunks), dim3(CO_THREADS), 0, s, job);
    hipLaunchKernelGGL(coarse_count_kernel, dim3(chunks), dim3(CO_THREADS), 0, s, job);
    hipLaunchKernelGGL(coarse_scan_kernel, dim3(2 * chunks), dim3(CO_THREADS), 0, s, job);
    hipLaunchKernelGGL(coarse_place_kernel, dim3(chunks), dim3(CO_THREADS), 0, s, job);
    return tpk_launch_status();
}

} // namespace
