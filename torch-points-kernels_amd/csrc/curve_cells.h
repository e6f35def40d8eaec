// Curve-ordered cells of point sets: the kernel that orders windows of at most CURVE_MAX_POINTS
// points along the curve (curve_order.h) and writes them out as cells of 64 records with their
// bounding boxes, for the searches that skip whole cells (nn_grid.hip) and for furthest point
// sampling of clouds too large for registers (fps.hip).
#pragma once

#include "curve_order.h"

namespace {

constexpr int NG_CELL = 64;           // points per cell = lanes of a wavefront
constexpr int NG_SORT_THREADS = 1024;
constexpr int NG_BOX = 10;            // float4 per cell: box of the cell, then of its four runs of 16 points

// A set of points to be ordered: `total` points in clouds of `cloud_points` consecutive points,
// every cloud cut into windows of `stride` consecutive points (the last window of a cloud may be
// shorter; a packed array of unequal clouds is one "cloud" whose windows hold whatever clouds
// lie there).  Every window gets stride / 64 (rounded up) cells of 64 records, in curve order; a record is (x, y, z, index inside the cloud), the
// padding records are infinitely far away with index 0x7FFFFFFF; a cell without points has an
// empty box (lo = +inf, hi = -inf).
struct PointSet
{
    const float* xyz;     // [total][3]
    const int64_t* group; // optional sorted cloud id per point (packed arrays), or nullptr
    int64_t total;
    int64_t cloud_points;
    int stride;
    float4* sorted;       // [windows][cells * 64]
    float4* boxes;        // [windows][cells][NG_BOX]: (lo.xyz, -), (hi.xyz, -) of the cell and of its quarters; or nullptr
    int* bin_ends;        // optional [windows][CURVE_BINS]: end of every bin of the counting sort
    float4* grid;         // optional [windows][2]: origin and scale of the window's 64^3 grid
    int* wide_first;      // optional (with boxes) [windows][cells]: the window's cells, those with much wider boxes than
                          // the window's average first - the cells whose queries take a search longest
    const int* only;      // optional [clouds]: a cloud whose word is 0 is left out (dense layout)
    const float4* records; // optional [total]: the points as (x, y, z, index) records to be read instead of xyz -
                           // an array that has been brought into a coarse order (coarse_order.h), whose records
                           // carry the numbers the points had before
};

__host__ __device__ inline int set_cells(const PointSet& s)
{
    return (s.stride + NG_CELL - 1) / NG_CELL;
}
__host__ __device__ inline int set_windows_per_cloud(const PointSet& s)
{
    return static_cast<int>((s.cloud_points + s.stride - 1) / s.stride);
}
__host__ __device__ inline int64_t set_windows(const PointSet& s)
{
    return s.total > 0 ? (s.total / s.cloud_points) * set_windows_per_cloud(s) : 0;
}

// The equal range [first, last) of value v in sorted a[0..len), found by the whole wavefront: 64
// samples per round instead of one, and both ends in the same rounds, so that their loads
// travel together.
__device__ __forceinline__ void wave_equal_range(const int64_t* __restrict__ a, int len, int64_t v, int lane,
                                                 int& first, int& last)
{
    int lo0 = 0, hi0 = len, lo1 = 0, hi1 = len;
    while (hi0 > lo0 || hi1 > lo1)
    {
        const int step0 = (hi0 - lo0 + TPK_WAVE - 1) / TPK_WAVE, step1 = (hi1 - lo1 + TPK_WAVE - 1) / TPK_WAVE;
        const int pos0 = lo0 + lane * step0, pos1 = lo1 + lane * step1;
        const bool in0 = pos0 < hi0, in1 = pos1 < hi1;
        const int64_t sample0 = a[in0 ? pos0 : 0], sample1 = a[in1 ? pos1 : 0];
        const unsigned long long ge0 = __ballot(!in0 || sample0 >= v);
        const unsigned long long ge1 = __ballot(!in1 || sample1 > v);
        if (hi0 > lo0)
        {
            const int f = ge0 ? __builtin_ctzll(ge0) : TPK_WAVE;
            const int next_lo = f > 0 ? lo0 + (f - 1) * step0 + 1 : lo0;
            hi0 = f < TPK_WAVE ? min(lo0 + f * step0, hi0) : hi0;
            lo0 = next_lo;
        }
        if (hi1 > lo1)
        {
            const int f = ge1 ? __builtin_ctzll(ge1) : TPK_WAVE;
            const int next_lo = f > 0 ? lo1 + (f - 1) * step1 + 1 : lo1;
            hi1 = f < TPK_WAVE ? min(lo1 + f * step1, hi1) : hi1;
            lo1 = next_lo;
        }
    }
    first = lo0;
    last = lo1;
}

// Work that rides along with an ordering launch, in workgroups of its own behind those of the
// windows: for every query of a packed call, the rows [x, y) of the support points that carry
// the query's cloud id (both id arrays sorted).  A wavefront takes 64 consecutive queries and
// searches once per distinct id among them - nearly always one.
struct CloudRows
{
    const int64_t* batch_x;
    const int64_t* batch_y;
    int size_x;
    int64_t size_y;
    int2* rows;
};

__device__ __forceinline__ void cloud_rows_job(const CloudRows& job, int64_t group, int tid)
{
    const int lane = tid & (TPK_WAVE - 1);
    const int64_t q = (group * (NG_SORT_THREADS / TPK_WAVE) + tid / TPK_WAVE) * TPK_WAVE + lane;
    const bool has = q < job.size_y;
    const int64_t mine = has ? job.batch_y[q] : 0;
    unsigned long long todo = __ballot(has);
    while (todo != 0)
    {
        const int64_t id = __shfl(mine, __builtin_ctzll(todo));
        int first, last;
        wave_equal_range(job.batch_x, job.size_x, id, lane, first, last);
        const bool same = has && mine == id;
        if (same)
            job.rows[q] = make_int2(first, last);
        todo &= ~__ballot(same); // (the lane that gave the id is among them: the loop ends)
    }
}

constexpr float CURVE_WIDE_FACTOR = 3.0f; // a cell is wide when its box's squared diagonal exceeds this many times the window's average

// One workgroup orders one window: the first windows_a blocks those of set_a, the rest set_b.
// `zero_word` (optional) is cleared by the first block: a counter used by the kernel that follows.
// The window's points are read once and stay in registers (16 per thread): bounding box, curve
// position of each point's cell of the 16^3 grid (a table in LDS), histogram and prefix sum over the
// 4096 bins, and then every thread takes a place in its points' bins (LDS integer atomics) and stores
// the records straight to their final positions.  The boxes of the cells are formed from the records
// read back in order (one more trip to the L2 instead of random gathers of the coordinates).
// Inside a bin (1/16 of the window's extent per axis) the order is that in which the atomics were
// served; it decides where a point sits inside its bin, never what a search over the cells returns.
// dynamic LDS: (2 * CURVE_BINS + 24 * cells) words.
__global__ __launch_bounds__(NG_SORT_THREADS) void curve_cells_kernel(PointSet set_a, PointSet set_b,
                                                                      int windows_a, int windows, int* zero_word,
                                                                      CloudRows rows_job)
{
    extern __shared__ unsigned bin_of_cell[];  // [CURVE_BINS] curve position of every cell of the 16^3 grid
    int* const bins = reinterpret_cast<int*>(bin_of_cell) + CURVE_BINS; // [CURVE_BINS]
    int* const run_boxes = bins + CURVE_BINS;  // [cells * 4][6] ordered ints: boxes of the runs of 16 records
    __shared__ int cloud_box[6];
    __shared__ int wave_totals[NG_SORT_THREADS / TPK_WAVE];
    __shared__ float wide_sums[NG_SORT_THREADS / TPK_WAVE];
    constexpr int PER = CURVE_MAX_POINTS / NG_SORT_THREADS; // points per thread
    static_assert(CURVE_BINS % NG_SORT_THREADS == 0, "every thread scans the same number of bins");

    if (static_cast<int>(blockIdx.x) >= windows)
    {
        cloud_rows_job(rows_job, static_cast<int>(blockIdx.x) - windows, threadIdx.x);
        return;
    }
    const bool first_set = static_cast<int>(blockIdx.x) < windows_a;
    const PointSet set = first_set ? set_a : set_b;
    const int64_t window = first_set ? blockIdx.x : blockIdx.x - windows_a;
    const int per_cloud = set_windows_per_cloud(set);
    const int64_t in_cloud = (window % per_cloud) * static_cast<int64_t>(set.stride);
    const int64_t start = (window / per_cloud) * set.cloud_points + in_cloud;
    const int n = static_cast<int>(tpk_min64(set.stride, set.cloud_points - in_cloud));
    const int cells = set_cells(set);
    const float* __restrict__ xyz = set.xyz + start * 3;
    const float4* __restrict__ records = set.records ? set.records + start : nullptr;
    const int64_t* __restrict__ group = set.group ? set.group + start : nullptr;
    float4* __restrict__ sorted = set.sorted + window * cells * NG_CELL;
    float4* __restrict__ boxes = set.boxes ? set.boxes + window * cells * NG_BOX : nullptr;
    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / TPK_WAVE);
    if (zero_word && blockIdx.x == 0 && tid == 0)
        *zero_word = 0;
    if (set.only && set.only[window / per_cloud] == 0)
        return; // (before the first barrier)

    // the points of this thread: tid, tid + 1024, ... (all loads issued before the first is used)
    float p[PER][3];
#pragma unroll
    for (int u = 0; u < PER; ++u)
    {
        const int k = min(tid + u * NG_SORT_THREADS, n - 1);
        if (records)
        {
            const float4 r = records[k];
            p[u][0] = r.x;
            p[u][1] = r.y;
            p[u][2] = r.z;
        }
        else
        {
#pragma unroll
            for (int a = 0; a < 3; ++a)
                p[u][a] = xyz[k * 3 + a];
        }
    }
    // (with cloud ids: how far a point's id lies above the window's first, cut at 7)
    int id_offset[PER];
    if (group)
    {
        const int64_t first_group = group[0];
#pragma unroll
        for (int u = 0; u < PER; ++u)
            id_offset[u] = static_cast<int>(tpk_min64(group[min(tid + u * NG_SORT_THREADS, n - 1)] - first_group, 7));
    }

    const int empty_lo = float_to_ordered_int(__builtin_inff());
    const int empty_hi = float_to_ordered_int(-__builtin_inff());
    if (tid < 6)
        cloud_box[tid] = tid < 3 ? empty_lo : empty_hi;
    for (int i = tid; i < CURVE_BINS; i += NG_SORT_THREADS)
    {
        bins[i] = 0;
        bin_of_cell[i] = curve_bin_table.bin[i]; // (= curve_bin_of_cell(i & 15, (i >> 4) & 15, i >> 8))
    }
    __syncthreads();
    {
        // box of the window (only to quantise coordinates for the curve); the clamped loads repeat a real point
        float lo[3], hi[3];
#pragma unroll
        for (int a = 0; a < 3; ++a)
        {
            lo[a] = hi[a] = p[0][a];
#pragma unroll
            for (int u = 1; u < PER; ++u)
            {
                lo[a] = fminf(lo[a], p[u][a]);
                hi[a] = fmaxf(hi[a], p[u][a]);
            }
            const int wave_lo = wave_min_i32(float_to_ordered_int(lo[a]));
            const int wave_hi = wave_max_i32(float_to_ordered_int(hi[a]));
            if (lane == 0)
            {
                atomicMin(&cloud_box[a], wave_lo);
                atomicMax(&cloud_box[3 + a], wave_hi);
            }
        }
    }
    __syncthreads();

    // the bin of every point: position on the curve of its cell of the 16^3 grid (with cloud ids: the
    // first 7 distinct-id offsets come first, one id after the other, each in curve order; the rest together)
    int bin[PER];
    {
        const CurveGrid grid = curve_grid(cloud_box);
#pragma unroll
        for (int u = 0; u < PER; ++u)
        {
            bin[u] = 0;
            if (u * NG_SORT_THREADS >= n) // (uniform over the workgroup: a short window has fewer rounds)
                continue;
            unsigned cell[3];
#pragma unroll
            for (int a = 0; a < 3; ++a)
                cell[a] = curve_grid_cell(p[u][a], grid.lo[a], grid.scale[a]);
            unsigned b = bin_of_cell[(cell[0] >> 2) | ((cell[1] >> 2) << 4) | ((cell[2] >> 2) << 8)];
            if (group)
            {
                b = (static_cast<unsigned>(id_offset[u]) << 9) | (b >> 3);
            }
            bin[u] = static_cast<int>(b);
            if (tid + u * NG_SORT_THREADS < n)
                atomicAdd(&bins[b], 1);
        }
    }
    __syncthreads();
    {
        // exclusive prefix sum over the bins: where every bin starts
        int count[CURVE_BINS / NG_SORT_THREADS];
        int sum = 0;
#pragma unroll
        for (int i = 0; i < CURVE_BINS / NG_SORT_THREADS; ++i)
        {
            count[i] = bins[tid * (CURVE_BINS / NG_SORT_THREADS) + i];
            sum += count[i];
        }
        const int before_in_wave = wave_exclusive_sum(sum);
        if (lane == TPK_WAVE - 1)
            wave_totals[wave] = before_in_wave + sum;
        __syncthreads();
        int run = before_in_wave;
        for (int w = 0; w < wave; ++w)
            run += wave_totals[w];
#pragma unroll
        for (int i = 0; i < CURVE_BINS / NG_SORT_THREADS; ++i)
        {
            bins[tid * (CURVE_BINS / NG_SORT_THREADS) + i] = run;
            run += count[i];
        }
    }
    __syncthreads();
    // every point takes the next place of its bin; its record goes straight there
    {
        int place[PER];
#pragma unroll
        for (int u = 0; u < PER; ++u)
            place[u] = tid + u * NG_SORT_THREADS < n ? atomicAdd(&bins[bin[u]], 1) : -1;
        // (records: the number a point had before the coarse order - read once more, the line is still near)
        int number[PER];
#pragma unroll
        for (int u = 0; u < PER; ++u)
            number[u] = static_cast<int>(in_cloud) + tid + u * NG_SORT_THREADS;
        if (records)
        {
#pragma unroll
            for (int u = 0; u < PER; ++u)
                if (place[u] >= 0)
                    number[u] = __float_as_int(records[tid + u * NG_SORT_THREADS].w);
        }
#pragma unroll
        for (int u = 0; u < PER; ++u)
            if (place[u] >= 0)
                sorted[place[u]] = make_float4(p[u][0], p[u][1], p[u][2], __int_as_float(number[u]));
    }
    const int padded = cells * NG_CELL;
    {
        // records behind the last point: infinitely far away
        const float inf = __builtin_inff();
        for (int q = n + tid; q < padded; q += NG_SORT_THREADS)
            sorted[q] = make_float4(inf, inf, inf, __int_as_float(0x7FFFFFFF));
    }
    // Every place is taken: `bins` now holds the end of every bin, and the records have been stored.  The barrier
    // orders memory at workgroup scope, which is all the read-back below needs: the wavefronts of a workgroup share
    // one L1, which holds no older copy of these lines (a wider fence would write the whole L2 back: 20 us).
    __syncthreads();
    if (boxes)
    {
        // The records in order, as the other wavefronts stored them: boxes of the runs of 16 (DPP row reductions).
        constexpr int BATCH = 16; // (all records of a thread are requested before the first is used: one trip to the L2)
        for (int q0 = tid; q0 < padded; q0 += NG_SORT_THREADS * BATCH)
        {
            float4 rec[BATCH];
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
                rec[u] = sorted[min(q0 + u * NG_SORT_THREADS, padded - 1)];
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
            {
                const int q = q0 + u * NG_SORT_THREADS;
                if (q >= padded) // uniform over the wavefront: cells are whole
                    continue;
                const bool real = __float_as_int(rec[u].w) != 0x7FFFFFFF;
                const float inf = __builtin_inff();
                const float v[3] = {rec[u].x, rec[u].y, rec[u].z};
                (void)inf;
                int lo[3], hi[3];
#pragma unroll
                for (int a = 0; a < 3; ++a)
                {
                    const int ordered = float_to_ordered_int(v[a]);
                    lo[a] = row_all_min_i32(real ? ordered : 0x7FFFFFFF);
                    hi[a] = row_all_max_i32(real ? ordered : INT_MIN);
                }
                if ((lane & 15) == 0)
                {
                    int* const run_box = run_boxes + (q / 16) * 6;
#pragma unroll
                    for (int a = 0; a < 3; ++a)
                    {
                        run_box[a] = lo[a];
                        run_box[3 + a] = hi[a];
                    }
                }
            }
        }
    }
    if (boxes)
    {
        // one thread per cell: the boxes of its four runs, and their union, to memory
        float diagonal2 = -1.f;
        __syncthreads();
        for (int c = tid; c < cells; c += NG_SORT_THREADS)
        {
            // (an empty run keeps (INT_MAX, INT_MIN), which map to NaN patterns: written as (+inf, -inf))
            auto as_lo = [](int o) { return o == 0x7FFFFFFF ? __builtin_inff() : ordered_int_to_float(o); };
            auto as_hi = [](int o) { return o == INT_MIN ? -__builtin_inff() : ordered_int_to_float(o); };
            int lo[3] = {0x7FFFFFFF, 0x7FFFFFFF, 0x7FFFFFFF}, hi[3] = {INT_MIN, INT_MIN, INT_MIN};
#pragma unroll
            for (int r = 0; r < 4; ++r)
            {
                const int* const run_box = run_boxes + (c * 4 + r) * 6;
                boxes[c * NG_BOX + 2 + r * 2 + 0] = make_float4(as_lo(run_box[0]), as_lo(run_box[1]), as_lo(run_box[2]), 0.f);
                boxes[c * NG_BOX + 2 + r * 2 + 1] = make_float4(as_hi(run_box[3]), as_hi(run_box[4]), as_hi(run_box[5]), 0.f);
#pragma unroll
                for (int a = 0; a < 3; ++a)
                {
                    lo[a] = min(lo[a], run_box[a]);
                    hi[a] = max(hi[a], run_box[3 + a]);
                }
            }
            boxes[c * NG_BOX + 0] = make_float4(as_lo(lo[0]), as_lo(lo[1]), as_lo(lo[2]), 0.f);
            boxes[c * NG_BOX + 1] = make_float4(as_hi(hi[0]), as_hi(hi[1]), as_hi(hi[2]), 0.f);
            if (c == tid && lo[0] != 0x7FFFFFFF) // (a cell that holds points: the squared diagonal of its box)
            {
                const float dx = as_hi(hi[0]) - as_lo(lo[0]), dy = as_hi(hi[1]) - as_lo(lo[1]), dz = as_hi(hi[2]) - as_lo(lo[2]);
                diagonal2 = __builtin_fmaf(dx, dx, __builtin_fmaf(dy, dy, dz * dz));
            }
        }
        if (set.wide_first) // (cells <= 256: one cell per thread of the first four wavefronts)
        {
            // the average over the cells that hold points, then the wide cells first, both groups in curve order
            const bool holds = diagonal2 >= 0.f;
            const float wave_sum = wave_sum_f32(holds ? diagonal2 : 0.f);
            const int wave_count = __builtin_popcountll(__ballot(holds));
            if (lane == 0)
            {
                wide_sums[wave] = wave_sum;
                wave_totals[wave] = wave_count;
            }
            __syncthreads();
            float sum = 0.f;
            int count = 0;
            for (int w = 0; w < NG_SORT_THREADS / TPK_WAVE; ++w)
            {
                sum += wide_sums[w];
                count += wave_totals[w];
            }
            const bool wide = holds && diagonal2 * count > CURVE_WIDE_FACTOR * sum;
            const unsigned long long wide_lanes = __ballot(wide);
            __syncthreads();
            if (lane == 0)
                wave_totals[wave] = __builtin_popcountll(wide_lanes);
            __syncthreads();
            int before = static_cast<int>(tpk_prefix_count(wide_lanes)), all_wide = 0;
            for (int w = 0; w < NG_SORT_THREADS / TPK_WAVE; ++w)
            {
                before += w < wave ? wave_totals[w] : 0;
                all_wide += wave_totals[w];
            }
            if (tid < cells)
                set.wide_first[window * cells + (wide ? before : all_wide + tid - before)] = tid;
        }
    }
    if (set.bin_ends)
    {
        // bins[i] is the end of bin i on the curve; the bin of a point is the leading 12 bits of
        // its position: the cell of the 16^3 grid it lies in (curve_bin_of_cell()).
        for (int i = tid; i < CURVE_BINS; i += NG_SORT_THREADS)
            set.bin_ends[window * CURVE_BINS + i] = bins[i];
        if (tid == 0)
        {
            const CurveGrid grid = curve_grid(cloud_box);
            set.grid[window * 2 + 0] = make_float4(grid.lo[0], grid.lo[1], grid.lo[2], 0.f);
            set.grid[window * 2 + 1] = make_float4(grid.scale[0], grid.scale[1], grid.scale[2], 0.f);
        }
    }
}

// Squared distance between two boxes / a point and a box (0 when they touch or overlap).
__device__ __forceinline__ float box_box_dist2(float4 alo, float4 ahi, float4 blo, float4 bhi)
{
    const float dx = fmaxf(fmaxf(blo.x - ahi.x, alo.x - bhi.x), 0.f);
    const float dy = fmaxf(fmaxf(blo.y - ahi.y, alo.y - bhi.y), 0.f);
    const float dz = fmaxf(fmaxf(blo.z - ahi.z, alo.z - bhi.z), 0.f);
    return __builtin_fmaf(dx, dx, __builtin_fmaf(dy, dy, dz * dz));
}
__device__ __forceinline__ float point_box_dist2(float x, float y, float z, float4 blo, float4 bhi)
{
    const float dx = fmaxf(fmaxf(blo.x - x, x - bhi.x), 0.f);
    const float dy = fmaxf(fmaxf(blo.y - y, y - bhi.y), 0.f);
    const float dz = fmaxf(fmaxf(blo.z - z, z - bhi.z), 0.f);
    return __builtin_fmaf(dx, dx, __builtin_fmaf(dy, dy, dz * dz));
}

int launch_curve_cells(const PointSet& a, const PointSet& c, int* zero_word, hipStream_t s,
                       const CloudRows& rows_job = CloudRows{nullptr, nullptr, 0, 0, nullptr})
{
    const int largest = a.stride > c.stride ? a.stride : c.stride;
    if (largest > CURVE_MAX_POINTS)
        return TPK_ERR_UNSUPPORTED; // (a thread holds 16 points of a window: windows of at most 16384 points)
    const int64_t windows_a = set_windows(a), windows_c = set_windows(c);
    const int64_t row_groups = tpk_ceil_div(rows_job.size_y, NG_SORT_THREADS);
    if (windows_a + windows_c + row_groups > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const size_t most_cells = static_cast<size_t>((largest + NG_CELL - 1) / NG_CELL);
    const size_t lds = (2 * static_cast<size_t>(CURVE_BINS) + 24 * most_cells) * sizeof(unsigned);
    const int allowed = tpk_allow_lds(reinterpret_cast<const void*>(curve_cells_kernel), lds);
    if (allowed != TPK_OK)
        return allowed;
    hipLaunchKernelGGL(curve_cells_kernel, dim3(static_cast<unsigned>(windows_a + windows_c + row_groups)),
                       dim3(NG_SORT_THREADS), lds, s, a, c, static_cast<int>(windows_a),
                       static_cast<int>(windows_a + windows_c), zero_word, rows_job);
    return tpk_launch_status();
}

} // namespace
