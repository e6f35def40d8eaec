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

// One workgroup orders one window: the first windows_a blocks those of set_a, the rest set_b.
// `zero_word` (optional) is cleared by the first block: a counter used by the kernel that follows.
__global__ __launch_bounds__(NG_SORT_THREADS) void curve_cells_kernel(PointSet set_a, PointSet set_b,
                                                                      int windows_a, int key_capacity,
                                                                      int* zero_word)
{
    extern __shared__ unsigned sort_keys[];
    unsigned* const unsorted = sort_keys + key_capacity;
    int* const bins = reinterpret_cast<int*>(unsorted + key_capacity);
    __shared__ int cloud_box[6];
    __shared__ int wave_totals[NG_SORT_THREADS / TPK_WAVE];

    const bool first_set = static_cast<int>(blockIdx.x) < windows_a;
    const PointSet set = first_set ? set_a : set_b;
    const int64_t window = first_set ? blockIdx.x : blockIdx.x - windows_a;
    const int per_cloud = set_windows_per_cloud(set);
    const int64_t in_cloud = (window % per_cloud) * static_cast<int64_t>(set.stride);
    const int64_t start = (window / per_cloud) * set.cloud_points + in_cloud;
    const int n = static_cast<int>(tpk_min64(set.stride, set.cloud_points - in_cloud));
    const int cells = set_cells(set);
    const float* __restrict__ xyz = set.xyz + start * 3;
    float4* __restrict__ sorted = set.sorted + window * cells * NG_CELL;
    float4* __restrict__ boxes = set.boxes ? set.boxes + window * cells * NG_BOX : nullptr;
    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    if (zero_word && blockIdx.x == 0 && tid == 0)
        *zero_word = 0;

    curve_order<NG_SORT_THREADS>(xyz, n, sort_keys, unsorted, bins, cloud_box, wave_totals,
                                 set.group ? set.group + start : nullptr);

    // Every wavefront writes whole cells; a batch of gathers is issued before any is used.
    int* const run_boxes = reinterpret_cast<int*>(unsorted); // (free now) [cells * 4][6] ordered ints
    constexpr int BATCH = 4;
    const int padded = cells * NG_CELL;
    for (int q0 = tid; q0 < padded; q0 += NG_SORT_THREADS * BATCH)
    {
        int k[BATCH];
        float v[BATCH][3];
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
        {
            const int q = q0 + u * NG_SORT_THREADS;
            k[u] = q < n ? static_cast<int>(sort_keys[q] & 0x3FFFu) : -1;
            const int kk = k[u] < 0 ? 0 : k[u];
#pragma unroll
            for (int a = 0; a < 3; ++a)
                v[u][a] = xyz[kk * 3 + a];
        }
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
        {
            const int q = q0 + u * NG_SORT_THREADS;
            if (q >= padded) // uniform over the wavefront: cells are whole
                continue;
            const bool real = k[u] >= 0;
            const float inf = __builtin_inff();
            sorted[q] = real ? make_float4(v[u][0], v[u][1], v[u][2], __int_as_float(static_cast<int>(in_cloud) + k[u]))
                             : make_float4(inf, inf, inf, __int_as_float(0x7FFFFFFF));
            if (!boxes) // uniform
                continue;
            // boxes of the four runs of 16 points (DPP row reductions), left in LDS
            int lo[3], hi[3];
#pragma unroll
            for (int a = 0; a < 3; ++a)
            {
                lo[a] = ~row_all_max_i32(~float_to_ordered_int(real ? v[u][a] : inf));
                hi[a] = row_all_max_i32(float_to_ordered_int(real ? v[u][a] : -inf));
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
    if (boxes)
    {
        // one thread per cell: the boxes of its four runs, and their union, to memory
        __syncthreads();
        for (int c = tid; c < cells; c += NG_SORT_THREADS)
        {
            int lo[3] = {0x7FFFFFFF, 0x7FFFFFFF, 0x7FFFFFFF}, hi[3] = {INT_MIN, INT_MIN, INT_MIN};
#pragma unroll
            for (int r = 0; r < 4; ++r)
            {
                const int* const run_box = run_boxes + (c * 4 + r) * 6;
                boxes[c * NG_BOX + 2 + r * 2 + 0] =
                    make_float4(ordered_int_to_float(run_box[0]), ordered_int_to_float(run_box[1]),
                                ordered_int_to_float(run_box[2]), 0.f);
                boxes[c * NG_BOX + 2 + r * 2 + 1] =
                    make_float4(ordered_int_to_float(run_box[3]), ordered_int_to_float(run_box[4]),
                                ordered_int_to_float(run_box[5]), 0.f);
#pragma unroll
                for (int a = 0; a < 3; ++a)
                {
                    lo[a] = min(lo[a], run_box[a]);
                    hi[a] = max(hi[a], run_box[3 + a]);
                }
            }
            boxes[c * NG_BOX + 0] = make_float4(ordered_int_to_float(lo[0]), ordered_int_to_float(lo[1]),
                                                ordered_int_to_float(lo[2]), 0.f);
            boxes[c * NG_BOX + 1] = make_float4(ordered_int_to_float(hi[0]), ordered_int_to_float(hi[1]),
                                                ordered_int_to_float(hi[2]), 0.f);
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

int launch_curve_cells(const PointSet& a, const PointSet& c, int* zero_word, hipStream_t s)
{
    const int largest = a.stride > c.stride ? a.stride : c.stride;
    const int key_capacity = largest > CURVE_BINS ? (largest + 63) & ~63 : CURVE_BINS; // (the ordering borrows CURVE_BINS words)
    const int64_t windows_a = set_windows(a), windows_c = set_windows(c);
    if (windows_a + windows_c > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const size_t lds = (2 * static_cast<size_t>(key_capacity) + CURVE_BINS) * sizeof(unsigned);
    const int allowed = tpk_allow_lds(reinterpret_cast<const void*>(curve_cells_kernel), lds);
    if (allowed != TPK_OK)
        return allowed;
    hipLaunchKernelGGL(curve_cells_kernel, dim3(static_cast<unsigned>(windows_a + windows_c)),
                       dim3(NG_SORT_THREADS), lds, s, a, c, static_cast<int>(windows_a), key_capacity,
                       zero_word);
    return tpk_launch_status();
}

} // namespace
