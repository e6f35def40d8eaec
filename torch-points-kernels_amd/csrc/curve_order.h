// Ordering of a point cloud along a Hilbert curve by one workgroup, in LDS, and the
// wavefront reductions it uses.  Shared by the kernels that cut a cloud into spatially compact
// cells so that whole cells can be skipped exactly (furthest point sampling, nearest-neighbour
// searches).
#pragma once

#include "tpk_device.h"

namespace {

// Row and wavefront minima, built like row_all_max_i32 / wave_max_i32.
__device__ __forceinline__ unsigned row_all_min_u32(unsigned v)
{
    v = min(v, static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true)));
    v = min(v, static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true)));
    v = min(v, static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, v, 0x124, 0xF, 0xF, true)));
    v = min(v, static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, v, 0x128, 0xF, 0xF, true)));
    return v;
}

// Minimum over each row of 16 lanes, in every lane of the row (built like row_all_max_i32).
__device__ __forceinline__ int row_all_min_i32(int v)
{
    v = min(v, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true));
    v = min(v, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true));
    v = min(v, __builtin_amdgcn_update_dpp(0, v, 0x124, 0xF, 0xF, true));
    v = min(v, __builtin_amdgcn_update_dpp(0, v, 0x128, 0xF, 0xF, true));
    return v;
}

__device__ __forceinline__ int wave_min_i32(int v)
{
    return ~wave_max_i32(~v);
}

__device__ __forceinline__ unsigned wave_min_u32(unsigned v)
{
    v = row_all_min_u32(v);
    const unsigned a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
    const unsigned c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
    return min(min(a, b), min(c, d));
}

__device__ __forceinline__ unsigned spread_bits_6(unsigned v) // abcdef -> a00b00c00d00e00f
{
    v &= 0x3Fu;
    v = (v | (v << 8)) & 0x300Fu;
    v = (v | (v << 4)) & 0x30C3u;
    v = (v | (v << 2)) & 0x9249u;
    return v;
}

// Position of grid cell (x0, x1, x2), BITS (<= 6) bits per axis, on the 3-D Hilbert curve through
// the grid (3 * BITS bits; Skilling's transposition: undo the excess rotations level by level, Gray-encode,
// interleave).  Consecutive positions are always adjacent cells, so a run of consecutive points
// is a compact blob - a Z-order run can straddle a jump across the whole cloud.
template <int BITS>
__device__ __forceinline__ unsigned hilbert_code(unsigned x0, unsigned x1, unsigned x2)
{
    unsigned x[3] = {x0, x1, x2};
#pragma unroll
    for (unsigned q = 1u << (BITS - 1); q > 1u; q >>= 1)
    {
        const unsigned p = q - 1u;
#pragma unroll
        for (int i = 0; i < 3; ++i)
        {
            const bool high = (x[i] & q) != 0;
            const unsigned t = (x[0] ^ x[i]) & p;
            const unsigned first = high ? x[0] ^ p : x[0] ^ t;
            if (i)
                x[i] = high ? x[i] : x[i] ^ t;
            x[0] = first;
        }
    }
    x[1] ^= x[0];
    x[2] ^= x[1];
    unsigned t = 0;
#pragma unroll
    for (unsigned q = 1u << (BITS - 1); q > 1u; q >>= 1)
        t ^= (x[2] & q) ? q - 1u : 0u;
    return (spread_bits_6(x[0] ^ t) << 2) | (spread_bits_6(x[1] ^ t) << 1) | spread_bits_6(x[2] ^ t);
}
// Bin of the counting sort that holds the points of cell (bx, by, bz) of the 16^3 grid: the
// position of that cell on the 4-bit curve (which is also the leading 12 bits of the position of
// any finer cell inside it: a Hilbert position starts with that of the enclosing coarser cell).
__device__ __forceinline__ unsigned curve_bin_of_cell(unsigned bx, unsigned by, unsigned bz)
{
    return hilbert_code<4>(bx, by, bz);
}

// The same position computed at compile time, and the table of all 4096 cells of the 16^3 grid (the ordering
// kernel copies it to LDS instead of computing 4096 positions per window).
constexpr unsigned spread_bits_6_const(unsigned v)
{
    v &= 0x3Fu;
    v = (v | (v << 8)) & 0x300Fu;
    v = (v | (v << 4)) & 0x30C3u;
    v = (v | (v << 2)) & 0x9249u;
    return v;
}
constexpr unsigned hilbert_code_const(int bits, unsigned x0, unsigned x1, unsigned x2)
{
    unsigned x[3] = {x0, x1, x2};
    for (unsigned q = 1u << (bits - 1); q > 1u; q >>= 1)
    {
        const unsigned p = q - 1u;
        for (int i = 0; i < 3; ++i)
        {
            const bool high = (x[i] & q) != 0;
            const unsigned t = (x[0] ^ x[i]) & p;
            const unsigned first = high ? x[0] ^ p : x[0] ^ t;
            if (i)
                x[i] = high ? x[i] : x[i] ^ t;
            x[0] = first;
        }
    }
    x[1] ^= x[0];
    x[2] ^= x[1];
    unsigned t = 0;
    for (unsigned q = 1u << (bits - 1); q > 1u; q >>= 1)
        t ^= (x[2] & q) ? q - 1u : 0u;
    return (spread_bits_6_const(x[0] ^ t) << 2) | (spread_bits_6_const(x[1] ^ t) << 1) | spread_bits_6_const(x[2] ^ t);
}
struct CurveBinTable
{
    unsigned short bin[4096]; // [bx | by << 4 | bz << 8]
};
constexpr CurveBinTable make_curve_bin_table()
{
    CurveBinTable t{};
    for (unsigned i = 0; i < 4096; ++i)
        t.bin[i] = static_cast<unsigned short>(hilbert_code_const(4, i & 15u, (i >> 4) & 15u, i >> 8));
    return t;
}
__device__ const CurveBinTable curve_bin_table = make_curve_bin_table();

// Order-preserving map of a float to a signed integer (for integer atomic min / max).
__device__ __forceinline__ int float_to_ordered_int(float f)
{
    const int b = __float_as_int(f);
    return b >= 0 ? b : b ^ 0x7FFFFFFF;
}
__device__ __forceinline__ float ordered_int_to_float(int b)
{
    return __int_as_float(b >= 0 ? b : b ^ 0x7FFFFFFF);
}

// The 64^3 grid over a cloud's bounding box in which curve positions are computed.
struct CurveGrid
{
    float lo[3], scale[3];
};

// From the box as the ordering left it in LDS (ordered ints: min x, y, z, then max x, y, z).
__device__ __forceinline__ CurveGrid curve_grid(const int* cloud_box)
{
    CurveGrid g;
#pragma unroll
    for (int a = 0; a < 3; ++a)
    {
        g.lo[a] = ordered_int_to_float(cloud_box[a]);
        const float ext = ordered_int_to_float(cloud_box[3 + a]) - g.lo[a];
        g.scale[a] = ext > 0.f ? 63.999f / ext : 0.f;
    }
    return g;
}

// Grid cell (0..63) of coordinate v along one axis; monotone in v; NaN goes to cell 0.
__device__ __forceinline__ unsigned curve_grid_cell(float v, float lo, float scale)
{
    float q = (v - lo) * scale;
    q = q >= 0.f ? q : 0.f;
    return q < 63.f ? static_cast<unsigned>(q) : 63u;
}

constexpr int CURVE_BINS = 4096;        // bins of the counting sort: the cells of a 16^3 grid, in curve order
constexpr int CURVE_MAX_POINTS = 16384; // the index of a point takes the low 14 bits of its sort key
constexpr int CURVE_LOAD_BATCH = 16;    // global loads in flight per thread

// Orders the n points (1 <= n <= CURVE_MAX_POINTS) of the cloud at `xyz` along the curve.  On
// return sort_keys[0..n) holds (bin << 20) | index, ascending in the bin - the position on the curve
// of the point's cell in a 16^3 grid over the cloud's box - and visible to the whole workgroup.
// All arrays are LDS: sort_keys max(n, CURVE_BINS) words, unsorted n words, bins CURVE_BINS words,
// cloud_box 6 words, wave_totals one word per wavefront.  Called by every thread of a workgroup
// of THREADS lanes (contains barriers).
// With `group` != nullptr (one sorted id per point: several clouds packed in one array) the points
// of the first 7 distinct-id offsets (group[k] - group[0] = 0..6) come first, one id after the
// other, each in curve order; the rest follow together.  Only the order changes, never its use.
template <int THREADS>
__device__ __forceinline__ void curve_order(const float* __restrict__ xyz, int n, unsigned* sort_keys,
                                            unsigned* unsorted, int* bins, int* cloud_box,
                                            int* wave_totals, const int64_t* __restrict__ group = nullptr)
{
    static_assert(CURVE_BINS % THREADS == 0, "every thread scans the same number of bins");
    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / TPK_WAVE);

    // box of the cloud (only to quantise coordinates for the curve)
    const int empty_lo = float_to_ordered_int(__builtin_inff());
    const int empty_hi = float_to_ordered_int(-__builtin_inff());
    if (tid < 6)
        cloud_box[tid] = tid < 3 ? empty_lo : empty_hi;
    for (int i = tid; i < CURVE_BINS; i += THREADS)
    {
        bins[i] = 0;
        // curve position of every cell of the 16^3 grid, computed once per cell instead of once
        // per point; the table borrows sort_keys, which the scatter fills only later
        sort_keys[i] = curve_bin_of_cell(i & 15, (i >> 4) & 15, i >> 8);
    }
    __syncthreads();
    {
        float lo[3] = {__builtin_inff(), __builtin_inff(), __builtin_inff()};
        float hi[3] = {-__builtin_inff(), -__builtin_inff(), -__builtin_inff()};
        // (loads in batches of CURVE_LOAD_BATCH points: the first touch of the cloud pays the full
        // memory latency, which must not be paid once per point)
        for (int k0 = tid; k0 < n; k0 += THREADS * CURVE_LOAD_BATCH)
        {
            float v[CURVE_LOAD_BATCH][3];
#pragma unroll
            for (int u = 0; u < CURVE_LOAD_BATCH; ++u)
            {
                const int k = min(k0 + u * THREADS, n - 1);
#pragma unroll
                for (int a = 0; a < 3; ++a)
                    v[u][a] = xyz[k * 3 + a];
            }
#pragma unroll
            for (int u = 0; u < CURVE_LOAD_BATCH; ++u)
#pragma unroll
                for (int a = 0; a < 3; ++a)
                {
                    lo[a] = fminf(lo[a], v[u][a]);
                    hi[a] = fmaxf(hi[a], v[u][a]);
                }
        }
#pragma unroll
        for (int a = 0; a < 3; ++a)
        {
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

    // sort keys = position on the curve, then the index.  Counting sort
    // on the leading 12 bits of the code: histogram, prefix sum, scatter through LDS atomics.
    // Inside a bin (1/16 of the cloud's extent per axis) the order is that in which the atomics
    // were served; it decides which lane holds which point, never which point is sampled.
    {
        const CurveGrid grid = curve_grid(cloud_box);
        for (int k0 = tid; k0 < n; k0 += THREADS * CURVE_LOAD_BATCH)
        {
            float v[CURVE_LOAD_BATCH][3];
#pragma unroll
            for (int u = 0; u < CURVE_LOAD_BATCH; ++u)
            {
                const int k = min(k0 + u * THREADS, n - 1);
#pragma unroll
                for (int a = 0; a < 3; ++a)
                    v[u][a] = xyz[k * 3 + a];
            }
#pragma unroll
            for (int u = 0; u < CURVE_LOAD_BATCH; ++u)
            {
                const int k = k0 + u * THREADS;
                unsigned cell[3];
#pragma unroll
                for (int a = 0; a < 3; ++a)
                    cell[a] = curve_grid_cell(v[u][a], grid.lo[a], grid.scale[a]);
                // the bin: position on the curve of the cell of the 16^3 grid
                unsigned bin = sort_keys[(cell[0] >> 2) | ((cell[1] >> 2) << 4) | ((cell[2] >> 2) << 8)];
                if (group && k < n)
                {
                    const int64_t offset = group[k] - group[0];
                    bin = (static_cast<unsigned>(offset < 7 ? offset : 7) << 9) | (bin >> 3);
                }
                const unsigned key = (bin << 20) | static_cast<unsigned>(k);
                if (k < n)
                {
                    unsorted[k] = key;
                    atomicAdd(&bins[key >> 20], 1);
                }
            }
        }
    }
    __syncthreads();
    {
        int count[CURVE_BINS / THREADS];
        int sum = 0;
#pragma unroll
        for (int i = 0; i < CURVE_BINS / THREADS; ++i)
        {
            count[i] = bins[tid * CURVE_BINS / THREADS + i];
            sum += count[i];
        }
        int scan = sum; // inclusive prefix sum over the wavefront
#pragma unroll
        for (int d = 1; d < TPK_WAVE; d <<= 1)
        {
            const int below = __shfl_up(scan, d);
            scan += lane >= d ? below : 0;
        }
        if (lane == TPK_WAVE - 1)
            wave_totals[wave] = scan;
        __syncthreads();
        int run = scan - sum;
        for (int w = 0; w < wave; ++w)
            run += wave_totals[w];
#pragma unroll
        for (int i = 0; i < CURVE_BINS / THREADS; ++i)
        {
            bins[tid * CURVE_BINS / THREADS + i] = run; // start of the bin
            run += count[i];
        }
    }
    __syncthreads();
    for (int k = tid; k < n; k += THREADS)
    {
        const unsigned key = unsorted[k];
        sort_keys[atomicAdd(&bins[key >> 20], 1)] = key;
    }
    __syncthreads();
}

} // namespace
