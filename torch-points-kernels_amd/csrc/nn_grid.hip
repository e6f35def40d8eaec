// Nearest-neighbour search over clouds cut into spatially compact cells.
//
// The all-pairs scans (chamfer.hip, three_nn.hip) test every query against every candidate.
// Here both clouds are first ordered along a Hilbert curve (curve_order.h) and cut into cells
// of 64 consecutive points, each with its bounding box.  A wavefront then serves the 64
// queries of one cell: it measures the distance from its cell's box to every candidate cell's
// box (one lane per candidate cell), scans the nearest candidate cell to get a first answer,
// and afterwards scans only candidate cells whose box is not further away than the worst
// current answer of its lanes.  A skipped cell cannot hold a nearer point, nor one at equal
// distance: the box distance is compared with a relative margin of 2e-6, several times the fp32
// rounding error of either side.  Distances of the pairs that are evaluated use the same
// operations in the same order as the all-pairs kernels, so values are bit-identical.
//
// The candidates are visited in curve order, not index order, so "the lowest index among equal
// distances" - what a serial first-strictly-smaller scan returns - is enforced explicitly: the
// scan keeps the minimum and the first group of 8 candidates that reached it, and flags a lane
// when another group reaches the same value; flagged lanes (duplicated points, lattices) take
// an extra pass that collects the lowest index among all candidates at that distance.
//
// Workspace per cloud: 16 bytes per point (x, y, z, original index) padded to whole cells, and
// 32 bytes per cell (box).  Clouds of up to 16384 points (the curve ordering works in LDS).
#include "curve_order.h"
#include "nn_grid.h"

namespace {

constexpr int NG_CELL = 64;                  // points per cell = lanes of a wavefront
constexpr int NG_MAX_CELLS = 256;            // candidate cells per cloud (their box distances sit in LDS)
constexpr int NG_SORT_THREADS = 1024;
constexpr int NG_SCAN_THREADS = 256;         // 4 wavefronts, each searching on its own
constexpr float NG_MARGIN = 0.999998f;
constexpr int NG_CHUNK = 8;

// A set of points to be ordered: `total` points cut into windows of `stride` consecutive points
// (a batch of equal clouds: stride = points per cloud; a packed array: windows of at most
// CURVE_MAX_POINTS points, whatever clouds they hold).  Every window gets stride / 64 (rounded
// up) cells of 64 records, in curve order; a record is (x, y, z, index inside the window), the
// padding records are infinitely far away with index 0x7FFFFFFF; a cell without points has an
// empty box (lo = +inf, hi = -inf).
struct PointSet
{
    const float* xyz;     // [total][3]
    const int64_t* group; // optional sorted cloud id per point (packed arrays), or nullptr
    int64_t total;
    int stride;
    float4* sorted;       // [windows][cells * 64]
    float4* boxes;        // [windows][cells][2]: (lo.xyz, -), (hi.xyz, -)
};

__host__ __device__ inline int set_cells(const PointSet& s)
{
    return (s.stride + NG_CELL - 1) / NG_CELL;
}
__host__ __device__ inline int64_t set_windows(const PointSet& s)
{
    return (s.total + s.stride - 1) / s.stride;
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
    const int64_t start = window * set.stride;
    const int n = static_cast<int>(tpk_min64(set.stride, set.total - start));
    const int cells = set_cells(set);
    const float* __restrict__ xyz = set.xyz + start * 3;
    float4* __restrict__ sorted = set.sorted + window * cells * NG_CELL;
    float4* __restrict__ boxes = set.boxes + window * cells * 2;
    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    if (zero_word && blockIdx.x == 0 && tid == 0)
        *zero_word = 0;

    curve_order<NG_SORT_THREADS>(xyz, n, sort_keys, unsorted, bins, cloud_box, wave_totals,
                                 set.group ? set.group + start : nullptr);

    // Every wavefront writes whole cells; a batch of gathers is issued before any is used.
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
            sorted[q] = real ? make_float4(v[u][0], v[u][1], v[u][2], __int_as_float(k[u]))
                             : make_float4(inf, inf, inf, __int_as_float(0x7FFFFFFF));
            float lo[3], hi[3];
#pragma unroll
            for (int a = 0; a < 3; ++a)
            {
                lo[a] = ordered_int_to_float(wave_min_i32(float_to_ordered_int(real ? v[u][a] : inf)));
                hi[a] = ordered_int_to_float(wave_max_i32(float_to_ordered_int(real ? v[u][a] : -inf)));
            }
            if (lane == 0)
            {
                boxes[(q / NG_CELL) * 2 + 0] = make_float4(lo[0], lo[1], lo[2], 0.f);
                boxes[(q / NG_CELL) * 2 + 1] = make_float4(hi[0], hi[1], hi[2], 0.f);
            }
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

// State of one lane's nearest-neighbour search.
struct Nearest
{
    float best; // smallest distance so far
    int chunk;  // first group of NG_CHUNK candidates (position / NG_CHUNK on the curve) that reached it
    bool tie;   // another group reached the same value
};

// Scans candidate cell `cell` for the 64 queries of the wavefront.  `stage` is the wavefront's
// own 64-entry LDS buffer, through which every lane sees every candidate (broadcast reads).
__device__ __forceinline__ void scan_cell(const float4* __restrict__ cand, int cell, float4* stage,
                                          int lane, float qx, float qy, float qz, Nearest& s)
{
    stage[lane] = cand[cell * NG_CELL + lane];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); // LDS serves a wavefront's requests in order
#pragma unroll 2
    for (int ch = 0; ch < NG_CELL / NG_CHUNK; ++ch)
    {
        float mn = 0.f;
#pragma unroll
        for (int c = 0; c < NG_CHUNK; ++c)
        {
            const float4 p = stage[ch * NG_CHUNK + c];
            // Operand order of the reference: (scanned - query), squares summed x, y, z.
            const float d = tpk_dist2(p.x, p.y, p.z, qx, qy, qz);
            mn = c == 0 ? d : fminf(mn, d);
        }
        const bool better = mn < s.best;
        const bool equal = mn == s.best;
        s.tie = better ? false : (s.tie || equal);
        s.chunk = better ? cell * (NG_CELL / NG_CHUNK) + ch : s.chunk;
        s.best = better ? mn : s.best;
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// One wavefront = the 64 queries of one cell.  Logical wavefront number (after the die-local
// block mapping) = cloud * (cells1 + cells2) + cell; the cells of cloud 1 query cloud 2 and
// write dist1 / idx1, those of cloud 2 the other way round.
__global__ __launch_bounds__(NG_SCAN_THREADS) void chamfer_grid_kernel(
    int n, int m, int clouds, const float4* __restrict__ sorted1,
    const float4* __restrict__ sorted2, const float4* __restrict__ boxes1,
    const float4* __restrict__ boxes2, float* __restrict__ dist1, float* __restrict__ dist2,
    int32_t* __restrict__ idx1, int32_t* __restrict__ idx2)
{
    __shared__ float4 stages[NG_SCAN_THREADS / TPK_WAVE][NG_CELL];
    __shared__ float lows_all[NG_SCAN_THREADS / TPK_WAVE][NG_MAX_CELLS];

    const int lane = threadIdx.x & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TPK_WAVE);
    const int cells1 = (n + NG_CELL - 1) / NG_CELL, cells2 = (m + NG_CELL - 1) / NG_CELL;
    const int per_cloud = cells1 + cells2;
    const int64_t task = static_cast<int64_t>(xcd_local_block(blockIdx.x, gridDim.x)) *
                             (NG_SCAN_THREADS / TPK_WAVE) + wave;
    if (task >= static_cast<int64_t>(per_cloud) * clouds)
        return; // (no workgroup barrier anywhere in this kernel)
    const int cloud = static_cast<int>(task / per_cloud);
    const int r = static_cast<int>(task - static_cast<int64_t>(cloud) * per_cloud);
    const bool second = r >= cells1;
    const int qcell = second ? r - cells1 : r;
    const int qcells = second ? cells2 : cells1;
    const int ccells = second ? cells1 : cells2;
    const int qcount = second ? m : n;
    const float4* __restrict__ qpts = (second ? sorted2 : sorted1) + static_cast<int64_t>(cloud) * qcells * NG_CELL;
    const float4* __restrict__ qbox = (second ? boxes2 : boxes1) + static_cast<int64_t>(cloud) * qcells * 2;
    const float4* __restrict__ cpts = (second ? sorted1 : sorted2) + static_cast<int64_t>(cloud) * ccells * NG_CELL;
    const float4* __restrict__ cbox = (second ? boxes1 : boxes2) + static_cast<int64_t>(cloud) * ccells * 2;
    float* __restrict__ dout = (second ? dist2 : dist1) + static_cast<int64_t>(cloud) * qcount;
    int32_t* __restrict__ iout = (second ? idx2 : idx1) + static_cast<int64_t>(cloud) * qcount;
    float4* const stage = stages[wave];
    float* const lows = lows_all[wave];

    const float4 query = qpts[qcell * NG_CELL + lane];
    const float qx = query.x, qy = query.y, qz = query.z;
    const int qindex = __float_as_int(query.w); // 0x7FFFFFFF: padding, nothing to store
    const float4 qlo = qbox[qcell * 2 + 0], qhi = qbox[qcell * 2 + 1];

    // Box distances to all candidate cells, kept in the wavefront's LDS row (lane l computes
    // cells l, 64 + l, ...); +inf marks a cell that does not exist or has been scanned.
    const int groups = (ccells + NG_CELL - 1) / NG_CELL;
    unsigned seed_key = 0xFFFFFFFFu;
    for (int g = 0; g < groups; ++g)
    {
        const int c = g * NG_CELL + lane;
        const bool valid = c < ccells;
        const int cc = valid ? c : 0;
        const float lb = box_box_dist2(qlo, qhi, cbox[cc * 2 + 0], cbox[cc * 2 + 1]);
        lows[c] = valid ? lb : __builtin_inff();
        // approximately the nearest cell (the two lowest bits of the distance carry g)
        const unsigned key = (static_cast<unsigned>(__float_as_int(lb)) & ~3u) | static_cast<unsigned>(g);
        seed_key = valid && key < seed_key ? key : seed_key;
    }
    Nearest s;
    s.best = __builtin_inff();
    s.chunk = 0;
    s.tie = false;
    {
        const unsigned lowest = wave_min_u32(seed_key);
        int seed = static_cast<int>(lowest & 3u) * NG_CELL + __builtin_ctzll(__ballot(seed_key == lowest));
        if (seed >= ccells) // no lane had a usable key (NaN boxes)
            seed = 0;
        scan_cell(cpts, seed, stage, lane, qx, qy, qz, s);
        if (lane == (seed & (NG_CELL - 1)))
            lows[seed] = __builtin_inff();
    }

    // First the cells whose boxes overlap the queries' box - they hold nearly all the answers -
    // then whatever the worst answer still admits.
    for (int phase = 0; phase < 2; ++phase)
        for (int g = 0; g < groups; ++g)
        {
            const float lw = lows[g * NG_CELL + lane];
            float bound = __int_as_float(wave_max_i32(__float_as_int(s.best)));
            unsigned long long live =
                __ballot(lw < __builtin_inff() && (phase == 0 ? lw == 0.f : lw * NG_MARGIN <= bound));
            while (live != 0)
            {
                const int bit = __builtin_ctzll(live);
                const int c = g * NG_CELL + bit;
                live &= live - 1;
                const float lb = point_box_dist2(qx, qy, qz, cbox[c * 2 + 0], cbox[c * 2 + 1]);
                if (__ballot(lb * NG_MARGIN <= s.best) == 0)
                {
                    // no lane can improve here now, and answers only get better: never again
                    if (lane == bit)
                        lows[c] = __builtin_inff();
                    continue;
                }
                scan_cell(cpts, c, stage, lane, qx, qy, qz, s);
                if (lane == bit)
                    lows[c] = __builtin_inff();
                if (phase)
                {
                    bound = __int_as_float(wave_max_i32(__float_as_int(s.best)));
                    live &= __ballot(lw * NG_MARGIN <= bound);
                }
            }
        }

    // The index: lowest original index among the candidates of the recorded group that are at
    // the minimum distance (re-evaluated with the same operations, hence the same bits).
    int bi = 0x7FFFFFFF;
#pragma unroll
    for (int c = 0; c < NG_CHUNK; ++c)
    {
        const float4 p = cpts[s.chunk * NG_CHUNK + c];
        const float d = tpk_dist2(p.x, p.y, p.z, qx, qy, qz);
        const int ci = __float_as_int(p.w);
        bi = (d == s.best && ci < bi) ? ci : bi;
    }
    if (__ballot(s.tie) != 0)
    {
        // Several groups reached the minimum (rare): lowest index over all cells that can hold it.
        for (int c = 0; c < ccells; ++c)
        {
            const float lb = point_box_dist2(qx, qy, qz, cbox[c * 2 + 0], cbox[c * 2 + 1]);
            if (__ballot(s.tie && lb * NG_MARGIN <= s.best) == 0)
                continue;
            stage[lane] = cpts[c * NG_CELL + lane];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            for (int k = 0; k < NG_CELL; ++k)
            {
                const float4 p = stage[k];
                const float d = tpk_dist2(p.x, p.y, p.z, qx, qy, qz);
                const int ci = __float_as_int(p.w);
                bi = (s.tie && d == s.best && ci < bi) ? ci : bi;
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    }
    if (qindex != 0x7FFFFFFF)
    {
        dout[qindex] = s.best;
        iout[qindex] = bi == 0x7FFFFFFF ? 0 : bi;
    }
}

// ---------------------------------------------------------------------------------------
// three_nn over cells: the three nearest known points of every unknown point.
//
// The running answer of a lane is a triple sorted by (distance, original index); a candidate
// enters where it is smaller in that order.  This is the order a serial scan in index order with
// strictly-smaller replacement (cuda/src/interpolate_gpu.cu:9-65) ends with, whatever order the
// candidates are visited in.  A cell is skipped when its box is further away than the third
// best of every lane.
// ---------------------------------------------------------------------------------------
struct Nearest3
{
    float b1, b2, b3;
    int i1, i2, i3;
};

__device__ __forceinline__ bool pair_less(float d, int ci, float b, int i)
{
    return d < b || (d == b && ci < i);
}

__device__ __forceinline__ void scan_cell3(const float4* __restrict__ cand, int cell, float4* stage,
                                           int lane, float qx, float qy, float qz, Nearest3& s)
{
    stage[lane] = cand[cell * NG_CELL + lane];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    for (int ch = 0; ch < NG_CELL / NG_CHUNK; ++ch)
    {
        float mn = 0.f;
#pragma unroll
        for (int c = 0; c < NG_CHUNK; ++c)
        {
            const float4 p = stage[ch * NG_CHUNK + c];
            const float d = tpk_dist2(qx, qy, qz, p.x, p.y, p.z);
            mn = c == 0 ? d : fminf(mn, d);
        }
        if (__ballot(mn <= s.b3) == 0)
            continue; // no candidate of this group enters any lane's triple
#pragma unroll
        for (int c = 0; c < NG_CHUNK; ++c)
        {
            const float4 p = stage[ch * NG_CHUNK + c];
            // Operand order of the reference: (query - scanned).
            const float d = tpk_dist2(qx, qy, qz, p.x, p.y, p.z);
            const int ci = __float_as_int(p.w);
            const bool l3 = pair_less(d, ci, s.b3, s.i3);
            if (__ballot(l3) == 0)
                continue;
            const bool l2 = pair_less(d, ci, s.b2, s.i2);
            const bool l1 = pair_less(d, ci, s.b1, s.i1);
            s.b3 = l2 ? s.b2 : (l3 ? d : s.b3);
            s.i3 = l2 ? s.i2 : (l3 ? ci : s.i3);
            s.b2 = l1 ? s.b1 : (l2 ? d : s.b2);
            s.i2 = l1 ? s.i1 : (l2 ? ci : s.i2);
            s.b1 = l1 ? d : s.b1;
            s.i1 = l1 ? ci : s.i1;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// One wavefront = the 64 unknown points of one cell; logical wavefront = cloud * qcells + cell.
__global__ __launch_bounds__(NG_SCAN_THREADS) void three_nn_grid_kernel(
    int n, int m, int clouds, const float4* __restrict__ sorted_unknown,
    const float4* __restrict__ sorted_known, const float4* __restrict__ boxes_unknown,
    const float4* __restrict__ boxes_known, float* __restrict__ dist2, int32_t* __restrict__ idx)
{
    __shared__ float4 stages[NG_SCAN_THREADS / TPK_WAVE][NG_CELL];
    __shared__ float lows_all[NG_SCAN_THREADS / TPK_WAVE][NG_MAX_CELLS];

    const int lane = threadIdx.x & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TPK_WAVE);
    const int qcells = (n + NG_CELL - 1) / NG_CELL, ccells = (m + NG_CELL - 1) / NG_CELL;
    const int64_t task = static_cast<int64_t>(xcd_local_block(blockIdx.x, gridDim.x)) *
                             (NG_SCAN_THREADS / TPK_WAVE) + wave;
    if (task >= static_cast<int64_t>(qcells) * clouds)
        return; // (no workgroup barrier anywhere in this kernel)
    const int cloud = static_cast<int>(task / qcells);
    const int qcell = static_cast<int>(task - static_cast<int64_t>(cloud) * qcells);
    const float4* __restrict__ qpts = sorted_unknown + static_cast<int64_t>(cloud) * qcells * NG_CELL;
    const float4* __restrict__ qbox = boxes_unknown + static_cast<int64_t>(cloud) * qcells * 2;
    const float4* __restrict__ cpts = sorted_known + static_cast<int64_t>(cloud) * ccells * NG_CELL;
    const float4* __restrict__ cbox = boxes_known + static_cast<int64_t>(cloud) * ccells * 2;
    dist2 += static_cast<int64_t>(cloud) * n * 3;
    idx += static_cast<int64_t>(cloud) * n * 3;
    float4* const stage = stages[wave];
    float* const lows = lows_all[wave];

    const float4 query = qpts[qcell * NG_CELL + lane];
    const float qx = query.x, qy = query.y, qz = query.z;
    const int qindex = __float_as_int(query.w); // 0x7FFFFFFF: padding, nothing to store
    const float4 qlo = qbox[qcell * 2 + 0], qhi = qbox[qcell * 2 + 1];

    const int groups = (ccells + NG_CELL - 1) / NG_CELL;
    unsigned seed_key = 0xFFFFFFFFu;
    for (int g = 0; g < groups; ++g)
    {
        const int c = g * NG_CELL + lane;
        const bool valid = c < ccells;
        const int cc = valid ? c : 0;
        const float lb = box_box_dist2(qlo, qhi, cbox[cc * 2 + 0], cbox[cc * 2 + 1]);
        lows[c] = valid ? lb : __builtin_inff();
        const unsigned key = (static_cast<unsigned>(__float_as_int(lb)) & ~3u) | static_cast<unsigned>(g);
        seed_key = valid && key < seed_key ? key : seed_key;
    }
    Nearest3 s;
    s.b1 = s.b2 = s.b3 = __builtin_inff();
    s.i1 = s.i2 = s.i3 = 0;
    {
        const unsigned lowest = wave_min_u32(seed_key);
        int seed = static_cast<int>(lowest & 3u) * NG_CELL + __builtin_ctzll(__ballot(seed_key == lowest));
        if (seed >= ccells)
            seed = 0;
        scan_cell3(cpts, seed, stage, lane, qx, qy, qz, s);
        if (lane == (seed & (NG_CELL - 1)))
            lows[seed] = __builtin_inff();
    }
    for (int phase = 0; phase < 2; ++phase)
        for (int g = 0; g < groups; ++g)
        {
            const float lw = lows[g * NG_CELL + lane];
            float bound = __int_as_float(wave_max_i32(__float_as_int(s.b3)));
            unsigned long long live =
                __ballot(lw < __builtin_inff() && (phase == 0 ? lw == 0.f : lw * NG_MARGIN <= bound));
            while (live != 0)
            {
                const int bit = __builtin_ctzll(live);
                const int c = g * NG_CELL + bit;
                live &= live - 1;
                const float lb = point_box_dist2(qx, qy, qz, cbox[c * 2 + 0], cbox[c * 2 + 1]);
                if (__ballot(lb * NG_MARGIN <= s.b3) != 0)
                    scan_cell3(cpts, c, stage, lane, qx, qy, qz, s);
                if (lane == bit)
                    lows[c] = __builtin_inff(); // scanned, or useless now and ever after
                if (phase)
                {
                    bound = __int_as_float(wave_max_i32(__float_as_int(s.b3)));
                    live &= __ballot(lw * NG_MARGIN <= bound);
                }
            }
        }
    if (qindex != 0x7FFFFFFF)
    {
        dist2[qindex * 3 + 0] = s.b1;
        dist2[qindex * 3 + 1] = s.b2;
        dist2[qindex * 3 + 2] = s.b3;
        idx[qindex * 3 + 0] = s.i1;
        idx[qindex * 3 + 1] = s.i2;
        idx[qindex * 3 + 2] = s.i3;
    }
}

// ---------------------------------------------------------------------------------------
// Ball query over cells, packed layout (several clouds back to back, sorted cloud id per point).
//
// Both packed arrays are cut into windows of CURVE_MAX_POINTS consecutive rows, each ordered on
// its own (curve_cells_kernel; inside a window the clouds come one after the other).  A
// wavefront serves the 64 queries of one cell: it looks up the support rows of its queries'
// clouds, walks the windows that hold them, and scans the cells whose box is within the radius
// of its own cell's box and of at least one of its queries.  A candidate is a hit when its
// squared distance is <= radius^2 and its row lies in the query's cloud.
// The result rows must hold the hits with the LOWEST rows, in ascending order (a serial scan in
// index order that stops after nsample hits, cuda/src/ball_query_gpu.cu:54-95).  A lane collects
// up to BQG_KEEP hits in LDS, sorts them, and the wavefront writes the rows (hits, then -1)
// with coalesced stores.  A query with more hits than that - or than nsample - is put on a
// list and answered by ball_query_overflow_kernel, one wavefront per query scanning its cloud
// in index order with early exit: dense neighbourhoods are exactly where that scan is short.
// ---------------------------------------------------------------------------------------
constexpr int BQG_KEEP = 16;          // hits a lane keeps in LDS
constexpr int BQG_PITCH = NG_CELL + 1; // LDS row pitch of the hit buffers (conflict-free both ways)
constexpr int BQG_LIST = 64;           // overflow list: word 0 = count, queries from word BQG_LIST on

// First position of sorted a[0..len) whose value is >= v, found by the whole wavefront:
// 64 samples per round instead of one.
__device__ __forceinline__ int wave_lower_bound(const int64_t* __restrict__ a, int len, int64_t v, int lane)
{
    int lo = 0, hi = len; // the answer lies in [lo, hi]
    while (hi > lo)
    {
        const int step = (hi - lo + TPK_WAVE - 1) / TPK_WAVE;
        const int pos = lo + lane * step;
        const bool in = pos < hi;
        const int64_t sample = a[in ? pos : lo];
        const unsigned long long ge = __ballot(!in || sample >= v);
        const int f = ge ? __builtin_ctzll(ge) : TPK_WAVE; // first lane whose sample is >= v
        const int next_lo = f > 0 ? lo + (f - 1) * step + 1 : lo;
        const int next_hi = f < TPK_WAVE ? min(lo + f * step, hi) : hi;
        lo = next_lo;
        hi = next_hi;
    }
    return lo;
}

__global__ __launch_bounds__(NG_SCAN_THREADS) void ball_query_grid_kernel(
    int size_x, int size_y, float radius2, int nsample, const float4* __restrict__ sorted_x,
    const float4* __restrict__ boxes_x, const float4* __restrict__ sorted_y,
    const float4* __restrict__ boxes_y, const int64_t* __restrict__ batch_x,
    const int64_t* __restrict__ batch_y, int64_t* __restrict__ idx, float* __restrict__ dist,
    int* __restrict__ overflow)
{
    constexpr int WAVES = NG_SCAN_THREADS / TPK_WAVE;
    constexpr int CELLS = CURVE_MAX_POINTS / NG_CELL; // cells per window
    __shared__ float4 stages[WAVES][NG_CELL];
    __shared__ int hit_rows[WAVES][BQG_KEEP * BQG_PITCH];
    __shared__ float hit_dists[WAVES][BQG_KEEP * BQG_PITCH];

    const int lane = threadIdx.x & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TPK_WAVE);
    const int windows_y = (size_y + CURVE_MAX_POINTS - 1) / CURVE_MAX_POINTS;
    const int64_t task = static_cast<int64_t>(xcd_local_block(blockIdx.x, gridDim.x)) * WAVES + wave;
    if (task >= static_cast<int64_t>(windows_y) * CELLS)
        return; // (no workgroup barrier anywhere in this kernel)
    const int wy = static_cast<int>(task / CELLS);
    const int qcell = static_cast<int>(task - static_cast<int64_t>(wy) * CELLS);
    float4* const stage = stages[wave];
    int* const my_rows = hit_rows[wave];
    float* const my_dists = hit_dists[wave];

    const float4 query = sorted_y[(static_cast<int64_t>(wy) * CELLS + qcell) * NG_CELL + lane];
    const float qx = query.x, qy = query.y, qz = query.z;
    const bool valid = __float_as_int(query.w) != 0x7FFFFFFF;
    if (__ballot(valid) == 0)
        return; // a cell past the end of its window
    const int qrow = wy * CURVE_MAX_POINTS + (valid ? __float_as_int(query.w) : 0);
    const float4 qlo = boxes_y[(static_cast<int64_t>(wy) * CELLS + qcell) * 2 + 0];
    const float4 qhi = boxes_y[(static_cast<int64_t>(wy) * CELLS + qcell) * 2 + 1];

    // Support rows [lo, hi) of every lane's cloud; usually all lanes share one cloud.
    const int64_t cloud = valid ? batch_y[qrow] : -1;
    int lo = 0, hi = 0;
    for (unsigned long long todo = __ballot(valid); todo != 0;)
    {
        const int l = __builtin_ctzll(todo);
        const int64_t c = (static_cast<int64_t>(__builtin_amdgcn_readlane(static_cast<int>(cloud >> 32), l)) << 32) |
                          static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(cloud), l));
        const int s0 = wave_lower_bound(batch_x, size_x, c, lane);
        const int s1 = wave_lower_bound(batch_x, size_x, c + 1, lane);
        const bool mine = valid && cloud == c;
        lo = mine ? s0 : lo;
        hi = mine ? s1 : hi;
        todo &= ~__ballot(mine);
    }
    const bool has_support = valid && hi > lo;
    const int first_row = wave_min_i32(has_support ? lo : 0x7FFFFFFF);
    const int last_row = wave_max_i32(has_support ? hi : 0);

    const int keep = nsample < BQG_KEEP ? nsample : BQG_KEEP;
    int cnt = 0;         // hits so far; keep + 1 = too many for this kernel
    bool active = has_support;
    if (last_row > first_row)
    {
        for (int wx = first_row / CURVE_MAX_POINTS; wx <= (last_row - 1) / CURVE_MAX_POINTS; ++wx)
        {
            const float4* __restrict__ cpts = sorted_x + static_cast<int64_t>(wx) * CELLS * NG_CELL;
            const float4* __restrict__ cbox = boxes_x + static_cast<int64_t>(wx) * CELLS * 2;
            const int row_base = wx * CURVE_MAX_POINTS;
            // box tests of the window's 256 cells first (their loads in flight together)
            static_assert(CELLS / NG_CELL == 4, "four groups of 64 cells per window");
            unsigned long long live_of[4];
#pragma unroll
            for (int g = 0; g < 4; ++g)
            {
                const int cc = g * NG_CELL + lane;
                const float lw = box_box_dist2(qlo, qhi, cbox[cc * 2 + 0], cbox[cc * 2 + 1]);
                live_of[g] = __ballot(lw * NG_MARGIN <= radius2); // empty boxes: +inf
            }
            for (int g = 0; g < 4; ++g)
            {
                unsigned long long live = g == 0 ? live_of[0] : g == 1 ? live_of[1] : g == 2 ? live_of[2] : live_of[3];
                while (live != 0)
                {
                    const int c = g * NG_CELL + __builtin_ctzll(live);
                    live &= live - 1;
                    const float lb = point_box_dist2(qx, qy, qz, cbox[c * 2 + 0], cbox[c * 2 + 1]);
                    if (__ballot(active && lb * NG_MARGIN <= radius2) == 0)
                        continue;
                    stage[lane] = cpts[c * NG_CELL + lane];
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    for (int k = 0; k < NG_CELL; ++k)
                    {
                        const float4 p = stage[k];
                        const float d = tpk_dist2(qx, qy, qz, p.x, p.y, p.z);
                        // (a padding record has index 0x7FFFFFFF: its row wraps out of every range)
                        const int row = static_cast<int>(static_cast<unsigned>(row_base) +
                                                         static_cast<unsigned>(__float_as_int(p.w)));
                        const bool hit = active && d <= radius2 && row >= lo && row < hi;
                        if (__ballot(hit) != 0 && hit)
                        {
                            if (cnt < keep)
                            {
                                my_rows[cnt * BQG_PITCH + lane] = row;
                                my_dists[cnt * BQG_PITCH + lane] = d;
                            }
                            ++cnt;
                            active = cnt <= keep;
                        }
                    }
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                }
            }
            if (__ballot(active) == 0)
                break;
        }
    }

    // Lanes with too many hits hand their query over; the others sort their hits by row.
    const bool handed_over = valid && cnt > keep;
    if (handed_over)
        overflow[BQG_LIST + atomicAdd(&overflow[0], 1)] = qrow;
    if (valid && !handed_over)
        for (int a = 1; a < cnt; ++a)
        {
            const int key = my_rows[a * BQG_PITCH + lane];
            const float kd = my_dists[a * BQG_PITCH + lane];
            int b = a - 1;
            while (b >= 0 && my_rows[b * BQG_PITCH + lane] > key)
            {
                my_rows[(b + 1) * BQG_PITCH + lane] = my_rows[b * BQG_PITCH + lane];
                my_dists[(b + 1) * BQG_PITCH + lane] = my_dists[b * BQG_PITCH + lane];
                --b;
            }
            my_rows[(b + 1) * BQG_PITCH + lane] = key;
            my_dists[(b + 1) * BQG_PITCH + lane] = kd;
        }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    // Rows are written by the whole wavefront, one query after the other: hits, then -1.
    const unsigned long long writers = __ballot(valid && !handed_over);
    for (unsigned long long todo = writers; todo != 0; todo &= todo - 1)
    {
        const int q = __builtin_ctzll(todo);
        const int64_t out = static_cast<int64_t>(__builtin_amdgcn_readlane(qrow, q)) * nsample;
        const int c = __builtin_amdgcn_readlane(cnt, q);
        for (int s = lane; s < nsample; s += TPK_WAVE)
        {
            const bool is_hit = s < c;
            const int at = (is_hit ? s : 0) * BQG_PITCH + q;
            idx[out + s] = is_hit ? static_cast<int64_t>(my_rows[at]) : -1;
            dist[out + s] = is_hit ? my_dists[at] : -1.0f;
        }
    }
}

// The queries handed over by ball_query_grid_kernel: one wavefront per query, the lanes hold 64
// consecutive support rows of the query's cloud; ballot + prefix count give the hits their slots
// in index order; the scan stops after nsample hits.
__global__ __launch_bounds__(NG_SCAN_THREADS) void ball_query_overflow_kernel(
    int size_x, float radius2, int nsample, const float* __restrict__ x, const float* __restrict__ y,
    const int64_t* __restrict__ batch_x, const int64_t* __restrict__ batch_y,
    int64_t* __restrict__ idx, float* __restrict__ dist, const int* __restrict__ overflow)
{
    constexpr int WAVES = NG_SCAN_THREADS / TPK_WAVE;
    const int lane = threadIdx.x & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TPK_WAVE);
    const int listed = overflow[0];
    for (int t = blockIdx.x * WAVES + wave; t < listed; t += gridDim.x * WAVES)
    {
        const int q = overflow[BQG_LIST + t];
        const float qx = to_vector_register(y[static_cast<int64_t>(q) * 3 + 0]);
        const float qy = to_vector_register(y[static_cast<int64_t>(q) * 3 + 1]);
        const float qz = to_vector_register(y[static_cast<int64_t>(q) * 3 + 2]);
        const int64_t c = batch_y[q];
        const int s0 = wave_lower_bound(batch_x, size_x, c, lane);
        const int s1 = wave_lower_bound(batch_x, size_x, c + 1, lane);
        const int64_t out = static_cast<int64_t>(q) * nsample;
        int cnt = 0;
        constexpr int BATCH = 4; // loads of four steps in flight
        for (int base = s0; base < s1 && cnt < nsample; base += BATCH * TPK_WAVE)
        {
            float px[BATCH], py[BATCH], pz[BATCH];
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
            {
                const int64_t pos = min(base + u * TPK_WAVE + lane, s1 - 1);
                px[u] = x[pos * 3 + 0];
                py[u] = x[pos * 3 + 1];
                pz[u] = x[pos * 3 + 2];
            }
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
            {
                const int pos = base + u * TPK_WAVE + lane;
                const float d = tpk_dist2(qx, qy, qz, px[u], py[u], pz[u]);
                const bool hit = pos < s1 && d <= radius2;
                const unsigned long long mask = __ballot(hit);
                const int slot = cnt + static_cast<int>(tpk_prefix_count(mask));
                if (hit && slot < nsample)
                {
                    idx[out + slot] = pos;
                    dist[out + slot] = d;
                }
                cnt += __builtin_popcountll(mask);
            }
        }
        for (int s = cnt + lane; s < nsample; s += TPK_WAVE)
        {
            idx[out + s] = -1;
            dist[out + s] = -1.0f;
        }
    }
}

struct GridLayout
{
    size_t sorted_a, sorted_b, boxes_a, boxes_b, total;
};

GridLayout grid_layout(int b, int n, int m)
{
    auto up = [](size_t v) { return (v + 255) & ~static_cast<size_t>(255); };
    const size_t cells_a = static_cast<size_t>((n + NG_CELL - 1) / NG_CELL);
    const size_t cells_b = static_cast<size_t>((m + NG_CELL - 1) / NG_CELL);
    GridLayout l;
    size_t pos = 0;
    l.sorted_a = pos;
    pos = up(pos + static_cast<size_t>(b) * cells_a * NG_CELL * sizeof(float4));
    l.sorted_b = pos;
    pos = up(pos + static_cast<size_t>(b) * cells_b * NG_CELL * sizeof(float4));
    l.boxes_a = pos;
    pos = up(pos + static_cast<size_t>(b) * cells_a * 2 * sizeof(float4));
    l.boxes_b = pos;
    pos = up(pos + static_cast<size_t>(b) * cells_b * 2 * sizeof(float4));
    l.total = pos;
    return l;
}

bool grid_supported(int b, int n, int m)
{
    // Small clouds are served as fast by the all-pairs scan; large ones do not fit the LDS sort.
    return b > 0 && n >= 512 && m >= 512 && n <= CURVE_MAX_POINTS && m <= CURVE_MAX_POINTS &&
           (m + NG_CELL - 1) / NG_CELL <= NG_MAX_CELLS && (n + NG_CELL - 1) / NG_CELL <= NG_MAX_CELLS;
}

int launch_curve_cells(const PointSet& a, const PointSet& c, int* zero_word, hipStream_t s)
{
    const int largest = a.stride > c.stride ? a.stride : c.stride;
    const int key_capacity = (largest + 63) & ~63;
    const int64_t windows_a = set_windows(a), windows_c = set_windows(c);
    if (windows_a + windows_c > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const size_t lds = (2 * static_cast<size_t>(key_capacity) + CURVE_BINS) * sizeof(unsigned);
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(curve_cells_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    if (e != hipSuccess)
        return static_cast<int>(e);
    hipLaunchKernelGGL(curve_cells_kernel, dim3(static_cast<unsigned>(windows_a + windows_c)),
                       dim3(NG_SORT_THREADS), lds, s, a, c, static_cast<int>(windows_a), key_capacity,
                       zero_word);
    return tpk_launch_status();
}

} // namespace

size_t tpk_grid_chamfer_workspace_bytes(int b, int n, int m)
{
    return grid_supported(b, n, m) ? grid_layout(b, n, m).total : 0;
}

int tpk_grid_chamfer_fwd(int b, int n, int m, const float* xyz1, const float* xyz2, float* dist1,
                         float* dist2, int32_t* idx1, int32_t* idx2, void* workspace,
                         size_t workspace_bytes, hipStream_t s)
{
    if (!grid_supported(b, n, m) || static_cast<int64_t>(b) * 2 > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const GridLayout l = grid_layout(b, n, m);
    if (!workspace || workspace_bytes < l.total || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return TPK_ERR_WORKSPACE;
    char* w = static_cast<char*>(workspace);
    PointSet a{xyz1, nullptr, static_cast<int64_t>(b) * n, n, reinterpret_cast<float4*>(w + l.sorted_a),
               reinterpret_cast<float4*>(w + l.boxes_a)};
    PointSet c{xyz2, nullptr, static_cast<int64_t>(b) * m, m, reinterpret_cast<float4*>(w + l.sorted_b),
               reinterpret_cast<float4*>(w + l.boxes_b)};
    int st = launch_curve_cells(a, c, nullptr, s);
    if (st != TPK_OK)
        return st;
    const int64_t waves = static_cast<int64_t>((n + NG_CELL - 1) / NG_CELL + (m + NG_CELL - 1) / NG_CELL) * b;
    const int64_t blocks = tpk_ceil_div(waves, NG_SCAN_THREADS / TPK_WAVE);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(chamfer_grid_kernel, dim3(static_cast<unsigned>(blocks)), dim3(NG_SCAN_THREADS), 0, s, n,
                       m, b, a.sorted, c.sorted, a.boxes, c.boxes, dist1, dist2, idx1, idx2);
    return tpk_launch_status();
}

size_t tpk_grid_three_nn_workspace_bytes(int b, int n, int m)
{
    return grid_supported(b, n, m) ? grid_layout(b, n, m).total : 0;
}

int tpk_grid_three_nn(int b, int n, int m, const float* unknown, const float* known, float* dist2,
                      int32_t* idx, void* workspace, size_t workspace_bytes, hipStream_t s)
{
    if (!grid_supported(b, n, m) || static_cast<int64_t>(b) * 2 > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const GridLayout l = grid_layout(b, n, m);
    if (!workspace || workspace_bytes < l.total || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return TPK_ERR_WORKSPACE;
    char* w = static_cast<char*>(workspace);
    PointSet a{unknown, nullptr, static_cast<int64_t>(b) * n, n, reinterpret_cast<float4*>(w + l.sorted_a),
               reinterpret_cast<float4*>(w + l.boxes_a)};
    PointSet c{known, nullptr, static_cast<int64_t>(b) * m, m, reinterpret_cast<float4*>(w + l.sorted_b),
               reinterpret_cast<float4*>(w + l.boxes_b)};
    int st = launch_curve_cells(a, c, nullptr, s);
    if (st != TPK_OK)
        return st;
    const int64_t waves = static_cast<int64_t>((n + NG_CELL - 1) / NG_CELL) * b;
    const int64_t blocks = tpk_ceil_div(waves, NG_SCAN_THREADS / TPK_WAVE);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(three_nn_grid_kernel, dim3(static_cast<unsigned>(blocks)), dim3(NG_SCAN_THREADS), 0, s, n,
                       m, b, a.sorted, c.sorted, a.boxes, c.boxes, dist2, idx);
    return tpk_launch_status();
}

namespace {

struct BallLayout
{
    size_t sorted_x, sorted_y, boxes_x, boxes_y, overflow, total;
};

BallLayout ball_layout(int64_t size_x, int64_t size_y)
{
    auto up = [](size_t v) { return (v + 255) & ~static_cast<size_t>(255); };
    const size_t wx = static_cast<size_t>((size_x + CURVE_MAX_POINTS - 1) / CURVE_MAX_POINTS);
    const size_t wy = static_cast<size_t>((size_y + CURVE_MAX_POINTS - 1) / CURVE_MAX_POINTS);
    const size_t cells = CURVE_MAX_POINTS / NG_CELL;
    BallLayout l;
    size_t pos = 0;
    l.sorted_x = pos;
    pos = up(pos + wx * CURVE_MAX_POINTS * sizeof(float4));
    l.sorted_y = pos;
    pos = up(pos + wy * CURVE_MAX_POINTS * sizeof(float4));
    l.boxes_x = pos;
    pos = up(pos + wx * cells * 2 * sizeof(float4));
    l.boxes_y = pos;
    pos = up(pos + wy * cells * 2 * sizeof(float4));
    l.overflow = pos;
    pos = up(pos + (static_cast<size_t>(size_y) + BQG_LIST) * sizeof(int));
    l.total = pos;
    return l;
}

bool ball_grid_supported(int64_t size_x, int64_t size_y, int nsample)
{
    // Small problems are served as fast by the all-pairs scan; rows are 32-bit here.
    return size_x >= 8192 && size_y >= 64 && nsample > 0 && size_x < (1LL << 30) && size_y < (1LL << 30);
}

} // namespace

size_t tpk_grid_ball_query_workspace_bytes(int64_t size_x, int64_t size_y, int nsample)
{
    return ball_grid_supported(size_x, size_y, nsample) ? ball_layout(size_x, size_y).total : 0;
}

int tpk_grid_ball_query_partial(int64_t size_x, int64_t size_y, float radius2, int nsample, const float* x,
                                const float* y, const int64_t* batch_x, const int64_t* batch_y,
                                int64_t* idx, float* dist, void* workspace, size_t workspace_bytes,
                                hipStream_t s)
{
    if (!ball_grid_supported(size_x, size_y, nsample))
        return TPK_ERR_UNSUPPORTED;
    const BallLayout l = ball_layout(size_x, size_y);
    if (!workspace || workspace_bytes < l.total || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return TPK_ERR_WORKSPACE;
    char* w = static_cast<char*>(workspace);
    PointSet px{x, batch_x, size_x, CURVE_MAX_POINTS, reinterpret_cast<float4*>(w + l.sorted_x),
                reinterpret_cast<float4*>(w + l.boxes_x)};
    PointSet py{y, batch_y, size_y, CURVE_MAX_POINTS, reinterpret_cast<float4*>(w + l.sorted_y),
                reinterpret_cast<float4*>(w + l.boxes_y)};
    int* overflow = reinterpret_cast<int*>(w + l.overflow);
    int st = launch_curve_cells(px, py, overflow, s);
    if (st != TPK_OK)
        return st;
    constexpr int WAVES = NG_SCAN_THREADS / TPK_WAVE;
    const int64_t waves = set_windows(py) * (CURVE_MAX_POINTS / NG_CELL);
    hipLaunchKernelGGL(ball_query_grid_kernel, dim3(static_cast<unsigned>(tpk_ceil_div(waves, WAVES))),
                       dim3(NG_SCAN_THREADS), 0, s, static_cast<int>(size_x), static_cast<int>(size_y), radius2,
                       nsample, px.sorted, px.boxes, py.sorted, py.boxes, batch_x, batch_y, idx, dist, overflow);
    st = tpk_launch_status();
    if (st != TPK_OK)
        return st;
    // The number of handed-over queries is known on the device only: a fixed grid walks the list.
    const unsigned blocks = static_cast<unsigned>(tpk_min64(tpk_ceil_div(size_y, WAVES), 2048));
    hipLaunchKernelGGL(ball_query_overflow_kernel, dim3(blocks), dim3(NG_SCAN_THREADS), 0, s,
                       static_cast<int>(size_x), radius2, nsample, x, y, batch_x, batch_y, idx, dist, overflow);
    return tpk_launch_status();
}
