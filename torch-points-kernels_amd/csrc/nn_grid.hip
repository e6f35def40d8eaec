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

struct CloudSet
{
    const float* xyz; // [clouds][count][3]
    int count;
    float4* sorted;   // [clouds][cells * 64]
    float4* boxes;    // [clouds][cells][2]: (lo.xyz, -), (hi.xyz, -)
};

// One workgroup orders one cloud of one set: blockIdx.x = cloud * sets + set.
__global__ __launch_bounds__(NG_SORT_THREADS) void curve_cells_kernel(CloudSet set_a, CloudSet set_b,
                                                                      int sets, int key_capacity)
{
    extern __shared__ unsigned sort_keys[];
    unsigned* const unsorted = sort_keys + key_capacity;
    int* const bins = reinterpret_cast<int*>(unsorted + key_capacity);
    __shared__ int cloud_box[6];
    __shared__ int wave_totals[NG_SORT_THREADS / TPK_WAVE];

    const int cloud = blockIdx.x / sets;
    const CloudSet set = (blockIdx.x - cloud * sets) ? set_b : set_a;
    const int n = set.count;
    const int cells = (n + NG_CELL - 1) / NG_CELL;
    const float* __restrict__ xyz = set.xyz + static_cast<int64_t>(cloud) * n * 3;
    float4* __restrict__ sorted = set.sorted + static_cast<int64_t>(cloud) * cells * NG_CELL;
    float4* __restrict__ boxes = set.boxes + static_cast<int64_t>(cloud) * cells * 2;
    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);

    curve_order<NG_SORT_THREADS>(xyz, n, sort_keys, unsorted, bins, cloud_box, wave_totals);

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
            // Padding: infinitely far away, with an index no real point has.
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

int launch_curve_cells(int b, CloudSet a, CloudSet c, hipStream_t s)
{
    const int largest = a.count > c.count ? a.count : c.count;
    const int key_capacity = (largest + 63) & ~63;
    const size_t lds = (2 * static_cast<size_t>(key_capacity) + CURVE_BINS) * sizeof(unsigned);
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(curve_cells_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    if (e != hipSuccess)
        return static_cast<int>(e);
    hipLaunchKernelGGL(curve_cells_kernel, dim3(static_cast<unsigned>(b) * 2), dim3(NG_SORT_THREADS), lds, s, a,
                       c, 2, key_capacity);
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
    CloudSet a{xyz1, n, reinterpret_cast<float4*>(w + l.sorted_a), reinterpret_cast<float4*>(w + l.boxes_a)};
    CloudSet c{xyz2, m, reinterpret_cast<float4*>(w + l.sorted_b), reinterpret_cast<float4*>(w + l.boxes_b)};
    int st = launch_curve_cells(b, a, c, s);
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
    CloudSet a{unknown, n, reinterpret_cast<float4*>(w + l.sorted_a), reinterpret_cast<float4*>(w + l.boxes_a)};
    CloudSet c{known, m, reinterpret_cast<float4*>(w + l.sorted_b), reinterpret_cast<float4*>(w + l.boxes_b)};
    int st = launch_curve_cells(b, a, c, s);
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
