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
// 160 bytes per cell (its box and those of its four runs of 16 points).  The curve ordering works
// in LDS on at most 16384 points: a larger cloud (up to 163840 points) is ordered in windows of
// 16384 consecutive points, which the search sees as more - and wider - cells of the same cloud.
#include "curve_cells.h"

#include <algorithm>
#include <cmath>
#include "nn_grid.h"
#include "topk.h"

namespace {

constexpr int NG_MAX_CELLS = 2560;           // candidate cells per cloud (their box distances sit in LDS)
constexpr int NG_WINDOW = CURVE_MAX_POINTS;  // larger clouds are ordered in windows of this many points
constexpr int NG_SCAN_THREADS = 256;         // 4 wavefronts, each searching on its own
constexpr float NG_MARGIN = 0.999998f;
constexpr int NG_CHUNK = 8;

// Box of the 64 queries of a wavefront (one query per lane; a padding lane - index 0x7FFFFFFF - holds none),
// the same value in every lane.  The ordering kernel forms no boxes for a set that is only queried.
__device__ __forceinline__ void query_box(float qx, float qy, float qz, bool real, float4& lo, float4& hi)
{
    const float v[3] = {qx, qy, qz};
    float l[3], h[3];
#pragma unroll
    for (int a = 0; a < 3; ++a)
    {
        const int ordered = float_to_ordered_int(v[a]);
        l[a] = ordered_int_to_float(wave_min_i32(real ? ordered : float_to_ordered_int(__builtin_inff())));
        h[a] = ordered_int_to_float(wave_max_i32(real ? ordered : float_to_ordered_int(-__builtin_inff())));
    }
    lo = make_float4(l[0], l[1], l[2], 0.f);
    hi = make_float4(h[0], h[1], h[2], 0.f);
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
__device__ __forceinline__ void scan_cell(const float4* __restrict__ cand, const float4* __restrict__ boxes,
                                          int cell, float4* stage, int lane, float qx, float qy, float qz,
                                          Nearest& s TPK_WORK_PARAM)
{
    stage[lane] = cand[cell * NG_CELL + lane];
    // (the boxes of the cell's four runs are requested together with its candidates: one wait, not five)
    float4 quarter[NG_BOX - 2];
#pragma unroll
    for (int i = 0; i < NG_BOX - 2; ++i)
        quarter[i] = boxes[cell * NG_BOX + 2 + i];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); // LDS serves a wavefront's requests in order
#pragma unroll
    for (int run = 0; run < NG_CELL / (2 * NG_CHUNK); ++run)
    {
        // a run of 16 candidates whose box no lane's answer reaches is passed over
        const float lb = point_box_dist2(qx, qy, qz, quarter[2 * run], quarter[2 * run + 1]);
        if (__ballot(lb * NG_MARGIN <= s.best) == 0)
            continue;
#pragma unroll
        for (int half = 0; half < 2; ++half)
        {
            const int ch = 2 * run + half;
            float mn = 0.f;
#pragma unroll
            for (int c = 0; c < NG_CHUNK; ++c)
            {
                const float4 p = stage[ch * NG_CHUNK + c];
                // Operand order of the reference: (scanned - query), squares summed x, y, z.
                const float d = tpk_dist2(p.x, p.y, p.z, qx, qy, qz);
                mn = c == 0 ? d : fminf(mn, d);
            }
            TPK_WORK_ADD(NG_CHUNK);
            const bool better = mn < s.best;
            const bool equal = mn == s.best;
            s.tie = better ? false : (s.tie || equal);
            s.chunk = better ? cell * (NG_CELL / NG_CHUNK) + ch : s.chunk;
            s.best = better ? mn : s.best;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// The same for a cell that only a few queries of the wavefront still ask for (an outlier among the
// queries keeps admitting cells that the other 63 have long turned down): one query at a time, the
// 64 candidates of the cell side by side in the lanes.  `want`: the lanes whose queries ask.
// A minimum reached in the cell by several groups of NG_CHUNK candidates, or equal to the query's
// answer so far, sets the tie flag exactly as the scan above would.
constexpr int NG_DEAL = 8;   // windows whose cells are dealt out together, wide cells first
constexpr int NG_FEW = 8; // (the scan above costs about as much as 14 queries served this way; 16: the same time, 24: slower)
__device__ __forceinline__ void scan_cell_few(const float4* __restrict__ cand, int cell, unsigned long long want,
                                              int lane, float qx, float qy, float qz, Nearest& s TPK_WORK_PARAM)
{
    const float4 p = cand[cell * NG_CELL + lane];
    while (want != 0)
    {
        const int q = __builtin_ctzll(want);
        want &= want - 1;
        TPK_WORK_ADD(1);
        const float ux = tpk_read_lane(qx, q), uy = tpk_read_lane(qy, q), uz = tpk_read_lane(qz, q);
        const float d = tpk_dist2(p.x, p.y, p.z, ux, uy, uz); // (a padding candidate lies at infinity)
        // distances are >= +0: their bit patterns order like integers (a NaN sorts above infinity)
        const float mn = __int_as_float(wave_min_i32(__float_as_int(d)));
        const unsigned long long at = __ballot(d == mn);
        if (at == 0)
            continue; // nothing but NaN
        const int first = __builtin_ctzll(at);
        const bool several = (at & ~(0xFFull << (first & ~(NG_CHUNK - 1)))) != 0;
        if (lane == q)
        {
            const bool better = mn < s.best;
            const bool equal = mn == s.best;
            s.tie = better ? several : (s.tie || equal);
            s.chunk = better ? cell * (NG_CELL / NG_CHUNK) + first / NG_CHUNK : s.chunk;
            s.best = better ? mn : s.best;
        }
    }
}

// One wavefront = the 64 queries of one cell.  Logical wavefront number (after the die-local
// block mapping) = cloud * (cells1 + cells2) + cell; the cells of cloud 1 query cloud 2 and
// write dist1 / idx1, those of cloud 2 the other way round.
__global__ __launch_bounds__(NG_SCAN_THREADS) void chamfer_grid_kernel(
    int n, int m, int cells1, int cells2, int clouds, const float4* __restrict__ sorted1,
    const float4* __restrict__ sorted2, const float4* __restrict__ boxes1,
    const float4* __restrict__ boxes2, float* __restrict__ dist1, float* __restrict__ dist2,
    int32_t* __restrict__ idx1, int32_t* __restrict__ idx2, const int* __restrict__ wide1,
    const int* __restrict__ wide2, int window_cells)
{
    __shared__ float4 stages[NG_SCAN_THREADS / TPK_WAVE][NG_CELL];
    extern __shared__ float lows_all[]; // [wavefronts][largest number of candidate cells, in whole groups of 64]

    const int lane = threadIdx.x & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TPK_WAVE);
    const int per_cloud = cells1 + cells2;
    const int64_t task = static_cast<int64_t>(xcd_local_block(blockIdx.x, gridDim.x)) *
                             (NG_SCAN_THREADS / TPK_WAVE) + wave;
    if (task >= static_cast<int64_t>(per_cloud) * clouds)
        return; // (no workgroup barrier anywhere in this kernel)
    int cloud = static_cast<int>(task / per_cloud);
    int r = static_cast<int>(task - static_cast<int64_t>(cloud) * per_cloud);
    if (window_cells > 0)
    {
        // Wavefronts start in the order of their numbers, and the call lasts as long as the wavefront that ends
        // last: the cells with the widest boxes - whose queries search longest - go first.  The cells of both
        // clouds' windows are dealt out in groups of NG_DEAL windows, window after window, every window
        // handing out its cells in the order the ordering kernel left: wide ones first.
        const int per_cloud_windows = per_cloud / window_cells;
        const int64_t all_windows = static_cast<int64_t>(per_cloud_windows) * clouds;
        const int64_t group = task / (NG_DEAL * window_cells);
        const int within = static_cast<int>(task - group * (NG_DEAL * window_cells));
        const int dealt = static_cast<int>(tpk_min64(NG_DEAL, all_windows - group * NG_DEAL));
        const int64_t window = group * NG_DEAL + within % dealt;
        const int rank = within / dealt;
        cloud = static_cast<int>(window / per_cloud_windows);
        const int k = static_cast<int>(window - static_cast<int64_t>(cloud) * per_cloud_windows);
        const int windows1 = cells1 / window_cells;
        const bool in_second = k >= windows1;
        const int own = in_second ? k - windows1 : k; // the window's number in its cloud
        const int* __restrict__ order = in_second ? wide2 + (static_cast<int64_t>(cloud) * (per_cloud_windows - windows1) + own) * window_cells
                                                  : wide1 + (static_cast<int64_t>(cloud) * windows1 + own) * window_cells;
        r = (in_second ? cells1 : 0) + own * window_cells + order[rank];
    }
    const bool second = r >= cells1;
    const int qcell = second ? r - cells1 : r;
    const int qcells = second ? cells2 : cells1;
    const int ccells = second ? cells1 : cells2;
    const int qcount = second ? m : n;
    const float4* __restrict__ qpts = (second ? sorted2 : sorted1) + static_cast<int64_t>(cloud) * qcells * NG_CELL;
    const float4* __restrict__ qbox = (second ? boxes2 : boxes1) + static_cast<int64_t>(cloud) * qcells * NG_BOX;
    const float4* __restrict__ cpts = (second ? sorted1 : sorted2) + static_cast<int64_t>(cloud) * ccells * NG_CELL;
    const float4* __restrict__ cbox = (second ? boxes1 : boxes2) + static_cast<int64_t>(cloud) * ccells * NG_BOX;
    float* __restrict__ dout = (second ? dist2 : dist1) + static_cast<int64_t>(cloud) * qcount;
    int32_t* __restrict__ iout = (second ? idx2 : idx1) + static_cast<int64_t>(cloud) * qcount;
    float4* const stage = stages[wave];
    float* const lows = lows_all + wave * ((max(cells1, cells2) + NG_CELL - 1) / NG_CELL * NG_CELL);
    TPK_WORK_DECL

    const float4 query = qpts[qcell * NG_CELL + lane];
    const float qx = query.x, qy = query.y, qz = query.z;
    const int qindex = __float_as_int(query.w); // 0x7FFFFFFF: padding, nothing to store
    if (__ballot(qindex != 0x7FFFFFFF) == 0)
        return; // a cell without points (the last window of a cloud may have some)
    const float4 qlo = qbox[qcell * NG_BOX + 0], qhi = qbox[qcell * NG_BOX + 1];

    // Box distances to all candidate cells, kept in the wavefront's LDS row (lane l computes
    // cells l, 64 + l, ...); +inf marks a cell that does not exist or has been scanned.
    const int groups = (ccells + NG_CELL - 1) / NG_CELL;
    unsigned seed_key = 0xFFFFFFFFu;
    for (int g = 0; g < groups; ++g)
    {
        const int c = g * NG_CELL + lane;
        const bool valid = c < ccells;
        const int cc = valid ? c : 0;
        const float4 clo = cbox[cc * NG_BOX + 0], chi = cbox[cc * NG_BOX + 1];
        const float lb = box_box_dist2(qlo, qhi, clo, chi);
        lows[c] = valid ? lb : __builtin_inff();
        // The first cell to scan: the one whose box centre is nearest to the centre of the queries'
        // box (many boxes overlap it; a good first answer lets the lanes turn most of them down).
        // The six lowest bits of the distance carry g.
        const float ex = (clo.x + chi.x) - (qlo.x + qhi.x), ey = (clo.y + chi.y) - (qlo.y + qhi.y);
        const float ez = (clo.z + chi.z) - (qlo.z + qhi.z);
        const float centre = __builtin_fmaf(ex, ex, __builtin_fmaf(ey, ey, ez * ez));
        const unsigned key = (static_cast<unsigned>(__float_as_int(centre)) & ~63u) | static_cast<unsigned>(g);
        seed_key = valid && lb < __builtin_inff() && key < seed_key ? key : seed_key;
    }
    Nearest s;
    s.best = qindex == 0x7FFFFFFF ? -1.f : __builtin_inff(); // (a padding lane never asks for a scan)
    s.chunk = 0;
    s.tie = false;
    {
        const unsigned lowest = wave_min_u32(seed_key);
        int seed = static_cast<int>(lowest & 63u) * NG_CELL + __builtin_ctzll(__ballot(seed_key == lowest));
        if (seed >= ccells) // no lane had a usable key (NaN boxes)
            seed = 0;
        scan_cell(cpts, cbox, seed, stage, lane, qx, qy, qz, s TPK_WORK_ARG);
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
                const float lb = point_box_dist2(qx, qy, qz, cbox[c * NG_BOX + 0], cbox[c * NG_BOX + 1]);
                const unsigned long long want = __ballot(lb * NG_MARGIN <= s.best);
                // scanned, or no lane can improve here now - and answers only get better: never again
                if (lane == bit)
                    lows[c] = __builtin_inff();
                if (want == 0)
                    continue;
                if (__builtin_popcountll(want) <= NG_FEW)
                    scan_cell_few(cpts, c, want, lane, qx, qy, qz, s TPK_WORK_ARG);
                else
                    scan_cell(cpts, cbox, c, stage, lane, qx, qy, qz, s TPK_WORK_ARG);
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
    // Several groups reached a query's minimum (about one query in 10^5 on random clouds, every query on a
    // lattice): the lowest index over all cells that can hold that distance.  One such query at a time: the
    // lanes test the boxes of all cells side by side, then the candidates of every cell that passes.
    for (unsigned long long tied = __ballot(s.tie); tied != 0; tied &= tied - 1)
    {
        const int q = __builtin_ctzll(tied);
        const float ux = tpk_read_lane(qx, q), uy = tpk_read_lane(qy, q), uz = tpk_read_lane(qz, q);
        const float ub = tpk_read_lane(s.best, q);
        int lowest = 0x7FFFFFFF;
        for (int g = 0; g < groups; ++g)
        {
            const int c = g * NG_CELL + lane;
            const int cc = c < ccells ? c : 0;
            const float lb = point_box_dist2(ux, uy, uz, cbox[cc * NG_BOX + 0], cbox[cc * NG_BOX + 1]);
            for (unsigned long long cells = __ballot(c < ccells && lb * NG_MARGIN <= ub); cells != 0; cells &= cells - 1)
            {
                const float4 p = cpts[(g * NG_CELL + __builtin_ctzll(cells)) * NG_CELL + lane];
                const float d = tpk_dist2(p.x, p.y, p.z, ux, uy, uz);
                TPK_WORK_ADD(1);
                lowest = min(lowest, wave_min_i32(d == ub ? __float_as_int(p.w) : 0x7FFFFFFF));
            }
        }
        bi = lane == q ? min(bi, lowest) : bi;
    }
    TPK_WORK_ADD(NG_CHUNK);
    TPK_WORK_FLUSH
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

__device__ __forceinline__ void scan_cell3(const float4* __restrict__ cand, const float4* __restrict__ boxes,
                                           int cell, float4* stage, int lane, float qx, float qy, float qz,
                                           Nearest3& s TPK_WORK_PARAM)
{
    stage[lane] = cand[cell * NG_CELL + lane];
    // (the boxes of the cell's four runs are requested together with its candidates: one wait, not five)
    float4 quarter[NG_BOX - 2];
#pragma unroll
    for (int i = 0; i < NG_BOX - 2; ++i)
        quarter[i] = boxes[cell * NG_BOX + 2 + i];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    bool reached = true;
#pragma unroll
    for (int ch = 0; ch < NG_CELL / NG_CHUNK; ++ch)
    {
        // a run of 16 candidates whose box no lane's third best reaches is passed over
        // (decided at the run's first group: `reached` carries it to the second)
        if ((ch & 1) == 0)
        {
            const float lb = point_box_dist2(qx, qy, qz, quarter[ch], quarter[ch + 1]);
            reached = __ballot(lb * NG_MARGIN <= s.b3) != 0;
        }
        if (!reached)
            continue;
        float mn = 0.f;
        float ds[NG_CHUNK];
        int cis[NG_CHUNK];
#pragma unroll
        for (int c = 0; c < NG_CHUNK; ++c)
        {
            const float4 p = stage[ch * NG_CHUNK + c];
            // Operand order of the reference: (query - scanned).
            ds[c] = tpk_dist2(qx, qy, qz, p.x, p.y, p.z);
            cis[c] = __float_as_int(p.w);
            mn = c == 0 ? ds[c] : fminf(mn, ds[c]);
        }
        TPK_WORK_ADD(NG_CHUNK);
        if (__ballot(mn <= s.b3) == 0)
            continue; // no candidate of this group enters any lane's triple
#pragma unroll
        for (int c = 0; c < NG_CHUNK; ++c)
        {
            const float d = ds[c];
            const int ci = cis[c];
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
// The same for a cell that only a few queries of the wavefront still ask for: one query at a time, the
// 64 candidates of the cell side by side in the lanes (`want`: the lanes whose queries ask).  The candidates
// that enter the query's triple are taken smallest first in the triple's order (distance, then index); no
// more than three of them can stay.
constexpr int NG_FEW3 = 8; // (uniform clouds, 16 x 16384 queries: 0 / 4 / 8 / 12 / 16: 98.7 / 95.1 / 94.9 / 95.6 / 99.8 us)
__device__ __forceinline__ void scan_cell3_few(const float4* __restrict__ cand, int cell, unsigned long long want,
                                               int lane, float qx, float qy, float qz, Nearest3& s TPK_WORK_PARAM)
{
    const float4 p = cand[cell * NG_CELL + lane];
    const int ci = __float_as_int(p.w);
    while (want != 0)
    {
        const int q = __builtin_ctzll(want);
        want &= want - 1;
        TPK_WORK_ADD(1);
        const float ux = tpk_read_lane(qx, q), uy = tpk_read_lane(qy, q), uz = tpk_read_lane(qz, q);
        // Operand order of the reference: (query - scanned).
        const float d = tpk_dist2(ux, uy, uz, p.x, p.y, p.z);
        unsigned long long in = __ballot(pair_less(d, ci, tpk_read_lane(s.b3, q), tpk_read_lane(s.i3, q)));
        for (int r = 0; r < 3 && in != 0; ++r)
        {
            // distances are >= +0: their bit patterns order like integers
            const bool mine = (in >> lane) & 1ull;
            const int least = wave_min_i32(mine ? __float_as_int(d) : 0x7FFFFFFF);
            unsigned long long at = __ballot(mine && __float_as_int(d) == least);
            if (at & (at - 1)) // equal distances: the lowest index
            {
                const bool tied = (at >> lane) & 1ull;
                const int first = wave_min_i32(tied ? ci : 0x7FFFFFFF);
                at = __ballot(tied && ci == first);
            }
            const int from = __builtin_ctzll(at);
            in &= ~(1ull << from);
            const float dv = __int_as_float(least);
            const int cv = tpk_read_lane(ci, from);
            if (lane == q)
            {
                const bool l3 = pair_less(dv, cv, s.b3, s.i3);
                const bool l2 = pair_less(dv, cv, s.b2, s.i2);
                const bool l1 = pair_less(dv, cv, s.b1, s.i1);
                s.b3 = l2 ? s.b2 : (l3 ? dv : s.b3);
                s.i3 = l2 ? s.i2 : (l3 ? cv : s.i3);
                s.b2 = l1 ? s.b1 : (l2 ? dv : s.b2);
                s.i2 = l1 ? s.i1 : (l2 ? cv : s.i2);
                s.b1 = l1 ? dv : s.b1;
                s.i1 = l1 ? cv : s.i1;
            }
        }
    }
}

__global__ __launch_bounds__(NG_SCAN_THREADS) void three_nn_grid_kernel(
    int n, int m, int qcells, int ccells, int clouds, const float4* __restrict__ sorted_unknown,
    const float4* __restrict__ sorted_known, const float4* __restrict__ boxes_known, float* __restrict__ dist2,
    int32_t* __restrict__ idx, const int* __restrict__ only)
{
    __shared__ float4 stages[NG_SCAN_THREADS / TPK_WAVE][NG_CELL];
    extern __shared__ float lows_all[]; // [wavefronts][candidate cells, in whole groups of 64]

    const int lane = threadIdx.x & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TPK_WAVE);
    const int64_t task = static_cast<int64_t>(xcd_local_block(blockIdx.x, gridDim.x)) *
                             (NG_SCAN_THREADS / TPK_WAVE) + wave;
    if (task >= static_cast<int64_t>(qcells) * clouds)
        return; // (no workgroup barrier anywhere in this kernel)
    const int cloud = static_cast<int>(task / qcells);
    if (only && only[cloud] == 0)
        return; // (a cloud that another kernel has answered)
    const int qcell = static_cast<int>(task - static_cast<int64_t>(cloud) * qcells);
    const float4* __restrict__ qpts = sorted_unknown + static_cast<int64_t>(cloud) * qcells * NG_CELL;
    const float4* __restrict__ cpts = sorted_known + static_cast<int64_t>(cloud) * ccells * NG_CELL;
    const float4* __restrict__ cbox = boxes_known + static_cast<int64_t>(cloud) * ccells * NG_BOX;
    dist2 += static_cast<int64_t>(cloud) * n * 3;
    idx += static_cast<int64_t>(cloud) * n * 3;
    float4* const stage = stages[wave];
    float* const lows = lows_all + wave * ((ccells + NG_CELL - 1) / NG_CELL * NG_CELL);
    TPK_WORK_DECL

    const float4 query = qpts[qcell * NG_CELL + lane];
    const float qx = query.x, qy = query.y, qz = query.z;
    const int qindex = __float_as_int(query.w); // 0x7FFFFFFF: padding, nothing to store
    if (__ballot(qindex != 0x7FFFFFFF) == 0)
        return; // a cell without points (the last window of a cloud may have some)
    float4 qlo, qhi;
    query_box(qx, qy, qz, qindex != 0x7FFFFFFF, qlo, qhi);

    const int groups = (ccells + NG_CELL - 1) / NG_CELL;
    unsigned seed_key = 0xFFFFFFFFu;
    for (int g = 0; g < groups; ++g)
    {
        const int c = g * NG_CELL + lane;
        const bool valid = c < ccells;
        const int cc = valid ? c : 0;
        const float4 clo = cbox[cc * NG_BOX + 0], chi = cbox[cc * NG_BOX + 1];
        const float lb = box_box_dist2(qlo, qhi, clo, chi);
        lows[c] = valid ? lb : __builtin_inff();
        // the first cell to scan: nearest box centre (the six lowest bits of the distance carry g)
        const float ex = (clo.x + chi.x) - (qlo.x + qhi.x), ey = (clo.y + chi.y) - (qlo.y + qhi.y);
        const float ez = (clo.z + chi.z) - (qlo.z + qhi.z);
        const float centre = __builtin_fmaf(ex, ex, __builtin_fmaf(ey, ey, ez * ez));
        const unsigned key = (static_cast<unsigned>(__float_as_int(centre)) & ~63u) | static_cast<unsigned>(g);
        seed_key = valid && lb < __builtin_inff() && key < seed_key ? key : seed_key;
    }
    Nearest3 s;
    s.b1 = s.b2 = s.b3 = qindex == 0x7FFFFFFF ? -1.f : __builtin_inff(); // (a padding lane never asks for a scan)
    s.i1 = s.i2 = s.i3 = 0;
    {
        const unsigned lowest = wave_min_u32(seed_key);
        int seed = static_cast<int>(lowest & 63u) * NG_CELL + __builtin_ctzll(__ballot(seed_key == lowest));
        if (seed >= ccells)
            seed = 0;
        scan_cell3(cpts, cbox, seed, stage, lane, qx, qy, qz, s TPK_WORK_ARG);
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
                const float lb = point_box_dist2(qx, qy, qz, cbox[c * NG_BOX + 0], cbox[c * NG_BOX + 1]);
                const unsigned long long want = __ballot(lb * NG_MARGIN <= s.b3);
                if (want != 0 && __builtin_popcountll(want) <= NG_FEW3)
                    scan_cell3_few(cpts, c, want, lane, qx, qy, qz, s TPK_WORK_ARG);
                else if (want != 0)
                    scan_cell3(cpts, cbox, c, stage, lane, qx, qy, qz, s TPK_WORK_ARG);
                if (lane == bit)
                    lows[c] = __builtin_inff(); // scanned, or useless now and ever after
                if (phase)
                {
                    bound = __int_as_float(wave_max_i32(__float_as_int(s.b3)));
                    live &= __ballot(lw * NG_MARGIN <= bound);
                }
            }
        }
    TPK_WORK_FLUSH
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
// k nearest neighbours over cells: three_nn's search with a list of up to 32 entries per lane
// (topk.h).  A larger k is served in rounds: round r finds the entries 32 r .. 32 r + 31, which
// are the smallest pairs after the last one of the round before.  A cell is skipped when its box
// is further away than the last kept entry of every lane.
// ---------------------------------------------------------------------------------------
template <int K>
__device__ __forceinline__ void scan_cell_k(const float4* __restrict__ cand, const float4* __restrict__ boxes,
                                            int cell, float4* stage, int lane, float qx, float qy, float qz,
                                            NearestK<K>& s)
{
    stage[lane] = cand[cell * NG_CELL + lane];
    float worst = s.worst(); // distance of the lane's last entry
    // The runs of 16 candidates whose box no lane's last entry reaches are passed over.  The four boxes are
    // requested together with the candidates and tested before the scan: one wait, not five.
    unsigned reached = 0;
    {
        float4 quarter[NG_BOX - 2];
#pragma unroll
        for (int i = 0; i < NG_BOX - 2; ++i)
            quarter[i] = boxes[cell * NG_BOX + 2 + i];
#pragma unroll
        for (int run = 0; run < (NG_BOX - 2) / 2; ++run)
        {
            const float lb = point_box_dist2(qx, qy, qz, quarter[2 * run], quarter[2 * run + 1]);
            reached |= __ballot(lb * NG_MARGIN <= worst) != 0 ? 1u << run : 0u;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    for (int ch = 0; ch < NG_CELL / NG_CHUNK; ++ch)
    {
        if (((reached >> (ch >> 1)) & 1u) == 0)
            continue;
        float mn = 0.f;
        float ds[NG_CHUNK];
        int cis[NG_CHUNK];
#pragma unroll
        for (int c = 0; c < NG_CHUNK; ++c)
        {
            const float4 p = stage[ch * NG_CHUNK + c];
            ds[c] = tpk_dist2(qx, qy, qz, p.x, p.y, p.z);
            cis[c] = __float_as_int(p.w);
            mn = c == 0 ? ds[c] : fminf(mn, ds[c]);
        }
        if (__ballot(mn <= worst) == 0)
            continue; // no candidate of this group enters any lane's list
#pragma unroll
        for (int c = 0; c < NG_CHUNK; ++c)
        {
            const unsigned long long cand = knn_key(ds[c], cis[c]);
            const bool in = s.admits(cand);
            if (__ballot(in) == 0)
                continue;
            if (in)
                s.insert(cand);
        }
        worst = s.worst();
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// One wavefront = the 64 queries of one cell; logical wavefront = cloud * qcells + cell.
// first: number of entries found by earlier rounds; count: entries this round finds (<= K).
template <int K>
__global__ __launch_bounds__(NG_SCAN_THREADS) void knn_grid_kernel(
    int n, int k, int first, int count, float limit, int qcells, int ccells, int clouds,
    const float4* __restrict__ sorted_query, const float4* __restrict__ sorted_support,
    const float4* __restrict__ boxes_support, float* __restrict__ dist2, int64_t* __restrict__ idx)
{
    __shared__ float4 stages[NG_SCAN_THREADS / TPK_WAVE][NG_CELL];
    extern __shared__ float lows_all[]; // [wavefronts][candidate cells, in whole groups of 64]

    const int lane = threadIdx.x & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TPK_WAVE);
    const int64_t task = static_cast<int64_t>(xcd_local_block(blockIdx.x, gridDim.x)) *
                             (NG_SCAN_THREADS / TPK_WAVE) + wave;
    if (task >= static_cast<int64_t>(qcells) * clouds)
        return; // (no workgroup barrier anywhere in this kernel)
    const int cloud = static_cast<int>(task / qcells);
    const int qcell = static_cast<int>(task - static_cast<int64_t>(cloud) * qcells);
    const float4* __restrict__ qpts = sorted_query + static_cast<int64_t>(cloud) * qcells * NG_CELL;
    const float4* __restrict__ cpts = sorted_support + static_cast<int64_t>(cloud) * ccells * NG_CELL;
    const float4* __restrict__ cbox = boxes_support + static_cast<int64_t>(cloud) * ccells * NG_BOX;
    dist2 += static_cast<int64_t>(cloud) * n * k;
    idx += static_cast<int64_t>(cloud) * n * k;
    float4* const stage = stages[wave];
    float* const lows = lows_all + wave * ((ccells + NG_CELL - 1) / NG_CELL * NG_CELL);

    const float4 query = qpts[qcell * NG_CELL + lane];
    const float qx = query.x, qy = query.y, qz = query.z;
    const int qindex = __float_as_int(query.w); // 0x7FFFFFFF: padding, nothing to store
    if (__ballot(qindex != 0x7FFFFFFF) == 0)
        return; // a cell without points (the last window of a cloud may have some)
    const bool real = qindex != 0x7FFFFFFF;
    float4 qlo, qhi;
    query_box(qx, qy, qz, real, qlo, qhi);

    NearestK<K> s;
    {
        // the last pair of the round before (rounds of one call run one after the other)
        const int64_t at = static_cast<int64_t>(real ? qindex : 0) * k + first - 1;
        const bool later = first > 0 && real;
        s.reset(first > 0, later ? dist2[at] : 0.f, later ? static_cast<int>(idx[at]) : 0, !real, limit);
    }

    const int groups = (ccells + NG_CELL - 1) / NG_CELL;
    unsigned seed_key = 0xFFFFFFFFu;
    for (int g = 0; g < groups; ++g)
    {
        const int c = g * NG_CELL + lane;
        const bool valid = c < ccells;
        const int cc = valid ? c : 0;
        const float4 clo = cbox[cc * NG_BOX + 0], chi = cbox[cc * NG_BOX + 1];
        const float lb = box_box_dist2(qlo, qhi, clo, chi);
        lows[c] = valid ? lb : __builtin_inff();
        // the first cell to scan: nearest box centre (the six lowest bits of the distance carry g)
        const float ex = (clo.x + chi.x) - (qlo.x + qhi.x), ey = (clo.y + chi.y) - (qlo.y + qhi.y);
        const float ez = (clo.z + chi.z) - (qlo.z + qhi.z);
        const float centre = __builtin_fmaf(ex, ex, __builtin_fmaf(ey, ey, ez * ez));
        const unsigned key = (static_cast<unsigned>(__float_as_int(centre)) & ~63u) | static_cast<unsigned>(g);
        seed_key = valid && lb < __builtin_inff() && key < seed_key ? key : seed_key;
    }
    {
        const unsigned lowest = wave_min_u32(seed_key);
        int seed = static_cast<int>(lowest & 63u) * NG_CELL + __builtin_ctzll(__ballot(seed_key == lowest));
        if (seed >= ccells)
            seed = 0;
        scan_cell_k<K>(cpts, cbox, seed, stage, lane, qx, qy, qz, s);
        if (lane == (seed & (NG_CELL - 1)))
            lows[seed] = __builtin_inff();
    }
    for (int phase = 0; phase < 2; ++phase)
        for (int g = 0; g < groups; ++g)
        {
            const float lw = lows[g * NG_CELL + lane];
            float bound = __int_as_float(wave_max_i32(__float_as_int(s.worst())));
            unsigned long long live =
                __ballot(lw < __builtin_inff() && (phase == 0 ? lw == 0.f : lw * NG_MARGIN <= bound));
            while (live != 0)
            {
                const int bit = __builtin_ctzll(live);
                const int c = g * NG_CELL + bit;
                live &= live - 1;
                const float lb = point_box_dist2(qx, qy, qz, cbox[c * NG_BOX + 0], cbox[c * NG_BOX + 1]);
                if (__ballot(lb * NG_MARGIN <= s.worst()) != 0)
                    scan_cell_k<K>(cpts, cbox, c, stage, lane, qx, qy, qz, s);
                if (lane == bit)
                    lows[c] = __builtin_inff(); // scanned, or useless now and ever after
                if (phase)
                {
                    bound = __int_as_float(wave_max_i32(__float_as_int(s.worst())));
                    live &= __ballot(lw * NG_MARGIN <= bound);
                }
            }
        }
    if (real)
    {
#pragma unroll
        for (int j = 0; j < K; ++j)
            if (j < count)
            {
                dist2[static_cast<int64_t>(qindex) * k + first + j] = s.dist(j);
                idx[static_cast<int64_t>(qindex) * k + first + j] = s.index(j);
            }
    }
}

constexpr int NG_RUN = 16; // consecutive cells that share a second-level box in the wavefront-per-query search

// ---------------------------------------------------------------------------------------
// Ball query over bins, packed layout (several clouds back to back, sorted cloud id per point).
//
// The support array is cut into windows of 8192 or 16384 (bqb_window_shift) consecutive rows, each ordered on its
// own (curve_cells_kernel), which groups a window's points by the cell of a 16^3 grid over the
// window's bounding box; the ordering kernel also leaves where each such bin ends.  One
// wavefront serves one query: it reads which support rows belong to the query's cloud (found for
// every query by workgroups that ride along with the ordering launch), and so the windows they
// lie in, and finds in every window the bins that the cube around the ball touches - a handful
// when the radius is small against the cloud - and tests their points, 64 per step, one per
// lane.  A candidate is a hit when its squared distance is <= radius^2 and its row lies in the
// query's cloud.  The hits (at most 64) are collected in LDS, ranked by row, and written in
// ascending row order, then -1: the rows a serial scan in index order that stops after nsample
// hits (cuda/src/ball_query_gpu.cu:54-95) would have produced.
// The (window, bin) pairs of a query are walked 64 at a time.  A query whose ball touches more
// than 64 bins of one window or 512 in all, or that has more than 64 hits, is answered by that
// serial scan itself, 64 rows per step with early exit: those are the dense
// neighbourhoods, where the scan ends soon.
// ---------------------------------------------------------------------------------------
// Rows per window of the packed ball query, as a shift.  Windows of 8192 rows are ordered faster and by twice as
// many workgroups (config 4: 15 windows of 16384 rows leave most of the chip idle while they are ordered: 61 ->
// 57 us with 8192, 58 with 4096); a lane per window limits a cloud to 64 windows, so arrays above 64 x 8192 rows
// keep windows of 16384.
constexpr int BQB_SMALL_SHIFT = 13;
inline int bqb_window_shift(int64_t size_x)
{
    return size_x <= (static_cast<int64_t>(TPK_WAVE) << BQB_SMALL_SHIFT) ? BQB_SMALL_SHIFT : 14;
}
static_assert((1 << 14) == CURVE_MAX_POINTS, "the larger window is what the ordering kernel holds at most");
constexpr int BQB_HITS = TPK_WAVE; // hits a wavefront collects before it falls back to the scan
constexpr int BQB_DENSE_MIN_POINTS = 8192; // dense layout: clouds above this take the bin walk (smaller ones fit in LDS whole)
constexpr int64_t BQB_DENSE_MIN_PAIRS = 40000000; // ... when the call has at least this many (query, point) pairs

// Range of 16^3-grid cells along one axis that [v - r, v + r] can touch.  The interval is widened
// by a few ulps of its ends so that a point the fp32 radius test accepts is never left out.
__device__ __forceinline__ void bin_range(float v, float r, float lo, float scale, int& first, int& last)
{
    const float slack = (fabsf(v) + r) * 1e-6f + 1e-30f;
    first = static_cast<int>(curve_grid_cell((v - r) - slack, lo, scale) >> 2);
    last = static_cast<int>(curve_grid_cell((v + r) + slack, lo, scale) >> 2);
}

// SORTED: the nsample (<= 64) NEAREST points with squared distance < radius2, nearest first, instead of the
// first nsample in row order with squared distance <= radius2: the wavefront keeps its 64 best (distance, row)
// keys sorted across the lanes and merges the hits of a step into them (as the wavefront-per-query kernel
// further down does with the points of a cell).
// DENSE (unsorted only): the dense layout's rules instead (cuda/src/ball_query_gpu.cu:9-52) - clouds of dense_n
// consecutive rows with dense_m consecutive queries each (no cloud_rows), a hit has squared distance < radius2
// (strict), indices count from the cloud's first row, and the slots behind the last hit repeat the first hit
// (0 without any) with distance -1.
template <bool SORTED, bool DENSE>
__global__ __launch_bounds__(NG_SCAN_THREADS) void ball_query_bins_kernel(
    int size_x, int size_y, int window_shift, float radius, float radius2, int nsample, const float* __restrict__ x,
    const float* __restrict__ y, const float4* __restrict__ sorted_x, const int* __restrict__ bin_ends,
    const float4* __restrict__ grids, const int2* __restrict__ cloud_rows, int64_t* __restrict__ idx,
    float* __restrict__ dist, int dense_n, int dense_m)
{
    static_assert(!(SORTED && DENSE), "the sorted query of the dense layout has a kernel of its own");
    constexpr int WAVES = NG_SCAN_THREADS / TPK_WAVE;
    __shared__ int hit_rows[WAVES][BQB_HITS];
    __shared__ float hit_dists[WAVES][BQB_HITS];
    __shared__ int slot_rows[WAVES][TPK_WAVE]; // pair descriptors, then candidate addresses

    const int lane = threadIdx.x & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TPK_WAVE);
    const int64_t q = static_cast<int64_t>(blockIdx.x) * WAVES + wave;
    if (q >= size_y)
        return; // (no workgroup barrier anywhere in this kernel)
    int* const rows = hit_rows[wave];
    float* const dists = hit_dists[wave];
    int* const slots = slot_rows[wave];

    const float ux = y[q * 3 + 0], uy = y[q * 3 + 1], uz = y[q * 3 + 2];
    const float qx = to_vector_register(ux), qy = to_vector_register(uy), qz = to_vector_register(uz);
    int s0, s1; // the support rows of the query's cloud
    if constexpr (DENSE)
    {
        s0 = static_cast<int>(q / dense_m) * dense_n;
        s1 = s0 + dense_n;
    }
    else
    {
        const int2 cloud = cloud_rows[q];
        s0 = cloud.x;
        s1 = cloud.y;
    }
    const int64_t out = q * nsample;
    TPK_WORK_DECL

    // The walk is laid out so that dependent loads are few: all windows at once (one lane each),
    // then all (window, bin) pairs at once, then the candidates 64 at a time.
    int cnt = 0;
    // SORTED: lane i holds the i-th smallest (distance, row) key so far; a hit must beat the nsample-th
    constexpr u64 NONE = ~0ull;
    u64 best = NONE, admit = NONE;
    auto offer = [&](bool hit, float d, int row) __attribute__((always_inline)) {
        u64 cand = hit ? knn_key(d, row) : NONE;
        cand = cand < admit ? cand : NONE;
        if (__ballot(cand != NONE) == 0)
            return;
        cand = wave_sort_keys(cand, lane, true);
        best = wave_merge_ascending(best < cand ? best : cand, lane);
        admit = read_lane_key(best, nsample - 1);
    };
    const int wx0 = s0 >> window_shift;
    const int windows = s1 > s0 ? ((s1 - 1) >> window_shift) - wx0 + 1 : 0;
    bool serial = windows > TPK_WAVE; // answer by the scan in index order instead
    if (!serial && windows > 0)
    {
        // lane w: the block of bins that the ball's cube touches in window wx0 + w
        int nbins = 0, block = 0;
        if (lane < windows)
        {
            const float4 origin = grids[(wx0 + lane) * 2 + 0], scale = grids[(wx0 + lane) * 2 + 1];
            int fx, lx, fy, ly, fz, lz;
            bin_range(ux, radius, origin.x, scale.x, fx, lx);
            bin_range(uy, radius, origin.y, scale.y, fy, ly);
            bin_range(uz, radius, origin.z, scale.z, fz, lz);
            const int nx = lx - fx + 1, ny = ly - fy + 1;
            nbins = nx * ny * (lz - fz + 1);
            block = fx | (fy << 4) | (fz << 8) | ((nx - 1) << 12) | ((ny - 1) << 16) | (lane << 26);
        }
        const int pairs_before = wave_exclusive_sum(nbins);
        const int pairs = __builtin_amdgcn_readlane(pairs_before + nbins, TPK_WAVE - 1);
        // (a ball that touches more than 64 bins of one window, or 512 in all, covers so much of
        // its cloud that the scan in index order ends early)
        serial = __ballot(nbins > TPK_WAVE) != 0 || pairs > 8 * TPK_WAVE;
        // 64 (window, bin) pairs at a time; nearly always there are no more than that
        auto walk_pairs = [&](int pair0) __attribute__((always_inline)) {
            // one descriptor per pair, written by the window's lane: a window's block holds a few bins, so a loop
            // is cheaper here than the marks used for the candidates below (64.6 against 62 us on 58750 queries)
            // (volatile: what a lane reads back was written by other lanes)
            volatile int* const marks = slots;
            for (int i = max(0, pair0 - pairs_before); i < nbins && pairs_before + i < pair0 + TPK_WAVE; ++i)
                marks[pairs_before + i - pair0] = block | (i << 20);
            // lane p: where the points of pair pair0 + p start in the ordered array, and how many
            int start = 0, size = 0;
            if (pair0 + lane < pairs)
            {
                const int d = marks[lane];
                const int i = (d >> 20) & 63, window = (d >> 26) & 63;
                const int fx = d & 15, fy = (d >> 4) & 15, fz = (d >> 8) & 15;
                const int nx = ((d >> 12) & 15) + 1, ny = ((d >> 16) & 15) + 1;
                const int wx = wx0 + window;
                // (the table of the ordering kernel: 8 KiB that every wavefront reads, at home in the caches)
                // (i = ix + nx * (iy + ny * iz), taken apart by float division: exact for these small numbers)
                const int iz = static_cast<int>((static_cast<float>(i) + 0.5f) * __builtin_amdgcn_rcpf(static_cast<float>(nx * ny)));
                const int in_plane = i - iz * nx * ny;
                const int iy = static_cast<int>((static_cast<float>(in_plane) + 0.5f) * __builtin_amdgcn_rcpf(static_cast<float>(nx)));
                const int ix = in_plane - iy * nx;
                const unsigned bin = curve_bin_table.bin[(fx + ix) | ((fy + iy) << 4) | ((fz + iz) << 8)];
                const int* __restrict__ ends = bin_ends + static_cast<int64_t>(wx) * CURVE_BINS;
                start = bin ? ends[bin - 1] : 0;
                size = ends[bin] - start;
                start += wx << window_shift;
            }
            const int before = wave_exclusive_sum(size);
            const int total = __builtin_amdgcn_readlane(before + size, TPK_WAVE - 1);
            const int origin = start - before; // candidate c of this walk lies at origin + c, for the c of this lane's pair
            for (int c0 = 0; c0 < total && !serial; c0 += TPK_WAVE)
            {
                // Which pair does candidate c0 + lane belong to?  Every pair's lane marks the slot of its first
                // candidate in this step with its own number; a running maximum over the slots carries the
                // number on to the pair's other candidates.
                marks[lane] = 0;
                if (size > 0 && before < c0 + TPK_WAVE && before + size > c0)
                    marks[max(before - c0, 0)] = lane;
                const int mark = marks[lane];
                const bool has = c0 + lane < total;
                const int at_x = __shfl(origin, wave_inclusive_max_i32(mark)) + c0 + lane;
                const float4 p = sorted_x[has ? at_x : 0];
                const float d = tpk_dist2(qx, qy, qz, p.x, p.y, p.z);
                TPK_WORK_ADD(1);
                const int row = __float_as_int(p.w);
                if constexpr (SORTED)
                {
                    offer(has && d < radius2 && row >= s0 && row < s1, d, row);
                    continue;
                }
                const bool hit = has && (DENSE ? d < radius2 : d <= radius2) && row >= s0 && row < s1;
                const unsigned long long mask = __ballot(hit);
                if (mask == 0)
                    continue;
                const int at = cnt + static_cast<int>(tpk_prefix_count(mask));
                if (hit && at < BQB_HITS)
                {
                    rows[at] = row;
                    dists[at] = d;
                }
                cnt += __builtin_popcountll(mask);
                serial = cnt > BQB_HITS;
            }
        };
        if (!serial)
            walk_pairs(0);
        for (int pair0 = TPK_WAVE; pair0 < pairs && !serial; pair0 += TPK_WAVE)
            walk_pairs(pair0);
    }

    if constexpr (SORTED)
    {
        if (serial)
        {
            // too many windows or bins for the walk: every row of the cloud, 64 per step
            constexpr int BATCH = 4;
            for (int base = s0; base < s1; base += BATCH * TPK_WAVE)
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
                    TPK_WORK_ADD(1);
                    offer(pos < s1 && d < radius2, d, pos);
                }
            }
        }
        if (lane < nsample)
        {
            const bool found = best != NONE;
            idx[out + lane] = found ? static_cast<int64_t>(best & 0xFFFFFFFFu) : -1;
            dist[out + lane] = found ? __int_as_float(static_cast<int>(best >> 32)) : -1.0f;
        }
        TPK_WORK_FLUSH
        return;
    }
    if (!serial)
    {
        // rank of every hit among the hits (rows are distinct), then hits in order, then -1
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        const int my_row = rows[lane < cnt ? lane : 0];
        const float my_dist = dists[lane < cnt ? lane : 0];
        int rank = 0;
        for (int j = 0; j < cnt; ++j)
            rank += rows[j] < my_row ? 1 : 0;
        if (lane < cnt && rank < nsample)
        {
            idx[out + rank] = DENSE ? my_row - s0 : my_row;
            dist[out + rank] = my_dist;
        }
        int64_t filler = -1;
        if constexpr (DENSE)
        {
            // the first hit of the scan in index order = the lowest row among the hits
            const unsigned long long lowest = __ballot(lane < cnt && rank == 0);
            filler = lowest ? __shfl(my_row, __builtin_ctzll(lowest)) - s0 : 0;
        }
        for (int s = cnt + lane; s < nsample; s += TPK_WAVE)
        {
            idx[out + s] = filler;
            dist[out + s] = -1.0f;
        }
        TPK_WORK_FLUSH
        return;
    }

    // Serial semantics directly: lanes hold 64 consecutive support rows; ballot + prefix count
    // give the hits their slots in index order; stop after nsample hits.
    cnt = 0;
    int first_hit = -1; // (dense layout: the row that fills the slots behind the last hit)
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
            TPK_WORK_ADD(1);
            const bool hit = pos < s1 && (DENSE ? d < radius2 : d <= radius2);
            const unsigned long long mask = __ballot(hit);
            const int slot = cnt + static_cast<int>(tpk_prefix_count(mask));
            if (hit && slot < nsample)
            {
                idx[out + slot] = DENSE ? pos - s0 : pos;
                dist[out + slot] = d;
            }
            if (DENSE && first_hit < 0 && mask != 0)
                first_hit = base + u * TPK_WAVE + __builtin_ctzll(mask) - s0;
            cnt += __builtin_popcountll(mask);
        }
    }
    for (int s = cnt + lane; s < nsample; s += TPK_WAVE)
    {
        idx[out + s] = DENSE ? max(first_hit, 0) : -1;
        dist[out + s] = -1.0f;
    }
    TPK_WORK_FLUSH
}

struct GridLayout
{
    size_t sorted_a, sorted_b, boxes_a, boxes_b, wide_a, wide_b, total;
};

// Cells of a cloud of n points: ordered whole up to NG_WINDOW points, else in windows of NG_WINDOW
// consecutive points (the last one padded with cells that hold nothing).
int grid_cells(int n)
{
    return n <= NG_WINDOW ? (n + NG_CELL - 1) / NG_CELL
                          : static_cast<int>(tpk_ceil_div(n, NG_WINDOW)) * (NG_WINDOW / NG_CELL);
}
int grid_stride(int n)
{
    return n <= NG_WINDOW ? n : NG_WINDOW;
}

GridLayout grid_layout(int b, int n, int m, bool wide_first = false)
{
    auto up = [](size_t v) { return (v + 255) & ~static_cast<size_t>(255); };
    const size_t cells_a = static_cast<size_t>(grid_cells(n));
    const size_t cells_b = static_cast<size_t>(grid_cells(m));
    GridLayout l;
    size_t pos = 0;
    l.sorted_a = pos;
    pos = up(pos + static_cast<size_t>(b) * cells_a * NG_CELL * sizeof(float4));
    l.sorted_b = pos;
    pos = up(pos + static_cast<size_t>(b) * cells_b * NG_CELL * sizeof(float4));
    l.boxes_a = pos;
    pos = up(pos + static_cast<size_t>(b) * cells_a * NG_BOX * sizeof(float4));
    l.boxes_b = pos;
    pos = up(pos + static_cast<size_t>(b) * cells_b * NG_BOX * sizeof(float4));
    l.wide_a = l.wide_b = pos;
    if (wide_first) // (the Chamfer search: the cells of every window, wide ones first)
    {
        pos = up(pos + static_cast<size_t>(b) * cells_a * sizeof(int));
        l.wide_b = pos;
        pos = up(pos + static_cast<size_t>(b) * cells_b * sizeof(int));
    }
    l.total = pos;
    return l;
}

bool grid_supported(int b, int n, int m)
{
    // Small clouds are served as fast by the all-pairs scan; the box distances of very large ones
    // do not fit in LDS.
    return b > 0 && n >= 512 && m >= 512 && grid_cells(n) <= NG_MAX_CELLS && grid_cells(m) <= NG_MAX_CELLS;
}

} // namespace

size_t tpk_grid_chamfer_workspace_bytes(int b, int n, int m)
{
    return grid_supported(b, n, m) ? grid_layout(b, n, m, true).total : 0;
}

int tpk_grid_chamfer_fwd(int b, int n, int m, const float* xyz1, const float* xyz2, float* dist1,
                         float* dist2, int32_t* idx1, int32_t* idx2, void* workspace,
                         size_t workspace_bytes, hipStream_t s)
{
    if (!grid_supported(b, n, m) || static_cast<int64_t>(b) * 2 > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const GridLayout l = grid_layout(b, n, m, true);
    if (!workspace || workspace_bytes < l.total || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return TPK_ERR_WORKSPACE;
    char* w = static_cast<char*>(workspace);
    PointSet a{xyz1, nullptr, static_cast<int64_t>(b) * n, n, grid_stride(n), reinterpret_cast<float4*>(w + l.sorted_a),
               reinterpret_cast<float4*>(w + l.boxes_a), nullptr, nullptr, nullptr};
    PointSet c{xyz2, nullptr, static_cast<int64_t>(b) * m, m, grid_stride(m), reinterpret_cast<float4*>(w + l.sorted_b),
               reinterpret_cast<float4*>(w + l.boxes_b), nullptr, nullptr, nullptr};
    // Both clouds' windows hold the same number of cells (clouds of one size class, the usual case): the cells
    // are handed to the wavefronts wide ones first.
    const int window_cells = set_cells(a) == set_cells(c) ? set_cells(a) : 0;
    if (window_cells > 0)
    {
        a.wide_first = reinterpret_cast<int*>(w + l.wide_a);
        c.wide_first = reinterpret_cast<int*>(w + l.wide_b);
    }
    int st = launch_curve_cells(a, c, nullptr, s);
    if (st != TPK_OK)
        return st;
    const int cells1 = grid_cells(n), cells2 = grid_cells(m);
    const int64_t waves = static_cast<int64_t>(cells1 + cells2) * b;
    const int64_t blocks = tpk_ceil_div(waves, NG_SCAN_THREADS / TPK_WAVE);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const size_t lds = static_cast<size_t>(NG_SCAN_THREADS / TPK_WAVE) *
                       ((std::max(cells1, cells2) + NG_CELL - 1) / NG_CELL * NG_CELL) * sizeof(float);
    hipLaunchKernelGGL(chamfer_grid_kernel, dim3(static_cast<unsigned>(blocks)), dim3(NG_SCAN_THREADS), lds, s, n,
                       m, cells1, cells2, b, a.sorted, c.sorted, a.boxes, c.boxes, dist1, dist2, idx1, idx2, a.wide_first,
                       c.wide_first, window_cells);
    return tpk_launch_status();
}

// (behind the ordered copies and boxes: one word per cloud, see tpk_grid_three_nn_flags)
size_t tpk_grid_three_nn_workspace_bytes(int b, int n, int m)
{
    return grid_supported(b, n, m) ? grid_layout(b, n, m).total + ((static_cast<size_t>(b) * sizeof(int) + 255) & ~static_cast<size_t>(255)) : 0;
}

int* tpk_grid_three_nn_flags(int b, int n, int m, void* workspace, size_t workspace_bytes)
{
    const size_t need = tpk_grid_three_nn_workspace_bytes(b, n, m);
    if (!need || !workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return nullptr;
    return reinterpret_cast<int*>(static_cast<char*>(workspace) + grid_layout(b, n, m).total);
}

int tpk_grid_three_nn(int b, int n, int m, const float* unknown, const float* known, float* dist2,
                      int32_t* idx, void* workspace, size_t workspace_bytes, bool flagged, hipStream_t s)
{
    if (!grid_supported(b, n, m) || static_cast<int64_t>(b) * 2 > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const GridLayout l = grid_layout(b, n, m);
    if (!workspace || workspace_bytes < tpk_grid_three_nn_workspace_bytes(b, n, m) || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return TPK_ERR_WORKSPACE;
    char* w = static_cast<char*>(workspace);
    const int* only = flagged ? reinterpret_cast<const int*>(w + l.total) : nullptr;
    // (the unknown points are only queried: no boxes of their cells - the search forms the box of its 64 queries)
    PointSet a{unknown, nullptr, static_cast<int64_t>(b) * n, n, grid_stride(n), reinterpret_cast<float4*>(w + l.sorted_a),
               nullptr, nullptr, nullptr, nullptr, only};
    PointSet c{known, nullptr, static_cast<int64_t>(b) * m, m, grid_stride(m), reinterpret_cast<float4*>(w + l.sorted_b),
               reinterpret_cast<float4*>(w + l.boxes_b), nullptr, nullptr, nullptr, only};
    int st = launch_curve_cells(a, c, nullptr, s);
    if (st != TPK_OK)
        return st;
    const int qcells = grid_cells(n), ccells = grid_cells(m);
    const int64_t waves = static_cast<int64_t>(qcells) * b;
    const int64_t blocks = tpk_ceil_div(waves, NG_SCAN_THREADS / TPK_WAVE);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const size_t lds = static_cast<size_t>(NG_SCAN_THREADS / TPK_WAVE) * ((ccells + NG_CELL - 1) / NG_CELL * NG_CELL) *
                       sizeof(float);
    hipLaunchKernelGGL(three_nn_grid_kernel, dim3(static_cast<unsigned>(blocks)), dim3(NG_SCAN_THREADS), lds, s, n,
                       m, qcells, ccells, b, a.sorted, c.sorted, c.boxes, dist2, idx, only);
    return tpk_launch_status();
}

namespace {

// Ball query with sorted neighbours, one wavefront per query: the nsample (<= 64) nearest support
// points with squared distance < limit.  The support points lie in curve-ordered cells of 64; a
// cell whose box is out of reach is skipped; the others are tested one point per lane.  The
// wavefront keeps its 64 best (distance, index) keys sorted across the lanes: the candidates of a
// cell that beat the current nsample-th key are sorted the other way round and merged in (minimum
// per lane, then one bitonic merge).  Dense neighbourhoods - hundreds of points inside the radius -
// cost a few such merges, not an insertion per point.
// Unused slots: packed layout -1 / -1; dense layout the nearest neighbour's index (0 without any)
// and -1.  Indices are raised by index_add.
__global__ __launch_bounds__(NG_SCAN_THREADS) void ball_sorted_wave_kernel(
    int64_t queries, int n, int ccells, int nsample, float limit, bool packed, int64_t index_add,
    const float* __restrict__ query, const float4* __restrict__ sorted_support,
    const float4* __restrict__ boxes_support, const float4* __restrict__ run_boxes, float* __restrict__ dist,
    int64_t* __restrict__ idx)
{
    const int lane = threadIdx.x & (TPK_WAVE - 1);
    const int64_t q = static_cast<int64_t>(blockIdx.x) * (NG_SCAN_THREADS / TPK_WAVE) + threadIdx.x / TPK_WAVE;
    if (q >= queries)
        return; // (no workgroup barrier anywhere in this kernel)
    const int64_t cloud = q / n;
    const float4* __restrict__ cpts = sorted_support + cloud * ccells * NG_CELL;
    const float4* __restrict__ cbox = boxes_support + cloud * ccells * NG_BOX;
    const float qx = query[q * 3 + 0], qy = query[q * 3 + 1], qz = query[q * 3 + 2];

    constexpr u64 NONE = ~0ull;
    u64 best = NONE;      // lane i: the i-th smallest key so far
    u64 admit = NONE;     // the nsample-th smallest: a candidate must beat it
    float reach = limit;  // squared distance beyond which a cell cannot help
    // One cell offered to the list, one point per lane.
    auto offer = [&](int cell) __attribute__((always_inline)) {
        const float4 p = cpts[static_cast<int64_t>(cell) * NG_CELL + lane];
        const float d = tpk_dist2(qx, qy, qz, p.x, p.y, p.z);
        u64 cand = d < limit ? knn_key(d, __float_as_int(p.w)) : NONE;
        cand = cand < admit ? cand : NONE;
        if (__ballot(cand != NONE) == 0)
            return;
        cand = wave_sort_keys(cand, lane, true);
        best = wave_merge_ascending(best < cand ? best : cand, lane);
        admit = read_lane_key(best, nsample - 1);
        if (admit != NONE)
            reach = __int_as_float(static_cast<int>(admit >> 32));
    };
    if (run_boxes == nullptr)
    {
        // few cells: the box of every cell is tested, one cell per lane
        for (int first = 0; first < ccells; first += NG_CELL)
        {
            const int c = first + lane;
            const bool valid = c < ccells;
            const int cc = valid ? c : 0;
            const float lb = point_box_dist2(qx, qy, qz, cbox[cc * NG_BOX + 0], cbox[cc * NG_BOX + 1]);
            u64 live = __ballot(valid && lb * NG_MARGIN <= reach);
            while (live != 0)
            {
                const int bit = __builtin_ctzll(live);
                live &= live - 1;
                if (tpk_read_lane(lb, bit) * NG_MARGIN <= reach) // (the list may have filled up with nearer points)
                    offer(first + bit);
            }
        }
    }
    else
    {
        // Two levels: the boxes of runs of 16 consecutive cells (neighbours on the curve, so compact), one run
        // per lane; then the cells of up to four runs in reach, one cell per lane.
        const int runs = (ccells + NG_RUN - 1) / NG_RUN;
        const float4* __restrict__ rbox = run_boxes + cloud * runs * 2;
        for (int first_run = 0; first_run < runs; first_run += NG_CELL)
        {
            const int r = first_run + lane;
            const int rr = r < runs ? r : 0;
            const float run_lb = point_box_dist2(qx, qy, qz, rbox[rr * 2 + 0], rbox[rr * 2 + 1]);
            u64 live_runs = __ballot(r < runs && run_lb * NG_MARGIN <= reach);
            while (live_runs != 0)
            {
                // the next four runs in reach: lanes 16 j .. 16 j + 15 take the cells of the j-th
                int mine = -1;
#pragma unroll
                for (int j = 0; j < TPK_WAVE / NG_RUN; ++j)
                {
                    const int bit = live_runs != 0 ? __builtin_ctzll(live_runs) : -1;
                    live_runs &= live_runs - 1; // (0 stays 0)
                    mine = (lane / NG_RUN) == j ? bit : mine;
                }
                const int c = mine < 0 ? ccells : (first_run + mine) * NG_RUN + (lane % NG_RUN);
                const bool valid = c < ccells;
                const int cc = valid ? c : 0;
                const float lb = point_box_dist2(qx, qy, qz, cbox[cc * NG_BOX + 0], cbox[cc * NG_BOX + 1]);
                u64 live = __ballot(valid && lb * NG_MARGIN <= reach);
                while (live != 0)
                {
                    const int bit = __builtin_ctzll(live);
                    live &= live - 1;
                    if (tpk_read_lane(lb, bit) * NG_MARGIN > reach)
                        continue; // the list has filled up with nearer points meanwhile
                    offer(__builtin_amdgcn_readlane(c, bit));
                }
            }
        }
    }
    if (lane < nsample)
    {
        const u64 nearest = read_lane_key(best, 0);
        const bool found = best != NONE;
        const int64_t o = q * nsample + lane;
        const int64_t pad = packed ? -1 : (nearest != NONE ? static_cast<int64_t>(nearest & 0xFFFFFFFFu) + index_add : 0);
        idx[o] = found ? static_cast<int64_t>(best & 0xFFFFFFFFu) + index_add : pad;
        dist[o] = found ? __int_as_float(static_cast<int>(best >> 32)) : -1.0f;
    }
}

// Box of every run of NG_RUN consecutive cells of a cloud: (lo, hi) as two float4.
__global__ __launch_bounds__(NG_SCAN_THREADS) void run_boxes_kernel(int64_t total_runs, int runs, int ccells,
                                                                    const float4* __restrict__ boxes,
                                                                    float4* __restrict__ run_boxes)
{
    const int64_t t = static_cast<int64_t>(blockIdx.x) * NG_SCAN_THREADS + threadIdx.x;
    if (t >= total_runs)
        return;
    const int64_t cloud = t / runs;
    const int r = static_cast<int>(t - cloud * runs);
    const float4* __restrict__ cbox = boxes + cloud * ccells * NG_BOX;
    const float inf = __builtin_inff();
    float4 lo = make_float4(inf, inf, inf, 0.f), hi = make_float4(-inf, -inf, -inf, 0.f);
    for (int c = r * NG_RUN; c < ccells && c < (r + 1) * NG_RUN; ++c)
    {
        const float4 a = cbox[c * NG_BOX + 0], b = cbox[c * NG_BOX + 1]; // (an empty cell: lo = +inf, hi = -inf)
        lo = make_float4(fminf(lo.x, a.x), fminf(lo.y, a.y), fminf(lo.z, a.z), 0.f);
        hi = make_float4(fmaxf(hi.x, b.x), fmaxf(hi.y, b.y), fmaxf(hi.z, b.z), 0.f);
    }
    run_boxes[t * 2 + 0] = lo;
    run_boxes[t * 2 + 1] = hi;
}

struct SupportLayout
{
    size_t sorted, boxes, runs, total;
};

SupportLayout support_layout(int b, int m)
{
    auto up = [](size_t v) { return (v + 255) & ~static_cast<size_t>(255); };
    const size_t cells = static_cast<size_t>(grid_cells(m));
    SupportLayout l;
    l.sorted = 0;
    l.boxes = up(static_cast<size_t>(b) * cells * NG_CELL * sizeof(float4));
    l.runs = l.boxes + up(static_cast<size_t>(b) * cells * NG_BOX * sizeof(float4));
    l.total = l.runs + up(static_cast<size_t>(b) * ((cells + NG_RUN - 1) / NG_RUN) * 2 * sizeof(float4));
    return l;
}

// Worth ordering the support points from this many on; below, all pairs are as fast.
bool ball_sorted_supported(int b, int m, int nsample)
{
    return b > 0 && m >= 512 && nsample >= 1 && nsample <= TPK_WAVE;
}

} // namespace

size_t tpk_grid_ball_sorted_workspace_bytes(int b, int m)
{
    return ball_sorted_supported(b, m, 1) ? support_layout(b, m).total : 0;
}

// n queries and m support points per cloud; outputs complete (padding included).
int tpk_grid_ball_sorted(int b, int n, int m, int nsample, float limit, bool packed, int64_t index_add,
                         const float* query, const float* support, float* dist, int64_t* idx, void* workspace,
                         size_t workspace_bytes, hipStream_t s)
{
    if (!ball_sorted_supported(b, m, nsample) || n < 1 || !(limit < __builtin_inff()))
        return TPK_ERR_UNSUPPORTED;
    const SupportLayout l = support_layout(b, m);
    if (!workspace || workspace_bytes < l.total || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return TPK_ERR_WORKSPACE;
    char* w = static_cast<char*>(workspace);
    PointSet none{nullptr, nullptr, 0, 1, 0, nullptr, nullptr, nullptr, nullptr};
    PointSet c{support, nullptr, static_cast<int64_t>(b) * m, m, grid_stride(m), reinterpret_cast<float4*>(w + l.sorted),
               reinterpret_cast<float4*>(w + l.boxes), nullptr, nullptr};
    int st = launch_curve_cells(none, c, nullptr, s);
    if (st != TPK_OK)
        return st;
    const int ccells = grid_cells(m), runs = (ccells + NG_RUN - 1) / NG_RUN;
    // second-level boxes pay from a few groups of 64 cells on
    float4* run_boxes = ccells > 4 * NG_CELL ? reinterpret_cast<float4*>(w + l.runs) : nullptr;
    if (run_boxes)
    {
        const int64_t total_runs = static_cast<int64_t>(b) * runs;
        hipLaunchKernelGGL(run_boxes_kernel, dim3(static_cast<unsigned>(tpk_ceil_div(total_runs, NG_SCAN_THREADS))),
                           dim3(NG_SCAN_THREADS), 0, s, total_runs, runs, ccells, c.boxes, run_boxes);
        st = tpk_launch_status();
        if (st != TPK_OK)
            return st;
    }
    const int64_t queries = static_cast<int64_t>(b) * n;
    const int64_t blocks = tpk_ceil_div(queries, NG_SCAN_THREADS / TPK_WAVE);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(ball_sorted_wave_kernel, dim3(static_cast<unsigned>(blocks)), dim3(NG_SCAN_THREADS), 0, s, queries,
                       n, ccells, nsample, limit, packed, index_add, query, c.sorted, c.boxes, run_boxes, dist, idx);
    return tpk_launch_status();
}

size_t tpk_grid_knn_workspace_bytes(int b, int n, int m)
{
    return grid_supported(b, n, m) ? grid_layout(b, n, m).total : 0;
}

namespace {

template <int K>
int launch_knn_grid(int b, int n, int k, float limit, int qcells, int ccells, const PointSet& a, const PointSet& c,
                    float* dist2, int64_t* idx, hipStream_t s)
{
    const int64_t waves = static_cast<int64_t>(qcells) * b;
    const int64_t blocks = tpk_ceil_div(waves, NG_SCAN_THREADS / TPK_WAVE);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const size_t lds = static_cast<size_t>(NG_SCAN_THREADS / TPK_WAVE) * ((ccells + NG_CELL - 1) / NG_CELL * NG_CELL) *
                       sizeof(float);
    for (int first = 0; first < k; first += K)
    {
        hipLaunchKernelGGL(knn_grid_kernel<K>, dim3(static_cast<unsigned>(blocks)), dim3(NG_SCAN_THREADS), lds, s, n,
                           k, first, k - first < K ? k - first : K, limit, qcells, ccells, b, a.sorted, c.sorted, c.boxes,
                           dist2, idx);
        const int st = tpk_launch_status();
        if (st != TPK_OK)
            return st;
    }
    return TPK_OK;
}

} // namespace

// n queries and m support points per cloud.
int tpk_grid_knn(int b, int n, int m, int k, float limit, const float* query, const float* support, float* dist2,
                 int64_t* idx, void* workspace, size_t workspace_bytes, hipStream_t s)
{
    if (!grid_supported(b, n, m) || static_cast<int64_t>(b) * 2 > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const GridLayout l = grid_layout(b, n, m);
    if (!workspace || workspace_bytes < l.total || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return TPK_ERR_WORKSPACE;
    char* w = static_cast<char*>(workspace);
    PointSet a{query, nullptr, static_cast<int64_t>(b) * n, n, grid_stride(n), reinterpret_cast<float4*>(w + l.sorted_a),
               nullptr, nullptr, nullptr};
    PointSet c{support, nullptr, static_cast<int64_t>(b) * m, m, grid_stride(m), reinterpret_cast<float4*>(w + l.sorted_b),
               reinterpret_cast<float4*>(w + l.boxes_b), nullptr, nullptr};
    int st = launch_curve_cells(a, c, nullptr, s);
    if (st != TPK_OK)
        return st;
    const int qcells = grid_cells(n), ccells = grid_cells(m);
    if (k <= 4)
        return launch_knn_grid<4>(b, n, k, limit, qcells, ccells, a, c, dist2, idx, s);
    if (k <= 8)
        return launch_knn_grid<8>(b, n, k, limit, qcells, ccells, a, c, dist2, idx, s);
    if (k <= 16)
        return launch_knn_grid<16>(b, n, k, limit, qcells, ccells, a, c, dist2, idx, s);
    return launch_knn_grid<KNN_MAX_K>(b, n, k, limit, qcells, ccells, a, c, dist2, idx, s);
}

namespace {

struct BallLayout
{
    size_t sorted_x, bin_ends, grids, cloud_rows, total;
};

BallLayout ball_layout(int64_t size_x, int64_t size_y)
{
    auto up = [](size_t v) { return (v + 255) & ~static_cast<size_t>(255); };
    const size_t window = static_cast<size_t>(1) << bqb_window_shift(size_x);
    const size_t wx = (static_cast<size_t>(size_x) + window - 1) / window;
    BallLayout l;
    size_t pos = 0;
    l.sorted_x = pos;
    pos = up(pos + wx * window * sizeof(float4));
    l.bin_ends = pos;
    pos = up(pos + wx * CURVE_BINS * sizeof(int));
    l.grids = pos;
    pos = up(pos + wx * 2 * sizeof(float4));
    l.cloud_rows = pos;
    pos = up(pos + static_cast<size_t>(size_y) * sizeof(int2));
    l.total = pos;
    return l;
}

bool ball_bins_supported(int64_t size_x, int64_t size_y, int nsample)
{
    // Small problems are served as fast by the all-pairs scan; rows are 32-bit here.
    return size_x >= 8192 && size_y > 0 && nsample > 0 && size_x < (1LL << 30);
}

} // namespace

size_t tpk_grid_ball_query_workspace_bytes(int64_t size_x, int64_t size_y, int nsample)
{
    return ball_bins_supported(size_x, size_y, nsample) ? ball_layout(size_x, size_y).total : 0;
}

int tpk_grid_ball_query_partial(int64_t size_x, int64_t size_y, float radius, float radius2, int nsample, bool sorted,
                                const float* x, const float* y, const int64_t* batch_x,
                                const int64_t* batch_y, int64_t* idx, float* dist, void* workspace,
                                size_t workspace_bytes, hipStream_t s)
{
    if (!ball_bins_supported(size_x, size_y, nsample) || (sorted && nsample > TPK_WAVE))
        return TPK_ERR_UNSUPPORTED;
    const BallLayout l = ball_layout(size_x, size_y);
    if (!workspace || workspace_bytes < l.total || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return TPK_ERR_WORKSPACE;
    char* w = static_cast<char*>(workspace);
    // (cloud ids are not used for the order: bins may mix the clouds of a window, rows tell them apart)
    const int window_shift = bqb_window_shift(size_x);
    PointSet px{x, nullptr, size_x, size_x, 1 << window_shift, reinterpret_cast<float4*>(w + l.sorted_x), nullptr,
                reinterpret_cast<int*>(w + l.bin_ends), reinterpret_cast<float4*>(w + l.grids)};
    PointSet none{nullptr, nullptr, 0, 1, CURVE_MAX_POINTS, nullptr, nullptr, nullptr, nullptr};
    const CloudRows rows{batch_x, batch_y, static_cast<int>(size_x), size_y, reinterpret_cast<int2*>(w + l.cloud_rows)};
    int st = launch_curve_cells(px, none, nullptr, s, rows);
    if (st != TPK_OK)
        return st;
    constexpr int WAVES = NG_SCAN_THREADS / TPK_WAVE;
    const int64_t blocks = tpk_ceil_div(size_y, WAVES);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    if (sorted)
        hipLaunchKernelGGL((ball_query_bins_kernel<true, false>), dim3(static_cast<unsigned>(blocks)), dim3(NG_SCAN_THREADS), 0, s,
                           static_cast<int>(size_x), static_cast<int>(size_y), window_shift, std::fabs(radius), radius2, nsample, x, y,
                           px.sorted, px.bin_ends, px.grid, rows.rows, idx, dist, 0, 0);
    else
        hipLaunchKernelGGL((ball_query_bins_kernel<false, false>), dim3(static_cast<unsigned>(blocks)), dim3(NG_SCAN_THREADS), 0, s,
                           static_cast<int>(size_x), static_cast<int>(size_y), window_shift, std::fabs(radius), radius2, nsample, x, y,
                           px.sorted, px.bin_ends, px.grid, rows.rows, idx, dist, 0, 0);
    return tpk_launch_status();
}

namespace {

// The dense layout takes the bin walk for clouds too large for the buckets of cells in LDS (ball_query.hip):
// the b clouds of n points are one array of b * n rows, cut into windows like the packed layout's.
bool ball_bins_dense_supported(int b, int n, int m, int nsample)
{
    // Ordering the points costs 17 - 30 us before the first query is answered, in which time the scan of all pairs
    // tests BQB_DENSE_MIN_PAIRS pairs: calls with fewer pairs keep the scan.  (What the host cannot know is how many
    // points a ball holds.  Where it holds hundreds, the scan in index order ends after a fraction of the cloud and
    // the walk over the bins has nothing to skip: measured 66 against 34 us for 4 x 20000 points, 5000 queries
    // each, 670 points per ball, and 222 against 162 us for 100000 points with 420 per ball - against 32 and 130 us,
    // 39 and 817 us where a ball holds a few points.)
    return n > BQB_DENSE_MIN_POINTS && b > 0 && m > 0 && nsample > 0 && static_cast<int64_t>(b) * n < (1LL << 30) &&
           static_cast<int64_t>(b) * m <= 0x7fffffffLL && static_cast<int64_t>(b) * n * m >= BQB_DENSE_MIN_PAIRS;
}

} // namespace

size_t tpk_grid_ball_query_dense_workspace_bytes(int b, int n, int m, int nsample)
{
    return ball_bins_dense_supported(b, n, m, nsample) ? ball_layout(static_cast<int64_t>(b) * n, 0).total : 0;
}

int tpk_grid_ball_query_dense(int b, int n, int m, float radius, float radius2, int nsample, const float* new_xyz,
                              const float* xyz, int64_t* idx, float* dist, void* workspace, size_t workspace_bytes,
                              hipStream_t s)
{
    if (!ball_bins_dense_supported(b, n, m, nsample))
        return TPK_ERR_UNSUPPORTED;
    const int64_t size_x = static_cast<int64_t>(b) * n, size_y = static_cast<int64_t>(b) * m;
    const BallLayout l = ball_layout(size_x, 0);
    if (!workspace || workspace_bytes < l.total || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return TPK_ERR_WORKSPACE;
    char* w = static_cast<char*>(workspace);
    const int window_shift = bqb_window_shift(size_x);
    PointSet px{xyz, nullptr, size_x, size_x, 1 << window_shift, reinterpret_cast<float4*>(w + l.sorted_x), nullptr,
                reinterpret_cast<int*>(w + l.bin_ends), reinterpret_cast<float4*>(w + l.grids)};
    PointSet none{nullptr, nullptr, 0, 1, CURVE_MAX_POINTS, nullptr, nullptr, nullptr, nullptr};
    int st = launch_curve_cells(px, none, nullptr, s);
    if (st != TPK_OK)
        return st;
    constexpr int WAVES = NG_SCAN_THREADS / TPK_WAVE;
    const int64_t blocks = tpk_ceil_div(size_y, WAVES);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((ball_query_bins_kernel<false, true>), dim3(static_cast<unsigned>(blocks)), dim3(NG_SCAN_THREADS), 0, s,
                       static_cast<int>(size_x), static_cast<int>(size_y), window_shift, std::fabs(radius), radius2, nsample, xyz,
                       new_xyz, px.sorted, px.bin_ends, px.grid, static_cast<const int2*>(nullptr), idx, dist, n, m);
    return tpk_launch_status();
}
