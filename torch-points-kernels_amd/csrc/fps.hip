// Furthest point sampling: npoint-1 dependent rounds of "update every point's distance to
// the chosen set, pick the point whose distance is largest".
//
// One workgroup (one compute unit) owns a cloud for the whole call; the rounds of a cloud
// depend on each other, so a call runs as many workgroups as there are clouds.  Four kernels
// by cloud size:
//   up to 512 points     fps_resident_kernel: one point per lane in registers, every point
//                        updated every round, one 24-byte LDS record per wavefront and one
//                        barrier per round (records double buffered);
//   up to 16384 points   fps_pruned_kernel: up to 32 points per lane in registers, cloud
//                        ordered along a space filling curve so that most updates can be
//                        skipped exactly (described at the kernel);
//   up to 163840 points  fps_cells_batched_kernel: the cloud ordered along the curve into cells of 64
//                        points that stay in memory (the caller's workspace); boxes, largest
//                        distance and best point of every cell in LDS; a round touches only
//                        the cells the new sample can change (described at the kernel);
//   larger clouds        fps_streaming_kernel: the selection code of the first kernel over
//                        points streamed from global memory, running minima in a workspace
//                        provided by the caller.
// In all of them the chosen point's coordinates travel through LDS with the selection: the
// chosen point is never re-read from memory.
//
// Semantics follow the reference kernel (cuda/src/sampling_gpu.cu:17-144): start at point
// 0; squared distances; points whose squared norm is <= 1e-3 are neither updated nor
// eligible; if no point is eligible the pick is 0.  Equal maxima resolve as its block
// reduction does: with BS = the reference's block size (largest power of two <= n, at
// most 512; cuda/include/cuda_utils.h:13-18), reference thread (k mod BS) keeps the lowest
// k among its own equal maxima, and the halving tree then prefers the thread whose number
// has the smaller bit-reversal.  Both rules together are "smallest tie key", with
//   key(k) = bitrev(k mod BS) * ceil(n / BS) + floor(k / BS).
#include "coarse_order.h"

#include <cmath>

namespace {

constexpr int FPS_THREADS = 1024;
constexpr int FPS_WAVES = FPS_THREADS / TPK_WAVE;
constexpr int FPS_REGISTER_POINTS = 16384; // largest cloud kept in registers

struct WaveRecord
{
    int val;     // bits of the wavefront's largest distance (-1.0f: no eligible point)
    unsigned tk; // tie key of the point holding it
    int k;       // its index in the cloud
    float x, y, z;
};

// Distances are >= 0 and the "nothing eligible" marker is -1.0f, so the bit patterns order
// like signed integers.
__device__ __forceinline__ int ordered_bits(float v)
{
    return __float_as_int(v);
}

// Lane of the wavefront holding the largest `val`; among equals the smallest tie key.
__device__ __forceinline__ int winning_lane(int val, unsigned tk, int& wave_val)
{
    wave_val = wave_max_i32(val);
    const unsigned long long top = __ballot(val == wave_val);
    if (__builtin_popcountll(top) == 1)
        return __builtin_ctzll(top);
    const unsigned cand = val == wave_val ? tk : 0xFFFFFFFFu;
    const unsigned lowest = wave_min_u32(cand);
    return __builtin_ctzll(__ballot(cand == lowest));
}

// Step 3: every wavefront reduces the 16 published records; returns the chosen point.
template <int WAVES>
__device__ __forceinline__ void reduce_records(const WaveRecord* __restrict__ rec, int lane,
                                               float p0x, float p0y, float p0z, int& k,
                                               float& sx, float& sy, float& sz, int& gv_out)
{
    const WaveRecord e = rec[lane & (WAVES - 1)];
    const int gv = __builtin_amdgcn_readfirstlane(row_all_max_i32(e.val));
    gv_out = gv;
    constexpr unsigned wave_bits = (1u << WAVES) - 1u;
    const unsigned top = static_cast<unsigned>(__ballot(e.val == gv)) & wave_bits;
    int w;
    if (__builtin_popcount(top) == 1)
    {
        w = __builtin_ctz(top);
    }
    else
    {
        const unsigned cand = e.val == gv ? e.tk : 0xFFFFFFFFu;
        const unsigned lowest = __builtin_amdgcn_readfirstlane(row_all_min_u32(cand));
        w = __builtin_ctz(static_cast<unsigned>(__ballot(cand == lowest)) & wave_bits);
    }
    k = __builtin_amdgcn_readlane(e.k, w);
    sx = tpk_read_lane(e.x, w);
    sy = tpk_read_lane(e.y, w);
    sz = tpk_read_lane(e.z, w);
    if (gv < 0)
    {
        // No eligible point in the whole cloud: the reference's reduction yields index 0.
        k = 0;
        sx = p0x;
        sy = p0y;
        sz = p0z;
    }
}

// A point takes part unless its squared norm is <= 1e-3 (compared in double precision, as
// the reference's literal makes it).
__device__ __forceinline__ bool eligible(float x, float y, float z)
{
    const float mag = (x * x) + (y * y) + (z * z);
    return !(static_cast<double>(mag) <= 1e-3);
}

// First slot whose value equals `value` (per lane; used only when lanes tie).
template <int PPT>
__device__ __forceinline__ int first_slot_equal(const int (&t)[PPT], int value)
{
    int slot = PPT - 1;
#pragma unroll
    for (int i = PPT - 2; i >= 0; --i)
        slot = t[i] == value ? i : slot;
    return slot;
}

template <int PPT, int THREADS>
__global__ __launch_bounds__(THREADS) void fps_resident_kernel(
    int n, int npoint, int log2_bs, int groups, const float* __restrict__ xyz,
    int32_t* __restrict__ out)
{
    constexpr int WAVES = THREADS / TPK_WAVE;
    constexpr int NG = PPT >= 4 ? PPT / 4 : 1; // slots are searched in groups of GS
    constexpr int GS = PPT / NG;
    __shared__ WaveRecord records[2][WAVES];

    xyz += static_cast<int64_t>(blockIdx.x) * n * 3;
    out += static_cast<int64_t>(blockIdx.x) * npoint;
    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / TPK_WAVE);

    // Lane `tid` owns points tid, tid + THREADS, ...: ascending slot = ascending tie key
    // (THREADS is a multiple of the reference's block size).  The running minimum of a point
    // is held as the bit pattern of a non-negative float, which orders like a signed
    // integer; an ineligible or absent point holds the pattern of -1.0f (negative as an
    // integer), which an integer min against any distance keeps forever.
    float x[PPT], y[PPT], z[PPT];
    int t[PPT];
#pragma unroll
    for (int i = 0; i < PPT; ++i)
    {
        const int k = tid + THREADS * i;
        bool ok = false;
        float px = 0.f, py = 0.f, pz = 0.f;
        if (k < n)
        {
            px = xyz[k * 3 + 0];
            py = xyz[k * 3 + 1];
            pz = xyz[k * 3 + 2];
            ok = eligible(px, py, pz);
        }
        x[i] = ok ? px : 0.f;
        y[i] = ok ? py : 0.f;
        z[i] = ok ? pz : 0.f;
        t[i] = ordered_bits(ok ? 1e10f : -1.0f);
    }

    const unsigned bs_mask = (1u << log2_bs) - 1u;
    const unsigned rev = log2_bs ? (__brev(tid & bs_mask) >> (32 - log2_bs)) : 0u;
    const unsigned tk_base = rev * static_cast<unsigned>(groups);

    const float p0x = xyz[0], p0y = xyz[1], p0z = xyz[2];
    float sx = p0x, sy = p0y, sz = p0z;
    if (tid == 0)
        out[0] = 0;

    for (int j = 1; j < npoint; ++j)
    {
        // 1. distance update: 8 double-rate fp32 operations + one integer min per point
        const float vx = to_vector_register(sx);
        const float vy = to_vector_register(sy);
        const float vz = to_vector_register(sz);
        int g[NG];
#pragma unroll
        for (int gi = 0; gi < NG; ++gi)
        {
#pragma unroll
            for (int e = 0; e < GS; ++e)
            {
                const int i = gi * GS + e;
                const float d = tpk_dist2(x[i], y[i], z[i], vx, vy, vz);
                t[i] = min(t[i], ordered_bits(d));
                g[gi] = e == 0 ? t[i] : max(g[gi], t[i]);
            }
        }
        int best = g[0];
#pragma unroll
        for (int gi = 1; gi < NG; ++gi)
            best = max(best, g[gi]);

        // 2. wavefront maximum and the lane that owns it
        const int wave_val = wave_max_i32(best);
        const unsigned long long top = __ballot(best == wave_val);
        int wl;
        if (__builtin_popcountll(top) == 1)
        {
            wl = __builtin_ctzll(top);
        }
        else
        {
            // several lanes hold the maximum: the smallest tie key decides
            const int bi = first_slot_equal<PPT>(t, best);
            const unsigned my_tk = tk_base + (static_cast<unsigned>(tid + THREADS * bi) >> log2_bs);
            const unsigned cand = best == wave_val ? my_tk : 0xFFFFFFFFu;
            const unsigned lowest = wave_min_u32(cand);
            wl = __builtin_ctzll(__ballot(cand == lowest));
        }
        // first slot of lane wl holding the maximum: its group first, then inside the group
        // (wave-uniform control flow; only lane reads, no per-lane bookkeeping in step 1)
        int grp = NG - 1;
#pragma unroll
        for (int gi = NG - 2; gi >= 0; --gi)
            grp = __builtin_amdgcn_readlane(g[gi], wl) == wave_val ? gi : grp;
        int slot = 0;
        float cx = 0.f, cy = 0.f, cz = 0.f;
#pragma unroll
        for (int gi = 0; gi < NG; ++gi)
            if (grp == gi)
            {
                int e_sel = GS - 1;
#pragma unroll
                for (int e = GS - 2; e >= 0; --e)
                    e_sel = __builtin_amdgcn_readlane(t[gi * GS + e], wl) == wave_val ? e : e_sel;
#pragma unroll
                for (int e = 0; e < GS; ++e)
                    if (e_sel == e)
                    {
                        slot = gi * GS + e;
                        cx = tpk_read_lane(x[gi * GS + e], wl);
                        cy = tpk_read_lane(y[gi * GS + e], wl);
                        cz = tpk_read_lane(z[gi * GS + e], wl);
                    }
            }
        const int win_tid = wave * TPK_WAVE + wl;
        const int win_k = win_tid + THREADS * slot;
        const unsigned win_rev = log2_bs ? (__brev(win_tid & bs_mask) >> (32 - log2_bs)) : 0u;
        WaveRecord r;
        r.val = wave_val;
        r.tk = win_rev * static_cast<unsigned>(groups) + (static_cast<unsigned>(win_k) >> log2_bs);
        r.k = win_k;
        r.x = cx;
        r.y = cy;
        r.z = cz;
        if (lane == 0)
            records[j & 1][wave] = r;
        __syncthreads();

        // 3. all wavefronts reduce the records
        int k;
        int gv_unused;
        reduce_records<WAVES>(records[j & 1], lane, p0x, p0y, p0z, k, sx, sy, sz, gv_unused);
        if (tid == 0)
            out[j] = k;
    }
}

// ---------------------------------------------------------------------------------------
// Register-resident kernel with exact pruning, for clouds of a few thousand to 16384 points.
//
// Pruning.  A point's running minimum changes in a round only if its distance to the new
// sample is smaller than that minimum, and no minimum exceeds the value that won the previous
// round.  So a set of points whose bounding box is further from the new sample than the square
// root of the previous winning value cannot change, and its update can be skipped without
// changing any result.  To make such sets exist, the kernel first orders the cloud along a
// Hilbert curve (12-bit position of its cell in a 16^3 grid, counting sort in LDS) and cuts the curve into cells of
// 64 * GS consecutive points.  A cell is GS registers of the 64 lanes of one wavefront; every
// wavefront holds NG cells, taken round-robin along the curve so that the cells around a
// sample belong to different wavefronts.  A wavefront tests its NG boxes at once, lane g
// testing the box of its group g, and updates only the live groups (wave-uniform branches).
// The fp32 box distance is compared with a relative margin of 2e-6, several times the rounding
// error of either side, so a skipped update is provably a no-op.
//
// Selection.  Each lane keeps the largest and second largest running minimum of every group; a
// wavefront publishes its two best points of different lanes (value, coordinates, sorted
// position: found per lane by compare/select, then through wave-uniform, GPR-indexed register
// reads) and the largest minimum it keeps to itself, and a round takes as many of the published
// points as follow each other as samples (described where the loop begins): several samples per
// round, each round's box tests one instruction sequence whatever their number.
//
// Equal maxima.  When several points hold the maximum, or no point is eligible, the round takes one
// sample by the reference's tie key over all points holding the maximum, through a copy of the
// running minima in LDS (slots are not in index order here, so the key is computed from the
// original index kept in the sort keys).
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ unsigned tie_key(int k, int log2_bs, int ref_groups)
{
    const unsigned bs_mask = (1u << log2_bs) - 1u;
    const unsigned rev = log2_bs ? (__brev(static_cast<unsigned>(k) & bs_mask) >> (32 - log2_bs)) : 0u;
    return rev * static_cast<unsigned>(ref_groups) + (static_cast<unsigned>(k) >> log2_bs);
}

// Register arrays of the sorted kernel are vector types: the winner's slot is a wave-uniform
// number known only at run time, and indexing a vector register tuple with a uniform index
// is one move in GPR-index mode (an array would be indexed through scratch memory).
template <int N>
struct RegisterVector
{
    typedef float floats __attribute__((ext_vector_type(N)));
    typedef int ints __attribute__((ext_vector_type(N)));
};

// The words of LDS through which the wavefronts of a workgroup agree on a round's winner.
struct RoundWords
{
    int max_val;      // atomic max of the running minima (bit patterns), starts at INT_MIN
    int winners;      // 1 when exactly one point holds max_val, more when several may
    unsigned min_tie; // atomic min of the tie keys of the points holding max_val (ties only)
    int pad;
};

// LDS atomics without return value, issued as written: one instruction for the active lanes
// (the compiler would otherwise wrap a same-address atomic in a loop over those lanes).
__device__ __forceinline__ unsigned lds_offset(const void* p)
{
    return static_cast<unsigned>(reinterpret_cast<unsigned long long>(
        (const __attribute__((address_space(3))) char*)p));
}
__device__ __forceinline__ void lds_atomic_max_i32(int* p, int v)
{
    asm volatile("ds_max_i32 %0, %1" ::"v"(lds_offset(p)), "v"(v) : "memory");
}
__device__ __forceinline__ void lds_atomic_add_u32(int* p, int v)
{
    asm volatile("ds_add_u32 %0, %1" ::"v"(lds_offset(p)), "v"(v) : "memory");
}

// Position on the sorted curve of member `e` of group `g` held by lane `lane` of wavefront `wave`.
template <int WAVES, int GS>
__device__ __forceinline__ int sorted_position(int g, int wave, int e, int lane)
{
    return ((g * WAVES + wave) * GS + e) * TPK_WAVE + lane;
}

template <int PPT, int THREADS, int GS>
__global__ __launch_bounds__(THREADS) void fps_pruned_kernel(
    int n, int npoint, int log2_bs, int ref_groups, int key_capacity,
    const float* __restrict__ xyz, int32_t* __restrict__ out)
{
    constexpr int WAVES = THREADS / TPK_WAVE;
    constexpr int NG = PPT / GS;
    static_assert(NG <= 16, "one DPP row of lanes tests the group boxes");
    static_assert(WAVES >= 2, "a cloud without eligible points must count several winners");
    // key_capacity keys (curve position << 20) | index in curve order, kept for the whole kernel; then
    // PPT * THREADS words (the unsorted keys during set-up, later the copy of the running minima
    // made when equal maxima have to be resolved); then the bins of the counting sort
    extern __shared__ unsigned sort_keys[];
    int* const t_copy = reinterpret_cast<int*>(sort_keys + key_capacity);
    unsigned* const unsorted = sort_keys + key_capacity;
    int* const bins = t_copy + PPT * THREADS; // CURVE_BINS words
    __shared__ int wave_totals[WAVES];
    __shared__ RoundWords words[2];
    __shared__ int cloud_box[6];      // ordered ints: min x,y,z then max x,y,z
    __shared__ int group_box[WAVES * NG * 6]; // the same per (wavefront, group) cell

    xyz += static_cast<int64_t>(blockIdx.x) * n * 3;
    out += static_cast<int64_t>(blockIdx.x) * npoint;
    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / TPK_WAVE);

    // ---- set-up 1 and 2: order the cloud along the curve (curve_order.h)
    if (tid < 2)
        words[tid] = RoundWords{INT_MIN, 0, 0xFFFFFFFFu, 0};
    curve_order<THREADS>(xyz, n, sort_keys, unsorted, bins, cloud_box, wave_totals);

    // ---- set-up 3: this lane's points.  The curve is cut into cells of 64 * GS consecutive
    // points; cell c belongs to wavefront c % WAVES as its group c / WAVES (neighbouring cells
    // go to different wavefronts, which spreads the work around a sample).  Slot i of a lane =
    // group (i / GS), member (i % GS); see sorted_position().
    typename RegisterVector<PPT>::floats x, y, z;
    typename RegisterVector<PPT>::ints t;
#pragma unroll
    for (int gi = 0; gi < NG; ++gi)
    {
        float lo[3] = {__builtin_inff(), __builtin_inff(), __builtin_inff()};
        float hi[3] = {-__builtin_inff(), -__builtin_inff(), -__builtin_inff()};
#pragma unroll
        for (int e = 0; e < GS; ++e)
        {
            const int i = gi * GS + e;
            const int q = sorted_position<WAVES, GS>(gi, wave, e, lane);
            const int k = static_cast<int>(sort_keys[q < n ? q : 0] & 0x3FFFu);
            const float px = xyz[k * 3 + 0], py = xyz[k * 3 + 1], pz = xyz[k * 3 + 2];
            const bool ok = q < n && eligible(px, py, pz);
            x[i] = ok ? px : 0.f;
            y[i] = ok ? py : 0.f;
            z[i] = ok ? pz : 0.f;
            t[i] = ordered_bits(ok ? 1e10f : -1.0f);
            lo[0] = ok ? fminf(lo[0], px) : lo[0];
            lo[1] = ok ? fminf(lo[1], py) : lo[1];
            lo[2] = ok ? fminf(lo[2], pz) : lo[2];
            hi[0] = ok ? fmaxf(hi[0], px) : hi[0];
            hi[1] = ok ? fmaxf(hi[1], py) : hi[1];
            hi[2] = ok ? fmaxf(hi[2], pz) : hi[2];
        }
        // the cell belongs to this wavefront alone: reduce over its lanes, plain store
#pragma unroll
        for (int a = 0; a < 3; ++a)
        {
            const int cell_lo = wave_min_i32(float_to_ordered_int(lo[a]));
            const int cell_hi = wave_max_i32(float_to_ordered_int(hi[a]));
            if (lane == 0)
            {
                group_box[(wave * NG + gi) * 6 + a] = cell_lo;
                group_box[(wave * NG + gi) * 6 + 3 + a] = cell_hi;
            }
        }
    }
    __syncthreads();
    // lane g of every 16-lane row tests this wavefront's group g; lanes beyond NG hold an empty box
    // (row g of the lanes tests group g, its lane k against sample k of the round)
    static_assert(NG <= 4, "one row of lanes per group");
    const int my_group = lane >> 4;
    float blo[3], bhi[3];
#pragma unroll
    for (int a = 0; a < 3; ++a)
    {
        blo[a] = my_group < NG ? ordered_int_to_float(group_box[(wave * NG + my_group) * 6 + a]) : __builtin_inff();
        bhi[a] = my_group < NG ? ordered_int_to_float(group_box[(wave * NG + my_group) * 6 + 3 + a]) : -__builtin_inff();
    }

    int g[NG]; // per-lane maximum of each group, kept across rounds
#pragma unroll
    for (int gi = 0; gi < NG; ++gi)
    {
        g[gi] = t[gi * GS];
#pragma unroll
        for (int e = 1; e < GS; ++e)
            g[gi] = max(g[gi], t[gi * GS + e]);
    }

    const float p0x = xyz[0], p0y = xyz[1], p0z = xyz[2];
    int bound = ordered_bits(__builtin_inff()); // no running minimum exceeds this
    const bool row_head = (lane & 15) == 0;
    int best = g[0]; // this lane's largest running minimum and that of its row of 16 lanes
#pragma unroll
    for (int gi = 1; gi < NG; ++gi)
        best = max(best, g[gi]);
    if (tid == 0)
        out[0] = 0;
    TPK_WORK_DECL

    {
        // Several samples per round.  After a round's updates let c0 > c1 > c2 ... be the points in the order of
        // their running minima.  c0 is the next sample.  If c1's minimum is not changed by c0 (c0 is no closer
        // to it than its minimum), then after c0's update c1 still holds what it held, nothing holds more, and
        // c1 is the sample after c0 - and so on: ck follows as long as none of c0 .. c(k-1) changes its minimum.
        // The largest minima sit in different corners of the cloud, far from each other, and a round takes eight
        // samples on average.  Every wavefront publishes its two best points and the largest minimum it does
        // not publish; after a barrier wavefront 0 sorts out the list - candidates above everything unpublished,
        // strictly ordered (equal minima are left to the exact resolution below, one sample at a time), each
        // unchanged by those before it - and after a second barrier all wavefronts apply the new samples'
        // updates together: which of a wavefront's groups a sample can change is one box test per (group,
        // sample), all of a round's in one instruction sequence.
        constexpr int FPB_T = WAVES >= 16 ? 16 : 8; // samples per round at most (16: one lane of a row each in the box tests)
        static_assert(FPB_T <= 16 && TPK_WAVE % FPB_T == 0, "the pair tests take whole rows of lanes");
        constexpr int FPB_PUB = 2; // points a wavefront publishes per round (3: 1 % faster at best)
        constexpr int CANDS = WAVES * FPB_PUB;
        static_assert(CANDS % 4 == 0 && CANDS <= TPK_WAVE && CANDS > FPB_T, "one lane per published point");
        __shared__ float4 cand_rec[2][CANDS];                // x, y, z, sorted position of the published points
        __shared__ __align__(16) int cand_val[2][CANDS];     // their running minima (INT_MIN: nothing published)
        __shared__ int hidden[2][WAVES];          // per wavefront: the largest minimum not published
        int g2[NG]; // per lane: second largest of each group (g: the largest)
#pragma unroll
        for (int gi = 0; gi < NG; ++gi)
        {
            int a1 = INT_MIN, a2 = INT_MIN;
#pragma unroll
            for (int e = 0; e < GS; ++e)
            {
                const int v = t[gi * GS + e];
                a2 = max(a2, min(a1, v));
                a1 = max(a1, v);
            }
            g2[gi] = a2;
        }
        // the samples whose updates are due: the round before's published points in the order of their minima
        // (first: point 0), and which of them may follow each other
        static_assert(FPB_PUB * CANDS <= TPK_WAVE && FPB_T <= WAVES, "a wavefront ranks its points in one step; one wavefront per place");
        __shared__ int order[2][CANDS];             // published point of every place
        __shared__ __align__(16) float4 taken[2][FPB_T]; // x, y, z, sorted position of the point of place k
        __shared__ int follows[2][FPB_T];           // 1: the point of place k may follow those before it
        __shared__ int largest[2];                  // the round's largest minimum
        if (tid == 0)
            taken[0][0] = make_float4(p0x, p0y, p0z, 0.f);
        __syncthreads();
        int ns = 1, from = 0;
        // Clouds with equal minima at the top in round after round (lattices, repeated points) gain nothing from the
        // list: after a round that had to fall back on the exact resolution the next `pause` rounds go there at
        // once, twice as many each time it happens again, until a round takes several samples.
        int pause = 0, penalty = 1, which = 0;
        int j = 1;
        for (int round = 1; j < npoint; ++round)
        {
            const int par = round & 1;
            // 1. the updates of the round before's samples.  Which groups can change?  Lane k < FPB_T fetches
            // sample k; row g of the lanes tests its lane's sample against group g.
            const float4 fetched = taken[from][lane < ns ? lane : 0];
            unsigned long long live;
            {
                const int k = lane & 15;
                const float sx = __shfl(fetched.x, k, TPK_WAVE), sy = __shfl(fetched.y, k, TPK_WAVE), sz = __shfl(fetched.z, k, TPK_WAVE);
                const float dx = fmaxf(fmaxf(blo[0] - sx, sx - bhi[0]), 0.f);
                const float dy = fmaxf(fmaxf(blo[1] - sy, sy - bhi[1]), 0.f);
                const float dz = fmaxf(fmaxf(blo[2] - sz, sz - bhi[2]), 0.f);
                const float lb = __builtin_fmaf(dx, dx, __builtin_fmaf(dy, dy, dz * dz)) * 0.999998f;
                // an empty box gives lb = +inf (never live); NaN compares false -> live
                live = __ballot(k < ns && !(lb >= __int_as_float(bound)));
            }
#pragma unroll
            for (int gi = 0; gi < NG; ++gi)
            {
                // samples that reach group gi, one bit each
                unsigned reach = static_cast<unsigned>(live >> (gi * 16)) & 0xFFFFu;
                if (reach == 0)
                    continue; // (uniform over the wavefront)
                while (reach != 0)
                {
                    const int k = __builtin_ctz(reach);
                    reach &= reach - 1;
                    const float sx = to_vector_register(tpk_read_lane(fetched.x, k)), sy = to_vector_register(tpk_read_lane(fetched.y, k));
                    const float sz = to_vector_register(tpk_read_lane(fetched.z, k));
                    TPK_WORK_ADD(GS);
#pragma unroll
                    for (int e = 0; e < GS; ++e)
                    {
                        const int i = gi * GS + e;
                        t[i] = min(t[i], ordered_bits(tpk_dist2(x[i], y[i], z[i], sx, sy, sz)));
                    }
                }
                int a1 = INT_MIN, a2 = INT_MIN;
#pragma unroll
                for (int e = 0; e < GS; ++e)
                {
                    const int v = t[gi * GS + e];
                    a2 = max(a2, min(a1, v));
                    a1 = max(a1, v);
                }
                g[gi] = a1;
                g2[gi] = a2;
            }
            // 2. the lane's largest and second largest minimum
            int b1 = INT_MIN, b2 = INT_MIN;
#pragma unroll
            for (int gi = 0; gi < NG; ++gi)
            {
                b2 = max(max(b2, min(b1, g[gi])), g2[gi]);
                b1 = max(b1, g[gi]);
            }
            best = b1;
            if (pause == 0)
            {
                // 3. the wavefront's FPB_PUB best points (of different lanes) and the largest minimum it keeps to itself
                // the slot of a lane's best point: group, then member (uniform indices into the registers)
                auto publish = [&](int from_lane, int place) __attribute__((always_inline)) {
                    int my_grp = 0;
#pragma unroll
                    for (int gi = NG - 1; gi >= 0; --gi)
                        my_grp = g[gi] == b1 ? gi : my_grp;
                    const int grp = __builtin_amdgcn_readlane(my_grp, from_lane);
                    int my_e = 0;
#pragma unroll
                    for (int e = GS - 1; e >= 0; --e)
                        my_e = t[grp * GS + e] == b1 ? e : my_e;
                    const int ce = __builtin_amdgcn_readlane(my_e, from_lane);
                    const int slot = grp * GS + ce;
                    const float cx = x[slot], cy = y[slot], cz = z[slot];
                    if (lane == from_lane)
                    {
                        cand_rec[par][place] = make_float4(cx, cy, cz, __int_as_float(sorted_position<WAVES, GS>(grp, wave, ce, lane)));
                        cand_val[par][place] = b1;
                    }
                };
                {
                    int left = b1;                   // the lane's best point not yet published
                    unsigned long long gone = 0ull;  // lanes whose best point is published
                    int most = wave_max_i32(left);
#pragma unroll
                    for (int p = 0; p < FPB_PUB; ++p)
                    {
                        const int from_lane = __builtin_ctzll(__ballot(left == most));
                        // (a lane's second point is not published: with it the list ends)
                        const bool fresh = ((gone >> from_lane) & 1ull) == 0ull;
                        if (fresh)
                        {
                            publish(from_lane, wave * FPB_PUB + p);
                            gone |= 1ull << from_lane;
                            left = lane == from_lane ? b2 : left;
                            most = wave_max_i32(left);
                        }
                        else if (lane == 0)
                            cand_val[par][wave * FPB_PUB + p] = INT_MIN;
                    }
                    if (lane == 0)
                        hidden[par][wave] = most;
                }
                lds_barrier();
                // 4. the list is sorted out by all wavefronts together, in two short steps.  First every wavefront
                // finds the places of its own published points among all of them (lane (c, o): is point o above my
                // point c? - equal values: the lower number first, so the places are distinct).
                {
                    const int c = lane / CANDS, o = lane % CANDS;
                    const int mine = wave * FPB_PUB + (c < FPB_PUB ? c : 0);
                    const int my_val = cand_val[par][mine], other = cand_val[par][o];
                    const unsigned long long above = __ballot(c < FPB_PUB && (other > my_val || (other == my_val && o < mine)));
                    if (o == 0 && c < FPB_PUB)
                        order[par][__builtin_popcountll((above >> (c * CANDS)) & ((1ull << CANDS) - 1ull))] = mine;
                }
                lds_barrier();
                // Then wavefront k looks at the point of place k: it may follow when its minimum is above everything
                // unpublished, strictly above the next one's (equal minima are left to the exact resolution below)
                // and a real minimum (>= 0), and when none of the points before it changes it (lane i: point i).
                if (wave < FPB_T)
                {
                    const int at = order[par][wave], next = order[par][wave + 1], before = order[par][lane < wave ? lane : 0];
                    const int val = cand_val[par][at], val_next = cand_val[par][next];
                    const float4 rec = cand_rec[par][at], earlier = cand_rec[par][before];
                    const int kept = wave_max_i32(lane < WAVES ? hidden[par][lane] : INT_MIN);
                    const bool spoiled = lane < wave && ordered_bits(tpk_dist2(rec.x, rec.y, rec.z, earlier.x, earlier.y, earlier.z)) < val;
                    // (after place 0 above 0: the samples before it drop to 0, and equal minima go by tie keys)
                    const bool may = __ballot(spoiled) == 0ull && val > kept && val > val_next && val >= (wave == 0 ? 0 : 1);
                    if (lane == 0)
                    {
                        taken[par][wave] = rec;
                        follows[par][wave] = may ? 1 : 0;
                        if (wave == 0)
                            largest[par] = val;
                    }
                }
                lds_barrier();
                const int accept = min(static_cast<int>(__builtin_ctzll(~__ballot(lane < FPB_T && follows[par][lane < FPB_T ? lane : 0] != 0))), npoint - j);
                if (accept > 0)
                {
                    if (wave == 0 && lane < accept) // (the others are on their way already)
                        out[j + lane] = static_cast<int>(sort_keys[__float_as_int(taken[par][lane].w)] & 0x3FFFu);
                    ns = accept;
                    from = par;
                    j += accept;
                    // (no minimum exceeds the round's largest; the new samples still hold theirs until their own updates)
                    bound = __builtin_amdgcn_readfirstlane(largest[par]);
                    penalty = accept > 1 ? 1 : penalty;
                    continue;
                }
                pause = penalty;
                penalty = min(2 * penalty, 32);
            }
            else
                --pause;

            // Equal minima at the top, or nothing eligible: one sample by the reference's tie key over all points
            // that hold the maximum (the key comes from the original index kept in the sort keys).
            if (tid == 0)
                words[which ^ 1] = RoundWords{INT_MIN, 0, 0xFFFFFFFFu, 0}; // (for the next time)
            const int row_best = row_all_max_i32(b1);
            if (row_head)
                lds_atomic_max_i32(&words[which].max_val, row_best);
            lds_barrier();
            const int gv = __builtin_amdgcn_readfirstlane(words[which].max_val);
            if (gv < 0)
            {
                // No eligible point in the whole cloud: the reference's reduction yields index 0.
                if (tid == 0)
                {
                    taken[par][0] = make_float4(p0x, p0y, p0z, 0.f);
                    out[j] = 0;
                }
            }
            else
            {
                unsigned my_tk = 0xFFFFFFFFu;
                int my_q = 0;
#pragma unroll
                for (int i = 0; i < PPT; ++i)
                {
                    const int q = sorted_position<WAVES, GS>(i / GS, wave, i % GS, lane);
                    if (t[i] == gv && q < n)
                    {
                        const unsigned tk = tie_key(static_cast<int>(sort_keys[q] & 0x3FFFu), log2_bs, ref_groups);
                        if (tk < my_tk)
                        {
                            my_tk = tk;
                            my_q = q;
                        }
                    }
                }
                if (my_tk != 0xFFFFFFFFu)
                    atomicMin(&words[which].min_tie, my_tk);
                lds_barrier();
                if (my_tk == words[which].min_tie) // tie keys are distinct: exactly one lane
                {
                    const int k = static_cast<int>(sort_keys[my_q] & 0x3FFFu);
                    taken[par][0] = make_float4(xyz[k * 3 + 0], xyz[k * 3 + 1], xyz[k * 3 + 2], __int_as_float(my_q));
                    out[j] = k;
                }
            }
            lds_barrier();
            which ^= 1;
            ns = 1;
            from = par;
            j += 1;
            bound = gv < 0 ? bound : gv;
        }
        TPK_WORK_FLUSH
        return;
    }
}

constexpr int FPS_CELL_WINDOW = CURVE_MAX_POINTS;            // points ordered together
constexpr int FPS_WINDOW_CELLS = FPS_CELL_WINDOW / NG_CELL;  // 256
constexpr int FPS_MAX_CELLS = 2560;                          // cells whose state fits in LDS
constexpr int FPS_CELL_POINTS = FPS_MAX_CELLS * NG_CELL;     // 163840
constexpr int FPS_LIVE_CAPACITY = (FPS_MAX_CELLS + FPS_THREADS - 1) / FPS_THREADS * TPK_WAVE; // live cells per wavefront

// Clouds too large for registers.  The cloud has been cut into windows of 16384 consecutive
// points, each ordered along the curve into 256 cells of 64 (curve_cells_kernel): records
// (x, y, z, index in the cloud) and the cells' boxes are in `sorted` / `boxes`; the running
// minima live in `temp`, in the same order (ineligible points and padding hold -1).  LDS keeps,
// for every cell, its box, its largest minimum, the tie key of the point holding it, and that
// point (x, y, z, index in the cloud).
// A minimum can only change if the new sample is closer than it, and no minimum of a cell
// exceeds the cell's largest: a cell whose box is not closer to the sample than its largest
// minimum is skipped (margin for rounding as in the register kernel), exactly.  Cell c belongs
// to wavefront c mod 16 (neighbours on the curve go to different wavefronts): the wavefront
// tests the boxes of its cells (one per lane and step), then updates the live ones - 64 points
// per cell, a few cells' loads in flight together - and renews their LDS entries.  After a
// Every wavefront then finds the best of its cells and the results are exchanged through LDS.
// Several samples are taken per round, as in fps_pruned_kernel: after a round's updates the points with the
// largest running minima follow each other as samples as long as none of them changes the next one's minimum.
// Here the order is by (minimum, then the reference's tie key), which is strict - equal minima need no separate
// path - and a candidate's coordinates are at hand in LDS (the best point of its cell).  LDS also keeps every
// cell's SECOND best point's minimum and key: what a wavefront does not publish - the best points of its other
// cells, the second best of all its cells - must stay below a candidate for it to count.  A live cell is loaded
// once per round and takes the updates of all samples that reach it.
// dynamic LDS: 56 bytes per cell + FPS_LIVE_CAPACITY * 16 * 4.
constexpr int FPC_T = 16;  // samples per round at most (one wavefront decides on each)
constexpr int FPC_PUB = 2; // points a wavefront publishes per round
constexpr int FPC_CANDS = FPS_WAVES * FPC_PUB;
#ifndef FPC_CELL_BATCH_N
#define FPC_CELL_BATCH_N 4
#endif
constexpr int FPC_CELL_BATCH = FPC_CELL_BATCH_N; // live cells in flight per wavefront
static_assert(FPC_T <= FPS_WAVES && FPC_T < FPC_CANDS && FPC_PUB * FPC_CANDS <= TPK_WAVE, "one wavefront per place, one lane per pair");

// (larger minimum first, among equals the smaller tie key)
__device__ __forceinline__ bool fps_above(int v, unsigned t, int w, unsigned u)
{
    return v > w || (v == w && t < u);
}

__global__ __launch_bounds__(FPS_THREADS) void fps_cells_batched_kernel(
    int n, int npoint, int log2_bs, int groups, int cells, const float* __restrict__ xyz,
    const float4* __restrict__ sorted, const float4* __restrict__ boxes, float* __restrict__ temp,
    int32_t* __restrict__ out)
{
    extern __shared__ float4 cell_best[];                                  // [cells] x, y, z, index
    float* const box = reinterpret_cast<float*>(cell_best + cells);        // [6][cells] lo.xyz, hi.xyz
    int* const cell_max = reinterpret_cast<int*>(box + 6 * cells);         // [cells] bits of the largest minimum
    unsigned* const cell_tie = reinterpret_cast<unsigned*>(cell_max + cells); // [cells] its point's tie key
    int* const cell_max2 = reinterpret_cast<int*>(cell_tie + cells);       // [cells] the same for the second best point
    unsigned* const cell_tie2 = reinterpret_cast<unsigned*>(cell_max2 + cells);
    unsigned* const live_all = cell_tie2 + cells;                          // per wavefront: live cell | samples that reach it << 16
    __shared__ int cand_val[2][FPC_CANDS];      // published points: minimum, tie key, cell
    __shared__ unsigned cand_tie[2][FPC_CANDS];
    __shared__ int cand_cell[2][FPC_CANDS];
    __shared__ int kept_val[2][FPS_WAVES];      // per wavefront: the best of what it does not publish
    __shared__ unsigned kept_tie[2][FPS_WAVES];
    __shared__ int order[2][FPC_CANDS];         // published point of every place
    __shared__ __align__(16) float4 taken[2][FPC_T]; // x, y, z, index of the point of place k
    __shared__ int follows[2][FPC_T];           // 1: the point of place k may follow those before it
    __shared__ __align__(16) float4 lone[2][FPS_WAVES]; // rounds with one sample: every wavefront's best point

    xyz += static_cast<int64_t>(blockIdx.x) * n * 3;
    sorted += static_cast<int64_t>(blockIdx.x) * cells * NG_CELL;
    boxes += static_cast<int64_t>(blockIdx.x) * cells * NG_BOX;
    temp += static_cast<int64_t>(blockIdx.x) * cells * NG_CELL;
    out += static_cast<int64_t>(blockIdx.x) * npoint;
    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / TPK_WAVE);
    unsigned* const live = live_all + wave * FPS_LIVE_CAPACITY;
    const int steps = (cells + FPS_THREADS - 1) / FPS_THREADS; // cells per lane
    const unsigned bs_mask = (1u << log2_bs) - 1u;
    auto tie_key = [&](unsigned k) __attribute__((always_inline)) {
        const unsigned rev = log2_bs ? (__brev(k & bs_mask) >> (32 - log2_bs)) : 0u;
        return rev * static_cast<unsigned>(groups) + (k >> log2_bs);
    };

    // Set-up: minima, boxes and largest minima (best points are found by the first update: it reaches every cell).
    for (int c = wave; c < cells; c += FPS_WAVES)
    {
        const float4 r = sorted[c * NG_CELL + lane];
        const bool takes_part = __float_as_int(r.w) != 0x7FFFFFFF && eligible(r.x, r.y, r.z);
        temp[c * NG_CELL + lane] = takes_part ? 1e10f : -1.0f;
        const bool any = __ballot(takes_part) != 0;
        if (lane < 6)
        {
            const float4 b = boxes[c * NG_BOX + lane / 3];
            const int a = lane % 3;
            box[lane * cells + c] = a == 0 ? b.x : a == 1 ? b.y : b.z;
        }
        if (lane == 6)
        {
            cell_max[c] = ordered_bits(any ? 1e10f : -1.0f);
            cell_tie[c] = 0xFFFFFFFFu;
            cell_max2[c] = ordered_bits(-1.0f);
            cell_tie2[c] = 0xFFFFFFFFu;
        }
    }
    const float p0x = xyz[0], p0y = xyz[1], p0z = xyz[2];
    if (tid == 0)
    {
        out[0] = 0;
        taken[0][0] = make_float4(p0x, p0y, p0z, 0.f);
    }
    __syncthreads();

    // Rounds in which only one point follows cost more this way than with one sample per round (two barriers
    // more, second bests): from the second such round in a row on, the next 1, 2, 4 .. 32 rounds take one sample
    // each, the plain way.
    int ns = 1, j = 1, pause = 0, penalty = 0;
    float4 fetched = taken[0][0]; // lane k < ns: sample k of the round before
    for (int round = 1; j < npoint; ++round)
    {
        const int par = round & 1;
        // 1. the live cells among this wavefront's, and which of the round before's samples reach each
        int count = 0;
        for (int step = 0; step < steps; ++step)
        {
            const int c = (step * TPK_WAVE + lane) * FPS_WAVES + wave;
            unsigned reach = 0;
            if (c < cells)
            {
                const float lx = box[0 * cells + c], ly = box[1 * cells + c], lz = box[2 * cells + c];
                const float hx = box[3 * cells + c], hy = box[4 * cells + c], hz = box[5 * cells + c];
                const float most = __int_as_float(cell_max[c]);
                for (int k = 0; k < ns; ++k)
                {
                    const float sx = tpk_read_lane(fetched.x, k), sy = tpk_read_lane(fetched.y, k), sz = tpk_read_lane(fetched.z, k);
                    const float dx = fmaxf(fmaxf(lx - sx, sx - hx), 0.f);
                    const float dy = fmaxf(fmaxf(ly - sy, sy - hy), 0.f);
                    const float dz = fmaxf(fmaxf(lz - sz, sz - hz), 0.f);
                    const float lb = __builtin_fmaf(dx, dx, __builtin_fmaf(dy, dy, dz * dz));
                    reach |= lb * 0.999998f < most ? 1u << k : 0u;
                }
            }
            const unsigned long long mask = __ballot(reach != 0);
            if (reach != 0)
                live[count + tpk_prefix_count(mask)] = static_cast<unsigned>(c) | (reach << 16);
            count += __builtin_popcountll(mask);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();

        // 2. their points: new minima, and the cell's best and second best point
        for (int i0 = 0; i0 < count; i0 += FPC_CELL_BATCH)
        {
            unsigned entry[FPC_CELL_BATCH];
            float4 r[FPC_CELL_BATCH];
            float m[FPC_CELL_BATCH];
#pragma unroll
            for (int u = 0; u < FPC_CELL_BATCH; ++u)
            {
                entry[u] = __builtin_amdgcn_readfirstlane(live[min(i0 + u, count - 1)]);
                const int c = static_cast<int>(entry[u] & 0xFFFFu);
                r[u] = sorted[c * NG_CELL + lane];
                m[u] = temp[c * NG_CELL + lane];
            }
#pragma unroll
            for (int u = 0; u < FPC_CELL_BATCH; ++u)
            {
                if (i0 + u >= count) // wave-uniform
                    break;
                const int c = static_cast<int>(entry[u] & 0xFFFFu);
                const int old_bits = ordered_bits(m[u]);
                int new_bits = old_bits;
                for (unsigned reach = entry[u] >> 16; reach != 0; reach &= reach - 1)
                {
                    const int k = __builtin_ctz(reach);
                    const float d = tpk_dist2(r[u].x, r[u].y, r[u].z, tpk_read_lane(fetched.x, k), tpk_read_lane(fetched.y, k),
                                              tpk_read_lane(fetched.z, k));
                    new_bits = min(ordered_bits(d), new_bits); // -1 stays -1
                }
                if (new_bits != old_bits)
                    temp[c * NG_CELL + lane] = __int_as_float(new_bits);
                const unsigned k = static_cast<unsigned>(__float_as_int(r[u].w));
                const unsigned tk = tie_key(k);
                int first_val, second_val;
                const int first = winning_lane(new_bits, tk, first_val);
                const int second = winning_lane(lane == first ? INT_MIN : new_bits, tk, second_val);
                if (lane == first)
                {
                    cell_max[c] = first_val;
                    cell_tie[c] = tk;
                    cell_best[c] = make_float4(r[u].x, r[u].y, r[u].z, __int_as_float(static_cast<int>(k)));
                }
                if (lane == second)
                {
                    cell_max2[c] = second_val;
                    cell_tie2[c] = tk;
                }
            }
        }

        // 3. the two best of this wavefront's cells, and the best of what it keeps to itself: per lane the best
        // cell (b1) and the best of everything else the lane knows of (b2: its other cells' best points and all
        // its cells' second best points)
        int b1v = INT_MIN, b2v = INT_MIN, b1c = 0;
        unsigned b1t = 0xFFFFFFFFu, b2t = 0xFFFFFFFFu;
        if (pause > 0) // wave-uniform, the same in all wavefronts
        {
            for (int step = 0; step < steps; ++step)
            {
                const int c = (step * TPK_WAVE + lane) * FPS_WAVES + wave;
                if (c < cells)
                {
                    const int v = cell_max[c];
                    const unsigned t = cell_tie[c];
                    if (fps_above(v, t, b1v, b1t))
                    {
                        b1v = v;
                        b1t = t;
                        b1c = c;
                    }
                }
            }
            int v1, all_v;
            const int l1 = winning_lane(b1v, b1t, v1);
            const unsigned t1 = __builtin_amdgcn_readlane(b1t, l1);
            const float4 mine = cell_best[__builtin_amdgcn_readlane(b1c, l1)];
            if (lane == 0)
            {
                cand_val[par][wave] = v1;
                cand_tie[par][wave] = t1;
                lone[par][wave] = mine;
            }
            lds_barrier();
            const int wl = winning_lane(lane < FPS_WAVES ? cand_val[par][lane] : INT_MIN,
                                        lane < FPS_WAVES ? cand_tie[par][lane] : 0xFFFFFFFFu, all_v);
            fetched = lone[par][wl];
            if (all_v < 0) // no eligible point in the whole cloud: the reference's reduction yields index 0
                fetched = make_float4(p0x, p0y, p0z, 0.f);
            if (tid == 0)
                out[j] = __float_as_int(fetched.w);
            ns = 1;
            j += 1;
            --pause;
            continue;
        }
        for (int step = 0; step < steps; ++step)
        {
            const int c = (step * TPK_WAVE + lane) * FPS_WAVES + wave;
            if (c < cells)
            {
                const int v = cell_max[c], v2 = cell_max2[c];
                const unsigned t = cell_tie[c], t2 = cell_tie2[c];
                if (fps_above(v, t, b1v, b1t))
                {
                    b2v = b1v;
                    b2t = b1t;
                    b1v = v;
                    b1t = t;
                    b1c = c;
                }
                else if (fps_above(v, t, b2v, b2t))
                {
                    b2v = v;
                    b2t = t;
                }
                if (fps_above(v2, t2, b2v, b2t))
                {
                    b2v = v2;
                    b2t = t2;
                }
            }
        }
        {
            int v1, v2, v3 = INT_MIN;
            const int l1 = winning_lane(b1v, b1t, v1);
            const unsigned t1 = __builtin_amdgcn_readlane(b1t, l1);
            const int c1 = __builtin_amdgcn_readlane(b1c, l1);
            const int left_v = lane == l1 ? b2v : b1v;
            const unsigned left_t = lane == l1 ? b2t : b1t;
            const int l2 = winning_lane(left_v, left_t, v2);
            const unsigned t2 = __builtin_amdgcn_readlane(left_t, l2);
            const int c2 = __builtin_amdgcn_readlane(b1c, l2);
            const bool two = l2 != l1; // (else the second best is something of the first lane's: not published)
            unsigned t3 = 0xFFFFFFFFu;
            if (two)
            {
                const int rest_v = (lane == l1 || lane == l2) ? b2v : b1v;
                const unsigned rest_t = (lane == l1 || lane == l2) ? b2t : b1t;
                const int l3 = winning_lane(rest_v, rest_t, v3);
                t3 = __builtin_amdgcn_readlane(rest_t, l3);
            }
            if (lane == 0)
            {
                cand_val[par][wave * 2 + 0] = v1;
                cand_tie[par][wave * 2 + 0] = t1;
                cand_cell[par][wave * 2 + 0] = c1;
                cand_val[par][wave * 2 + 1] = two ? v2 : INT_MIN;
                cand_tie[par][wave * 2 + 1] = two ? t2 : 0xFFFFFFFFu;
                cand_cell[par][wave * 2 + 1] = two ? c2 : 0;
                kept_val[par][wave] = two ? v3 : v2;
                kept_tie[par][wave] = two ? t3 : t2;
            }
        }
        lds_barrier();

        // 4. the list is sorted out by all wavefronts together.  First every wavefront finds the places of its own
        // published points among all of them (lane (c, o): is point o above my point c?).
        {
            const int c = lane / FPC_CANDS, o = lane % FPC_CANDS;
            const int mine = wave * FPC_PUB + (c < FPC_PUB ? c : 0);
            const int mv = cand_val[par][mine], ov = cand_val[par][o];
            const unsigned mt = cand_tie[par][mine], ot = cand_tie[par][o];
            // (points that are not published are all alike: the lower number first)
            const bool higher = fps_above(ov, ot, mv, mt) || (ov == mv && ot == mt && o < mine);
            const unsigned long long above = __ballot(c < FPC_PUB && higher);
            if (o == 0 && c < FPC_PUB)
                order[par][__builtin_popcountll((above >> (c * FPC_CANDS)) & ((1ull << FPC_CANDS) - 1ull))] = mine;
        }
        lds_barrier();
        // Then wavefront k looks at the point of place k: the point of place 0 is the reference's choice; a later
        // one may follow when it is above everything unpublished and none of the points before it changes its
        // minimum (lane i: point i).
        if (wave < FPC_T)
        {
            const int at = order[par][wave], before = order[par][lane < wave ? lane : 0];
            const int val = cand_val[par][at];
            const unsigned tie = cand_tie[par][at];
            float4 rec = cell_best[cand_cell[par][at]];
            const float4 earlier = cell_best[cand_cell[par][before]];
            int kept_v;
            const int hv = lane < FPS_WAVES ? kept_val[par][lane] : INT_MIN;
            const unsigned ht = lane < FPS_WAVES ? kept_tie[par][lane] : 0xFFFFFFFFu;
            const int kl = winning_lane(hv, ht, kept_v);
            const unsigned kept_t = __builtin_amdgcn_readlane(ht, kl);
            const bool spoiled = lane < wave && ordered_bits(tpk_dist2(rec.x, rec.y, rec.z, earlier.x, earlier.y, earlier.z)) < val;
            // (its minimum must be above 0: the samples before it drop to 0 and keep their tie keys)
            const bool may = wave == 0 || (__ballot(spoiled) == 0ull && fps_above(val, tie, kept_v, kept_t) && val > 0);
            if (wave == 0 && val < 0) // no eligible point in the whole cloud: the reference's reduction yields index 0
                rec = make_float4(p0x, p0y, p0z, 0.f);
            if (lane == 0)
            {
                taken[par][wave] = rec;
                follows[par][wave] = may ? 1 : 0;
            }
        }
        lds_barrier();
        int accept = static_cast<int>(__builtin_ctzll(~__ballot(lane < FPC_T && follows[par][lane < FPC_T ? lane : 0] != 0)));
        accept = min(accept, npoint - j); // (>= 1: the point of place 0 always follows)
        if (wave == 0 && lane < accept)
            out[j + lane] = __float_as_int(taken[par][lane].w);
        fetched = taken[par][lane < accept ? lane : 0];
        ns = accept;
        j += accept;
        if (accept > 1)
            penalty = 0;
        else
        {
            pause = penalty;
            penalty = penalty ? min(2 * penalty, 32) : 1;
        }
    }
}

// Clouds too large for registers: points and running minima stream from global memory.
__global__ __launch_bounds__(FPS_THREADS) void fps_streaming_kernel(
    int n, int npoint, int log2_bs, int groups, const float* __restrict__ xyz,
    float* __restrict__ temp, int32_t* __restrict__ out)
{
    __shared__ WaveRecord records[2][FPS_WAVES];

    xyz += static_cast<int64_t>(blockIdx.x) * n * 3;
    temp += static_cast<int64_t>(blockIdx.x) * n;
    out += static_cast<int64_t>(blockIdx.x) * npoint;
    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / TPK_WAVE);

    for (int k = tid; k < n; k += FPS_THREADS)
        temp[k] = 1e10f;

    const unsigned bs_mask = (1u << log2_bs) - 1u;
    const unsigned rev = log2_bs ? (__brev(tid & bs_mask) >> (32 - log2_bs)) : 0u;
    const unsigned tk_base = rev * static_cast<unsigned>(groups);

    const float p0x = xyz[0], p0y = xyz[1], p0z = xyz[2];
    float sx = p0x, sy = p0y, sz = p0z;
    if (tid == 0)
        out[0] = 0;

    for (int j = 1; j < npoint; ++j)
    {
        float best = -1.0f;
        int bk = tid < n ? tid : 0;
        for (int k = tid; k < n; k += FPS_THREADS)
        {
            const float px = xyz[k * 3 + 0], py = xyz[k * 3 + 1], pz = xyz[k * 3 + 2];
            if (!eligible(px, py, pz))
                continue;
            const float d = tpk_dist2(px, py, pz, sx, sy, sz);
            const float d2 = fminf(d, temp[k]);
            temp[k] = d2;
            bk = d2 > best ? k : bk;
            best = d2 > best ? d2 : best;
        }
        const unsigned my_tk = tk_base + (static_cast<unsigned>(bk) >> log2_bs);

        int wave_val;
        const int wl = winning_lane(ordered_bits(best), my_tk, wave_val);
        WaveRecord r;
        r.val = wave_val;
        r.tk = __builtin_amdgcn_readlane(my_tk, wl);
        r.k = __builtin_amdgcn_readlane(bk, wl);
        r.x = xyz[r.k * 3 + 0];
        r.y = xyz[r.k * 3 + 1];
        r.z = xyz[r.k * 3 + 2];
        if (lane == 0)
            records[j & 1][wave] = r;
        __syncthreads();

        int k;
        int gv_unused;
        reduce_records<FPS_WAVES>(records[j & 1], lane, p0x, p0y, p0z, k, sx, sy, sz, gv_unused);
        if (tid == 0)
            out[j] = k;
    }
}

__global__ __launch_bounds__(256) void fill_zero_i32_kernel(int32_t* p, int64_t count)
{
    int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (; t < count; t += stride)
        p[t] = 0;
}

// The reference's block size for n points (cuda/include/cuda_utils.h:13-18), as a log2.
int reference_log2_block(int n)
{
    const int pow_2 = static_cast<int>(std::log(static_cast<double>(n)) / std::log(2.0));
    int v = 1 << pow_2;
    if (v > 512)
        v = 512;
    if (v < 1)
        v = 1;
    int l = 0;
    while ((1 << l) < v)
        ++l;
    return l;
}

template <int PPT, int THREADS>
void launch_resident(int b, int n, int npoint, int log2_bs, int groups, const float* xyz,
                     int32_t* out, hipStream_t s)
{
    hipLaunchKernelGGL((fps_resident_kernel<PPT, THREADS>), dim3(b), dim3(THREADS), 0, s, n,
                       npoint, log2_bs, groups, xyz, out);
}


template <int PPT, int THREADS, int GS>
int launch_pruned(int b, int n, int npoint, int log2_bs, int groups, const float* xyz,
                  int32_t* out, hipStream_t s)
{
    const int key_capacity = n > CURVE_BINS ? (n + 63) & ~63 : CURVE_BINS; // (the ordering borrows CURVE_BINS words)
    const size_t lds = (static_cast<size_t>(key_capacity) + static_cast<size_t>(PPT) * THREADS + CURVE_BINS) * sizeof(unsigned);
    auto kernel = fps_pruned_kernel<PPT, THREADS, GS>;
    const int allowed = tpk_allow_lds(reinterpret_cast<const void*>(kernel), lds);
    if (allowed != TPK_OK)
        return allowed;
    hipLaunchKernelGGL(kernel, dim3(b), dim3(THREADS), lds, s, n, npoint, log2_bs, groups, key_capacity,
                       xyz, out);
    return tpk_launch_status();
}

// Workspace of the cell kernel: ordered records, boxes, minima (each 256-byte aligned).
struct CellLayout
{
    int cells; // per cloud
    size_t sorted, boxes, temp, coarse, total;
};
// Clouds of more than one window are brought into a coarse order first (coarse_order.h), in batches it can index.
bool fps_coarse_first(int b, int n)
{
    return n >= CO_MIN_ROWS && static_cast<int64_t>(b) * n < (1LL << 30);
}
CellLayout cell_layout(int b, int n)
{
    auto up = [](size_t v) { return (v + 255) & ~static_cast<size_t>(255); };
    CellLayout l;
    l.cells = static_cast<int>(tpk_ceil_div(n, FPS_CELL_WINDOW)) * FPS_WINDOW_CELLS;
    const size_t all = static_cast<size_t>(b) * l.cells;
    l.sorted = 0;
    l.boxes = up(all * NG_CELL * sizeof(float4));
    l.temp = up(l.boxes + all * NG_BOX * sizeof(float4));
    l.coarse = up(l.temp + all * NG_CELL * sizeof(float));
    l.total = fps_coarse_first(b, n) ? up(l.coarse + coarse_layout(static_cast<int64_t>(b) * n).total) : l.coarse;
    return l;
}

size_t streaming_bytes(int b, int n)
{
    return static_cast<size_t>(b) * static_cast<size_t>(n) * sizeof(float);
}

} // namespace

extern "C" size_t tpk_fps_workspace_bytes(int b, int n)
{
    if (b <= 0 || n <= FPS_REGISTER_POINTS)
        return 0;
    return n <= FPS_CELL_POINTS ? cell_layout(b, n).total : streaming_bytes(b, n);
}

extern "C" int tpk_fps_f32(int b, int n, int npoint, const float* xyz, void* workspace,
                           size_t workspace_bytes, int32_t* idx_out, void* stream)
{
    if (b < 0 || n < 0 || npoint < 0)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || npoint == 0)
        return TPK_OK;
    if (!idx_out)
        return TPK_ERR_INVALID_ARG;
    hipStream_t s = tpk_stream(stream);
    if (n == 0)
    {
        // Nothing to sample from: the reference returns its zero-initialised output.
        const int64_t count = static_cast<int64_t>(b) * npoint;
        hipLaunchKernelGGL(fill_zero_i32_kernel,
                           dim3(static_cast<unsigned>(tpk_min64(tpk_ceil_div(count, 256), 4096))),
                           dim3(256), 0, s, idx_out, count);
        return tpk_launch_status();
    }
    if (!xyz)
        return TPK_ERR_INVALID_ARG;
    if (static_cast<int64_t>(n) * 3 > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const int log2_bs = reference_log2_block(n);
    const int groups = static_cast<int>(tpk_ceil_div(n, 1 << log2_bs));

    // Tiny clouds: one point per lane, no sorting.  Up to 16384 points: registers of a workgroup of 512 or
    // 1024 lanes, curve order and pruning (cells of 64, 128 or 256 points).  Shapes as measured: sixteen
    // wavefronts with half as many points each shorten a round (fewer cells per wavefront to update, fewer
    // groups for the winner to search) except between 4097 and 8192 points.
    if (n <= 512)
        launch_resident<1, FPS_THREADS>(b, n, npoint, log2_bs, groups, xyz, idx_out, s);
    else if (n <= 512 * 2)
        return launch_pruned<2, 512, 1>(b, n, npoint, log2_bs, groups, xyz, idx_out, s);
    else if (n <= 512 * 4)
        return launch_pruned<2, 1024, 2>(b, n, npoint, log2_bs, groups, xyz, idx_out, s);
    else if (n <= 512 * 8)
        return launch_pruned<4, 1024, 4>(b, n, npoint, log2_bs, groups, xyz, idx_out, s);
    else if (n <= 512 * 16)
        return launch_pruned<16, 512, 4>(b, n, npoint, log2_bs, groups, xyz, idx_out, s);
    else if (n <= FPS_REGISTER_POINTS)
        return launch_pruned<16, 1024, 4>(b, n, npoint, log2_bs, groups, xyz, idx_out, s);
    else if (n <= FPS_CELL_POINTS && workspace && workspace_bytes >= cell_layout(b, n).total)
    {
        // Cells of 64 points in memory, their summaries in LDS.
        const CellLayout l = cell_layout(b, n);
        char* const w = static_cast<char*>(workspace);
        PointSet cloud{xyz, nullptr, static_cast<int64_t>(b) * n, n, FPS_CELL_WINDOW,
                       reinterpret_cast<float4*>(w + l.sorted), reinterpret_cast<float4*>(w + l.boxes), nullptr, nullptr};
        PointSet none{nullptr, nullptr, 0, 1, FPS_CELL_WINDOW, nullptr, nullptr, nullptr, nullptr};
        int st = TPK_OK;
        if (fps_coarse_first(b, n))
        {
            // windows that are neighbourhoods instead of samples of the whole cloud: cells half as wide
            st = launch_coarse_order(xyz, static_cast<int64_t>(b) * n, n, w + l.coarse, s);
            if (st != TPK_OK)
                return st;
            cloud.records = reinterpret_cast<const float4*>(w + l.coarse);
        }
        st = launch_curve_cells(cloud, none, nullptr, s);
        if (st != TPK_OK)
            return st;
        const size_t lds = static_cast<size_t>(l.cells) * 56 + FPS_LIVE_CAPACITY * FPS_WAVES * sizeof(unsigned);
        auto kernel = fps_cells_batched_kernel;
        st = tpk_allow_lds(reinterpret_cast<const void*>(kernel), lds);
        if (st != TPK_OK)
            return st;
        hipLaunchKernelGGL(kernel, dim3(b), dim3(FPS_THREADS), lds, s, n, npoint, log2_bs, groups, l.cells,
                           xyz, cloud.sorted, cloud.boxes, reinterpret_cast<float*>(w + l.temp), idx_out);
    }
    else
    {
        // (also serves callers that sized the workspace for the minima only)
        const size_t need = streaming_bytes(b, n);
        if (!workspace || workspace_bytes < need)
            return TPK_ERR_WORKSPACE;
        hipLaunchKernelGGL(fps_streaming_kernel, dim3(b), dim3(FPS_THREADS), 0, s, n, npoint,
                           log2_bs, groups, xyz, static_cast<float*>(workspace), idx_out);
    }
    return tpk_launch_status();
}
