// Chamfer distance: nearest-neighbour distance and index in both directions, and the
// gradient of those distances with respect to both clouds.
//
// Forward.  Both directions run in ONE launch (the first part of the grid scans cloud 2
// for the points of cloud 1, the rest the other way round).  A lane owns Q query points;
// the scanned cloud streams through LDS as tiles of (x, y, z, pad), read by all lanes at
// the same address (broadcast).  The scan is a plain all-pairs fp32/fp64 VALU reduction;
// the inner dimension is 3 and the products must round as the reference's do, so the
// matrix cores are not used.
//
// Per pair the work is 8 flops for the distance; keeping "which candidate was it" next to
// the minimum would add a compare and two selects per pair.  Instead the scan keeps only
// the minimum of each group of CHUNK consecutive candidates (min3: half an operation per
// pair), compares it once per group with the running best (strictly smaller replaces, so
// the earliest group holding the minimum wins) and remembers the group.  After the scan
// each lane re-evaluates the CHUNK candidates of its winning group and takes the first
// whose distance equals the minimum: the same candidate a serial first-strictly-smaller
// scan (cuda/src/chamfer_dist_gpu.cu:9-155) ends on.
//
// Backward (cuda/src/chamfer_dist_gpu.cu:187-245).  A point's gradient is its own term,
// 2*g*(p - nearest), plus one term from every point of the other cloud that chose it as
// nearest neighbour.  The reference scatters those with float atomics.  Here the two
// nearest-neighbour index arrays are inverted into per-target lists (lists.h) and one
// kernel, one lane per point, adds the own term and walks the point's list: no atomics, no
// zero fill, every output written once.  Without workspace for the lists the scatter falls
// back to hardware float atomics (own terms stored first by one kernel, scattered terms
// added by a second).
#include "lists.h"
#include "nn_grid.h"

namespace {

constexpr int CH_THREADS = 256;
constexpr int CH_TILE = 1024; // scanned points per LDS tile
constexpr int CH_CHUNK = 8;   // candidates per "which group held the minimum" record

template <typename T>
struct Point4
{
    T x, y, z, w;
};

template <typename T>
__device__ __forceinline__ T tpk_min(T a, T b);
template <>
__device__ __forceinline__ float tpk_min<float>(float a, float b)
{
    return fminf(a, b);
}
template <>
__device__ __forceinline__ double tpk_min<double>(double a, double b)
{
    return fmin(a, b);
}

template <typename T>
__device__ __forceinline__ T tpk_inf();
template <>
__device__ __forceinline__ float tpk_inf<float>()
{
    return __builtin_inff();
}
template <>
__device__ __forceinline__ double tpk_inf<double>()
{
    return __builtin_inf();
}

template <typename T, int Q>
__global__ __launch_bounds__(CH_THREADS) void chamfer_fwd_kernel(
    int n, int m, int blocks_per_cloud1, int blocks_per_cloud2, int blocks_dir1,
    const T* __restrict__ xyz1, const T* __restrict__ xyz2, T* __restrict__ dist1,
    T* __restrict__ dist2, int32_t* __restrict__ idx1, int32_t* __restrict__ idx2)
{
    __shared__ Point4<T> tile[CH_TILE];

    // Direction 1: queries = cloud 1 (n points), scanned = cloud 2 (m points); direction 2
    // swaps the roles.
    int bid = blockIdx.x;
    const bool dir2 = bid >= blocks_dir1;
    if (dir2)
        bid -= blocks_dir1;
    const int nq = dir2 ? m : n;
    const int nc = dir2 ? n : m;
    const int bpc = dir2 ? blocks_per_cloud2 : blocks_per_cloud1;
    const int cloud = bid / bpc;
    const int blk = bid - cloud * bpc;
    const T* __restrict__ qs = (dir2 ? xyz2 : xyz1) + static_cast<int64_t>(cloud) * nq * 3;
    const T* __restrict__ cs = (dir2 ? xyz1 : xyz2) + static_cast<int64_t>(cloud) * nc * 3;
    T* __restrict__ dout = (dir2 ? dist2 : dist1) + static_cast<int64_t>(cloud) * nq;
    int32_t* __restrict__ iout = (dir2 ? idx2 : idx1) + static_cast<int64_t>(cloud) * nq;

    const int tid = threadIdx.x;
    const int j0 = blk * (CH_THREADS * Q) + tid;

    T qx[Q], qy[Q], qz[Q], best[Q];
    int bgroup[Q];
#pragma unroll
    for (int q = 0; q < Q; ++q)
    {
        int j = j0 + q * CH_THREADS;
        j = j < nq ? j : nq - 1; // lanes past the end shadow the last query and store nothing
        qx[q] = qs[static_cast<int64_t>(j) * 3 + 0];
        qy[q] = qs[static_cast<int64_t>(j) * 3 + 1];
        qz[q] = qs[static_cast<int64_t>(j) * 3 + 2];
        best[q] = tpk_inf<T>();
        bgroup[q] = 0;
    }
    TPK_WORK_DECL

    for (int base = 0; base < nc; base += CH_TILE)
    {
        const int cnt = min(CH_TILE, nc - base);
        __syncthreads(); // the previous tile has been consumed by every wave
        for (int t = tid; t < CH_TILE; t += CH_THREADS)
        {
            Point4<T> p;
            if (t < cnt)
            {
                const T* src = cs + static_cast<int64_t>(base + t) * 3;
                p.x = src[0];
                p.y = src[1];
                p.z = src[2];
            }
            else
            {
                // Padding: an infinitely distant point never lowers a minimum.
                p.x = p.y = p.z = tpk_inf<T>();
            }
            p.w = 0;
            tile[t] = p;
        }
        __syncthreads();

        const int cnt_groups = (cnt + CH_CHUNK - 1) / CH_CHUNK;
        for (int g = 0; g < cnt_groups; ++g)
        {
            T mn[Q];
#pragma unroll
            for (int c = 0; c < CH_CHUNK; ++c)
            {
                const Point4<T> p = tile[g * CH_CHUNK + c];
#pragma unroll
                for (int q = 0; q < Q; ++q)
                {
                    // Operand order of the reference: (scanned - query), squares summed x,y,z.
                    const T d = tpk_dist2(p.x, p.y, p.z, qx[q], qy[q], qz[q]);
                    mn[q] = c == 0 ? d : tpk_min(mn[q], d);
                }
            }
            TPK_WORK_ADD(CH_CHUNK * Q);
            const int group = base / CH_CHUNK + g;
#pragma unroll
            for (int q = 0; q < Q; ++q)
            {
                const bool better = mn[q] < best[q];
                best[q] = better ? mn[q] : best[q];
                bgroup[q] = better ? group : bgroup[q];
            }
        }
    }

    TPK_WORK_FLUSH
    // Recover the index: first candidate of the winning group whose distance equals the
    // minimum (re-evaluated with the same operations, hence the same bits).
#pragma unroll
    for (int q = 0; q < Q; ++q)
    {
        const int j = j0 + q * CH_THREADS;
        if (j >= nq)
            continue;
        T bd = best[q];
        int bi = bgroup[q] * CH_CHUNK;
        if (nc == 0)
        {
            bd = 0;
            bi = 0;
        }
        else
        {
            const int k0 = bgroup[q] * CH_CHUNK;
            bool found = false;
#pragma unroll
            for (int c = 0; c < CH_CHUNK; ++c)
            {
                const int k = k0 + c;
                if (k < nc)
                {
                    const T* src = cs + static_cast<int64_t>(k) * 3;
                    const T d = tpk_dist2(src[0], src[1], src[2], qx[q], qy[q], qz[q]);
                    if (!found && d == bd)
                    {
                        found = true;
                        bi = k;
                    }
                }
            }
        }
        dout[j] = bd;
        iout[j] = bi;
    }
}

// Own term of every point: grad[j] = 2 * grad_dist[j] * (p[j] - other[idx[j]]), stored.
template <typename T>
__global__ __launch_bounds__(256) void chamfer_bwd_own_kernel(
    int64_t total1, int64_t total2, int n, int m, const T* __restrict__ xyz1,
    const T* __restrict__ xyz2, const int32_t* __restrict__ idx1,
    const int32_t* __restrict__ idx2, const T* __restrict__ grad_dist1,
    const T* __restrict__ grad_dist2, T* __restrict__ grad_xyz1, T* __restrict__ grad_xyz2)
{
    int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (; t < total1 + total2; t += stride)
    {
        const bool second = t >= total1;
        const int64_t p = second ? t - total1 : t; // flat point number (cloud * npts + j)
        const int npts = second ? m : n;
        const int nother = second ? n : m;
        const int64_t cloud = p / npts;
        const T* a = (second ? xyz2 : xyz1) + p * 3;
        const int j2 = (second ? idx2 : idx1)[p];
        const T* o = (second ? xyz1 : xyz2) + (cloud * nother + j2) * 3;
        const T g = (second ? grad_dist2 : grad_dist1)[p] * 2;
        T* out = (second ? grad_xyz2 : grad_xyz1) + p * 3;
        out[0] = g * (a[0] - o[0]);
        out[1] = g * (a[1] - o[1]);
        out[2] = g * (a[2] - o[2]);
    }
}

// Scattered term: grad_other[idx[j]] += -(2 * grad_dist[j] * (p[j] - other[idx[j]])).
template <typename T>
__global__ __launch_bounds__(256) void chamfer_bwd_scatter_kernel(
    int64_t total1, int64_t total2, int n, int m, const T* __restrict__ xyz1,
    const T* __restrict__ xyz2, const int32_t* __restrict__ idx1,
    const int32_t* __restrict__ idx2, const T* __restrict__ grad_dist1,
    const T* __restrict__ grad_dist2, T* grad_xyz1, T* grad_xyz2)
{
    int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (; t < total1 + total2; t += stride)
    {
        const bool second = t >= total1;
        const int64_t p = second ? t - total1 : t;
        const int npts = second ? m : n;
        const int nother = second ? n : m;
        const int64_t cloud = p / npts;
        const T* a = (second ? xyz2 : xyz1) + p * 3;
        const int j2 = (second ? idx2 : idx1)[p];
        const int64_t op = cloud * nother + j2;
        const T* o = (second ? xyz1 : xyz2) + op * 3;
        const T g = (second ? grad_dist2 : grad_dist1)[p] * 2;
        T* out = (second ? grad_xyz1 : grad_xyz2) + op * 3;
        unsafeAtomicAdd(out + 0, -(g * (a[0] - o[0])));
        unsafeAtomicAdd(out + 1, -(g * (a[1] - o[1])));
        unsafeAtomicAdd(out + 2, -(g * (a[2] - o[2])));
    }
}

// Backward without float atomics and without workspace.  A workgroup owns a range of points
// ("targets") of one cloud of one pair.  It first threads the points of the OTHER cloud that
// chose one of its targets as nearest neighbour into per-target chains held in LDS: one LDS
// integer exchange per point (head[target] <- entry, next[entry] <- old head).  Then one lane per
// target adds the target's own term and walks its chain (most chains hold zero to two points).
// Every output is written once, nothing is zero-filled.  The order of a chain is the order in
// which the exchanges happened to be served, so - as with the reference's atomics - the sum of
// a point with several terms may differ in the last bits from run to run.
//
// What a chain holds: the workgroup reads the other cloud's indices in order anyway, so for a point that chose one
// of its targets it reads the point's coordinates and gradient in the same pass - consecutive addresses - and
// keeps them in LDS as the chain's entry (x, y, z, 2 g; next).  The walk then reads LDS only, and the one
// scattered read per target that remains is the target's own nearest point.  (Entries that name the other
// cloud's points, their coordinates and gradients fetched during the walk, were the first version: four scattered
// 4- and 12-byte reads per target, and a compute unit serves a scattered read at about 1.7 clocks per lane
// whatever its width - 8800 of 10500 clocks per 1024 targets.)  A range's share of the other cloud is about
// range / points of it; room is kept for `capacity` entries, and a workgroup that meets more (a range that
// much of the other cloud chose) builds chains of point numbers instead, as before.
// dynamic LDS: lds_ints ints.
constexpr int CHB_THREADS = 1024;
constexpr int CHB_LDS_INTS = 38912; // 152 KiB

// LDS words of one entry: four values and the link.
template <typename T>
constexpr int chb_entry_ints()
{
    return 4 * static_cast<int>(sizeof(T) / sizeof(int)) + 1;
}

template <typename T>
__global__ __launch_bounds__(CHB_THREADS) void chamfer_bwd_chains_kernel(
    int n, int m, int clouds, int splits, int range1, int range2, int lds_ints, const T* __restrict__ xyz1,
    const T* __restrict__ xyz2, const int32_t* __restrict__ idx1, const int32_t* __restrict__ idx2,
    const T* __restrict__ grad_dist1, const T* __restrict__ grad_dist2, T* __restrict__ grad_xyz1,
    T* __restrict__ grad_xyz2)
{
    extern __shared__ __align__(16) int chain_lds[];
    __shared__ int entries; // entries asked for (may exceed the room)
    // logical workgroup = ((cloud * 2 + direction) * splits + split); those of a pair run on one
    // die, whose L2 then serves the random reads into the pair's points
    const int lin = static_cast<int>(xcd_local_block(blockIdx.x, gridDim.x));
    const int cloud = lin / (2 * splits);
    const int rem = lin - cloud * 2 * splits;
    const bool second = rem >= splits;
    const int split = second ? rem - splits : rem;
    const int npts = second ? m : n;
    const int nother = second ? n : m;
    const int range = second ? range2 : range1;
    const int t0 = split * range;
    const int t1 = min(t0 + range, npts);
    if (t0 >= t1)
        return; // (the whole workgroup: no barrier has been passed yet)
    const int tid = threadIdx.x;
    const T* __restrict__ own = (second ? xyz2 : xyz1) + static_cast<int64_t>(cloud) * npts * 3;
    const T* __restrict__ other = (second ? xyz1 : xyz2) + static_cast<int64_t>(cloud) * nother * 3;
    const int32_t* __restrict__ own_idx = (second ? idx2 : idx1) + static_cast<int64_t>(cloud) * npts;
    const int32_t* __restrict__ other_idx = (second ? idx1 : idx2) + static_cast<int64_t>(cloud) * nother;
    const T* __restrict__ own_g = (second ? grad_dist2 : grad_dist1) + static_cast<int64_t>(cloud) * npts;
    const T* __restrict__ other_g = (second ? grad_dist1 : grad_dist2) + static_cast<int64_t>(cloud) * nother;
    T* __restrict__ out = (second ? grad_xyz2 : grad_xyz1) + static_cast<int64_t>(cloud) * npts * 3;

    // entries in LDS: values [capacity][4], links [capacity], heads [range]
    const int capacity = min(nother, (lds_ints - range) / chb_entry_ints<T>());
    T* const values = reinterpret_cast<T*>(chain_lds);
    int* const links = chain_lds + capacity * (chb_entry_ints<T>() - 1);
    int* head = links + capacity;
    for (int t = tid; t < t1 - t0; t += CHB_THREADS)
        head[t] = -1;
    if (tid == 0)
        entries = 0;
    __syncthreads();
    constexpr int BATCH = 8; // index loads in flight per thread
    for (int j0 = tid; j0 < nother; j0 += BATCH * CHB_THREADS)
    {
        int k[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
        {
            const int j = j0 + u * CHB_THREADS;
            k[u] = j < nother ? other_idx[j] : -1;
        }
        // (read by every lane, wanted or not: a wavefront's 64 consecutive points cost a few lines, where reads
        // under the test cost as much as scattered ones - a lane at a time)
        T ox[BATCH], oy[BATCH], oz[BATCH], og[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
        {
            const int j = min(j0 + u * CHB_THREADS, nother - 1);
            ox[u] = other[j * 3 + 0];
            oy[u] = other[j * 3 + 1];
            oz[u] = other[j * 3 + 2];
            og[u] = other_g[j] * 2;
        }
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
            if (k[u] >= t0 && k[u] < t1)
            {
                // (one request per entry: a request for all of a lane's entries of the batch at once - lanes
                // asking for different numbers - was slower, 20 against 15.5 us)
                const int e = atomicAdd(&entries, 1);
                if (e < capacity)
                {
                    links[e] = atomicExch(&head[k[u] - t0], e);
                    values[e * 4 + 0] = ox[u];
                    values[e * 4 + 1] = oy[u];
                    values[e * 4 + 2] = oz[u];
                    values[e * 4 + 3] = og[u];
                }
            }
    }
    __syncthreads();
    const bool in_lds = entries <= capacity;
    int* const next = chain_lds; // (chains of point numbers: links [nother], heads [range])
    if (!in_lds)
    {
        __syncthreads(); // (every wavefront has read the count)
        head = chain_lds + nother;
        for (int t = tid; t < t1 - t0; t += CHB_THREADS)
            head[t] = -1;
        __syncthreads();
        for (int j0 = tid; j0 < nother; j0 += BATCH * CHB_THREADS)
        {
            int k[BATCH];
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
            {
                const int j = j0 + u * CHB_THREADS;
                k[u] = j < nother ? other_idx[j] : -1;
            }
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
                if (k[u] >= t0 && k[u] < t1)
                {
                    const int j = j0 + u * CHB_THREADS;
                    next[j] = atomicExch(&head[k[u] - t0], j);
                }
        }
        __syncthreads();
    }
    if (in_lds)
    {
        // Several targets per lane at a time, so that their dependent reads (own index -> that point) travel together.
        constexpr int TPT = 4;
        for (int kb = t0 + tid; kb < t1; kb += TPT * CHB_THREADS)
        {
            T px[TPT], py[TPT], pz[TPT], g[TPT];
            int j2[TPT], j[TPT];
#pragma unroll
            for (int u = 0; u < TPT; ++u)
            {
                const int k = min(kb + u * CHB_THREADS, t1 - 1);
                px[u] = own[k * 3 + 0];
                py[u] = own[k * 3 + 1];
                pz[u] = own[k * 3 + 2];
                j2[u] = own_idx[k];
                g[u] = own_g[k] * 2;
                j[u] = kb + u * CHB_THREADS < t1 ? head[k - t0] : -1;
            }
            T qx[TPT], qy[TPT], qz[TPT];
#pragma unroll
            for (int u = 0; u < TPT; ++u)
            {
                qx[u] = other[j2[u] * 3 + 0];
                qy[u] = other[j2[u] * 3 + 1];
                qz[u] = other[j2[u] * 3 + 2];
            }
#pragma unroll
            for (int u = 0; u < TPT; ++u)
            {
                T ax = g[u] * (px[u] - qx[u]);
                T ay = g[u] * (py[u] - qy[u]);
                T az = g[u] * (pz[u] - qz[u]);
                int e = j[u];
                while (e >= 0)
                {
                    const T vx = values[e * 4 + 0], vy = values[e * 4 + 1], vz = values[e * 4 + 2], vg = values[e * 4 + 3];
                    e = links[e];
                    ax = ax + -(vg * (vx - px[u]));
                    ay = ay + -(vg * (vy - py[u]));
                    az = az + -(vg * (vz - pz[u]));
                }
                const int k = kb + u * CHB_THREADS;
                if (k < t1)
                {
                    out[k * 3 + 0] = ax;
                    out[k * 3 + 1] = ay;
                    out[k * 3 + 2] = az;
                }
            }
        }
        return;
    }
    for (int k = t0 + tid; k < t1; k += CHB_THREADS)
    {
        const T px = own[k * 3 + 0], py = own[k * 3 + 1], pz = own[k * 3 + 2];
        const int j2 = own_idx[k];
        const T g = own_g[k] * 2;
        int j = head[k - t0];
        T ax = g * (px - other[j2 * 3 + 0]);
        T ay = g * (py - other[j2 * 3 + 1]);
        T az = g * (pz - other[j2 * 3 + 2]);
        {
            // The chains are followed in LDS first, CHAIN links at a time, and the points they name are
            // requested together: the reads from memory do not wait for one another.
            constexpr int CHAIN = 2;
            while (j >= 0)
            {
                int link[CHAIN];
#pragma unroll
                for (int l = 0; l < CHAIN; ++l)
                {
                    link[l] = j;
                    j = j >= 0 ? next[j] : -1;
                }
                T gj[CHAIN], ox[CHAIN], oy[CHAIN], oz[CHAIN];
#pragma unroll
                for (int l = 0; l < CHAIN; ++l)
                {
                    const int jj = link[l] >= 0 ? link[l] : 0;
                    gj[l] = other_g[jj] * 2;
                    ox[l] = other[jj * 3 + 0];
                    oy[l] = other[jj * 3 + 1];
                    oz[l] = other[jj * 3 + 2];
                }
#pragma unroll
                for (int l = 0; l < CHAIN; ++l)
                    if (link[l] >= 0)
                    {
                        ax = ax + -(gj[l] * (ox[l] - px));
                        ay = ay + -(gj[l] * (oy[l] - py));
                        az = az + -(gj[l] * (oz[l] - pz));
                    }
            }
        }
        out[k * 3 + 0] = ax;
        out[k * 3 + 1] = ay;
        out[k * 3 + 2] = az;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void fill_zero_kernel(T* p, int64_t count)
{
    int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (; t < count; t += stride)
        p[t] = 0;
}

template <typename T, int Q>
int launch_fwd(int b, int n, int m, const T* xyz1, const T* xyz2, T* dist1, T* dist2,
               int32_t* idx1, int32_t* idx2, hipStream_t s)
{
    const int64_t bpc1 = tpk_ceil_div(n, CH_THREADS * Q);
    const int64_t bpc2 = tpk_ceil_div(m, CH_THREADS * Q);
    const int64_t blocks1 = bpc1 * b;
    const int64_t blocks2 = bpc2 * b;
    if (blocks1 + blocks2 > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    if (blocks1 + blocks2 == 0)
        return TPK_OK;
    hipLaunchKernelGGL((chamfer_fwd_kernel<T, Q>), dim3(static_cast<unsigned>(blocks1 + blocks2)),
                       dim3(CH_THREADS), 0, s, n, m, static_cast<int>(bpc1 ? bpc1 : 1),
                       static_cast<int>(bpc2 ? bpc2 : 1), static_cast<int>(blocks1), xyz1, xyz2,
                       dist1, dist2, idx1, idx2);
    return tpk_launch_status();
}

template <typename T>
int chamfer_fwd(int b, int n, int m, const T* xyz1, const T* xyz2, T* dist1, T* dist2,
                int32_t* idx1, int32_t* idx2, void* stream)
{
    if (b < 0 || n < 0 || m < 0)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || (n == 0 && m == 0))
        return TPK_OK;
    if ((n > 0 && (!xyz1 || !dist1 || !idx1)) || (m > 0 && (!xyz2 || !dist2 || !idx2)))
        return TPK_ERR_INVALID_ARG;
    hipStream_t s = tpk_stream(stream);
    const int64_t queries = static_cast<int64_t>(b) * (static_cast<int64_t>(n) + m);
    if (queries >= 4LL * CH_THREADS * 1024)
        return launch_fwd<T, 4>(b, n, m, xyz1, xyz2, dist1, dist2, idx1, idx2, s);
    if (queries >= 2LL * CH_THREADS * 1024)
        return launch_fwd<T, 2>(b, n, m, xyz1, xyz2, dist1, dist2, idx1, idx2, s);
    return launch_fwd<T, 1>(b, n, m, xyz1, xyz2, dist1, dist2, idx1, idx2, s);
}

template <typename T>
int chamfer_bwd(int b, int n, int m, const T* xyz1, const T* xyz2, const int32_t* idx1,
                const int32_t* idx2, const T* grad_dist1, const T* grad_dist2, T* grad_xyz1,
                T* grad_xyz2, void* workspace, size_t workspace_bytes, void* stream)
{
    if (b < 0 || n < 0 || m < 0)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || (n == 0 && m == 0))
        return TPK_OK;
    if ((n > 0 && (!xyz1 || !idx1 || !grad_dist1 || !grad_xyz1)) ||
        (m > 0 && (!xyz2 || !idx2 || !grad_dist2 || !grad_xyz2)))
        return TPK_ERR_INVALID_ARG;
    hipStream_t s = tpk_stream(stream);
    const int64_t total1 = static_cast<int64_t>(b) * n;
    const int64_t total2 = static_cast<int64_t>(b) * m;
    if (n == 0 || m == 0)
    {
        // One cloud is empty: no pairs exist; the reference returns its zero-initialised
        // gradients.
        const int64_t count = (total1 + total2) * 3;
        T* p = n == 0 ? grad_xyz2 : grad_xyz1;
        const unsigned blocks = static_cast<unsigned>(tpk_min64(tpk_ceil_div(count, 256), 4096));
        hipLaunchKernelGGL(fill_zero_kernel<T>, dim3(blocks), dim3(256), 0, s, p, count);
        return tpk_launch_status();
    }
    (void)workspace;
    (void)workspace_bytes;
    // Chains in LDS (no workspace): as many target ranges per cloud as give every compute unit one
    // workgroup and none a second (config 5: 256 workgroups 19.7 us, 320 or 1024: 24 us, 512: 20.4 us),
    // each of at least 1024 targets; clouds too large for LDS scatter with atomics.
    {
        const int larger = n > m ? n : m;
        int splits = TPK_COMPUTE_UNITS / (2 * b);
        const int most = static_cast<int>(tpk_ceil_div(larger, CHB_THREADS));
        splits = splits > most ? most : splits;
        splits = splits < 1 ? 1 : splits;
        while (larger + tpk_ceil_div(larger, splits) > CHB_LDS_INTS && splits < most)
            ++splits;
        // (room for the entries a range expects - its share of the other cloud - and a third more)
        auto with_entries = [&](int parts) {
            const int64_t range = tpk_ceil_div(larger, parts);
            return range + chb_entry_ints<T>() * (range + range / 3 + 64);
        };
        while (with_entries(splits) > CHB_LDS_INTS && splits < most)
            ++splits;
        const int range1 = static_cast<int>(tpk_ceil_div(n, splits)), range2 = static_cast<int>(tpk_ceil_div(m, splits));
        const int range = range1 > range2 ? range1 : range2;
        const int64_t groups = 2 * static_cast<int64_t>(b) * splits;
        if (larger + range <= CHB_LDS_INTS && groups <= 0x7fffffffLL && static_cast<int64_t>(larger) * 3 <= 0x7fffffffLL)
        {
            // every point of the other cloud as an entry where that fits; else all of the LDS
            const int64_t all = range + static_cast<int64_t>(chb_entry_ints<T>()) * larger;
            const int lds_ints = static_cast<int>(all <= CHB_LDS_INTS ? (all > larger + range ? all : larger + range) : CHB_LDS_INTS);
            const size_t lds = static_cast<size_t>(lds_ints) * sizeof(int);
            const int allowed = allow_lds(chamfer_bwd_chains_kernel<T>, lds);
            if (allowed != TPK_OK)
                return allowed;
            hipLaunchKernelGGL(chamfer_bwd_chains_kernel<T>, dim3(static_cast<unsigned>(groups)), dim3(CHB_THREADS), lds, s,
                               n, m, b, splits, range1, range2, lds_ints, xyz1, xyz2, idx1, idx2, grad_dist1, grad_dist2,
                               grad_xyz1, grad_xyz2);
            return tpk_launch_status();
        }
    }
    const unsigned blocks =
        static_cast<unsigned>(tpk_min64(tpk_ceil_div(total1 + total2, 256), 1 << 20));
    hipLaunchKernelGGL(chamfer_bwd_own_kernel<T>, dim3(blocks), dim3(256), 0, s, total1, total2,
                       n, m, xyz1, xyz2, idx1, idx2, grad_dist1, grad_dist2, grad_xyz1,
                       grad_xyz2);
    int st = tpk_launch_status();
    if (st != TPK_OK)
        return st;
    hipLaunchKernelGGL(chamfer_bwd_scatter_kernel<T>, dim3(blocks), dim3(256), 0, s, total1,
                       total2, n, m, xyz1, xyz2, idx1, idx2, grad_dist1, grad_dist2, grad_xyz1,
                       grad_xyz2);
    return tpk_launch_status();
}

} // namespace

extern "C" size_t tpk_chamfer_fwd_workspace_bytes(int b, int n, int m)
{
    return tpk_grid_chamfer_workspace_bytes(b, n, m);
}

extern "C" int tpk_chamfer_fwd_f32(int b, int n, int m, const float* xyz1, const float* xyz2,
                                   float* dist1, float* dist2, int32_t* idx1, int32_t* idx2,
                                   void* workspace, size_t workspace_bytes, void* stream)
{
    if (workspace && b > 0 && n > 0 && m > 0 && xyz1 && xyz2 && dist1 && dist2 && idx1 && idx2)
    {
        // Search over curve-ordered cells where it applies; otherwise all pairs.
        const int st = tpk_grid_chamfer_fwd(b, n, m, xyz1, xyz2, dist1, dist2, idx1, idx2, workspace,
                                            workspace_bytes, tpk_stream(stream));
        if (st != TPK_ERR_UNSUPPORTED)
            return st;
    }
    return chamfer_fwd<float>(b, n, m, xyz1, xyz2, dist1, dist2, idx1, idx2, stream);
}

extern "C" int tpk_chamfer_fwd_f64(int b, int n, int m, const double* xyz1, const double* xyz2,
                                   double* dist1, double* dist2, int32_t* idx1, int32_t* idx2,
                                   void* stream)
{
    return chamfer_fwd<double>(b, n, m, xyz1, xyz2, dist1, dist2, idx1, idx2, stream);
}

extern "C" int tpk_chamfer_bwd_f32(int b, int n, int m, const float* xyz1, const float* xyz2,
                                   const int32_t* idx1, const int32_t* idx2,
                                   const float* grad_dist1, const float* grad_dist2,
                                   float* grad_xyz1, float* grad_xyz2, void* workspace,
                                   size_t workspace_bytes, void* stream)
{
    return chamfer_bwd<float>(b, n, m, xyz1, xyz2, idx1, idx2, grad_dist1, grad_dist2, grad_xyz1,
                            grad_xyz2, workspace, workspace_bytes, stream);
}

extern "C" int tpk_chamfer_bwd_f64(int b, int n, int m, const double* xyz1, const double* xyz2,
                                   const int32_t* idx1, const int32_t* idx2,
                                   const double* grad_dist1, const double* grad_dist2,
                                   double* grad_xyz1, double* grad_xyz2, void* workspace,
                                   size_t workspace_bytes, void* stream)
{
    return chamfer_bwd<double>(b, n, m, xyz1, xyz2, idx1, idx2, grad_dist1, grad_dist2, grad_xyz1,
                            grad_xyz2, workspace, workspace_bytes, stream);
}

extern "C" size_t tpk_chamfer_bwd_workspace_bytes(int b, int n, int m)
{
    (void)b;
    (void)n;
    (void)m;
    return 0; // the backward pass keeps its chains in LDS
}
