// three_nn: for every "unknown" point the three nearest "known" points of the same cloud.
//
// Work split: one lane owns Q query points and keeps their running best three (distance,
// index) in registers; the known points of the cloud stream through LDS in tiles of
// float4 (x, y, z, pad), so every lane of a wavefront reads the same LDS address at the
// same time (a broadcast read, no bank conflicts) and one LDS read feeds Q distance
// evaluations.  Insertion into the sorted triple happens only in lanes whose distance
// beats their current third best, which after the first few hundred candidates is rare.
//
// Semantics follow the reference kernel (cuda/src/interpolate_gpu.cu:9-65): candidates are
// visited in index order and replace an entry only when strictly smaller, so equal
// distances keep the lower index first.  The reference holds its running bests as doubles
// initialised to 1e40; every distance is an fp32 value, so fp32 running bests initialised
// to +inf select identically and store identical values.
#include "lds_grid.h"
#include "nn_grid.h"

#include <algorithm>
#include <mutex>

namespace {

constexpr int NN_THREADS = 256;
constexpr int NN_TILE = 1024; // known points per LDS tile (16 KiB)

template <int Q>
__global__ __launch_bounds__(NN_THREADS) void three_nn_kernel(
    int n, int m, int blocks_per_cloud, const float* __restrict__ unknown,
    const float* __restrict__ known, float* __restrict__ dist2, int32_t* __restrict__ idx)
{
    __shared__ float4 tile[NN_TILE];

    const int cloud = blockIdx.x / blocks_per_cloud;
    const int blk = blockIdx.x - cloud * blocks_per_cloud;
    unknown += static_cast<int64_t>(cloud) * n * 3;
    known += static_cast<int64_t>(cloud) * m * 3;
    dist2 += static_cast<int64_t>(cloud) * n * 3;
    idx += static_cast<int64_t>(cloud) * n * 3;

    const int tid = threadIdx.x;
    const int j0 = blk * (NN_THREADS * Q) + tid;

    float ux[Q], uy[Q], uz[Q];
    float b1[Q], b2[Q], b3[Q];
    int i1[Q], i2[Q], i3[Q];
#pragma unroll
    for (int q = 0; q < Q; ++q)
    {
        int j = j0 + q * NN_THREADS;
        j = j < n ? j : n - 1; // lanes past the end shadow the last query and store nothing
        ux[q] = unknown[j * 3 + 0];
        uy[q] = unknown[j * 3 + 1];
        uz[q] = unknown[j * 3 + 2];
        b1[q] = b2[q] = b3[q] = __builtin_inff();
        i1[q] = i2[q] = i3[q] = 0;
    }
    TPK_WORK_DECL

    for (int base = 0; base < m; base += NN_TILE)
    {
        const int cnt = min(NN_TILE, m - base);
        __syncthreads(); // the previous tile has been consumed by every wave
        for (int t = tid; t < NN_TILE; t += NN_THREADS)
        {
            float4 p;
            if (t < cnt)
            {
                const float* src = known + static_cast<int64_t>(base + t) * 3;
                p = make_float4(src[0], src[1], src[2], 0.f);
            }
            else
            {
                // Padding: an infinitely distant point never beats a running best.
                p = make_float4(__builtin_inff(), __builtin_inff(), __builtin_inff(), 0.f);
            }
            tile[t] = p;
        }
        __syncthreads();

        const int cnt4 = (cnt + 3) & ~3;
        TPK_WORK_ADD(cnt4 * Q);
#pragma unroll 4
        for (int k = 0; k < cnt4; ++k)
        {
            const float4 c = tile[k];
            const int kk = base + k;
#pragma unroll
            for (int q = 0; q < Q; ++q)
            {
                const float d = tpk_dist2(ux[q], uy[q], uz[q], c.x, c.y, c.z);
                if (d < b3[q])
                {
                    // Sorted insert written as selects: one short block, no nested divergence.
                    const bool lt1 = d < b1[q];
                    const bool lt2 = d < b2[q];
                    b3[q] = lt2 ? b2[q] : d;
                    i3[q] = lt2 ? i2[q] : kk;
                    b2[q] = lt1 ? b1[q] : (lt2 ? d : b2[q]);
                    i2[q] = lt1 ? i1[q] : (lt2 ? kk : i2[q]);
                    b1[q] = lt1 ? d : b1[q];
                    i1[q] = lt1 ? kk : i1[q];
                }
            }
        }
    }

    TPK_WORK_FLUSH
#pragma unroll
    for (int q = 0; q < Q; ++q)
    {
        const int j = j0 + q * NN_THREADS;
        if (j < n)
        {
            dist2[j * 3 + 0] = b1[q];
            dist2[j * 3 + 1] = b2[q];
            dist2[j * 3 + 2] = b3[q];
            idx[j * 3 + 0] = i1[q];
            idx[j * 3 + 1] = i2[q];
            idx[j * 3 + 2] = i3[q];
        }
    }
}

template <int Q>
int launch_three_nn(int b, int n, int m, const float* unknown, const float* known, float* dist2,
                    int32_t* idx, hipStream_t stream)
{
    const int64_t blocks_per_cloud = tpk_ceil_div(n, NN_THREADS * Q);
    const int64_t blocks = blocks_per_cloud * b;
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(three_nn_kernel<Q>, dim3(static_cast<unsigned>(blocks)), dim3(NN_THREADS),
                       0, stream, n, m, static_cast<int>(blocks_per_cloud), unknown, known, dist2,
                       idx);
    return tpk_launch_status();
}

// ---------------------------------------------------------------------------------------------
// Known clouds of TNC_MIN_KNOWN .. TNC_MAX_KNOWN points: a grid in LDS (lds_grid.h), one lane per query.
//
// Every workgroup (16 wavefronts) sorts its cloud's known points into the cells of a grid in LDS; all workgroups
// of a cloud repeat this (a few microseconds; the cloud comes from the L2); no launch in front, no workspace, and
// the queries need no order.  Then every lane takes a query and walks the cells around it, keeping its best three
// (distance, index).  Selection by (distance, index) gives what the reference's scan in index order with
// strictly-smaller replacement gives (cuda/src/interpolate_gpu.cu:9-65) whatever the visiting order.
// ---------------------------------------------------------------------------------------------
constexpr int TNC_MIN_KNOWN = 1024;
constexpr int TNC_MAX_KNOWN = LG_MAX_POINTS;
constexpr float TNC_CROWDED = 12.0f; // points per cell, as a point sees them, from which the grid is given up

// The best three (squared distance, index) keys of a lane, ascending.  Unused entries are (inf, 0): no candidate
// at infinite distance, or with a NaN, is smaller.
struct Best3
{
    unsigned long long k1, k2, k3;
    __device__ __forceinline__ void clear() { k1 = k2 = k3 = lg_key(__builtin_inff(), 0); }
    __device__ __forceinline__ float bound() const { return __int_as_float(static_cast<int>(k3 >> 32)); }
    __device__ __forceinline__ void offer(unsigned long long k)
    {
        if (k < k3)
        {
            const bool lt1 = k < k1, lt2 = k < k2;
            k3 = lt2 ? k2 : k;
            k2 = lt1 ? k1 : (lt2 ? k : k2);
            k1 = lt1 ? k : k1;
        }
    }
};

__global__ __launch_bounds__(LG_THREADS) void three_nn_cells_kernel(
    int n, int m, int blocks_per_cloud, int queries_per_block, const float* __restrict__ unknown,
    const float* __restrict__ known, float* __restrict__ dist2, int32_t* __restrict__ idx, int* __restrict__ general)
{
    extern __shared__ __align__(16) unsigned char tnc_lds[];
    const int tid = threadIdx.x;
    const int cloud = blockIdx.x / blocks_per_cloud;
    const int blk = blockIdx.x - cloud * blocks_per_cloud;
    unknown += static_cast<int64_t>(cloud) * n * 3;
    known += static_cast<int64_t>(cloud) * m * 3;
    dist2 += static_cast<int64_t>(cloud) * n * 3;
    idx += static_cast<int64_t>(cloud) * n * 3;
    TPK_WORK_DECL

    LdsGrid grid;
    lds_grid_build(grid, tnc_lds, known, m, 0);
    // Points per cell as a point sees them (3 in a cloud of even density): above TNC_CROWDED the grid is a poor
    // fit - dense cells cost their queries many candidates, empty ones many steps of widening - and, where the
    // caller enqueues it behind this kernel, the search over curve-ordered cells answers the cloud instead.
    // Without it: on with the grid; when 40 points cost a lane what the whole cloud costs by broadcast reads,
    // every lane scans the cloud.
    if (general)
    {
        const bool hand_over = grid.crowd > TNC_CROWDED;
        if (blk == 0 && tid == 0)
            general[cloud] = hand_over ? 1 : 0;
        if (hand_over)
            return;
    }
    const bool crowded = grid.crowd * 40.0f > static_cast<float>(m);

    // ---- queries: one lane each, no workgroup barrier from here on ----
    const int q_end = min(n, (blk + 1) * queries_per_block);
    for (int j = blk * queries_per_block + tid; j < q_end; j += LG_THREADS)
    {
        const float qx = unknown[j * 3 + 0], qy = unknown[j * 3 + 1], qz = unknown[j * 3 + 2];
        Best3 best;
        best.clear();
        if (crowded)
            lds_grid_scan_all(grid, m, qx, qy, qz, best TPK_WORK_ARG);
        else
            lds_grid_search(grid, qx, qy, qz, best TPK_WORK_ARG);
        dist2[j * 3 + 0] = __int_as_float(static_cast<int>(best.k1 >> 32));
        dist2[j * 3 + 1] = __int_as_float(static_cast<int>(best.k2 >> 32));
        dist2[j * 3 + 2] = best.bound();
        idx[j * 3 + 0] = static_cast<int>(best.k1 & 0xFFFFFFFFu);
        idx[j * 3 + 1] = static_cast<int>(best.k2 & 0xFFFFFFFFu);
        idx[j * 3 + 2] = static_cast<int>(best.k3 & 0xFFFFFFFFu);
    }
    TPK_WORK_FLUSH
}

int launch_three_nn_cells(int b, int n, int m, const float* unknown, const float* known, float* dist2, int32_t* idx,
                          int* general, hipStream_t stream)
{
    // one workgroup per compute unit where the queries allow it (every workgroup sorts its cloud)
    const int64_t per_cloud = std::max<int64_t>(1, std::min<int64_t>(tpk_ceil_div(n, LG_THREADS), TPK_COMPUTE_UNITS / b));
    const int per_block = static_cast<int>(tpk_ceil_div(n, per_cloud));
    const int64_t bpc = tpk_ceil_div(n, per_block);
    if (bpc * b > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const size_t lds = lg_lds_bytes(m);
    const int st = tpk_allow_lds(reinterpret_cast<const void*>(&three_nn_cells_kernel), lds);
    if (st != TPK_OK)
        return st;
    hipLaunchKernelGGL(three_nn_cells_kernel, dim3(static_cast<unsigned>(bpc * b)), dim3(LG_THREADS), lds, stream, n, m,
                       static_cast<int>(bpc), per_block, unknown, known, dist2, idx, general);
    return tpk_launch_status();
}

} // namespace

extern "C" size_t tpk_three_nn_workspace_bytes(int b, int n, int m)
{
    return tpk_grid_three_nn_workspace_bytes(b, n, m);
}

extern "C" int tpk_three_nn_f32(int b, int n, int m, const float* unknown, const float* known,
                                float* dist2, int32_t* idx, void* workspace, size_t workspace_bytes,
                                void* stream)
{
    if (b < 0 || n < 0 || m < 0)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || n == 0)
        return TPK_OK;
    if (!unknown || !dist2 || !idx || (m > 0 && !known))
        return TPK_ERR_INVALID_ARG;
    if (static_cast<int64_t>(n) * 3 > 0x7fffffffLL || static_cast<int64_t>(m) * 3 > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipStream_t s = tpk_stream(stream);
    if (m >= TNC_MIN_KNOWN && m <= TNC_MAX_KNOWN)
    {
        // The known cloud fits in LDS: a grid there, one lane per query.  It notes the clouds it gives up (uneven
        // density) in the workspace, and the search over curve-ordered cells, enqueued behind it, answers those.
        int* const general = tpk_grid_three_nn_flags(b, n, m, workspace, workspace_bytes);
        const int st = launch_three_nn_cells(b, n, m, unknown, known, dist2, idx, general, s);
        if (st != TPK_OK || !general)
            return st;
        return tpk_grid_three_nn(b, n, m, unknown, known, dist2, idx, workspace, workspace_bytes, true, s);
    }
    if (workspace)
    {
        // Search over curve-ordered cells where it applies; otherwise all pairs.
        const int st = tpk_grid_three_nn(b, n, m, unknown, known, dist2, idx, workspace, workspace_bytes, false, s);
        if (st != TPK_ERR_UNSUPPORTED)
            return st;
    }
    return tpk_three_nn_all_pairs_f32(b, n, m, unknown, known, dist2, idx, stream);
}

extern "C" int tpk_three_nn_all_pairs_f32(int b, int n, int m, const float* unknown, const float* known,
                                          float* dist2, int32_t* idx, void* stream)
{
    if (b < 0 || n < 0 || m < 0)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || n == 0)
        return TPK_OK;
    if (!unknown || !dist2 || !idx || (m > 0 && !known))
        return TPK_ERR_INVALID_ARG;
    if (static_cast<int64_t>(n) * 3 > 0x7fffffffLL || static_cast<int64_t>(m) * 3 > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipStream_t s = tpk_stream(stream);
    // Queries per lane: as many as still leave a few workgroups per compute unit.
    const int64_t queries = static_cast<int64_t>(b) * n;
    if (queries >= 4LL * NN_THREADS * 2048)
        return launch_three_nn<4>(b, n, m, unknown, known, dist2, idx, s);
    if (queries >= 2LL * NN_THREADS * 2048)
        return launch_three_nn<2>(b, n, m, unknown, known, dist2, idx, s);
    return launch_three_nn<1>(b, n, m, unknown, known, dist2, idx, s);
}

// ---------------------------------------------------------------------------------------------
// three_nn for callers that may not allocate device memory (code under graph capture, serving
// loops, harnesses that forbid it).  The curve-ordered copy of both clouds and the cell boxes,
// which tpk_three_nn_f32 takes as a caller-provided workspace, live in a fixed array in device
// memory instead.  Every GPU the library runs on holds its own copy of the array at its own
// address until the process ends; that address is looked up once per device, with that device
// current, and host code uses the looked-up pointer only (the array's name is not a device
// address on the host).  The search overwrites whatever an earlier call left there (nothing has
// to start at zero), so calls that overlap on one GPU - on different streams or from different
// threads - race on it.
// ---------------------------------------------------------------------------------------------
namespace {

constexpr size_t THREE_NN_STATIC_BYTES = TPK_THREE_NN_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[THREE_NN_STATIC_BYTES];

constexpr int SCRATCH_MAX_DEVICES = 64;
std::mutex scratch_lock;
void* scratch_address[SCRATCH_MAX_DEVICES]; // per device, filled at the first call on that device

// Device address of `scratch` on the current device (looked up once per device).
int static_scratch(void** out)
{
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess)
        return static_cast<int>(e);
    if (device < 0 || device >= SCRATCH_MAX_DEVICES)
        return TPK_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (!scratch_address[device])
    {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess)
            return static_cast<int>(e);
        if (!p || (reinterpret_cast<uintptr_t>(p) & 255u))
            return TPK_ERR_WORKSPACE;
        scratch_address[device] = p;
    }
    *out = scratch_address[device];
    return TPK_OK;
}

} // namespace

extern "C" size_t tpk_three_nn_static_scratch_bytes(void)
{
    return THREE_NN_STATIC_BYTES;
}

extern "C" int tpk_three_nn_static_f32(int b, int n, int m, const float* unknown, const float* known,
                                       float* dist2, int32_t* idx, void* stream)
{
    if (b < 0 || n < 0 || m < 0)
        return TPK_ERR_INVALID_ARG;
    const size_t need = tpk_grid_three_nn_workspace_bytes(b, n, m);
    if (need > THREE_NN_STATIC_BYTES)
        return TPK_ERR_TOO_LARGE;
    if (need == 0) // shapes the cell search does not serve use no scratch memory at all
        return tpk_three_nn_f32(b, n, m, unknown, known, dist2, idx, nullptr, 0, stream);
    void* ptr = nullptr;
    const int st = static_scratch(&ptr);
    if (st != TPK_OK)
        return st;
    return tpk_three_nn_f32(b, n, m, unknown, known, dist2, idx, ptr, THREE_NN_STATIC_BYTES, stream);
}
