// Furthest point sampling: npoint-1 dependent rounds of "update every point's distance to
// the chosen set, pick the point whose distance is largest".
//
// One 1024-lane workgroup (16 wavefronts, one compute unit) owns a cloud for the whole
// call.  Up to 16 points per lane (16384 per cloud) stay in registers for all rounds -
// coordinates and running minimum distance - so a round touches no memory except one
// 24-byte LDS record per wavefront:
//   1. every lane updates its points against the last chosen point and keeps its first
//      largest value (strict >, points in ascending index order);
//   2. the wavefront finds its largest value with DPP row reductions + four lane reads,
//      picks the owning lane (ballot; the tie key below only when two lanes tie), and
//      lane 0 publishes (value, tie key, point index, x, y, z) of the winner to LDS;
//   3. after the round's single barrier every wavefront reduces the 16 records the same
//      way (16 records = one DPP row) and continues with the winner's coordinates taken
//      from the record: the chosen point is never re-read from memory.
// Records are double buffered so that one barrier per round suffices.
//
// Clouds that do not fit in registers use the same selection code over points streamed
// from global memory with the running minima in a caller-provided workspace.
//
// Semantics follow the reference kernel (cuda/src/sampling_gpu.cu:17-144): start at point
// 0; squared distances; points whose squared norm is <= 1e-3 are neither updated nor
// eligible; if no point is eligible the pick is 0.  Equal maxima resolve as its block
// reduction does: with BS = the reference's block size (largest power of two <= n, at
// most 512; cuda/include/cuda_utils.h:13-18), reference thread (k mod BS) keeps the lowest
// k among its own equal maxima, and the halving tree then prefers the thread whose number
// has the smaller bit-reversal.  Both rules together are "smallest tie key", with
//   key(k) = bitrev(k mod BS) * ceil(n / BS) + floor(k / BS).
#include "tpk_device.h"

#include <cmath>

namespace {

constexpr int FPS_THREADS = 1024;
constexpr int FPS_WAVES = FPS_THREADS / TPK_WAVE;
constexpr int FPS_MAX_PPT = 16; // points per lane kept in registers

struct WaveRecord
{
    int val;     // bits of the wavefront's largest distance (-1.0f: no eligible point)
    unsigned tk; // tie key of the point holding it
    int k;       // its index in the cloud
    float x, y, z;
};

// DPP controls: quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_ror:4, row_ror:8.  After the
// four steps every lane of a 16-lane row holds the row's result.
__device__ __forceinline__ int row_all_max_i32(int v)
{
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x124, 0xF, 0xF, true));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x128, 0xF, 0xF, true));
    return v;
}

__device__ __forceinline__ unsigned row_all_min_u32(unsigned v)
{
    v = min(v, static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true)));
    v = min(v, static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true)));
    v = min(v, static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, v, 0x124, 0xF, 0xF, true)));
    v = min(v, static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, v, 0x128, 0xF, 0xF, true)));
    return v;
}

__device__ __forceinline__ int wave_max_i32(int v)
{
    v = row_all_max_i32(v);
    const int a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
    const int c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
    return max(max(a, b), max(c, d));
}

__device__ __forceinline__ unsigned wave_min_u32(unsigned v)
{
    v = row_all_min_u32(v);
    const unsigned a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
    const unsigned c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
    return min(min(a, b), min(c, d));
}

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
                                               float& sx, float& sy, float& sz)
{
    const WaveRecord e = rec[lane & (WAVES - 1)];
    const int gv = __builtin_amdgcn_readfirstlane(row_all_max_i32(e.val));
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
        reduce_records<WAVES>(records[j & 1], lane, p0x, p0y, p0z, k, sx, sy, sz);
        if (tid == 0)
            out[j] = k;
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
        reduce_records<FPS_WAVES>(records[j & 1], lane, p0x, p0y, p0z, k, sx, sy, sz);
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

} // namespace

extern "C" size_t tpk_fps_workspace_bytes(int b, int n)
{
    if (b <= 0 || n <= FPS_THREADS * FPS_MAX_PPT)
        return 0;
    return static_cast<size_t>(b) * static_cast<size_t>(n) * sizeof(float);
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

    if (n <= FPS_THREADS * 1)
        launch_resident<1, FPS_THREADS>(b, n, npoint, log2_bs, groups, xyz, idx_out, s);
    else if (n <= FPS_THREADS * 2)
        launch_resident<2, FPS_THREADS>(b, n, npoint, log2_bs, groups, xyz, idx_out, s);
    else if (n <= FPS_THREADS * 4)
        launch_resident<4, FPS_THREADS>(b, n, npoint, log2_bs, groups, xyz, idx_out, s);
    else if (n <= FPS_THREADS * 8)
        launch_resident<8, FPS_THREADS>(b, n, npoint, log2_bs, groups, xyz, idx_out, s);
    else if (n <= FPS_THREADS * 16)
        // 8 wavefronts x 32 points per lane: the per-round selection work is paid by half as
        // many wavefronts as with 16 x 16 (measured 6.20 ms against 6.35 ms per batch of 16 clouds)
        launch_resident<32, 512>(b, n, npoint, log2_bs, groups, xyz, idx_out, s);
    else
    {
        const size_t need = tpk_fps_workspace_bytes(b, n);
        if (!workspace || workspace_bytes < need)
            return TPK_ERR_WORKSPACE;
        hipLaunchKernelGGL(fps_streaming_kernel, dim3(b), dim3(FPS_THREADS), 0, s, n, npoint,
                           log2_bs, groups, xyz, static_cast<float*>(workspace), idx_out);
    }
    return tpk_launch_status();
}
