// Bandwidth-bound gathers and their scatter-add backward passes:
//   three_interpolate      out[b,c,j] = sum_t points[b,c,idx[b,j,t]] * weight[b,j,t]   (K=3)
//   grouping_operation     out[b,c,j] = features[b,c,idx[b,j]]  (j = p*nsample + s)     (K=1)
//
// The source of a gather is one feature row (b, c, :) of m floats, and every output column
// j uses the same K positions in each of the c rows of its cloud.  A workgroup therefore
// stages R whole rows of one cloud in LDS (R*m*4 bytes, up to 128 KiB of the 160 KiB a
// gfx950 workgroup may use), reads the (idx, weight) of a column once and serves the
// K*R random reads from LDS; global memory sees only streaming traffic: rows in once,
// (idx, weight) once per row block, outputs written once, consecutive lanes writing
// consecutive columns.
//
// Backward.  Scattering grad_out into the rows needs float accumulation at random positions;
// LDS float atomics are far too slow on gfx950 for that (a wavefront-wide ds_add_f32 takes
// about 190 cycles whatever the address pattern, against 8 for a random LDS read), so the
// scatter is turned into a gather: a first kernel inverts the index of each cloud into
// per-target lists (for target position i the columns j that reference it, with their
// weights) using LDS *integer* atomics, which are fast, and an LDS prefix sum; the main
// kernel then stages R rows of grad_out in LDS (rows of n floats) and sums, for every
// target, the listed columns - 16 lanes share one target, read 16 list entries at a time
// (one contiguous 128-byte piece) and combine with a DPP row reduction.  No float atomics,
// no zero fill, each output written once.  The lists cost 8 bytes (4 unweighted) per index
// entry of workspace, passed in by the caller.  The order in which a target's terms are
// added differs from run to run only through the order of its list, as with the
// reference's global atomics (cuda/src/interpolate_gpu.cu:122-152): results agree to
// rounding.
//
// Rows too long for LDS, or a call without workspace, take a direct path: gathers from
// global memory (forward), zero fill + global float atomics (backward).
//
// Forward arithmetic follows cuda/src/interpolate_gpu.cu:78-107: ((p1*w1) + (p2*w2)) +
// (p3*w3), every operation rounded on its own.  The grouping forward is a pure copy
// (torch_points_kernels/torchpoints.py:129-146 expresses it as torch.gather).
#include "lists.h"

namespace {

constexpr int G_MAX_ROWS = 8;
constexpr int G_LDS_BUDGET = 131072; // bytes of LDS for the staged rows

template <int K, bool WEIGHTED, typename IdxT>
struct Column
{
    int i[K];
    float w[K];

    __device__ __forceinline__ void load(const IdxT* __restrict__ idx,
                                         const float* __restrict__ weight, int64_t j)
    {
#pragma unroll
        for (int t = 0; t < K; ++t)
        {
            i[t] = static_cast<int>(idx[j * K + t]);
            w[t] = WEIGHTED ? weight[j * K + t] : 1.0f;
        }
    }

    // Value of this column in the row starting at `row` (LDS or global memory).
    __device__ __forceinline__ float combine(const float* row) const
    {
        if (!WEIGHTED)
            return row[i[0]];
        float acc = row[i[0]] * w[0];
#pragma unroll
        for (int t = 1; t < K; ++t)
            acc = acc + row[i[t]] * w[t];
        return acc;
    }
};

// Cooperative copy of `count` floats from global memory into LDS by the whole workgroup.
// Loads are issued in batches of eight per thread before any is written (one memory
// latency per batch, not per element), 16 bytes per lane when both sides are 16-byte
// aligned.
__device__ __forceinline__ void stage_copy(float* dst, const float* __restrict__ src, unsigned count)
{
    const unsigned tid = threadIdx.x;
    constexpr unsigned T = G_THREADS;
    const bool aligned = ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0;
    if (aligned)
    {
        const unsigned n4 = count >> 2;
        const float4* __restrict__ s4 = reinterpret_cast<const float4*>(src);
        float4* d4 = reinterpret_cast<float4*>(dst);
        unsigned t = tid;
        for (; t + 7 * T < n4; t += 8 * T)
        {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                v[u] = s4[t + u * T];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                d4[t + u * T] = v[u];
        }
        for (; t < n4; t += T)
            d4[t] = s4[t];
        for (t = (n4 << 2) + tid; t < count; t += T)
            dst[t] = src[t];
    }
    else
    {
        unsigned t = tid;
        for (; t + 7 * T < count; t += 8 * T)
        {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                v[u] = src[t + u * T];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                dst[t + u * T] = v[u];
        }
        for (; t < count; t += T)
            dst[t] = src[t];
    }
}

// grid: (clouds * row_blocks * jsplit).  dynamic LDS: R * m floats.
template <int K, bool WEIGHTED, typename IdxT, bool XCD_LOCAL>
__global__ __launch_bounds__(G_THREADS) void gather_fwd_lds_kernel(
    int c, int m, int64_t n, int rows_per_block, int row_blocks, int jsplit, int64_t jlen,
    const float* __restrict__ src, const IdxT* __restrict__ idx,
    const float* __restrict__ weight, float* __restrict__ out)
{
    extern __shared__ float rows[];
    int bid = XCD_LOCAL ? static_cast<int>(xcd_local_block(blockIdx.x, gridDim.x)) : static_cast<int>(blockIdx.x);
    const int jpart = bid % jsplit;
    bid /= jsplit;
    const int rb = bid % row_blocks;
    const int cloud = bid / row_blocks;
    const int c0 = rb * rows_per_block;
    const int nrows = min(rows_per_block, c - c0);

    const float* __restrict__ s = src + (static_cast<int64_t>(cloud) * c + c0) * m;
    stage_copy(rows, s, static_cast<unsigned>(nrows) * static_cast<unsigned>(m));
    __syncthreads();

    idx += static_cast<int64_t>(cloud) * n * K;
    if (WEIGHTED)
        weight += static_cast<int64_t>(cloud) * n * K;
    float* __restrict__ o = out + (static_cast<int64_t>(cloud) * c + c0) * n;

    const int64_t jbeg = static_cast<int64_t>(jpart) * jlen;
    const int64_t jend = tpk_min64(n, jbeg + jlen);
    for (int64_t j = jbeg + threadIdx.x; j < jend; j += G_THREADS)
    {
        Column<K, WEIGHTED, IdxT> col;
        col.load(idx, weight, j);
#pragma unroll
        for (int r = 0; r < G_MAX_ROWS; ++r)
            if (r < nrows)
                o[static_cast<int64_t>(r) * n + j] = col.combine(rows + r * m);
    }
}

// DPP helpers on 16-lane rows.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}

// Transposing reduction over a 16-lane row: every lane brings 16 partial sums t[0..15]
// (t[s] = its share of target s of the row); lane l leaves with the row-wide sum of target
// l.  Four exchange steps with the lanes l^15, l^7, l^3, l^1 (DPP row_mirror,
// row_half_mirror and two quad permutations); in each step a lane keeps the half of its
// values whose target agrees with its own lane number in the bit being resolved and
// receives the partner's partials of exactly those targets: 15 additions instead of the 64
// that 16 separate row reductions take.
__device__ __forceinline__ float row_transpose_sum(float (&t)[16], int l)
{
    const bool b3 = l & 8, b2 = l & 4, b1 = l & 2, b0 = l & 1;
    float u[8];
#pragma unroll
    for (int s = 0; s < 8; ++s)
    {
        const float keepv = b3 ? t[s + 8] : t[s];
        const float send = b3 ? t[s] : t[s + 8];
        u[s] = keepv + dpp_f32<0x140>(send); // row_mirror: partner l ^ 15
    }
    float v[4];
#pragma unroll
    for (int s = 0; s < 4; ++s)
    {
        const float keepv = b2 ? u[s + 4] : u[s];
        const float send = b2 ? u[s] : u[s + 4];
        v[s] = keepv + dpp_f32<0x141>(send); // row_half_mirror: partner l ^ 7
    }
    float w[2];
#pragma unroll
    for (int s = 0; s < 2; ++s)
    {
        const float keepv = b1 ? v[s + 2] : v[s];
        const float send = b1 ? v[s] : v[s + 2];
        w[s] = keepv + dpp_f32<0x1B>(send); // quad_perm [3,2,1,0]: partner l ^ 3
    }
    const float keepv = b0 ? w[1] : w[0];
    const float send = b0 ? w[0] : w[1];
    return keepv + dpp_f32<0xB1>(send); // quad_perm [1,0,3,2]: partner l ^ 1
}

// Value of lane S of the caller's 16-lane row (DPP row_newbcast).
template <int S>
__device__ __forceinline__ int row_broadcast(int v)
{
    return dpp_i32<0x150 + S>(v);
}

template <int K, bool WEIGHTED, int R, int S>
struct ListRound
{
    // Loads entry (round*16 + l) of target S of the row for every S (recursively unrolled,
    // so that the 16 loads are independent and issued together).
    __device__ __forceinline__ static void load(const ListEntry<WEIGHTED>* __restrict__ entries,
                                                int my_beg, int my_end, int first, int l,
                                                ListEntry<WEIGHTED> (&e)[16], bool (&ok)[16])
    {
        const int beg = row_broadcast<S>(my_beg);
        const int end = row_broadcast<S>(my_end);
        const unsigned p = static_cast<unsigned>(beg + first + l);
        ok[S] = static_cast<int>(p) < end;
        e[S] = entries[ok[S] ? p : 0u];
        if constexpr (S + 1 < 16)
            ListRound<K, WEIGHTED, R, S + 1>::load(entries, my_beg, my_end, first, l, e, ok);
    }
};

// grid: (clouds * row_blocks).  dynamic LDS: R rows of grad_out, n floats each.
// A wavefront takes 64 consecutive targets at a time.  Lane L first fetches the list bounds
// of target base+L (one coalesced read).  Then each of the wavefront's four 16-lane rows
// serves its 16 targets: for target s of the row, lane l reads list entry l (a contiguous
// 128-byte piece per row; the reads of the 16 targets are independent and issued
// together) and multiplies the staged grad_out value; the transposing row reduction above
// leaves the sum of target l in lane l, so the 64 results leave as one contiguous store per
// feature row.  Lists longer than 16 take further rounds.
template <int K, bool WEIGHTED, int R>
__global__ __launch_bounds__(G_THREADS) void gather_bwd_lists_kernel(
    int c, int m, int64_t n, int row_blocks, const float* __restrict__ grad_out,
    const int* __restrict__ offsets, const ListEntry<WEIGHTED>* __restrict__ entries,
    float* __restrict__ grad_src)
{
    extern __shared__ float rows[];
    const int bid = blockIdx.x;
    const int rb = bid % row_blocks;
    const int cloud = bid / row_blocks;
    const int c0 = rb * R;
    const int nrows = min(R, c - c0);
    const unsigned ni = static_cast<unsigned>(n);

    const int lane = threadIdx.x & (TPK_WAVE - 1);
    const int wave = threadIdx.x / TPK_WAVE;
    const int l = lane & 15;
    constexpr int WAVES = G_THREADS / TPK_WAVE;

    offsets += static_cast<int64_t>(cloud) * (m + 1);
    entries += static_cast<int64_t>(cloud) * n * K;
    float* __restrict__ d = grad_src + (static_cast<int64_t>(cloud) * c + c0) * m;

    // list bounds of the first block of targets: requested before the rows are staged
    int base = wave * TPK_WAVE;
    int my_beg = 0, my_end = 0;
    if (base + lane < m)
    {
        my_beg = offsets[base + lane];
        my_end = offsets[base + lane + 1];
    }

    // Staged rows have a stride of a little more than n floats: slot n of every row holds 0
    // and is what lanes without a list entry read, so that no read in the loop below is
    // conditional.  Rows beyond the last feature row are all zeros.
    const unsigned stride = (ni + 4u) & ~3u;
    const float* __restrict__ g = grad_out + (static_cast<int64_t>(cloud) * c + c0) * n;
    for (int r = 0; r < R; ++r)
    {
        if (r < nrows)
        {
            stage_copy(rows + r * stride, g + static_cast<int64_t>(r) * n, ni);
            for (unsigned t = ni + threadIdx.x; t < stride; t += G_THREADS)
                rows[r * stride + t] = 0.f;
        }
        else
        {
            for (unsigned t = threadIdx.x; t < stride; t += G_THREADS)
                rows[r * stride + t] = 0.f;
        }
    }
    __syncthreads();

    for (; base < m; base += WAVES * TPK_WAVE)
    {
        const int tgt = base + lane;
        // bounds of the next block, in flight while this one is processed
        const int next = tgt + WAVES * TPK_WAVE;
        int next_beg = 0, next_end = 0;
        if (next < m)
        {
            next_beg = offsets[next];
            next_end = offsets[next + 1];
        }

        float keep[R];
#pragma unroll
        for (int r = 0; r < R; ++r)
            keep[r] = 0.f;

        const int longest = my_end - my_beg;
        for (int first = 0; __any(longest > first); first += 16)
        {
            ListEntry<WEIGHTED> e[16];
            bool ok[16];
            ListRound<K, WEIGHTED, R, 0>::load(entries, my_beg, my_end, first, l, e, ok);
            unsigned col[16];
            float wv[16];
#pragma unroll
            for (int s = 0; s < 16; ++s)
            {
                col[s] = ok[s] ? static_cast<unsigned>(e[s].j) : ni; // ni = the zero slot
                if constexpr (WEIGHTED)
                    wv[s] = ok[s] ? e[s].w : 0.f;
            }
#pragma unroll
            for (int r = 0; r < R; ++r)
            {
                float t[16];
#pragma unroll
                for (int s = 0; s < 16; ++s)
                {
                    const float v = rows[static_cast<unsigned>(r) * stride + col[s]];
                    if constexpr (WEIGHTED)
                        t[s] = v * wv[s];
                    else
                        t[s] = v;
                }
                keep[r] += row_transpose_sum(t, l);
            }
        }
        if (tgt < m)
        {
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (r < nrows)
                    d[static_cast<int64_t>(r) * m + tgt] = keep[r];
        }
        my_beg = next_beg;
        my_end = next_end;
    }
}

// Direct paths for rows that do not fit in LDS.  One thread per (row, column).
template <int K, bool WEIGHTED, typename IdxT>
__global__ __launch_bounds__(256) void gather_fwd_direct_kernel(
    int c, int m, int64_t n, const float* __restrict__ src, const IdxT* __restrict__ idx,
    const float* __restrict__ weight, float* __restrict__ out, int64_t total)
{
    int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (; t < total; t += stride)
    {
        const int64_t j = t % n;
        const int64_t row = t / n; // cloud * c + channel
        const int64_t cloud = row / c;
        Column<K, WEIGHTED, IdxT> col;
        col.load(idx + cloud * n * K, WEIGHTED ? weight + cloud * n * K : weight, j);
        out[t] = col.combine(src + row * m);
    }
}

template <int K, bool WEIGHTED, typename IdxT>
__global__ __launch_bounds__(256) void gather_bwd_direct_kernel(
    int c, int m, int64_t n, const float* __restrict__ grad_out, const IdxT* __restrict__ idx,
    const float* __restrict__ weight, float* grad_src, int64_t total)
{
    int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (; t < total; t += stride)
    {
        const int64_t j = t % n;
        const int64_t row = t / n;
        const int64_t cloud = row / c;
        Column<K, WEIGHTED, IdxT> col;
        col.load(idx + cloud * n * K, WEIGHTED ? weight + cloud * n * K : weight, j);
        const float gv = grad_out[t];
#pragma unroll
        for (int k = 0; k < K; ++k)
            unsafeAtomicAdd(grad_src + row * m + col.i[k], WEIGHTED ? gv * col.w[k] : gv);
    }
}

__global__ __launch_bounds__(256) void fill_zero_f32_kernel(float* p, int64_t count)
{
    int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (; t < count; t += stride)
        p[t] = 0.0f;
}

// Rows staged per workgroup for rows of m floats; 0 = does not fit.
int rows_for(int m, int c)
{
    if (m <= 0)
        return 0;
    int r = G_LDS_BUDGET / (4 * m);
    if (r > G_MAX_ROWS)
        r = G_MAX_ROWS;
    if (r > c)
        r = c;
    return r;
}

template <int K, bool WEIGHTED, typename IdxT>
int gather_fwd(int b, int c, int m, int64_t n, const float* src, const IdxT* idx,
               const float* weight, float* out, hipStream_t s)
{
    if (b < 0 || c < 0 || m < 0 || n < 0)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || c == 0 || n == 0)
        return TPK_OK;
    if (m == 0)
        return TPK_ERR_INVALID_ARG; // columns to fill but nothing to gather from
    if (!src || !idx || !out || (WEIGHTED && !weight))
        return TPK_ERR_INVALID_ARG;
    const int r = rows_for(m, c);
    if (r > 0)
    {
        const int row_blocks = static_cast<int>(tpk_ceil_div(c, r));
        // Split the columns so that a few hundred workgroups exist, but keep each part at
        // least as long as a row (so staging a row block stays the smaller share of traffic).
        int64_t jsplit = tpk_ceil_div(WEIGHTED ? 256 : 512, static_cast<int64_t>(row_blocks) * b);
        const int64_t max_split = n / (m > G_THREADS ? m : G_THREADS);
        if (jsplit > max_split)
            jsplit = max_split;
        if (jsplit < 1)
            jsplit = 1;
        const int64_t jlen = tpk_ceil_div(n, jsplit);
        const int64_t blocks = static_cast<int64_t>(b) * row_blocks * jsplit;
        if (blocks > 0x7fffffffLL)
            return TPK_ERR_UNSUPPORTED;
        const size_t lds = static_cast<size_t>(r) * m * sizeof(float);
        // Measured on MI355X: the weighted 3-neighbour gather (LDS-read bound) is fastest with one
        // workgroup per compute unit and die-local cloud placement; the plain gather (store
        // bound) with two rounds of workgroups and the default placement.
        auto kernel = gather_fwd_lds_kernel<K, WEIGHTED, IdxT, WEIGHTED>;
        int st = allow_lds(kernel, lds);
        if (st != TPK_OK)
            return st;
        hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(blocks)), dim3(G_THREADS), lds, s, c,
                           m, n, r, row_blocks, static_cast<int>(jsplit), jlen, src, idx, weight,
                           out);
        return tpk_launch_status();
    }
    const int64_t total = static_cast<int64_t>(b) * c * n;
    const unsigned blocks = static_cast<unsigned>(tpk_min64(tpk_ceil_div(total, 256), 1 << 20));
    hipLaunchKernelGGL((gather_fwd_direct_kernel<K, WEIGHTED, IdxT>), dim3(blocks), dim3(256), 0,
                       s, c, m, n, src, idx, weight, out, total);
    return tpk_launch_status();
}

// Workspace of the list-based backward: offsets (b, m+1) ints, then the list entries.
template <int K, bool WEIGHTED>
size_t lists_workspace_bytes(int b, int m, int64_t n)
{
    if (b <= 0 || m <= 0 || n <= 0)
        return 0;
    const size_t off = (static_cast<size_t>(b) * (static_cast<size_t>(m) + 1) * sizeof(int) + 255) &
                       ~static_cast<size_t>(255);
    return off + static_cast<size_t>(b) * static_cast<size_t>(n) * K * sizeof(ListEntry<WEIGHTED>);
}

template <int K, bool WEIGHTED, int R>
int launch_bwd_lists(int b, int c, int m, int64_t n, const float* grad_out, const int* offsets,
                     const ListEntry<WEIGHTED>* entries, float* grad_src, hipStream_t s)
{
    const int row_blocks = static_cast<int>(tpk_ceil_div(c, R));
    const int64_t blocks = static_cast<int64_t>(b) * row_blocks;
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const size_t lds = static_cast<size_t>(R) * ((n + 4) & ~static_cast<int64_t>(3)) * sizeof(float);
    auto kernel = gather_bwd_lists_kernel<K, WEIGHTED, R>;
    int st = allow_lds(kernel, lds);
    if (st != TPK_OK)
        return st;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(blocks)), dim3(G_THREADS), lds, s, c, m, n,
                       row_blocks, grad_out, offsets, entries, grad_src);
    return tpk_launch_status();
}

template <int K, bool WEIGHTED, typename IdxT>
int gather_bwd(int b, int c, int m, int64_t n, const float* grad_out, const IdxT* idx,
               const float* weight, float* grad_src, void* workspace, size_t workspace_bytes,
               hipStream_t s)
{
    if (b < 0 || c < 0 || m < 0 || n < 0)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || c == 0 || m == 0)
        return TPK_OK;
    if (!grad_src || (n > 0 && (!grad_out || !idx || (WEIGHTED && !weight))))
        return TPK_ERR_INVALID_ARG;
    // The list path needs: a row of grad_out (n floats) in LDS, the counters of one cloud
    // (m ints) in LDS, entry positions that fit an int, and the workspace.
    const int64_t row_bytes = n * static_cast<int64_t>(sizeof(float));
    const bool fits = n > 0 && row_bytes <= G_LDS_BUDGET &&
                      m <= 16 * static_cast<int64_t>(L_MAX_TARGETS) && n * K <= 0x7fffffffLL;
    const size_t need = lists_workspace_bytes<K, WEIGHTED>(b, m, n);
    if (fits && workspace && workspace_bytes >= need)
    {
        int* offsets = static_cast<int*>(workspace);
        const size_t off = (static_cast<size_t>(b) * (static_cast<size_t>(m) + 1) * sizeof(int) + 255) &
                           ~static_cast<size_t>(255);
        auto* entries = reinterpret_cast<ListEntry<WEIGHTED>*>(static_cast<char*>(workspace) + off);
        int st = launch_build_lists<K, WEIGHTED, IdxT>(b, m, n * K, idx, weight, offsets, entries, s);
        if (st != TPK_OK)
            return st;
        const int r = static_cast<int>(G_LDS_BUDGET / row_bytes);
        if (r >= 4 && c >= 4)
            return launch_bwd_lists<K, WEIGHTED, 4>(b, c, m, n, grad_out, offsets, entries, grad_src, s);
        if (r >= 2 && c >= 2)
            return launch_bwd_lists<K, WEIGHTED, 2>(b, c, m, n, grad_out, offsets, entries, grad_src, s);
        return launch_bwd_lists<K, WEIGHTED, 1>(b, c, m, n, grad_out, offsets, entries, grad_src, s);
    }
    const int64_t count = static_cast<int64_t>(b) * c * m;
    hipLaunchKernelGGL(fill_zero_f32_kernel,
                       dim3(static_cast<unsigned>(tpk_min64(tpk_ceil_div(count, 256), 1 << 16))),
                       dim3(256), 0, s, grad_src, count);
    int st = tpk_launch_status();
    if (st != TPK_OK || n == 0)
        return st;
    const int64_t total = static_cast<int64_t>(b) * c * n;
    const unsigned blocks = static_cast<unsigned>(tpk_min64(tpk_ceil_div(total, 256), 1 << 20));
    hipLaunchKernelGGL((gather_bwd_direct_kernel<K, WEIGHTED, IdxT>), dim3(blocks), dim3(256), 0,
                       s, c, m, n, grad_out, idx, weight, grad_src, total);
    return tpk_launch_status();
}

} // namespace

extern "C" int tpk_three_interpolate_f32(int b, int c, int m, int n, const float* points,
                                         const int32_t* idx, const float* weight, float* out,
                                         void* stream)
{
    return gather_fwd<3, true, int32_t>(b, c, m, n, points, idx, weight, out, tpk_stream(stream));
}

extern "C" size_t tpk_three_interpolate_grad_workspace_bytes(int b, int n, int m)
{
    return lists_workspace_bytes<3, true>(b, m, n);
}

extern "C" int tpk_three_interpolate_grad_f32(int b, int c, int n, int m, const float* grad_out,
                                              const int32_t* idx, const float* weight,
                                              float* grad_points, void* workspace,
                                              size_t workspace_bytes, void* stream)
{
    return gather_bwd<3, true, int32_t>(b, c, m, n, grad_out, idx, weight, grad_points, workspace,
                                        workspace_bytes, tpk_stream(stream));
}

extern "C" int tpk_group_f32(int b, int c, int n, int npoint, int nsample, const float* features,
                             const int64_t* idx, float* out, void* stream)
{
    if (npoint < 0 || nsample < 0)
        return TPK_ERR_INVALID_ARG;
    return gather_fwd<1, false, int64_t>(b, c, n, static_cast<int64_t>(npoint) * nsample, features,
                                         idx, nullptr, out, tpk_stream(stream));
}

extern "C" size_t tpk_group_grad_workspace_bytes(int b, int n, int npoint, int nsample)
{
    if (npoint < 0 || nsample < 0)
        return 0;
    return lists_workspace_bytes<1, false>(b, n, static_cast<int64_t>(npoint) * nsample);
}

extern "C" int tpk_group_grad_f32(int b, int c, int n, int npoint, int nsample,
                                  const float* grad_out, const int64_t* idx, float* grad_features,
                                  void* workspace, size_t workspace_bytes, void* stream)
{
    if (npoint < 0 || nsample < 0)
        return TPK_ERR_INVALID_ARG;
    return gather_bwd<1, false, int64_t>(b, c, n, static_cast<int64_t>(npoint) * nsample, grad_out,
                                         idx, nullptr, grad_features, workspace, workspace_bytes,
                                         tpk_stream(stream));
}
