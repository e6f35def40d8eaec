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
// weights) using LDS *integer* atomics, which are fast, and an LDS prefix sum, laid out so that
// one lane per target can walk them with coalesced reads (lists.h); the main kernel then
// stages rows of grad_out in LDS - four rows in pieces of 8192 columns, or one longer row in
// pieces of 16384 columns, with lists per piece - and every lane sums the listed columns of
// its target.  No float atomics, no zero fill, each output written by one lane.  The lists cost
// about 3 entries of 8 bytes (4 unweighted) per index entry of workspace, passed in by the
// caller.  The order in which a target's terms are added differs from run to run only through
// the order of its list, as with the reference's global atomics
// (cuda/src/interpolate_gpu.cu:122-152): results agree to rounding.
//
// Forward rows too long for LDS, or a backward call without workspace, take a direct path:
// gathers from global memory (forward), zero fill + global float atomics (backward).
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

// Cooperative copy of `rows` pieces of `count` floats each from global memory into LDS by T
// threads (`tid` = 0..T-1); consecutive pieces lie src_stride / dst_stride floats apart.  The
// pieces are treated as one run of elements: loads are issued in batches of BATCH per thread
// before any is written (one memory latency per batch, not per element or per piece), 16 bytes
// per lane when everything is 16-byte aligned.
template <unsigned T, int BATCH>
__device__ __forceinline__ void stage_rows_by(float* dst, unsigned dst_stride, const float* __restrict__ src,
                                              int64_t src_stride, unsigned rows, unsigned count, unsigned tid)
{
    const bool aligned = ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0 &&
                         ((src_stride | dst_stride | count) & 3) == 0;
    if (aligned)
    {
        const unsigned per_row = count >> 2;
        const unsigned total = per_row * rows;
        for (unsigned base = tid; base < total; base += BATCH * T)
        {
            float4 v[BATCH];
            unsigned at[BATCH];
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
            {
                // (every load is issued, out-of-range ones at the last element: no branches
                // between the loads)
                const unsigned i = min(base + u * T, total - 1u);
                const unsigned r = rows > 1u ? i / per_row : 0u, col = i - r * per_row;
                at[u] = base + u * T < total ? r * dst_stride + col * 4u : ~0u;
                v[u] = *reinterpret_cast<const float4*>(src + r * src_stride + col * 4u);
            }
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
                if (at[u] != ~0u)
                    *reinterpret_cast<float4*>(dst + at[u]) = v[u];
        }
    }
    else
    {
        const unsigned total = count * rows;
        for (unsigned base = tid; base < total; base += BATCH * T)
        {
            float v[BATCH];
            unsigned at[BATCH];
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
            {
                const unsigned i = min(base + u * T, total - 1u);
                const unsigned r = rows > 1u ? i / count : 0u, col = i - r * count;
                at[u] = base + u * T < total ? r * dst_stride + col : ~0u;
                v[u] = src[r * src_stride + col];
            }
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
                if (at[u] != ~0u)
                    dst[at[u]] = v[u];
        }
    }
}

__device__ __forceinline__ void stage_copy(float* dst, const float* __restrict__ src, unsigned count)
{
    stage_rows_by<G_THREADS, 8>(dst, count, src, count, 1u, count, threadIdx.x);
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

constexpr int GB_BUFFER_FLOATS = 16384; // floats of grad_out a workgroup stages at a time (64 KiB)
constexpr int GB_STEPS = L_WIDTH_STEP;  // list slots per request group (widths are multiples of it)

// grid: (clouds * row_groups).  A workgroup takes R feature rows of one cloud and goes through
// the parts of `part_len` columns (the lists are built per part, lists.h): it stages the piece
// of grad_out in LDS, then every wavefront takes the lists of 64 consecutive targets at a time,
// one target per lane: in step i the lanes read slot i of their lists - consecutive entries -
// and the staged values these refer to; padding entries refer to a staged zero (slot part_len
// of every row).  The few lists longer than the block's padded part are then summed by the
// whole wavefront, 64 entries at a time.  Results leave as one contiguous store per feature
// row; parts after the first add to what the same lane stored for the part before.
// With pieces of 64 KiB two workgroups share a compute unit (64 registers each): one stages
// while the other walks its lists, and 32 wavefronts hide the latency of the entry reads.
// dynamic LDS: R * (part_len + 4) floats.
template <int K, bool WEIGHTED, int R>
__global__ __launch_bounds__(G_THREADS, 2) void gather_bwd_lists_kernel(
    int c, int m, int64_t n, int parts, int part_len, int row_groups, const float* __restrict__ grad_out,
    Lists<WEIGHTED> lists, float* __restrict__ grad_src)
{
    extern __shared__ float rows[];
    const unsigned stride = static_cast<unsigned>(part_len) + 4u;
    const int lane = threadIdx.x & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TPK_WAVE); // (a scalar for the compiler)
    constexpr int WAVES = G_THREADS / TPK_WAVE;
    constexpr int STEPS = WEIGHTED ? GB_STEPS : 2 * GB_STEPS; // list slots requested per block at a time
    const int nblocks = (m + L_BLOCK - 1) / L_BLOCK;

    // consecutive workgroups of a die work on consecutive row groups: one cloud's lists per L2
    const int group = static_cast<int>(xcd_local_block(blockIdx.x, gridDim.x));
    const int cloud = group / row_groups;
    const int c0 = (group % row_groups) * R;
    const int nrows = min(R, c - c0);
    float* __restrict__ d = grad_src + (static_cast<int64_t>(cloud) * c + c0) * m;

    for (unsigned t = threadIdx.x; t < R * 4u; t += G_THREADS)
        rows[(t >> 2) * stride + static_cast<unsigned>(part_len) + (t & 3u)] = 0.f;

    for (int part = 0; part < parts; ++part)
    {
        const int64_t col0 = static_cast<int64_t>(part) * part_len;
        const unsigned len = static_cast<unsigned>(tpk_min64(part_len, n - col0));
        if (part > 0)
            __syncthreads(); // everybody is done with the piece before
        stage_rows_by<G_THREADS, 4>(rows, stride, grad_out + (static_cast<int64_t>(cloud) * c + c0) * n + col0, n,
                                    static_cast<unsigned>(nrows), len, threadIdx.x);
        __syncthreads();

        const int64_t cloud_part = static_cast<int64_t>(cloud) * parts + part;
        const int* __restrict__ counts = lists.counts + cloud_part * nblocks * L_BLOCK;
        const int2* __restrict__ blocks = lists.blocks + cloud_part * nblocks;
        const ListEntry<WEIGHTED>* __restrict__ entries = lists.entries + cloud_part * lists.capacity;
        auto add_entry = [&](const ListEntry<WEIGHTED>& e, float (&sum)[R]) __attribute__((always_inline)) {
#pragma unroll
            for (int r = 0; r < R; ++r)
            {
                const float v = rows[static_cast<unsigned>(r) * stride + static_cast<unsigned>(e.j)];
                if constexpr (WEIGHTED)
                    sum[r] += v * e.w;
                else
                    sum[r] += v;
            }
        };

        ListBlock lb = list_block(blocks, min(wave, nblocks - 1));
        for (int blk = wave; blk < nblocks; blk += WAVES)
        {
            // (the next block's description is requested before this block's work starts)
            const ListBlock next_lb = list_block(blocks, min(blk + WAVES, nblocks - 1));
            const ListEntry<WEIGHTED>* __restrict__ e = entries + lb.start + lane;
            const int tgt = blk * L_BLOCK + lane;
            // (what the parts before stored for these targets is requested now, needed at the end)
            float acc[R], old[R];
#pragma unroll
            for (int r = 0; r < R; ++r)
            {
                acc[r] = 0.f;
                old[r] = part > 0 && tgt < m && r < nrows ? d[static_cast<int64_t>(r) * m + tgt] : 0.f;
            }
            for (int i = 0; i < lb.width; i += STEPS)
            {
                // all requests of this round, then all the sums (widths are multiples of
                // GB_STEPS: a round is one or two whole groups of that many slots)
                ListEntry<WEIGHTED> ent[STEPS];
#pragma unroll
                for (int h = 0; h < STEPS; h += GB_STEPS)
                    if (i + h < lb.width)
                    {
#pragma unroll
                        for (int u = h; u < h + GB_STEPS; ++u)
                            ent[u] = e[(i + u) * L_BLOCK];
                    }
#pragma unroll
                for (int h = 0; h < STEPS; h += GB_STEPS)
                    if (i + h < lb.width)
                    {
#pragma unroll
                        for (int u = h; u < h + GB_STEPS; ++u)
                            add_entry(ent[u], acc);
                    }
            }
            if (lb.longer)
            {
                int extra, extra_at;
                list_extra(counts[tgt], lb.width, extra, extra_at);
                const ListEntry<WEIGHTED>* __restrict__ rest = entries + lb.start + lb.width * L_BLOCK;
                for (unsigned long long todo = __ballot(extra > 0); todo; todo &= todo - 1)
                {
                    const int owner = __builtin_ctzll(todo);
                    const int count = __builtin_amdgcn_readlane(extra, owner);
                    const int at = __builtin_amdgcn_readlane(extra_at, owner);
                    float rest_sum[R];
#pragma unroll
                    for (int r = 0; r < R; ++r)
                        rest_sum[r] = 0.f;
                    for (int p = lane; p < count; p += TPK_WAVE)
                        add_entry(rest[at + p], rest_sum);
#pragma unroll
                    for (int r = 0; r < R; ++r)
                    {
                        const float total = wave_sum_f32(rest_sum[r]);
                        if (lane == owner)
                            acc[r] += total;
                    }
                }
            }
            // (an empty block has nothing to add after the first part)
            if (tgt < m && (part == 0 || lb.width > 0 || lb.longer))
            {
#pragma unroll
                for (int r = 0; r < R; ++r)
                    if (r < nrows)
                        d[static_cast<int64_t>(r) * m + tgt] = old[r] + acc[r];
            }
            lb = next_lb;
        }
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

// Rows of grad_out staged together and columns per part, for rows of n floats.
struct BwdShape
{
    int rows;
    int part_len;
    int parts;
};
BwdShape bwd_shape(int64_t n)
{
    BwdShape sh;
    // Measured on MI355X (config shapes): rows of up to 16384 floats go four at a time in pieces of
    // 8192 columns (one workgroup per compute unit: the lists of a piece are read once per four
    // rows); longer rows one at a time in pieces of 16384 columns, two workgroups per compute unit.
    sh.rows = n <= GB_BUFFER_FLOATS ? 4 : 1;
    const int64_t n4 = (n + 3) & ~static_cast<int64_t>(3);
    sh.part_len = static_cast<int>(tpk_min64(n4, sh.rows == 4 ? GB_BUFFER_FLOATS / 2 : GB_BUFFER_FLOATS));
    sh.parts = static_cast<int>(tpk_min64(tpk_ceil_div(n, sh.part_len), 0x7fffffff));
    return sh;
}

// Workspace of the list-based backward: the lists of every (cloud, part) (lists.h).
template <int K, bool WEIGHTED>
size_t lists_workspace_bytes(int b, int m, int64_t n)
{
    if (b <= 0 || m <= 0 || n <= 0)
        return 0;
    const BwdShape sh = bwd_shape(n);
    if (static_cast<int64_t>(b) * sh.parts > 0x7fffffffLL)
        return 0;
    return lists_bytes<WEIGHTED>(b * sh.parts, m, static_cast<int64_t>(sh.part_len) * K);
}

template <int K, bool WEIGHTED, int R>
int launch_bwd_lists(int b, int c, int m, int64_t n, const BwdShape& sh, const float* grad_out,
                     const Lists<WEIGHTED>& lists, float* grad_src, hipStream_t s)
{
    const int row_groups = static_cast<int>(tpk_ceil_div(c, R));
    const int64_t groups_total = static_cast<int64_t>(b) * row_groups;
    if (groups_total > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    const size_t lds = static_cast<size_t>(R) * (sh.part_len + 4) * sizeof(float);
    auto kernel = gather_bwd_lists_kernel<K, WEIGHTED, R>;
    int st = allow_lds(kernel, lds);
    if (st != TPK_OK)
        return st;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(groups_total)), dim3(G_THREADS), lds, s, c, m, n,
                       sh.parts, sh.part_len, row_groups, grad_out, lists, grad_src);
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
    // The list path needs entry positions that fit an int, and the workspace.
    const BwdShape sh = bwd_shape(n > 0 ? n : 1);
    const bool fits = n > 0 && n * K <= 0x7fffffffLL &&
                      static_cast<int64_t>(b) * sh.parts <= 0x7fffffffLL;
    const size_t need = lists_workspace_bytes<K, WEIGHTED>(b, m, n);
    if (fits && workspace && need > 0 && workspace_bytes >= need)
    {
        const int64_t part_total = static_cast<int64_t>(sh.part_len) * K;
        const Lists<WEIGHTED> lists = lists_at<WEIGHTED>(workspace, b * sh.parts, m, part_total);
        int st = launch_build_lists<K, WEIGHTED, IdxT>(b, m, n * K, part_total, sh.part_len, idx, weight, lists, s);
        if (st == TPK_OK)
        {
            if (sh.rows == 4)
                return launch_bwd_lists<K, WEIGHTED, 4>(b, c, m, n, sh, grad_out, lists, grad_src, s);
            return launch_bwd_lists<K, WEIGHTED, 1>(b, c, m, n, sh, grad_out, lists, grad_src, s);
        }
        if (st != TPK_ERR_UNSUPPORTED)
            return st;
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
