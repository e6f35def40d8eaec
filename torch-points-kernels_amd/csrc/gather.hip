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
// Backward: the same row block lives in LDS as an accumulator, zeroed at the start, fed
// with LDS float atomics and written out once - no global atomics and no separate zero
// fill of the result.  The order of the additions is not fixed (as with the reference's
// global atomics, cuda/src/interpolate_gpu.cu:122-152), so results agree to rounding.
//
// Rows too long for LDS take a direct path: gathers from global memory (forward), zero
// fill + global float atomics (backward).
//
// Forward arithmetic follows cuda/src/interpolate_gpu.cu:78-107: ((p1*w1) + (p2*w2)) +
// (p3*w3), every operation rounded on its own.  The grouping forward is a pure copy
// (torch_points_kernels/torchpoints.py:129-146 expresses it as torch.gather).
#include "tpk_device.h"

namespace {

constexpr int G_THREADS = 1024;
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

// grid: (clouds * row_blocks * jsplit).  dynamic LDS: R * m floats.
template <int K, bool WEIGHTED, typename IdxT>
__global__ __launch_bounds__(G_THREADS) void gather_fwd_lds_kernel(
    int c, int m, int64_t n, int rows_per_block, int row_blocks, int jsplit, int64_t jlen,
    const float* __restrict__ src, const IdxT* __restrict__ idx,
    const float* __restrict__ weight, float* __restrict__ out)
{
    extern __shared__ float rows[];
    int bid = blockIdx.x;
    const int jpart = bid % jsplit;
    bid /= jsplit;
    const int rb = bid % row_blocks;
    const int cloud = bid / row_blocks;
    const int c0 = rb * rows_per_block;
    const int nrows = min(rows_per_block, c - c0);

    const float* __restrict__ s = src + (static_cast<int64_t>(cloud) * c + c0) * m;
    const int total = nrows * m;
    for (int t = threadIdx.x; t < total; t += G_THREADS)
        rows[t] = s[t];
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

// grid: (clouds * row_blocks).  dynamic LDS: R * m floats (accumulators).
template <int K, bool WEIGHTED, typename IdxT>
__global__ __launch_bounds__(G_THREADS) void gather_bwd_lds_kernel(
    int c, int m, int64_t n, int rows_per_block, int row_blocks,
    const float* __restrict__ grad_out, const IdxT* __restrict__ idx,
    const float* __restrict__ weight, float* __restrict__ grad_src)
{
    extern __shared__ float rows[];
    const int rb = blockIdx.x % row_blocks;
    const int cloud = blockIdx.x / row_blocks;
    const int c0 = rb * rows_per_block;
    const int nrows = min(rows_per_block, c - c0);
    const int total = nrows * m;
    for (int t = threadIdx.x; t < total; t += G_THREADS)
        rows[t] = 0.0f;
    __syncthreads();

    idx += static_cast<int64_t>(cloud) * n * K;
    if (WEIGHTED)
        weight += static_cast<int64_t>(cloud) * n * K;
    const float* __restrict__ g = grad_out + (static_cast<int64_t>(cloud) * c + c0) * n;

    for (int64_t j = threadIdx.x; j < n; j += G_THREADS)
    {
        Column<K, WEIGHTED, IdxT> col;
        col.load(idx, weight, j);
#pragma unroll
        for (int r = 0; r < G_MAX_ROWS; ++r)
            if (r < nrows)
            {
                const float gv = g[static_cast<int64_t>(r) * n + j];
#pragma unroll
                for (int t = 0; t < K; ++t)
                {
                    const float v = WEIGHTED ? gv * col.w[t] : gv;
                    __hip_atomic_fetch_add(&rows[r * m + col.i[t]], v, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            }
    }
    __syncthreads();
    float* __restrict__ d = grad_src + (static_cast<int64_t>(cloud) * c + c0) * m;
    for (int t = threadIdx.x; t < total; t += G_THREADS)
        d[t] = rows[t];
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

template <typename Kernel>
int allow_lds(Kernel kernel, size_t bytes)
{
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       static_cast<int>(bytes));
    return e == hipSuccess ? TPK_OK : static_cast<int>(e);
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
        int64_t jsplit = tpk_ceil_div(512, static_cast<int64_t>(row_blocks) * b);
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
        auto kernel = gather_fwd_lds_kernel<K, WEIGHTED, IdxT>;
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

template <int K, bool WEIGHTED, typename IdxT>
int gather_bwd(int b, int c, int m, int64_t n, const float* grad_out, const IdxT* idx,
               const float* weight, float* grad_src, hipStream_t s)
{
    if (b < 0 || c < 0 || m < 0 || n < 0)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || c == 0 || m == 0)
        return TPK_OK;
    if (!grad_src || (n > 0 && (!grad_out || !idx || (WEIGHTED && !weight))))
        return TPK_ERR_INVALID_ARG;
    const int r = rows_for(m, c);
    if (r > 0)
    {
        const int row_blocks = static_cast<int>(tpk_ceil_div(c, r));
        const int64_t blocks = static_cast<int64_t>(b) * row_blocks;
        if (blocks > 0x7fffffffLL)
            return TPK_ERR_UNSUPPORTED;
        const size_t lds = static_cast<size_t>(r) * m * sizeof(float);
        auto kernel = gather_bwd_lds_kernel<K, WEIGHTED, IdxT>;
        int st = allow_lds(kernel, lds);
        if (st != TPK_OK)
            return st;
        hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(blocks)), dim3(G_THREADS), lds, s, c,
                           m, n, r, row_blocks, grad_out, idx, weight, grad_src);
        return tpk_launch_status();
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

extern "C" int tpk_three_interpolate_grad_f32(int b, int c, int n, int m, const float* grad_out,
                                              const int32_t* idx, const float* weight,
                                              float* grad_points, void* stream)
{
    return gather_bwd<3, true, int32_t>(b, c, m, n, grad_out, idx, weight, grad_points,
                                        tpk_stream(stream));
}

extern "C" int tpk_group_f32(int b, int c, int n, int npoint, int nsample, const float* features,
                             const int64_t* idx, float* out, void* stream)
{
    if (npoint < 0 || nsample < 0)
        return TPK_ERR_INVALID_ARG;
    return gather_fwd<1, false, int64_t>(b, c, n, static_cast<int64_t>(npoint) * nsample, features,
                                         idx, nullptr, out, tpk_stream(stream));
}

extern "C" int tpk_group_grad_f32(int b, int c, int n, int npoint, int nsample,
                                  const float* grad_out, const int64_t* idx, float* grad_features,
                                  void* stream)
{
    if (npoint < 0 || nsample < 0)
        return TPK_ERR_INVALID_ARG;
    return gather_bwd<1, false, int64_t>(b, c, n, static_cast<int64_t>(npoint) * nsample, grad_out,
                                         idx, nullptr, grad_features, tpk_stream(stream));
}
