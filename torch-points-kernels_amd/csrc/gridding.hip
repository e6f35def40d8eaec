// GRNet's two grid operators: gridding (points -> occupancy grid by trilinear weights, and its
// gradient) and cubic feature sampling (features of the grid vertices around a point, and its
// gradient).  Reference: cuda/src/gridding_gpu.cu:29-331, cuda/src/cubic_feature_sampling_gpu.cu:
// 23-210.  The reference runs one block per cloud; here every launch spreads over all points
// (or output elements) of all clouds.  Sums into the grid are float / double atomics in no fixed
// order, as in the reference; the gridding gradient of a point is one thread's sum in the
// reference's order, so it is reproduced bit for bit.
//
// Vertices outside the grid: the reference forms the linear index regardless (and writes out of
// bounds or into a neighbouring row); here such a vertex gets index -1, adds nothing to the grid
// and contributes no gradient.
#include "tpk_device.h"

namespace {

constexpr int GR_THREADS = 256;

template <typename T>
__global__ __launch_bounds__(GR_THREADS) void fill_zero_kernel(int64_t count, T* __restrict__ out)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * GR_THREADS + threadIdx.x;
    if (i < count)
        out[i] = T(0);
}

template <typename T>
int fill_zero(int64_t count, T* out, hipStream_t s)
{
    if (count == 0)
        return TPK_OK;
    const int64_t blocks = tpk_ceil_div(count, GR_THREADS);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(fill_zero_kernel<T>, dim3(static_cast<unsigned>(blocks)), dim3(GR_THREADS), 0, s, count, out);
    return tpk_launch_status();
}

// The two grid planes a coordinate lies between (cuda/src/gridding_gpu.cu:47-67): floor and
// ceil, the upper one raised by one when the coordinate is integral.
template <typename T>
__device__ __forceinline__ void planes(T v, int* lower, int* upper)
{
    *lower = static_cast<int>(floor(v));
    *upper = static_cast<int>(ceil(v));
    if (*lower == *upper)
        *upper += 1;
}

template <typename T>
__device__ __forceinline__ T axis_weight(T v, int plane)
{
    return T(1) - fabs(v - static_cast<T>(plane));
}

// cuda/src/gridding_gpu.cu:29-191.  One thread per point.
template <typename T>
__global__ __launch_bounds__(GR_THREADS) void gridding_kernel(
    int64_t total_pts, int n_pts, int n_grid_vertices, float min_x, float min_y, float min_z, int len_x, int len_y,
    int len_z, const T* __restrict__ ptcloud, T* __restrict__ grid_weights, T* __restrict__ grid_pt_weights,
    int* __restrict__ grid_pt_indexes)
{
    const int64_t j = static_cast<int64_t>(blockIdx.x) * GR_THREADS + threadIdx.x;
    if (j >= total_pts)
        return;
    T* grid = grid_weights + (j / n_pts) * n_grid_vertices;
    const T px = ptcloud[j * 3 + 0], py = ptcloud[j * 3 + 1], pz = ptcloud[j * 3 + 2];
    int plane[3][2];
    planes(px, &plane[0][0], &plane[0][1]);
    planes(py, &plane[1][0], &plane[1][1]);
    planes(pz, &plane[2][0], &plane[2][1]);
    // int - float -> float -> int, as the reference's expressions convert
    int off[3][2];
    T w[3][2];
#pragma unroll
    for (int side = 0; side < 2; ++side)
    {
        off[0][side] = static_cast<int>(plane[0][side] - min_x);
        off[1][side] = static_cast<int>(plane[1][side] - min_y);
        off[2][side] = static_cast<int>(plane[2][side] - min_z);
        w[0][side] = axis_weight(px, plane[0][side]);
        w[1][side] = axis_weight(py, plane[1][side]);
        w[2][side] = axis_weight(pz, plane[2][side]);
    }
    // vertex v = 4 * (x upper) + 2 * (y upper) + (z upper): LLL, LLU, LUL, LUU, ULL, ULU, UUL, UUU
#pragma unroll
    for (int v = 0; v < 8; ++v)
    {
        const int sx = v >> 2, sy = (v >> 1) & 1, sz = v & 1;
        const bool inside = off[0][sx] >= 0 && off[0][sx] < len_x && off[1][sy] >= 0 && off[1][sy] < len_y &&
                            off[2][sz] >= 0 && off[2][sz] < len_z;
        const int index = inside ? off[0][sx] * len_y * len_z + off[1][sy] * len_z + off[2][sz] : -1;
        grid_pt_indexes[j * 8 + v] = index;
        grid_pt_weights[j * 24 + v * 3 + 0] = w[0][sx];
        grid_pt_weights[j * 24 + v * 3 + 1] = w[1][sy];
        grid_pt_weights[j * 24 + v * 3 + 2] = w[2][sz];
        if (inside)
            atomicAdd(&grid[index], w[0][sx] * w[1][sy] * w[2][sz]);
    }
}

// cuda/src/gridding_gpu.cu:205-305: the gradient of a point is the sum over its 8 vertices, in
// the reference's order and with its signs (upper side +, lower side -).
template <typename T>
__global__ __launch_bounds__(GR_THREADS) void gridding_grad_kernel(
    int64_t total_pts, int n_pts, int n_grid_vertices, const T* __restrict__ grid_pt_weights,
    const int* __restrict__ grid_pt_indexes, const T* __restrict__ grad_grid, T* __restrict__ grad_ptcloud)
{
    const int64_t j = static_cast<int64_t>(blockIdx.x) * GR_THREADS + threadIdx.x;
    if (j >= total_pts)
        return;
    const T* grad = grad_grid + (j / n_pts) * n_grid_vertices;
    T gx = T(0), gy = T(0), gz = T(0);
#pragma unroll
    for (int v = 0; v < 8; ++v)
    {
        const int index = grid_pt_indexes[j * 8 + v];
        const T g = index >= 0 && index < n_grid_vertices ? grad[index] : T(0);
        const T wx = grid_pt_weights[j * 24 + v * 3 + 0];
        const T wy = grid_pt_weights[j * 24 + v * 3 + 1];
        const T wz = grid_pt_weights[j * 24 + v * 3 + 2];
        const T sx = (v >> 2) ? g : -g, sy = ((v >> 1) & 1) ? g : -g, sz = (v & 1) ? g : -g;
        gx += sx * wy * wz;
        gy += sy * wx * wz;
        gz += sz * wx * wy;
    }
    grad_ptcloud[j * 3 + 0] = gx;
    grad_ptcloud[j * 3 + 1] = gy;
    grad_ptcloud[j * 3 + 2] = gz;
}

// cuda/src/cubic_feature_sampling_gpu.cu:23-105.  First kernel: the vertex indices of every
// point (-1 outside the grid); second kernel: one thread per output element, channel fastest.
template <typename T>
__global__ __launch_bounds__(GR_THREADS) void cubic_indexes_kernel(int64_t total_pts, int scale, int neighborhood_size,
                                                                   int n_vertices, const T* __restrict__ ptcloud,
                                                                   int* __restrict__ grid_pt_indexes)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * GR_THREADS + threadIdx.x;
    if (i >= total_pts)
        return;
    int lx, ux, ly, uy, lz, uz;
    planes(ptcloud[i * 3 + 0], &lx, &ux);
    planes(ptcloud[i * 3 + 1], &ly, &uy);
    planes(ptcloud[i * 3 + 2], &lz, &uz);
    const int ns = neighborhood_size - 1;
    int at = 0;
    for (int j = lx - ns; j <= ux + ns; ++j)
        for (int k = ly - ns; k <= uy + ns; ++k)
            for (int m = lz - ns; m <= uz + ns; ++m)
            {
                const bool outside = j < 0 || j >= scale || k < 0 || k >= scale || m < 0 || m >= scale;
                if (at < n_vertices)
                    grid_pt_indexes[i * n_vertices + at] = outside ? -1 : j * scale * scale + k * scale + m;
                ++at;
            }
}

template <typename T>
__global__ __launch_bounds__(GR_THREADS) void cubic_gather_kernel(
    int64_t total, int n_pts, int n_vertices, int channels, int64_t cub_scale, const T* __restrict__ cubic_features,
    const int* __restrict__ grid_pt_indexes, T* __restrict__ point_features)
{
    // consecutive logical blocks (one cloud's) run on one die, whose L2 then holds that cloud's feature map
    const int64_t e = static_cast<int64_t>(xcd_local_block(blockIdx.x, gridDim.x)) * GR_THREADS + threadIdx.x;
    if (e >= total)
        return;
    const int k = static_cast<int>(e % channels);
    const int64_t pv = e / channels; // point * n_vertices + vertex, over all clouds
    const int64_t cloud = pv / (static_cast<int64_t>(n_pts) * n_vertices);
    const int vertex = grid_pt_indexes[pv];
    point_features[e] = vertex < 0 ? T(0) : cubic_features[(cloud * channels + k) * cub_scale + vertex];
}

// cuda/src/cubic_feature_sampling_gpu.cu:138-175
template <typename T>
__global__ __launch_bounds__(GR_THREADS) void cubic_scatter_kernel(
    int64_t total, int n_pts, int n_vertices, int channels, int64_t cub_scale,
    const T* __restrict__ grad_point_features, const int* __restrict__ grid_pt_indexes,
    T* __restrict__ grad_cubic_features)
{
    const int64_t e = static_cast<int64_t>(blockIdx.x) * GR_THREADS + threadIdx.x;
    if (e >= total)
        return;
    const int k = static_cast<int>(e % channels);
    const int64_t pv = e / channels;
    const int64_t cloud = pv / (static_cast<int64_t>(n_pts) * n_vertices);
    const int vertex = grid_pt_indexes[pv];
    if (vertex >= 0 && vertex < cub_scale)
        atomicAdd(&grad_cubic_features[(cloud * channels + k) * cub_scale + vertex], grad_point_features[e]);
}

// The same sum with the destination in LDS: a workgroup owns `group` channels of one cloud's
// feature map (group * scale^3 accumulators), walks all (point, vertex) entries of the cloud
// and adds its channels' gradients with LDS atomics, then writes the map out in order.  One
// global atomic per term (a cache line each, at device scope) is what makes the kernel above slow.
constexpr int CS_THREADS = 1024; // LDS atomics are slow: many wavefronts keep the unit busy

template <typename T>
__global__ __launch_bounds__(CS_THREADS) void cubic_scatter_lds_kernel(
    int n_pts, int n_vertices, int channels, int group, int64_t cub_scale, const T* __restrict__ grad_point_features,
    const int* __restrict__ grid_pt_indexes, T* __restrict__ grad_cubic_features)
{
    extern __shared__ __align__(16) unsigned char cubic_lds[];
    T* sums = reinterpret_cast<T*>(cubic_lds);
    // the workgroups of one cloud read the same lines of the gradient (each its own channels): they
    // are kept on one die, so that one L2 serves them
    const int groups = (channels + group - 1) / group;
    const int block = static_cast<int>(xcd_local_block(blockIdx.x, gridDim.x));
    const int cloud = block / groups;
    const int k0 = (block - cloud * groups) * group;
    const int width = min(group, channels - k0);
    const int64_t cells = static_cast<int64_t>(width) * cub_scale;
    for (int64_t t = threadIdx.x; t < cells; t += CS_THREADS)
        sums[t] = T(0);
    __syncthreads();
    const int64_t entries = static_cast<int64_t>(n_pts) * n_vertices;
    const int* indexes = grid_pt_indexes + cloud * entries;
    const T* grads = grad_point_features + cloud * entries * channels;
    // consecutive threads take the channels of one entry, then the next entry
    for (int64_t t = threadIdx.x; t < entries * width; t += CS_THREADS)
    {
        const int64_t entry = t / width;
        const int k = static_cast<int>(t - entry * width);
        const int vertex = indexes[entry];
        if (vertex >= 0 && vertex < cub_scale)
            atomicAdd(&sums[k * cub_scale + vertex], grads[entry * channels + k0 + k]);
    }
    __syncthreads();
    T* out = grad_cubic_features + (static_cast<int64_t>(cloud) * channels + k0) * cub_scale;
    for (int64_t t = threadIdx.x; t < cells; t += CS_THREADS)
        out[t] = sums[t];
}

template <typename T>
int gridding_fwd(int b, int n_pts, float min_x, float max_x, float min_y, float max_y, float min_z, float max_z,
                 const T* ptcloud, T* grid_weights, T* grid_pt_weights, int32_t* grid_pt_indexes, hipStream_t s)
{
    if (b < 0 || n_pts < 0)
        return TPK_ERR_INVALID_ARG;
    // cuda/src/gridding_gpu.cu:199-202
    const int len_x = static_cast<int>(max_x - min_x + 1), len_y = static_cast<int>(max_y - min_y + 1);
    const int len_z = static_cast<int>(max_z - min_z + 1);
    if (len_x <= 0 || len_y <= 0 || len_z <= 0)
        return TPK_ERR_INVALID_ARG;
    const int64_t vertices = static_cast<int64_t>(len_x) * len_y * len_z;
    if (vertices > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    if (b == 0)
        return TPK_OK;
    if (!grid_weights || (n_pts > 0 && (!ptcloud || !grid_pt_weights || !grid_pt_indexes)))
        return TPK_ERR_INVALID_ARG;
    int st = fill_zero<T>(static_cast<int64_t>(b) * vertices, grid_weights, s);
    if (st != TPK_OK || n_pts == 0)
        return st;
    const int64_t total = static_cast<int64_t>(b) * n_pts;
    const int64_t blocks = tpk_ceil_div(total, GR_THREADS);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(gridding_kernel<T>, dim3(static_cast<unsigned>(blocks)), dim3(GR_THREADS), 0, s, total, n_pts,
                       static_cast<int>(vertices), min_x, min_y, min_z, len_x, len_y, len_z, ptcloud, grid_weights,
                       grid_pt_weights, grid_pt_indexes);
    return tpk_launch_status();
}

template <typename T>
int gridding_bwd(int b, int n_pts, int n_grid_vertices, const T* grid_pt_weights, const int32_t* grid_pt_indexes,
                 const T* grad_grid, T* grad_ptcloud, hipStream_t s)
{
    if (b < 0 || n_pts < 0 || n_grid_vertices < 0)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || n_pts == 0)
        return TPK_OK;
    if (!grid_pt_weights || !grid_pt_indexes || !grad_ptcloud || (n_grid_vertices > 0 && !grad_grid))
        return TPK_ERR_INVALID_ARG;
    const int64_t total = static_cast<int64_t>(b) * n_pts;
    const int64_t blocks = tpk_ceil_div(total, GR_THREADS);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(gridding_grad_kernel<T>, dim3(static_cast<unsigned>(blocks)), dim3(GR_THREADS), 0, s, total,
                       n_pts, n_grid_vertices, grid_pt_weights, grid_pt_indexes, grad_grid, grad_ptcloud);
    return tpk_launch_status();
}

// (2 * neighborhood_size)^3, or -1 when that does not fit
int64_t cubic_vertices(int neighborhood_size)
{
    if (neighborhood_size < 1 || neighborhood_size > 64)
        return -1;
    const int64_t side = 2 * static_cast<int64_t>(neighborhood_size);
    return side * side * side;
}

template <typename T>
int cubic_fwd(int b, int n_pts, int channels, int scale, int neighborhood_size, const T* ptcloud,
              const T* cubic_features, T* point_features, int32_t* grid_pt_indexes, hipStream_t s)
{
    const int64_t nv = cubic_vertices(neighborhood_size);
    if (b < 0 || n_pts < 0 || channels < 0 || scale <= 0 || nv < 0 || scale > 1290)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || n_pts == 0)
        return TPK_OK;
    if (!ptcloud || !grid_pt_indexes || (channels > 0 && (!cubic_features || !point_features)))
        return TPK_ERR_INVALID_ARG;
    const int64_t total_pts = static_cast<int64_t>(b) * n_pts;
    const int64_t total = total_pts * nv * channels;
    const int64_t blocks_pts = tpk_ceil_div(total_pts, GR_THREADS), blocks = tpk_ceil_div(total, GR_THREADS);
    if (blocks > 0x7fffffffLL || nv > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(cubic_indexes_kernel<T>, dim3(static_cast<unsigned>(blocks_pts)), dim3(GR_THREADS), 0, s,
                       total_pts, scale, neighborhood_size, static_cast<int>(nv), ptcloud, grid_pt_indexes);
    int st = tpk_launch_status();
    if (st != TPK_OK || total == 0)
        return st;
    hipLaunchKernelGGL(cubic_gather_kernel<T>, dim3(static_cast<unsigned>(blocks)), dim3(GR_THREADS), 0, s, total, n_pts,
                       static_cast<int>(nv), channels, static_cast<int64_t>(scale) * scale * scale, cubic_features,
                       grid_pt_indexes, point_features);
    return tpk_launch_status();
}

template <typename T>
int cubic_bwd(int b, int n_pts, int channels, int scale, int neighborhood_size, const T* grad_point_features,
              const int32_t* grid_pt_indexes, T* grad_ptcloud, T* grad_cubic_features, hipStream_t s)
{
    const int64_t nv = cubic_vertices(neighborhood_size);
    if (b < 0 || n_pts < 0 || channels < 0 || scale <= 0 || nv < 0 || scale > 1290)
        return TPK_ERR_INVALID_ARG;
    if (b == 0)
        return TPK_OK;
    const int64_t cub = static_cast<int64_t>(scale) * scale * scale;
    if ((n_pts > 0 && !grad_ptcloud) || (channels > 0 && !grad_cubic_features))
        return TPK_ERR_INVALID_ARG;
    // the coordinates only choose the vertices (floor and ceil): their gradient is zero
    // (cuda/src/cubic_feature_sampling_gpu.cu:165-170)
    int st = fill_zero<T>(static_cast<int64_t>(b) * n_pts * 3, grad_ptcloud, s);
    if (st != TPK_OK)
        return st;
    const int64_t total = static_cast<int64_t>(b) * n_pts * nv * channels;
    if (total > 0 && (!grad_point_features || !grid_pt_indexes))
        return TPK_ERR_INVALID_ARG;
    // Feature maps that fit in LDS (at least one channel of scale^3 sums in 128 KiB) are summed there.
    const int64_t fit = (128 * 1024) / (cub * static_cast<int64_t>(sizeof(T)));
    if (fit >= 1 && channels > 0 && nv <= 0x7fffffffLL)
    {
        // as many channels per workgroup as fit (the fewer workgroups share a line of the gradient, the
        // less often it is read), but a workgroup for every compute unit
        int64_t group = fit < channels ? fit : channels;
        while (group > 1 && static_cast<int64_t>(b) * tpk_ceil_div(channels, group) < 256)
            group = (group + 1) / 2;
        const int64_t blocks = static_cast<int64_t>(b) * tpk_ceil_div(channels, group);
        if (blocks <= 0x7fffffffLL)
        {
            const size_t lds = static_cast<size_t>(group * cub) * sizeof(T);
            const int allowed = tpk_allow_lds(reinterpret_cast<const void*>(cubic_scatter_lds_kernel<T>), lds);
            if (allowed != TPK_OK)
                return allowed;
            hipLaunchKernelGGL(cubic_scatter_lds_kernel<T>, dim3(static_cast<unsigned>(blocks)), dim3(CS_THREADS), lds, s, n_pts, static_cast<int>(nv), channels,
                               static_cast<int>(group), cub, grad_point_features, grid_pt_indexes, grad_cubic_features);
            return tpk_launch_status();
        }
    }
    st = fill_zero<T>(static_cast<int64_t>(b) * channels * cub, grad_cubic_features, s);
    if (st != TPK_OK || total == 0)
        return st;
    const int64_t blocks = tpk_ceil_div(total, GR_THREADS);
    if (blocks > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(cubic_scatter_kernel<T>, dim3(static_cast<unsigned>(blocks)), dim3(GR_THREADS), 0, s, total, n_pts,
                       static_cast<int>(nv), channels, cub, grad_point_features, grid_pt_indexes, grad_cubic_features);
    return tpk_launch_status();
}

} // namespace

extern "C" int tpk_gridding_f32(int b, int n_pts, float min_x, float max_x, float min_y, float max_y, float min_z,
                                float max_z, const float* ptcloud, float* grid_weights, float* grid_pt_weights,
                                int32_t* grid_pt_indexes, void* stream)
{
    return gridding_fwd<float>(b, n_pts, min_x, max_x, min_y, max_y, min_z, max_z, ptcloud, grid_weights,
                               grid_pt_weights, grid_pt_indexes, tpk_stream(stream));
}

extern "C" int tpk_gridding_f64(int b, int n_pts, float min_x, float max_x, float min_y, float max_y, float min_z,
                                float max_z, const double* ptcloud, double* grid_weights, double* grid_pt_weights,
                                int32_t* grid_pt_indexes, void* stream)
{
    return gridding_fwd<double>(b, n_pts, min_x, max_x, min_y, max_y, min_z, max_z, ptcloud, grid_weights,
                                grid_pt_weights, grid_pt_indexes, tpk_stream(stream));
}

extern "C" int tpk_gridding_grad_f32(int b, int n_pts, int n_grid_vertices, const float* grid_pt_weights,
                                     const int32_t* grid_pt_indexes, const float* grad_grid, float* grad_ptcloud,
                                     void* stream)
{
    return gridding_bwd<float>(b, n_pts, n_grid_vertices, grid_pt_weights, grid_pt_indexes, grad_grid, grad_ptcloud,
                               tpk_stream(stream));
}

extern "C" int tpk_gridding_grad_f64(int b, int n_pts, int n_grid_vertices, const double* grid_pt_weights,
                                     const int32_t* grid_pt_indexes, const double* grad_grid, double* grad_ptcloud,
                                     void* stream)
{
    return gridding_bwd<double>(b, n_pts, n_grid_vertices, grid_pt_weights, grid_pt_indexes, grad_grid, grad_ptcloud,
                                tpk_stream(stream));
}

extern "C" int tpk_cubic_feature_sampling_f32(int b, int n_pts, int channels, int scale, int neighborhood_size,
                                              const float* ptcloud, const float* cubic_features, float* point_features,
                                              int32_t* grid_pt_indexes, void* stream)
{
    return cubic_fwd<float>(b, n_pts, channels, scale, neighborhood_size, ptcloud, cubic_features, point_features,
                            grid_pt_indexes, tpk_stream(stream));
}

extern "C" int tpk_cubic_feature_sampling_f64(int b, int n_pts, int channels, int scale, int neighborhood_size,
                                              const double* ptcloud, const double* cubic_features,
                                              double* point_features, int32_t* grid_pt_indexes, void* stream)
{
    return cubic_fwd<double>(b, n_pts, channels, scale, neighborhood_size, ptcloud, cubic_features, point_features,
                             grid_pt_indexes, tpk_stream(stream));
}

extern "C" int tpk_cubic_feature_sampling_grad_f32(int b, int n_pts, int channels, int scale, int neighborhood_size,
                                                   const float* grad_point_features, const int32_t* grid_pt_indexes,
                                                   float* grad_ptcloud, float* grad_cubic_features, void* stream)
{
    return cubic_bwd<float>(b, n_pts, channels, scale, neighborhood_size, grad_point_features, grid_pt_indexes,
                            grad_ptcloud, grad_cubic_features, tpk_stream(stream));
}

extern "C" int tpk_cubic_feature_sampling_grad_f64(int b, int n_pts, int channels, int scale, int neighborhood_size,
                                                   const double* grad_point_features, const int32_t* grid_pt_indexes,
                                                   double* grad_ptcloud, double* grad_cubic_features, void* stream)
{
    return cubic_bwd<double>(b, n_pts, channels, scale, neighborhood_size, grad_point_features, grid_pt_indexes,
                             grad_ptcloud, grad_cubic_features, tpk_stream(stream));
}
