/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar CPU restatement of what the reference's CUDA kernels compute for the
 * spatial-search path, used only as the checker in tests/, in
 * __graft_entry__.smoke() and as the timed "port" leg of bench.py.  The shipped
 * library never links, loads or calls this file.
 *
 * Arithmetic: fp32, every product and sum rounded separately (build with
 * -ffp-contract=off), evaluated left to right as the reference's C source
 * reads.  Integer outputs of the HIP kernels are required to equal these bit
 * for bit.
 *
 * Each function cites the reference lines it follows (paths relative to the
 * reference checkout).  How each function is pinned (known-answer vectors of
 * the reference's own tests, the reference's compiled CPU module, brute force
 * in numpy/float64, closed forms) is listed in tests/test_oracle_pinning.py;
 * no function of this file is "parity unpinned".
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------- */
/* ball query, dense layout.  cuda/src/ball_query_gpu.cu:9-52 (kernel),       */
/* cuda/src/ball_query.cpp:26-29 (idx pre-zeroed, dist pre-filled with -1).    */
/* new_xyz (b,m,3) queries, xyz (b,n,3) support, idx (b,m,nsample) int64,      */
/* dist (b,m,nsample).  scan_pairs (may be NULL) receives the number of        */
/* distance evaluations the serial scan performs (early exit included).        */
/* ------------------------------------------------------------------------- */
void tpk_oracle_ball_query_dense(int b, int n, int m, float radius, int nsample,
                                 const float* new_xyz, const float* xyz, int64_t* idx,
                                 float* dist, int64_t* scan_pairs)
{
    const float radius2 = radius * radius;
    int64_t pairs = 0;
    for (int64_t t = 0; t < (int64_t)b * m * nsample; ++t)
    {
        idx[t] = 0;
        dist[t] = -1.0f;
    }
    for (int bi = 0; bi < b; ++bi)
    {
        const float* sx = xyz + (int64_t)bi * n * 3;
        const float* qx = new_xyz + (int64_t)bi * m * 3;
        int64_t* io = idx + (int64_t)bi * m * nsample;
        float* dout = dist + (int64_t)bi * m * nsample;
        for (int j = 0; j < m; ++j)
        {
            const float new_x = qx[j * 3 + 0], new_y = qx[j * 3 + 1], new_z = qx[j * 3 + 2];
            for (int k = 0, cnt = 0; k < n && cnt < nsample; ++k)
            {
                const float x = sx[k * 3 + 0], y = sx[k * 3 + 1], z = sx[k * 3 + 2];
                const float d2 = (new_x - x) * (new_x - x) + (new_y - y) * (new_y - y) +
                                 (new_z - z) * (new_z - z);
                ++pairs;
                if (d2 < radius2)
                {
                    if (cnt == 0)
                        for (int l = 0; l < nsample; ++l)
                            io[(int64_t)j * nsample + l] = k;
                    io[(int64_t)j * nsample + cnt] = k;
                    dout[(int64_t)j * nsample + cnt] = d2;
                    ++cnt;
                }
            }
        }
    }
    if (scan_pairs)
        *scan_pairs = pairs;
}

/* ------------------------------------------------------------------------- */
/* ball query, packed variable-length layout.                                  */
/* cuda/src/ball_query_gpu.cu:54-95 (kernel: non-strict <=, global indices,    */
/* dist accumulated from 0), cuda/src/ball_query.cpp:58-73 (idx and dist       */
/* pre-filled with -1; cloud count = batch_x[last]+1; offsets = exclusive      */
/* prefix sum of per-cloud counts).  x (size_x,3) support, y (size_y,3)        */
/* queries, batch_x/batch_y sorted cloud ids.  Returns the cloud count, or -1  */
/* on allocation failure.                                                      */
/* ------------------------------------------------------------------------- */
int64_t tpk_oracle_ball_query_partial(int64_t size_x, int64_t size_y, float radius, int nsample,
                                      const float* x, const float* y, const int64_t* batch_x,
                                      const int64_t* batch_y, int64_t* idx, float* dist,
                                      int64_t* scan_pairs)
{
    const float radius2 = radius * radius;
    int64_t pairs = 0;
    for (int64_t t = 0; t < size_y * nsample; ++t)
    {
        idx[t] = -1;
        dist[t] = -1.0f;
    }
    if (size_x == 0)
    {
        if (scan_pairs)
            *scan_pairs = 0;
        return 0;
    }
    const int64_t batch_size = batch_x[size_x - 1] + 1;
    int64_t* off_x = (int64_t*)calloc((size_t)batch_size + 1, sizeof(int64_t));
    int64_t* off_y = (int64_t*)calloc((size_t)batch_size + 1, sizeof(int64_t));
    if (!off_x || !off_y)
    {
        free(off_x);
        free(off_y);
        return -1;
    }
    /* degree() + cumsum + leading zero */
    for (int64_t i = 0; i < size_x; ++i)
        if (batch_x[i] >= 0 && batch_x[i] < batch_size)
            off_x[batch_x[i] + 1] += 1;
    for (int64_t i = 0; i < size_y; ++i)
        if (batch_y[i] >= 0 && batch_y[i] < batch_size)
            off_y[batch_y[i] + 1] += 1;
    for (int64_t c = 0; c < batch_size; ++c)
    {
        off_x[c + 1] += off_x[c];
        off_y[c + 1] += off_y[c];
    }
    for (int64_t c = 0; c < batch_size; ++c)
    {
        for (int64_t n_y = off_y[c]; n_y < off_y[c + 1]; ++n_y)
        {
            int64_t count = 0;
            for (int64_t n_x = off_x[c]; n_x < off_x[c + 1]; ++n_x)
            {
                float d = 0;
                for (int t = 0; t < 3; ++t)
                    d += (x[n_x * 3 + t] - y[n_y * 3 + t]) * (x[n_x * 3 + t] - y[n_y * 3 + t]);
                ++pairs;
                if (d <= radius2)
                {
                    idx[n_y * nsample + count] = n_x;
                    dist[n_y * nsample + count] = d;
                    count++;
                }
                if (count >= nsample)
                    break;
            }
        }
    }
    free(off_x);
    free(off_y);
    if (scan_pairs)
        *scan_pairs = pairs;
    return batch_size;
}

/* ------------------------------------------------------------------------- */
/* furthest point sampling.  cuda/src/sampling_gpu.cu:17-144 (kernel),         */
/* :6-12 (pairwise merge), cuda/src/sampling.cpp:14-18 (out zeroed, running    */
/* minimum initialised to 1e10), cuda/include/cuda_utils.h:13-18 (block size   */
/* = largest power of two <= n, at most 512).                                  */
/*                                                                             */
/* The kernel's result depends on its thread layout when two points tie, so    */
/* the layout is restated literally: "thread" t owns points t, t+BS, ... and   */
/* keeps its first strict maximum; the per-thread results are merged by the    */
/* same halving tree, a slot keeping its own entry unless the partner's value  */
/* is strictly larger.                                                         */
/* xyz (b,n,3), out (b,m) int32.                                               */
/* ------------------------------------------------------------------------- */
static int tpk_oracle_block_size(int work_size)
{
    int pow_2 = (int)(log((double)work_size) / log(2.0));
    int v = 1 << pow_2;
    if (v > 512)
        v = 512;
    if (v < 1)
        v = 1;
    return v;
}

int tpk_oracle_fps(int b, int n, int m, const float* xyz, int32_t* out)
{
    if (b <= 0 || m <= 0)
        return 0;
    memset(out, 0, sizeof(int32_t) * (size_t)b * (size_t)m);
    if (n <= 0)
        return 0;
    const int bs = tpk_oracle_block_size(n);
    float* temp = (float*)malloc(sizeof(float) * (size_t)n);
    float dists[512];
    int dists_i[512];
    if (!temp)
        return -1;
    for (int bi = 0; bi < b; ++bi)
    {
        const float* p = xyz + (int64_t)bi * n * 3;
        int32_t* idxs = out + (int64_t)bi * m;
        for (int k = 0; k < n; ++k)
            temp[k] = 1e10f;
        int old = 0;
        idxs[0] = old;
        for (int j = 1; j < m; ++j)
        {
            const float x1 = p[old * 3 + 0], y1 = p[old * 3 + 1], z1 = p[old * 3 + 2];
            for (int tid = 0; tid < bs; ++tid)
            {
                int besti = 0;
                float best = -1;
                for (int k = tid; k < n; k += bs)
                {
                    const float x2 = p[k * 3 + 0], y2 = p[k * 3 + 1], z2 = p[k * 3 + 2];
                    const float mag = (x2 * x2) + (y2 * y2) + (z2 * z2);
                    if (mag <= 1e-3) /* double comparison, as in the kernel */
                        continue;
                    const float d = (x2 - x1) * (x2 - x1) + (y2 - y1) * (y2 - y1) +
                                    (z2 - z1) * (z2 - z1);
                    const float d2 = fminf(d, temp[k]);
                    temp[k] = d2;
                    besti = d2 > best ? k : besti;
                    best = d2 > best ? d2 : best;
                }
                dists[tid] = best;
                dists_i[tid] = besti;
            }
            for (int stride = bs / 2; stride >= 1; stride /= 2)
            {
                for (int tid = 0; tid < stride; ++tid)
                {
                    const float v1 = dists[tid], v2 = dists[tid + stride];
                    const int i1 = dists_i[tid], i2 = dists_i[tid + stride];
                    dists[tid] = fmaxf(v1, v2);
                    dists_i[tid] = v2 > v1 ? i2 : i1;
                }
            }
            old = dists_i[0];
            idxs[j] = old;
        }
    }
    free(temp);
    return 0;
}

/* ------------------------------------------------------------------------- */
/* k nearest neighbours, dense layout: the three_nn scan above with k entries.   */
/* The reference has this operator on the CPU only (torch_points_kernels/       */
/* knn.py:4-18, cpu/src/knn.cpp:8-62, nanoflann's knnSearch underneath); the     */
/* support points are visited in index order and enter the list only when        */
/* strictly smaller than an entry, so equal distances keep the lower index       */
/* first (nanoflann leaves the order of exactly equal distances open).           */
/* support (b,n,3), query (b,m,3); idx (b,m,k) int64, dist2 (b,m,k) ascending.   */
/* Returns -1 when k > n (cpu/src/knn.cpp:12-14 raises), else 0.                 */
/* ------------------------------------------------------------------------- */
int tpk_oracle_knn(int b, int n, int m, int k, const float* support, const float* query,
                   int64_t* idx, float* dist2)
{
    if (k > n)
        return -1;
    for (int bi = 0; bi < b; ++bi)
    {
        const float* s = support + (int64_t)bi * n * 3;
        const float* q = query + (int64_t)bi * m * 3;
        for (int j = 0; j < m; ++j)
        {
            const float ux = q[j * 3 + 0], uy = q[j * 3 + 1], uz = q[j * 3 + 2];
            float* d = dist2 + ((int64_t)bi * m + j) * k;
            int64_t* ix = idx + ((int64_t)bi * m + j) * k;
            int have = 0;
            for (int p = 0; p < n; ++p)
            {
                const float x = s[p * 3 + 0], y = s[p * 3 + 1], z = s[p * 3 + 2];
                const float dd = (ux - x) * (ux - x) + (uy - y) * (uy - y) + (uz - z) * (uz - z);
                if (have == k && !(dd < d[k - 1]))
                    continue;
                int at = have < k ? have : k - 1;
                while (at > 0 && dd < d[at - 1])
                {
                    d[at] = d[at - 1];
                    ix[at] = ix[at - 1];
                    --at;
                }
                d[at] = dd;
                ix[at] = p;
                if (have < k)
                    ++have;
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* three nearest neighbours.  cuda/src/interpolate_gpu.cu:9-65; outputs        */
/* zero-initialised (cuda/src/interpolate.cpp:22-25).  unknown (b,n,3), known  */
/* (b,m,3); dist2 (b,n,3) squared distances ascending, idx (b,n,3) int32.      */
/* The running bests are doubles initialised to 1e40, as in the kernel.        */
/* ------------------------------------------------------------------------- */
void tpk_oracle_three_nn(int b, int n, int m, const float* unknown, const float* known,
                         float* dist2, int32_t* idx)
{
    for (int bi = 0; bi < b; ++bi)
    {
        const float* u = unknown + (int64_t)bi * n * 3;
        const float* kn = known + (int64_t)bi * m * 3;
        float* d2o = dist2 + (int64_t)bi * n * 3;
        int32_t* io = idx + (int64_t)bi * n * 3;
        for (int j = 0; j < n; ++j)
        {
            const float ux = u[j * 3 + 0], uy = u[j * 3 + 1], uz = u[j * 3 + 2];
            double best1 = 1e40, best2 = 1e40, best3 = 1e40;
            int besti1 = 0, besti2 = 0, besti3 = 0;
            for (int k = 0; k < m; ++k)
            {
                const float x = kn[k * 3 + 0], y = kn[k * 3 + 1], z = kn[k * 3 + 2];
                const float d = (ux - x) * (ux - x) + (uy - y) * (uy - y) + (uz - z) * (uz - z);
                if (d < best1)
                {
                    best3 = best2;
                    besti3 = besti2;
                    best2 = best1;
                    besti2 = besti1;
                    best1 = d;
                    besti1 = k;
                }
                else if (d < best2)
                {
                    best3 = best2;
                    besti3 = besti2;
                    best2 = d;
                    besti2 = k;
                }
                else if (d < best3)
                {
                    best3 = d;
                    besti3 = k;
                }
            }
            d2o[j * 3 + 0] = (float)best1;
            d2o[j * 3 + 1] = (float)best2;
            d2o[j * 3 + 2] = (float)best3;
            io[j * 3 + 0] = besti1;
            io[j * 3 + 1] = besti2;
            io[j * 3 + 2] = besti3;
        }
    }
}

/* ------------------------------------------------------------------------- */
/* three_interpolate forward.  cuda/src/interpolate_gpu.cu:78-107.             */
/* points (b,c,m), idx (b,n,3) int32, weight (b,n,3), out (b,c,n).             */
/* ------------------------------------------------------------------------- */
void tpk_oracle_three_interpolate(int b, int c, int m, int n, const float* points,
                                  const int32_t* idx, const float* weight, float* out)
{
    for (int bi = 0; bi < b; ++bi)
    {
        const float* p = points + (int64_t)bi * m * c;
        const int32_t* id = idx + (int64_t)bi * n * 3;
        const float* w = weight + (int64_t)bi * n * 3;
        float* o = out + (int64_t)bi * n * c;
        for (int64_t i = 0; i < (int64_t)c * n; ++i)
        {
            const int64_t l = i / n, j = i % n;
            const float w1 = w[j * 3 + 0], w2 = w[j * 3 + 1], w3 = w[j * 3 + 2];
            const int i1 = id[j * 3 + 0], i2 = id[j * 3 + 1], i3 = id[j * 3 + 2];
            o[i] = p[l * m + i1] * w1 + p[l * m + i2] * w2 + p[l * m + i3] * w3;
        }
    }
}

/* ------------------------------------------------------------------------- */
/* three_interpolate backward.  cuda/src/interpolate_gpu.cu:122-152; output    */
/* zero-initialised (cuda/src/interpolate.cpp:68).  The kernel adds with       */
/* atomics in no fixed order; this restatement adds in index order, and        */
/* parity is to tolerance.  grad_out (b,c,n) -> grad_points (b,c,m).           */
/* ------------------------------------------------------------------------- */
void tpk_oracle_three_interpolate_grad(int b, int c, int n, int m, const float* grad_out,
                                       const int32_t* idx, const float* weight,
                                       float* grad_points)
{
    memset(grad_points, 0, sizeof(float) * (size_t)b * (size_t)c * (size_t)m);
    for (int bi = 0; bi < b; ++bi)
    {
        const float* go = grad_out + (int64_t)bi * n * c;
        const int32_t* id = idx + (int64_t)bi * n * 3;
        const float* w = weight + (int64_t)bi * n * 3;
        float* gp = grad_points + (int64_t)bi * m * c;
        for (int64_t i = 0; i < (int64_t)c * n; ++i)
        {
            const int64_t l = i / n, j = i % n;
            const float w1 = w[j * 3 + 0], w2 = w[j * 3 + 1], w3 = w[j * 3 + 2];
            const int i1 = id[j * 3 + 0], i2 = id[j * 3 + 1], i3 = id[j * 3 + 2];
            gp[l * m + i1] += go[i] * w1;
            gp[l * m + i2] += go[i] * w2;
            gp[l * m + i3] += go[i] * w3;
        }
    }
}

/* ------------------------------------------------------------------------- */
/* grouping_operation forward / backward.                                      */
/* torch_points_kernels/torchpoints.py:129-146: out[b,c,p,s] =                 */
/* features[b,c,idx[b,p,s]] (a gather along the last axis); the backward of a  */
/* gather accumulates grad_out into the gathered positions.                    */
/* features (b,c,n), idx (b,np,ns) int64, out (b,c,np,ns).                     */
/* ------------------------------------------------------------------------- */
void tpk_oracle_group(int b, int c, int n, int64_t npts, const float* features,
                      const int64_t* idx, float* out)
{
    for (int bi = 0; bi < b; ++bi)
        for (int ci = 0; ci < c; ++ci)
        {
            const float* f = features + ((int64_t)bi * c + ci) * n;
            const int64_t* id = idx + (int64_t)bi * npts;
            float* o = out + ((int64_t)bi * c + ci) * npts;
            for (int64_t t = 0; t < npts; ++t)
                o[t] = f[id[t]];
        }
}

void tpk_oracle_group_grad(int b, int c, int n, int64_t npts, const float* grad_out,
                           const int64_t* idx, float* grad_features)
{
    memset(grad_features, 0, sizeof(float) * (size_t)b * (size_t)c * (size_t)n);
    for (int bi = 0; bi < b; ++bi)
        for (int ci = 0; ci < c; ++ci)
        {
            float* gf = grad_features + ((int64_t)bi * c + ci) * n;
            const int64_t* id = idx + (int64_t)bi * npts;
            const float* go = grad_out + ((int64_t)bi * c + ci) * npts;
            for (int64_t t = 0; t < npts; ++t)
                gf[id[t]] += go[t];
        }
}

/* ------------------------------------------------------------------------- */
/* Chamfer distance, one direction: for every point of cloud 1 the squared     */
/* distance to, and index of, its nearest point of cloud 2.                    */
/* cuda/src/chamfer_dist_gpu.cu:9-155: cloud 2 is walked in tiles of 512;      */
/* inside a tile the first point starts the minimum and later ones replace it  */
/* only when strictly smaller; a later tile replaces the stored result only    */
/* when strictly smaller.  Outputs zero-initialised (:162-165).                */
/* The wrapper (:157-184) runs it twice with the clouds swapped.               */
/* ------------------------------------------------------------------------- */
#define TPK_ORACLE_CHAMFER_ONE_DIRECTION(NAME, T)                                                  \
    static void NAME(int batch_size, int n, const T* xyz1, int m, const T* xyz2, T* dist,          \
                     int32_t* indexes)                                                             \
    {                                                                                              \
        const int tile = 512;                                                                      \
        for (int64_t t = 0; t < (int64_t)batch_size * n; ++t)                                      \
        {                                                                                          \
            dist[t] = 0;                                                                           \
            indexes[t] = 0;                                                                        \
        }                                                                                          \
        for (int i = 0; i < batch_size; ++i)                                                       \
            for (int k2 = 0; k2 < m; k2 += tile)                                                   \
            {                                                                                      \
                const int end_k = (m < k2 + tile ? m : k2 + tile) - k2;                            \
                const T* buf = xyz2 + ((int64_t)i * m + k2) * 3;                                   \
                for (int j = 0; j < n; ++j)                                                        \
                {                                                                                  \
                    const T x1 = xyz1[((int64_t)i * n + j) * 3 + 0];                               \
                    const T y1 = xyz1[((int64_t)i * n + j) * 3 + 1];                               \
                    const T z1 = xyz1[((int64_t)i * n + j) * 3 + 2];                               \
                    T best_dist = 0;                                                               \
                    int best_dist_index = 0;                                                       \
                    for (int k = 0; k < end_k; ++k)                                                \
                    {                                                                              \
                        const T x2 = buf[k * 3 + 0] - x1;                                          \
                        const T y2 = buf[k * 3 + 1] - y1;                                          \
                        const T z2 = buf[k * 3 + 2] - z1;                                          \
                        const T d = x2 * x2 + y2 * y2 + z2 * z2;                                   \
                        if (k == 0 || d < best_dist)                                               \
                        {                                                                          \
                            best_dist = d;                                                         \
                            best_dist_index = k + k2;                                              \
                        }                                                                          \
                    }                                                                              \
                    if (k2 == 0 || dist[(int64_t)i * n + j] > best_dist)                           \
                    {                                                                              \
                        dist[(int64_t)i * n + j] = best_dist;                                      \
                        indexes[(int64_t)i * n + j] = best_dist_index;                             \
                    }                                                                              \
                }                                                                                  \
            }                                                                                      \
    }

TPK_ORACLE_CHAMFER_ONE_DIRECTION(chamfer_dir_f32, float)
TPK_ORACLE_CHAMFER_ONE_DIRECTION(chamfer_dir_f64, double)

void tpk_oracle_chamfer_fwd_f32(int batch_size, int n, int m, const float* xyz1,
                                const float* xyz2, float* dist1, float* dist2, int32_t* idx1,
                                int32_t* idx2)
{
    chamfer_dir_f32(batch_size, n, xyz1, m, xyz2, dist1, idx1);
    chamfer_dir_f32(batch_size, m, xyz2, n, xyz1, dist2, idx2);
}

void tpk_oracle_chamfer_fwd_f64(int batch_size, int n, int m, const double* xyz1,
                                const double* xyz2, double* dist1, double* dist2, int32_t* idx1,
                                int32_t* idx2)
{
    chamfer_dir_f64(batch_size, n, xyz1, m, xyz2, dist1, idx1);
    chamfer_dir_f64(batch_size, m, xyz2, n, xyz1, dist2, idx2);
}

/* ------------------------------------------------------------------------- */
/* Chamfer backward.  cuda/src/chamfer_dist_gpu.cu:187-213 (one direction:     */
/* g = 2*grad_dist[j]; grad_xyz1[j] += g*(p1-p2); grad_xyz2[idx[j]] -= same),  */
/* :215-245 (zero-initialised outputs; run twice with the clouds and their     */
/* gradients swapped).  The kernel's additions are atomic and unordered; this  */
/* restatement adds in index order, and parity is to tolerance.                */
/* ------------------------------------------------------------------------- */
#define TPK_ORACLE_CHAMFER_GRAD_ONE_DIRECTION(NAME, T)                                             \
    static void NAME(int b, int n, const T* xyz1, int m, const T* xyz2, const T* grad_dist1,       \
                     const int32_t* idx1, T* grad_xyz1, T* grad_xyz2)                              \
    {                                                                                              \
        for (int i = 0; i < b; ++i)                                                                \
            for (int j = 0; j < n; ++j)                                                            \
            {                                                                                      \
                const T x1 = xyz1[((int64_t)i * n + j) * 3 + 0];                                   \
                const T y1 = xyz1[((int64_t)i * n + j) * 3 + 1];                                   \
                const T z1 = xyz1[((int64_t)i * n + j) * 3 + 2];                                   \
                const int j2 = idx1[(int64_t)i * n + j];                                           \
                const T x2 = xyz2[((int64_t)i * m + j2) * 3 + 0];                                  \
                const T y2 = xyz2[((int64_t)i * m + j2) * 3 + 1];                                  \
                const T z2 = xyz2[((int64_t)i * m + j2) * 3 + 2];                                  \
                const T g = grad_dist1[(int64_t)i * n + j] * 2;                                    \
                grad_xyz1[((int64_t)i * n + j) * 3 + 0] += g * (x1 - x2);                          \
                grad_xyz1[((int64_t)i * n + j) * 3 + 1] += g * (y1 - y2);                          \
                grad_xyz1[((int64_t)i * n + j) * 3 + 2] += g * (z1 - z2);                          \
                grad_xyz2[((int64_t)i * m + j2) * 3 + 0] += -(g * (x1 - x2));                      \
                grad_xyz2[((int64_t)i * m + j2) * 3 + 1] += -(g * (y1 - y2));                      \
                grad_xyz2[((int64_t)i * m + j2) * 3 + 2] += -(g * (z1 - z2));                      \
            }                                                                                      \
    }

TPK_ORACLE_CHAMFER_GRAD_ONE_DIRECTION(chamfer_grad_dir_f32, float)
TPK_ORACLE_CHAMFER_GRAD_ONE_DIRECTION(chamfer_grad_dir_f64, double)

void tpk_oracle_chamfer_bwd_f32(int b, int n, int m, const float* xyz1, const float* xyz2,
                                const int32_t* idx1, const int32_t* idx2,
                                const float* grad_dist1, const float* grad_dist2,
                                float* grad_xyz1, float* grad_xyz2)
{
    memset(grad_xyz1, 0, sizeof(float) * (size_t)b * (size_t)n * 3);
    memset(grad_xyz2, 0, sizeof(float) * (size_t)b * (size_t)m * 3);
    chamfer_grad_dir_f32(b, n, xyz1, m, xyz2, grad_dist1, idx1, grad_xyz1, grad_xyz2);
    chamfer_grad_dir_f32(b, m, xyz2, n, xyz1, grad_dist2, idx2, grad_xyz2, grad_xyz1);
}

void tpk_oracle_chamfer_bwd_f64(int b, int n, int m, const double* xyz1, const double* xyz2,
                                const int32_t* idx1, const int32_t* idx2,
                                const double* grad_dist1, const double* grad_dist2,
                                double* grad_xyz1, double* grad_xyz2)
{
    memset(grad_xyz1, 0, sizeof(double) * (size_t)b * (size_t)n * 3);
    memset(grad_xyz2, 0, sizeof(double) * (size_t)b * (size_t)m * 3);
    chamfer_grad_dir_f64(b, n, xyz1, m, xyz2, grad_dist1, idx1, grad_xyz1, grad_xyz2);
    chamfer_grad_dir_f64(b, m, xyz2, n, xyz1, grad_dist2, idx2, grad_xyz2, grad_xyz1);
}

/* ------------------------------------------------------------------------- */
/* Clusters grown over a neighbour matrix (torch_points_kernels/cluster.py:9-37, */
/* the numba routine behind grow_proximity).  neighbours (n, nsample) int64,     */
/* each row ends at its first -1.  Points are taken in index order; an unseen    */
/* point starts a cluster and a stack; the last entry of the stack is taken off  */
/* and its row read left to right, every unseen neighbour being marked, put on   */
/* the stack and appended to the cluster at once.  Clusters with at least        */
/* min_cluster_size members are kept, in the order of their first point.         */
/* members (n) receives the kept clusters one after the other, starts            */
/* (up to n + 1) their offsets; returns the number of kept clusters.             */
/* ------------------------------------------------------------------------- */
int64_t tpk_oracle_grow_proximity(int64_t n, int nsample, const int64_t* neighbours,
                                  int64_t min_cluster_size, int64_t* members, int64_t* starts)
{
    unsigned char* seen = (unsigned char*)calloc((size_t)(n > 0 ? n : 1), 1);
    int64_t* stack = (int64_t*)malloc(sizeof(int64_t) * (size_t)(n > 0 ? n : 1));
    int64_t clusters = 0, filled = 0;
    starts[0] = 0;
    for (int64_t i = 0; i < n; ++i)
    {
        if (seen[i])
            continue;
        int64_t* cluster = members + filled;
        int64_t size = 0, top = 0;
        seen[i] = 1;
        stack[top++] = i;
        cluster[size++] = i;
        while (top > 0)
        {
            const int64_t k = stack[--top];
            const int64_t* row = neighbours + k * nsample;
            for (int j = 0; j < nsample; ++j)
            {
                const int64_t nei = row[j];
                if (nei == -1)
                    break;
                if (!seen[nei])
                {
                    seen[nei] = 1;
                    stack[top++] = nei;
                    cluster[size++] = nei;
                }
            }
        }
        if (size >= min_cluster_size)
        {
            filled += size;
            starts[++clusters] = filled;
        }
    }
    free(stack);
    free(seen);
    return clusters;
}

/* ------------------------------------------------------------------------- */
/* Ball query with sorted neighbours: what the reference computes for CPU      */
/* tensors with sort=True (and refuses for CUDA tensors,                       */
/* torch_points_kernels/torchpoints.py:152-153, :163-164).                      */
/* cpu/src/neighbors.cpp:8-136 (dense, per cloud) and :139-310 (packed):       */
/* nanoflann's radiusSearch keeps a support point when its squared distance,   */
/* accumulated as ((dx*dx) + dy*dy) + dz*dz in the points' type, is            */
/* < radius*radius (a float product, :19 and :153), sorts the matches by       */
/* distance, and the first max_num = nsample are written.  nanoflann sorts by  */
/* distance only; here equal distances keep the lower index first.             */
/* Unused slots: dense - index of the first (nearest) match, distance -1, and  */
/* index 0 when there is no match (:60-61, :88-105); packed - index -1,        */
/* distance -1 (:248-275).  In the packed layout a query searches the support  */
/* points that carry its own cloud id (the reference walks both batch vectors  */
/* in step, which is the same thing when every cloud has queries).             */
/* first/last (per query) delimit the support range searched.                  */
/* ------------------------------------------------------------------------- */
static void sorted_hits(const float* q, const float* support, int64_t first, int64_t last,
                        float radius2, int nsample, int64_t* idx, float* dist, int* found)
{
    int have = 0;
    for (int64_t p = first; p < last; ++p)
    {
        float d = 0;
        for (int t = 0; t < 3; ++t)
            d += (q[t] - support[p * 3 + t]) * (q[t] - support[p * 3 + t]);
        if (!(d < radius2))
            continue;
        if (have == nsample && !(d < dist[nsample - 1]))
            continue;
        int at = have < nsample ? have : nsample - 1;
        while (at > 0 && d < dist[at - 1])
        {
            dist[at] = dist[at - 1];
            idx[at] = idx[at - 1];
            --at;
        }
        dist[at] = d;
        idx[at] = p;
        if (have < nsample)
            ++have;
    }
    *found = have;
}

void tpk_oracle_ball_query_sorted_dense(int b, int n, int m, float radius, int nsample,
                                        const float* new_xyz, const float* xyz, int64_t* idx, float* dist)
{
    const float radius2 = radius * radius;
    if (nsample <= 0)
        return;
    for (int bi = 0; bi < b; ++bi)
        for (int j = 0; j < m; ++j)
        {
            int64_t* io = idx + ((int64_t)bi * m + j) * nsample;
            float* dout = dist + ((int64_t)bi * m + j) * nsample;
            int found = 0;
            sorted_hits(new_xyz + ((int64_t)bi * m + j) * 3, xyz + (int64_t)bi * n * 3, 0, n, radius2, nsample,
                        io, dout, &found);
            const int64_t token = found > 0 ? io[0] : 0;
            for (int s = found; s < nsample; ++s)
            {
                io[s] = token;
                dout[s] = -1.0f;
            }
        }
}

void tpk_oracle_ball_query_sorted_partial(int64_t size_x, int64_t size_y, float radius, int nsample,
                                          const float* x, const float* y, const int64_t* batch_x,
                                          const int64_t* batch_y, int64_t* idx, float* dist)
{
    const float radius2 = radius * radius;
    if (nsample <= 0)
        return;
    for (int64_t j = 0; j < size_y; ++j)
    {
        int64_t first = 0, last;
        while (first < size_x && batch_x[first] < batch_y[j])
            ++first;
        last = first;
        while (last < size_x && batch_x[last] == batch_y[j])
            ++last;
        int found = 0;
        sorted_hits(y + j * 3, x, first, last, radius2, nsample, idx + j * nsample, dist + j * nsample, &found);
        for (int s = found; s < nsample; ++s)
        {
            idx[j * nsample + s] = -1;
            dist[j * nsample + s] = -1.0f;
        }
    }
}

/* ------------------------------------------------------------------------- */
/* IoU between proposed instances and ground-truth instances.                  */
/* cuda/src/metrics_gpu.cu:9-43 (kernel), cuda/src/metrics.cpp:37-39 (output   */
/* pre-zeroed).  proposals_idx: the proposals' point indices one after the     */
/* other, proposals_offset (n_proposals + 1) their boundaries; labels (per     */
/* point; ground-truth instance k of a sample carries label k + 1, 0 and       */
/* negative values mean "none"); batch (per point) the sample of a point;      */
/* n_instances / instance_offset (per sample) count and first column of the    */
/* sample's instances; instance_pointnum (per column) their sizes.  A          */
/* proposal is compared with the instances of the sample of its first point.   */
/* The quotient is formed as the kernel's expression types dictate: float      */
/* operands, the 1e-5 a double, the result stored as float.                    */
/* iou (n_proposals, total_instances).                                         */
/* ------------------------------------------------------------------------- */
void tpk_oracle_instance_iou(int64_t total_instances, int64_t n_proposals, const int64_t* n_instances,
                             const int64_t* proposals_idx, const int64_t* proposals_offset,
                             const int64_t* labels, const int64_t* instance_offset, const int64_t* batch,
                             const int64_t* instance_pointnum, float* iou)
{
    for (int64_t t = 0; t < n_proposals * total_instances; ++t)
        iou[t] = 0.0f;
    for (int64_t p = 0; p < n_proposals; ++p)
    {
        const int start = (int)proposals_offset[p], end = (int)proposals_offset[p + 1];
        if (end <= start)
            continue; /* the kernel would read past the proposal; every quotient is 0 anyway */
        const int sample = (int)batch[proposals_idx[start]];
        const int count = (int)n_instances[sample];
        const int first = (int)instance_offset[sample];
        const int proposal_total = end - start;
        for (int k = 0; k < count; ++k)
        {
            const int instance_total = (int)instance_pointnum[first + k];
            int intersection = 0;
            for (int i = start; i < end; ++i)
                if ((int)labels[proposals_idx[i]] == k + 1)
                    ++intersection;
            iou[first + k + p * total_instances] =
                (float)((float)intersection / ((float)(proposal_total + instance_total - intersection) + 1e-5));
        }
    }
}

/* ------------------------------------------------------------------------- */
/* Gridding and cubic feature sampling (GRNet).  cuda/src/gridding_gpu.cu:    */
/* 29-191 (forward), :205-305 (gradient); cuda/src/cubic_feature_sampling_    */
/* gpu.cu:23-105 (forward), :138-175 (gradient).  Both exist for float and     */
/* double (AT_DISPATCH_FLOATING_TYPES).  Sums are formed in point order here;  */
/* the kernels add atomically in no fixed order.  Vertices outside the grid    */
/* (where the reference forms an index regardless and writes out of bounds or  */
/* into a neighbouring row) get index -1 and take no part.                     */
/* ------------------------------------------------------------------------- */
#define TPK_GRID_OPS(T, SUFFIX, FLOOR, CEIL, FABS)                                                          \
    static void planes_##SUFFIX(T v, int* lower, int* upper)                                                \
    {                                                                                                       \
        *lower = (int)FLOOR(v);                                                                             \
        *upper = (int)CEIL(v);                                                                              \
        if (*lower == *upper)                                                                               \
            *upper += 1;                                                                                    \
    }                                                                                                       \
    void tpk_oracle_gridding_##SUFFIX(int b, int n_pts, float min_x, float max_x, float min_y, float max_y, \
                                      float min_z, float max_z, const T* ptcloud, T* grid_weights,          \
                                      T* grid_pt_weights, int32_t* grid_pt_indexes)                         \
    {                                                                                                       \
        const int len_x = (int)(max_x - min_x + 1), len_y = (int)(max_y - min_y + 1);                       \
        const int len_z = (int)(max_z - min_z + 1);                                                         \
        const int64_t vertices = (int64_t)len_x * len_y * len_z;                                            \
        for (int64_t t = 0; t < b * vertices; ++t)                                                          \
            grid_weights[t] = 0;                                                                            \
        for (int64_t j = 0; j < (int64_t)b * n_pts; ++j)                                                    \
        {                                                                                                   \
            T* grid = grid_weights + (j / n_pts) * vertices;                                                \
            const T p[3] = {ptcloud[j * 3 + 0], ptcloud[j * 3 + 1], ptcloud[j * 3 + 2]};                    \
            const float lo[3] = {min_x, min_y, min_z};                                                      \
            const int len[3] = {len_x, len_y, len_z};                                                       \
            int plane[3][2], off[3][2];                                                                     \
            T w[3][2];                                                                                      \
            for (int a = 0; a < 3; ++a)                                                                     \
            {                                                                                               \
                planes_##SUFFIX(p[a], &plane[a][0], &plane[a][1]);                                          \
                for (int s = 0; s < 2; ++s)                                                                 \
                {                                                                                           \
                    off[a][s] = (int)(plane[a][s] - lo[a]);                                                 \
                    w[a][s] = 1 - FABS(p[a] - (T)plane[a][s]);                                              \
                }                                                                                           \
            }                                                                                               \
            for (int v = 0; v < 8; ++v)                                                                     \
            {                                                                                               \
                const int s[3] = {v >> 2, (v >> 1) & 1, v & 1};                                             \
                int inside = 1;                                                                             \
                for (int a = 0; a < 3; ++a)                                                                 \
                    inside = inside && off[a][s[a]] >= 0 && off[a][s[a]] < len[a];                          \
                const int index = inside ? off[0][s[0]] * len_y * len_z + off[1][s[1]] * len_z + off[2][s[2]] : -1; \
                grid_pt_indexes[j * 8 + v] = index;                                                         \
                for (int a = 0; a < 3; ++a)                                                                 \
                    grid_pt_weights[j * 24 + v * 3 + a] = w[a][s[a]];                                       \
                if (inside)                                                                                 \
                    grid[index] += w[0][s[0]] * w[1][s[1]] * w[2][s[2]];                                    \
            }                                                                                               \
        }                                                                                                   \
    }                                                                                                       \
    void tpk_oracle_gridding_grad_##SUFFIX(int b, int n_pts, int n_grid_vertices, const T* grid_pt_weights, \
                                           const int32_t* grid_pt_indexes, const T* grad_grid,             \
                                           T* grad_ptcloud)                                                 \
    {                                                                                                       \
        for (int64_t j = 0; j < (int64_t)b * n_pts; ++j)                                                    \
        {                                                                                                   \
            const T* grad = grad_grid + (j / n_pts) * n_grid_vertices;                                      \
            T gx = 0, gy = 0, gz = 0;                                                                       \
            for (int v = 0; v < 8; ++v)                                                                     \
            {                                                                                               \
                const int index = grid_pt_indexes[j * 8 + v];                                               \
                const T g = index >= 0 && index < n_grid_vertices ? grad[index] : 0;                        \
                const T wx = grid_pt_weights[j * 24 + v * 3 + 0], wy = grid_pt_weights[j * 24 + v * 3 + 1]; \
                const T wz = grid_pt_weights[j * 24 + v * 3 + 2];                                           \
                /* upper side +, lower side - (gridding_gpu.cu:228-303) */                                  \
                gx += ((v >> 2) ? g : -g) * wy * wz;                                                        \
                gy += (((v >> 1) & 1) ? g : -g) * wx * wz;                                                  \
                gz += ((v & 1) ? g : -g) * wx * wy;                                                         \
            }                                                                                               \
            grad_ptcloud[j * 3 + 0] = gx;                                                                   \
            grad_ptcloud[j * 3 + 1] = gy;                                                                   \
            grad_ptcloud[j * 3 + 2] = gz;                                                                   \
        }                                                                                                   \
    }                                                                                                       \
    void tpk_oracle_cubic_feature_sampling_##SUFFIX(int b, int n_pts, int channels, int scale,              \
                                                    int neighborhood_size, const T* ptcloud,                \
                                                    const T* cubic_features, T* point_features,             \
                                                    int32_t* grid_pt_indexes)                               \
    {                                                                                                       \
        const int side = 2 * neighborhood_size, nv = side * side * side, ns = neighborhood_size - 1;        \
        const int64_t cub = (int64_t)scale * scale * scale;                                                 \
        for (int64_t i = 0; i < (int64_t)b * n_pts; ++i)                                                    \
        {                                                                                                   \
            const T* feats = cubic_features + (i / n_pts) * channels * cub;                                 \
            int lx, ux, ly, uy, lz, uz, at = 0;                                                             \
            planes_##SUFFIX(ptcloud[i * 3 + 0], &lx, &ux);                                                  \
            planes_##SUFFIX(ptcloud[i * 3 + 1], &ly, &uy);                                                  \
            planes_##SUFFIX(ptcloud[i * 3 + 2], &lz, &uz);                                                  \
            for (int j = lx - ns; j <= ux + ns; ++j)                                                        \
                for (int k = ly - ns; k <= uy + ns; ++k)                                                    \
                    for (int m = lz - ns; m <= uz + ns; ++m)                                                \
                    {                                                                                       \
                        const int out = j < 0 || j >= scale || k < 0 || k >= scale || m < 0 || m >= scale;  \
                        grid_pt_indexes[i * nv + at++] = out ? -1 : j * scale * scale + k * scale + m;      \
                    }                                                                                       \
            for (int j = 0; j < nv; ++j)                                                                    \
                for (int k = 0; k < channels; ++k)                                                          \
                {                                                                                           \
                    const int vertex = grid_pt_indexes[i * nv + j];                                         \
                    point_features[(i * nv + j) * channels + k] = vertex == -1 ? 0 : feats[k * cub + vertex]; \
                }                                                                                           \
        }                                                                                                   \
    }                                                                                                       \
    void tpk_oracle_cubic_feature_sampling_grad_##SUFFIX(int b, int n_pts, int channels, int scale,         \
                                                         int neighborhood_size, const T* grad_point_features, \
                                                         const int32_t* grid_pt_indexes, T* grad_ptcloud,   \
                                                         T* grad_cubic_features)                            \
    {                                                                                                       \
        const int side = 2 * neighborhood_size, nv = side * side * side;                                    \
        const int64_t cub = (int64_t)scale * scale * scale;                                                 \
        for (int64_t t = 0; t < (int64_t)b * n_pts * 3; ++t)                                                \
            grad_ptcloud[t] = 0;                                                                            \
        for (int64_t t = 0; t < b * channels * cub; ++t)                                                    \
            grad_cubic_features[t] = 0;                                                                     \
        for (int64_t i = 0; i < (int64_t)b * n_pts; ++i)                                                    \
            for (int j = 0; j < nv; ++j)                                                                    \
            {                                                                                               \
                const int vertex = grid_pt_indexes[i * nv + j];                                             \
                if (vertex == -1)                                                                           \
                    continue;                                                                               \
                for (int k = 0; k < channels; ++k)                                                          \
                    grad_cubic_features[((i / n_pts) * channels + k) * cub + vertex] +=                     \
                        grad_point_features[(i * nv + j) * channels + k];                                   \
            }                                                                                               \
    }

TPK_GRID_OPS(float, f32, floorf, ceilf, fabsf)
TPK_GRID_OPS(double, f64, floor, ceil, fabs)
