/*
 * tpk.h - C ABI of libtpk_hip.so: the spatial-search kernels of torch-points-kernels for
 * AMD MI355X (gfx950).
 *
 * Every entry point takes plain device pointers and sizes, launches on the HIP stream
 * passed as `stream` (a hipStream_t cast to void*; NULL = the null stream), never
 * allocates, never synchronises the host (exceptions, documented below: tpk_grow_proximity and
 * tpk_ball_query_sorted_partial_f32 with a workspace and nsample > 64) and keeps no state between calls
 * (exception: tpk_three_nn_static_f32, whose scratch memory is an array inside the library that all calls on a GPU
 * share).  The first call of a kernel on a device makes a few runtime calls on the host (the kernel's LDS limit;
 * for tpk_three_nn_static_f32 also the address of its array): a caller that captures HIP graphs makes one call
 * of the same shape outside the capture first.  The caller owns all memory.  All arrays are dense row-major ("contiguous").  Outputs need not be
 * initialised: every element of every output array is written by the call.
 *
 * Return value: TPK_OK (0); a negative TPK_ERR_* for a rejected argument (nothing was
 * launched); or a positive hipError_t reported by the launch.  tpk_status_string() turns
 * any of them into text.
 *
 * Each declaration names the interface of the reference (torch-points3d/
 * torch-points-kernels, paths relative to its checkout) that it stands in for: the
 * `*_kernel_wrapper` launchers its pybind host functions call.
 */
#ifndef TPK_H
#define TPK_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TPK_OK 0
#define TPK_ERR_INVALID_ARG (-1) /* negative size, NULL pointer with non-empty data, ... */
#define TPK_ERR_UNSUPPORTED (-2) /* valid request outside what the kernels cover */
#define TPK_ERR_WORKSPACE (-3)   /* workspace missing or too small */
#define TPK_ERR_TOO_LARGE (-4)   /* problem needs more scratch memory than the library's fixed array holds */

/* Library version, major*10000 + minor*100 + patch. */
int tpk_version(void);

/* Text for a status returned by any entry point (static storage). */
const char* tpk_status_string(int status);

/* ---------------------------------------------------------------------------------------
 * Furthest point sampling.
 * Replaces furthest_point_sampling_kernel_wrapper(b, n, m, dataset, temp, idxs)
 * (cuda/src/sampling_gpu.cu:146-201, declared cuda/src/sampling.cpp:5-6).
 *   xyz  (b, n, 3) float32          idx_out (b, npoint) int32
 * Starts at point 0; squared distances; points with x*x+y*y+z*z <= 1e-3 are never
 * updated nor selected; ties resolve as the reference's block reduction does.
 * `workspace` replaces the reference's `temp` tensor: it is needed only when n exceeds
 * what one workgroup keeps in registers (16384 points); tpk_fps_workspace_bytes() says how
 * many bytes (0 = none needed, NULL may be passed).  Up to 163840 points it also holds the
 * cloud in curve order and what orders it (45 - 52 bytes per point); with 4 bytes per point
 * or more, but less than that, the call still works, several times slower.
 * ------------------------------------------------------------------------------------- */
size_t tpk_fps_workspace_bytes(int b, int n);
int tpk_fps_f32(int b, int n, int npoint, const float* xyz, void* workspace,
                size_t workspace_bytes, int32_t* idx_out, void* stream);

/* ---------------------------------------------------------------------------------------
 * Ball query, dense layout.
 * Replaces query_ball_point_kernel_dense_wrapper(b, n, m, radius, nsample, new_xyz, xyz,
 * idx, dist_out) (cuda/src/ball_query_gpu.cu:97-106, declared cuda/src/ball_query.cpp:5-7).
 *   new_xyz (b, m, 3) query centres   xyz (b, n, 3) support
 *   idx (b, m, nsample) int64         dist (b, m, nsample) float32 (squared)
 * First `nsample` support points in index order with d2 < radius*radius; unused idx slots
 * repeat the first hit (0 when there is none), unused dist slots are -1.
 * Clouds of 1024 .. 8192 points are searched through buckets of cells that every workgroup
 * builds in LDS.  Larger clouds need a `workspace` for anything better than a scan of all
 * pairs (tpk_ball_query_dense_workspace_bytes() bytes - 0 for sizes not served that way -,
 * 256-byte aligned, contents arbitrary before and after): the points are ordered in windows
 * along a space filling curve and a query only looks into the bins its ball touches, as in the
 * packed layout below.  tpk_ball_query_dense_f32 is the call without a workspace.  Same results
 * every way.
 * ------------------------------------------------------------------------------------- */
int tpk_ball_query_dense_f32(int b, int n, int m, float radius, int nsample,
                             const float* new_xyz, const float* xyz, int64_t* idx, float* dist,
                             void* stream);
size_t tpk_ball_query_dense_workspace_bytes(int b, int n, int m, int nsample);
int tpk_ball_query_dense_ws_f32(int b, int n, int m, float radius, int nsample,
                                const float* new_xyz, const float* xyz, int64_t* idx, float* dist,
                                void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------
 * Ball query, packed variable-length layout.
 * Replaces query_ball_point_kernel_partial_wrapper(batch_size, size_x, size_y, radius,
 * nsample, x, y, batch_x, batch_y, idx_out, dist_out) (cuda/src/ball_query_gpu.cu:108-118,
 * declared cuda/src/ball_query.cpp:9-13) together with the offset construction in front of
 * it (cuda/src/ball_query.cpp:64-73): this entry takes the SORTED per-point cloud ids
 * themselves and finds each cloud's range on the device, so no device-to-host copy and no
 * cloud count are needed.
 *   x (size_x, 3) support   y (size_y, 3) queries   batch_x (size_x) / batch_y (size_y) int64
 *   idx (size_y, nsample) int64 (indices into x)    dist (size_y, nsample) float32
 * First `nsample` points of the query's own cloud in index order with d2 <= radius*radius;
 * unused slots are -1 in both outputs.
 * With a `workspace` (tpk_ball_query_partial_workspace_bytes() bytes - 0 for sizes not served
 * that way -, 256-byte aligned, contents arbitrary before and after) both arrays are ordered
 * along a space filling curve and a query only visits cells within its radius; queries with
 * more than 16 neighbours in the radius are then answered by a scan in index order that stops
 * after nsample hits.  With workspace == NULL every query scans its whole cloud (same results).
 * ------------------------------------------------------------------------------------- */
size_t tpk_ball_query_partial_workspace_bytes(int64_t size_x, int64_t size_y, int nsample);
int tpk_ball_query_partial_f32(int64_t size_x, int64_t size_y, float radius, int nsample,
                               const float* x, const float* y, const int64_t* batch_x,
                               const int64_t* batch_y, int64_t* idx, float* dist,
                               void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------
 * Ball query with sorted neighbours, dense and packed layouts: the `nsample` nearest support
 * points with d2 < radius*radius, nearest first (equal distances: lower index first).
 * The reference computes this for CPU tensors only, with sort=True: nanoflann_neighbors() /
 * batch_nanoflann_neighbors() (cpu/src/neighbors.cpp:8-136, :139-310, reached through
 * dense_ball_query / batch_ball_query, cpu/src/ball_query.cpp:127-146, :65-124); for CUDA
 * tensors torch_points_kernels/torchpoints.py:152-153 and :163-164 raise.
 * Shapes and dtypes as for tpk_ball_query_dense_f32 / tpk_ball_query_partial_f32.  Unused
 * slots: dense - idx repeats the nearest neighbour (0 when there is none), dist -1; packed -
 * both -1.  With a `workspace` (tpk_ball_query_sorted_*_workspace_bytes() bytes - 0 for
 * shapes not served that way -, 256-byte aligned) the support points are ordered along a
 * space filling curve and a query only visits cells within its radius (clouds of 512 support
 * points or more; up to 64 neighbours one wavefront serves a query; dense layout, clouds of
 * 1024 .. 8192 points, up to 64 neighbours: buckets of cells in LDS, workspace not used), same results as the all
 * pairs scan used otherwise.  In the packed layout up to 64 neighbours are found by the walk
 * over bins of tpk_ball_query_partial_f32 (no wait for the stream); more than 64 cloud by
 * cloud (clouds of up to 163840 points, cloud ids below 1024; others by all pairs), and only
 * then the call waits for the stream once, to read where the clouds start.
 * ------------------------------------------------------------------------------------- */
size_t tpk_ball_query_sorted_dense_workspace_bytes(int b, int n, int m);
int tpk_ball_query_sorted_dense_f32(int b, int n, int m, float radius, int nsample,
                                    const float* new_xyz, const float* xyz, int64_t* idx, float* dist,
                                    void* workspace, size_t workspace_bytes, void* stream);
size_t tpk_ball_query_sorted_partial_workspace_bytes(int64_t size_x, int64_t size_y);
int tpk_ball_query_sorted_partial_f32(int64_t size_x, int64_t size_y, float radius, int nsample,
                                      const float* x, const float* y, const int64_t* batch_x,
                                      const int64_t* batch_y, int64_t* idx, float* dist,
                                      void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------
 * Three nearest neighbours.
 * Replaces three_nn_kernel_wrapper(b, n, m, unknown, known, dist2, idx)
 * (cuda/src/interpolate_gpu.cu:67-76, declared cuda/src/interpolate.cpp:5-6).
 *   unknown (b, n, 3)   known (b, m, 3)
 *   dist2 (b, n, 3) float32 squared distances, ascending   idx (b, n, 3) int32
 * Equal distances keep the lower index first; with m < 3 the missing entries are
 * (+inf, 0).
 * Known clouds of 1024 .. 8192 points are sorted into a grid that every workgroup builds in its
 * local memory, and a query looks at the cells around it only.  With a `workspace`
 * (tpk_three_nn_workspace_bytes() bytes - 0 for shapes not served that way -, 256-byte aligned,
 * contents arbitrary before and after) other shapes, and clouds whose density is too uneven for
 * that grid, are ordered along a space filling curve and only nearby cells are searched; with
 * workspace == NULL the grid answers uneven clouds as well (slower there), and for other shapes
 * all pairs are tested.  Same results every way.
 * tpk_three_nn_all_pairs_f32: the scan of all pairs itself, for any shape (what the reference
 * kernel does; here for measurements and as a check).
 * ------------------------------------------------------------------------------------- */
size_t tpk_three_nn_workspace_bytes(int b, int n, int m);
int tpk_three_nn_f32(int b, int n, int m, const float* unknown, const float* known,
                     float* dist2, int32_t* idx, void* workspace, size_t workspace_bytes,
                     void* stream);
int tpk_three_nn_all_pairs_f32(int b, int n, int m, const float* unknown, const float* known,
                               float* dist2, int32_t* idx, void* stream);

/* ---------------------------------------------------------------------------------------
 * Three nearest neighbours without any allocation.
 * No counterpart in the reference.  It is for callers that cannot allocate device memory (not
 * even a workspace to pass in): code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  Same arguments and results as tpk_three_nn_f32 with a workspace, but
 * the workspace (curve-ordered copies of both clouds, a word per cloud) is an array of
 * TPK_THREE_NN_STATIC_SCRATCH_BYTES bytes of device memory that is part of the library (every GPU
 * the library runs on holds one until the process ends).  The call allocates and frees nothing.
 * Shapes whose workspace (tpk_three_nn_workspace_bytes()) exceeds the array are rejected with
 * TPK_ERR_TOO_LARGE before anything is launched; shapes that need no workspace run the all
 * pairs scan.  All calls on one GPU share that GPU's array, its contents (the per-cloud words
 * included) are whatever the last call left: calls that overlap there (different streams or host
 * threads) race; calls on one stream are safe.  The first call on a device looks up the array's
 * address and sets the kernels' LDS limits (host runtime calls, no allocation): make one call per
 * device before capturing a graph that contains this entry point.
 * ------------------------------------------------------------------------------------- */
#define TPK_THREE_NN_STATIC_SCRATCH_BYTES (8u << 20)
size_t tpk_three_nn_static_scratch_bytes(void);
int tpk_three_nn_static_f32(int b, int n, int m, const float* unknown, const float* known,
                            float* dist2, int32_t* idx, void* stream);

/* ---------------------------------------------------------------------------------------
 * k nearest neighbours, dense layout.
 * Replaces dense_knn(support, query, k) (cpu/src/knn.cpp:43-62, bound in
 * cpu/src/bindings.cpp; torch_points_kernels/knn.py:4-18 refuses CUDA tensors: the reference
 * has no GPU implementation of this operator).
 *   support (b, n_support, 3)   query (b, m_query, 3)
 *   idx (b, m_query, k) int64   dist2 (b, m_query, k) float32 squared distances
 * Entries ascend by (squared distance, index): equal distances keep the lower index first, the
 * rule of three_nn (nanoflann leaves that order open).  k > n_support is TPK_ERR_INVALID_ARG
 * (cpu/src/knn.cpp:12-14 raises).  `workspace` (tpk_knn_workspace_bytes() bytes - 0 for shapes
 * not served that way -, 256-byte aligned): search over curve-ordered cells instead of all
 * pairs, same results.
 * ------------------------------------------------------------------------------------- */
size_t tpk_knn_workspace_bytes(int b, int n_support, int m_query);
int tpk_knn_f32(int b, int n_support, int m_query, int k, const float* support, const float* query,
                int64_t* idx, float* dist2, void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------
 * Three-point interpolation, forward and backward.
 * Replace three_interpolate_kernel_wrapper(b, c, m, n, points, idx, weight, out) and
 * three_interpolate_grad_kernel_wrapper(b, c, n, m, grad_out, idx, weight, grad_points)
 * (cuda/src/interpolate_gpu.cu:109-118 and :154-164, declared cuda/src/interpolate.cpp:7-10).
 *   points (b, c, m)   idx (b, n, 3) int32 in [0, m)   weight (b, n, 3)
 *   out (b, c, n) = sum_t points[b, c, idx[b, n, t]] * weight[b, n, t]
 *   grad_points (b, c, m) += grad_out (b, c, n) scattered back (fully written, no pre-zero)
 * The backward pass inverts the index into per-target lists held in `workspace`
 * (tpk_three_interpolate_grad_workspace_bytes() bytes, 256-byte aligned; contents need not
 * be initialised and are garbage afterwards; about one entry of 8 bytes per index entry and
 * per target).  With workspace == NULL, or for shapes the lists do not serve (m above about
 * 36000: the sums of one row then leave no room in LDS; tpk_..._workspace_bytes() returns 0),
 * it falls back to global float atomics - same result to rounding, much slower.
 * Index values outside [0, m) are ignored by the list path.
 * ------------------------------------------------------------------------------------- */
int tpk_three_interpolate_f32(int b, int c, int m, int n, const float* points,
                              const int32_t* idx, const float* weight, float* out, void* stream);
size_t tpk_three_interpolate_grad_workspace_bytes(int b, int n, int m);
int tpk_three_interpolate_grad_f32(int b, int c, int n, int m, const float* grad_out,
                                   const int32_t* idx, const float* weight, float* grad_points,
                                   void* workspace, size_t workspace_bytes, void* stream);
/* The two halves of tpk_three_interpolate_grad_f32 on their own, for callers that know at the
 * time of the FORWARD pass that a backward pass will follow (autograd is recording): the lists
 * depend on (idx, weight) only, so they can be built then, the backward pass is the walk alone, and
 * several backward passes share one inversion.  `lists`: tpk_three_interpolate_grad_workspace_bytes()
 * bytes, 256-byte aligned, kept by the caller from one call to the other (read-only in the second, so
 * one set of lists serves any number of backward passes).  TPK_ERR_UNSUPPORTED: the lists do not serve
 * the shape (the size function returns 0); use tpk_three_interpolate_grad_f32.  The reference has no
 * counterpart: its backward is three_interpolate_grad_kernel_wrapper with atomics
 * (cuda/src/interpolate_gpu.cu:122-164). */
int tpk_three_interpolate_lists_f32(int b, int n, int m, const int32_t* idx, const float* weight,
                                    void* lists, size_t lists_bytes, void* stream);
int tpk_three_interpolate_grad_lists_f32(int b, int c, int n, int m, const float* grad_out,
                                         void* lists, size_t lists_bytes, float* grad_points,
                                         void* stream);

/* ---------------------------------------------------------------------------------------
 * Grouping (gather of feature columns), forward and backward.
 * The reference has no native code for this: it is `features.gather(2, idx repeated over
 * channels)` plus autograd (torch_points_kernels/torchpoints.py:129-146).  These two entry
 * points compute the same without materialising the repeated index.
 *   features (b, c, n)   idx (b, npoint, nsample) int64 in [0, n)
 *   out (b, c, npoint, nsample) = features[b, c, idx[b, p, s]]
 *   grad_features (b, c, n) = scatter-add of grad_out (fully written, no pre-zero)
 * `workspace`: as for tpk_three_interpolate_grad_f32 (tpk_group_grad_workspace_bytes()).
 * ------------------------------------------------------------------------------------- */
int tpk_group_f32(int b, int c, int n, int npoint, int nsample, const float* features,
                  const int64_t* idx, float* out, void* stream);
size_t tpk_group_grad_workspace_bytes(int b, int n, int npoint, int nsample);
int tpk_group_grad_f32(int b, int c, int n, int npoint, int nsample, const float* grad_out,
                       const int64_t* idx, float* grad_features, void* workspace,
                       size_t workspace_bytes, void* stream);
/* The two halves of tpk_group_grad_f32 on their own, as for the interpolation above (`lists`:
 * tpk_group_grad_workspace_bytes() bytes). */
int tpk_group_lists(int b, int n, int npoint, int nsample, const int64_t* idx, void* lists,
                    size_t lists_bytes, void* stream);
int tpk_group_grad_lists_f32(int b, int c, int n, int npoint, int nsample, const float* grad_out,
                             void* lists, size_t lists_bytes, float* grad_features, void* stream);

/* ---------------------------------------------------------------------------------------
 * Chamfer distance, forward (both directions) and backward.
 * Replace chamfer_dist_kernel_wrapper(xyz1, xyz2) and chamfer_dist_grad_kernel_wrapper(
 * xyz1, xyz2, idx1, idx2, grad_dist1, grad_dist2) (cuda/src/chamfer_dist_gpu.cu:157-184 and
 * :215-245, declared cuda/include/chamfer_dist.h:4-15), which take tensors; here they take
 * the raw arrays.
 *   xyz1 (b, n, 3)  xyz2 (b, m, 3)
 *   dist1 (b, n) squared distance of each xyz1 point to its nearest xyz2 point, idx1 (b, n)
 *   int32 its index (lowest index on ties); dist2 (b, m), idx2 (b, m) the other direction.
 *   grad_xyz1 (b, n, 3), grad_xyz2 (b, m, 3): fully written, no pre-zero needed.
 * n == 0 or m == 0 yields zeros, as the reference's zero-initialised outputs do.
 * The float32 forward pass orders both clouds along a space filling curve into `workspace`
 * (tpk_chamfer_fwd_workspace_bytes() bytes - 0 for shapes it does not serve that way -, 256-byte
 * aligned, contents arbitrary before and after) and searches only nearby cells; with
 * workspace == NULL, and always in float64, it tests all pairs (same results, slower).
 * The backward pass needs no workspace (tpk_chamfer_bwd_workspace_bytes() returns 0; the
 * arguments are kept for callers written against earlier versions and are ignored): the points
 * that chose a point as nearest neighbour are chained to it in LDS.  Clouds of more than about
 * 38000 points scatter with hardware float atomics instead.
 * ------------------------------------------------------------------------------------- */
size_t tpk_chamfer_fwd_workspace_bytes(int b, int n, int m);
int tpk_chamfer_fwd_f32(int b, int n, int m, const float* xyz1, const float* xyz2, float* dist1,
                        float* dist2, int32_t* idx1, int32_t* idx2, void* workspace,
                        size_t workspace_bytes, void* stream);
int tpk_chamfer_fwd_f64(int b, int n, int m, const double* xyz1, const double* xyz2,
                        double* dist1, double* dist2, int32_t* idx1, int32_t* idx2,
                        void* stream);
size_t tpk_chamfer_bwd_workspace_bytes(int b, int n, int m);
int tpk_chamfer_bwd_f32(int b, int n, int m, const float* xyz1, const float* xyz2,
                        const int32_t* idx1, const int32_t* idx2, const float* grad_dist1,
                        const float* grad_dist2, float* grad_xyz1, float* grad_xyz2,
                        void* workspace, size_t workspace_bytes, void* stream);
int tpk_chamfer_bwd_f64(int b, int n, int m, const double* xyz1, const double* xyz2,
                        const int32_t* idx1, const int32_t* idx2, const double* grad_dist1,
                        const double* grad_dist2, double* grad_xyz1, double* grad_xyz2,
                        void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------
 * Clusters grown over a neighbour matrix (PointGroup's region growing).
 * Replaces _grow_proximity_core(neighbours, min_cluster_size), the numba routine that
 * grow_proximity() runs on the host after copying the matrix there
 * (torch_points_kernels/cluster.py:9-37, called at :40-45 and from region_grow() at :48-109);
 * the reference has no device code for it.
 *   neighbours (n, nsample) int64: row i lists neighbours of point i and ends at its first -1
 *     (what ball_query_partial_dense returns for a self query); entries in [-1, n), a row
 *     repeats no index.
 *   members (n) int64: the clusters with at least min_cluster_size members, one after the
 *     other, ordered by their first (smallest) point as the reference orders them;
 *     starts (n + 1) int64: their offsets into `members`, then the total.
 *   found (2, HOST memory): number of clusters, number of members written.  Only that many
 *     entries of starts (+1) and members are defined.
 *   member_order: TPK_MEMBERS_AS_REFERENCE - inside a cluster, the order of the reference's
 *     lists (the order its stack walk appends points; a serial walk per cluster, clusters in
 *     parallel); TPK_MEMBERS_BY_INDEX - ascending index (all steps data-parallel; same
 *     clusters, same cluster order).
 * `workspace`: tpk_grow_proximity_workspace_bytes(n, nsample) bytes (0 when n is 0, beyond 2^30, or
 * no device is present to size the sort's temporary storage), 256-byte aligned, required.
 * This entry point waits for the stream (several times): the number of label sweeps and the
 * output sizes depend on the data.
 * ------------------------------------------------------------------------------------- */
#define TPK_MEMBERS_AS_REFERENCE 0
#define TPK_MEMBERS_BY_INDEX 1
size_t tpk_grow_proximity_workspace_bytes(int64_t n, int nsample);
int tpk_grow_proximity(int64_t n, int nsample, const int64_t* neighbours, int64_t min_cluster_size,
                       int member_order, int64_t* members, int64_t* starts, int64_t* found,
                       void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------
 * IoU between proposed instances and ground-truth instances.
 * Replaces instance_iou_kernel_wrapper(total_gt_instances, max_gt_instances, nInstance,
 * nProposal, proposals_idx, proposals_offset, instance_labels, offset_num_gt_instances, batch,
 * instance_pointnum, proposals_iou) (cuda/src/metrics_gpu.cu:50-61, declared
 * cuda/src/metrics.cpp:5-10; max_gt_instances only sized the reference's blocks).
 *   proposals_idx (sum of proposal sizes) int64: point indices, proposal after proposal
 *   proposals_offset (n_proposals + 1) int64     instance_labels (n_points) int64: k + 1 for
 *   ground-truth instance k of the point's sample, 0 or negative for none
 *   batch (n_points) int64: sample of a point     num_gt_instances, offset_num_gt_instances
 *   (n_samples, n_samples + 1) int64: instances per sample and their first output column
 *   instance_pointnum (total_gt_instances) int64: points per ground-truth instance
 *   proposals_iou (n_proposals, total_gt_instances) float32: intersection / (union + 1e-5)
 *   with the instances of the sample of the proposal's first point, 0 elsewhere.
 * n_points and n_samples bound what the kernel reads; indices outside are ignored.
 * ------------------------------------------------------------------------------------- */
int tpk_instance_iou(int64_t total_gt_instances, int64_t n_proposals, int64_t n_points, int64_t n_samples,
                     const int64_t* num_gt_instances, const int64_t* proposals_idx,
                     const int64_t* proposals_offset, const int64_t* instance_labels,
                     const int64_t* offset_num_gt_instances, const int64_t* batch,
                     const int64_t* instance_pointnum, float* proposals_iou, void* stream);

/* ---------------------------------------------------------------------------------------
 * Gridding (GRNet): point clouds to occupancy grids by trilinear weights, and the gradient.
 * Replaces gridding_kernel_warpper(min_x, max_x, min_y, max_y, min_z, max_z, ptcloud, stream)
 * and gridding_grad_kernel_warpper(grid_pt_weights, grid_pt_indexes, grad_grid, stream)
 * (cuda/src/gridding_gpu.cu:193-218, :307-331; host functions cuda/src/gridding.cpp:4-26).
 *   ptcloud (b, n_pts, 3) in grid units; the grid spans [min, max] per axis, len = max-min+1
 *   grid_weights (b, len_x*len_y*len_z): sum over points of wx*wy*wz at the 8 vertices around
 *   a point, w = 1 - |coordinate - vertex|; grid_pt_weights (b, n_pts, 8, 3) the three factors,
 *   grid_pt_indexes (b, n_pts, 8) int32 the vertices (order LLL, LLU, LUL, LUU, ULL, ULU, UUL,
 *   UUU; -1 for a vertex outside the grid, where the reference computes an index regardless).
 *   grad_grid (b, n_grid_vertices) -> grad_ptcloud (b, n_pts, 3).
 * float32 and float64 (the reference dispatches on both).  Sums into the grid are atomic, in
 * no fixed order; the gradient is summed in the reference's order.
 * ------------------------------------------------------------------------------------- */
int tpk_gridding_f32(int b, int n_pts, float min_x, float max_x, float min_y, float max_y, float min_z,
                     float max_z, const float* ptcloud, float* grid_weights, float* grid_pt_weights,
                     int32_t* grid_pt_indexes, void* stream);
int tpk_gridding_f64(int b, int n_pts, float min_x, float max_x, float min_y, float max_y, float min_z,
                     float max_z, const double* ptcloud, double* grid_weights, double* grid_pt_weights,
                     int32_t* grid_pt_indexes, void* stream);
int tpk_gridding_grad_f32(int b, int n_pts, int n_grid_vertices, const float* grid_pt_weights,
                          const int32_t* grid_pt_indexes, const float* grad_grid, float* grad_ptcloud,
                          void* stream);
int tpk_gridding_grad_f64(int b, int n_pts, int n_grid_vertices, const double* grid_pt_weights,
                          const int32_t* grid_pt_indexes, const double* grad_grid, double* grad_ptcloud,
                          void* stream);

/* ---------------------------------------------------------------------------------------
 * Cubic feature sampling (GRNet): the features of the grid vertices around every point.
 * Replaces cubic_feature_sampling_kernel_wrapper(scale, neighborhood_size, ptcloud,
 * cubic_features, stream) and cubic_feature_sampling_grad_kernel_wrapper(scale,
 * neighborhood_size, grad_point_features, grid_pt_indexes, stream)
 * (cuda/src/cubic_feature_sampling_gpu.cu:107-136, :177-210; host functions
 * cuda/src/cubic_feature_sampling.cpp:4-30).
 *   ptcloud (b, n_pts, 3) in grid units   cubic_features (b, channels, scale, scale, scale)
 *   point_features (b, n_pts, n_vertices, channels), n_vertices = (2*neighborhood_size)^3:
 *   the features at the vertices floor-(ns-1) .. ceil+(ns-1) per axis, x slowest; 0 where the
 *   vertex lies outside the grid; grid_pt_indexes (b, n_pts, n_vertices) int32, -1 outside.
 *   Gradient: grad_cubic_features (b, channels, scale^3) = scatter-add of grad_point_features;
 *   grad_ptcloud (b, n_pts, 3) = 0 (the coordinates only choose vertices).
 * ------------------------------------------------------------------------------------- */
int tpk_cubic_feature_sampling_f32(int b, int n_pts, int channels, int scale, int neighborhood_size,
                                   const float* ptcloud, const float* cubic_features, float* point_features,
                                   int32_t* grid_pt_indexes, void* stream);
int tpk_cubic_feature_sampling_f64(int b, int n_pts, int channels, int scale, int neighborhood_size,
                                   const double* ptcloud, const double* cubic_features, double* point_features,
                                   int32_t* grid_pt_indexes, void* stream);
int tpk_cubic_feature_sampling_grad_f32(int b, int n_pts, int channels, int scale, int neighborhood_size,
                                        const float* grad_point_features, const int32_t* grid_pt_indexes,
                                        float* grad_ptcloud, float* grad_cubic_features, void* stream);
int tpk_cubic_feature_sampling_grad_f64(int b, int n_pts, int channels, int scale, int neighborhood_size,
                                        const double* grad_point_features, const int32_t* grid_pt_indexes,
                                        double* grad_ptcloud, double* grad_cubic_features, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TPK_H */
