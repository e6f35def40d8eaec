// Nearest-neighbour searches over curve-ordered cells (nn_grid.hip), as seen by the entry
// points of the all-pairs kernels, which hand suitable problems over when a workspace is given.
#pragma once

#include "tpk_device.h"

// Bytes of workspace tpk_grid_chamfer_fwd needs for b pairs of n- and m-point clouds; 0 when it
// does not serve that shape (callers then use the all-pairs scan).
size_t tpk_grid_chamfer_workspace_bytes(int b, int n, int m);

// Chamfer forward, both directions, float32.  TPK_ERR_UNSUPPORTED when the shape is not served,
// TPK_ERR_WORKSPACE when the workspace is missing, too small or not 256-byte aligned.
int tpk_grid_chamfer_fwd(int b, int n, int m, const float* xyz1, const float* xyz2, float* dist1,
                         float* dist2, int32_t* idx1, int32_t* idx2, void* workspace,
                         size_t workspace_bytes, hipStream_t stream);

// three_nn, float32: same conventions.  The workspace ends with one word per cloud
// (tpk_grid_three_nn_flags: its address, or nullptr when the workspace does not serve the shape); with
// `flagged` only the clouds whose word is not 0 are searched - a kernel enqueued before has answered the others.
size_t tpk_grid_three_nn_workspace_bytes(int b, int n, int m);
int* tpk_grid_three_nn_flags(int b, int n, int m, void* workspace, size_t workspace_bytes);
int tpk_grid_three_nn(int b, int n, int m, const float* unknown, const float* known, float* dist2,
                      int32_t* idx, void* workspace, size_t workspace_bytes, bool flagged, hipStream_t stream);

// k nearest neighbours, float32 (n queries, m support points per cloud; idx int64, both outputs
// (b, n, k), ascending by (squared distance, index)): same conventions.  Only support points with
// squared distance < limit count (+inf: all); entries that stay empty are written as (limit, 0).
size_t tpk_grid_knn_workspace_bytes(int b, int n, int m);
int tpk_grid_knn(int b, int n, int m, int k, float limit, const float* query, const float* support, float* dist2,
                 int64_t* idx, void* workspace, size_t workspace_bytes, hipStream_t stream);

// Ball query with sorted neighbours, float32, one wavefront per query: the nsample (<= 64) nearest of the
// m support points of the query's cloud with squared distance < limit, nearest first; only the support
// points are ordered (workspace for b clouds of m points).  Writes every slot: unused ones are -1 / -1
// when `packed`, else (index of the nearest, or 0) / -1; indices are raised by index_add.
size_t tpk_grid_ball_sorted_workspace_bytes(int b, int m);
int tpk_grid_ball_sorted(int b, int n, int m, int nsample, float limit, bool packed, int64_t index_add,
                         const float* query, const float* support, float* dist, int64_t* idx, void* workspace,
                         size_t workspace_bytes, hipStream_t stream);

// Ball query, packed layout (a hit has squared distance <= radius2 = radius * radius as the caller
// rounds it): same conventions.  Queries with dense neighbourhoods are answered by a scan in
// index order inside the same kernel.  `sorted`: the nsample (<= 64) nearest points with squared
// distance < radius2 instead, nearest first (equal distances: lower row first), -1 behind them.
size_t tpk_grid_ball_query_workspace_bytes(int64_t size_x, int64_t size_y, int nsample);
int tpk_grid_ball_query_partial(int64_t size_x, int64_t size_y, float radius, float radius2, int nsample, bool sorted,
                                const float* x, const float* y, const int64_t* batch_x,
                                const int64_t* batch_y, int64_t* idx, float* dist, void* workspace,
                                size_t workspace_bytes, hipStream_t stream);

// Ball query, dense layout (b clouds of n points, m queries each; cuda/src/ball_query_gpu.cu:9-52), for clouds
// above 8192 points: the bin walk of the packed layout under the dense layout's rules (hit: squared distance
// < radius2; indices inside the cloud; the slots behind the last hit repeat the first, 0 without any; distance -1).
size_t tpk_grid_ball_query_dense_workspace_bytes(int b, int n, int m, int nsample);
int tpk_grid_ball_query_dense(int b, int n, int m, float radius, float radius2, int nsample, const float* new_xyz,
                              const float* xyz, int64_t* idx, float* dist, void* workspace, size_t workspace_bytes,
                              hipStream_t stream);
