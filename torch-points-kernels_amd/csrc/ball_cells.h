// Ball query, dense layout, over buckets of cells in LDS (ball_query.hip): clouds of 1024 .. 8192 support
// points.  `sorted`: the nsample (<= 64) nearest points inside the radius, nearest first, instead of the
// first nsample in index order.  TPK_ERR_UNSUPPORTED (nothing launched) for other shapes.
#pragma once

#include <cstdint>
#include <hip/hip_runtime.h>

int tpk_cells_ball_query_dense(int b, int n, int m, float radius, float radius2, int nsample, bool sorted,
                               const float* new_xyz, const float* xyz, int64_t* idx, float* dist, hipStream_t s);
