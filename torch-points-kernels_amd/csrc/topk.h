// The k nearest candidates of one query, kept by one lane: K entries sorted by (squared distance,
// index), for the k-nearest-neighbour kernels (knn.hip: all pairs; nn_grid.hip: search over
// curve-ordered cells).  The order by (distance, index) is the one a serial scan in index
// order with strictly-smaller insertion ends with (the rule of the reference's three_nn kernel,
// cuda/src/interpolate_gpu.cu:9-65), whatever order the candidates arrive in.
#pragma once

#include "tpk_device.h"

namespace {

constexpr int KNN_MAX_K = 32; // entries a lane keeps; larger k is served in rounds of this many

__device__ __forceinline__ bool knn_pair_less(float d, int ci, float b, int i)
{
    return d < b || (d == b && ci < i);
}

template <int K>
struct NearestK
{
    float d[K];
    int i[K];
    // Entries must come after this pair (the last one found by the round before; (-1, -1) in the
    // first round: every distance is >= 0).
    float after_d;
    int after_i;

    __device__ __forceinline__ void reset(float from_d, int from_i, bool inert)
    {
#pragma unroll
        for (int j = 0; j < K; ++j)
        {
            d[j] = inert ? -1.f : __builtin_inff(); // (an inert lane never admits a candidate)
            i[j] = inert ? -1 : 0x7FFFFFFF;
        }
        after_d = from_d;
        after_i = from_i;
    }
    // True when (dist, ci) belongs into the list.
    __device__ __forceinline__ bool admits(float dist, int ci) const
    {
        return knn_pair_less(dist, ci, d[K - 1], i[K - 1]) && knn_pair_less(after_d, after_i, dist, ci);
    }
    // Inserts a pair that admits() accepted.
    __device__ __forceinline__ void insert(float dist, int ci)
    {
#pragma unroll
        for (int j = K - 1; j > 0; --j)
        {
            const bool before_prev = knn_pair_less(dist, ci, d[j - 1], i[j - 1]);
            const bool before_this = knn_pair_less(dist, ci, d[j], i[j]);
            d[j] = before_prev ? d[j - 1] : (before_this ? dist : d[j]);
            i[j] = before_prev ? i[j - 1] : (before_this ? ci : i[j]);
        }
        const bool first = knn_pair_less(dist, ci, d[0], i[0]);
        d[0] = first ? dist : d[0];
        i[0] = first ? ci : i[0];
    }
};

} // namespace
