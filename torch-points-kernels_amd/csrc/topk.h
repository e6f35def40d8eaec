// The k nearest candidates of one query, kept by one lane: K entries sorted by (squared distance,
// index), for the k-nearest-neighbour kernels (knn.hip: all pairs; nn_grid.hip: search over
// curve-ordered cells).  The order by (distance, index) is the one a serial scan in index
// order with strictly-smaller insertion ends with (the rule of the reference's three_nn kernel,
// cuda/src/interpolate_gpu.cu:9-65), whatever order the candidates arrive in.
#pragma once

#include "tpk_device.h"

namespace {

constexpr int KNN_MAX_K = 32; // entries a lane keeps; larger k is served in rounds of this many

// A (squared distance, index) pair as one integer: distances are >= 0, so their bit patterns
// order like unsigned integers, and one 64-bit comparison orders by distance, then index.
__device__ __forceinline__ unsigned long long knn_key(float d, int i)
{
    return (static_cast<unsigned long long>(static_cast<unsigned>(__float_as_int(d))) << 32) |
           static_cast<unsigned>(i);
}

using u64 = unsigned long long;

// The 64 keys of a wavefront sorted across its lanes (bitonic network; lane i ends with the i-th
// smallest, or the i-th largest when `descending`).
__device__ __forceinline__ u64 wave_sort_keys(u64 key, int lane, bool descending)
{
#pragma unroll
    for (int k = 2; k <= TPK_WAVE; k <<= 1)
#pragma unroll
        for (int j = k >> 1; j > 0; j >>= 1)
        {
            const u64 other = __shfl_xor(key, j, TPK_WAVE);
            const bool up = ((lane & k) == 0) != descending;
            const bool keep_min = ((lane & j) == 0) == up;
            key = (keep_min == (key < other)) ? key : other;
        }
    return key;
}

// A bitonic sequence across the lanes put into ascending order.
__device__ __forceinline__ u64 wave_merge_ascending(u64 key, int lane)
{
#pragma unroll
    for (int j = TPK_WAVE / 2; j > 0; j >>= 1)
    {
        const u64 other = __shfl_xor(key, j, TPK_WAVE);
        key = (((lane & j) == 0) == (key < other)) ? key : other;
    }
    return key;
}

__device__ __forceinline__ u64 read_lane_key(u64 key, int from)
{
    const unsigned lo = __builtin_amdgcn_readlane(static_cast<int>(key & 0xFFFFFFFFu), from);
    const unsigned hi = __builtin_amdgcn_readlane(static_cast<int>(key >> 32), from);
    return (static_cast<u64>(hi) << 32) | lo;
}

template <int K>
struct NearestK
{
    unsigned long long key[K]; // ascending
    // Entries must come after this pair (the last one found by the round before; 0 with
    // `from_start` in the first round).
    unsigned long long after;
    bool from_start;

    // An inert lane (no query) never admits a candidate.  Only candidates closer than `limit`
    // (squared; +inf for a plain k-nearest search) are admitted; entries that stay empty read
    // (limit, 0), which no candidate equals.
    __device__ __forceinline__ void reset(bool later_round, float last_d, int last_i, bool inert, float limit)
    {
        const unsigned long long empty = knn_key(limit, limit == __builtin_inff() ? 0x7FFFFFFF : 0);
#pragma unroll
        for (int j = 0; j < K; ++j)
            key[j] = inert ? 0ull : empty;
        after = later_round ? knn_key(last_d, last_i) : 0ull;
        from_start = !later_round;
    }
    // Squared distance of the last entry (the limit while the list is not full; -1 for an inert lane).
    __device__ __forceinline__ float worst() const
    {
        return key[K - 1] == 0ull ? -1.f : __int_as_float(static_cast<int>(key[K - 1] >> 32));
    }
    // True when the pair belongs into the list.
    __device__ __forceinline__ bool admits(unsigned long long cand) const
    {
        return cand < key[K - 1] && (from_start || cand > after);
    }
    // Inserts a pair that admits() accepted.
    __device__ __forceinline__ void insert(unsigned long long cand)
    {
        bool before_this = true; // cand < key[K - 1]
#pragma unroll
        for (int j = K - 1; j > 0; --j)
        {
            const bool before_prev = cand < key[j - 1];
            key[j] = before_prev ? key[j - 1] : (before_this ? cand : key[j]);
            before_this = before_prev;
        }
        key[0] = before_this ? cand : key[0];
    }
    __device__ __forceinline__ float dist(int j) const
    {
        return __int_as_float(static_cast<int>(key[j] >> 32));
    }
    __device__ __forceinline__ int index(int j) const
    {
        return static_cast<int>(key[j] & 0xFFFFFFFFull);
    }
};

} // namespace
