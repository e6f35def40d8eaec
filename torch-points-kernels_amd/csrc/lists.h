// Inverted index ("lists"): for every target position of a cloud, the entries that refer to
// it.  The backward passes that would otherwise scatter with float atomics (three_interpolate,
// grouping) gather along these lists instead.
//
// Layout, made for the walk of gather.hip (one wavefront per span of targets, 64 lanes that
// each add up a run of consecutive entries):
//   * The index entries of one cloud - or of one column part of it - are sorted by target.
//     A target nobody refers to gets one empty entry, so every target owns at least one entry
//     and the last entry of every list is marked: a walker that counts these marks knows which
//     target a sum belongs to, and every output element gets written (no zero fill).
//   * The targets are cut into L_SPANS spans of equal size; span s is walked by wavefront s.
//     Its sorted entries, `len` of them, are dealt to the 64 lanes in runs of
//     c = ceil(len / 64) consecutive entries: the entry of rank q goes to lane q / c as its
//     step q % c, stored at  base + (q % c) * 64 + q / c  - one step of all lanes is one
//     contiguous row of 64 entries; the places behind rank len - 1 hold entries that refer to
//     nothing.  Runs are equally long whatever the lists look like; a list may cross from one
//     lane's run into the next, which the walker resolves with one scan over the lanes at the end.
//   * regions[cloud_part][span]              (base, len, c, 0)
//     first_target[cloud_part][span][lane]   target of the lane's first entry
//     entries[cloud_part][capacity]
#pragma once

#include "tpk_device.h"

namespace {

constexpr int G_THREADS = 1024;

template <typename Kernel>
int allow_lds(Kernel kernel, size_t bytes)
{
    return tpk_allow_lds(reinterpret_cast<const void*>(kernel), bytes);
}

// One entry of a target's list: the column that references it and the weight it carries.  The
// column is stored the way the walker uses it: as the byte offset of that column's value in a
// staged row, column * 4.  Bit 31 marks the last entry of a list.  An entry that refers to
// nothing (the entry of an empty list, the entries that fill a span's last row) carries
// L_NOTHING, an offset beyond the LDS: reads there return zero on gfx950, as on every GCN / CDNA
// part, and never fault.
template <bool WEIGHTED>
struct ListEntry;
template <>
struct ListEntry<true>
{
    int j;
    float w;
};
template <>
struct ListEntry<false>
{
    int j;
};
constexpr int L_LAST = static_cast<int>(0x80000000u);
constexpr int L_NOTHING = 0x7ffffffc - 3 * 0x40000; // (rows further down, at multiples of the row size, stay out of range too)
// The walker multiplies the offset by the number of rows it stages side by side (1, 2 or 4), in 32 bits: every
// product has to stay beyond the LDS.
static_assert(static_cast<uint32_t>(L_NOTHING) * 1u >= TPK_LDS_BYTES && static_cast<uint32_t>(L_NOTHING) * 2u >= TPK_LDS_BYTES &&
                  static_cast<uint32_t>(L_NOTHING) * 4u >= TPK_LDS_BYTES,
              "an entry that refers to nothing must read beyond the LDS whatever the number of staged rows");

constexpr int L_SPANS = G_THREADS / TPK_WAVE; // spans of targets per cloud: one per wavefront of the walker
constexpr int L_MAX_SPAN = 15360;             // targets of a span: their bookkeeping (2 ints each) fits in LDS
constexpr int L_REGION_GAP = 128;             // entry slots between the regions of consecutive spans
constexpr int L_CACHED = 48;                  // index values a thread keeps in registers between the two passes
constexpr int L_QUEUE = 128;                  // places of a wavefront's queue of entries inside the span (a power of two >= 128)

template <bool WEIGHTED>
struct Lists
{
    int4* regions;
    int* first_target;
    ListEntry<WEIGHTED>* entries;
    int64_t capacity; // entry slots per cloud part
};

inline size_t list_align(size_t v)
{
    return (v + 255) & ~static_cast<size_t>(255);
}
// Entry slots of one cloud part with m targets and `total` index entries: every entry, one
// empty entry per target at most, the rounding of every region to whole rows of 64 and the gaps.
inline int64_t list_capacity(int m, int64_t total)
{
    return ((total + m + 63) & ~static_cast<int64_t>(63)) + static_cast<int64_t>(L_REGION_GAP) * L_SPANS + 64;
}
// Workspace bytes of the lists of `clouds` cloud parts with m targets and `total` index entries each.
template <bool WEIGHTED>
size_t lists_bytes(int64_t clouds, int m, int64_t total)
{
    const size_t c = static_cast<size_t>(clouds);
    return list_align(c * L_SPANS * sizeof(int4)) + list_align(c * L_SPANS * TPK_WAVE * sizeof(int)) +
           list_align(c * static_cast<size_t>(list_capacity(m, total)) * sizeof(ListEntry<WEIGHTED>));
}
template <bool WEIGHTED>
Lists<WEIGHTED> lists_at(void* workspace, int64_t clouds, int m, int64_t total)
{
    const size_t c = static_cast<size_t>(clouds);
    char* p = static_cast<char*>(workspace);
    Lists<WEIGHTED> l;
    l.regions = reinterpret_cast<int4*>(p);
    p += list_align(c * L_SPANS * sizeof(int4));
    l.first_target = reinterpret_cast<int*>(p);
    p += list_align(c * L_SPANS * TPK_WAVE * sizeof(int));
    l.entries = reinterpret_cast<ListEntry<WEIGHTED>*>(p);
    l.capacity = list_capacity(m, total);
    return l;
}

// The job of inverting the index of `clouds` clouds: the `cloud_total` index entries of a cloud
// (K per column) are cut into `parts` runs of `part_total` entries (a multiple of K; the last may
// be shorter), and every (cloud, part) gets lists of its own, stored as cloud part number
// cloud * parts + part; the columns in its entries count from the first column of the part.
template <bool WEIGHTED, typename IdxT>
struct ListJob
{
    int m, cloud_total, parts, part_total, span, workgroups;
    const IdxT* idx;
    const float* weight;
    Lists<WEIGHTED> lists;
};

// grid: (clouds * parts * L_SPANS); workgroup (cloud part, s) builds the lists of the targets
// [s * span, (s + 1) * span).  It reads every index entry of its part (keeping the first
// L_CACHED values per thread in registers for the second pass), counts those inside its span
// with LDS integer atomics and those below it - their number fixes where its region starts, so
// no workgroup waits for another -, prefix-sums the list lengths (empty lists count as one
// entry) and places its entries in a second pass.  Index values outside [0, m) are dropped.
// dynamic LDS: (2 * span + G_THREADS / 64 + 2) ints + the queues (L_QUEUE x 8 bytes per wavefront).
template <int K, bool WEIGHTED, typename IdxT>
__global__ __launch_bounds__(G_THREADS) void build_lists_kernel(ListJob<WEIGHTED, IdxT> job)
{
    const int m = job.m, cloud_total = job.cloud_total, parts = job.parts, part_total = job.part_total, span = job.span;
    const IdxT* __restrict__ idx = job.idx;
    const float* __restrict__ weight = job.weight;

    extern __shared__ int counters[];           // [span] list lengths, in the second pass the places still free
    int* const ends = counters + span;          // [span] rank behind every list's last entry inside the span
    int* const scan = ends + span;              // [G_THREADS / 64], then below_total
    int* const below_total = scan + G_THREADS / TPK_WAVE;
    const int tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int wave = tid / TPK_WAVE;
    const int cloud_part = blockIdx.x / L_SPANS;
    const int s = blockIdx.x - cloud_part * L_SPANS;
    const int part = cloud_part % parts;
    const int total = min(part_total, cloud_total - part * part_total);
    const int i0 = min(s * span, m);
    const int i1 = min(i0 + span, m);
    const int width = i1 - i0;
    const int64_t first_entry = static_cast<int64_t>(cloud_part / parts) * cloud_total + static_cast<int64_t>(part) * part_total;
    idx += first_entry;
    if (WEIGHTED)
        weight += first_entry;

    for (int t = tid; t < width; t += G_THREADS)
        counters[t] = 0;
    if (tid == 0)
        *below_total = 0;
    __syncthreads();

    // First pass.  Entry e of the part is read by thread e % G_THREADS in its round e / G_THREADS.
    int cached[L_CACHED];
    int below = 0; // valid entries whose target lies before this span
    auto count_one = [&](int v) {
        below += (v >= 0 && v < i0) ? 1 : 0;
        if (v >= i0 && v < i1)
            atomicAdd(&counters[v - i0], 1);
    };
    // (a value that does not fit 32 bits is outside every cloud: -1, like an entry behind the part's last)
    auto index_value = [&](int e) {
        const int64_t v = static_cast<int64_t>(idx[min(e, total - 1)]);
        return (e < total && v >= 0 && v < m) ? static_cast<int>(v) : -1;
    };
    constexpr int BATCH = 16; // index loads in flight per thread
    static_assert(L_CACHED % BATCH == 0, "the cached rounds are whole batches");
#pragma unroll
    for (int b = 0; b < L_CACHED; b += BATCH)
    {
        if (b * G_THREADS < total) // (wave-uniform)
        {
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
                cached[b + u] = index_value((b + u) * G_THREADS + tid);
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
                count_one(cached[b + u]);
        }
        else
        {
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
                cached[b + u] = -1;
        }
    }
    for (int e0 = L_CACHED * G_THREADS + tid; e0 < total; e0 += BATCH * G_THREADS)
    {
        int iv[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
            iv[u] = index_value(e0 + u * G_THREADS);
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
            count_one(iv[u]);
    }
    {
        const int below_before = wave_exclusive_sum(below);
        if (lane == TPK_WAVE - 1)
            atomicAdd(below_total, below_before + below);
    }
    __syncthreads();

    // Prefix sum of the list lengths, an empty list counting as one entry (every thread owns a run of
    // `per` consecutive targets; sums inside a wavefront by DPP, across wavefronts through LDS).
    const int per = (width + G_THREADS - 1) / G_THREADS;
    const int lo = min(tid * per, width), hi = min(lo + per, width);
    int sum = 0;
    for (int t = lo; t < hi; ++t)
        sum += max(counters[t], 1);
    const int before_in_wave = wave_exclusive_sum(sum);
    if (lane == TPK_WAVE - 1)
        scan[wave] = before_in_wave + sum;
    __syncthreads();
    int run = before_in_wave, len = 0;
    for (int w = 0; w < G_THREADS / TPK_WAVE; ++w)
    {
        run += w < wave ? scan[w] : 0;
        len += scan[w];
    }
    // Where this span's region starts: behind all entries and all possible empty entries of the spans before it,
    // on a multiple of 64, with a gap that absorbs the rounding of the earlier regions to whole rows.
    const int base = ((*below_total + i0 + 63) & ~63) + L_REGION_GAP * s;
    const int c = (len + TPK_WAVE - 1) / TPK_WAVE; // steps of a lane; 0 for a span without targets
    ListEntry<WEIGHTED>* __restrict__ entries = job.lists.entries + static_cast<int64_t>(cloud_part) * job.lists.capacity;
    int* __restrict__ first_target = job.lists.first_target + (static_cast<int64_t>(cloud_part) * L_SPANS + s) * TPK_WAVE;
    if (tid == 0)
        job.lists.regions[static_cast<int64_t>(cloud_part) * L_SPANS + s] = make_int4(base, len, c, 0);
    // (rank -> lane and step: a division by c through the reciprocal in float, corrected; ranks stay below 2^24)
    const float per_c = c > 0 ? 1.0f / static_cast<float>(c) : 0.f;
    auto place = [&](int rank, int target, ListEntry<WEIGHTED> entry) {
        int ln = static_cast<int>(static_cast<float>(rank) * per_c);
        int step = rank - ln * c;
        if (step < 0)
        {
            --ln;
            step += c;
        }
        if (step >= c)
        {
            ++ln;
            step -= c;
        }
        entries[base + step * TPK_WAVE + ln] = entry;
        if (step == 0)
            first_target[ln] = target;
    };
    for (int t = lo; t < hi; ++t)
    {
        const int n = counters[t];
        run += max(n, 1);
        ends[t] = run;
        if (n == 0) // the empty list's entry: refers to nothing, ends the list
        {
            ListEntry<WEIGHTED> entry;
            entry.j = L_NOTHING | L_LAST;
            if constexpr (WEIGHTED)
                entry.w = 0.f;
            place(run - 1, i0 + t, entry);
        }
    }
    // the places behind the span's last entry, up to the end of the lanes' runs: entries that refer to nothing
    for (int rank = len + tid; rank < c * TPK_WAVE; rank += G_THREADS)
    {
        ListEntry<WEIGHTED> entry;
        entry.j = L_NOTHING;
        if constexpr (WEIGHTED)
            entry.w = 0.f;
        place(rank, 0, entry);
    }
    __syncthreads();

    // Second pass.  Only one entry in L_SPANS lies inside the span: a wavefront first gathers those of its lanes
    // into a queue of its own in LDS (ballot + prefix count), and whenever 64 are waiting every lane takes one:
    // the next free place of its list, front to back.  `counters` holds the number of places still free, so the
    // entry that takes the last one knows that it ends the list.
    int2* const queue = reinterpret_cast<int2*>(below_total + 2) + wave * L_QUEUE;
    int queued = 0, placed = 0; // (wave-uniform)
    // An entry's weight is a trip to memory: the 64 entries taken from the queue wait for theirs while the next
    // ones are queued, and go to their places when the queue has filled again (or at the end).
    bool waiting = false; // per lane: an entry taken from the queue, not yet placed
    int waiting_rank = 0, waiting_target = 0;
    ListEntry<WEIGHTED> waiting_entry;
    auto place_waiting = [&]() {
        if (waiting)
            place(waiting_rank, waiting_target, waiting_entry);
        waiting = false;
    };
    auto place_queued = [&](int count) {
        place_waiting();
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        if (lane < count)
        {
            const int2 item = queue[(placed + lane) & (L_QUEUE - 1)];
            const int e = item.x, t = item.y - i0;
            const int left = atomicSub(&counters[t], 1); // places free before this entry took one
            waiting_entry.j = ((e / K) * 4) | (left == 1 ? L_LAST : 0);
            if constexpr (WEIGHTED)
                waiting_entry.w = weight[e];
            waiting_rank = ends[t] - left;
            waiting_target = item.y;
            waiting = true;
        }
        placed += count;
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    };
    auto enqueue = [&](int e, int v) {
        const bool mine = v >= i0 && v < i1;
        const unsigned long long mask = __ballot(mine);
        if (mask == 0) // (wave-uniform)
            return;
        if (mine)
            queue[(queued + static_cast<int>(tpk_prefix_count(mask))) & (L_QUEUE - 1)] = make_int2(e, v);
        queued += __builtin_popcountll(mask);
        if (queued - placed >= TPK_WAVE)
            place_queued(TPK_WAVE);
    };
#pragma unroll
    for (int b = 0; b < L_CACHED; b += BATCH)
        if (b * G_THREADS < total) // (wave-uniform)
        {
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
                enqueue((b + u) * G_THREADS + tid, cached[b + u]);
        }
    // (the rounds behind the cached ones; the trip count is the same for every lane of a wavefront)
    for (int e0 = L_CACHED * G_THREADS + tid; e0 - tid < total; e0 += BATCH * G_THREADS)
    {
        int iv[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
            iv[u] = index_value(e0 + u * G_THREADS);
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
            enqueue(e0 + u * G_THREADS, iv[u]);
    }
    place_queued(queued - placed);
    place_waiting();
}

// Describes the job of building the lists of `clouds` clouds of `m` targets and `cloud_total`
// index entries each, in parts of `part_total` entries (`lists` sized for clouds * parts cloud
// parts of part_total entries).  Returns TPK_ERR_UNSUPPORTED when a span of targets would not
// fit in LDS or entry positions would not fit an int.
template <int K, bool WEIGHTED, typename IdxT>
int make_list_job(int clouds, int m, int64_t cloud_total, int64_t part_total, const IdxT* idx, const float* weight,
                  const Lists<WEIGHTED>& lists, ListJob<WEIGHTED, IdxT>* job)
{
    *job = ListJob<WEIGHTED, IdxT>{};
    if (clouds <= 0 || m <= 0 || cloud_total <= 0)
        return TPK_OK; // nothing to build: no workgroups
    if (part_total <= 0 || part_total % K != 0)
        return TPK_ERR_INVALID_ARG;
    const int64_t parts = tpk_ceil_div(cloud_total, part_total);
    const int64_t span = tpk_ceil_div(m, L_SPANS);
    // (ranks inside a span must stay below 2^24 for the float division of the builder)
    if (span > L_MAX_SPAN || part_total + span >= (1 << 24) || list_capacity(m, part_total) * 8 > 0x7fffffffLL ||
        cloud_total > 0x7fffffffLL || clouds * parts * L_SPANS > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    job->m = m;
    job->cloud_total = static_cast<int>(cloud_total);
    job->parts = static_cast<int>(parts);
    job->part_total = static_cast<int>(part_total);
    job->span = static_cast<int>(span);
    job->workgroups = static_cast<int>(clouds * parts * L_SPANS);
    job->idx = idx;
    job->weight = weight;
    job->lists = lists;
    return TPK_OK;
}

template <int K, bool WEIGHTED, typename IdxT>
int launch_build_lists(int clouds, int m, int64_t cloud_total, int64_t part_total, const IdxT* idx,
                       const float* weight, const Lists<WEIGHTED>& lists, hipStream_t s)
{
    ListJob<WEIGHTED, IdxT> job;
    const int st = make_list_job<K, WEIGHTED, IdxT>(clouds, m, cloud_total, part_total, idx, weight, lists, &job);
    if (st != TPK_OK || job.workgroups == 0)
        return st;
    const size_t lds = (2 * static_cast<size_t>(job.span) + G_THREADS / TPK_WAVE + 2) * sizeof(int) +
                       static_cast<size_t>(G_THREADS / TPK_WAVE) * L_QUEUE * sizeof(int2);
    auto build = build_lists_kernel<K, WEIGHTED, IdxT>;
    const int allowed = allow_lds(build, lds);
    if (allowed != TPK_OK)
        return allowed;
    hipLaunchKernelGGL(build, dim3(static_cast<unsigned>(job.workgroups)), dim3(G_THREADS), lds, s, job);
    return tpk_launch_status();
}

} // namespace
