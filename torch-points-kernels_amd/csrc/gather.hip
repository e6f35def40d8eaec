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
// weights) using LDS *integer* atomics, which are fast, and deals the sorted entries to the
// lanes of sixteen wavefronts in equally long runs (lists.h); the main kernel then stages
// whole rows of grad_out in LDS - four, two or one at a time, whatever leaves room for the
// sums -, every lane adds up its run, one random LDS read per entry and row, and the sums
// leave as contiguous stores.  No float atomics, no zero fill, each output written once.  The
// lists cost about one entry of 8 bytes (4 unweighted) per index entry and target of
// workspace, passed in by the caller.  The order in which a target's terms are added differs
// from run to run only through the order of its list, as with the reference's global atomics
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
constexpr int G_PLAIN_BLOCKS = 1024; // workgroups the plain gather aims at (four per compute unit, two at a time)

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

    idx += static_cast<int64_t>(cloud) * n * K;
    if (WEIGHTED)
        weight += static_cast<int64_t>(cloud) * n * K;
    float* __restrict__ o = out + (static_cast<int64_t>(cloud) * c + c0) * n;
    const int64_t jbeg = static_cast<int64_t>(jpart) * jlen;
    const int64_t jend = tpk_min64(n, jbeg + jlen);
    const float* __restrict__ s = src + (static_cast<int64_t>(cloud) * c + c0) * m;

    if (WEIGHTED)
    {
        // Bound by the random LDS reads: a column's indices and weights are requested one column ahead, the
        // first before the rows are staged, so that no lane waits for them between its reads.
        int64_t j = jbeg + threadIdx.x;
        Column<K, WEIGHTED, IdxT> next;
        if (j < jend)
            next.load(idx, weight, j);
        stage_copy(rows, s, static_cast<unsigned>(nrows) * static_cast<unsigned>(m));
        __syncthreads();
        for (; j < jend; j += G_THREADS)
        {
            const Column<K, WEIGHTED, IdxT> col = next;
            next.load(idx, weight, tpk_min64(j + G_THREADS, jend - 1));
#pragma unroll
            for (int r = 0; r < G_MAX_ROWS; ++r)
                if (r < nrows)
                    o[static_cast<int64_t>(r) * n + j] = col.combine(rows + r * m);
        }
        return;
    }
    stage_copy(rows, s, static_cast<unsigned>(nrows) * static_cast<unsigned>(m));
    __syncthreads();
    for (int64_t j = jbeg + threadIdx.x; j < jend; j += G_THREADS)
    {
        Column<K, WEIGHTED, IdxT> col;
        col.load(idx, weight, j);
#pragma unroll
        for (int r = 0; r < G_MAX_ROWS; ++r)
            if (r < nrows)
                // (written once, read by nobody here: past the caches, -3 % on config 3b)
                __builtin_nontemporal_store(col.combine(rows + r * m), &o[static_cast<int64_t>(r) * n + j]);
    }
}

constexpr int GB_LDS_FLOATS = TPK_LDS_BYTES / 4; // floats of LDS a workgroup of the backward walk may use (all 160 KiB)
constexpr int GB_STAGE_FLOATS = 32768; // at most this many of them hold the staged piece of grad_out (128 KiB)
constexpr int GB_FETCH = GB_STAGE_FLOATS / 4 / G_THREADS; // 16-byte loads per lane that bring in a piece: 8
constexpr int GB_AHEAD = 8;            // rows of list entries a wavefront has requested ahead of the one it adds
constexpr int GB_HOLD = 36;            // rows of list entries a lane keeps in registers where a piece's entries are held
// The walk that holds a piece's entries in registers: one row per pass, 4-byte entries.
template <int K, bool WEIGHTED, int R>
constexpr bool GB_HOLD_FOR = K == 1 && !WEIGHTED && R == 1;

typedef int int2_vec __attribute__((ext_vector_type(2)));

// A run of device memory as a buffer resource: a load whose offset lies beyond it returns zero and
// fetches nothing, a store beyond it is dropped.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t memory_buffer(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
}

// Sum over the lanes before this one, back to and including the nearest lane whose `starts` is set
// (all lanes before it if there is none): what the lists that began in earlier lanes' runs carry into
// this lane's run.  `open` = what a lane's run adds to the list that is still open at its end;
// `starts` = the run ended at least one list, so that `open` begins a new sum.
template <int R>
__device__ __forceinline__ void carried_in(const float (&open)[R], bool starts, int lane, float (&carry)[R])
{
    float val[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
        val[r] = open[r];
    int flag = starts ? 1 : 0;
    // inside rows of 16 lanes: row_shr:1, 2, 4, 8 (a source outside the row reads as zero / no flag)
#define TPK_ROW_SHR(x, d)                                                                  \
    ((d) == 0   ? __builtin_amdgcn_update_dpp(0, (x), 0x111, 0xF, 0xF, false)              \
     : (d) == 1 ? __builtin_amdgcn_update_dpp(0, (x), 0x112, 0xF, 0xF, false)              \
     : (d) == 2 ? __builtin_amdgcn_update_dpp(0, (x), 0x114, 0xF, 0xF, false)              \
                : __builtin_amdgcn_update_dpp(0, (x), 0x118, 0xF, 0xF, false))
#pragma unroll
    for (int d = 0; d < 4; ++d)
    {
        const int pf = TPK_ROW_SHR(flag, d);
#pragma unroll
        for (int r = 0; r < R; ++r)
        {
            const int pv = TPK_ROW_SHR(__float_as_int(val[r]), d);
            val[r] += flag ? 0.f : __int_as_float(pv);
        }
        flag |= pf;
    }
#undef TPK_ROW_SHR
    // across the rows, one after the other: the sum at the end of the row before is final by then
#pragma unroll
    for (int k = 1; k < 4; ++k)
    {
        const bool take = (lane >> 4) == k && flag == 0;
#pragma unroll
        for (int r = 0; r < R; ++r)
        {
            const float before = tpk_read_lane(val[r], 16 * k - 1);
            val[r] += take ? before : 0.f;
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
    {
        const float up = __shfl_up(val[r], 1);
        carry[r] = lane == 0 ? 0.f : up;
    }
}

// grid: workgroups that each take `units_per_group` consecutive units; a unit = R feature rows
// (c0 .. c0 + R - 1) of one cloud.  A unit is processed in `parts` pieces of `part_len` columns (the
// lists are built per part, lists.h).  For a piece the workgroup holds the R x part_len values of
// grad_out in LDS; wavefront s walks the lists of span s of the targets: every lane adds up its run
// of consecutive list entries, one entry per step - the entries of a step are one contiguous row,
// requested GB_AHEAD steps ahead - and reads the staged values they refer to (an entry that refers
// to nothing carries an address beyond the LDS, which reads as zero).  Where an entry ends a list the
// lane puts its sum into the span's output row in LDS, at the target it has counted up to, and starts
// the next sum.  The first list a lane ends may have begun in the runs of the lanes before it: when
// the walk is over one scan over the lanes tells every lane what was carried into its run, and the
// lane adds that to the first sum it put.  Then the span's sums leave as contiguous stores - every
// target has at least one entry (lists.h), so the first part writes every output element; later
// parts (rows longer than the LDS holds) add to what is there, the same wavefront at the same place.
//
// grad_out streams from memory while the lists are walked: every lane requests its 16-byte loads of
// the NEXT piece into registers during the walk (a wavefront's loads complete in order, so the entry
// requests behind them wait for them: every wavefront does this at another point of its walk) and
// writes them to LDS between the two barriers that end the piece.  (Lists without weights over whole rows, one
// row per pass: the entries of a piece fit in registers and are requested a piece ahead - see GB_HOLD_FOR.)
// dynamic LDS: R * part_len floats (the piece) + R * L_SPANS * span floats (the sums).
template <int K, bool WEIGHTED, int R>
__global__ __launch_bounds__(G_THREADS, 1) void gather_bwd_lists_kernel(
    int c, int m, int64_t n, int parts, int part_len, int span, int row_groups, int units, int units_per_group,
    bool vector_loads, const float* __restrict__ grad_out, Lists<WEIGHTED> lists, float* __restrict__ grad_src)
{
    extern __shared__ float rows[];
    const unsigned tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / TPK_WAVE); // (a scalar for the compiler)
    constexpr uint32_t ENTRY_BYTES = sizeof(ListEntry<WEIGHTED>);
    // the sums of this wavefront's span: sums[(target - t0) * R + r]
    float* const sums = rows + static_cast<unsigned>(R) * static_cast<unsigned>(part_len) +
                        static_cast<unsigned>(wave) * static_cast<unsigned>(span) * R;
    const int t0 = min(wave * span, m), width = min(span, m - t0);

    // consecutive workgroups of a die work on consecutive units: one cloud's lists per L2
    const int group = static_cast<int>(xcd_local_block(blockIdx.x, gridDim.x));
    const int unit0 = group * units_per_group;
    const int unit1 = min(unit0 + units_per_group, units);
    const int pieces = (unit1 - unit0) * parts;

    // The next piece on its way into registers: 16-byte load k of a lane covers the columns
    // ((k / R) * G_THREADS + tid) * 4 .. + 3 of row k % R of the piece (part_len is a multiple of 4 here).
    float4 fetched[GB_FETCH];
    auto piece_source = [&](int piece, int& nrows, unsigned& len) __attribute__((always_inline)) {
        const int unit = unit0 + piece / parts, part = piece - (piece / parts) * parts;
        const int cloud = unit / row_groups, c0 = (unit - cloud * row_groups) * R;
        nrows = min(R, c - c0);
        const int64_t col0 = static_cast<int64_t>(part) * part_len;
        len = static_cast<unsigned>(tpk_min64(part_len, n - col0));
        return grad_out + (static_cast<int64_t>(cloud) * c + c0) * n + col0;
    };
    auto fetch = [&](int piece) __attribute__((always_inline)) {
        if (piece >= pieces)
            return;
        int nrows;
        unsigned len;
        const float* __restrict__ src = piece_source(piece, nrows, len);
#pragma unroll
        for (int k = 0; k < GB_FETCH; ++k)
        {
            const unsigned r = static_cast<unsigned>(k % R), col = (static_cast<unsigned>(k / R) * G_THREADS + tid) * 4u;
            fetched[k] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (r < static_cast<unsigned>(nrows) && col < len)
                fetched[k] = *reinterpret_cast<const float4*>(src + static_cast<int64_t>(r) * n + col);
        }
    };
    auto stage_fetched = [&]() __attribute__((always_inline)) {
        // the R rows side by side: value (row r, column col) at rows[col * R + r], so that the walk reads the
        // R values an entry refers to with one LDS instruction
        static_assert(GB_FETCH % R == 0, "a lane holds all R rows of its columns");
#pragma unroll
        for (int g = 0; g < GB_FETCH / R; ++g)
        {
            const unsigned col = (static_cast<unsigned>(g) * G_THREADS + tid) * 4u;
            if (col >= static_cast<unsigned>(part_len))
                continue;
            float* const to = rows + col * R;
            if constexpr (R == 1)
                *reinterpret_cast<float4*>(to) = fetched[g];
            else if constexpr (R == 2)
            {
                const float4 a = fetched[g * 2 + 0], b = fetched[g * 2 + 1];
                *reinterpret_cast<float4*>(to + 0) = make_float4(a.x, b.x, a.y, b.y);
                *reinterpret_cast<float4*>(to + 4) = make_float4(a.z, b.z, a.w, b.w);
            }
            else
            {
                const float4 a = fetched[g * 4 + 0], b = fetched[g * 4 + 1], cc = fetched[g * 4 + 2], d = fetched[g * 4 + 3];
                *reinterpret_cast<float4*>(to + 0) = make_float4(a.x, b.x, cc.x, d.x);
                *reinterpret_cast<float4*>(to + 4) = make_float4(a.y, b.y, cc.y, d.y);
                *reinterpret_cast<float4*>(to + 8) = make_float4(a.z, b.z, cc.z, d.z);
                *reinterpret_cast<float4*>(to + 12) = make_float4(a.w, b.w, cc.w, d.w);
            }
        }
    };
    auto stage_slowly = [&](int piece) __attribute__((always_inline)) {
        int nrows;
        unsigned len;
        const float* __restrict__ src = piece_source(piece, nrows, len);
        for (unsigned i = tid; i < R * static_cast<unsigned>(part_len); i += G_THREADS)
        {
            const unsigned r = i / static_cast<unsigned>(part_len), col = i - r * static_cast<unsigned>(part_len);
            rows[col * R + r] = (r < static_cast<unsigned>(nrows) && col < len) ? src[static_cast<int64_t>(r) * n + col] : 0.f;
        }
    };

    if constexpr (GB_HOLD_FOR<K, WEIGHTED, R>)
    {
        // Entries held in registers (this instance: 4-byte entries, whole rows as pieces).  A wavefront's loads
        // complete in order, so an entry requested behind the 16-byte loads of the next piece waits for that
        // piece - for most of the time a piece takes.  Here a piece's entries are all requested before the next
        // piece is, right after the walk of the piece before, and kept in registers: the walk itself then asks
        // memory for nothing, and the next piece is requested at its very beginning, by all wavefronts at once.
        // (Spans of more than GB_HOLD rows of entries fetch the rest one row at a time.)
        if (vector_loads)
        {
            struct Span
            {
                __amdgpu_buffer_rsrc_t ebuf;
                uint32_t first;
                int steps, first_slot;
            };
            auto describe = [&](int piece) __attribute__((always_inline)) {
                const int unit = unit0 + piece / parts, part = piece - (piece / parts) * parts;
                const int64_t cloud_part = static_cast<int64_t>(unit / row_groups) * parts + part;
                const int4 region = lists.regions[cloud_part * L_SPANS + wave];
                Span sp;
                sp.steps = __builtin_amdgcn_readfirstlane(region.z);
                sp.first_slot = (lists.first_target[(cloud_part * L_SPANS + wave) * TPK_WAVE + lane] - t0) * (R * 4);
                sp.ebuf = memory_buffer(lists.entries + cloud_part * lists.capacity, static_cast<uint32_t>(lists.capacity) * ENTRY_BYTES);
                sp.first = (static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(region.x)) + static_cast<uint32_t>(lane)) * ENTRY_BYTES;
                return sp;
            };
            auto entry = [&](const Span& sp, int i) __attribute__((always_inline)) {
                const uint32_t row = static_cast<uint32_t>(min(i, sp.steps - 1)) * (TPK_WAVE * ENTRY_BYTES); // wave-uniform
                return __builtin_amdgcn_raw_buffer_load_b32(sp.ebuf, sp.first, row, 0);
            };
            int held[GB_HOLD];
            auto request_all = [&](const Span& sp) __attribute__((always_inline)) {
                if (sp.steps > 0)
                {
#pragma unroll
                    for (int u = 0; u < GB_HOLD; ++u)
                        held[u] = entry(sp, u);
                }
            };
            fetch(0);
            Span cur = describe(0);
            request_all(cur);
            stage_fetched();
            for (int piece = 0; piece < pieces; ++piece)
            {
                const int unit = unit0 + piece / parts, part = piece - (piece / parts) * parts;
                const int cloud = unit / row_groups, c0 = (unit - cloud * row_groups) * R;
                const int nrows = min(R, c - c0);
                // (what the next piece's entries are found by, requested before the next piece itself)
                Span next = cur;
                if (piece + 1 < pieces)
                    next = describe(piece + 1);
                lds_barrier(); // the piece is in LDS
                const char* const staged = reinterpret_cast<const char*>(rows);
                char* const put_at = reinterpret_cast<char*>(sums);
                float acc = 0.f;
                int slot = cur.first_slot;
                auto take = [&](int j) __attribute__((always_inline)) {
                    acc += *reinterpret_cast<const float*>(staged + (static_cast<unsigned>(j) & 0x7fffffffu));
                    const bool ends = j < 0; // the entry ends a list
                    if (ends)
                        *reinterpret_cast<float*>(put_at + slot) = acc;
                    acc = ends ? 0.f : acc;
                    slot += ends ? 4 : 0;
                };
                // The next piece is requested while this one is walked, a load every few steps: a compute unit takes
                // requests at 64 bytes a clock, 2000 clocks for a piece, and a wavefront that issues its eight loads
                // in one go stands still that long.
                int next_source_rows;
                unsigned next_len;
                const float* __restrict__ next_source = piece + 1 < pieces ? piece_source(piece + 1, next_source_rows, next_len) : nullptr;
                constexpr int EVERY = GB_HOLD / GB_FETCH; // steps between two loads
#pragma unroll
                for (int u = 0; u < GB_HOLD; ++u)
                {
                    if (u % EVERY == 0 && u / EVERY < GB_FETCH)
                    {
                        const unsigned col = (static_cast<unsigned>(u / EVERY) * G_THREADS + tid) * 4u;
                        fetched[u / EVERY] = make_float4(0.f, 0.f, 0.f, 0.f);
                        if (next_source && col < next_len)
                            fetched[u / EVERY] = *reinterpret_cast<const float4*>(next_source + col);
                    }
                    if (u < cur.steps) // (wave-uniform)
                        take(held[u]);
                }
                for (int i = GB_HOLD; i < cur.steps; ++i)
                    take(entry(cur, i));
                // the first list every lane ended, with what the lanes before carried into it
                float open[1] = {acc}, carry[1];
                const bool ended_one = slot != cur.first_slot;
                carried_in<1>(open, ended_one, lane, carry);
                if (ended_one)
                    *reinterpret_cast<float*>(put_at + cur.first_slot) += carry[0];
                float* __restrict__ d = grad_src + (static_cast<int64_t>(cloud) * c + c0) * m + t0;
                for (int t = lane; t < width; t += TPK_WAVE)
                {
                    if (0 < nrows)
                    {
                        const float v = sums[t];
                        float* const at = d + t;
                        *at = part == 0 ? v : *at + v;
                    }
                }
                // (the next piece's entries, behind the stores: requested before them, or one by one during the walk, the
                // call was 2.5 us slower)
                if (piece + 1 < pieces)
                    request_all(next);
                cur = next;
                lds_barrier(); // everybody is done with the piece
                stage_fetched();
            }
            return;
        }
    }
    if (vector_loads)
    {
        fetch(0);
        stage_fetched();
    }
    for (int piece = 0; piece < pieces; ++piece)
    {
        const int unit = unit0 + piece / parts, part = piece - (piece / parts) * parts;
        const int cloud = unit / row_groups, c0 = (unit - cloud * row_groups) * R;
        const int nrows = min(R, c - c0);
        const int64_t cloud_part = static_cast<int64_t>(cloud) * parts + part;

        // this wavefront's span of the lists of (cloud, part)
        const int4 region = lists.regions[cloud_part * L_SPANS + wave];
        const int base = __builtin_amdgcn_readfirstlane(region.x);
        const int steps = __builtin_amdgcn_readfirstlane(region.z);
        // where this lane puts its next sum: the target of its first entry, as a byte offset into `sums`
        const int first_slot = (lists.first_target[(cloud_part * L_SPANS + wave) * TPK_WAVE + lane] - t0) * (R * 4);
        const __amdgpu_buffer_rsrc_t ebuf =
            memory_buffer(lists.entries + cloud_part * lists.capacity, static_cast<uint32_t>(lists.capacity) * ENTRY_BYTES);
        const uint32_t first = (static_cast<uint32_t>(base) + static_cast<uint32_t>(lane)) * ENTRY_BYTES;
        auto request = [&](int i) __attribute__((always_inline)) {
            // (rows behind the last are never used: the last row again)
            const uint32_t row = static_cast<uint32_t>(min(i, steps - 1)) * (TPK_WAVE * ENTRY_BYTES); // wave-uniform
            ListEntry<WEIGHTED> e;
            if constexpr (WEIGHTED)
            {
                const int2_vec v = __builtin_amdgcn_raw_buffer_load_b64(ebuf, first, row, 0);
                e.j = v.x;
                e.w = __int_as_float(v.y);
            }
            else
                e.j = __builtin_amdgcn_raw_buffer_load_b32(ebuf, first, row, 0);
            return e;
        };
        // (list entries do not depend on the staged values: the first rows are requested before the barrier)
        ListEntry<WEIGHTED> ahead[GB_AHEAD];
        if (steps > 0)
        {
#pragma unroll
            for (int u = 0; u < GB_AHEAD; ++u)
                ahead[u] = request(u);
        }

        if (!vector_loads)
        {
            // rows that do not start on 16-byte boundaries: the piece is staged before its walk, nothing overlaps
            __syncthreads();
            stage_slowly(piece);
        }
        lds_barrier(); // the piece is in LDS
        const int fetch_at = vector_loads ? ((wave * steps / L_SPANS) / GB_AHEAD) * GB_AHEAD : -1;
        if (vector_loads && steps == 0)
            fetch(piece + 1);

        const char* const staged = reinterpret_cast<const char*>(rows);
        char* const put_at = reinterpret_cast<char*>(sums);
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; ++r)
            acc[r] = 0.f;
        int slot = first_slot;
        for (int i0 = 0; i0 < steps; i0 += GB_AHEAD)
        {
            if (i0 == fetch_at) // (wave-uniform)
                fetch(piece + 1);
#pragma unroll
            for (int u = 0; u < GB_AHEAD; ++u)
            {
                if (i0 + u >= steps) // (wave-uniform)
                    break;
                const ListEntry<WEIGHTED> e = ahead[u];
                ahead[u] = request(i0 + u + GB_AHEAD);
                const unsigned at = (static_cast<unsigned>(e.j) & 0x7fffffffu) * R; // (column * 4 bytes in the entry)
                float v[R];
                if constexpr (R == 1)
                    v[0] = *reinterpret_cast<const float*>(staged + at);
                else if constexpr (R == 2)
                {
                    const float2 both = *reinterpret_cast<const float2*>(staged + at);
                    v[0] = both.x;
                    v[1] = both.y;
                }
                else
                {
                    const float4 all = *reinterpret_cast<const float4*>(staged + at);
                    v[0] = all.x;
                    v[1] = all.y;
                    v[2] = all.z;
                    v[3] = all.w;
                }
#pragma unroll
                for (int r = 0; r < R; ++r)
                {
                    if constexpr (WEIGHTED)
                        acc[r] = __builtin_fmaf(v[r], e.w, acc[r]); // (one rounding instead of the reference's two: within its tolerance)
                    else
                        acc[r] += v[r];
                }
                const bool ends = e.j < 0; // the entry ends a list
                if (ends)
                {
#pragma unroll
                    for (int r = 0; r < R; ++r)
                        *reinterpret_cast<float*>(put_at + slot + r * 4) = acc[r];
                }
#pragma unroll
                for (int r = 0; r < R; ++r)
                    acc[r] = ends ? 0.f : acc[r];
                slot += ends ? R * 4 : 0;
            }
        }
        // the first list every lane ended, with what the lanes before carried into it
        float carry[R];
        const bool ended_one = slot != first_slot;
        carried_in<R>(acc, ended_one, lane, carry);
        if (ended_one)
        {
#pragma unroll
            for (int r = 0; r < R; ++r)
                *reinterpret_cast<float*>(put_at + first_slot + r * 4) += carry[r];
        }
        // the span's sums leave in order (a wavefront's LDS accesses are executed in order: no barrier needed)
        float* __restrict__ d = grad_src + (static_cast<int64_t>(cloud) * c + c0) * m + t0;
        for (int t = lane; t < width; t += TPK_WAVE)
        {
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (r < nrows)
                {
                    const float v = sums[t * R + r];
                    float* const at = d + static_cast<int64_t>(r) * m + t;
                    *at = part == 0 ? v : *at + v;
                }
        }
        lds_barrier(); // everybody is done with the piece
        if (vector_loads)
            stage_fetched();
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
    int r = rows_for(m, c);
    // The plain gather is bound by its stores and gains from two workgroups per compute unit that stage and store
    // at different times, and from row blocks that are not split by columns (every split stages the rows again):
    // fewer rows per workgroup while that gives more workgroups, down to two rows (with one row the indices, read
    // once per row block, become the larger stream).  Config 3b: 8 rows x 2 column parts 62 us, 4 rows 59, 2 rows 55,
    // 1 row 78.
    if (!WEIGHTED)
        while (r > 2 && static_cast<int64_t>(b) * tpk_ceil_div(c, r) < G_PLAIN_BLOCKS)
            r = (r + 1) / 2;
    if (r > 0)
    {
        const int row_blocks = static_cast<int>(tpk_ceil_div(c, r));
        // Split the columns so that a few hundred workgroups exist, but keep each part at
        // least as long as a row (so staging a row block stays the smaller share of traffic).
        int64_t jsplit = tpk_ceil_div(WEIGHTED ? 256 : G_PLAIN_BLOCKS, static_cast<int64_t>(row_blocks) * b);
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
        // bound) with two workgroups per compute unit at a time and the default placement.
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

// Rows of grad_out staged together and columns per part, for rows of n floats and m targets.
struct BwdShape
{
    int rows;     // 0: the shape does not fit (too many targets)
    int part_len;
    int parts;
    int span;     // targets per wavefront
};
BwdShape bwd_shape(int64_t n, int m)
{
    BwdShape sh;
    // The LDS holds rows x part_len staged values and rows x (16 spans) sums.  As many rows at a time as
    // leave room for whole rows of grad_out (the lists are read once per row group): four, two or one; rows
    // longer than that go one at a time in parts.
    sh.span = static_cast<int>(tpk_ceil_div(m, L_SPANS));
    const int64_t sums = static_cast<int64_t>(sh.span) * L_SPANS;
    const int64_t n4 = (n + 3) & ~static_cast<int64_t>(3);
    sh.rows = 0;
    sh.part_len = 0;
    sh.parts = 0;
    for (int r = 4; r >= 1; r /= 2)
    {
        const int64_t room = tpk_min64(GB_LDS_FLOATS / r - sums, GB_STAGE_FLOATS / r) & ~static_cast<int64_t>(3);
        if (room >= n4 || (r == 1 && room >= 4096))
        {
            sh.rows = r;
            sh.part_len = static_cast<int>(tpk_min64(n4, room));
            sh.parts = static_cast<int>(tpk_min64(tpk_ceil_div(n, sh.part_len), 0x7fffffff));
            break;
        }
    }
    return sh;
}

// Workspace of the list-based backward: the lists of every (cloud, part) (lists.h).
template <int K, bool WEIGHTED>
size_t lists_workspace_bytes(int b, int m, int64_t n)
{
    if (b <= 0 || m <= 0 || n <= 0)
        return 0;
    const BwdShape sh = bwd_shape(n, m);
    if (sh.rows == 0 || static_cast<int64_t>(b) * sh.parts > 0x7fffffffLL)
        return 0;
    return lists_bytes<WEIGHTED>(static_cast<int64_t>(b) * sh.parts, m, static_cast<int64_t>(sh.part_len) * K);
}

template <int K, bool WEIGHTED, int R>
int launch_bwd_lists(int b, int c, int m, int64_t n, const BwdShape& sh, const float* grad_out,
                     const Lists<WEIGHTED>& lists, float* grad_src, hipStream_t s)
{
    const int row_groups = static_cast<int>(tpk_ceil_div(c, R));
    const int64_t units = static_cast<int64_t>(b) * row_groups;
    if (units > 0x7fffffffLL)
        return TPK_ERR_UNSUPPORTED;
    // One workgroup per compute unit (its LDS holds one piece): every workgroup takes the same
    // number of consecutive units, so that it can request its next piece while it works.
    const int per_group = static_cast<int>(tpk_ceil_div(units, 256));
    const int groups = static_cast<int>(tpk_ceil_div(units, per_group));
    const size_t lds = static_cast<size_t>(R) * (static_cast<size_t>(sh.part_len) + static_cast<size_t>(sh.span) * L_SPANS) * sizeof(float);
    // 16-byte loads need rows that start on 16-byte boundaries
    const bool vector_loads = (n & 3) == 0 && (reinterpret_cast<uintptr_t>(grad_out) & 15u) == 0;
    auto kernel = gather_bwd_lists_kernel<K, WEIGHTED, R>;
    int st = allow_lds(kernel, lds);
    if (st != TPK_OK)
        return st;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(groups)), dim3(G_THREADS), lds, s, c, m, n, sh.parts,
                       sh.part_len, sh.span, row_groups, static_cast<int>(units), per_group, vector_loads, grad_out, lists,
                       grad_src);
    return tpk_launch_status();
}

// The shape of the list path for (b, n, m), or rows == 0 where the lists do not serve it.
template <int K>
BwdShape list_shape(int b, int m, int64_t n)
{
    BwdShape sh = bwd_shape(n > 0 ? n : 1, m);
    if (n <= 0 || m <= 0 || n * K > 0x7fffffffLL || static_cast<int64_t>(b) * sh.parts > 0x7fffffffLL)
        sh.rows = 0;
    return sh;
}

// Inverts the index of every cloud into `lists` (lists_workspace_bytes() bytes).  TPK_ERR_UNSUPPORTED: the
// list path does not serve this shape.
template <int K, bool WEIGHTED, typename IdxT>
int gather_lists(int b, int m, int64_t n, const IdxT* idx, const float* weight, void* lists_memory, size_t lists_bytes,
                 hipStream_t s)
{
    const BwdShape sh = list_shape<K>(b, m, n);
    const size_t need = lists_workspace_bytes<K, WEIGHTED>(b, m, n);
    if (sh.rows == 0 || need == 0)
        return TPK_ERR_UNSUPPORTED;
    if (!lists_memory || lists_bytes < need || (reinterpret_cast<uintptr_t>(lists_memory) & 15u))
        return TPK_ERR_WORKSPACE;
    const int64_t part_total = static_cast<int64_t>(sh.part_len) * K;
    const Lists<WEIGHTED> lists = lists_at<WEIGHTED>(lists_memory, static_cast<int64_t>(b) * sh.parts, m, part_total);
    return launch_build_lists<K, WEIGHTED, IdxT>(b, m, n * K, part_total, idx, weight, lists, s);
}

// The backward pass over lists that gather_lists() built for the same (b, n, m).
template <int K, bool WEIGHTED>
int gather_bwd_from_lists(int b, int c, int m, int64_t n, const float* grad_out, void* lists_memory, size_t lists_bytes,
                          float* grad_src, hipStream_t s)
{
    const BwdShape sh = list_shape<K>(b, m, n);
    const size_t need = lists_workspace_bytes<K, WEIGHTED>(b, m, n);
    if (sh.rows == 0 || need == 0)
        return TPK_ERR_UNSUPPORTED;
    if (!lists_memory || lists_bytes < need || (reinterpret_cast<uintptr_t>(lists_memory) & 15u))
        return TPK_ERR_WORKSPACE;
    const Lists<WEIGHTED> lists =
        lists_at<WEIGHTED>(lists_memory, static_cast<int64_t>(b) * sh.parts, m, static_cast<int64_t>(sh.part_len) * K);
    if (sh.rows == 4)
        return launch_bwd_lists<K, WEIGHTED, 4>(b, c, m, n, sh, grad_out, lists, grad_src, s);
    if (sh.rows == 2)
        return launch_bwd_lists<K, WEIGHTED, 2>(b, c, m, n, sh, grad_out, lists, grad_src, s);
    return launch_bwd_lists<K, WEIGHTED, 1>(b, c, m, n, sh, grad_out, lists, grad_src, s);
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
    const size_t need = lists_workspace_bytes<K, WEIGHTED>(b, m, n);
    if (n > 0 && workspace && need > 0 && workspace_bytes >= need && list_shape<K>(b, m, n).rows > 0)
    {
        int st = gather_lists<K, WEIGHTED, IdxT>(b, m, n, idx, weight, workspace, workspace_bytes, s);
        if (st == TPK_OK)
            return gather_bwd_from_lists<K, WEIGHTED>(b, c, m, n, grad_out, workspace, workspace_bytes, grad_src, s);
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

extern "C" int tpk_three_interpolate_lists_f32(int b, int n, int m, const int32_t* idx, const float* weight, void* lists,
                                               size_t lists_bytes, void* stream)
{
    if (b < 0 || n < 0 || m < 0)
        return TPK_ERR_INVALID_ARG;
    if (b > 0 && n > 0 && m > 0 && (!idx || !weight))
        return TPK_ERR_INVALID_ARG;
    return gather_lists<3, true, int32_t>(b, m, n, idx, weight, lists, lists_bytes, tpk_stream(stream));
}

extern "C" int tpk_three_interpolate_grad_lists_f32(int b, int c, int n, int m, const float* grad_out, void* lists,
                                                    size_t lists_bytes, float* grad_points, void* stream)
{
    if (b < 0 || c < 0 || n < 0 || m < 0)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || c == 0 || m == 0)
        return TPK_OK;
    if (!grad_out || !grad_points)
        return TPK_ERR_INVALID_ARG;
    return gather_bwd_from_lists<3, true>(b, c, m, n, grad_out, lists, lists_bytes, grad_points, tpk_stream(stream));
}

extern "C" int tpk_group_lists(int b, int n, int npoint, int nsample, const int64_t* idx, void* lists, size_t lists_bytes,
                               void* stream)
{
    if (b < 0 || n < 0 || npoint < 0 || nsample < 0)
        return TPK_ERR_INVALID_ARG;
    const int64_t columns = static_cast<int64_t>(npoint) * nsample;
    if (b > 0 && n > 0 && columns > 0 && !idx)
        return TPK_ERR_INVALID_ARG;
    return gather_lists<1, false, int64_t>(b, n, columns, idx, nullptr, lists, lists_bytes, tpk_stream(stream));
}

extern "C" int tpk_group_grad_lists_f32(int b, int c, int n, int npoint, int nsample, const float* grad_out, void* lists,
                                        size_t lists_bytes, float* grad_features, void* stream)
{
    if (b < 0 || c < 0 || n < 0 || npoint < 0 || nsample < 0)
        return TPK_ERR_INVALID_ARG;
    if (b == 0 || c == 0 || n == 0)
        return TPK_OK;
    if (!grad_out || !grad_features)
        return TPK_ERR_INVALID_ARG;
    return gather_bwd_from_lists<1, false>(b, c, n, static_cast<int64_t>(npoint) * nsample, grad_out, lists, lists_bytes,
                                           grad_features, tpk_stream(stream));
}
