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
// weights) using LDS *integer* atomics, which are fast, and an LDS prefix sum, laid out so that
// one lane per target can walk them with coalesced reads (lists.h); the main kernel then
// stages rows of grad_out in LDS - four rows in pieces of 8192 columns, or one longer row in
// pieces of 16384 columns, with lists per piece - and every lane sums the listed columns of
// its target.  No float atomics, no zero fill, each output written by one lane.  The lists cost
// about 3 entries of 8 bytes (4 unweighted) per index entry of workspace, passed in by the
// caller.  The order in which a target's terms are added differs from run to run only through
// the order of its list, as with the reference's global atomics
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

    const float* __restrict__ s = src + (static_cast<int64_t>(cloud) * c + c0) * m;
    stage_copy(rows, s, static_cast<unsigned>(nrows) * static_cast<unsigned>(m));
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

constexpr int GB_STAGE_FLOATS = 32768; // floats of grad_out a workgroup keeps in LDS (128 KiB)
constexpr int GB_WAVES = G_THREADS / TPK_WAVE;
constexpr int GB_WALK_WAVES = GB_WAVES;
constexpr int GB_FETCH = GB_STAGE_FLOATS / 4 / G_THREADS; // 16-byte loads per lane that bring in a piece: 8
constexpr int GB_KEPT_BLOCKS = 4;      // blocks of 64 targets per wavefront whose sums stay in registers
constexpr int GB_STEPS = L_WIDTH_STEP / 2; // list slots requested together (widths are multiples of twice that)

typedef int int2_vec __attribute__((ext_vector_type(2)));

// The entries of a cloud's lists as a buffer resource: a load whose offset lies beyond the buffer
// returns zero and fetches nothing, so a lane without an entry in some step is given such an
// offset instead of a branch around the load.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t entry_buffer(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
}
constexpr uint32_t GB_NO_ENTRY = 0x80000000u; // a byte offset beyond every entry buffer (and below 2^32 with a round's offsets added)

// What a walking wavefront does for one piece (see gather_bwd_lists_kernel): the sums of the lists of
// its blocks (block walker + 16 b) over the columns of the piece.  KEEP: added to `kept` (lane = target)
// and stored after the unit's last part; otherwise added to what the parts before stored.
// STRIDE: floats from one staged row to the next when known at compile time, else 0 (`stride`).
// `between(b)` is called once per block position b = 0 .. GB_KEPT_BLOCKS - 1 (KEEP) after that block's first
// entries have been requested: the place for other memory requests that should not hold the walk up.
template <int K, bool WEIGHTED, int R, bool KEEP, unsigned STRIDE, typename Between>
__device__ __forceinline__ void walk_piece(const float* rows, unsigned stride, int piece, int unit0, int parts,
                                           int row_groups, int c, int m, int nblocks, int walker, int lane,
                                           const Lists<WEIGHTED>& lists, float* __restrict__ grad_src,
                                           float (*kept)[R], Between&& between)
{
    const unsigned row_bytes = (STRIDE ? STRIDE : stride) * 4u;
    const char* const staged = reinterpret_cast<const char*>(rows);
    constexpr int STEPS = GB_STEPS; // list slots requested per round
    constexpr uint32_t ENTRY_BYTES = sizeof(ListEntry<WEIGHTED>);
    const int unit = unit0 + piece / parts, part = piece - (piece / parts) * parts;
    const int cloud = unit / row_groups, c0 = (unit - cloud * row_groups) * R;
    const int nrows = min(R, c - c0);
    float* __restrict__ d = grad_src + (static_cast<int64_t>(cloud) * c + c0) * m;
    const int64_t cloud_part = static_cast<int64_t>(cloud) * parts + part;
    const int* __restrict__ meta = lists.meta + cloud_part * nblocks * L_BLOCK;
    const int2* __restrict__ blocks = lists.blocks + cloud_part * nblocks;
    const ListEntry<WEIGHTED>* __restrict__ entries = lists.entries + cloud_part * lists.capacity;
    const __amdgpu_buffer_rsrc_t ebuf = entry_buffer(entries, static_cast<uint32_t>(lists.capacity) * ENTRY_BYTES);

    // (the lane's offset decides whether the load is inside the buffer; `uniform` is added to the address)
    auto load_entry = [&](uint32_t offset, uint32_t uniform) __attribute__((always_inline)) {
        ListEntry<WEIGHTED> e;
        if constexpr (WEIGHTED)
        {
            const int2_vec v = __builtin_amdgcn_raw_buffer_load_b64(ebuf, offset, uniform, 0);
            e.j = v.x;
            e.w = __int_as_float(v.y);
        }
        else
            e.j = __builtin_amdgcn_raw_buffer_load_b32(ebuf, offset, uniform, 0);
        return e;
    };
    // The staged value an entry refers to, in row r (a lane without entry was given the entry (0, 0): it
    // reads the zero in front of the row).  Rows in pairs: an LDS instruction's own offset reaches the
    // next row, not the one after.
    auto staged_value = [&](const ListEntry<WEIGHTED>& e, int r) __attribute__((always_inline)) {
        const char* const pair = staged + static_cast<unsigned>(e.j) + static_cast<unsigned>(r / 2) * (2u * row_bytes);
        return *reinterpret_cast<const float*>(pair + static_cast<unsigned>(r % 2) * row_bytes);
    };
    auto add_value = [&](const ListEntry<WEIGHTED>& e, float v, float& sum) __attribute__((always_inline)) {
        if constexpr (WEIGHTED)
            sum = __builtin_fmaf(v, e.w, sum); // (one rounding instead of the reference's two: within its tolerance)
        else
            sum += v;
    };
    auto add_entry = [&](const ListEntry<WEIGHTED>& e, float (&sum)[R]) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < R; ++r)
            add_value(e, staged_value(e, r), sum[r]);
    };
    // Sums of the lists of a block over this piece, lane = position in the block's lane order.
    auto walk_block = [&](int word, const ListBlock& lb, float (&sum)[R], auto&& after_first_request) __attribute__((always_inline)) {
        const int count = word & L_COUNT_MASK;
        const int slots = min(count, lb.width); // entries of this lane in the slot-major part
        const uint32_t first = (static_cast<uint32_t>(lb.start) + static_cast<uint32_t>(lane)) * ENTRY_BYTES;
        auto request = [&](int i, ListEntry<WEIGHTED> (&ent)[STEPS]) __attribute__((always_inline)) {
            const uint32_t round = first + static_cast<uint32_t>(i) * (L_BLOCK * ENTRY_BYTES);
#pragma unroll
            for (int u = 0; u < STEPS; ++u)
                ent[u] = load_entry(i + u < slots ? round : GB_NO_ENTRY, static_cast<uint32_t>(u) * (L_BLOCK * ENTRY_BYTES));
        };
        // (all reads of a round are issued before the first sum; the compiler is kept from mixing the
        // phases of a round, which would make every read wait for the one before)
        auto add_round = [&](const ListEntry<WEIGHTED> (&ent)[STEPS]) __attribute__((always_inline)) {
            float v[STEPS][R];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < STEPS; ++u)
#pragma unroll
                for (int r = 0; r < R; ++r)
                    v[u][r] = staged_value(ent[u], r);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < STEPS; ++u)
#pragma unroll
                for (int r = 0; r < R; ++r)
                    add_value(ent[u], v[u][r], sum[r]);
            __builtin_amdgcn_sched_barrier(0);
        };
#pragma unroll
        for (int r = 0; r < R; ++r)
            sum[r] = 0.f;
        // Two sets of registers take turns: while one round's entries are used, the next round's are
        // on their way (beyond the width every lane asks for nothing and is given zeros).
        ListEntry<WEIGHTED> even[STEPS], odd[STEPS];
        request(0, even);
        after_first_request();
        for (int i = 0; i < lb.width; i += 2 * STEPS) // (widths are multiples of 2 * STEPS)
        {
            request(i + STEPS, odd);
            add_round(even);
            request(i + 2 * STEPS, even);
            add_round(odd);
        }
        if (lb.longer)
        {
            int extra, extra_at;
            list_extra(count, lb.width, extra, extra_at);
            const uint32_t rest = (static_cast<uint32_t>(lb.start) + static_cast<uint32_t>(lb.width) * L_BLOCK) * ENTRY_BYTES;
            for (unsigned long long todo = __ballot(extra > 0); todo; todo &= todo - 1)
            {
                const int owner = __builtin_ctzll(todo);
                const int number = __builtin_amdgcn_readlane(extra, owner);
                const int at = __builtin_amdgcn_readlane(extra_at, owner);
                float rest_sum[R];
#pragma unroll
                for (int r = 0; r < R; ++r)
                    rest_sum[r] = 0.f;
                for (int p = lane; p < number; p += TPK_WAVE)
                    add_entry(load_entry(rest + static_cast<uint32_t>(at + p) * ENTRY_BYTES, 0u), rest_sum);
#pragma unroll
                for (int r = 0; r < R; ++r)
                {
                    const float total = wave_sum_f32(rest_sum[r]);
                    if (lane == owner)
                        sum[r] += total;
                }
            }
        }
    };

    if constexpr (KEEP)
    {
        const bool last_part = part == parts - 1;
        // (the descriptions of all blocks are requested together)
        int words[GB_KEPT_BLOCKS];
        ListBlock lbs[GB_KEPT_BLOCKS];
#pragma unroll
        for (int b = 0; b < GB_KEPT_BLOCKS; ++b)
        {
            const int blk = min(walker + b * GB_WALK_WAVES, nblocks - 1);
            words[b] = meta[blk * L_BLOCK + lane];
            lbs[b] = list_block(blocks, blk);
        }
#pragma unroll
        for (int b = 0; b < GB_KEPT_BLOCKS; ++b)
        {
            const int blk = walker + b * GB_WALK_WAVES;
            if (blk >= nblocks)
                between(b);
            if (blk < nblocks)
            {
                float sum[R];
                walk_block(words[b], lbs[b], sum, [&]() __attribute__((always_inline)) { between(b); });
                // from the block's lane order to target order: lane T takes the sums of the lane that served target T
                const int serving = static_cast<int>(static_cast<unsigned>(words[b]) >> 26);
#pragma unroll
                for (int r = 0; r < R; ++r)
                    kept[b][r] += __int_as_float(__builtin_amdgcn_ds_bpermute(serving * 4, __float_as_int(sum[r])));
                if (last_part)
                {
                    const int tgt = blk * L_BLOCK + lane;
#pragma unroll
                    for (int r = 0; r < R; ++r)
                    {
                        if (tgt < m && r < nrows)
                            d[static_cast<int64_t>(r) * m + tgt] = kept[b][r];
                        kept[b][r] = 0.f;
                    }
                }
            }
        }
    }
    else
    {
        between(0);
        for (int blk = walker; blk < nblocks; blk += GB_WALK_WAVES)
        {
            const int word = meta[blk * L_BLOCK + lane];
            const ListBlock lb = list_block(blocks, blk);
            const int tgt = blk * L_BLOCK + lane;
            // (what the parts before stored for these targets is requested now, needed at the end)
            float old[R];
#pragma unroll
            for (int r = 0; r < R; ++r)
                old[r] = part > 0 && tgt < m && r < nrows ? d[static_cast<int64_t>(r) * m + tgt] : 0.f;
            float sum[R];
            walk_block(word, lb, sum, [] {});
            const int serving = static_cast<int>(static_cast<unsigned>(word) >> 26);
#pragma unroll
            for (int r = 0; r < R; ++r)
            {
                const float mine = __int_as_float(__builtin_amdgcn_ds_bpermute(serving * 4, __float_as_int(sum[r])));
                if (tgt < m && r < nrows)
                    d[static_cast<int64_t>(r) * m + tgt] = old[r] + mine;
            }
        }
    }
}

// grid: workgroups that each take `units_per_group` consecutive units; a unit = R feature rows
// (c0 .. c0 + R - 1) of one cloud.  A unit is processed in `parts` pieces of `part_len` columns
// (the lists are built per part, lists.h).  For a piece the workgroup holds the R x part_len
// values of grad_out in LDS, and every wavefront takes blocks of 64 targets, one target per lane
// (in the block's order of descending list length): in step i the lanes that still have an entry
// read slot i of their lists - one contiguous run - and the staged values these refer to.  Two
// sets of registers take turns, so the entries of a round are requested a round ahead.  The few
// lists longer than the block's slot-major part are then summed by the whole wavefront.
//
// grad_out streams from memory while the lists are walked: every lane requests its eight 16-byte
// loads of the NEXT piece (1024 lanes x 8 = the 128 KiB of a piece) into registers during the walk
// and writes them to LDS between the two barriers that end a piece.  A wavefront's loads complete in
// order, so the entry requests that follow those loads wait for them: each wavefront issues them
// during one of its blocks only, a different one from wavefront to wavefront, and at any time
// most wavefronts walk while some wait for memory.
//
// KEEP: the sums of every block stay in registers across the parts of a unit and are stored
// once (m <= 64 * 16 * GB_KEPT_BLOCKS targets); otherwise a block's sums of one part are added
// to what the parts before stored.
// dynamic LDS: R * (part_len + 4) floats.
template <int K, bool WEIGHTED, int R, bool KEEP>
__global__ __launch_bounds__(G_THREADS, 1) void gather_bwd_lists_kernel(
    int c, int m, int64_t n, int parts, int part_len, int row_groups, int units, int units_per_group, bool vector_loads,
    const float* __restrict__ grad_out, Lists<WEIGHTED> lists, float* __restrict__ grad_src)
{
    extern __shared__ float rows[];
    const unsigned stride = static_cast<unsigned>(part_len) + 4u;
    const unsigned tid = threadIdx.x;
    const int lane = tid & (TPK_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / TPK_WAVE); // (a scalar for the compiler)
    const int nblocks = (m + L_BLOCK - 1) / L_BLOCK;

    // consecutive workgroups of a die work on consecutive units: one cloud's lists per L2
    const int group = static_cast<int>(xcd_local_block(blockIdx.x, gridDim.x));
    const int unit0 = group * units_per_group;
    const int unit1 = min(unit0 + units_per_group, units);
    const int pieces = (unit1 - unit0) * parts;

    // what a lane without entry reads: four zeros in front of every staged row
    for (unsigned t = tid; t < R * 4u; t += G_THREADS)
        rows[(t >> 2) * stride + (t & 3u)] = 0.f;

    float kept[KEEP ? GB_KEPT_BLOCKS : 1][R]; // sums of this wavefront's blocks over the parts so far, lane = target
#pragma unroll
    for (int b = 0; b < (KEEP ? GB_KEPT_BLOCKS : 1); ++b)
#pragma unroll
        for (int r = 0; r < R; ++r)
            kept[b][r] = 0.f;

    if (!vector_loads)
    {
        // Rows that do not start on 16-byte boundaries, or pieces shorter than the LDS holds: the
        // piece is staged before its walk, nothing overlaps.
        for (int piece = 0; piece < pieces; ++piece)
        {
            const int unit = unit0 + piece / parts, part = piece - (piece / parts) * parts;
            const int cloud = unit / row_groups, c0 = (unit - cloud * row_groups) * R;
            const int64_t col0 = static_cast<int64_t>(part) * part_len;
            __syncthreads();
            stage_rows_by<G_THREADS, 4>(rows + 4, stride, grad_out + (static_cast<int64_t>(cloud) * c + c0) * n + col0, n,
                                        static_cast<unsigned>(min(R, c - c0)),
                                        static_cast<unsigned>(tpk_min64(part_len, n - col0)), tid);
            __syncthreads();
            walk_piece<K, WEIGHTED, R, KEEP, 0>(rows, stride, piece, unit0, parts, row_groups, c, m, nblocks, wave, lane, lists,
                                                grad_src, kept, [](int) {});
        }
        return;
    }

    // (on this path part_len = GB_STAGE_FLOATS / R: load k of a lane lies in row k / CHUNKS of the
    // piece, at a column that is the same for the whole workgroup plus four times the lane's number)
    constexpr unsigned PART = GB_STAGE_FLOATS / R;
    constexpr unsigned CHUNK = G_THREADS * 4; // columns covered by one load of all lanes
    constexpr unsigned CHUNKS = PART / CHUNK;
    float4 fetched[GB_FETCH];
    auto fetch = [&](int piece) __attribute__((always_inline)) {
        if (piece >= pieces)
            return;
        const int unit = unit0 + piece / parts, part = piece - (piece / parts) * parts;
        const int cloud = unit / row_groups, c0 = (unit - cloud * row_groups) * R;
        const int nrows = min(R, c - c0);
        const int64_t col0 = static_cast<int64_t>(part) * PART;
        const unsigned len = static_cast<unsigned>(tpk_min64(PART, n - col0));
        const float* __restrict__ src = grad_out + (static_cast<int64_t>(cloud) * c + c0) * n + col0;
#pragma unroll
        for (int k = 0; k < GB_FETCH; ++k)
        {
            const unsigned r = static_cast<unsigned>(k) / CHUNKS, col = (static_cast<unsigned>(k) % CHUNKS) * CHUNK + tid * 4u;
            fetched[k] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (r < static_cast<unsigned>(nrows) && col < len)
                fetched[k] = *reinterpret_cast<const float4*>(src + static_cast<int64_t>(r) * n + col);
        }
    };
    auto stage_fetched = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int k = 0; k < GB_FETCH; ++k)
        {
            const unsigned r = static_cast<unsigned>(k) / CHUNKS, col = (static_cast<unsigned>(k) % CHUNKS) * CHUNK + tid * 4u;
            *reinterpret_cast<float4*>(rows + r * (PART + 4u) + 4u + col) = fetched[k];
        }
    };
    fetch(0);
    stage_fetched();
    const int my_turn = KEEP ? (wave & (GB_KEPT_BLOCKS - 1)) : 0; // the block position during which this wavefront fetches
    for (int piece = 0; piece < pieces; ++piece)
    {
        lds_barrier(); // the piece is in LDS
        walk_piece<K, WEIGHTED, R, KEEP, PART + 4>(rows, stride, piece, unit0, parts, row_groups, c, m, nblocks, wave, lane, lists,
                                                   grad_src, kept, [&](int b) __attribute__((always_inline)) {
                                                       if (b == my_turn)
                                                           fetch(piece + 1);
                                                   });
        lds_barrier(); // everybody is done with the piece
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
    const int r = rows_for(m, c);
    if (r > 0)
    {
        const int row_blocks = static_cast<int>(tpk_ceil_div(c, r));
        // Split the columns so that a few hundred workgroups exist, but keep each part at
        // least as long as a row (so staging a row block stays the smaller share of traffic).
        int64_t jsplit = tpk_ceil_div(WEIGHTED ? 256 : 512, static_cast<int64_t>(row_blocks) * b);
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
        // bound) with two rounds of workgroups and the default placement.
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

// Rows of grad_out staged together and columns per part, for rows of n floats.
struct BwdShape
{
    int rows;
    int part_len;
    int parts;
};
BwdShape bwd_shape(int64_t n)
{
    BwdShape sh;
    // 128 KiB of LDS hold rows x part_len values.  Rows of up to 16384 floats go four at a time in
    // pieces of 8192 columns (the lists of a piece are read once per four rows), rows of up to
    // 32768 floats two at a time in pieces of 16384 columns, longer rows one at a time.
    sh.rows = n <= GB_STAGE_FLOATS ? 4 : 1;
    const int64_t n4 = (n + 3) & ~static_cast<int64_t>(3);
    sh.part_len = static_cast<int>(tpk_min64(n4, GB_STAGE_FLOATS / sh.rows));
    sh.parts = static_cast<int>(tpk_min64(tpk_ceil_div(n, sh.part_len), 0x7fffffff));
    return sh;
}

// Workspace of the list-based backward: the lists of every (cloud, part) (lists.h).
template <int K, bool WEIGHTED>
size_t lists_workspace_bytes(int b, int m, int64_t n)
{
    if (b <= 0 || m <= 0 || n <= 0)
        return 0;
    const BwdShape sh = bwd_shape(n);
    if (static_cast<int64_t>(b) * sh.parts > 0x7fffffffLL)
        return 0;
    return lists_bytes<WEIGHTED>(b * sh.parts, m, static_cast<int64_t>(sh.part_len) * K);
}

template <int K, bool WEIGHTED, int R, bool KEEP>
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
    const size_t lds = static_cast<size_t>(R) * (sh.part_len + 4) * sizeof(float);
    // 16-byte loads need rows that start on 16-byte boundaries
    // the fetching wavefronts need rows that start on 16-byte boundaries and full-size pieces
    const bool vector_loads = (n & 3) == 0 && (reinterpret_cast<uintptr_t>(grad_out) & 15u) == 0 &&
                              static_cast<int64_t>(sh.part_len) * R == GB_STAGE_FLOATS;
    auto kernel = gather_bwd_lists_kernel<K, WEIGHTED, R, KEEP>;
    int st = allow_lds(kernel, lds);
    if (st != TPK_OK)
        return st;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(groups)), dim3(G_THREADS), lds, s, c, m, n, sh.parts,
                       sh.part_len, row_groups, static_cast<int>(units), per_group, vector_loads, grad_out, lists,
                       grad_src);
    return tpk_launch_status();
}

template <int K, bool WEIGHTED, int R>
int launch_bwd_lists_rows(int b, int c, int m, int64_t n, const BwdShape& sh, const float* grad_out,
                          const Lists<WEIGHTED>& lists, float* grad_src, hipStream_t s)
{
    if (list_blocks(m) <= GB_KEPT_BLOCKS * GB_WALK_WAVES)
        return launch_bwd_lists<K, WEIGHTED, R, true>(b, c, m, n, sh, grad_out, lists, grad_src, s);
    return launch_bwd_lists<K, WEIGHTED, R, false>(b, c, m, n, sh, grad_out, lists, grad_src, s);
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
    const BwdShape sh = bwd_shape(n > 0 ? n : 1);
    const bool fits = n > 0 && n * K <= 0x7fffffffLL &&
                      static_cast<int64_t>(b) * sh.parts <= 0x7fffffffLL;
    const size_t need = lists_workspace_bytes<K, WEIGHTED>(b, m, n);
    if (fits && workspace && need > 0 && workspace_bytes >= need)
    {
        const int64_t part_total = static_cast<int64_t>(sh.part_len) * K;
        const Lists<WEIGHTED> lists = lists_at<WEIGHTED>(workspace, b * sh.parts, m, part_total);
        int st = launch_build_lists<K, WEIGHTED, IdxT>(b, m, n * K, part_total, idx, weight, lists, s);
        if (st == TPK_OK)
        {
            if (sh.rows == 4)
                return launch_bwd_lists_rows<K, WEIGHTED, 4>(b, c, m, n, sh, grad_out, lists, grad_src, s);
            if (sh.rows == 2)
                return launch_bwd_lists_rows<K, WEIGHTED, 2>(b, c, m, n, sh, grad_out, lists, grad_src, s);
            return launch_bwd_lists_rows<K, WEIGHTED, 1>(b, c, m, n, sh, grad_out, lists, grad_src, s);
        }
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
