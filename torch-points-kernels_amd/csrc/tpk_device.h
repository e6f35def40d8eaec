// Shared pieces of the gfx950 kernels: launch bookkeeping and wavefront helpers.
//
// Arithmetic rule for every distance in this library: fp32 (or fp64), each product and
// each sum rounded on its own, evaluated left to right.  The translation units are
// compiled with -ffp-contract=off and additionally carry the pragma below, so no
// multiply-add is ever fused; integer outputs (neighbour indices, sample indices) depend
// on it.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstring>
#include <map>
#include <mutex>
#include <utility>

#include "../../include/tpk.h"

#pragma clang fp contract(off)

#define TPK_WAVE 64

// LDS a workgroup may use on gfx950 (160 KiB); the kernels stay below it.
#define TPK_LDS_BYTES 163840

// Compute units of an MI355X (8 dies of 32).
#define TPK_COMPUTE_UNITS 256

static inline hipStream_t tpk_stream(void* s)
{
    return reinterpret_cast<hipStream_t>(s);
}

// Status of the launch just made: 0, or the hipError_t it raised.
static inline int tpk_launch_status()
{
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? TPK_OK : static_cast<int>(e);
}

// Lets `kernel` use up to `bytes` of dynamic LDS on the current device.  The runtime call behind it
// is made once per kernel and device (again only when a larger size is asked for): a launch on
// the hot path does a table look-up instead of a driver call.
static inline int tpk_allow_lds(const void* kernel, size_t bytes)
{
    static std::mutex lock;
    static std::map<std::pair<const void*, int>, size_t> allowed;
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess)
        return static_cast<int>(e);
    std::lock_guard<std::mutex> guard(lock);
    size_t& have = allowed[std::make_pair(kernel, device)];
    if (bytes <= have)
        return TPK_OK;
    // (sizes are rounded up so that slightly larger requests later seldom come back here)
    size_t ask = (bytes + 16383) & ~static_cast<size_t>(16383);
    if (ask > TPK_LDS_BYTES)
        ask = bytes > TPK_LDS_BYTES ? bytes : TPK_LDS_BYTES;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(ask));
    if (e != hipSuccess && ask != bytes)
    {
        // (the rounded size did not fit next to the kernel's static LDS: the exact one)
        (void)hipGetLastError();
        ask = bytes;
        e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(ask));
    }
    if (e != hipSuccess)
        return static_cast<int>(e);
    have = ask;
    return TPK_OK;
}

// Copies `bytes` (at most TPK_READ_BACK_BYTES) from device memory at `src` to `dst` behind the work on `stream` and
// waits for them: for the entry points whose next step depends on what the device computed.  The copy lands in a
// small pinned buffer that every host thread allocates once and keeps (a copy into pageable memory is staged by the
// runtime, which blocks the host for longer than the data takes).
constexpr size_t TPK_READ_BACK_BYTES = 32768;
static inline int tpk_read_back(void* dst, const void* src, size_t bytes, hipStream_t stream)
{
    static thread_local void* pinned = nullptr;
    if (bytes > TPK_READ_BACK_BYTES)
        return TPK_ERR_INVALID_ARG;
    if (!pinned)
    {
        const hipError_t made = hipHostMalloc(&pinned, TPK_READ_BACK_BYTES, hipHostMallocDefault);
        if (made != hipSuccess)
        {
            pinned = nullptr;
            return static_cast<int>(made);
        }
    }
    hipError_t e = hipMemcpyAsync(pinned, src, bytes, hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess)
        e = hipStreamSynchronize(stream);
    if (e != hipSuccess)
        return static_cast<int>(e);
    memcpy(dst, pinned, bytes);
    return TPK_OK;
}

static inline int64_t tpk_ceil_div(int64_t a, int64_t b)
{
    return (a + b - 1) / b;
}

__host__ __device__ __forceinline__ int64_t tpk_min64(int64_t a, int64_t b)
{
    return a < b ? a : b;
}

// Number of lanes below this one whose bit is set in `mask` (a wave64 ballot).
__device__ __forceinline__ unsigned tpk_prefix_count(unsigned long long mask)
{
    return __builtin_amdgcn_mbcnt_hi(static_cast<unsigned>(mask >> 32),
                                     __builtin_amdgcn_mbcnt_lo(static_cast<unsigned>(mask), 0u));
}

__device__ __forceinline__ unsigned tpk_lane_id()
{
    return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// Value of `v` in lane `lane` (wave-uniform lane number), as a wave-uniform scalar.
__device__ __forceinline__ float tpk_read_lane(float v, int lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

__device__ __forceinline__ int tpk_read_lane(int v, int lane)
{
    return __builtin_amdgcn_readlane(v, lane);
}

// Squared distance, unfused, in the order ((dx*dx + dy*dy) + dz*dz).
template <typename T>
__device__ __forceinline__ T tpk_dist2(T ax, T ay, T az, T bx, T by, T bz)
{
    const T dx = ax - bx;
    const T dy = ay - by;
    const T dz = az - bz;
    return dx * dx + dy * dy + dz * dz;
}

// A wave-uniform value copied into a vector register.  On gfx950 fp32 add / sub / mul issue
// at twice the rate of other VALU instructions, but only when no operand is a scalar
// register; wave-uniform coordinates that enter a distance loop are therefore copied into
// vector registers first.
__device__ __forceinline__ float to_vector_register(float uniform_value)
{
    float v;
    asm volatile("v_mov_b32 %0, %1" : "=v"(v) : "s"(uniform_value));
    return v;
}

// Workgroups are handed to the 8 accelerator dies (XCDs) round-robin, and each die has its own
// L2.  This turns the hardware block number into a logical one such that consecutive logical
// blocks - which work on the same cloud and re-read the same index / list data - run on the
// same die, so that data is served by one L2 instead of being fetched into all eight.
__device__ __forceinline__ unsigned xcd_local_block(unsigned bid, unsigned blocks)
{
    constexpr unsigned XCDS = 8;
    const unsigned even = blocks - blocks % XCDS;
    return bid < even ? (bid % XCDS) * (even / XCDS) + bid / XCDS : bid;
}

// DPP controls: quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_ror:4, row_ror:8.  After the
// four steps every lane of a 16-lane row holds the row's result.
__device__ __forceinline__ int row_all_max_i32(int v)
{
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x124, 0xF, 0xF, true));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x128, 0xF, 0xF, true));
    return v;
}

__device__ __forceinline__ int wave_max_i32(int v)
{
    v = row_all_max_i32(v);
    const int a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
    const int c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
    return max(max(a, b), max(c, d));
}

// Sum of v over the lanes below this one (DPP prefix sum inside every row of 16 lanes, then
// the totals of the rows before).
__device__ __forceinline__ int wave_exclusive_sum(int v)
{
    int s = v;
    s += __builtin_amdgcn_update_dpp(0, s, 0x111, 0xF, 0xF, false); // row_shr:1
    s += __builtin_amdgcn_update_dpp(0, s, 0x112, 0xF, 0xF, false); // row_shr:2
    s += __builtin_amdgcn_update_dpp(0, s, 0x114, 0xF, 0xF, false); // row_shr:4
    s += __builtin_amdgcn_update_dpp(0, s, 0x118, 0xF, 0xF, false); // row_shr:8
    const int r0 = __builtin_amdgcn_readlane(s, 15), r1 = __builtin_amdgcn_readlane(s, 31);
    const int r2 = __builtin_amdgcn_readlane(s, 47);
    const int row = (threadIdx.x & (TPK_WAVE - 1)) >> 4;
    s += (row > 0 ? r0 : 0) + (row > 1 ? r1 : 0) + (row > 2 ? r2 : 0);
    return s - v;
}

// Largest of the values v >= 0 of this lane and the lanes below it (the same steps with a maximum).
__device__ __forceinline__ int wave_inclusive_max_i32(int v)
{
    int s = v;
    s = max(s, __builtin_amdgcn_update_dpp(0, s, 0x111, 0xF, 0xF, false)); // row_shr:1
    s = max(s, __builtin_amdgcn_update_dpp(0, s, 0x112, 0xF, 0xF, false)); // row_shr:2
    s = max(s, __builtin_amdgcn_update_dpp(0, s, 0x114, 0xF, 0xF, false)); // row_shr:4
    s = max(s, __builtin_amdgcn_update_dpp(0, s, 0x118, 0xF, 0xF, false)); // row_shr:8
    const int r0 = __builtin_amdgcn_readlane(s, 15);
    const int r1 = max(r0, __builtin_amdgcn_readlane(s, 31));
    const int r2 = max(r1, __builtin_amdgcn_readlane(s, 47));
    const int row = (threadIdx.x & (TPK_WAVE - 1)) >> 4;
    return max(s, row == 0 ? 0 : row == 1 ? r0 : row == 2 ? r1 : r2);
}

// Sum of v over the wavefront, the same value in every lane (row rotations, then the four row
// totals added in lane order: the result does not depend on which lanes call it).
__device__ __forceinline__ float wave_sum_f32(float v)
{
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xF, 0xF, true));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, true));
    return ((tpk_read_lane(v, 0) + tpk_read_lane(v, 16)) + tpk_read_lane(v, 32)) + tpk_read_lane(v, 48);
}

// Workgroup barrier that orders LDS traffic only: global loads and stores a wavefront has in
// flight stay in flight across it.
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): also covers LDS atomics without return value
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}


// ---------------------------------------------------------------------------------------------
// Work counters.  The library is also built a second time with -DTPK_COUNT_WORK
// (libtpk_hip_counting.so): there the distance scans add up the pair evaluations their lanes
// execute (one count = one lane forming one squared distance, or one running minimum updated by
// furthest point sampling), so that a benchmark can divide EXECUTED work by time.  Every
// translation unit has its own device counter, registered with the reader in status.hip.  In the
// shipping build all of this expands to nothing.
// ---------------------------------------------------------------------------------------------
#ifdef TPK_COUNT_WORK
namespace {
__device__ unsigned long long tpk_work_cell;
int tpk_work_cell_read_reset(unsigned long long* out)
{
    const unsigned long long zero = 0;
    hipError_t e = hipMemcpyFromSymbol(out, HIP_SYMBOL(tpk_work_cell), sizeof(*out));
    if (e == hipSuccess)
        e = hipMemcpyToSymbol(HIP_SYMBOL(tpk_work_cell), &zero, sizeof(zero));
    return static_cast<int>(e);
}
} // namespace
extern "C" void tpk_work_register(int (*read_reset)(unsigned long long*));
namespace {
struct TpkWorkRegistration
{
    TpkWorkRegistration() { tpk_work_register(&tpk_work_cell_read_reset); }
} tpk_work_registration;
} // namespace
#define TPK_WORK_DECL unsigned long long tpk_work = 0;
#define TPK_WORK_ADD(n) (tpk_work += static_cast<unsigned long long>(n))
#define TPK_WORK_FLUSH atomicAdd(&tpk_work_cell, tpk_work);
#define TPK_WORK_PARAM , unsigned long long& tpk_work
#define TPK_WORK_ARG , tpk_work
#else
#define TPK_WORK_DECL
#define TPK_WORK_ADD(n) ((void)0)
#define TPK_WORK_FLUSH
#define TPK_WORK_PARAM
#define TPK_WORK_ARG
#endif
