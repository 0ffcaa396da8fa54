// Device-side building blocks shared by the kernels: wave64 scans, the decoupled look-back
// protocol, and the K-gram key load. gfx950 only (wavefront = 64 lanes).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint64_t u64;
typedef uint32_t u32;
typedef uint16_t u16;
typedef uint8_t u8;

namespace csa {

constexpr int WAVE = 64;

// Values of the device error word (0 = no error). Kernels report a broken invariant there instead of
// reading or writing out of bounds; the host turns it into CSA_ERR_INTERNAL.
constexpr unsigned DEV_ERR_LOOKBACK_TIMEOUT = 1;
constexpr unsigned DEV_ERR_SMALLSORT_TABLES = 2;
constexpr unsigned DEV_ERR_PLACE_RANGE = 3;
constexpr unsigned DEV_ERR_RERANK_RANGE = 4;

__device__ __forceinline__ u32 lane_id() { return __lane_id(); }

// ---- wave64 inclusive scans by shuffles ----

__device__ __forceinline__ u32 wave_incl_sum(u32 v)
{
    const u32 lane = lane_id();
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {
        const u32 t = __shfl_up(v, o);
        if (lane >= (u32)o)
            v += t;
    }
    return v;
}

__device__ __forceinline__ u32 wave_incl_max(u32 v)
{
    const u32 lane = lane_id();
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {
        const u32 t = __shfl_up(v, o);
        if (lane >= (u32)o)
            v = v > t ? v : t;
    }
    return v;
}

// ---- decoupled look-back ----
//
// One 64-bit word per (tile, chain): [63:34] epoch of the launch, [33:32] status, [31:0] value.
// A word whose epoch is not the launch's own is "not written yet", so the array is never cleared
// between launches. Words are read and written with relaxed agent-scope atomics only: status and
// value travel in the same word, so no fence is needed and the accesses are coherent across XCDs.
// Tiles are numbered by an atomic ticket taken when a workgroup starts, hence every predecessor
// of a waiting tile is already resident or finished.

constexpr u32 LB_AGG = 1;  // value = this tile's aggregate
constexpr u32 LB_INCL = 2; // value = aggregate of tiles [0, tile]
constexpr u32 LB_SPIN_LIMIT = 1u << 24;

__device__ __forceinline__ u64 lb_pack(u32 epoch, u32 status, u32 value)
{
    return ((u64)epoch << 34) | ((u64)status << 32) | (u64)value;
}

__device__ __forceinline__ void lb_store(u64* p, u64 v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ u64 lb_load(const u64* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The protocol in two steps, so that a kernel can publish its aggregate as soon as it is known and wait
// for its predecessors as late as possible.
// Step 1: publish `aggregate` of `tile` on the chain whose word for tile t lives at chain[t * stride].
__device__ __forceinline__ void lb_publish(u64* chain, u32 stride, u32 tile, u32 epoch, u32 aggregate)
{
    lb_store(chain + (u64)tile * stride, lb_pack(epoch, tile == 0 ? LB_INCL : LB_AGG, aggregate));
}

// Step 2: returns the combination of the aggregates of tiles [0, tile) and upgrades the tile's own word
// to "inclusive". Combination is max if IS_MAX, else a 32-bit sum. On a spin timeout (a predecessor never
// published) sets *err and returns what it has, so that every wave still leaves the kernel.
template <bool IS_MAX>
__device__ __forceinline__ u32 lb_wait_exclusive(u64* chain, u32 stride, u32 tile, u32 epoch, u32 aggregate, u32* err)
{
    if (tile == 0)
        return 0;
    u32 excl = 0;
    u32 t = tile;
    while (t > 0) {
        --t;
        u64 w = 0;
        u32 spins = 0;
        for (;;) {
            w = lb_load(chain + (u64)t * stride);
            if ((u32)(w >> 34) == epoch && ((w >> 32) & 3u) != 0)
                break;
            if (++spins >= LB_SPIN_LIMIT) {
                atomicExch(err, 1u);
                return excl;
            }
            __builtin_amdgcn_s_sleep(1);
        }
        const u32 v = (u32)w;
        excl = IS_MAX ? (excl > v ? excl : v) : excl + v;
        if (((w >> 32) & 3u) == LB_INCL)
            break;
    }
    const u32 incl = IS_MAX ? (excl > aggregate ? excl : aggregate) : excl + aggregate;
    lb_store(chain + (u64)tile * stride, lb_pack(epoch, LB_INCL, incl));
    return excl;
}

template <bool IS_MAX>
__device__ __forceinline__ u32 lb_exclusive_prefix(u64* chain, u32 stride, u32 tile, u32 epoch, u32 aggregate, u32* err)
{
    lb_publish(chain, stride, tile, epoch, aggregate);
    return lb_wait_exclusive<IS_MAX>(chain, stride, tile, epoch, aggregate, err);
}

// ---- K-gram key: four uint16 symbols of the zero-padded text, the first one most significant ----

__device__ __forceinline__ u64 load_kgram(const u16* __restrict__ T, u32 n, u32 j, u32 word)
{
    const u64 p = (u64)j + 4ull * word;
    if (p + 4 <= (u64)n) {
        u64 raw; // little-endian: s0 | s1 << 16 | s2 << 32 | s3 << 48
        __builtin_memcpy(&raw, T + p, 8);
        return (raw << 48) | ((raw & 0xFFFF0000ull) << 16) | ((raw >> 16) & 0xFFFF0000ull) | (raw >> 48);
    }
    u64 k = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const u64 s = (p + q < (u64)n) ? (u64)T[p + q] : 0ull;
        k = (k << 16) | s;
    }
    return k;
}

} // namespace csa
