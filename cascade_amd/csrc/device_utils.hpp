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
constexpr unsigned DEV_ERR_UNEXPECTED_LARGE_GROUP = 5;
constexpr unsigned DEV_ERR_JOIN_TABLE_FULL = 6;

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
// of a waiting tile is already resident or finished and the waits end whatever else shares the device.
// (The radix pass may instead derive the tile from the workgroup index, for callers that have the device to
// themselves: a predecessor may then belong to a workgroup that is dispatched later, which only ends if enough
// workgroups of the launch are resident together.)
// Every wait has a spin limit that turns a predecessor that never shows up into an error word, and gives up
// early once another wait has failed; the kernels that wait leave at once when the word is set.

constexpr u32 LB_AGG = 1;  // value = this tile's aggregate
constexpr u32 LB_INCL = 2; // value = aggregate of tiles [0, tile]
#ifndef CSA_LB_SPIN_LIMIT
#define CSA_LB_SPIN_LIMIT (1u << 21) // polls of one word; a poll takes a microsecond or more
#endif
constexpr u32 LB_SPIN_LIMIT = CSA_LB_SPIN_LIMIT;

// After a device invariant has failed, the arrays downstream of the failure hold neither a valid order nor valid
// indices: the kernels that wait for other workgroups leave at once, and the host reports the code when it reads the
// word back at the end of the step. (Kernels without a wait check the indices they are given instead, and raise the
// word themselves: reading it first would put a memory round trip in front of every workgroup.)
__device__ __forceinline__ bool dev_failed(const u32* err)
{
    return err != nullptr && __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
}

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

// Publishes `aggregate` of `tile` on the chain whose word for tile t lives at chain[t * stride] (tile 0's aggregate is
// its inclusive prefix). A kernel publishes as soon as the aggregate is known and waits for its predecessors as late
// as possible; the walk below does the waiting.
__device__ __forceinline__ void lb_publish(u64* chain, u32 stride, u32 tile, u32 epoch, u32 aggregate)
{
    lb_store(chain + (u64)tile * stride, lb_pack(epoch, tile == 0 ? LB_INCL : LB_AGG, aggregate));
}

// ---- two-level look-back (one chain per thread, many chains per tile: the radix pass) ----
//
// With one level, every waiting tile walks back over all the unresolved tiles in flight, re-reading their words
// over the fabric; the walks grow with the number of resident tiles and end up costing more traffic and time
// than the data. Here tiles form groups of LB_GROUP consecutive tiles. A tile sums the aggregates of the
// (at most LB_GROUP - 1) earlier tiles of its own group: those are published early by tiles that started
// together with it, so nothing there waits for a resolution. The last tile of a group publishes the group's
// total and chains the groups with the ordinary protocol; every tile adds the inclusive prefix of the group
// before its own. Group words arrive LB_GROUP times more slowly than tile words, so that chain stays short.

constexpr u32 LB_GROUP = 16;

// spins until the word is published for this launch; returns it (0 after a timeout, with *err set)
__device__ __forceinline__ u64 lb_wait_word(const u64* p, u32 epoch, u32* err)
{
    u32 idle = 0;
    for (;;) {
        const u64 w = lb_load(p);
        if ((u32)(w >> 34) == epoch && ((w >> 32) & 3u) != 0)
            return w;
        if (++idle >= LB_SPIN_LIMIT) {
            atomicExch(err, DEV_ERR_LOOKBACK_TIMEOUT);
            return 0;
        }
        if ((idle & 1023u) == 0u && dev_failed(err))
            return 0; // another wait has failed: the launch is lost, leave without waiting out the limit
        __builtin_amdgcn_s_sleep(2);
    }
}

// tile_chain: word of tile t at tile_chain[t * stride]; it only ever holds the tile's own aggregate (lb2_publish).
// group_chain: word of group g at group_chain[g * stride]. lb2_wait_exclusive returns the sum of the aggregates of
// tiles [0, tile).
__device__ __forceinline__ void lb2_publish(u64* tile_chain, u32 stride, u32 tile, u32 epoch, u32 aggregate)
{
    lb_store(tile_chain + (u64)tile * stride, lb_pack(epoch, LB_AGG, aggregate));
}

__device__ __forceinline__ u32 lb2_wait_exclusive(u64* tile_chain, u64* group_chain, u32 stride, u32 tile, u32 epoch,
                                                  u32 aggregate, u32* err)
{
    const u32 j = tile % LB_GROUP, g = tile / LB_GROUP;
    // aggregates of the earlier tiles of this group: all loads in flight together, stragglers polled one by one
    u64 word[LB_GROUP - 1];
#pragma unroll
    for (u32 k = 1; k < LB_GROUP; ++k)
        word[k - 1] = k <= j ? lb_load(tile_chain + (u64)(tile - k) * stride) : 0ull;
    // the words of the two groups before this one travel together with the tile words: the walk over the groups below
    // then starts from words that are already here, instead of paying a round trip of its own for each
    constexpr u32 PROBES = 2;
    u64 probe[PROBES];
#pragma unroll
    for (u32 k = 0; k < PROBES; ++k)
        probe[k] = g > k ? lb_load(group_chain + (u64)(g - 1 - k) * stride) : 0ull;
    u32 within = 0;
#pragma unroll
    for (u32 k = 1; k < LB_GROUP; ++k) {
        if (k <= j) {
            u64 w = word[k - 1];
            if ((u32)(w >> 34) != epoch || ((w >> 32) & 3u) == 0)
                w = lb_wait_word(tile_chain + (u64)(tile - k) * stride, epoch, err);
            within += (u32)w;
        }
    }
    const bool closes_group = j == LB_GROUP - 1;
    const u32 total = within + aggregate;
    if (closes_group)
        lb_store(group_chain + (u64)g * stride, lb_pack(epoch, g == 0 ? LB_INCL : LB_AGG, total));
    // inclusive prefix of the groups before this one
    u32 gexcl = 0;
    for (u32 gi = g; gi > 0;) {
        --gi;
        u64 w = g - 1 - gi < PROBES ? probe[g - 1 - gi] : 0ull;
        if ((u32)(w >> 34) != epoch || ((w >> 32) & 3u) == 0)
            w = lb_wait_word(group_chain + (u64)gi * stride, epoch, err);
        gexcl += (u32)w;
        if (((w >> 32) & 3u) == LB_INCL || w == 0)
            break;
    }
    if (closes_group && g > 0)
        lb_store(group_chain + (u64)g * stride, lb_pack(epoch, LB_INCL, gexcl + total));
    return gexcl + within;
}

// ---- wave-wide reduction ----

__device__ __forceinline__ u32 wave_reduce_sum(u32 v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o);
    return v;
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

// LDS whose size is given at launch: `extern __shared__` on the device; the CPU emulation of the kernels hands out
// one buffer per launch instead.
#ifdef HIPEMU
#define CSA_DYNAMIC_LDS(T, name) T* name = reinterpret_cast<T*>(hipemu::dynamic_lds())
#else
#define CSA_DYNAMIC_LDS(T, name) extern __shared__ T name[]
#endif

// ---- a stretch of the text in LDS ----
//
// Consecutive suffixes share all but one symbol of their K-grams, and the text is only 2-byte aligned, so kernels
// that build the keys of a run of consecutive positions stage the stretch once: symbols [p0, p0 + count) of the text
// (zero past its end, the key padding) are copied into s_words with aligned 8-byte loads by the `block` threads of the
// workgroup. Returns sym_off: after a __syncthreads(), symbol p0 + i is 16-bit element sym_off + i of s_words.
// s_words needs room for (count + 6) / 4 + 1 words.
__device__ __forceinline__ u32 stage_text(const u16* __restrict__ text, u64 text_len, u64 p0, u32 count, u64* s_words, u32 t,
                                          u32 block)
{
    const u32 sym_off = (u32)(((uintptr_t)(text + p0) & 7u) >> 1); // symbols between the aligned word boundary and p0
    const long long first_pos = (long long)p0 - (long long)sym_off;
    const u32 nw = (sym_off + count + 3u) / 4u;
    for (u32 i = t; i < nw; i += block) {
        const long long q0 = first_pos + 4ll * i;
        u64 wv = 0;
        if (q0 >= 0 && q0 + 4 <= (long long)text_len) {
            wv = *reinterpret_cast<const u64*>(text + q0); // 8-byte aligned by construction, wholly inside the text
        } else {
#pragma unroll
            for (int sy = 0; sy < 4; ++sy) {
                const long long q = q0 + sy;
                if (q >= 0 && q < (long long)text_len)
                    wv |= (u64)text[q] << (16 * sy);
            }
        }
        s_words[i] = wv;
    }
    return sym_off;
}

// K-gram word (four symbols, the first most significant) that starts at 16-bit element sidx of a staged stretch.
// Reads three 32-bit LDS words; the stretch must extend one word past the last symbol used.
__device__ __forceinline__ u64 staged_kgram(const u32* s_dw, u32 sidx)
{
    const u32 dw = sidx >> 1;
    const u64 lo = (u64)s_dw[dw] | ((u64)s_dw[dw + 1] << 32);
    const u64 raw = (sidx & 1u) ? (lo >> 16) | ((u64)s_dw[dw + 2] << 48) : lo; // s0 | s1 << 16 | s2 << 32 | s3 << 48
    return (raw << 48) | ((raw & 0xFFFF0000ull) << 16) | ((raw >> 16) & 0xFFFF0000ull) | (raw >> 48);
}

} // namespace csa
