// Rank-propagation messages between partitions, for partitions that are sorted one at a time and exchange ranks
// through the host (the reference's scheme, README.md:26; kernels include/GPU_SACA.cuh:283-389). A partition whose
// text and ranks are resident in HBM does not need them (it gathers rank[x + h] by text position); these kernels
// serve the per-generation entry points that keep the reference's slab interface.
//
// At the end of a generation that resolved `ctx` symbols, every cohort member j (sorted list SA, keys K, routing
// tags beta) sends
//   its rank to j - ctx, via the partition in the low half of beta, unless j < ctx or the recipient has retired;
//     the rank carries the poison-pill bit if j itself retired in this generation (list index >= *active_sz);
//   and, if its own key had received a pill, the secondary of that key as a pill to j - ctx / 2, via the high half.
// Messages are collated by destination: msg_off[q] must hold, before the emission, the exclusive prefix sum of the
// per-destination counts, and holds the exclusive END of q's group afterwards. The order inside a group is arbitrary.
#pragma once

#include "device_utils.hpp"

namespace csa {

constexpr u64 MSG_VAL_MASK = (1ull << 48) - 1ull;    // suffix in a word (include/bit-layout.hpp:44,109)
constexpr u64 MSG_PILL_RECEIPT = 1ull << 62;         // a key that received a pill (include/bit-layout.hpp:57)
constexpr u32 MSG_PILL_BIT = 1u << 31;               // finality of a message's rank (include/message.hpp:22)
constexpr u32 MSG_RETIRED = 0x8000u;                 // recipient retired, in a half of beta (include/bit-layout.hpp:135)
constexpr int MSG_BLOCK = 256;
constexpr int MSG_ITEMS = 4;
constexpr int MSG_TILE = MSG_BLOCK * MSG_ITEMS;
constexpr u32 MSG_LDS_PARTS = 2048; // destinations counted in LDS (more: one global atomic per message, as the reference)

struct MessageArgs {
    const u64* sa;
    const u64* keys;
    const u32* beta;
    u64 n;
    u64 ctx;
    int packed; // keys are composite (primary << 31 | secondary, pill receipt in bit 62), not plain ranks
    const unsigned long long* active_sz;
    u32 p;
    u8* msg_target;
    u32* msg_rank;
    u32* msg_off; // count kernel: per-destination counters to add to
    u32 tiles;
};

struct Message {
    u32 dest;   // 0xFFFFFFFF: none
    u64 target;
    u32 rank;
};

// the (at most) two messages of list element i (include/GPU_SACA.cuh:300-307, 334-352)
__device__ __forceinline__ void messages_of(const MessageArgs& a, u64 i, u64 active_sz, Message& pay, Message& fwd)
{
    pay.dest = fwd.dest = 0xFFFFFFFFu;
    const u64 j = a.sa[i] & MSG_VAL_MASK;
    const u64 k = a.keys[i];
    const u32 beta = a.beta[i];
    if (j >= a.ctx && !(beta & MSG_RETIRED)) {
        const u32 primary = a.packed ? (u32)((k >> 31) & 0x7FFFFFFFull) : (u32)k;
        pay.dest = beta & 0xFFFFu;
        pay.target = j - a.ctx;
        pay.rank = i < active_sz ? primary : (primary | MSG_PILL_BIT);
    }
    if (a.packed && (k & MSG_PILL_RECEIPT) && j >= (a.ctx >> 1) && !((beta >> 16) & MSG_RETIRED)) {
        fwd.dest = beta >> 16;
        fwd.target = j - (a.ctx >> 1);
        fwd.rank = (u32)(k & 0x7FFFFFFFull) | MSG_PILL_BIT;
    }
}

// msg_off[q] += messages bound for partition q. Workgroups stride over the tiles and flush their LDS counters once.
__global__ __launch_bounds__(MSG_BLOCK) void count_messages_kernel(MessageArgs a)
{
    __shared__ u32 s_cnt[MSG_LDS_PARTS];
    const u32 t = threadIdx.x;
    const bool lds = a.p <= MSG_LDS_PARTS;
    if (lds)
        for (u32 q = t; q < a.p; q += MSG_BLOCK)
            s_cnt[q] = 0;
    __syncthreads();
    for (u32 tile = blockIdx.x; tile < a.tiles; tile += gridDim.x) {
#pragma unroll
        for (int k = 0; k < MSG_ITEMS; ++k) {
            const u64 i = (u64)tile * MSG_TILE + (u64)k * MSG_BLOCK + t;
            if (i >= a.n)
                continue;
            Message pay, fwd;
            messages_of(a, i, ~0ull, pay, fwd); // the destinations do not depend on the active size
            // a destination outside [0, p) would be a corrupt routing tag: not counted (and not emitted either)
            if (pay.dest < a.p)
                atomicAdd(lds ? &s_cnt[pay.dest] : &a.msg_off[pay.dest], 1u);
            if (fwd.dest < a.p)
                atomicAdd(lds ? &s_cnt[fwd.dest] : &a.msg_off[fwd.dest], 1u);
        }
    }
    if (lds) {
        __syncthreads();
        for (u32 q = t; q < a.p; q += MSG_BLOCK)
            if (s_cnt[q])
                atomicAdd(&a.msg_off[q], s_cnt[q]);
    }
}

// Writes the messages: a tile of EMIT_TILE list elements counts its messages per destination in LDS, reserves one range
// per destination with a single global atomic, orders its messages by destination in LDS and stores them as runs: the
// messages of one destination leave together, lane after lane, instead of as single 5-byte and 4-byte stores all over
// the outbox. With more than MSG_LDS_PARTS destinations every message takes its slot with a global atomic and is
// stored where it falls, as the reference does.
constexpr u32 EMIT_FEW_PARTS = 256;
constexpr int EMIT_BLOCK = 512;
constexpr int EMIT_ITEMS = 4;
constexpr int EMIT_TILE = EMIT_BLOCK * EMIT_ITEMS;
constexpr int EMIT_CAP = 2 * EMIT_TILE; // a payload and a forwarded pill per element

// PARTS: the destinations the LDS tables hold (fewer: more workgroups per CU).
template <u32 PARTS>
__global__ __launch_bounds__(EMIT_BLOCK) void emit_messages_kernel(MessageArgs a)
{
    __shared__ u32 s_cnt[PARTS];  // the tile's messages per destination
    __shared__ u32 s_excl[PARTS]; // where they start in the ordered tile
    __shared__ u32 s_base[PARTS]; // where they go in the outbox
    __shared__ u32 s_low[EMIT_CAP];
    __shared__ u32 s_rank[EMIT_CAP];
    __shared__ u16 s_dest[EMIT_CAP];
    __shared__ u8 s_high[EMIT_CAP];
    __shared__ u32 s_wave[EMIT_BLOCK / 64 + 1];
    const u32 t = threadIdx.x, lane = t & 63u, w = t >> 6;
    const bool lds = a.p <= PARTS;
    const u64 active_sz = *a.active_sz;
    const u64 tiles = (a.n + EMIT_TILE - 1) / EMIT_TILE;
    const u32 per = (a.p + EMIT_BLOCK - 1) / EMIT_BLOCK; // destinations per thread in the scan
    for (u64 tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        if (lds)
            for (u32 q = t; q < a.p; q += EMIT_BLOCK)
                s_cnt[q] = 0;
        __syncthreads(); // also: the ordered tile of the round before has been stored
        Message m[2 * EMIT_ITEMS];
        u32 slot[2 * EMIT_ITEMS];
#pragma unroll
        for (int k = 0; k < EMIT_ITEMS; ++k) {
            const u64 i = tile * EMIT_TILE + (u64)k * EMIT_BLOCK + t;
            m[2 * k].dest = m[2 * k + 1].dest = 0xFFFFFFFFu;
            if (i < a.n)
                messages_of(a, i, active_sz, m[2 * k], m[2 * k + 1]);
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                Message& mm = m[2 * k + e];
                if (mm.dest >= a.p)
                    mm.dest = 0xFFFFFFFFu;
                else
                    slot[2 * k + e] = atomicAdd(lds ? &s_cnt[mm.dest] : &a.msg_off[mm.dest], 1u);
            }
        }
        if (!lds) {
#pragma unroll
            for (int e = 0; e < 2 * EMIT_ITEMS; ++e) {
                if (m[e].dest == 0xFFFFFFFFu)
                    continue;
                const u64 s = slot[e];
#pragma unroll
                for (int b = 0; b < 5; ++b)
                    a.msg_target[5 * s + b] = (u8)(m[e].target >> (8 * b));
                a.msg_rank[s] = m[e].rank;
            }
            continue;
        }
        __syncthreads();
        // exclusive prefix sums of the counts over the destinations; one range of the outbox per destination
        const u32 first = t * per < a.p ? t * per : a.p;
        const u32 last = first + per < a.p ? first + per : a.p;
        u32 sum = 0;
        for (u32 q = first; q < last; ++q)
            sum += s_cnt[q];
        const u32 incl = wave_incl_sum(sum);
        if (lane == 63u)
            s_wave[w] = incl;
        __syncthreads();
        u32 run = incl - sum;
        for (u32 ww = 0; ww < w; ++ww)
            run += s_wave[ww];
        if (t == EMIT_BLOCK - 1)
            s_wave[EMIT_BLOCK / 64] = run + sum; // the tile's messages
        for (u32 q = first; q < last; ++q) {
            const u32 c = s_cnt[q];
            s_excl[q] = run;
            if (c)
                s_base[q] = atomicAdd(&a.msg_off[q], c);
            run += c;
        }
        __syncthreads();
        const u32 total = s_wave[EMIT_BLOCK / 64];
#pragma unroll
        for (int e = 0; e < 2 * EMIT_ITEMS; ++e) {
            if (m[e].dest == 0xFFFFFFFFu)
                continue;
            const u32 at = s_excl[m[e].dest] + slot[e];
            s_low[at] = (u32)m[e].target;
            s_high[at] = (u8)(m[e].target >> 32);
            s_rank[at] = m[e].rank;
            s_dest[at] = (u16)m[e].dest;
        }
        __syncthreads();
        for (u32 j = t; j < total; j += EMIT_BLOCK) {
            const u32 d = s_dest[j];
            const u64 s = (u64)s_base[d] + (j - s_excl[d]);
            const u32 low = s_low[j];
#pragma unroll
            for (int b = 0; b < 4; ++b)
                a.msg_target[5 * s + b] = (u8)(low >> (8 * b));
            a.msg_target[5 * s + 4] = s_high[j];
            a.msg_rank[s] = s_rank[j];
        }
    }
}

// In-place exclusive prefix sum of `count` counters (count <= 32769: one per partition and one more), one workgroup.
// Replaces cub::DeviceScan::ExclusiveSum over the p + 1 message counters (src/GPU_SACA.cu:1278-1283).
__global__ __launch_bounds__(1024) void message_offsets_kernel(u32* v, u32 count)
{
    __shared__ u32 s_w[16];
    const u32 t = threadIdx.x, lane = t & 63u, w = t >> 6;
    const u32 per = (count + 1023u) / 1024u;
    const u32 first = t * per < count ? t * per : count;
    const u32 last = first + per < count ? first + per : count;
    u32 sum = 0;
    for (u32 i = first; i < last; ++i)
        sum += v[i];
    const u32 incl = wave_incl_sum(sum);
    if (lane == 63u)
        s_w[w] = incl;
    __syncthreads();
    u32 run = incl - sum;
    for (u32 ww = 0; ww < w; ++ww)
        run += s_w[ww];
    for (u32 i = first; i < last; ++i) {
        const u32 c = v[i];
        v[i] = run;
        run += c;
    }
}

// A directory over the suffix-ordered cohort SA[0, n): dir[b] = first place whose suffix is >= b << shift, for b in
// [0, 2^dir_log2], where shift spreads the directory over the values up to the cohort's largest suffix. A search for a
// target then starts inside one bucket (a few neighbouring entries, one or two cache lines) instead of walking the whole
// array, which would cost a cache line from HBM for every level below the cached top of the search tree.
__device__ __forceinline__ u32 join_directory_shift(const u64* __restrict__ sa, u64 n, u32 dir_log2)
{
    const u64 largest = sa[n - 1] & MSG_VAL_MASK;
    const u32 span = 64u - (u32)__builtin_clzll(largest | 1ull);
    return span > dir_log2 ? span - dir_log2 : 0u;
}

__global__ __launch_bounds__(256) void join_directory_kernel(const u64* __restrict__ sa, u64 n, u32 dir_log2, u32* __restrict__ dir)
{
    const u64 b = (u64)blockIdx.x * 256 + threadIdx.x;
    if (b > (1ull << dir_log2))
        return;
    const u64 v = b << join_directory_shift(sa, n, dir_log2);
    u64 low = 0, high = n;
    while (low < high) {
        const u64 mid = low + (high - low) / 2;
        if ((sa[mid] & MSG_VAL_MASK) < v)
            low = mid + 1;
        else
            high = mid;
    }
    dir[b] = (u32)low;
}

// Delivers every message to its recipient in the suffix-ordered cohort SA[0, n): K[pos] = primary[pos] << 31 |
// received rank, marked if the message is a pill; a recipient that is not in the cohort has retired and the
// message is dropped (include/GPU_SACA.cuh:362-389).
// The targets come as 5-byte lanes (msg_target) or, when the inbox was sorted by target first, as 64-bit words
// (target_words): sorted targets probe neighbouring places of the cohort, so that the probes of a wave share
// cache lines instead of each costing a line from HBM. With a directory (dir != null, from join_directory_kernel) the
// search is confined to the target's bucket.
__global__ __launch_bounds__(256) void join_messages_kernel(const u8* __restrict__ msg_target,
                                                            const u64* __restrict__ target_words,
                                                            const u32* __restrict__ msg_rank, u32 msg_c,
                                                            const u64* __restrict__ sa, const u32* __restrict__ primary,
                                                            u64* keys, u64 n, const u32* __restrict__ dir, u32 dir_log2)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i >= msg_c)
        return;
    u64 tgt = 0;
    if (target_words) {
        tgt = target_words[i] & MSG_VAL_MASK;
    } else {
#pragma unroll
        for (int b = 0; b < 5; ++b)
            tgt |= (u64)msg_target[5 * i + b] << (8 * b);
    }
    u64 low = 0, high = n;
    if (dir) {
        const u64 b = tgt >> join_directory_shift(sa, n, dir_log2);
        if (b >= (1ull << dir_log2))
            return; // beyond the cohort's largest suffix
        low = dir[b];
        high = dir[b + 1];
    }
    const u64 end = high;
    while (low < high) {
        const u64 mid = low + (high - low) / 2;
        if ((sa[mid] & MSG_VAL_MASK) < tgt)
            low = mid + 1;
        else
            high = mid;
    }
    // a target that is absent from its bucket is absent from the cohort: the next bucket starts above it
    if (low == end || (sa[low] & MSG_VAL_MASK) != tgt)
        return;
    const u32 r = msg_rank[i];
    u64 key = ((u64)primary[low] << 31) | (u64)(r & ~MSG_PILL_BIT);
    if (r & MSG_PILL_BIT)
        key |= MSG_PILL_RECEIPT;
    keys[low] = key;
}

// ---- the join through a hash table over the cohort's suffixes (the per-generation step) ----
//
// The step receives its cohort in rank order and needs it in suffix order for nothing but the join. Instead of sorting
// it by suffix (five radix passes and two gathers, src/GPU_SACA.cu:1769-1800) and searching, the cohort's suffixes go into
// an open-addressed table (linear probing; a slot holds the 40-bit suffix, a parallel array the member's list place), and
// every message probes it: a message whose recipient has retired, which most are, ends at an empty slot of the line it
// read first, instead of a directory line and a line of the sorted cohort. What a message delivers is the 32-bit rank
// word as it came (pill bit included) at the recipient's list place; the composite keys are put together afterwards in
// one streaming pass. Same outcome as join_messages_kernel (include/GPU_SACA.cuh:362-389).
constexpr u64 JOIN_EMPTY = ~0ull;      // no suffix is all ones (suffixes are below 2^40)
constexpr u32 JOIN_NOTHING = ~0u;      // no rank word is all ones: ranks are below 2^31 - 1 (only the forwarded pill of a member that
                                       // no message joined would be, which the exchange scheme excludes; it counts as nothing)

__device__ __forceinline__ u64 join_home(u64 suffix, u64 slots)
{
    return __umul64hi(suffix * 0x9E3779B97F4A7C15ull, slots); // the high word of a 128-bit product: in [0, slots)
}

__device__ __forceinline__ u64 lane_value(const u8* __restrict__ lanes, u64 i)
{
    u64 v = 0;
#pragma unroll
    for (int b = 0; b < 5; ++b)
        v |= (u64)lanes[5 * i + b] << (8 * b);
    return v;
}

// table[s] = suffix of list place place_of[s]; `slots` >= m entries, all JOIN_EMPTY before the launch
__global__ __launch_bounds__(256) void join_table_insert_kernel(const u8* __restrict__ suf40, u64 m, unsigned long long* table,
                                                                u32* __restrict__ place_of, u64 slots, u32* err)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i >= m)
        return;
    const u64 suffix = lane_value(suf40, i);
    u64 s = join_home(suffix, slots);
    for (u64 step = 0; step < slots; ++step) {
        // an atomic costs several times a load: only a slot that reads empty is tried
        if (*(volatile unsigned long long*)&table[s] == JOIN_EMPTY &&
            atomicCAS(&table[s], (unsigned long long)JOIN_EMPTY, (unsigned long long)suffix) == JOIN_EMPTY) {
            place_of[s] = (u32)i;
            return;
        }
        s = s + 1 == slots ? 0 : s + 1;
    }
    atomicExch(err, DEV_ERR_JOIN_TABLE_FULL); // more members than slots: the caller sized the table wrongly
}

// sec[place] = rank word of the message whose target is the member at that list place (sec is JOIN_NOTHING-filled)
__global__ __launch_bounds__(256) void join_table_probe_kernel(const u8* __restrict__ msg_target, const u32* __restrict__ msg_rank, u32 msg_c,
                                                               const unsigned long long* __restrict__ table, const u32* __restrict__ place_of,
                                                               u64 slots, u32* __restrict__ sec)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i >= msg_c)
        return;
    const u64 target = lane_value(msg_target, i);
    u64 s = join_home(target, slots);
    for (u64 step = 0; step < slots; ++step) {
        const u64 v = table[s];
        if (v == JOIN_EMPTY)
            return; // the recipient is not in the cohort: it has retired, the message is dropped
        if (v == target) {
            sec[place_of[s]] = msg_rank[i];
            return;
        }
        s = s + 1 == slots ? 0 : s + 1;
    }
}

// keys[i] = primary[i] << 31 | received rank, marked if the message was a pill; all ones where nothing arrived
// (src/GPU_SACA.cu:1826, include/GPU_SACA.cuh:383-387)
__global__ __launch_bounds__(256) void compose_join_keys_kernel(const u32* __restrict__ primary, const u32* __restrict__ sec, u64 m,
                                                                u64* __restrict__ keys)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i >= m)
        return;
    const u32 r = sec[i];
    u64 key = ~0ull;
    if (r != JOIN_NOTHING) {
        key = ((u64)primary[i] << 31) | (u64)(r & ~MSG_PILL_BIT);
        if (r & MSG_PILL_BIT)
            key |= MSG_PILL_RECEIPT;
    }
    keys[i] = key;
}

// words[i] = suffix of list place perm[i] (5-byte lanes gathered through a permutation)
__global__ __launch_bounds__(256) void gather_lanes_kernel(const u8* __restrict__ lanes, const u32* __restrict__ perm, u64 count,
                                                           u64* __restrict__ words)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i < count)
        words[i] = lane_value(lanes, perm[i]);
}

// 5-byte lanes -> 64-bit words (the keys of the inbox sort)
__global__ __launch_bounds__(256) void unpack_lanes_kernel(const u8* __restrict__ lanes, u64 count, u64* __restrict__ words)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i >= count)
        return;
    u64 v = 0;
#pragma unroll
    for (int b = 0; b < 5; ++b)
        v |= (u64)lanes[5 * i + b] << (8 * b);
    words[i] = v;
}

} // namespace csa
