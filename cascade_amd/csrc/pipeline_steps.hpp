// Kernels of the per-generation partition steps that keep the reference's exchange scheme: a partition arrives as
// (key | rank, suffix lane, routing tags [, inbox]) and leaves as (rank, suffix lane) in "active first, retired after"
// order plus an outbox of rank messages (reference: GPU_SACA::sort_and_init_rank_and_filter and
// GPU_SACA::sort_and_re_rank_and_filter, src/GPU_SACA.cu:1112-1331 and 1715-1995). The sorts are the library's radix
// sort on (64-bit key, 32-bit permutation) pairs, as the reference sorts with cub; the kernels here are the glue:
// lane unpacking, gathers through the permutation, run ranking with the active/retired split, narrowing.
#pragma once

#include "device_utils.hpp"
#include "doubling.hpp"
#include "messages.hpp"

namespace csa {

constexpr int STEP_BLOCK = 256;
constexpr int STEP_ITEMS = 4;
constexpr int STEP_TILE = STEP_BLOCK * STEP_ITEMS;
constexpr u64 STEP_KEY62 = (1ull << 62) - 1ull;    // (primary, secondary): the sorted bits of a composite key
constexpr u64 STEP_SECONDARY = (1ull << 31) - 1ull;

__global__ __launch_bounds__(256) void iota_kernel(u32* p, u64 count)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i < count)
        p[i] = (u32)i;
}

// keys[i] = forward tag of suffix i: the high half of its routing-tag pair (include/bit-layout.hpp:141-145)
__global__ __launch_bounds__(256) void tag_keys_kernel(const u32* __restrict__ beta, u64 count, u64* __restrict__ keys)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i < count)
        keys[i] = beta[i] >> 16;
}

// dst[i] = src[perm[i] * stride + offset]
__global__ __launch_bounds__(256) void gather_u64_kernel(const u64* __restrict__ src, const u32* __restrict__ perm, u64 count,
                                                         u32 stride, u32 offset, u64* __restrict__ dst)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i < count)
        dst[i] = src[(u64)perm[i] * stride + offset];
}

__global__ __launch_bounds__(256) void gather_u32_kernel(const u32* __restrict__ src, const u32* __restrict__ perm, u64 count,
                                                         u32* __restrict__ dst)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i < count)
        dst[i] = src[perm[i]];
}

// keys[i] = forward tag of suffix perm[i]
__global__ __launch_bounds__(256) void gather_tag_keys_kernel(const u32* __restrict__ beta, const u32* __restrict__ perm, u64 count,
                                                              u64* __restrict__ keys)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i < count)
        keys[i] = beta[perm[i]] >> 16;
}

// dst[pos[i]] = src[i] (pos strictly increasing: the places of the tied entries in the sorted list)
__global__ __launch_bounds__(256) void scatter_u32_kernel(const u32* __restrict__ src, const u32* __restrict__ pos, u64 count, u64 m,
                                                          u32* __restrict__ dst, u32* err)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i >= count)
        return;
    const u32 at = pos[i];
    if (at < m)
        dst[at] = src[i];
    else
        atomicExch(err, DEV_ERR_RERANK_RANGE);
}

// Entries of a list sorted by its first key word that tie with a neighbour on that word, compacted in order: their
// places in the list and the suffixes (permutation entries) at those places. Only they can change places when the later
// key words and the forward tag are taken into account, and they stay inside their run. Two launches around
// rerank_scan_kernel (count, apply), like the rank step.
struct TieArgs {
    const u64* keys; // sorted
    const u32* perm;
    u64 m;
    u32* pos_out;
    u32* perm_out;
    u32* tile_agg;    // [tiles][4]: slot 2 carries the count
    u32* tile_splits; // [tiles]
    const u32* tile_prefix;
    const u32* slab_total;
    u32 slab;
    u32 slabs;
    unsigned long long* total_out;
};

template <bool APPLY>
__global__ __launch_bounds__(STEP_BLOCK) void tie_kernel(TieArgs a)
{
    constexpr int WAVES = STEP_BLOCK / WAVE;
    __shared__ u32 s_w[WAVES];
    const u32 t = threadIdx.x, lane = t & 63u, w = t >> 6;
    const u32 tile = blockIdx.x;
    const u64 base = (u64)tile * STEP_TILE + (u64)t * STEP_ITEMS;
    u64 key[STEP_ITEMS + 2]; // entries base - 1 .. base + STEP_ITEMS
#pragma unroll
    for (int k = 0; k < STEP_ITEMS + 2; ++k) {
        const u64 c = base + k;
        key[k] = (c >= 1 && c - 1 < a.m) ? a.keys[c - 1] : 0;
    }
    u32 tied = 0, cnt = 0;
#pragma unroll
    for (int k = 0; k < STEP_ITEMS; ++k) {
        const u64 i = base + k;
        if (i < a.m) {
            const bool left = i >= 1 && key[k] == key[k + 1], right = i + 1 < a.m && key[k + 2] == key[k + 1];
            if (left || right) {
                tied |= 1u << k;
                cnt++;
            }
        }
    }
    const u32 ic = wave_incl_sum(cnt);
    if (lane == 63u)
        s_w[w] = ic;
    __syncthreads();
    u32 before = ic - cnt, total = 0;
    for (u32 ww = 0; ww < WAVES; ++ww) {
        if (ww < w)
            before += s_w[ww];
        total += s_w[ww];
    }
    if (!APPLY) {
        if (t == 0) {
            a.tile_agg[(u64)tile * 4 + 0] = 0;
            a.tile_agg[(u64)tile * 4 + 1] = 0;
            a.tile_agg[(u64)tile * 4 + 2] = total;
            a.tile_agg[(u64)tile * 4 + 3] = 0;
            a.tile_splits[tile] = 0;
        }
        return;
    }
    u32 at = a.tile_prefix[(u64)tile * 4 + 2] + slabs_before(a.slab_total, tile / a.slab).sum2 + before;
    const u32 all = slabs_before(a.slab_total, a.slabs).sum2;
    if (tile == 0 && t == 0)
        *a.total_out = all;
#pragma unroll
    for (int k = 0; k < STEP_ITEMS; ++k) {
        if (tied & (1u << k)) {
            const u64 i = base + k;
            a.pos_out[at] = (u32)i;
            a.perm_out[at] = a.perm[i];
            at++;
        }
    }
}

// words[i] = suffix of lane perm[i] (or i), with the forward tag of its routing tags in the top 16 bits when with_tag
// (reference: unpack_tagged_lanes_kernel / unpack_lanes_kernel, include/GPU_SACA.cuh:94-119); beta_out[i] = beta[perm[i]].
__global__ __launch_bounds__(256) void unpack_words_kernel(const u8* __restrict__ lanes, const u32* __restrict__ beta,
                                                           const u32* __restrict__ perm, u64 count, int with_tag,
                                                           u64* __restrict__ words, u32* __restrict__ beta_out)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i >= count)
        return;
    const u64 j = perm ? perm[i] : i;
    u64 v = 0;
#pragma unroll
    for (int b = 0; b < 5; ++b)
        v |= (u64)lanes[5 * j + b] << (8 * b);
    const u32 bt = beta ? beta[j] : 0u;
    words[i] = with_tag ? (v | ((u64)(bt >> 16) << 48)) : v;
    if (beta_out)
        beta_out[i] = bt;
}

// carried[i] = (suffix of lane i with the forward tag in the top 16 bits, routing tags of suffix i): what generation 0
// moves along with a suffix, in one 16-byte record
__global__ __launch_bounds__(256) void pack_carried_kernel(const u8* __restrict__ lanes, const u32* __restrict__ beta, u64 count,
                                                           uint4* __restrict__ carried)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i >= count)
        return;
    u64 v = 0;
#pragma unroll
    for (int b = 0; b < 5; ++b)
        v |= (u64)lanes[5 * i + b] << (8 * b);
    const u32 bt = beta[i];
    v |= (u64)(bt >> 16) << 48;
    carried[i] = make_uint4((u32)v, (u32)(v >> 32), bt, 0u);
}

// keys[i] = forward tag of suffix i, from its carried record
__global__ __launch_bounds__(256) void carried_tag_keys_kernel(const uint4* __restrict__ carried, u64 count, u64* __restrict__ keys)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i < count)
        keys[i] = carried[i].z >> 16;
}

// words[i], beta_out[i] = the record of suffix perm[i]
__global__ __launch_bounds__(256) void gather_carried_kernel(const uint4* __restrict__ carried, const u32* __restrict__ perm, u64 count,
                                                             u64* __restrict__ words, u32* __restrict__ beta_out)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i >= count)
        return;
    const uint4 r = carried[perm[i]];
    words[i] = (u64)r.x | ((u64)r.y << 32);
    beta_out[i] = r.z;
}

// Run ranking with the active / retired split, in the three launches of the rank step (count, rerank_scan_kernel, apply).
// Generation 0: the list is sorted by (key words, forward tag); rank = offset of the head of the run of equal
// (key, tag), stored as a plain rank (include/GPU_SACA.cuh:191-208). Generation t: the list is sorted by the composite
// key; refined primary = primary + (head of the key run - head of the primary run), secondary and pill receipt kept
// (include/GPU_SACA.cuh:218-280). An entry is active iff its run is longer than one. Active entries go first, in
// order; retired ones follow (reference: cub::DevicePartition::Flagged, which reverses them: their order carries nothing).
struct StepRankArgs {
    const u64* key0;  // generation 0: sorted key word 0; generation t: sorted composite keys
    const u64* key1;  // generation 0 with keys of two or more words: sorted key word 1, else null
    const u64* keys_src; // generation 0 with keys of three or four words: the caller's keys (key_words per suffix) ...
    const u32* perm;     // ... and the permutation that sorted them: words 2 and 3 are compared through it where words 0
    int key_words;       //     and 1 tie
    const u64* words; // suffix words in the same order (generation 0: forward tag in the top 16 bits)
    const u32* beta;
    u64 m;
    u64* key_out;
    u64* words_out;
    u32* beta_out;
    u32* tile_agg;    // [tiles][4]
    u32* tile_splits; // [tiles]
    u32* tile_prefix; // [tiles][4]
    u32* slab_total;  // [RERANK_SLABS][5]
    u32 slab;
    u32 slabs;
    unsigned long long* active_out; // size of the active set
    // generation t: what the reference counts and checks under -DTESTS (include/GPU_SACA.cuh:234-249): cohort members no
    // message joined, members a poison pill joined, and neighbours with equal (primary, secondary) of which only one
    // carries a pill receipt
    unsigned long long* unserved_out;
    unsigned long long* pills_out;
    u32* incoherent_out;
};

template <bool GEN0>
__device__ __forceinline__ bool step_same_key(const StepRankArgs& a, u64 i, u64 j)
{
    if (GEN0) {
        bool same = a.key0[i] == a.key0[j] && (!a.key1 || a.key1[i] == a.key1[j]) && (a.words[i] >> 48) == (a.words[j] >> 48);
        for (int w = 2; same && w < a.key_words; ++w)
            same = a.keys_src[(u64)a.perm[i] * a.key_words + w] == a.keys_src[(u64)a.perm[j] * a.key_words + w];
        return same;
    }
    return a.key0[i] == a.key0[j]; // whole words: tied entries agree on the pill receipt
}

template <bool GEN0>
__device__ __forceinline__ bool step_same_primary(const StepRankArgs& a, u64 i, u64 j)
{
    if (GEN0)
        return true; // one primary group: the partition
    return ((a.key0[i] & STEP_KEY62) >> 31) == ((a.key0[j] & STEP_KEY62) >> 31);
}

template <bool GEN0, bool APPLY>
__global__ __launch_bounds__(STEP_BLOCK) void step_rank_kernel(StepRankArgs a)
{
    constexpr int WAVES = STEP_BLOCK / WAVE;
    __shared__ u32 s_w[WAVES][5];
    const u32 t = threadIdx.x, lane = t & 63u, w = t >> 6;
    const u32 tile = blockIdx.x;
    const u64 base = (u64)tile * STEP_TILE + (u64)t * STEP_ITEMS;
    // heads are 1-based positions (0 = none so far)
    bool kh[STEP_ITEMS + 1], ph[STEP_ITEMS];
    u32 la = 0, lb = 0, lact = 0, lun = 0, lpill = 0;
#pragma unroll
    for (int k = 0; k < STEP_ITEMS + 1; ++k) {
        const u64 i = base + k;
        kh[k] = i < a.m ? (i == 0 || !step_same_key<GEN0>(a, i, i - 1)) : true; // the end of the list closes the last run
    }
#pragma unroll
    for (int k = 0; k < STEP_ITEMS; ++k) {
        const u64 i = base + k;
        ph[k] = i < a.m && (i == 0 || !step_same_primary<GEN0>(a, i, i - 1));
        if (i < a.m) {
            if (kh[k])
                la = (u32)i + 1u;
            if (ph[k])
                lb = (u32)i + 1u;
            lact += (kh[k] && kh[k + 1]) ? 0u : 1u;
            if (!GEN0 && !APPLY) {
                const u64 key = a.key0[i];
                if ((key & STEP_SECONDARY) == STEP_SECONDARY)
                    lun++;
                else if (key & MSG_PILL_RECEIPT)
                    lpill++;
                if (i > 0) {
                    const u64 differ = key ^ a.key0[i - 1];
                    if ((differ & STEP_KEY62) == 0 && (differ & MSG_PILL_RECEIPT))
                        atomicAdd(a.incoherent_out, 1u);
                }
            }
        }
    }
    const u32 ia = wave_incl_max(la), ib = wave_incl_max(lb), ic = wave_incl_sum(lact);
    if (!GEN0 && !APPLY) {
        lun = wave_reduce_sum(lun);
        lpill = wave_reduce_sum(lpill);
    }
    if (lane == 63u) {
        s_w[w][0] = ia;
        s_w[w][1] = ib;
        s_w[w][2] = ic;
        s_w[w][3] = lun;
        s_w[w][4] = lpill;
    }
    __syncthreads();
    u32 xa = __shfl_up(ia, 1), xb = __shfl_up(ib, 1), xc = __shfl_up(ic, 1);
    if (lane == 0)
        xa = xb = xc = 0;
    u32 ta = 0, tb = 0, tc = 0;
    for (u32 ww = 0; ww < WAVES; ++ww) {
        if (ww < w) {
            xa = xa > s_w[ww][0] ? xa : s_w[ww][0];
            xb = xb > s_w[ww][1] ? xb : s_w[ww][1];
            xc += s_w[ww][2];
        }
        ta = ta > s_w[ww][0] ? ta : s_w[ww][0];
        tb = tb > s_w[ww][1] ? tb : s_w[ww][1];
        tc += s_w[ww][2];
    }
    if (!APPLY) {
        if (t == 0) {
            u32 tun = 0, tpill = 0;
            for (u32 ww = 0; ww < WAVES; ++ww) {
                tun += s_w[ww][3];
                tpill += s_w[ww][4];
            }
            a.tile_agg[(u64)tile * 4 + 0] = ta;
            a.tile_agg[(u64)tile * 4 + 1] = tb;
            a.tile_agg[(u64)tile * 4 + 2] = tc;
            a.tile_agg[(u64)tile * 4 + 3] = tun;  // summed by the scan like the active count
            a.tile_splits[tile] = tpill;          // at most STEP_TILE: the scan adds the low 16 bits up per slab
        }
        return;
    }
    u32 pre_a = a.tile_prefix[(u64)tile * 4 + 0], pre_b = a.tile_prefix[(u64)tile * 4 + 1];
    u32 pre_c = a.tile_prefix[(u64)tile * 4 + 2];
    const SlabPrefix sp = slabs_before(a.slab_total, tile / a.slab);
    pre_a = pre_a > sp.max0 ? pre_a : sp.max0;
    pre_b = pre_b > sp.max1 ? pre_b : sp.max1;
    pre_c += sp.sum2;
    const SlabPrefix all = slabs_before(a.slab_total, a.slabs);
    const u32 total_active = all.sum2;
    if (tile == 0 && w == 0) {
        u32 pills = lane < a.slabs ? a.slab_total[lane * 5 + 4] : 0u; // one slab per lane
        pills = wave_reduce_sum(pills);
        if (lane == 0) {
            *a.active_out = total_active;
            if (!GEN0) {
                *a.unserved_out = all.sum3;
                *a.pills_out = pills;
            }
        }
    }
    u32 ra = xa > pre_a ? xa : pre_a, rb = xb > pre_b ? xb : pre_b;
    u32 act_before = pre_c + xc; // active entries before this thread's first
    // everything the thread moves is read before its first store: the outputs may alias the inputs as far as the
    // compiler can tell, and loads behind a store would wait for it
    u64 old_key[STEP_ITEMS], old_word[STEP_ITEMS];
    u32 old_beta[STEP_ITEMS];
#pragma unroll
    for (int k = 0; k < STEP_ITEMS; ++k) {
        const u64 i = base + k;
        old_key[k] = i < a.m ? a.key0[i] : 0ull;
        old_word[k] = i < a.m ? a.words[i] : 0ull;
        old_beta[k] = i < a.m ? a.beta[i] : 0u;
    }
#pragma unroll
    for (int k = 0; k < STEP_ITEMS; ++k) {
        const u64 i = base + k;
        if (i >= a.m)
            continue;
        if (kh[k])
            ra = (u32)i + 1u;
        if (ph[k])
            rb = (u32)i + 1u;
        const bool active = !(kh[k] && kh[k + 1]);
        const u64 old = old_key[k];
        u64 key;
        if (GEN0) {
            key = (u64)(ra - 1u); // plain rank: offset of the run's head
        } else {
            const u64 primary = ((old & STEP_KEY62) >> 31) + (u64)(ra - rb);
            key = (primary << 31) | (old & STEP_SECONDARY) | (old & MSG_PILL_RECEIPT);
        }
        const u64 dest = active ? (u64)act_before : (u64)total_active + (i - act_before);
        a.key_out[dest] = key;
        a.words_out[dest] = old_word[k];
        a.beta_out[dest] = old_beta[k];
        act_before += active ? 1u : 0u;
    }
}

// What a step persists per suffix: its partition-local rank narrowed to 32 bits and its 5-byte lane
// (reference: extract_primary_keys_kernel, include/GPU_SACA.cuh:397-409; pack_lanes_kernel, :126-133).
__global__ __launch_bounds__(256) void narrow_and_pack_kernel(const u64* __restrict__ keys, const u64* __restrict__ words, u64 count,
                                                              int packed, u32* __restrict__ rank_out, u8* __restrict__ lanes_out)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i >= count)
        return;
    const u64 k = keys[i];
    rank_out[i] = packed ? (u32)((k & STEP_KEY62) >> 31) : (u32)k;
    const u64 v = words[i];
#pragma unroll
    for (int b = 0; b < 5; ++b)
        lanes_out[5 * i + b] = (u8)(v >> (8 * b));
}

__global__ __launch_bounds__(256) void fill_u64_kernel(u64* p, u64 count, u64 v)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i < count)
        p[i] = v;
}

} // namespace csa
