// Kernels of the prefix-doubling generations: rank assignment / compaction after a sort, the in-tile
// sort of small groups (which gathers rank[x + h]), the return of radix-sorted large groups, sa40
// emission, K-gram packing and the device-side suffix-array check.
#pragma once

#include "device_utils.hpp"

namespace csa {

// ---------------------------------------------------------------------------------------------
// Generation 0: rank assignment + compaction of the sorted K-gram keys in three launches: per-tile aggregates, a scan
// of the aggregates over the tiles, and the pass that applies them. (A single launch with a decoupled look-back
// was measured at 2.5 to 4 times the duration of these three on this part: with 8 XCDs the look-back words travel
// over the fabric, and the few resident workgroups per CU spent most of their life waiting for their predecessors.)
//
// Input: all suffixes sorted by key, keys[c] / sufs[c] for c in [0, n). The rank of a suffix is the index of the
// head of its run of equal keys (reference: include/GPU_SACA.cuh:191-208; the max-scan of src/GPU_SACA.cu:1241-1247
// is the max chain here). A suffix whose run has length 1 retires: its rank is final, and the sorted index array
// already holds it at its place of the suffix array. The others are compacted, in order, into the first active list
// (reference: cub::DevicePartition::Flagged, src/GPU_SACA.cu:1253-1261), each with the dense id of its group.
// ---------------------------------------------------------------------------------------------

constexpr u32 NO_RANK = 0xFFFFFFFFu; // ranks are below 2^31

// The tiles of a rank step are scanned in RERANK_SLABS slabs (rerank_scan_kernel): a tile's prefix is its prefix inside
// its slab combined with the totals (max, max, sum, sum, -) of the slabs before. One slab per lane: a wave fetches the
// totals in one round trip and reduces them, instead of walking them one after the other (up to 63 dependent loads
// at the head of every workgroup of kernels that live on latency). Call with all 64 lanes; the same values return in each.
constexpr u32 RERANK_SLABS = 64;
static_assert(RERANK_SLABS == WAVE, "one slab total per lane");

struct SlabPrefix {
    u32 max0, max1, sum2, sum3;
};

__device__ __forceinline__ SlabPrefix slabs_before(const u32* __restrict__ slab_total, u32 slabs_before_mine)
{
    const u32 lane = threadIdx.x & 63u;
    SlabPrefix p = {0u, 0u, 0u, 0u};
    if (lane < slabs_before_mine) {
        p.max0 = slab_total[lane * 5 + 0];
        p.max1 = slab_total[lane * 5 + 1];
        p.sum2 = slab_total[lane * 5 + 2];
        p.sum3 = slab_total[lane * 5 + 3];
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const u32 o0 = __shfl_xor(p.max0, o), o1 = __shfl_xor(p.max1, o);
        p.max0 = p.max0 > o0 ? p.max0 : o0;
        p.max1 = p.max1 > o1 ? p.max1 : o1;
        p.sum2 += __shfl_xor(p.sum2, o);
        p.sum3 += __shfl_xor(p.sum3, o);
    }
    return p;
}

constexpr u32 MAX_LEVELS = 4, LEVEL_SLOTS = 64;

struct RerankArgs {
    const u64* keys;
    const u32* sufs;
    u32 m;         // = n: generation 0 ranks every suffix
    int key_words; // 1..4 (the words after the first are re-read from the text where the first words tie)
    u32 n;         // partition size
    u32 ell;       // symbols in the generation-0 key
    // Packed keys of many symbols (packed_text.hpp): the counting pass also counts what the list would leave at shorter
    // contexts. Level i looks at the key bits above level_drop[i] and sets apart the suffixes that run off the text inside
    // level_ell[i] symbols; its survivors and groups are added to level_totals[slot * 8 + 2 i] and [.. + 1], slot = tile
    // % LEVEL_SLOTS (spread so that the additions of neighbouring tiles do not queue on one address; zeroed by the caller).
    u32 levels; // <= MAX_LEVELS
    u32 level_drop[4];
    u32 level_ell[4];
    unsigned long long* level_totals;
    const u16* text;
    u32* rank;     // [n] by text position
    // Deferred rank update: instead of the scattered write rank[x] = r, the suffix at sorted index c leaves the record
    // (x << 32) | r at rank_recs[c] (a coalesced stream). The records then go through radix passes on the high bits of
    // x before they are written to rank[], so that those writes fall into one window of rank[] at a time.
    u64* rank_recs; // null: write rank[x] directly
    // 0: the value kept for suffix x is its rank (index of the head of its key run). 1: it is the run's ordinal, the
    // number of key runs before it (the ranks renumbered 0, 1, 2, ...): what the next generation wants when it sorts the
    // whole partition again by pairs of these values read in text order (rank_pair_key with a radix). Counted without
    // a scan of its own: runs before a place = groups begun before it + singletons before it, and an element that is
    // not a survivor is a singleton.
    u32 ordinals;
    u32* sufs_out;  // first active list
    u32* gids_out;
    u32* gprim_out;
    u32* gstart_out; // index in the active list where each group starts; [groups] = survivors
    u32* tile_agg;    // [tiles][4]: last key-run head (1-based, 0 = none), unused, survivors, groups of each tile
    u32* tile_splits; // [tiles]: changed-rank counts for the scan (zero here: generation 0 writes every rank)
    u32* tile_prefix; // [tiles][4]: the aggregates combined over the earlier tiles of the tile's slab (max, -, sum, sum)
    u32* slab_total;  // [RERANK_SLABS][5]: combination over each slab of tiles
    u32 slab;         // tiles per slab
    u32* err;
};

// Elements base - 1 .. base + ITEMS of the sorted (key, suffix) list, m elements long, for the thread that owns
// elements base .. base + ITEMS - 1 (base a multiple of ITEMS): its own in whole 16-byte loads where they all exist,
// zeros outside the list.
template <int ITEMS>
__device__ __forceinline__ void load_with_neighbours(const u64* __restrict__ keys, const u32* __restrict__ sufs, u64 base, u32 m,
                                                     u64 (&key)[ITEMS + 2], u32 (&suf)[ITEMS + 2])
{
    if (ITEMS % 4 == 0 && base + ITEMS <= m) {
        const uint4* k4 = reinterpret_cast<const uint4*>(keys + base);
        const uint4* s4 = reinterpret_cast<const uint4*>(sufs + base);
#pragma unroll
        for (int k = 0; k < ITEMS; k += 2) {
            const uint4 v = k4[k / 2];
            key[k + 1] = (u64)v.x | ((u64)v.y << 32);
            key[k + 2] = (u64)v.z | ((u64)v.w << 32);
        }
#pragma unroll
        for (int k = 0; k < ITEMS; k += 4) {
            const uint4 v = s4[k / 4];
            suf[k + 1] = v.x;
            suf[k + 2] = v.y;
            suf[k + 3] = v.z;
            suf[k + 4] = v.w;
        }
        key[0] = base >= 1 ? keys[base - 1] : 0;
        suf[0] = base >= 1 ? sufs[base - 1] : 0;
        const bool last_in = base + ITEMS < m;
        key[ITEMS + 1] = last_in ? keys[base + ITEMS] : 0;
        suf[ITEMS + 1] = last_in ? sufs[base + ITEMS] : 0;
    } else {
#pragma unroll
        for (int k = 0; k < ITEMS + 2; ++k) {
            const u64 c = base + k; // element c - 1
            const bool in = c >= 1 && c - 1 < m;
            key[k] = in ? keys[c - 1] : 0;
            suf[k] = in ? sufs[c - 1] : 0;
        }
    }
}

// The counting pass of generation 0 on its own: the per-tile aggregates need no ordering inside the tile, so every
// thread reads its ITEMS elements and their two neighbours straight from the arrays (no exchange through LDS, one
// barrier) and the tile reduces instead of scanning. Same run and tail rules as rerank_kernel below.
template <int BLOCK, int ITEMS>
__global__ __launch_bounds__(BLOCK) void rerank_count_kernel(RerankArgs a)
{
    constexpr int TILE = BLOCK * ITEMS;
    constexpr int WAVES = BLOCK / WAVE;
    __shared__ u32 s_wagg[WAVES][3];
    const u32 t = threadIdx.x;
    const u32 lane = t & 63u;
    const u32 w = t >> 6;
    const u32 tile = blockIdx.x;
    const u64 base = (u64)tile * TILE + (u64)t * ITEMS;
    const u32 m = a.m;
    u64 key[ITEMS + 2]; // elements base - 1 .. base + ITEMS
    u32 suf[ITEMS + 2];
    load_with_neighbours<ITEMS>(a.keys, a.sufs, base, m, key, suf);
    u32 la = 0, lcnt = 0, lheads = 0;
    bool prev_eq = false;
#pragma unroll
    for (int k = 0; k < ITEMS + 1; ++k) {
        const u64 c = base + k; // right element of the pair (c - 1, c)
        bool e = c >= 1 && c < m && key[k] == key[k + 1];
        for (int word = 1; e && word < a.key_words; ++word)
            e = load_kgram(a.text, a.n, suf[k], (u32)word) == load_kgram(a.text, a.n, suf[k + 1], (u32)word);
        // a suffix that runs off the text inside its key ties with nobody (include/bit-layout.hpp:99-100)
        if (e && ((u64)suf[k] + a.ell >= a.n || (u64)suf[k + 1] + a.ell >= a.n))
            e = false;
        if (k >= 1 && c - 1 < m) { // element c - 1 = base + k - 1: prev_eq ties it to its left, e to its right
            const bool ka = !prev_eq;
            const bool single = ka && !e;
            if (ka)
                la = (u32)(c - 1) + 1u;
            lcnt += single ? 0u : 1u;
            lheads += (ka && !single) ? 1u : 0u;
        }
        prev_eq = e;
    }
    // the same counts at the shorter contexts of packed keys (one-word keys: nothing is read from the text)
    __shared__ u32 s_level[WAVES][MAX_LEVELS];
    for (u32 i = 0; i < a.levels; ++i) {
        const u32 drop = a.level_drop[i];
        const u64 lell = a.level_ell[i];
        u32 cs = 0, ch = 0;
        bool pe = false;
#pragma unroll
        for (int k = 0; k < ITEMS + 1; ++k) {
            const u64 c = base + k;
            const bool e = c >= 1 && c < m && ((key[k] ^ key[k + 1]) >> drop) == 0 && (u64)suf[k] + lell < a.n && (u64)suf[k + 1] + lell < a.n;
            if (k >= 1 && c - 1 < m) {
                const bool ka = !pe;
                const bool single = ka && !e;
                cs += single ? 0u : 1u;
                ch += (ka && !single) ? 1u : 0u;
            }
            pe = e;
        }
        const u32 packed = wave_reduce_sum(cs | (ch << 16)); // at most 64 * ITEMS each
        if (lane == 0)
            s_level[w][i] = packed;
    }
    u32 ra = la, rc = lcnt, rh = lheads;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const u32 oa = __shfl_xor(ra, o);
        ra = ra > oa ? ra : oa;
        rc += __shfl_xor(rc, o);
        rh += __shfl_xor(rh, o);
    }
    if (lane == 0) {
        s_wagg[w][0] = ra;
        s_wagg[w][1] = rc;
        s_wagg[w][2] = rh;
    }
    __syncthreads();
    if (t == 0) {
        u32 ta = 0, tc = 0, th = 0;
        for (int ww = 0; ww < WAVES; ++ww) {
            ta = ta > s_wagg[ww][0] ? ta : s_wagg[ww][0];
            tc += s_wagg[ww][1];
            th += s_wagg[ww][2];
        }
        a.tile_agg[(u64)tile * 4 + 0] = ta;
        a.tile_agg[(u64)tile * 4 + 1] = 0;
        a.tile_agg[(u64)tile * 4 + 2] = tc;
        a.tile_agg[(u64)tile * 4 + 3] = th;
        a.tile_splits[tile] = 0;
    }
    if (t < a.levels) {
        u32 sv = 0, hd = 0;
        for (int ww = 0; ww < WAVES; ++ww) {
            sv += s_level[ww][t] & 0xFFFFu;
            hd += s_level[ww][t] >> 16;
        }
        unsigned long long* slot = a.level_totals + (u64)(tile % LEVEL_SLOTS) * 8 + 2 * t;
        if (sv)
            atomicAdd(slot, (unsigned long long)sv);
        if (hd)
            atomicAdd(slot + 1, (unsigned long long)hd);
    }
}

// The applying pass: reads the tile's exclusive prefix from tile_prefix (rerank_count_kernel and rerank_scan_kernel
// before it) and does the work. What the tile produces is collected in LDS and leaves in striped order (consecutive
// lanes, consecutive elements).
template <int BLOCK, int ITEMS>
__global__ __launch_bounds__(BLOCK) void rerank_kernel(RerankArgs a)
{
    constexpr int TILE = BLOCK * ITEMS;
    constexpr int WAVES = BLOCK / WAVE;
    __shared__ u32 s_osuf[TILE];       // survivors of the tile, compacted
    __shared__ u32 s_ogid[TILE];       // their group ids
    __shared__ u32 s_oprim[TILE / 2];  // first rank of each group of the tile
    __shared__ u32 s_ostart[TILE / 2]; // and its start in the active list
    __shared__ u32 s_wagg[WAVES][3];

    const u32 t = threadIdx.x;
    const u32 lane = t & 63u;
    const u32 w = t >> 6;
    const u32 tile = blockIdx.x;
    const u64 tile_base = (u64)tile * TILE;
    const u64 base = tile_base + (u64)t * ITEMS;
    const u32 m = a.m;

    // every thread reads its ITEMS elements (whole 16-byte loads where the tile is full) and their two neighbours
    // straight from the arrays: elements base - 1 .. base + ITEMS
    u64 key[ITEMS + 2];
    u32 suf[ITEMS + 2];
    load_with_neighbours<ITEMS>(a.keys, a.sufs, base, m, key, suf);
    // eq[k]: elements (base+k-1) and (base+k) exist and belong to one run of equal keys
    bool eq[ITEMS + 1];
#pragma unroll
    for (int k = 0; k < ITEMS + 1; ++k) {
        const u64 c = base + k; // right element of the pair
        bool e = c >= 1 && c < m && key[k] == key[k + 1];
        for (int word = 1; e && word < a.key_words; ++word)
            e = load_kgram(a.text, a.n, suf[k], (u32)word) == load_kgram(a.text, a.n, suf[k + 1], (u32)word);
        // a suffix that runs off the text inside its key ties with nobody (include/bit-layout.hpp:99-100)
        if (e && ((u64)suf[k] + a.ell >= a.n || (u64)suf[k + 1] + a.ell >= a.n))
            e = false;
        eq[k] = e;
    }

    // thread-local aggregates; head positions are kept 1-based (c + 1), so that 0 means "no head so far"
    u32 la = 0, lcnt = 0, lheads = 0;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u64 c = base + k;
        if (c < m) {
            const bool ka = !eq[k];
            const bool single = ka && !eq[k + 1];
            if (ka)
                la = (u32)c + 1u;
            lcnt += single ? 0u : 1u;
            lheads += (ka && !single) ? 1u : 0u;
        }
    }

    // block-wide exclusive prefix of (max a, sum cnt, sum heads)
    const u32 ia = wave_incl_max(la), ic = wave_incl_sum(lcnt), ih = wave_incl_sum(lheads);
    if (lane == 63u) {
        s_wagg[w][0] = ia;
        s_wagg[w][1] = ic;
        s_wagg[w][2] = ih;
    }
    __syncthreads();
    u32 xa = __shfl_up(ia, 1), xc = __shfl_up(ic, 1), xh = __shfl_up(ih, 1);
    if (lane == 0)
        xa = xc = xh = 0;
    u32 tile_total_surv = 0, tile_total_heads = 0;
    for (u32 ww = 0; ww < WAVES; ++ww) {
        if (ww < w) {
            xa = xa > s_wagg[ww][0] ? xa : s_wagg[ww][0];
            xc += s_wagg[ww][1];
            xh += s_wagg[ww][2];
        }
        tile_total_surv += s_wagg[ww][1];
        tile_total_heads += s_wagg[ww][2];
    }
    // prefix of the tile = totals of the slabs before its slab, combined with its prefix inside the slab
    u32 pre_a = a.tile_prefix[(u64)tile * 4 + 0];
    u32 tile_rc = a.tile_prefix[(u64)tile * 4 + 2], tile_rh = a.tile_prefix[(u64)tile * 4 + 3];
    const SlabPrefix sp = slabs_before(a.slab_total, tile / a.slab);
    pre_a = pre_a > sp.max0 ? pre_a : sp.max0;
    tile_rc += sp.sum2;
    tile_rh += sp.sum3;
    if (t == 0 && tile_base + TILE >= m) // the last tile knows the totals
        a.gstart_out[tile_rh + tile_total_heads] = tile_rc + tile_total_surv; // gstart[groups] = survivors
    u32 ra = xa > pre_a ? xa : pre_a;
    u32 rc = xc; // tile-local from here on
    u32 rh = xh;
    u64 rec[ITEMS]; // (position << 32 | rank) records of the thread's elements (deferred rank update)
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u64 c = base + k;
        rec[k] = 0;
        if (c < m) {
            const bool ka = !eq[k];
            const bool single = ka && !eq[k + 1];
            if (ka)
                ra = (u32)c + 1u;
            const u32 x = suf[k + 1];
            const u32 nr = ra - 1u; // element 0 is always a head, so ra >= 1 here
            if (ra == 0 || nr >= a.n || x >= a.n) { // a corrupt sorted list: report it instead of writing out of bounds
                atomicExch(a.err, DEV_ERR_RERANK_RANGE);
                continue;
            }
            // runs before this element's own: (groups begun before its run) + (singletons before its run); for a group
            // member at place c with S survivors before it, S - (c - head) of them precede the head
            const u32 begun = tile_rh + rh + ((!single && ka) ? 1u : 0u); // group heads up to and including its own run's
            const u32 ordinal = (single ? begun : begun - 1u) + ((u32)c - (tile_rc + rc));
            const u32 value = a.ordinals ? ordinal : nr;
            if (a.rank_recs)
                rec[k] = ((u64)x << 32) | value;
            else
                a.rank[x] = value;
            if (!single) {
                if (ka) {
                    s_oprim[rh] = nr;
                    s_ostart[rh] = tile_rc + rc;
                    rh++;
                }
                s_osuf[rc] = x;
                s_ogid[rc] = tile_rh + rh - 1;
                rc++;
            }
        }
    }
    // a thread's ITEMS records are neighbours in memory: whole 16-byte stores where the tile is full
    if (a.rank_recs) {
        if (ITEMS % 2 == 0 && tile_base + TILE <= m) {
            uint4* out = reinterpret_cast<uint4*>(a.rank_recs + base); // base is a multiple of ITEMS: 16-byte aligned
#pragma unroll
            for (int k = 0; k < ITEMS; k += 2)
                out[k / 2] = make_uint4((u32)rec[k], (u32)(rec[k] >> 32), (u32)rec[k + 1], (u32)(rec[k + 1] >> 32));
        } else {
#pragma unroll
            for (int k = 0; k < ITEMS; ++k)
                if (base + k < m)
                    a.rank_recs[base + k] = rec[k];
        }
    }
    __syncthreads();
    // striped write-out of what the tile produced
    const u32 n_surv = tile_total_surv, n_heads = tile_total_heads;
    for (u32 i = t; i < n_surv; i += BLOCK) {
        a.sufs_out[tile_rc + i] = s_osuf[i];
        a.gids_out[tile_rc + i] = s_ogid[i];
    }
    for (u32 i = t; i < n_heads; i += BLOCK) {
        a.gprim_out[tile_rh + i] = s_oprim[i];
        a.gstart_out[tile_rh + i] = s_ostart[i];
    }
}

// Exclusive combination of the tile aggregates (max, max, sum, sum) over the tiles of one slab: workgroup s handles
// tiles [s * slab, (s + 1) * slab) and writes each tile's prefix relative to the slab start plus the slab's total.
// The applying pass adds the totals of the slabs before its own (at most RERANK_SLABS of them).

__global__ __launch_bounds__(1024) void rerank_scan_kernel(const u32* __restrict__ tile_agg, u32* __restrict__ tile_prefix,
                                                           u32 tiles, u32 slab, u32* __restrict__ slab_total,
                                                           const u32* __restrict__ tile_splits)
{
    __shared__ u32 s_w[16][4];
    __shared__ u32 s_sp[16];
    const u32 t = threadIdx.x, lane = t & 63u, w = t >> 6;
    const u32 slab_first = blockIdx.x * slab;
    const u32 slab_last = slab_first + slab < tiles ? slab_first + slab : tiles;
    const u32 per = (slab + 1023) / 1024;
    const u32 first = slab_first + t * per < slab_last ? slab_first + t * per : slab_last;
    const u32 last = first + per < slab_last ? first + per : slab_last;
    const uint4* agg4 = reinterpret_cast<const uint4*>(tile_agg);
    uint4* pre4 = reinterpret_cast<uint4*>(tile_prefix);
    u32 ra = 0, rb = 0, rc = 0, rh = 0, sp = 0;
    for (u32 i = first; i < last; ++i) {
        const uint4 v = agg4[i];
        ra = ra > v.x ? ra : v.x;
        rb = rb > v.y ? rb : v.y;
        rc += v.z;
        rh += v.w;
    }
    const u32 ia = wave_incl_max(ra), ib = wave_incl_max(rb), ic = wave_incl_sum(rc), ih = wave_incl_sum(rh);
    if (lane == 63u) {
        s_w[w][0] = ia;
        s_w[w][1] = ib;
        s_w[w][2] = ic;
        s_w[w][3] = ih;
    }
    __syncthreads();
    u32 xa = __shfl_up(ia, 1), xb = __shfl_up(ib, 1), xc = __shfl_up(ic, 1), xh = __shfl_up(ih, 1);
    if (lane == 0)
        xa = xb = xc = xh = 0;
    u32 ta = 0, tb = 0, tc = 0, th = 0;
    for (u32 ww = 0; ww < 16; ++ww) {
        if (ww < w) {
            xa = xa > s_w[ww][0] ? xa : s_w[ww][0];
            xb = xb > s_w[ww][1] ? xb : s_w[ww][1];
            xc += s_w[ww][2];
            xh += s_w[ww][3];
        }
        ta = ta > s_w[ww][0] ? ta : s_w[ww][0];
        tb = tb > s_w[ww][1] ? tb : s_w[ww][1];
        tc += s_w[ww][2];
        th += s_w[ww][3];
    }
    for (u32 i = first; i < last; ++i) {
        const uint4 v = agg4[i];
        pre4[i] = make_uint4(xa, xb, xc, xh);
        // changed ranks of the tile; its undecided elements change if the slab so far ends inside a split group
        // (what the slabs before left open is ignored: the sum only steers a choice between two correct paths)
        const u32 packed = tile_splits[i];
        sp += (packed & 0xFFFFu) + (xa > xb ? packed >> 16 : 0u);
        xa = xa > v.x ? xa : v.x;
        xb = xb > v.y ? xb : v.y;
        xc += v.z;
        xh += v.w;
    }
    const u32 wsp = wave_reduce_sum(sp);
    if (lane == 0)
        s_sp[w] = wsp;
    __syncthreads();
    if (t == 0) {
        u32 tsp = 0;
        for (u32 ww = 0; ww < 16; ++ww)
            tsp += s_sp[ww];
        slab_total[blockIdx.x * 5 + 0] = ta;
        slab_total[blockIdx.x * 5 + 1] = tb;
        slab_total[blockIdx.x * 5 + 2] = tc;
        slab_total[blockIdx.x * 5 + 3] = th;
        slab_total[blockIdx.x * 5 + 4] = tsp;
    }
}

// Last step of the deferred rank update. The (text position << 32 | rank) records of generation 0 arrive sorted by
// the high bits of the position; the positions are a permutation of [0, n), so the records of window w (positions
// [w * S, (w + 1) * S), S = 1 << window_log2) are exactly records [w * S, (w + 1) * S) of the list. One workgroup
// per window scatters the ranks into an LDS image of the window and writes the image out in full lines.
template <int MAX_LOG2>
__global__ __launch_bounds__(1024) void place_ranks_kernel(const u64* __restrict__ recs, u32 n, int window_log2,
                                                           u32* __restrict__ rank)
{
    __shared__ u32 s_win[1 << MAX_LOG2];
    const u32 S = 1u << window_log2;
    const u64 first = (u64)blockIdx.x << window_log2;
    const u32 count = (u32)((u64)n - first < S ? (u64)n - first : S);
    for (u32 i = threadIdx.x; i < count; i += 1024) {
        const u64 r = recs[first + i];
        const u32 off = (u32)(r >> 32) - (u32)first;
        if (off < count) // always, for a permutation sorted by window
            s_win[off] = (u32)r;
    }
    __syncthreads();
    for (u32 i = threadIdx.x; i < count; i += 1024)
        rank[first + i] = s_win[i];
}

// Bucketed rank update of a later generation. The changed ranks of a generation are few or many: when they are
// many, the (text position, rank) pairs of the whole sorted list go through ONE radix pass on the position bits
// above the window size, after which consecutive workgroups scatter into one window of rank[] at a time. Random
// 4-byte writes into a window that the last-level cache holds (here 128 MB) run about four times faster than
// writes spread over a multi-GB array.
constexpr int POS_BINS = 256; // digits of the one bucket pass are at most 8 bits wide

__global__ __launch_bounds__(256) void position_hist_kernel(const u32* __restrict__ pos, u32 m, int shift, int bits,
                                                            u32* ghist)
{
    __shared__ u32 s_hist[POS_BINS * 8];
    for (int i = threadIdx.x; i < POS_BINS * 8; i += 256)
        s_hist[i] = 0;
    __syncthreads();
    const u32 copy = threadIdx.x & 7u;
    const u32 mask = (1u << bits) - 1u;
    // four positions per thread and round (one 16-byte load where they all exist: the lists are 16-byte aligned)
    const u64 stride = (u64)gridDim.x * 256 * 4;
    for (u64 i = ((u64)blockIdx.x * 256 + threadIdx.x) * 4; i < m; i += stride) {
        u32 x[4];
        const int have = m - i < 4 ? (int)(m - i) : 4;
        if (have == 4 && (reinterpret_cast<uintptr_t>(pos) & 15u) == 0) {
            const uint4 v = *reinterpret_cast<const uint4*>(pos + i);
            x[0] = v.x, x[1] = v.y, x[2] = v.z, x[3] = v.w;
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k)
                x[k] = k < have ? pos[i + k] : 0u;
        }
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (k < have)
                atomicAdd(&s_hist[((x[k] >> shift) & mask) * 8 + copy], 1u);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < POS_BINS; i += 256) {
        u32 v = 0;
#pragma unroll
        for (int c = 0; c < 8; ++c)
            v += s_hist[i * 8 + c];
        if (v)
            atomicAdd(&ghist[i], v);
    }
}

__global__ __launch_bounds__(256) void scatter_ranks_kernel(const u32* __restrict__ pos, const u32* __restrict__ val, u32 m,
                                                            u32 n, u32* __restrict__ rank, u32* err)
{
    const u64 i0 = ((u64)blockIdx.x * 256 + threadIdx.x) * 4;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const u64 i = i0 + k;
        if (i < m) {
            const u32 v = val[i];
            if (v != NO_RANK) {
                const u32 x = pos[i];
                if (x < n && v < n)
                    rank[x] = v;
                else
                    atomicExch(err, DEV_ERR_RERANK_RANGE);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Generation t >= 1: gather rank[x + h], and sort inside every small group in the same pass.
//
// The active list is grouped (members of a group are contiguous, group g = [gstart[g], gstart[g + 1])).
// A tile stages the gathered ranks of its elements plus a halo of MAXG elements on either side in LDS. For a group
// of at most MAXG members, each member then derives from its group, all by itself:
//   its place in the sorted group   = members with a smaller rank[x + h], ties kept in list order;
//   its refined rank                = gprim[g] + members with a smaller rank[x + h]
//                                     (reference: include/GPU_SACA.cuh:277, new = old + key-run head - group head);
// and writes (suffix, refined rank) to its place of the sorted list. Equal refined ranks are equal keys: a group owns
// the rank range [gprim, gprim + size), so ranks of different groups cannot meet. No key is written at all.
// Members of larger groups go, in list order, to a list of (key, suffix) pairs that goes through the radix sort
// instead (place_big_kernel brings them back in the same (suffix, refined rank) form). List order matters: the sort
// is stable, so members that tie keep the order they had, here as in the small groups; a list whose large groups are
// in order of rank[x + h] already (place_presorted_kernel) stays recognisable as such generation after generation.
// Replaces, for small groups, the 62-bit key sort of the reference (src/GPU_SACA.cu:1841-1871).
//
// COUNT instantiation (lists known to hold small groups only): the kernel also adds, to the tile of the sorted list
// that each member lands in, the survivor / new-group / changed-rank counts the apply step needs, so that no
// counting pass over the sorted list runs at all.
// ---------------------------------------------------------------------------------------------

struct SmallSortArgs {
    const u32* sufs;   // active list
    const u32* gids;
    const u32* gstart; // [groups + 1]
    const u32* gprim;  // [groups] first rank of each group
    const u32* rank;
    u32 m, n, h;
    u32 groups;
    int sec_bits;
    u32* err; // set to a DEV_ERR_* code if an invariant of the group tables is violated
    u32* sufs_out; // sorted active list: suffix ...
    u32* nr_out;   // ... and its refined rank, bit 31 set if it differs from the old rank
    u64* big_keys; // elements of groups larger than MAXG: (group id << sec_bits) | rank[x + h], in list order:
    u32* big_sufs; // the member at list place e of large group g goes to big_first[g] + (e - gstart[g])
    u32 side_list; // 0: the two arrays above are not written (the caller expects every large group to be in order already, as
                   //    in the generation before, and runs the kernel again if the marks say otherwise)
    const u32* big_first; // [groups]: members of large groups before group g (big_prefix_kernel)
    u32* tile_agg;    // COUNT: [tiles][4], zero before the launch: [2] survivors, [3] new groups per tile of the sorted list
    u32* tile_splits; // COUNT: [tiles], zero before the launch: changed ranks
    // !COUNT: is the list already in order inside its large groups? The gathered rank of every member of a large group
    // is kept at its list place in big_sec, and a large group in which some member's gathered rank is below (above) its
    // predecessor's gets its size written to not_asc (not_desc) at the group's mark index, big_first[g] / MAXG: a large
    // group has more than MAXG members, so no two share an index, and m / MAXG + 2 entries cover every list. Both zero
    // before the launch.
    u32* big_sec;
    u32* not_asc;
    u32* not_desc;
};

template <int BLOCK, int ITEMS, int MAXG, bool COUNT>
__global__ __launch_bounds__(BLOCK) void smallsort_kernel(SmallSortArgs a)
{
    constexpr int TILE = BLOCK * ITEMS;
    constexpr int SPAN = TILE + 2 * MAXG;
    __shared__ u32 s_sec[SPAN];

    const u32 t = threadIdx.x;
    const long long t0 = (long long)blockIdx.x * TILE;
    const long long lo = t0 - MAXG; // list index of s_sec[0]

    u32 x[ITEMS], sec[ITEMS];
    // own elements (striped: consecutive lanes hold consecutive elements) and the two halos
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const long long e = t0 + k * BLOCK + t;
        x[k] = 0;
        sec[k] = 0;
        if (e < (long long)a.m) {
            x[k] = a.sufs[e];
            const u64 src = (u64)x[k] + a.h;
            sec[k] = src < a.n ? a.rank[src] : 0u;
            s_sec[MAXG + k * BLOCK + t] = sec[k];
        }
    }
    // A halo element matters only if its group reaches into the tile, i.e. if it shares the group of the tile's
    // first (left halo) or last (right halo) element; the others would be random reads for nothing.
    // A member of a large group needs no other member's rank, except the one before it in the list (is the group in
    // order already?): of a large group at the tile's border only that one element of the halo is read.
    const long long last_own = t0 + TILE - 1 < (long long)a.m - 1 ? t0 + TILE - 1 : (long long)a.m - 1;
    const u32 gid_first = a.gids[t0], gid_last = a.gids[last_own];
    bool first_small = true, last_small = true;
    if (gid_first < a.groups && gid_last < a.groups) { // (checked again, and reported, below)
        first_small = a.gstart[gid_first + 1] - a.gstart[gid_first] <= (u32)MAXG;
        last_small = a.gstart[gid_last + 1] - a.gstart[gid_last] <= (u32)MAXG;
    }
    for (int i = t; i < 2 * MAXG; i += BLOCK) {
        const int slot = i < MAXG ? i : TILE + i; // [0, MAXG) and [MAXG + TILE, SPAN)
        const long long e = lo + slot;
        const bool wanted = i < MAXG ? (first_small || (!COUNT && i == MAXG - 1)) : last_small;
        if (wanted && e >= 0 && e < (long long)a.m && a.gids[e] == (i < MAXG ? gid_first : gid_last)) {
            const u64 src = (u64)a.sufs[e] + a.h;
            s_sec[slot] = src < a.n ? a.rank[src] : 0u;
        }
    }
    __syncthreads();

    // group of every own element; members of large groups are counted so that the block reserves their slots in
    // the large-group list with ONE atomic (one atomic per wave on a single counter serialises the whole launch
    // when most of the list is in large groups)
    u32 g[ITEMS], gs[ITEMS], ge[ITEMS];
    u32 kind = 0; // 2 bits per item: 0 = not mine, 1 = small group, 2 = large group
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const long long e = t0 + k * BLOCK + t;
        g[k] = gs[k] = ge[k] = 0;
        if (e < (long long)a.m) {
            g[k] = a.gids[e];
            bool ok = g[k] < a.groups;
            if (ok) {
                gs[k] = a.gstart[g[k]];
                ge[k] = a.gstart[g[k] + 1];
                ok = (long long)gs[k] <= e && e < (long long)ge[k] && ge[k] <= a.m;
            }
            if (!ok) {
                atomicExch(a.err, DEV_ERR_SMALLSORT_TABLES); // the element is not inside its group's range
            } else if (ge[k] - gs[k] > (u32)MAXG) {
                kind |= 2u << (2 * k);
            } else {
                kind |= 1u << (2 * k);
            }
        }
    }
    const u32 lane = t & 63u;

    // COUNT: survivors, new groups, changed ranks bound for the own tile (registers) or, for a group that straddles
    // a tile border, for the tile before / after (LDS)
    __shared__ u32 s_nb[2][3];
    __shared__ u32 s_own[3];
    if constexpr (COUNT) {
        if (t < 6)
            (&s_nb[0][0])[t] = 0;
        if (t < 3)
            s_own[t] = 0;
        __syncthreads();
    }
    u32 c_surv = 0, c_head = 0, c_chg = 0;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const long long e = t0 + k * BLOCK + t;
        const u32 what = (kind >> (2 * k)) & 3u;
        if (what == 2u) {
            if constexpr (COUNT) {
                atomicExch(a.err, DEV_ERR_UNEXPECTED_LARGE_GROUP); // groups only split: cannot happen after an all-small list
            } else {
                const u32 first = a.big_first[g[k]];
                const u32 slot = first + ((u32)e - gs[k]);
                if (a.side_list) {
                    a.big_keys[slot] = ((u64)g[k] << a.sec_bits) | (u64)sec[k];
                    a.big_sufs[slot] = x[k];
                }
                a.big_sec[e] = sec[k];
                if (e > (long long)gs[k]) { // the member before it in the list belongs to the same group
                    const u32 before = s_sec[MAXG + (e - 1 - t0)]; // an own element, or the last one of the left halo
                    const u32 mark = first / (u32)MAXG;
                    // (plain stores of one value by whoever sees it first: no atomics, and soon only cached reads)
                    if (before > sec[k] && a.not_asc[mark] == 0)
                        a.not_asc[mark] = ge[k] - gs[k];
                    if (before < sec[k] && a.not_desc[mark] == 0)
                        a.not_desc[mark] = ge[k] - gs[k];
                }
            }
            continue;
        }
        if (what != 1u)
            continue;
        u32 less = 0, eq_before = 0, eq_after = 0;
        for (u32 j = gs[k]; j < ge[k]; ++j) {
            const u32 v = s_sec[(long long)j - lo];
            less += v < sec[k] ? 1u : 0u;
            if (v == sec[k]) {
                eq_before += (long long)j < e ? 1u : 0u;
                eq_after += (long long)j > e ? 1u : 0u;
            }
        }
        const u32 pos = gs[k] + less + eq_before;
        const u32 nr = a.gprim[g[k]] + less;
        if (nr >= a.n || x[k] >= a.n) {
            atomicExch(a.err, DEV_ERR_RERANK_RANGE);
            continue;
        }
        a.sufs_out[pos] = x[k];
        a.nr_out[pos] = nr | (less ? 0x80000000u : 0u);
        if constexpr (COUNT) {
            const bool single = eq_before + eq_after == 0;
            const u32 surv = single ? 0u : 1u, head = (!single && eq_before == 0) ? 1u : 0u, chg = less ? 1u : 0u;
            const long long dest_tile = (long long)pos / TILE;
            if (dest_tile == (long long)blockIdx.x) {
                c_surv += surv;
                c_head += head;
                c_chg += chg;
            } else {
                const int side = dest_tile < (long long)blockIdx.x ? 0 : 1;
                if (surv)
                    atomicAdd(&s_nb[side][0], 1u);
                if (head)
                    atomicAdd(&s_nb[side][1], 1u);
                if (chg)
                    atomicAdd(&s_nb[side][2], 1u);
            }
        }
    }
    if constexpr (COUNT) {
        // per wave at most 64 * ITEMS of each: three 10-bit fields travel in one reduction
        static_assert(64 * ITEMS < 1024, "three counts are packed into one 32-bit word");
        const u32 packed = wave_reduce_sum(c_surv | (c_head << 10) | (c_chg << 20));
        if (lane == 0) {
            atomicAdd(&s_own[0], packed & 1023u);
            atomicAdd(&s_own[1], (packed >> 10) & 1023u);
            atomicAdd(&s_own[2], packed >> 20);
        }
        __syncthreads();
        if (t < 9) {
            const u32 which = t / 3, field = t % 3; // 0: own tile, 1: the tile before, 2: the tile after
            const u32 v = which == 0 ? s_own[field] : s_nb[which - 1][field];
            const long long tile = (long long)blockIdx.x + (which == 0 ? 0 : (which == 1 ? -1 : 1));
            if (v && tile >= 0 && tile < (long long)gridDim.x)
                atomicAdd(field < 2 ? &a.tile_agg[tile * 4 + 2 + field] : &a.tile_splits[tile], v);
        }
    }
}

// Counts of the sorted list (suffix, refined rank) per tile, for generations in which large groups came back through
// the radix sort: survivors (members whose rank is shared), new groups, changed ranks. Reads 4 bytes per member.
template <int BLOCK, int ITEMS>
__global__ __launch_bounds__(BLOCK) void count_ranks_kernel(const u32* __restrict__ nr, u32 m, u32* __restrict__ tile_agg,
                                                            u32* __restrict__ tile_splits)
{
    constexpr int TILE = BLOCK * ITEMS;
    constexpr int WAVES = BLOCK / WAVE;
    __shared__ u32 s_w[WAVES];
    const u32 t = threadIdx.x;
    // blocked: thread t owns places base .. base + ITEMS - 1 and reads them, with the two places next to them, straight
    // from the list (whole 16-byte loads where they all exist)
    const u64 base = (u64)blockIdx.x * TILE + (u64)t * ITEMS;
    u32 nrw[ITEMS + 2]; // places base - 1 .. base + ITEMS
    if (ITEMS % 4 == 0 && base + ITEMS <= m) {
        const uint4* n4 = reinterpret_cast<const uint4*>(nr + base); // base is a multiple of ITEMS
#pragma unroll
        for (int k = 0; k < ITEMS; k += 4) {
            const uint4 v = n4[k / 4];
            nrw[k + 1] = v.x;
            nrw[k + 2] = v.y;
            nrw[k + 3] = v.z;
            nrw[k + 4] = v.w;
        }
        nrw[0] = base >= 1 ? nr[base - 1] : 0u;
        nrw[ITEMS + 1] = base + ITEMS < m ? nr[base + ITEMS] : 0u;
    } else {
#pragma unroll
        for (int k = 0; k < ITEMS + 2; ++k) {
            const u64 c = base + k; // place c - 1
            nrw[k] = (c >= 1 && c - 1 < m) ? nr[c - 1] : 0u;
        }
    }
    u32 c_surv = 0, c_head = 0, c_chg = 0;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u64 c = base + k;
        if (c < m) {
            const u32 word = nrw[k + 1], me = word & 0x7FFFFFFFu;
            const bool head = c == 0 || (nrw[k] & 0x7FFFFFFFu) != me;
            const bool last = c + 1 == m || (nrw[k + 2] & 0x7FFFFFFFu) != me;
            const bool surv = !(head && last);
            c_surv += surv ? 1u : 0u;
            c_head += (head && surv) ? 1u : 0u;
            c_chg += word >> 31;
        }
    }
    static_assert(64 * ITEMS < 1024, "three counts are packed into one 32-bit word");
    const u32 packed = wave_reduce_sum(c_surv | (c_head << 10) | (c_chg << 20));
    if ((t & 63u) == 0)
        s_w[t >> 6] = packed;
    __syncthreads();
    if (t == 0) {
        u32 sv = 0, hd = 0, ch = 0;
        for (int ww = 0; ww < WAVES; ++ww) {
            sv += s_w[ww] & 1023u;
            hd += (s_w[ww] >> 10) & 1023u;
            ch += s_w[ww] >> 20;
        }
        tile_agg[(u64)blockIdx.x * 4 + 0] = 0;
        tile_agg[(u64)blockIdx.x * 4 + 1] = 0;
        tile_agg[(u64)blockIdx.x * 4 + 2] = sv;
        tile_agg[(u64)blockIdx.x * 4 + 3] = hd;
        tile_splits[blockIdx.x] = ch;
    }
}

// Second half of a generation t >= 1: the sorted list carries, at every place, the suffix and its refined rank.
// Equal ranks are equal keys, so run heads, singletons and new groups follow from neighbour comparison of the
// ranks: a singleton retires to its final place in the suffix array, the others are compacted, in order, into the
// next active list (reference: cub::DevicePartition::Flagged, src/GPU_SACA.cu:1917-1925) with the tile prefixes of
// rerank_scan_kernel, each with the dense id of its new group; changed ranks are written to rank[] (or handed to
// the bucketed update). Tiles must be those the counts were attributed to (TILE = the small-group kernel's).
struct ApplySmallArgs {
    const u32* sufs;
    const u32* nr; // bit 31: the rank changed
    u32 m, n;
    u32* rank;
    u32* rank_vals; // null: write rank[x] directly; else the rank of list place c goes to rank_vals[c] (NO_RANK where unchanged)
    u32* sa32;      // suffix array under construction
    u32* sufs_out;
    u32* gids_out;
    u32* gprim_out;
    u32* gstart_out;
    const u32* tile_prefix; // [tiles][4]
    const u32* slab_total;  // [RERANK_SLABS][5]
    u32 slab;
    u32* err;
};

template <int BLOCK, int ITEMS>
__global__ __launch_bounds__(BLOCK) void apply_small_kernel(ApplySmallArgs a)
{
    constexpr int TILE = BLOCK * ITEMS;
    constexpr int WAVES = BLOCK / WAVE;
    __shared__ u32 s_w[WAVES][2];
    __shared__ u32 s_suf[TILE], s_gid[TILE], s_head_rank[TILE], s_head_start[TILE];
    const u32 t = threadIdx.x, lane = t & 63u, w = t >> 6;
    const u32 tile = blockIdx.x;
    const u64 tile_base = (u64)tile * TILE;
    const u32 m = a.m;
    // blocked: thread t owns places tile_base + t * ITEMS + k and reads them, with the refined ranks of the two places
    // next to them, straight from the lists (whole 16-byte loads where the tile is full)
    const u64 base = tile_base + (u64)t * ITEMS;
    u32 nrw[ITEMS + 2]; // places base - 1 .. base + ITEMS
    u32 xs[ITEMS];
    if (ITEMS % 4 == 0 && base + ITEMS <= m) {
        const uint4* n4 = reinterpret_cast<const uint4*>(a.nr + base); // base is a multiple of ITEMS
        const uint4* x4 = reinterpret_cast<const uint4*>(a.sufs + base);
#pragma unroll
        for (int k = 0; k < ITEMS; k += 4) {
            const uint4 v = n4[k / 4], xv = x4[k / 4];
            nrw[k + 1] = v.x;
            nrw[k + 2] = v.y;
            nrw[k + 3] = v.z;
            nrw[k + 4] = v.w;
            xs[k] = xv.x;
            xs[k + 1] = xv.y;
            xs[k + 2] = xv.z;
            xs[k + 3] = xv.w;
        }
        nrw[0] = base >= 1 ? a.nr[base - 1] : 0u;
        nrw[ITEMS + 1] = base + ITEMS < m ? a.nr[base + ITEMS] : 0u;
    } else {
#pragma unroll
        for (int k = 0; k < ITEMS + 2; ++k) {
            const u64 c = base + k; // place c - 1
            nrw[k] = (c >= 1 && c - 1 < m) ? a.nr[c - 1] : 0u;
        }
#pragma unroll
        for (int k = 0; k < ITEMS; ++k)
            xs[k] = base + k < m ? a.sufs[base + k] : 0u;
    }
    u32 flags = 0; // 2 bits per item: bit 0 survivor, bit 1 head of a new group
    u32 lsurv = 0, lhead = 0;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u64 c = base + k;
        if (c < m) {
            const u32 me = nrw[k + 1] & 0x7FFFFFFFu;
            const bool head = c == 0 || (nrw[k] & 0x7FFFFFFFu) != me;
            const bool last = c + 1 == m || (nrw[k + 2] & 0x7FFFFFFFu) != me;
            const bool surv = !(head && last);
            flags |= (surv ? 1u : 0u) << (2 * k);
            flags |= ((head && surv) ? 2u : 0u) << (2 * k);
            lsurv += surv ? 1u : 0u;
            lhead += (head && surv) ? 1u : 0u;
        }
    }
    const u32 is = wave_incl_sum(lsurv), ih = wave_incl_sum(lhead);
    if (lane == 63u) {
        s_w[w][0] = is;
        s_w[w][1] = ih;
    }
    __syncthreads();
    u32 rc = is - lsurv, rh = ih - lhead; // exclusive inside the tile
    u32 tot_s = 0, tot_h = 0;
    for (u32 ww = 0; ww < WAVES; ++ww) {
        if (ww < w) {
            rc += s_w[ww][0];
            rh += s_w[ww][1];
        }
        tot_s += s_w[ww][0];
        tot_h += s_w[ww][1];
    }
    u32 tile_rc = a.tile_prefix[(u64)tile * 4 + 2], tile_rh = a.tile_prefix[(u64)tile * 4 + 3];
    const SlabPrefix sp = slabs_before(a.slab_total, tile / a.slab);
    tile_rc += sp.sum2;
    tile_rh += sp.sum3;
    if (t == 0 && tile_base + TILE >= m)
        a.gstart_out[tile_rh + tot_h] = tile_rc + tot_s; // gstart[groups] = survivors
    // The survivors of a tile and its new groups land in one contiguous stretch each of the next list and of the next
    // group table: they are compacted in LDS first, so that the stores below go out lane after lane (a thread owns
    // ITEMS consecutive places, and its own stores would each touch a line that three more stores touch again).
    const bool full = ITEMS % 4 == 0 && base + ITEMS <= m;
    u32 rv[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u64 c = base + k;
        rv[k] = NO_RANK;
        if (c >= m)
            continue;
        const u32 word = nrw[k + 1], nr = word & 0x7FFFFFFFu, x = xs[k];
        const u32 f = (flags >> (2 * k)) & 3u;
        if (nr >= a.n || x >= a.n) {
            atomicExch(a.err, DEV_ERR_RERANK_RANGE);
            // (a survivor still takes its slot below, so that every slot of the stretch is written: with a value in range)
            if (f & 2u) {
                s_head_rank[rh] = 0;
                s_head_start[rh] = rc;
                rh++;
            }
            if (f & 1u) {
                s_suf[rc] = 0;
                s_gid[rc] = rh - 1;
                rc++;
            }
            continue;
        }
        if (a.rank_vals)
            rv[k] = (word >> 31) ? nr : NO_RANK;
        else if (word >> 31)
            a.rank[x] = nr;
        if (!(f & 1u))
            a.sa32[nr] = x; // alone with its key: the rank is final
        if (f & 2u) {
            s_head_rank[rh] = nr;
            s_head_start[rh] = rc;
            rh++;
        }
        if (f & 1u) {
            s_suf[rc] = x;
            s_gid[rc] = rh - 1; // (-1 wraps for members of a group that began in an earlier tile: added to tile_rh below)
            rc++;
        }
    }
    if (a.rank_vals) {
        if (full && (reinterpret_cast<uintptr_t>(a.rank_vals) & 15u) == 0) {
            uint4* out4 = reinterpret_cast<uint4*>(a.rank_vals + base);
#pragma unroll
            for (int k = 0; k < ITEMS; k += 4)
                out4[k / 4] = make_uint4(rv[k], rv[k + 1], rv[k + 2], rv[k + 3]);
        } else {
#pragma unroll
            for (int k = 0; k < ITEMS; ++k)
                if (base + k < m)
                    a.rank_vals[base + k] = rv[k];
        }
    }
    __syncthreads();
    for (u32 i = t; i < tot_s; i += BLOCK) {
        a.sufs_out[tile_rc + i] = s_suf[i];
        a.gids_out[tile_rc + i] = tile_rh + s_gid[i];
    }
    for (u32 i = t; i < tot_h; i += BLOCK) {
        a.gprim_out[tile_rh + i] = s_head_rank[i];
        a.gstart_out[tile_rh + i] = tile_rc + s_head_start[i];
    }
}

// big_first[g] = members of groups larger than maxg among the groups before g, the place of g's first member in the list
// of large-group members; *total = that count over all groups. From the group table alone (4 bytes per group), in the
// three launches of the rank step: per-tile sums, rerank_scan_kernel, the pass that writes the prefixes.
template <bool APPLY>
__global__ __launch_bounds__(256) void big_prefix_kernel(const u32* __restrict__ gstart, u32 groups, u32 maxg, u32* __restrict__ big_first,
                                                         u32* __restrict__ tile_agg, u32* __restrict__ tile_splits,
                                                         const u32* __restrict__ tile_prefix, const u32* __restrict__ slab_total, u32 slab,
                                                         u32 slabs, u32* __restrict__ total)
{
    constexpr int ITEMS = 4, TILE = 256 * ITEMS, WAVES = 256 / WAVE;
    __shared__ u32 s_w[WAVES];
    const u32 t = threadIdx.x, lane = t & 63u, w = t >> 6;
    const u32 tile = blockIdx.x;
    const u64 base = (u64)tile * TILE + (u64)t * ITEMS;
    u32 size[ITEMS], mine = 0;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u64 g = base + k;
        size[k] = 0;
        if (g < groups) {
            const u32 sz = gstart[g + 1] - gstart[g];
            size[k] = sz > maxg ? sz : 0u;
        }
        mine += size[k];
    }
    const u32 incl = wave_incl_sum(mine);
    if (lane == 63u)
        s_w[w] = incl;
    __syncthreads();
    u32 before = incl - mine, tile_total = 0;
    for (u32 ww = 0; ww < WAVES; ++ww) {
        if (ww < w)
            before += s_w[ww];
        tile_total += s_w[ww];
    }
    if (!APPLY) {
        if (t == 0) {
            tile_agg[(u64)tile * 4 + 0] = 0;
            tile_agg[(u64)tile * 4 + 1] = 0;
            tile_agg[(u64)tile * 4 + 2] = tile_total;
            tile_agg[(u64)tile * 4 + 3] = 0;
            tile_splits[tile] = 0;
        }
        return;
    }
    before += tile_prefix[(u64)tile * 4 + 2] + slabs_before(slab_total, tile / slab).sum2;
    const u32 all = slabs_before(slab_total, slabs).sum2;
    if (tile == 0 && t == 0)
        *total = all;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u64 g = base + k;
        if (g < groups)
            big_first[g] = before;
        before += size[k];
    }
}

// Members of large groups whose gathered ranks are out of order: the sizes of the large groups that carry both marks
// (`marks` entries of the two mark arrays of the small-group kernel). Zero means every large group of the list is in
// non-decreasing or in non-increasing order of rank[x + h] as it stands, and none of them needs the radix sort.
__global__ __launch_bounds__(256) void group_order_kernel(const u32* __restrict__ not_asc, const u32* __restrict__ not_desc, u32 marks,
                                                          u32* __restrict__ unordered)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    u32 mine = (i < marks && not_asc[i] && not_desc[i]) ? not_asc[i] : 0u;
    mine = wave_reduce_sum(mine);
    if ((threadIdx.x & 63u) == 0 && mine)
        atomicAdd(unordered, mine);
}

// The large groups of a list in which every one of them is in order already (group_order_kernel counted nothing):
// no sort. Place p of a large group g takes the member at list place p if the group's gathered ranks do not decrease
// along the list, and the member at the mirrored place gstart[g] + gstart[g + 1] - 1 - p if they do not increase (a
// token run followed by a smaller symbol: the deeper into the run, the smaller); its refined rank is gprim[g] + (head
// of its run of equal gathered ranks - gstart[g]), the heads being a running maximum over the places, found in the
// three launches of the rank step (per-tile maxima, rerank_scan_kernel, apply). Members that tie keep whatever mutual
// order this leaves them in: they share a rank, and the next generation sorts them by what it gathers.
// Replaces, for such lists, the sort of the reference's 62-bit keys (src/GPU_SACA.cu:1841-1871).
struct PresortedArgs {
    const u32* sufs; // the active list ...
    const u32* gids; // ... its groups ...
    const u32* big_sec; // ... and, at the places of large groups, the gathered ranks
    const u32* gstart;
    const u32* gprim;
    const u32* big_first; // members of large groups before each group: big_first[g] / maxg is the group's mark index
    const u32* not_asc;   // set at the mark index where the group's gathered ranks decrease somewhere (then they never increase)
    u32 m, n, groups, maxg;
    u32* sufs_out;
    u32* nr_out;
    u32* tile_agg;    // [tiles][4]: [0] last run head of the tile, as place + 1 (0: none)
    u32* tile_splits; // [tiles]: zeroed for the scan
    const u32* tile_prefix;
    const u32* slab_total;
    u32 slab;
    u32* err;
};

template <int BLOCK, int ITEMS, bool APPLY>
__global__ __launch_bounds__(BLOCK) void place_presorted_kernel(PresortedArgs a)
{
    constexpr int TILE = BLOCK * ITEMS;
    constexpr int WAVES = BLOCK / WAVE;
    __shared__ u32 s_wagg[WAVES];
    const u32 t = threadIdx.x, lane = t & 63u, w = t >> 6;
    const u32 tile = blockIdx.x;
    const u64 base = (u64)tile * TILE + (u64)t * ITEMS;
    u32 g[ITEMS], gs[ITEMS], src[ITEMS], sec[ITEMS];
    u32 big = 0, heads = 0; // one bit per item
    u32 lh = 0;             // last run head among this thread's places, as place + 1
    // The loads of a thread's places are issued in rounds (group ids, then the groups' tables, then the gathered ranks)
    // rather than place after place: the four chains of dependent loads run side by side.
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u64 p = base + k;
        gs[k] = src[k] = sec[k] = 0;
        g[k] = p < a.m ? a.gids[p] : 0xFFFFFFFFu;
    }
    // neighbouring places mostly lie in one group: its tables are looked up once per thread, not once per place
    u32 ge[ITEMS];
    bool mirrored[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u64 p = base + k;
        ge[k] = 0;
        mirrored[k] = false;
        if (p >= a.m)
            continue;
        if (g[k] >= a.groups) {
            atomicExch(a.err, DEV_ERR_SMALLSORT_TABLES);
            continue;
        }
        const bool same_group = k > 0 && (big & (1u << (k - 1))) && g[k - 1] == g[k];
        gs[k] = same_group ? gs[k - 1] : a.gstart[g[k]];
        ge[k] = same_group ? ge[k - 1] : a.gstart[g[k] + 1];
        if (!(gs[k] <= p && p < ge[k] && ge[k] <= a.m)) {
            atomicExch(a.err, DEV_ERR_SMALLSORT_TABLES);
            continue;
        }
        if (ge[k] - gs[k] <= a.maxg)
            continue; // a small group: the small-group kernel has placed it
        big |= 1u << k;
        mirrored[k] = same_group ? mirrored[k - 1] : a.not_asc[a.big_first[g[k]] / a.maxg] != 0;
        src[k] = mirrored[k] ? gs[k] + (ge[k] - 1u - (u32)p) : (u32)p;
    }
#pragma unroll
    for (int k = 0; k < ITEMS; ++k)
        if (big & (1u << k))
            sec[k] = a.big_sec[src[k]];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u64 p = base + k;
        if (!(big & (1u << k)))
            continue;
        bool head = p == gs[k];
        if (!head) { // the member at the place before this one, in the same order
            const u32 before = (k > 0 && (big & (1u << (k - 1))) && g[k - 1] == g[k]) ? sec[k - 1]
                                                                                     : a.big_sec[mirrored[k] ? src[k] + 1u : src[k] - 1u];
            head = before != sec[k];
        }
        if (head) {
            heads |= 1u << k;
            lh = (u32)p + 1u;
        }
    }
    const u32 ih = wave_incl_max(lh);
    if (lane == 63u)
        s_wagg[w] = ih;
    __syncthreads();
    if (!APPLY) {
        if (t == 0) {
            u32 ah = 0;
            for (int ww = 0; ww < WAVES; ++ww)
                ah = ah > s_wagg[ww] ? ah : s_wagg[ww];
            a.tile_agg[(u64)tile * 4 + 0] = ah;
            a.tile_agg[(u64)tile * 4 + 1] = 0;
            a.tile_agg[(u64)tile * 4 + 2] = 0;
            a.tile_agg[(u64)tile * 4 + 3] = 0;
            a.tile_splits[tile] = 0;
        }
        return;
    }
    u32 xh = __shfl_up(ih, 1);
    if (lane == 0)
        xh = 0;
    for (u32 ww = 0; ww < w; ++ww)
        xh = xh > s_wagg[ww] ? xh : s_wagg[ww];
    u32 pre = a.tile_prefix[(u64)tile * 4 + 0];
    const SlabPrefix sp = slabs_before(a.slab_total, tile / a.slab);
    pre = pre > sp.max0 ? pre : sp.max0;
    u32 head_at = xh > pre ? xh : pre; // place + 1 of the last run head before this thread's places
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u64 p = base + k;
        if (p >= a.m || !(big & (1u << k)))
            continue;
        if (heads & (1u << k))
            head_at = (u32)p + 1u;
        // (a large group opens with a head of its own, so the running maximum never reaches back into another group)
        const u32 khead = head_at - 1u;
        const u32 x = a.sufs[src[k]];
        const u32 nr = a.gprim[g[k]] + (khead - gs[k]);
        if (head_at == 0 || khead < gs[k] || khead > (u32)p || nr >= a.n || x >= a.n) {
            atomicExch(a.err, DEV_ERR_PLACE_RANGE);
            continue;
        }
        a.sufs_out[p] = x;
        a.nr_out[p] = nr | (khead != gs[k] ? 0x80000000u : 0u);
    }
}

// Brings the radix-sorted members of the large groups back into the sorted active list, in the (suffix, refined
// rank) form of the small groups: the k-th sorted member of group g goes to place gstart[g] + (k - index of g's first
// member in the sorted large-group list), and its refined rank is gprim[g] + (index of the head of its key run -
// index of g's first member). The two heads are running maxima over the list; like the rank step of generation 0
// they are found in three launches (per-tile maxima, rerank_scan_kernel over the tiles, the pass that applies them),
// which on this part beats one launch with look-back chains by a wide margin when the list is long.
struct PlaceArgs {
    const u64* big_keys; // sorted by (group id, rank[x + h])
    const u32* big_sufs;
    u32 mb;
    u32 m;      // size of the active list
    u32 n;
    u32 groups; // its groups
    int sec_bits;
    const u32* gstart;
    const u32* gprim;
    u32* sufs_out;
    u32* nr_out;
    u32* tile_agg;    // [tiles][4]: last group head, last key-run head of the tile (0: none, or element 0), 0, 0
    u32* tile_splits; // [tiles]: zeroed for the scan
    const u32* tile_prefix; // [tiles][4]: the maxima over the earlier tiles of the tile's slab
    const u32* slab_total;  // [RERANK_SLABS][5]
    u32 slab;               // tiles per slab
    u32* err;
};

// APPLY = false: writes the tile's maxima to tile_agg. APPLY = true: reads their exclusive prefix and does the work.
template <int BLOCK, int ITEMS, bool APPLY>
__global__ __launch_bounds__(BLOCK) void place_big_kernel(PlaceArgs a)
{
    constexpr int TILE = BLOCK * ITEMS;
    constexpr int WAVES = BLOCK / WAVE;
    __shared__ u32 s_wagg[WAVES][2];
    const u32 t = threadIdx.x;
    const u32 lane = t & 63u;
    const u32 w = t >> 6;
    const u32 tile = blockIdx.x;
    const u64 base = (u64)tile * TILE + (u64)t * ITEMS;

    u64 key[ITEMS + 1]; // element base - 1 first
#pragma unroll
    for (int k = 0; k < ITEMS + 1; ++k) {
        const u64 c = base + k;
        key[k] = (c >= 1 && c - 1 < a.mb) ? a.big_keys[c - 1] : 0;
    }
    u32 lg = 0, lk = 0; // last group head / key-run head among this thread's elements (0: none, or element 0)
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u64 c = base + k;
        if (c < a.mb) {
            if (c == 0 || (key[k] >> a.sec_bits) != (key[k + 1] >> a.sec_bits))
                lg = (u32)c;
            if (c == 0 || key[k] != key[k + 1])
                lk = (u32)c;
        }
    }
    const u32 ig = wave_incl_max(lg), ik = wave_incl_max(lk);
    if (lane == 63u) {
        s_wagg[w][0] = ig;
        s_wagg[w][1] = ik;
    }
    __syncthreads();
    if (!APPLY) {
        if (t == 0) {
            u32 ag = 0, ak = 0;
            for (int ww = 0; ww < WAVES; ++ww) {
                ag = ag > s_wagg[ww][0] ? ag : s_wagg[ww][0];
                ak = ak > s_wagg[ww][1] ? ak : s_wagg[ww][1];
            }
            a.tile_agg[(u64)tile * 4 + 0] = ag;
            a.tile_agg[(u64)tile * 4 + 1] = ak;
            a.tile_agg[(u64)tile * 4 + 2] = 0;
            a.tile_agg[(u64)tile * 4 + 3] = 0;
            a.tile_splits[tile] = 0;
        }
        return;
    }
    u32 xg = __shfl_up(ig, 1), xk = __shfl_up(ik, 1);
    if (lane == 0)
        xg = xk = 0;
    for (u32 ww = 0; ww < w; ++ww) {
        xg = xg > s_wagg[ww][0] ? xg : s_wagg[ww][0];
        xk = xk > s_wagg[ww][1] ? xk : s_wagg[ww][1];
    }
    // prefix of the tile = totals of the slabs before its slab, combined with its prefix inside the slab
    u32 pre_g = a.tile_prefix[(u64)tile * 4 + 0], pre_k = a.tile_prefix[(u64)tile * 4 + 1];
    const SlabPrefix sp = slabs_before(a.slab_total, tile / a.slab);
    pre_g = pre_g > sp.max0 ? pre_g : sp.max0;
    pre_k = pre_k > sp.max1 ? pre_k : sp.max1;
    u32 ghead = xg > pre_g ? xg : pre_g;
    u32 khead = xk > pre_k ? xk : pre_k;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u64 c = base + k;
        if (c < a.mb) {
            const u32 g = (u32)(key[k + 1] >> a.sec_bits);
            if (c == 0 || (key[k] >> a.sec_bits) != g)
                ghead = (u32)c;
            if (c == 0 || key[k] != key[k + 1])
                khead = (u32)c;
            const bool ok = g < a.groups && ghead <= khead && khead <= (u32)c;
            const u32 dest = ok ? a.gstart[g] + ((u32)c - ghead) : a.m;
            const u32 nr = ok ? a.gprim[g] + (khead - ghead) : a.n;
            if (dest >= a.m || nr >= a.n) {
                atomicExch(a.err, DEV_ERR_PLACE_RANGE);
                continue;
            }
            a.sufs_out[dest] = a.big_sufs[c];
            a.nr_out[dest] = nr | (khead != ghead ? 0x80000000u : 0u);
        }
    }
}

// Four suffix-array entries per thread: 16 bytes in, 20 bytes out (include/lane.hpp:69-79, include/sa40.hpp:72-75).
__global__ __launch_bounds__(256) void emit_sa40_kernel(const u32* __restrict__ sa32, u32 n, u64 index_base,
                                                        u8* __restrict__ out, int aligned4)
{
    const u64 q = ((u64)blockIdx.x * 256 + threadIdx.x) * 4;
    if (q >= n)
        return;
    if (aligned4 && q + 4 <= n) {
        u64 v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k)
            v[k] = index_base + sa32[q + k];
        u32* o = reinterpret_cast<u32*>(out + 5 * q); // 20 * (q / 4): 4-byte aligned
        o[0] = (u32)v[0];
        o[1] = (u32)(v[0] >> 32) | ((u32)v[1] << 8);
        o[2] = (u32)(v[1] >> 24) | ((u32)v[2] << 16);
        o[3] = (u32)(v[2] >> 16) | ((u32)v[3] << 24);
        o[4] = (u32)(v[3] >> 8);
    } else {
        for (u64 r = q; r < q + 4 && r < n; ++r) {
            const u64 v = index_base + sa32[r];
#pragma unroll
            for (int b = 0; b < 5; ++b)
                out[5 * r + b] = (u8)(v >> (8 * b));
        }
    }
}

__device__ __forceinline__ u64 load_sa40(const u8* sa, u64 r);

// One 5-byte entry to its place (plain byte stores: a 4 + 1 byte split measured the same).
__device__ __forceinline__ void store_sa40(u8* __restrict__ out, u64 r, u64 v)
{
#pragma unroll
    for (int b = 0; b < 5; ++b)
        out[5 * r + b] = (u8)(v >> (8 * b));
}

// Rank-order scatter of a partition that arrives as (suffix lane, local rank) pairs in any order:
// out lane[rank[i]] = lane[i]. The reference scatters into 8-byte words and packs the lanes in a second kernel
// (include/GPU_SACA.cuh:167-182 and :126-133, src/GPU_SACA.cu:2133-2143); here the 5 bytes go straight to their place.
// `bad` is set if a rank is out of range (the reference traps under -DTESTS).
__global__ __launch_bounds__(256) void scatter_lanes_kernel(const u8* __restrict__ suf, const u32* __restrict__ rank, u64 n,
                                                           u8* __restrict__ out, u32* bad)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i >= n)
        return;
    const u64 r = rank[i];
    if (r >= n) {
        atomicExch(bad, 1u);
        return;
    }
    store_sa40(out, r, load_sa40(suf, i));
}

// The same scatter for large partitions, bucketed: 5-byte writes spread over gigabytes run at the rate of scattered
// write requests, writes confined to a window that the last-level cache holds run about four times faster (the same
// finding as for the rank updates above). Step 1 turns every pair into key = (window of its rank) << 40 | suffix and
// value = rank; one radix pass on the window bits groups the pairs by window, in the order of the windows; step 3
// writes the lanes of one window after the other.
__global__ __launch_bounds__(256) void scatter_window_keys_kernel(const u8* __restrict__ suf, const u32* __restrict__ rank, u64 n,
                                                                 int window_log2, u64* __restrict__ keys, u32* __restrict__ vals,
                                                                 u32* bad)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i >= n)
        return;
    u32 r = rank[i];
    if (r >= n) {
        atomicExch(bad, 1u);
        r = 0; // keeps the pass in range; the call fails anyway
    }
    keys[i] = load_sa40(suf, i) | ((u64)(r >> window_log2) << 40);
    vals[i] = r;
}

__global__ __launch_bounds__(256) void scatter_window_lanes_kernel(const u64* __restrict__ keys, const u32* __restrict__ vals, u64 n,
                                                                  u8* __restrict__ out)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i >= n)
        return;
    const u64 v = keys[i];
    const u64 r = vals[i];
    store_sa40(out, r, v);
}

// Standalone K-gram packing (reference: include/utility.hpp:147-162, include/Packed_Prefix.hpp:91-104).
__global__ __launch_bounds__(256) void pack_keys_kernel(const u16* __restrict__ text, u32 n, int key_words,
                                                        u64* __restrict__ keys)
{
    const u64 j = (u64)blockIdx.x * 256 + threadIdx.x;
    if (j >= n)
        return;
    for (int w = 0; w < key_words; ++w)
        keys[j * key_words + w] = load_kgram(text, n, (u32)j, (u32)w);
}

__global__ __launch_bounds__(256) void fill_u32_kernel(u32* p, u64 count, u32 v)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i < count)
        p[i] = v;
}

__device__ __forceinline__ u64 load_sa40(const u8* sa, u64 r)
{
    u64 v = 0;
#pragma unroll
    for (int b = 0; b < 5; ++b)
        v |= (u64)sa[5 * r + b] << (8 * b);
    return v;
}

// Verifier, step 1: inverse[sa[r]] = r, flagging entries out of range.
__global__ __launch_bounds__(256) void verify_invert_kernel(const u8* __restrict__ sa40, u32 n, u64 index_base,
                                                            u32* inverse, u32* bad)
{
    const u64 r = (u64)blockIdx.x * 256 + threadIdx.x;
    if (r >= n)
        return;
    const u64 v = load_sa40(sa40, r);
    if (v < index_base || v - index_base >= n) {
        atomicExch(bad, 1u);
        return;
    }
    inverse[v - index_base] = (u32)r;
}

// Verifier, step 2: every position was hit (so sa is a permutation) and adjacent entries are in order
// (test/end-to-end.cpp:60-76).
__global__ __launch_bounds__(256) void verify_order_kernel(const u8* __restrict__ sa40, const u16* __restrict__ text,
                                                           u32 n, u64 index_base, const u32* __restrict__ inverse,
                                                           u32* bad)
{
    const u64 r = (u64)blockIdx.x * 256 + threadIdx.x;
    if (r >= n)
        return;
    if (inverse[r] == 0xFFFFFFFFu) {
        atomicExch(bad, 1u);
        return;
    }
    if (r == 0)
        return;
    const u64 x = load_sa40(sa40, r - 1) - index_base, y = load_sa40(sa40, r) - index_base;
    if (x >= n || y >= n)
        return; // already flagged by step 1
    const u16 tx = text[x], ty = text[y];
    if (tx < ty)
        return;
    if (tx > ty) {
        atomicExch(bad, 1u);
        return;
    }
    const long long nx = x + 1 < n ? (long long)inverse[x + 1] : -1;
    const long long ny = y + 1 < n ? (long long)inverse[y + 1] : -1;
    if (nx >= ny)
        atomicExch(bad, 1u);
}

} // namespace csa
