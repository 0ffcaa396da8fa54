// Kernels of the prefix-doubling generations: rank assignment / compaction after a sort, the
// rank[x + h] gather that builds the next generation's keys, sa40 emission, K-gram packing and the
// device-side suffix-array check.
#pragma once

#include "device_utils.hpp"

namespace csa {

// ---------------------------------------------------------------------------------------------
// Rank assignment + compaction, one pass with decoupled look-back (four chains).
//
// Input: the active suffixes sorted by key, keys[c] / sufs[c] for c in [0, m).
//   generation 0 : key = packed K-gram(s); one primary group (the whole partition, rank 0)
//   generation t : key = (group id << sec_bits) | rank[x + h]; group g starts at rank gprim_in[g]
// With a(c) = index of the head of c's run of equal keys and b(c) = index of the head of c's run of
// equal group ids, the refined rank is  prim + a(c) - b(c)  (reference: include/GPU_SACA.cuh:191-208
// for generation 0, :218-280 for the later ones; the two max-scans of src/GPU_SACA.cu:1241-1247,
// 1888-1902 are the look-back chains "a" and "b" here). A suffix whose run has length 1 retires:
// its rank is final and it is written to its place in the suffix array. The others are compacted,
// in order, into the next active list (reference: cub::DevicePartition::Flagged,
// src/GPU_SACA.cu:1253-1261,1917-1925), each with the dense id of its new group.
// ---------------------------------------------------------------------------------------------

struct RerankArgs {
    const u64* keys;
    const u32* sufs;
    u32 m;
    int gen0;      // 1: generation 0 rules
    int key_words; // generation 0: 1 or 2 (the low word is re-read from the text when 2)
    int sec_bits;  // generation t: low bits of the key that hold rank[x + h]
    u32 n;         // partition size
    u32 ell;       // symbols in the generation-0 key
    const u16* text;
    const u32* gprim_in; // generation t: first rank of each incoming group
    u32* rank;           // [n] by text position
    u32* sa32;           // [n] suffix array under construction
    u32* sufs_out;       // next active list
    u32* gids_out;
    u32* gprim_out;
    u32* counts; // [0] = survivors, [1] = their groups (written by the last tile)
    u64* lookback; // [tiles][4]
    u32* ticket;
    u32 epoch;
    u32* err;
};

template <int BLOCK, int ITEMS>
__global__ __launch_bounds__(BLOCK) void rerank_kernel(RerankArgs a)
{
    constexpr int TILE = BLOCK * ITEMS;
    constexpr int WAVES = BLOCK / WAVE;
    __shared__ u32 s_wagg[WAVES][4];
    __shared__ u32 s_tileprefix[4];
    __shared__ u32 s_tile;

    const u32 t = threadIdx.x;
    const u32 lane = t & 63u;
    const u32 w = t >> 6;
    if (t == 0)
        s_tile = atomicAdd(a.ticket, 1u);
    __syncthreads();
    const u32 tile = s_tile;
    const u64 base = (u64)tile * TILE + (u64)t * ITEMS;
    const u32 m = a.m;

    // keys of c-1 .. c+ITEMS, and whether two neighbours are tied
    u64 key[ITEMS + 2];
    u32 suf[ITEMS + 2];
#pragma unroll
    for (int k = 0; k < ITEMS + 2; ++k) {
        const u64 c = base + k; // index c-1 of the array, shifted by one
        const bool in = c >= 1 && c - 1 < m;
        key[k] = in ? a.keys[c - 1] : 0;
        suf[k] = in ? a.sufs[c - 1] : 0;
    }
    // eq[k]: elements (base+k-1) and (base+k) exist and belong to one run of equal keys
    // pq[k]: ... and to one primary group
    bool eq[ITEMS + 1], pq[ITEMS + 1];
#pragma unroll
    for (int k = 0; k < ITEMS + 1; ++k) {
        const u64 c = base + k; // right element of the pair
        const bool both = c >= 1 && c < m;
        bool e = both && key[k] == key[k + 1];
        bool p = both;
        if (a.gen0) {
            if (e && a.key_words == 2)
                e = load_kgram(a.text, a.n, suf[k], 1) == load_kgram(a.text, a.n, suf[k + 1], 1);
            // a suffix that runs off the text inside its key ties with nobody (include/bit-layout.hpp:99-100)
            if (e && ((u64)suf[k] + a.ell >= a.n || (u64)suf[k + 1] + a.ell >= a.n))
                e = false;
        } else {
            p = both && (key[k] >> a.sec_bits) == (key[k + 1] >> a.sec_bits);
        }
        eq[k] = e;
        pq[k] = p;
    }

    // thread-local aggregates
    u32 la = 0, lb = 0, lcnt = 0, lheads = 0;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u64 c = base + k;
        if (c < m) {
            const bool ka = !eq[k];
            const bool pb = !pq[k];
            const bool single = ka && !eq[k + 1];
            if (ka)
                la = (u32)c;
            if (pb)
                lb = (u32)c;
            lcnt += single ? 0u : 1u;
            lheads += (ka && !single) ? 1u : 0u;
        }
    }

    // block-wide exclusive prefix of (max a, max b, sum cnt, sum heads)
    const u32 ia = wave_incl_max(la), ib = wave_incl_max(lb), ic = wave_incl_sum(lcnt), ih = wave_incl_sum(lheads);
    if (lane == 63u) {
        s_wagg[w][0] = ia;
        s_wagg[w][1] = ib;
        s_wagg[w][2] = ic;
        s_wagg[w][3] = ih;
    }
    __syncthreads();
    u32 xa = __shfl_up(ia, 1), xb = __shfl_up(ib, 1), xc = __shfl_up(ic, 1), xh = __shfl_up(ih, 1);
    if (lane == 0)
        xa = xb = xc = xh = 0;
    for (u32 ww = 0; ww < w; ++ww) {
        xa = xa > s_wagg[ww][0] ? xa : s_wagg[ww][0];
        xb = xb > s_wagg[ww][1] ? xb : s_wagg[ww][1];
        xc += s_wagg[ww][2];
        xh += s_wagg[ww][3];
    }
    // tile aggregate -> look-back, one lane per chain
    if (w == 0 && lane < 4) {
        u32 agg = 0;
        for (int ww = 0; ww < WAVES; ++ww)
            agg = lane < 2 ? (agg > s_wagg[ww][lane] ? agg : s_wagg[ww][lane]) : agg + s_wagg[ww][lane];
        u32 excl;
        if (lane < 2)
            excl = lb_exclusive_prefix<true>(a.lookback + lane, 4, tile, a.epoch, agg, a.err);
        else
            excl = lb_exclusive_prefix<false>(a.lookback + lane, 4, tile, a.epoch, agg, a.err);
        s_tileprefix[lane] = excl;
        if ((u64)(tile + 1) * TILE >= m && lane >= 2) // the last tile knows the totals
            a.counts[lane - 2] = excl + agg;
    }
    __syncthreads();
    u32 ra = xa > s_tileprefix[0] ? xa : s_tileprefix[0];
    u32 rb = xb > s_tileprefix[1] ? xb : s_tileprefix[1];
    u32 rc = xc + s_tileprefix[2];
    u32 rh = xh + s_tileprefix[3];

#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u64 c = base + k;
        if (c < m) {
            const bool ka = !eq[k];
            const bool pb = !pq[k];
            const bool single = ka && !eq[k + 1];
            if (ka)
                ra = (u32)c;
            if (pb)
                rb = (u32)c;
            const u32 x = suf[k + 1];
            u32 prim = 0;
            if (!a.gen0)
                prim = a.gprim_in[(u32)(key[k + 1] >> a.sec_bits)];
            const u32 nr = prim + (ra - rb);
            if (a.gen0 || ra != rb)
                a.rank[x] = nr;
            if (single) {
                if (!a.gen0)
                    a.sa32[nr] = x;
            } else {
                if (ka) {
                    a.gprim_out[rh] = nr;
                    rh++;
                }
                a.sufs_out[rc] = x;
                a.gids_out[rc] = rh - 1;
                rc++;
            }
        }
    }
}

// key[c] = (group id << sec_bits) | rank[x + h]; every active x has x + h < n
// (reference: the joined key of include/GPU_SACA.cuh:362-389 with secondary = the rank of suffix x + ctx/2,
// include/bit-layout.hpp:128; here the rank is read straight from HBM by text position).
__global__ __launch_bounds__(256) void gather_keys_kernel(const u32* __restrict__ sufs, const u32* __restrict__ gids,
                                                          const u32* __restrict__ rank, u32 m, u32 n, u32 h,
                                                          int sec_bits, u64* __restrict__ keys)
{
    const u64 c = (u64)blockIdx.x * 256 + threadIdx.x;
    if (c >= m)
        return;
    const u64 src = (u64)sufs[c] + h;
    const u32 sec = src < n ? rank[src] : 0u;
    keys[c] = ((u64)gids[c] << sec_bits) | (u64)sec;
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
