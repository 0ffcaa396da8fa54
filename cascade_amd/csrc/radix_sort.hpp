// One-sweep LSD radix sort of (64-bit key, 32-bit value) pairs for gfx950.
//
// Per sort: one histogram kernel counts every pass's digits at once, a one-block kernel turns the
// counts into digit bases, then one kernel per pass reads each pair once and writes it once
// ("one sweep"): wave64 ballot/popcount ranks equal digits inside a wave, per-wave counters in LDS
// stitch the waves of a tile together, and a decoupled look-back over per-tile digit counts gives
// each tile its global offsets without a second read of the data.
//
// Replaces cub::DeviceRadixSort::SortPairs of the reference (src/GPU_SACA.cu:1175-1210,1783-1789,1849-1855).
#pragma once

#include "device_utils.hpp"

namespace csa {

constexpr int RADIX_BITS = 8;
constexpr int RADIX_BINS = 1 << RADIX_BITS;
constexpr int MAX_PASSES = 8;

struct PassPlan {
    int num_passes;
    int shift[MAX_PASSES];
    int bits[MAX_PASSES];
};

// How a pass obtains its input pairs.
enum : int {
    SRC_PAIRS = 0, // keys_in[i], vals_in[i]
    SRC_TEXT = 1,  // generation 0, first pass: the pair of virtual position i is built from the text
    SRC_TEXT_IDX = 2 // key word `word` of suffix vals_in[i], rebuilt from the text (128-bit keys, second phase)
};

// Generation 0 feeds the suffixes in the order (n-1, n-2, ..., n-tail, 0, 1, ..., n-tail-1): the last
// `tail` suffixes run off the text inside their key, must each stay a group of one and sort
// shorter-first before any real suffix with the same (zero-padded) key. Putting them first, shortest
// first, makes the stable sort produce exactly that (the reference reaches the same order with a
// separate tag sort, include/bit-layout.hpp:99-100, src/GPU_SACA.cu:1165-1181).
__device__ __forceinline__ u32 virtual_to_suffix(u32 i, u32 n, u32 tail)
{
    return i < tail ? n - 1 - i : i - tail;
}

struct HistArgs {
    const u64* keys;
    const u32* vals;
    const u16* text;
    u32 n;      // pairs
    u32 text_n; // symbols in the text
    u32 word;   // key word to build from the text
    PassPlan plan;
    u32* ghist; // [MAX_PASSES][256], zeroed by the caller
};

template <int SRC>
__global__ __launch_bounds__(256) void radix_hist_kernel(HistArgs a)
{
    __shared__ u32 s_hist[MAX_PASSES * RADIX_BINS];
    for (int i = threadIdx.x; i < MAX_PASSES * RADIX_BINS; i += 256)
        s_hist[i] = 0;
    __syncthreads();
    const u64 stride = (u64)gridDim.x * 256;
    for (u64 i = (u64)blockIdx.x * 256 + threadIdx.x; i < a.n; i += stride) {
        u64 key;
        if (SRC == SRC_PAIRS)
            key = a.keys[i];
        else if (SRC == SRC_TEXT)
            key = load_kgram(a.text, a.text_n, (u32)i, a.word); // a histogram does not care about the order
        else
            key = load_kgram(a.text, a.text_n, a.vals[i], a.word);
        for (int p = 0; p < a.plan.num_passes; ++p) {
            const u32 d = (u32)(key >> a.plan.shift[p]) & ((1u << a.plan.bits[p]) - 1u);
            atomicAdd(&s_hist[p * RADIX_BINS + d], 1u);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < a.plan.num_passes * RADIX_BINS; i += 256) {
        const u32 v = s_hist[i];
        if (v)
            atomicAdd(&a.ghist[i], v);
    }
}

// digit_base[p][d] = number of pairs whose pass-p digit is < d.
__global__ __launch_bounds__(256) void radix_scan_hist_kernel(const u32* ghist, u32* digit_base, int num_passes)
{
    __shared__ u32 s_wave[4];
    const u32 t = threadIdx.x;
    for (int p = 0; p < num_passes; ++p) {
        const u32 c = ghist[p * RADIX_BINS + t];
        const u32 incl = wave_incl_sum(c);
        if ((t & 63u) == 63u)
            s_wave[t >> 6] = incl;
        __syncthreads();
        u32 prefix = 0;
        for (u32 w = 0; w < (t >> 6); ++w)
            prefix += s_wave[w];
        digit_base[p * RADIX_BINS + t] = prefix + incl - c;
        __syncthreads();
    }
}

struct OnesweepArgs {
    const u64* keys_in;
    const u32* vals_in;
    u64* keys_out;
    u32* vals_out;
    const u16* text;
    u32 n;      // pairs
    u32 text_n; // symbols in the text (SRC_TEXT*)
    u32 tail;   // suffixes that run off the text inside their key (SRC_TEXT)
    u32 word;   // key word to build (SRC_TEXT*)
    int shift;
    int bits;
    const u32* digit_base; // [256] for this pass
    u64* lookback;         // [tiles][256]
    u32* ticket;           // zero before the launch
    u32 epoch;
    u32* err;
};

template <int BLOCK, int ITEMS, int SRC>
__global__ __launch_bounds__(BLOCK) void onesweep_kernel(OnesweepArgs a)
{
    constexpr int TILE = BLOCK * ITEMS;
    constexpr int WAVES = BLOCK / WAVE;
    static_assert(BLOCK >= RADIX_BINS, "one thread per digit is assumed");

    __shared__ u64 s_keys[TILE];
    __shared__ u32 s_whist[WAVES * RADIX_BINS];
    __shared__ u32 s_binstart[RADIX_BINS];
    __shared__ u32 s_delta[RADIX_BINS];
    __shared__ u32 s_wsum[WAVES];
    __shared__ u32 s_tile;

    const u32 t = threadIdx.x;
    const u32 lane = t & 63u;
    const u32 w = t >> 6;

    if (t == 0)
        s_tile = atomicAdd(a.ticket, 1u);
    for (int i = t; i < WAVES * RADIX_BINS; i += BLOCK)
        s_whist[i] = 0;
    __syncthreads();
    const u32 tile = s_tile;
    const u64 base = (u64)tile * TILE;
    const u32 valid = (u32)((u64)a.n - base < (u64)TILE ? (u64)a.n - base : (u64)TILE);
    const u32 mask = (1u << a.bits) - 1u;

    // ---- load: wave-striped, so that consecutive lanes read consecutive pairs ----
    u64 key[ITEMS];
    u32 val[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u32 local = w * (WAVE * ITEMS) + k * WAVE + lane;
        const u64 i = base + local;
        if (local < valid) {
            if (SRC == SRC_PAIRS) {
                key[k] = a.keys_in[i];
                val[k] = a.vals_in[i];
            } else if (SRC == SRC_TEXT) {
                val[k] = virtual_to_suffix((u32)i, a.text_n, a.tail);
                key[k] = load_kgram(a.text, a.text_n, val[k], a.word);
            } else {
                val[k] = a.vals_in[i];
                key[k] = load_kgram(a.text, a.text_n, val[k], a.word);
            }
        } else {
            key[k] = ~0ull; // padding: largest digit, and behind every real pair of the tile
            val[k] = 0;
        }
    }

    // ---- rank each pair among the pairs of its wave that share its digit ----
    volatile u32* whist = s_whist + w * RADIX_BINS;
    const u64 lt_mask = (1ull << lane) - 1ull;
    u32 pos[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u32 d = (u32)(key[k] >> a.shift) & mask;
        u64 same = ~0ull;
#pragma unroll
        for (int b = 0; b < RADIX_BITS; ++b) {
            const bool bit = (d >> b) & 1u;
            const u64 bal = __ballot(bit);
            same &= bit ? bal : ~bal;
        }
        const u32 before = __popcll(same & lt_mask);
        const u32 prev = whist[d];
        __builtin_amdgcn_wave_barrier();
        if (before == 0)
            whist[d] = prev + __popcll(same);
        __builtin_amdgcn_wave_barrier();
        pos[k] = prev + before;
    }
    __syncthreads();

    // ---- one thread per digit: offsets of the waves inside the tile, tile totals, look-back ----
    u32 total = 0;
    if (t < RADIX_BINS) {
#pragma unroll
        for (int ww = 0; ww < WAVES; ++ww) {
            const u32 c = s_whist[ww * RADIX_BINS + t];
            s_whist[ww * RADIX_BINS + t] = total;
            total += c;
        }
    }
    // exclusive scan of the 256 totals (padding included: it occupies LDS slots too)
    {
        const u32 incl = wave_incl_sum(total);
        if (t < RADIX_BINS && lane == 63u)
            s_wsum[w] = incl;
        __syncthreads();
        if (t < RADIX_BINS) {
            u32 prefix = 0;
            for (u32 ww = 0; ww < w; ++ww)
                prefix += s_wsum[ww];
            const u32 binstart = prefix + incl - total;
            s_binstart[t] = binstart;
            u32 real = total;
            if (t == mask)
                real -= (u32)TILE - valid; // padding pairs all carry the largest digit
            const u32 excl = lb_exclusive_prefix<false>(a.lookback + t, RADIX_BINS, tile, a.epoch, real, a.err);
            s_delta[t] = a.digit_base[t] + excl - binstart; // wraps; added back to an LDS slot below
        }
    }
    __syncthreads();

    // ---- order the tile in LDS, then write runs of equal digits to their global places ----
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u32 d = (u32)(key[k] >> a.shift) & mask;
        pos[k] += s_binstart[d] + s_whist[w * RADIX_BINS + d];
        s_keys[pos[k]] = key[k];
    }
    __syncthreads();
    u32 dst[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u32 q = k * BLOCK + t;
        if (q < valid) {
            const u64 kk = s_keys[q];
            const u32 d = (u32)(kk >> a.shift) & mask;
            dst[k] = q + s_delta[d];
            a.keys_out[dst[k]] = kk;
        }
    }
    __syncthreads();
    u32* s_vals = reinterpret_cast<u32*>(s_keys);
#pragma unroll
    for (int k = 0; k < ITEMS; ++k)
        s_vals[pos[k]] = val[k];
    __syncthreads();
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u32 q = k * BLOCK + t;
        if (q < valid)
            a.vals_out[dst[k]] = s_vals[q];
    }
}

} // namespace csa
