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
#include "packed_text.hpp"

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
    SRC_RANKS = 2, // a dense later generation, first pass: pair i = ((rank[i], rank[i + hop]), i), built from rank[]
    SRC_PACKED = 3 // generation 0 over a small alphabet, first pass: the key of virtual position i is cut from the code stream
};

// Key of text position i in a dense generation: its rank, then the rank of the suffix `hop` symbols on (0 past the
// end of the text; no tied suffix reaches there). radix = 0: the two ranks side by side in the two halves of the key.
// radix = D > 0: rank[] holds ordinals below D (the ranks renumbered 0, 1, 2, ... in their order), and the key is the
// two-digit number rank[i] * D + rank[i + hop], which takes as few bits as two ordinals can: the passes of the sort
// follow the bits in use, and a partition whose suffixes share a few hundred ranks sorts in three passes instead of eight.
__device__ __forceinline__ u64 rank_pair_key(const u32* __restrict__ rank, u32 n, u32 hop, u32 i, u32 radix)
{
    const u64 j = (u64)i + hop;
    const u64 second = j < (u64)n ? rank[j] : 0u;
    return radix ? (u64)rank[i] * radix + second : ((u64)rank[i] << 32) | second;
}

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
    const u32* rank = nullptr; // non-null: the keys are rank_pair_key(rank, n, hop, i, radix) instead of keys[i]
    u32 hop = 0;
    u32 radix = 0;
};

// Digit counters live in LDS as hist[pass][bin][copy]: a lane adds to copy (lane % COPIES), so the lanes of
// a wave that meet on one hot digit (Zipf tokens, runs, group ids) spread over COPIES addresses in COPIES
// banks instead of serialising on one.
constexpr int HIST_COPIES = 8;

__global__ __launch_bounds__(256) void radix_hist_kernel(HistArgs a)
{
    __shared__ u32 s_hist[MAX_PASSES * RADIX_BINS * HIST_COPIES];
    for (int i = threadIdx.x; i < MAX_PASSES * RADIX_BINS * HIST_COPIES; i += 256)
        s_hist[i] = 0;
    __syncthreads();
    const u32 copy = threadIdx.x & (HIST_COPIES - 1);
    // four keys per thread and round, as two 16-byte loads where they all exist: a thread with one 8-byte load in
    // flight per round leaves the kernel waiting on latency (1.6 TB/s)
    const bool aligned16 = (reinterpret_cast<uintptr_t>(a.keys) & 15u) == 0; // a caller's array need not be
    const u64 stride = (u64)gridDim.x * 256 * 4;
    for (u64 i = ((u64)blockIdx.x * 256 + threadIdx.x) * 4; i < a.n; i += stride) {
        u64 key[4];
        const int have = a.n - i < 4 ? (int)(a.n - i) : 4;
        if (!a.rank && have == 4 && aligned16) {
            const uint4 lo = *reinterpret_cast<const uint4*>(a.keys + i), hi = *reinterpret_cast<const uint4*>(a.keys + i + 2);
            key[0] = (u64)lo.x | ((u64)lo.y << 32);
            key[1] = (u64)lo.z | ((u64)lo.w << 32);
            key[2] = (u64)hi.x | ((u64)hi.y << 32);
            key[3] = (u64)hi.z | ((u64)hi.w << 32);
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k)
                key[k] = k < have ? (a.rank ? rank_pair_key(a.rank, a.n, a.hop, (u32)(i + k), a.radix) : a.keys[i + k]) : 0;
        }
        for (int p = 0; p < a.plan.num_passes; ++p) {
            const int sh = a.plan.shift[p];
            const u32 mask = (1u << a.plan.bits[p]) - 1u;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (k < have)
                    atomicAdd(&s_hist[(p * RADIX_BINS + ((u32)(key[k] >> sh) & mask)) * HIST_COPIES + copy], 1u);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < a.plan.num_passes * RADIX_BINS; i += 256) {
        u32 v = 0;
#pragma unroll
        for (int c = 0; c < HIST_COPIES; ++c)
            v += s_hist[i * HIST_COPIES + c];
        if (v)
            atomicAdd(&a.ghist[i], v);
    }
}

// Digit histograms of rank[begin .. end): out[p][d] counts the entries whose digit (rank >> shift[p]) & mask[p] is d, for up
// to four digits of a 32-bit rank. The keys (rank[i], rank[i + hop]) of a dense generation need no histogram of their own:
// their high halves are rank[0 .. n), their low halves rank[hop .. n) and min(hop, n) zeros (rank_hist_combine_kernel).
constexpr int RANK_HIST_PASSES = 4;
constexpr int RANK_HIST_COPIES = 16;

struct RankHistArgs {
    const u32* rank;
    u32 begin, end;
    int num_passes; // <= RANK_HIST_PASSES
    int shift[RANK_HIST_PASSES];
    int bits[RANK_HIST_PASSES];
    u32* out; // [num_passes][256], zeroed by the caller
};

__global__ __launch_bounds__(256) void rank_hist_kernel(RankHistArgs a)
{
    __shared__ u32 s_hist[RANK_HIST_PASSES * RADIX_BINS * RANK_HIST_COPIES];
    for (int i = threadIdx.x; i < RANK_HIST_PASSES * RADIX_BINS * RANK_HIST_COPIES; i += 256)
        s_hist[i] = 0;
    __syncthreads();
    const u32 copy = threadIdx.x & (RANK_HIST_COPIES - 1);
    // eight ranks per thread and round (two 16-byte loads where they all exist and are aligned)
    const bool aligned16 = (reinterpret_cast<uintptr_t>(a.rank + a.begin) & 15u) == 0;
    const u64 stride = (u64)gridDim.x * 256 * 8;
    for (u64 i = (u64)a.begin + ((u64)blockIdx.x * 256 + threadIdx.x) * 8; i < a.end; i += stride) {
        u32 r[8];
        const int have = a.end - i < 8 ? (int)(a.end - i) : 8;
        if (have == 8 && aligned16) {
            const uint4 lo = *reinterpret_cast<const uint4*>(a.rank + i), hi = *reinterpret_cast<const uint4*>(a.rank + i + 4);
            r[0] = lo.x, r[1] = lo.y, r[2] = lo.z, r[3] = lo.w, r[4] = hi.x, r[5] = hi.y, r[6] = hi.z, r[7] = hi.w;
        } else {
#pragma unroll
            for (int k = 0; k < 8; ++k)
                r[k] = k < have ? a.rank[i + k] : 0u;
        }
        for (int p = 0; p < a.num_passes; ++p) {
            const int sh = a.shift[p];
            const u32 mask = (1u << a.bits[p]) - 1u;
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (k < have)
                    atomicAdd(&s_hist[(p * RADIX_BINS + ((r[k] >> sh) & mask)) * RANK_HIST_COPIES + copy], 1u);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < a.num_passes * RADIX_BINS; i += 256) {
        u32 v = 0;
#pragma unroll
        for (int c = 0; c < RANK_HIST_COPIES; ++c)
            v += s_hist[i * RANK_HIST_COPIES + c];
        if (v)
            atomicAdd(&a.out[i], v);
    }
}

// ghist rows [half, 2 half) hold the histograms of rank[0 .. n) (the high halves of the keys), rows [0, half) those of
// rank[0 .. cut), cut = min(hop, n). Rows [0, half) become the histograms of the low halves: all entries but the first
// cut, plus cut zeros.
__global__ __launch_bounds__(256) void rank_hist_combine_kernel(u32* ghist, int half, u32 cut)
{
    const u32 d = threadIdx.x;
    for (int p = 0; p < half; ++p) {
        const u32 all = ghist[(half + p) * RADIX_BINS + d], head = ghist[p * RADIX_BINS + d];
        ghist[p * RADIX_BINS + d] = all - head + (d == 0 ? cut : 0u);
    }
}

// Histogram of the low and of the high byte of every symbol of the text: bytehist[0][d], bytehist[1][d].
// The eight digit histograms of a K-gram key word follow from these two (text_hist_expand_kernel).
constexpr int TEXT_HIST_COPIES = 16;

__global__ __launch_bounds__(256) void text_byte_hist_kernel(const u16* __restrict__ text, u32 n, u32* bytehist)
{
    __shared__ u32 s_hist[2 * RADIX_BINS * TEXT_HIST_COPIES];
    for (int i = threadIdx.x; i < 2 * RADIX_BINS * TEXT_HIST_COPIES; i += 256)
        s_hist[i] = 0;
    __syncthreads();
    const u32 copy = threadIdx.x & (TEXT_HIST_COPIES - 1);
    const u64 stride = (u64)gridDim.x * 256 * 16;
    const bool aligned16 = (reinterpret_cast<uintptr_t>(text) & 15u) == 0;
    for (u64 i = ((u64)blockIdx.x * 256 + threadIdx.x) * 16; i < n; i += stride) {
        u16 sym[16];
        if (i + 16 <= n && aligned16) { // two 16-byte loads in flight per thread
            const uint4* p4 = reinterpret_cast<const uint4*>(text + i);
            const uint4 v0 = p4[0], v1 = p4[1];
            __builtin_memcpy(sym, &v0, 16);
            __builtin_memcpy(sym + 8, &v1, 16);
        } else {
#pragma unroll
            for (int k = 0; k < 16; ++k)
                sym[k] = i + k < n ? text[i + k] : 0;
        }
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            if (i + k < n) {
                atomicAdd(&s_hist[(0 * RADIX_BINS + (sym[k] & 0xFFu)) * TEXT_HIST_COPIES + copy], 1u);
                atomicAdd(&s_hist[(1 * RADIX_BINS + (sym[k] >> 8)) * TEXT_HIST_COPIES + copy], 1u);
            }
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 2 * RADIX_BINS; i += 256) {
        u32 v = 0;
#pragma unroll
        for (int c = 0; c < TEXT_HIST_COPIES; ++c)
            v += s_hist[i * TEXT_HIST_COPIES + c];
        if (v)
            atomicAdd(&bytehist[i], v);
    }
}

// ghist[p][d] for the 8 byte-wide passes of key word `word` over all n suffixes. Pass p looks at byte (p & 1) of
// the symbol at offset pos = 4 * word + 3 - p / 2 of each suffix, i.e. at T[pos .. n) followed by min(pos, n) padding
// zeros: the whole-text byte histogram minus the first min(pos, n) symbols, plus that many zeros.
__global__ __launch_bounds__(256) void text_hist_expand_kernel(const u16* __restrict__ text, u32 n, u32 word,
                                                               const u32* __restrict__ bytehist, u32* ghist)
{
    const u32 d = threadIdx.x;
    for (int p = 0; p < 8; ++p) {
        const u32 byte = p & 1;
        const u32 pos = 4 * word + 3 - p / 2;
        const u32 cut = pos < n ? pos : n;
        u32 v = bytehist[byte * RADIX_BINS + d];
        for (u32 i = 0; i < cut; ++i) {
            const u32 b = byte ? (text[i] >> 8) : (text[i] & 0xFFu);
            if (b == d)
                --v;
        }
        if (d == 0)
            v += cut;
        ghist[p * RADIX_BINS + d] = v;
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
    const void* keys_in; // u64 keys, or u32 keys for the narrow instantiation
    const u32* vals_in;  // unused by the instantiations without values, like vals_out
    void* keys_out;
    u32* vals_out;
    const u16* text;
    u32 n;      // pairs
    u32 text_n; // symbols in the text (SRC_TEXT)
    u32 tail;   // suffixes that run off the text inside their key (SRC_TEXT)
    u32 word;   // key word to build (SRC_TEXT)
    int shift;
    int bits;
    const u32* digit_base; // [256] for this pass
    u64* lookback;         // [tiles][256]
    u64* lookback_groups;  // [ceil(tiles / LB_GROUP)][256]
    u32* ticket;           // zero before the launch (TILES_BY_ARRIVAL)
    u32 order;             // TILES_BY_ARRIVAL or TILES_STATIC_CHUNKS
    u32 xcd_chunk;         // TILES_STATIC_CHUNKS: consecutive tiles given to one XCD
    u32 tiles;             // tiles of the pass = workgroups of the launch
    u32 epoch;
    u32* err;
    const u32* rank = nullptr; // SRC_RANKS: rank[] by text position ...
    u32 hop = 0;               // ... the distance to the second rank of a key ...
    u32 radix = 0;             // ... and how the two make the key (rank_pair_key)
    const u32* stream = nullptr; // SRC_PACKED: the code stream of the text (packed_text.hpp), stream_words words of it ...
    u64 stream_words = 0;
    u32 sym_bits = 0;            // ... with sym_bits bits per symbol ...
    u32 key_bits = 0;            // ... and keys of key_bits bits
};

// How the workgroups of a radix pass come by their tiles (one each). Whatever the order, a tile waits for the tiles
// before it.
//  TILES_BY_ARRIVAL     numbered by an atomic ticket: every predecessor of a tile has started, so every wait ends
//                       whatever else shares the device.
//  TILES_STATIC_CHUNKS  numbered from the workgroup index so that XCD x (workgroup b runs on XCD b % 8) works on chunks
//                       of xcd_chunk consecutive tiles: the runs of one digit written by neighbouring tiles then meet in
//                       one L2 and leave it as full lines (measured 15% faster per pass at chunks of 16). A predecessor
//                       may belong to a workgroup that is dispatched up to 8 (xcd_chunk - 1) places later: the waits only
//                       end if that many workgroups of the launch are resident at once, which holds on a device that
//                       runs nothing else and not, in general, next to other launches (their waiting workgroups can
//                       fill the places this launch needs). The host selects it only for a caller that has declared the
//                       device its own. Tiles past the last whole group of 8 chunks are numbered by workgroup index.
constexpr u32 TILES_BY_ARRIVAL = 0, TILES_STATIC_CHUNKS = 1;
constexpr u32 NO_TILE = 0xFFFFFFFFu;

// Thread 0 of a workgroup: its tile, or NO_TILE when the step is lost already and the workgroup is to leave.
__device__ __forceinline__ u32 onesweep_tile_number(const OnesweepArgs& a)
{
    const bool failed = dev_failed(a.err); // read while the ticket is on its way
    u32 tl;
    if (a.order == TILES_BY_ARRIVAL) {
        tl = atomicAdd(a.ticket, 1u);
    } else {
        const u32 b = blockIdx.x;
        const u32 span = 8u * a.xcd_chunk;
        const u32 whole = (a.tiles / span) * span;
        tl = b;
        if (b < whole) {
            const u32 x = b % 8u, q = b / 8u;
            tl = ((q / a.xcd_chunk) * 8u + x) * a.xcd_chunk + q % a.xcd_chunk;
        }
    }
    return failed || tl >= a.tiles ? NO_TILE : tl;
}

// predecessors a digit's look-back inspects per round
#ifndef CSA_SORT_LB_W
#define CSA_SORT_LB_W 8
#endif

// minimum waves per SIMD the compiler must leave room for (caps the VGPR budget of the radix pass)
#ifndef CSA_SORT_MIN_WAVES
#define CSA_SORT_MIN_WAVES 1
#endif

// KeyT is u64 (the suffix-sort keys) or u32 (the (text position, rank) pairs of the bucketed rank update).
// HI selects the 32-bit half of a 64-bit key that holds this pass's digit (digits never straddle the halves),
// so that the digit is one bit-field extract of a 32-bit register.
// VALS = false: the keys travel alone (records whose payload sits in the key bits that are not sorted on).
template <typename KeyT, int BLOCK, int ITEMS, int SRC, int HI, bool VALS = true>
__global__ __launch_bounds__(BLOCK, CSA_SORT_MIN_WAVES) void onesweep_kernel(OnesweepArgs a)
{
    static_assert(VALS || SRC == SRC_PAIRS, "the passes that build their keys make the suffix indices");
    constexpr int TILE = BLOCK * ITEMS;
    constexpr int WAVES = BLOCK / WAVE;
    static_assert(BLOCK >= RADIX_BINS, "one thread per digit is assumed");
    static_assert(sizeof(KeyT) == 8 || (SRC == SRC_PAIRS && HI == 0), "narrow keys are plain pairs");
    auto rank_key = [&](u32 i) -> u64 { return rank_pair_key(a.rank, a.n, a.hop, i, a.radix); }; // SRC_RANKS: pair i is text position i
    const KeyT* __restrict__ keys_in = static_cast<const KeyT*>(a.keys_in);
    KeyT* __restrict__ keys_out = static_cast<KeyT*>(a.keys_out);

    __shared__ KeyT s_keys[TILE];
    __shared__ u32 s_whist[WAVES * RADIX_BINS];
    __shared__ u32 s_binstart[RADIX_BINS];
    __shared__ u32 s_delta[RADIX_BINS];
    __shared__ u32 s_wsum[WAVES];
    __shared__ u32 s_tile;

    const u32 t = threadIdx.x;
    const u32 lane = t & 63u;
    const u32 w = t >> 6;

    if (t == 0)
        s_tile = onesweep_tile_number(a);
    for (int i = t; i < WAVES * RADIX_BINS; i += BLOCK)
        s_whist[i] = 0;
    __syncthreads();
    const u32 tile = s_tile;
    if (tile == NO_TILE)
        return;
    const u64 base = (u64)tile * TILE;
    const u32 valid = (u32)((u64)a.n - base < (u64)TILE ? (u64)a.n - base : (u64)TILE);
    const u32 sh = (u32)a.shift & 31u;
    const u32 bits = (u32)a.bits;
    const u32 mask = (1u << bits) - 1u;
#define CSA_DIGIT(kk) __builtin_amdgcn_ubfe(HI ? (u32)((u64)(kk) >> 32) : (u32)(kk), sh, bits)
#ifdef __HIP_DEVICE_COMPILE__
#define CSA_LDS_ORDER() asm volatile("" ::: "memory")
#define CSA_OPAQUE(x) asm volatile("" : "+v"(x))
#else
#define CSA_LDS_ORDER() __builtin_amdgcn_wave_barrier() /* CPU emulation: lanes are threads, order them for real */
#define CSA_OPAQUE(x) ((void)0)
#endif
    // ---- first pass of generation 0: stage the tile's stretch of the text in LDS ----
    // The tile covers consecutive virtual positions, i.e. (after the few tail suffixes of tile 0) consecutive text
    // positions j0, j0 + 1, ...; the (still unused) reorder buffer holds the stretch, and each key is assembled
    // from three LDS words instead of four narrow global loads.
    u32 j0 = 0, sym_off = 0;
    if constexpr (SRC == SRC_TEXT) {
        const u32 first_virtual = (u32)base > a.tail ? (u32)base : a.tail;
        j0 = first_virtual - a.tail;
        const u32 count = (u32)TILE - (first_virtual - (u32)base) + 3u; // the last key reaches 3 symbols further
        static_assert(sizeof(KeyT) * TILE >= 8 * ((TILE + 3 + 6) / 4 + 2), "the staged text must fit the reorder buffer");
        sym_off = stage_text(a.text, a.text_n, (u64)j0 + 4ull * a.word, count, reinterpret_cast<u64*>(s_keys), t, BLOCK);
        __syncthreads();
    }
    // the same over a small alphabet: the tile's stretch of the code stream (TILE * sym_bits bits and a key's worth more)
    u64 stream_bit0 = 0;
    if constexpr (SRC == SRC_PACKED) {
        const u32 first_virtual = (u32)base > a.tail ? (u32)base : a.tail;
        const u64 first_word = ((u64)(first_virtual - a.tail) * a.sym_bits) >> 5;
        stream_bit0 = first_word << 5;
        const u32 count = (u32)((((u64)TILE * a.sym_bits + a.key_bits) >> 5) + 3u);
        static_assert(sizeof(KeyT) * TILE >= 4 * (TILE * 8 / 32 + 6), "the staged codes must fit the reorder buffer");
        u32* s_codes = reinterpret_cast<u32*>(s_keys);
        for (u32 i = t; i < count; i += BLOCK)
            s_codes[i] = first_word + i < a.stream_words ? a.stream[first_word + i] : 0u;
        __syncthreads();
    }
    auto text_key = [&](u32 i) -> u64 { // key of virtual position i of this tile (SRC_TEXT, SRC_PACKED)
        if constexpr (SRC == SRC_PACKED) {
            if (i < a.tail)
                return packed_window(a.stream, (u64)(a.text_n - 1u - i) * a.sym_bits, a.key_bits);
            return packed_window(reinterpret_cast<const u32*>(s_keys), (u64)(i - a.tail) * a.sym_bits - stream_bit0, a.key_bits);
        }
        if (i < a.tail)
            return load_kgram(a.text, a.text_n, a.text_n - 1u - i, a.word);
        return staged_kgram(reinterpret_cast<const u32*>(s_keys), (i - a.tail) - j0 + sym_off);
    };

    // ---- load: wave-striped, so that consecutive lanes read consecutive pairs ----
    // (the values are fetched, or computed, only when they are needed: held from here they would cost ITEMS registers
    // through the ranking, which is where the kernel is tightest)
    KeyT key[ITEMS];
    const u32 first_local = w * (WAVE * ITEMS) + lane;
    if (valid == (u32)TILE) { // every tile but the last: no bounds checks, all loads in flight at once
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            const u64 i = base + first_local + k * WAVE;
            if (SRC == SRC_PAIRS)
                key[k] = keys_in[i];
            else if (SRC == SRC_RANKS)
                key[k] = (KeyT)rank_key((u32)i);
            else
                key[k] = (KeyT)text_key((u32)i);
        }
    } else {
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            const u32 local = first_local + k * WAVE;
            const u64 i = base + local;
            key[k] = ~(KeyT)0; // padding: largest digit, and behind every real pair of the tile
            if (local < valid) {
                if (SRC == SRC_PAIRS)
                    key[k] = keys_in[i];
                else if (SRC == SRC_RANKS)
                    key[k] = (KeyT)rank_key((u32)i);
                else
                    key[k] = (KeyT)text_key((u32)i);
            }
        }
    }

    // ---- rank each pair among the pairs of its wave that share its digit ----
    // For every digit bit, (ballot of "bit set") XOR (all-ones if my own bit is set) has a 0 exactly at the lanes
    // that agree with me on that bit; `same` keeps the lanes that agree on every bit, i.e. whose digit is mine.
    // The per-wave counters are plain LDS words: a wave executes its LDS instructions in order, so the counter
    // update of one item is seen by the next item's read; the empty asm statements only keep the compiler from
    // moving those accesses across each other.
    u32* whist = s_whist + w * RADIX_BINS;
    u32 pos[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u32 d = CSA_DIGIT(key[k]);
        u32 same_lo = ~0u, same_hi = ~0u;
#pragma unroll
        for (int b = 0; b < RADIX_BITS; ++b) {
            u32 mine = (u32)__builtin_amdgcn_sbfe(d, b, 1); // 0 or 0xFFFFFFFF
            CSA_OPAQUE(mine); // the ballot tests this register (one compare), not a second extraction of the bit
            const u64 bal = __ballot((int)mine < 0);
            // same &= ~(bal ^ mine): one three-input bit operation per half (table of a & ~(b ^ c): 0x90)
            same_lo = __builtin_amdgcn_bitop3_b32(same_lo, (u32)bal, mine, 0x90);
            same_hi = __builtin_amdgcn_bitop3_b32(same_hi, (u32)(bal >> 32), mine, 0x90);
        }
        const u32 before = __builtin_amdgcn_mbcnt_hi(same_hi, __builtin_amdgcn_mbcnt_lo(same_lo, 0u));
        const u32 prev = whist[d];
        CSA_LDS_ORDER();
        if (before == 0)
            whist[d] = prev + __popc(same_lo) + __popc(same_hi);
        CSA_LDS_ORDER();
        pos[k] = prev + before;
    }
    __syncthreads();

    // ---- one thread per digit: offsets of the waves inside the tile, tile totals; publish them at once ----
    u32 total = 0, real = 0;
    if (t < RADIX_BINS) {
#pragma unroll
        for (int ww = 0; ww < WAVES; ++ww) {
            const u32 c = s_whist[ww * RADIX_BINS + t];
            s_whist[ww * RADIX_BINS + t] = total;
            total += c;
        }
        real = total;
        if (t == mask)
            real -= (u32)TILE - valid; // padding pairs all carry the largest digit
        lb2_publish(a.lookback + t, RADIX_BINS, tile, a.epoch, real);
    }
    // exclusive scan of the 256 totals (padding included: it occupies LDS slots too)
    u32 binstart = 0;
    {
        const u32 incl = wave_incl_sum(total);
        if (t < RADIX_BINS && lane == 63u)
            s_wsum[w] = incl;
        __syncthreads();
        if (t < RADIX_BINS) {
            u32 prefix = 0;
            for (u32 ww = 0; ww < w; ++ww)
                prefix += s_wsum[ww];
            binstart = prefix + incl - total;
            s_binstart[t] = binstart;
        }
    }
    __syncthreads();

    // ---- order the tile in LDS (needs tile-local offsets only), then wait for the tiles before this one ----
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u32 d = CSA_DIGIT(key[k]);
        pos[k] += s_binstart[d] + s_whist[w * RADIX_BINS + d];
        s_keys[pos[k]] = key[k];
    }
    if (t < RADIX_BINS) {
        const u32 excl = lb2_wait_exclusive(a.lookback + t, a.lookback_groups + t, RADIX_BINS, tile, a.epoch, real, a.err);
        s_delta[t] = a.digit_base[t] + excl - binstart; // wraps; added back to an LDS slot below
    }
    __syncthreads();

    // the values are asked for now: their way from HBM overlaps the writes of the keys below (asked for before the
    // look-back they would delay its words, which come back in the order of issue)
    u32 val[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u32 local = first_local + k * WAVE;
        val[k] = 0;
        if (VALS && local < valid)
            val[k] = (SRC == SRC_TEXT || SRC == SRC_PACKED) ? virtual_to_suffix((u32)(base + local), a.text_n, a.tail)
                     : SRC == SRC_RANKS                     ? (u32)(base + local)
                                                            : a.vals_in[base + local];
    }
    // ---- write runs of equal digits to their global places ----
    u32 dst[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const u32 q = k * BLOCK + t;
        if (q < valid) {
            const KeyT kk = s_keys[q];
            dst[k] = q + s_delta[CSA_DIGIT(kk)];
            keys_out[dst[k]] = kk;
        }
    }
    if (!VALS)
        return;
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
#undef CSA_DIGIT
#undef CSA_LDS_ORDER
#undef CSA_OPAQUE
}

// Sorted pairs that ended in the ping-pong partner go back to the caller's arrays (a kernel rather than a copy call,
// so that a sort recorded into a graph consists of kernel launches only).
__global__ __launch_bounds__(256) void copy_pairs_kernel(const u64* __restrict__ keys_in, const u32* __restrict__ vals_in, u64 n,
                                                        u64* __restrict__ keys_out, u32* __restrict__ vals_out)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        keys_out[i] = keys_in[i];
        vals_out[i] = vals_in[i];
    }
}

} // namespace csa
