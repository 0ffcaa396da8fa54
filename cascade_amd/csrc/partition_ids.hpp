// Partition ids of the suffixes of a text against sorted pivots, their bit-packed map and the partition sizes, in
// one pass over the text. The reference does this with two kernels and one global atomic per suffix
// (include/GPU_SACA.cuh:23-74 compute_partition_IDs_kernel, :82-91 pack_partition_IDs_kernel; host loop
// src/GPU_SACA.cu:854-1000); the packed layout is that of include/Partition_ID_Map.hpp:158-177.
#pragma once

#include "device_utils.hpp"

namespace csa {

struct PartitionIdArgs {
    const u16* text;
    u64 n;        // suffixes: text positions [0, n)
    u64 text_len; // symbols readable at `text` (>= n); the text reads as zero beyond them
    const u64* pivots; // [p - 1][W] packed K-grams, first symbols most significant, ascending; inclusive upper bounds
    u32 p;        // partitions
    u32 bits;     // bits per entry of the packed map (the id, then a clear retirement flag)
    u16* pid;     // [n] partition id of every suffix, or null
    u64* packed;  // the packed map (`bits` words per 64 suffixes), or null
    unsigned long long* psz; // [p] partition sizes, added to; or null
    u32 tiles;
    u32 hist_copies_log2; // LDS histogram: counters per partition (hot partitions spread over them)
};

constexpr int PID_BLOCK = 256;
constexpr int PID_ITEMS = 8; // groups of 64 suffixes per wave and tile
constexpr int PID_TILE = PID_BLOCK * PID_ITEMS;
constexpr u32 PID_LDS_PIVOT_WORDS = 4096; // pivots are searched in LDS when they fit
constexpr u32 PID_LDS_BINS = 4096;        // partition sizes are counted in LDS when they fit

// LDS bytes of a workgroup, and the histogram replication that goes with them: at most 16 counters per partition and
// at most 16 KB of histogram.
// words of the packed map that one tile fills: PID_TILE / 64 groups of `bits` 64-bit words
__host__ __device__ inline u32 partition_ids_pack_words(u32 bits) { return (u32)(PID_TILE / 64) * bits; }

inline u32 partition_ids_lds_bytes(int W, u32 p, bool piv_lds, bool want_sizes, bool want_packed, u32 bits, u32* copies_log2)
{
    u32 c = 0;
    const bool hist_lds = want_sizes && p <= PID_LDS_BINS;
    while (hist_lds && c < 4 && (p << (c + 1)) <= PID_LDS_BINS)
        ++c;
    *copies_log2 = c;
    const u32 text_words = (PID_TILE + 4 * W + 6) / 4 + 2;
    u32 steps = 0;
    while (((p - 1u) >> steps) != 0)
        ++steps;
    return text_words * 8u + (piv_lds ? ((1u << steps) - 1u) * (u32)W * 8u : 0u) + (want_packed ? partition_ids_pack_words(bits) * 8u : 0u) +
           (hist_lds ? (p << c) * 4u : 0u);
}

// W: 64-bit words per pivot (the reference's K_WORDS, include/Packed_Prefix.hpp:26-34). PIV_LDS: the pivots fit in LDS.
// A wave handles 64 consecutive suffixes at a time: exactly one group of the packed map. The map is a bit stream (entry e
// of a group takes bits [e * bits, (e + 1) * bits) of the group's `bits` words, least significant first): every lane ORs
// its entry into an image of the tile's stretch of the map in LDS (one or two 32-bit LDS atomics), and after a barrier
// the workgroup stores the image as one contiguous run of words. (One shuffle and one ballot per word and group, the
// first form, was 45 % of the kernel's instructions at 9 bits per entry.) The searches of a thread's PID_ITEMS suffixes advance
// together, one pivot probe each per step, so that their LDS (or cache) latencies overlap. Workgroups stride over
// the tiles so that the LDS histogram is flushed once per workgroup, not once per tile; it is replicated so that
// the lanes of a wave that meet in one hot partition spread over several counters.
template <int W, bool PIV_LDS>
__global__ __launch_bounds__(PID_BLOCK) void partition_ids_kernel(PartitionIdArgs a)
{
    // LDS is sized at launch (partition_ids_lds_bytes): the staged text, then the pivots (PIV_LDS), then the
    // histogram copies. A workgroup that needs little of it leaves room for more workgroups per CU, which is what
    // hides the latency of the stage -> search -> write chain of a tile.
    CSA_DYNAMIC_LDS(u64, s_dyn);
    constexpr u32 TEXT_WORDS = (PID_TILE + 4 * W + 6) / 4 + 2;
    u64* s_text = s_dyn;
    const u32 np = a.p - 1u; // pivots
    int steps = 0; // bits of the pivot count: probes per search
    while ((np >> steps) != 0)
        ++steps;
    const u32 piv_slots = PIV_LDS ? ((1u << steps) - 1u) * (u32)W : 0u; // the table, filled up with all-ones keys
    u64* s_piv = s_dyn + TEXT_WORDS;
    u64* s_pack = s_piv + piv_slots;
    const u32 pack_words = a.packed ? partition_ids_pack_words(a.bits) : 0u;
    u32* s_hist = reinterpret_cast<u32*>(s_pack + pack_words);
    const u32 t = threadIdx.x, lane = t & 63u, w = t >> 6;
    const bool hist_lds = a.psz != nullptr && a.p <= PID_LDS_BINS;
    const u32 copies_log2 = a.hist_copies_log2; // counters per partition in the LDS histogram
    // word j of pivot i at s_piv[j * slots + i]: the first words of all pivots lie together
    const u32 slots = PIV_LDS ? (1u << steps) - 1u : 1u;
    for (u32 i = t; i < piv_slots; i += PID_BLOCK) {
        const u32 j = i / slots, pv = i - j * slots;
        s_piv[i] = pv < np ? a.pivots[(u64)pv * W + j] : ~0ull;
    }
    if (hist_lds)
        for (u32 i = t; i < (a.p << copies_log2); i += PID_BLOCK)
            s_hist[i] = 0;
    __syncthreads();

    for (u32 tile = blockIdx.x; tile < a.tiles; tile += gridDim.x) {
        const u64 tile_base = (u64)tile * PID_TILE;
        const u32 count = (u32)(a.n - tile_base < (u64)PID_TILE ? a.n - tile_base : (u64)PID_TILE);
        const u32 sym_off = stage_text(a.text, a.text_len, tile_base, count + 4u * W - 1u, s_text, t, PID_BLOCK);
        for (u32 i = t; i < pack_words; i += PID_BLOCK)
            s_pack[i] = 0;
        __syncthreads();
        const u32* s_dw = reinterpret_cast<const u32*>(s_text);

        // keys of this thread's suffixes (zero for lanes past the end: never used)
        // (with the pivots in LDS the words after the first are taken from the staged text only where they are needed)
        u64 key[PID_ITEMS][PIV_LDS ? 1 : W];
        u32 id[PID_ITEMS];
#pragma unroll
        for (int k = 0; k < PID_ITEMS; ++k) {
            const u32 local = (w * PID_ITEMS + (u32)k) * 64u + lane;
            id[k] = 0;
#pragma unroll
            for (int j = 0; j < (PIV_LDS ? 1 : W); ++j)
                key[k][j] = local < count ? staged_kgram(s_dw, sym_off + local + 4u * j) : 0ull;
        }
        // id = number of pivots below the key = the smallest id with key <= pivots[id], p - 1 if there is none
        // (test/partitioning.cpp:21-31), found by fixing the bits of the answer from the top. In LDS the table is filled up
        // to 2^steps - 1 entries with all-ones keys, which are below no key: no probe needs a bounds check.
        if (PIV_LDS) {
            // First by the first word alone (one LDS word and one compare per probe): the number of pivots whose first
            // word is below the key's. Only a key whose first word equals that of the pivot it stopped at (a K-gram that
            // some pivot starts with: few suffixes of a text) is placed again, by all W words.
            for (int b = steps - 1; b >= 0; --b) {
#pragma unroll
                for (int k = 0; k < PID_ITEMS; ++k) {
                    const u32 cand = id[k] + (1u << b);
                    id[k] = s_piv[cand - 1u] < key[k][0] ? cand : id[k];
                }
            }
            if (W > 1) {
#pragma unroll
                for (int k = 0; k < PID_ITEMS; ++k) {
                    const u32 local = (w * PID_ITEMS + (u32)k) * 64u + lane;
                    if (local < count && id[k] < np && s_piv[id[k]] == key[k][0]) {
                        u64 whole[W];
#pragma unroll
                        for (int j = 0; j < W; ++j)
                            whole[j] = staged_kgram(s_dw, sym_off + local + 4u * j);
                        u32 again = 0;
                        for (int b = steps - 1; b >= 0; --b) {
                            const u32 cand = again + (1u << b);
                            bool below = false, decided = false; // pivot < key, by the first word that differs
#pragma unroll
                            for (int j = 0; j < W; ++j) {
                                const u64 x = s_piv[(u32)j * slots + cand - 1u];
                                below = decided ? below : x < whole[j];
                                decided = decided || x != whole[j];
                            }
                            again = below ? cand : again;
                        }
                        id[k] = again;
                    }
                }
            }
        } else {
            for (int b = steps - 1; b >= 0; --b) {
#pragma unroll
                for (int k = 0; k < PID_ITEMS; ++k) {
                    const u32 cand = id[k] + (1u << b);
                    if (cand <= np) {
                        const u64* pv = a.pivots + (u64)(cand - 1u) * W;
                        bool below = false;
#pragma unroll
                        for (int j = 0; j < W; ++j) {
                            const u64 x = pv[j];
                            if (x != key[k][j]) {
                                below = x < key[k][j];
                                break;
                            }
                        }
                        if (below)
                            id[k] = cand;
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < PID_ITEMS; ++k) {
            const u32 group_local = (w * PID_ITEMS + (u32)k) * 64u; // wave-uniform
            if (group_local >= count)
                break;
            const u32 local = group_local + lane;
            if (local < count) {
                if (a.pid)
                    a.pid[tile_base + local] = (u16)id[k];
                if (a.psz) {
                    if (hist_lds)
                        atomicAdd(&s_hist[(id[k] << copies_log2) + (lane & ((1u << copies_log2) - 1u))], 1u);
                    else
                        atomicAdd(&a.psz[id[k]], 1ull);
                }
            } else {
                id[k] = 0;
            }
            if (a.packed && id[k] != 0) {
                // Entries fill the words least significant bits first (include/Partition_ID_Map.hpp:158-177): entry e of the
                // group is bits [e * bits, (e + 1) * bits) of its words. Lanes past the end of the text hold id 0 and add
                // nothing, which is what the reference's partial last word carries there.
                u32* image = reinterpret_cast<u32*>(s_pack + (u64)(w * PID_ITEMS + (u32)k) * a.bits);
                const u32 bit = lane * a.bits;
                const u64 v = (u64)id[k] << (bit & 31u); // at most 17 bits, shifted by at most 31
                atomicOr(&image[bit >> 5], (u32)v);
                if ((u32)(v >> 32))
                    atomicOr(&image[(bit >> 5) + 1u], (u32)(v >> 32));
            }
        }
        if (a.packed) {
            __syncthreads();
            // whole groups take `bits` words each; a partial last group only the words its entries reach
            const u32 full = count / 64u, rest = count % 64u;
            const u32 words = full * a.bits + (rest * a.bits + 63u) / 64u;
            u64* out = a.packed + (tile_base / 64u) * a.bits;
            for (u32 i = t; i < words; i += PID_BLOCK)
                out[i] = s_pack[i];
        }
        __syncthreads(); // the staged text is replaced in the next round
    }
    if (hist_lds) {
        for (u32 i = t; i < a.p; i += PID_BLOCK) {
            u32 v = 0;
            for (u32 c = 0; c < (1u << copies_log2); ++c)
                v += s_hist[(i << copies_log2) + c];
            if (v)
                atomicAdd(&a.psz[i], (unsigned long long)v);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Staging of a partition's suffixes on the device: what the reference's host threads do per slab before every
// upload (GPU_SACA::stage_slab, src/GPU_SACA.cu:1611-1692). For the suffix j of every 5-byte lane:
//   generation 0 : key = its packed K-gram (W words) gathered from the text in HBM;
//                  beta = (route of j - ell) | forward tag of j + ell << 16
//   generation t : beta = (route of j - ctx) | route of j - ctx / 2 << 16
// route(x) = partition id of x, with bit 15 set if x has retired; 0 where x would lie before the text
// (include/bit-layout.hpp:137-152). Forward tag: id + ell, or n + ell - 1 - tgt past the end of the text (:99-100).
// Ids and retirement flags are read from the packed partition-id map.
// ---------------------------------------------------------------------------------------------

struct StageArgs {
    const u16* text;
    u64 n; // symbols in the text
    const u8* suf40;
    u64 count;
    const u64* pid_map; // packed map of the whole text
    u32 bits;           // bits per map entry
    u64 ctx;            // context of the generation (ell at generation 0)
    u32 ell;
    int gen0;
    u64* keys; // [count][W], generation 0 only; may be null
    u32* beta; // [count]
};

// entry i of the packed map: id in the low bits - 1 bits, retirement flag on top (include/Partition_ID_Map.hpp:180-196)
__device__ __forceinline__ u32 pid_map_entry(const u64* __restrict__ map, u32 bits, u64 i)
{
    const u64 bit = i * bits, off = bit & 63u;
    u64 v = map[bit >> 6] >> off;
    if (off + bits > 64)
        v |= map[(bit >> 6) + 1] << (64 - off);
    return (u32)(v & ((1ull << bits) - 1ull));
}

__device__ __forceinline__ u32 pid_route(const u64* __restrict__ map, u32 bits, u64 x)
{
    const u32 e = pid_map_entry(map, bits, x);
    const u32 id = e & ((1u << (bits - 1)) - 1u);
    return (e >> (bits - 1)) ? (id | 0x8000u) : id; // BETA_RETIRED, include/bit-layout.hpp:135
}

template <int W>
__global__ __launch_bounds__(256) void stage_slab_kernel(StageArgs a)
{
    const u64 i = (u64)blockIdx.x * 256 + threadIdx.x;
    if (i >= a.count)
        return;
    u64 j = 0;
#pragma unroll
    for (int b = 0; b < 5; ++b)
        j |= (u64)a.suf40[5 * i + b] << (8 * b);
    if (a.gen0 && a.keys) {
#pragma unroll
        for (int w = 0; w < W; ++w) {
            // one 8-byte load where the four symbols exist (the suffixes of a slab are in no order: every load of a wave
            // is 64 separate lines, so four narrow loads per word cost four times the requests)
            const u64 pos = j + 4ull * w;
            u64 k = 0;
            if (pos + 4 <= a.n) {
                u64 raw; // little-endian: s0 | s1 << 16 | s2 << 32 | s3 << 48
                __builtin_memcpy(&raw, a.text + pos, 8);
                k = (raw << 48) | ((raw & 0xFFFF0000ull) << 16) | ((raw >> 16) & 0xFFFF0000ull) | (raw >> 48);
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    k = (k << 16) | (pos + q < a.n ? (u64)a.text[pos + q] : 0ull);
            }
            a.keys[i * W + w] = k;
        }
    }
    const u32 cur = j < a.ctx ? 0u : pid_route(a.pid_map, a.bits, j - a.ctx);
    u32 prev;
    if (a.gen0) {
        const u64 tgt = j + a.ell;
        const u64 tag = tgt < a.n ? (u64)(pid_map_entry(a.pid_map, a.bits, tgt) & ((1u << (a.bits - 1)) - 1u)) + a.ell
                                  : a.n + a.ell - 1 - tgt;
        prev = (u32)tag & 0xFFFFu; // the tag travels in a 16-bit half (include/bit-layout.hpp:137)
    } else {
        const u64 stride = a.ctx / 2;
        prev = j < stride ? 0u : pid_route(a.pid_map, a.bits, j - stride);
    }
    a.beta[i] = (prev << 16) | cur;
}

} // namespace csa
