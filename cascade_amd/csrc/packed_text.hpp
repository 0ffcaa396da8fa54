// Texts over a small alphabet: generation 0 on keys of many symbols.
//
// A K-gram key of the reference holds 4 symbols of 16 bits per word (include/bit-layout.hpp:20-47). When the text uses at
// most 256 different symbols, a symbol fits a code of b = 1, 2, 4 or 8 bits that keeps the order of the symbols, and one
// 64-bit key holds S = 64 / b of them (or the largest 4 W 2^j that fits, W the key words of the caller): the first sort
// then resolves S symbols, which is the state prefix doubling reaches after j more generations of gathers and sorts
// (4 W -> 8 W -> ... -> S symbols; suffixes that run off the text inside the key tie with nobody and sort shorter-first,
// the same rule at every context length, see virtual_to_suffix). A four-letter text packs 32 symbols into a key and
// starts where the reference stands after its generation 3.
//
// The text is encoded once into a stream of codes, most significant first inside 32-bit words (symbol y takes bits
// [y b, y b + b) counted from the top of the word sequence); the key of position y is the S b bits from bit y b on,
// zero codes past the end of the text (the key padding of the reference). The digit of radix pass p of such a key is the
// 8-bit window of the stream that starts 8 p bits before the end of the key: every pass counts the same windows, shifted,
// so one histogram of all 8-bit windows of the stream (taken while encoding) gives every pass's digit counts.
#pragma once

#include "device_utils.hpp"

namespace csa {

// code(s) = hi[s >> 8] * nlo + lo[s & 255]: the ranks of the two bytes of a symbol among the byte values that occur
// (zero counted as occurring: it is the padding), which keeps the order of the symbols.
struct SymbolCodes {
    u8 hi[256];
    u8 lo[256];
    u32 nlo;
    u32 bits;     // b: bits per code, a power of two <= 8
    u32 key_syms; // S: symbols per key, S * b <= 64 and a multiple of 8
};

__device__ __forceinline__ u32 symbol_code(const SymbolCodes& c, u32 s)
{
    return (u32)c.hi[s >> 8] * c.nlo + (u32)c.lo[s & 255u];
}

// The key_bits (8..64) bits of the code stream `w` from bit `bitpos` on (bits counted from the top of word 0), right
// aligned. Reads words bitpos / 32 .. bitpos / 32 + 2.
template <typename Words>
__device__ __forceinline__ u64 packed_window(Words w, u64 bitpos, u32 key_bits)
{
    const u64 idx = bitpos >> 5;
    const u32 sh = (u32)bitpos & 31u;
    const u64 hi = ((u64)w[idx] << 32) | (u64)w[idx + 1];
    const u64 top = sh ? (hi << sh) | ((u64)w[idx + 2] >> (32u - sh)) : hi;
    return top >> (64u - key_bits);
}

constexpr int ENCODE_BLOCK = 256;
constexpr int ENCODE_COPIES = 16;

// stream[wd] for wd < words: the codes of symbols [wd * 32 / b, (wd + 1) * 32 / b), zero past the text; the caller sizes the
// stream so that three words past the last symbol exist (and are written here, as zeros). gramhist[d] += positions
// y < n whose 8-bit window (the codes of symbols y .. y + 8 / b - 1) is d.
__global__ __launch_bounds__(ENCODE_BLOCK) void encode_text_kernel(const u16* __restrict__ text, u32 n, SymbolCodes codes, u32* __restrict__ stream,
                                                                   u64 words, u32* __restrict__ gramhist)
{
    constexpr int MAX_SPW = 32; // symbols per word at b = 1
    __shared__ u64 s_text[(ENCODE_BLOCK * MAX_SPW + 8 + 6) / 4 + 2];
    __shared__ u32 s_hist[256 * ENCODE_COPIES];
    __shared__ SymbolCodes s_codes;
    const u32 t = threadIdx.x;
    for (u32 i = t; i < sizeof(SymbolCodes) / 4; i += ENCODE_BLOCK)
        reinterpret_cast<u32*>(&s_codes)[i] = reinterpret_cast<const u32*>(&codes)[i];
    for (u32 i = t; i < 256 * ENCODE_COPIES; i += ENCODE_BLOCK)
        s_hist[i] = 0;
    const u32 b = codes.bits;
    const u32 spw = 32u / b;  // symbols per word
    const u32 gram = 8u / b;  // symbols per 8-bit window
    const u32 copy = t & (ENCODE_COPIES - 1);
    const u64 blocks = (words + ENCODE_BLOCK - 1) / ENCODE_BLOCK;
    for (u64 blk = blockIdx.x; blk < blocks; blk += gridDim.x) {
        const u64 w0 = blk * ENCODE_BLOCK;
        const u64 p0 = w0 * spw; // first symbol of the block's stretch
        __syncthreads();         // the tables are in place; the stretch of the round before has been read
        const u32 count = ENCODE_BLOCK * spw + gram - 1u;
        const u32 sym_off = stage_text(text, n, p0, count, s_text, t, ENCODE_BLOCK);
        __syncthreads();
        const u16* s16 = reinterpret_cast<const u16*>(s_text) + sym_off + t * spw;
        u64 ext = 0; // the thread's word, then the codes of the next gram - 1 symbols
        for (u32 k = 0; k < spw + gram - 1u; ++k)
            ext |= (u64)symbol_code(s_codes, s16[k]) << (64u - b * (k + 1u));
        const u64 wd = w0 + t;
        if (wd < words)
            stream[wd] = (u32)(ext >> 32);
        const u64 y0 = p0 + (u64)t * spw;
        for (u32 k = 0; k < spw; ++k)
            if (y0 + k < n)
                atomicAdd(&s_hist[((u32)(ext >> (56u - b * k)) & 0xFFu) * ENCODE_COPIES + copy], 1u);
    }
    __syncthreads();
    for (u32 d = t; d < 256; d += ENCODE_BLOCK) {
        u32 v = 0;
#pragma unroll
        for (int c = 0; c < ENCODE_COPIES; ++c)
            v += s_hist[d * ENCODE_COPIES + c];
        if (v)
            atomicAdd(&gramhist[d], v);
    }
}

// ghist[p][d] for the passes of the packed keys of all n suffixes: pass p looks at the window that starts off_p =
// S - (p + 1) * 8 / b symbols into each key, i.e. at the windows of positions off_p .. n + off_p - 1: all windows but
// the first min(off_p, n), plus that many windows past the end of the text (all padding: digit 0).
__global__ __launch_bounds__(256) void packed_hist_expand_kernel(const u32* __restrict__ stream, u32 n, u32 bits, u32 key_syms, int passes,
                                                                 const u32* __restrict__ gramhist, u32* __restrict__ ghist)
{
    const u32 d = threadIdx.x;
    const u32 gram = 8u / bits;
    for (int p = 0; p < passes; ++p) {
        const u32 off = key_syms - (u32)(p + 1) * gram;
        const u32 cut = off < n ? off : n;
        u32 v = gramhist[d];
        for (u32 y = 0; y < cut; ++y)
            if ((u32)packed_window(stream, (u64)y * bits, 8u) == d)
                --v;
        if (d == 0)
            v += cut;
        ghist[p * 256 + d] = v;
    }
}

} // namespace csa
