/*
 * CPU oracle for the per-partition suffix sort: TEST INFRASTRUCTURE ONLY (see cascade_oracle.h).
 * Plain C restatement of the reference's algorithm; nothing in the product links this file.
 */
#include "cascade_oracle.h"

#include <stdlib.h>
#include <string.h>

/* ---------- order of two suffixes: include/CPU_Reference.hpp:107-123 ---------- */

int orc_cmp_suffixes_u16(const uint16_t* T, uint64_t n, uint64_t i, uint64_t j, uint64_t max_cmp)
{
    const uint64_t len_i = n - i, len_j = n - j;
    const uint64_t len = len_i < len_j ? len_i : len_j;
    const uint64_t lim = len < max_cmp ? len : max_cmp;
    for (uint64_t k = 0; k < lim; ++k)
        if (T[i + k] != T[j + k])
            return T[i + k] < T[j + k] ? -1 : 1;
    if (lim == max_cmp && len > max_cmp)
        return 0; /* undecided within max_cmp symbols */
    return len_i < len_j ? -1 : 1; /* the exhausted suffix is the smaller one */
}

/* ---------- 5-byte little-endian lanes: include/sa40.hpp:46-75, include/lane.hpp:51-79 ---------- */

void orc_sa40_store(uint8_t* SA, uint64_t r, uint64_t v)
{
    uint8_t* p = SA + ORC_SA_WIDTH * r;
    for (int b = 0; b < ORC_SA_WIDTH; ++b)
        p[b] = (uint8_t)(v >> (8 * b));
}

uint64_t orc_sa40_load(const uint8_t* SA, uint64_t r)
{
    const uint8_t* p = SA + ORC_SA_WIDTH * r;
    uint64_t v = 0;
    for (int b = 0; b < ORC_SA_WIDTH; ++b)
        v |= (uint64_t)p[b] << (8 * b);
    return v;
}

/* ---------- a comparison sort over indices with a context (bottom-up merge sort) ---------- */

typedef int (*orc_less_fn)(const void* ctx, uint64_t a, uint64_t b);

static void merge_sort_u64(uint64_t* a, uint64_t n, orc_less_fn less, const void* ctx)
{
    if (n < 2)
        return;
    uint64_t* tmp = (uint64_t*)malloc(n * sizeof(uint64_t));
    uint64_t* src = a;
    uint64_t* dst = tmp;
    for (uint64_t w = 1; w < n; w *= 2) {
        for (uint64_t lo = 0; lo < n; lo += 2 * w) {
            uint64_t mid = lo + w < n ? lo + w : n;
            uint64_t hi = lo + 2 * w < n ? lo + 2 * w : n;
            uint64_t i = lo, j = mid, k = lo;
            while (i < mid && j < hi)
                dst[k++] = less(ctx, src[j], src[i]) ? src[j++] : src[i++]; /* stable */
            while (i < mid)
                dst[k++] = src[i++];
            while (j < hi)
                dst[k++] = src[j++];
        }
        uint64_t* t = src;
        src = dst;
        dst = t;
    }
    if (src != a)
        memcpy(a, src, n * sizeof(uint64_t));
    free(tmp);
}

/* ---------- the reference CPU suffix sort: test/query.cpp:42-55 ---------- */

typedef struct {
    const uint16_t* T;
    uint64_t n;
} text_ctx;

static int suffix_less(const void* c, uint64_t i, uint64_t j)
{
    const text_ctx* t = (const text_ctx*)c;
    return orc_cmp_suffixes_u16(t->T, t->n, i, j, t->n) < 0;
}

void orc_build_sa40_u16(const uint16_t* T, uint64_t n, uint8_t* SA)
{
    uint64_t* sa = (uint64_t*)malloc((n ? n : 1) * sizeof(uint64_t));
    for (uint64_t i = 0; i < n; ++i)
        sa[i] = i;
    text_ctx ctx = {T, n};
    merge_sort_u64(sa, n, suffix_less, &ctx);
    memset(SA, 0, ORC_SA_WIDTH * n + ORC_SA_PAD_BYTES);
    for (uint64_t r = 0; r < n; ++r)
        orc_sa40_store(SA, r, sa[r]);
    free(sa);
}

/* ---------- the O(n) verifier: test/end-to-end.cpp:13-80 ---------- */

int orc_is_permutation(const uint64_t* sa, uint64_t n)
{
    uint8_t* present = (uint8_t*)calloc(n ? n : 1, 1);
    int ok = 1;
#pragma omp parallel for schedule(static) reduction(&& : ok)
    for (uint64_t i = 0; i < n; ++i) {
        if (sa[i] >= n)
            ok = 0;
        else
            present[sa[i]] = 1;
    }
    if (ok) {
#pragma omp parallel for schedule(static) reduction(&& : ok)
        for (uint64_t i = 0; i < n; ++i)
            if (!present[i])
                ok = 0;
    }
    free(present);
    return ok;
}

int orc_is_correct_sa_u16(const uint64_t* sa, const uint16_t* T, uint64_t n)
{
    if (!orc_is_permutation(sa, n))
        return 0;
    uint64_t* rank = (uint64_t*)malloc((n ? n : 1) * sizeof(uint64_t));
#pragma omp parallel for schedule(static)
    for (uint64_t i = 0; i < n; ++i)
        rank[sa[i]] = i;
    int sorted = 1;
#pragma omp parallel for schedule(static) reduction(&& : sorted)
    for (uint64_t i = 1; i < n; ++i) {
        const uint64_t x = sa[i - 1], y = sa[i];
        if (T[x] < T[y])
            continue;
        if (T[x] > T[y]) {
            sorted = 0;
        } else {
            const int64_t nx = x + 1 < n ? (int64_t)rank[x + 1] : -1; /* past the end sorts first */
            const int64_t ny = y + 1 < n ? (int64_t)rank[y + 1] : -1;
            if (nx >= ny)
                sorted = 0;
        }
    }
    free(rank);
    return sorted;
}

int orc_is_correct_sa40_u16(const uint8_t* sa40, const uint16_t* T, uint64_t n)
{
    uint64_t* sa = (uint64_t*)malloc((n ? n : 1) * sizeof(uint64_t));
#pragma omp parallel for schedule(static)
    for (uint64_t i = 0; i < n; ++i)
        sa[i] = orc_sa40_load(sa40, i);
    const int ok = orc_is_correct_sa_u16(sa, T, n);
    free(sa);
    return ok;
}

/* ---------- K-gram key packing: include/utility.hpp:147-162, include/Packed_Prefix.hpp:91-104 ---------- */

uint64_t orc_pack_word_u16(const uint16_t* T)
{
    uint64_t w = 0;
    for (int k = 0; k < 4; ++k)
        w = (w << 16) | T[k]; /* the first symbol ends in the most significant bits */
    return w;
}

void orc_pack_prefix_u16(const uint16_t* T, uint64_t n, uint64_t j, int key_words, uint64_t* words)
{
    for (int w = 0; w < key_words; ++w) {
        uint16_t s[4];
        for (int k = 0; k < 4; ++k) {
            const uint64_t p = j + 4 * (uint64_t)w + k;
            s[k] = p < n ? T[p] : 0; /* zero padding of the tail: src/GPU_SACA.cu:223-236 */
        }
        words[w] = orc_pack_word_u16(s);
    }
}

/* ---------- forward tag, single partition: include/bit-layout.hpp:99-100 ---------- */

uint64_t orc_fwd_tag(uint64_t tgt, uint64_t n, uint64_t ell)
{
    return tgt < n ? 0 + ell : (n + ell - 1 - tgt);
}

/* ---------- prefix doubling over one partition ---------- */

typedef struct {
    const uint64_t* kw; /* n * key_words packed words */
    const uint64_t* tag;
    int key_words;
} gen0_ctx;

static int gen0_cmp(const gen0_ctx* g, uint64_t a, uint64_t b)
{
    for (int w = 0; w < g->key_words; ++w) {
        const uint64_t x = g->kw[a * g->key_words + w], y = g->kw[b * g->key_words + w];
        if (x != y)
            return x < y ? -1 : 1;
    }
    if (g->tag[a] != g->tag[b])
        return g->tag[a] < g->tag[b] ? -1 : 1;
    return 0;
}

static int gen0_less(const void* c, uint64_t a, uint64_t b)
{
    return gen0_cmp((const gen0_ctx*)c, a, b) < 0;
}

typedef struct {
    const uint64_t* prim; /* indexed by text position */
    const uint64_t* sec;
} gent_ctx;

static int gent_less(const void* c, uint64_t a, uint64_t b)
{
    const gent_ctx* g = (const gent_ctx*)c;
    if (g->prim[a] != g->prim[b])
        return g->prim[a] < g->prim[b];
    return g->sec[a] < g->sec[b];
}

int orc_prefix_doubling_u16(const uint16_t* T, uint64_t n, int key_words, uint64_t* sa_out,
                            uint64_t* active_counts, int max_gens)
{
    if (n == 0)
        return 0;
    const uint64_t ell = 4 * (uint64_t)key_words;
    uint64_t* kw = (uint64_t*)malloc(n * key_words * sizeof(uint64_t));
    uint64_t* tag = (uint64_t*)malloc(n * sizeof(uint64_t));
    uint64_t* order = (uint64_t*)malloc(n * sizeof(uint64_t));
    uint64_t* rank = (uint64_t*)malloc(n * sizeof(uint64_t));
    uint64_t* sec = (uint64_t*)malloc(n * sizeof(uint64_t));
    uint64_t* act = (uint64_t*)malloc(n * sizeof(uint64_t));
    uint64_t* nxt = (uint64_t*)malloc(n * sizeof(uint64_t));
    uint64_t* newrank = (uint64_t*)malloc(n * sizeof(uint64_t));

    for (uint64_t j = 0; j < n; ++j) {
        orc_pack_prefix_u16(T, n, j, key_words, kw + j * key_words);
        tag[j] = orc_fwd_tag(j + ell, n, ell);
        order[j] = j;
    }
    int gens = 0;
    if (gens < max_gens)
        active_counts[gens] = n;
    gens++;

    /* generation 0: include/GPU_SACA.cuh:191-208 + the max-scan of src/GPU_SACA.cu:1241-1247 */
    gen0_ctx g0 = {kw, tag, key_words};
    merge_sort_u64(order, n, gen0_less, &g0);
    uint64_t m = 0;
    {
        uint64_t head = 0;
        for (uint64_t i = 0; i < n; ++i) {
            if (i == 0 || gen0_cmp(&g0, order[i - 1], order[i]) != 0)
                head = i;
            rank[order[i]] = head;
        }
        for (uint64_t i = 0; i < n; ++i) {
            const int tied_prev = i > 0 && rank[order[i - 1]] == rank[order[i]];
            const int tied_next = i + 1 < n && rank[order[i + 1]] == rank[order[i]];
            if (tied_prev || tied_next)
                act[m++] = order[i]; /* stable: the active set stays in rank order */
        }
    }

    /* generations t >= 1: src/GPU_SACA.cu:1999-2103 drives, include/GPU_SACA.cuh:218-280 ranks */
    for (uint64_t h = ell; m > 0; h *= 2) {
        if (gens < max_gens)
            active_counts[gens] = m;
        gens++;
        for (uint64_t c = 0; c < m; ++c) {
            const uint64_t x = act[c];
            sec[x] = x + h < n ? rank[x + h] : 0; /* every active x has x + h < n */
        }
        gent_ctx gt = {rank, sec};
        merge_sort_u64(act, m, gent_less, &gt);
        uint64_t a = 0, b = 0; /* heads of the key run and of the primary run, in the sorted active array */
        for (uint64_t c = 0; c < m; ++c) {
            const uint64_t x = act[c];
            if (c == 0 || rank[act[c - 1]] != rank[x])
                a = b = c;
            else if (sec[act[c - 1]] != sec[x])
                a = c;
            newrank[x] = rank[x] + (a - b); /* include/GPU_SACA.cuh:277 */
        }
        for (uint64_t c = 0; c < m; ++c) /* ranks change only after every key was gathered from the old ones */
            rank[act[c]] = newrank[act[c]];
        uint64_t m2 = 0;
        for (uint64_t c = 0; c < m; ++c) {
            const uint64_t x = act[c];
            const int tied_prev = c > 0 && rank[act[c - 1]] == rank[x];
            const int tied_next = c + 1 < m && rank[act[c + 1]] == rank[x];
            if (tied_prev || tied_next)
                nxt[m2++] = x;
        }
        uint64_t* t = act;
        act = nxt;
        nxt = t;
        m = m2;
    }

    for (uint64_t j = 0; j < n; ++j) /* include/GPU_SACA.cuh:181 */
        sa_out[rank[j]] = j;

    free(kw), free(tag), free(order), free(rank), free(sec), free(act), free(nxt), free(newrank);
    return gens;
}

/* ---------- retirement generations from the finished SA: src/sa_structure.cpp:295-306,375 ---------- */

static int link_level(uint64_t a, uint64_t b, uint64_t l, uint64_t n, uint64_t ell)
{
    if (l < ell)
        return -1;
    const int t = 63 - __builtin_clzll(l / ell);
    const uint64_t c = ell << t;
    if (a + c < n && b + c < n)
        return t;
    return t - 1;
}

void orc_retire_generations_u16(const uint16_t* T, uint64_t n, const uint64_t* sa, uint64_t ell, uint8_t* d_out)
{
    int prev = -1; /* link of the pair (r - 1, r) */
    for (uint64_t r = 0; r < n; ++r) {
        int next = -1;
        if (r + 1 < n) {
            const uint64_t a = sa[r], b = sa[r + 1];
            uint64_t l = 0;
            while (a + l < n && b + l < n && T[a + l] == T[b + l])
                ++l;
            next = link_level(a, b, l, n, ell);
        }
        d_out[sa[r]] = (uint8_t)(1 + (prev > next ? prev : next));
        prev = next;
    }
}

/* ---------- stable LSD radix sort on a bit range (the contract of cub::DeviceRadixSort::SortPairs) ---------- */

void orc_stable_sort_pairs_u64_u32(uint64_t* keys, uint32_t* vals, uint64_t n, int begin_bit, int end_bit)
{
    uint64_t* k2 = (uint64_t*)malloc((n ? n : 1) * sizeof(uint64_t));
    uint32_t* v2 = (uint32_t*)malloc((n ? n : 1) * sizeof(uint32_t));
    for (int shift = begin_bit; shift < end_bit; shift += 8) {
        const int bits = end_bit - shift < 8 ? end_bit - shift : 8;
        const uint64_t mask = (1u << bits) - 1;
        uint64_t count[257] = {0};
        for (uint64_t i = 0; i < n; ++i)
            count[((keys[i] >> shift) & mask) + 1]++;
        for (int d = 0; d < 256; ++d)
            count[d + 1] += count[d];
        for (uint64_t i = 0; i < n; ++i) {
            const uint64_t p = count[(keys[i] >> shift) & mask]++;
            k2[p] = keys[i];
            v2[p] = vals[i];
        }
        memcpy(keys, k2, n * sizeof(uint64_t));
        memcpy(vals, v2, n * sizeof(uint32_t));
    }
    free(k2), free(v2);
}

/* ---------- partition ids ---------- */

uint32_t orc_partition_id_bits(uint32_t p)
{
    /* util::math::bits_for(x) = ceil(log2 x), 0 for x <= 1 (include/utility.hpp:118-121) */
    uint32_t id_bits = 0;
    while (id_bits < 32 && ((uint64_t)1 << id_bits) < (uint64_t)p)
        ++id_bits;
    return (id_bits < 1 ? 1 : id_bits) + 1; /* max(1, bits) + the retirement flag: include/Partition_ID_Map.hpp:79 */
}

/* include/Packed_Prefix.hpp:122-135: a <= b, most significant word first */
static int prefix_le(const uint64_t* a, const uint64_t* b, int words)
{
    for (int w = 0; w < words; ++w)
        if (a[w] != b[w])
            return a[w] < b[w];
    return 1;
}

void orc_partition_ids_u16(const uint16_t* T, uint64_t n, uint64_t text_len, const uint64_t* pivots, int words, uint32_t p,
                           uint16_t* pid, uint64_t* psz)
{
    uint64_t key[64];
    for (uint64_t i = 0; i < n; ++i) {
        orc_pack_prefix_u16(T, text_len, i, words, key);
        /* test/partitioning.cpp:21-31 */
        uint32_t low = 0, high = p - 1;
        while (low < high) {
            const uint32_t mid = low + (high - low) / 2;
            if (prefix_le(key, pivots + (uint64_t)mid * words, words))
                high = mid;
            else
                low = mid + 1;
        }
        pid[i] = (uint16_t)low;
        if (psz)
            psz[low]++;
    }
}

void orc_pack_partition_ids(const uint16_t* pid, uint64_t n, uint32_t bits, uint64_t* out)
{
    for (uint64_t off = 0; off < n; off += 64) { /* one "thread" per group: include/GPU_SACA.cuh:86-90 */
        const uint64_t sz = n - off < 64 ? n - off : 64;
        uint64_t* dst = out + (off / 64) * bits;
        /* include/Partition_ID_Map.hpp:160-176 */
        uint64_t acc = 0;
        uint32_t fill = 0;
        for (uint64_t i = 0; i < sz; ++i) {
            const uint64_t id = pid[off + i];
            acc |= id << fill;
            fill += bits;
            if (fill >= 64) {
                *dst++ = acc;
                fill -= 64;
                acc = fill > 0 ? id >> (bits - fill) : 0;
            }
        }
        if (fill > 0)
            *dst = acc;
    }
}

uint16_t orc_partition_id_map_get(const uint64_t* words, uint32_t bits, uint64_t i)
{
    const uint64_t mask = ((uint64_t)1 << (bits - 1)) - 1; /* the id's bits; the flag is the entry's top bit */
    const uint64_t bit = i * bits, off = bit % 64;
    const uint64_t lo = words[bit / 64] >> off;
    const uint64_t hi = off + bits - 1 > 64 ? words[bit / 64 + 1] << (64 - off) : 0;
    return (uint16_t)((lo | hi) & mask);
}

/* ---------- after the partition sort ---------- */

int orc_scatter_to_rank_order(const uint8_t* suf, const uint32_t* rank, uint64_t n, uint8_t* out)
{
    for (uint64_t i = 0; i < n; ++i) {
        if (rank[i] >= n)
            return -1; /* include/GPU_SACA.cuh:176-179 */
        orc_sa40_store(out, rank[i], orc_sa40_load(suf, i)); /* SA[rank[i]] = suffix; then lane::store of each word */
    }
    return 0;
}

static uint64_t u64_min(uint64_t a, uint64_t b) { return a < b ? a : b; }
static uint64_t u64_max(uint64_t a, uint64_t b) { return a > b ? a : b; }

void orc_output_cut(uint64_t lo, uint64_t hi, uint64_t chunk_bytes, uint64_t c, uint64_t chunk_c, uint64_t out[6])
{
    const uint64_t B = 4096; /* Direct_File::DISK_BLOCK, include/Direct_File.hpp:27 */
    const uint64_t base = lo / B * B, mid_lo = (lo + B - 1) / B * B, mid_hi = u64_max(mid_lo, hi / B * B);
    for (int i = 0; i < 6; ++i)
        out[i] = 0;
    out[0] = u64_min(u64_max(mid_lo, base + c * chunk_bytes), mid_hi);
    out[1] = u64_max(out[0], u64_min(mid_hi, base + (c + 1) * chunk_bytes));
    if (c == 0) {
        out[2] = lo;
        out[3] = u64_min(hi, mid_lo);
    }
    if (c + 1 == chunk_c) {
        out[4] = u64_max(mid_lo, hi / B * B);
        out[5] = u64_max(out[4], hi);
    }
}

/* ---------- slab staging ---------- */

static uint16_t orc_route(uint16_t p_id, int retired)
{
    return retired ? (uint16_t)(p_id | 0x8000u) : p_id; /* include/bit-layout.hpp:135,152 */
}

void orc_stage_slab_u16(const uint16_t* T, uint64_t n, const uint8_t* suf40, uint64_t count, int key_words,
                        const uint16_t* pid, const uint8_t* retired, uint64_t ctx, int generation0, uint64_t* keys,
                        uint32_t* beta)
{
    const uint64_t ell = 4 * (uint64_t)key_words, stride = ctx / 2;
    for (uint64_t i = 0; i < count; ++i) {
        const uint64_t j = orc_sa40_load(suf40, i);
        if (generation0 && keys)
            orc_pack_prefix_u16(T, n, j, key_words, keys + i * key_words); /* src/GPU_SACA.cu:1683 */
        /* src/GPU_SACA.cu:1688-1690 */
        const uint16_t cur = j < ctx ? 0 : orc_route(pid[j - ctx], retired[j - ctx]);
        uint16_t prev;
        if (generation0) {
            const uint64_t tgt = j + ell;
            prev = (uint16_t)(tgt < n ? (uint64_t)pid[tgt] + ell : n + ell - 1 - tgt); /* include/bit-layout.hpp:100 */
        } else {
            prev = j < stride ? 0 : orc_route(pid[j - stride], retired[j - stride]);
        }
        beta[i] = ((uint32_t)prev << 16) | cur; /* include/bit-layout.hpp:137 */
    }
}

/* ---------- rank messages ---------- */

#define ORC_VAL_MASK (((uint64_t)1 << 48) - 1)       /* include/bit-layout.hpp:44 */
#define ORC_PILL_RECEIPT ((uint64_t)1 << 62)         /* include/bit-layout.hpp:57 */
#define ORC_MSG_PILL ((uint32_t)1 << 31)             /* include/message.hpp:22 */
#define ORC_BETA_RETIRED 0x8000u                     /* include/bit-layout.hpp:135 */

void orc_messages_of(uint64_t sa_word, uint64_t key, uint32_t beta, uint64_t i, uint64_t active_sz, uint64_t ctx, int packed,
                     uint64_t out[6])
{
    const uint64_t j = sa_word & ORC_VAL_MASK;
    out[0] = out[3] = 0xFFFFFFFFu;
    out[1] = out[2] = out[4] = out[5] = 0;
    if (j >= ctx && !(beta & ORC_BETA_RETIRED)) { /* include/GPU_SACA.cuh:334 */
        const uint32_t primary = packed ? (uint32_t)((key >> 31) & 0x7FFFFFFFu) : (uint32_t)key;
        out[0] = beta & 0xFFFFu;
        out[1] = j - ctx;
        out[2] = i < active_sz ? primary : (primary | ORC_MSG_PILL); /* :342 */
    }
    if (packed && (key & ORC_PILL_RECEIPT) && j >= (ctx >> 1) && !((beta >> 16) & ORC_BETA_RETIRED)) { /* :345 */
        out[3] = beta >> 16;
        out[4] = j - (ctx >> 1);
        out[5] = (uint32_t)(key & 0x7FFFFFFFu) | ORC_MSG_PILL; /* :349-351 */
    }
}

void orc_count_messages(const uint64_t* sa, const uint64_t* keys, const uint32_t* beta, uint64_t n, uint64_t ctx, int packed,
                        uint32_t* msg_count)
{
    uint64_t m[6];
    for (uint64_t i = 0; i < n; ++i) {
        /* the count kernel tests the pill receipt whatever the key kind (include/GPU_SACA.cuh:306); plain ranks never
         * carry bit 62, so this is the same set of messages */
        orc_messages_of(sa[i], keys[i], beta[i], i, ~(uint64_t)0, ctx, packed, m);
        if (m[0] != 0xFFFFFFFFu)
            msg_count[m[0]]++;
        if (m[3] != 0xFFFFFFFFu)
            msg_count[m[3]]++;
    }
}

void orc_emit_messages(const uint64_t* sa, const uint64_t* keys, const uint32_t* beta, uint64_t n, uint64_t ctx, int packed,
                       uint64_t active_sz, uint8_t* msg_target, uint32_t* msg_rank, uint32_t* msg_off)
{
    uint64_t m[6];
    for (uint64_t i = 0; i < n; ++i) {
        orc_messages_of(sa[i], keys[i], beta[i], i, active_sz, ctx, packed, m);
        for (int e = 0; e < 2; ++e)
            if (m[3 * e] != 0xFFFFFFFFu) {
                const uint32_t slot = msg_off[m[3 * e]]++;
                orc_sa40_store(msg_target, slot, m[3 * e + 1]);
                msg_rank[slot] = (uint32_t)m[3 * e + 2];
            }
    }
}

void orc_join_messages(const uint8_t* msg_target, const uint32_t* msg_rank, uint32_t msg_c, const uint64_t* sa,
                       const uint32_t* primary, uint64_t* keys, uint64_t n)
{
    for (uint32_t i = 0; i < msg_c; ++i) {
        const uint64_t tgt = orc_sa40_load(msg_target, i) & ORC_VAL_MASK;
        uint64_t low = 0, high = n;
        while (low < high) { /* include/GPU_SACA.cuh:373-381 */
            const uint64_t mid = low + (high - low) / 2;
            if ((sa[mid] & ORC_VAL_MASK) < tgt)
                low = mid + 1;
            else
                high = mid;
        }
        if (low == n || (sa[low] & ORC_VAL_MASK) != tgt)
            continue; /* the recipient has retired */
        uint64_t key = ((uint64_t)primary[low] << 31) | (msg_rank[i] & ~ORC_MSG_PILL);
        if (msg_rank[i] & ORC_MSG_PILL)
            key |= ORC_PILL_RECEIPT;
        keys[low] = key;
    }
}
