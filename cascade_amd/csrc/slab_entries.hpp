// The three per-partition members of the reference's builder in the form its pipeline calls them: the partition
// arrives as a chain of pinned host slabs, is uploaded slab by slab, goes through the device step, and what the step
// leaves is downloaded slab by slab (reference: src/GPU_SACA.cu:1112-1331, 1715-1995, 2107-2164; slab layout
// include/Staging_Slab.hpp:20-119). Host code only; included by cascade_hip.hip after the handle's definition.
#pragma once

namespace {

// Device image of a partition's slabs, allocated by the first slab call of a handle and kept until csa_destroy:
// the columns going in, the columns coming out, and the counters of the outbox.
struct SlabArena {
    unsigned char* base = nullptr;
    u64 bytes = 0;
    u64* key = nullptr;        // generation 0: key_words words per suffix; later: the u32 ranks kept from the step before
    u8* suf = nullptr;         // 5-byte lanes
    u32* beta = nullptr;
    u8* inbox_target = nullptr;
    u32* inbox_rank = nullptr;
    u32* rank_out = nullptr;
    u8* suf_out = nullptr;
    u8* msg_target = nullptr;  // room for 2 * cap messages
    u32* msg_rank = nullptr;
    u32* msg_off = nullptr;    // p + 1 counters
};

constexpr u64 arena_align(u64 v) { return (v + 255u) & ~(u64)255u; }

// Lays the arena out for `cap` suffixes, keys of `key_words` words and p partitions; (re)allocates when it has to grow.
int slab_arena(csa_handle* h, int key_words, u32 p, SlabArena** out)
{
    const u64 cap = h->cap;
    u64 off = 0;
    auto take = [&](u64 bytes) {
        const u64 at = off;
        off = arena_align(off + bytes);
        return at;
    };
    const u64 o_key = take(cap * 8 * (u64)key_words), o_suf = take(cap * 5), o_beta = take(cap * 4), o_it = take(cap * 5),
              o_ir = take(cap * 4), o_ro = take(cap * 4), o_so = take(cap * 5), o_mt = take(cap * 10), o_mr = take(cap * 8),
              o_mo = take(((u64)p + 1) * 4);
    SlabArena* a = h->slab_arena;
    if (!a) {
        a = new SlabArena();
        h->slab_arena = a;
    }
    if (a->bytes < off) {
        if (a->base)
            HIP_TRY(hipFree(a->base));
        a->base = nullptr;
        a->bytes = 0;
        HIP_TRY(hipMalloc((void**)&a->base, off));
        a->bytes = off;
    }
    a->key = reinterpret_cast<u64*>(a->base + o_key);
    a->suf = a->base + o_suf;
    a->beta = reinterpret_cast<u32*>(a->base + o_beta);
    a->inbox_target = a->base + o_it;
    a->inbox_rank = reinterpret_cast<u32*>(a->base + o_ir);
    a->rank_out = reinterpret_cast<u32*>(a->base + o_ro);
    a->suf_out = a->base + o_so;
    a->msg_target = a->base + o_mt;
    a->msg_rank = reinterpret_cast<u32*>(a->base + o_mr);
    a->msg_off = reinterpret_cast<u32*>(a->base + o_mo);
    *out = a;
    return CSA_OK;
}

void free_slab_arena(csa_handle* h)
{
    if (!h->slab_arena)
        return;
    if (h->slab_arena->base)
        (void)hipFree(h->slab_arena->base);
    delete h->slab_arena;
    h->slab_arena = nullptr;
}

// The slabs must lie inside the partition and carry all of it.
int check_slabs(const char* who, const csa_handle* h, const csa_slab* slabs, u32 slab_c, u64 part_sz, u64 chunk_cap, bool need_beta)
{
    if (!h)
        return fail(CSA_ERR_ARG, "%s: null handle", who);
    if (part_sz > h->cap)
        return fail(CSA_ERR_ARG, "%s: %llu suffixes exceed the handle's capacity %llu", who, (unsigned long long)part_sz,
                    (unsigned long long)h->cap);
    if (chunk_cap == 0)
        return fail(CSA_ERR_ARG, "%s: chunk_cap is 0", who);
    if (slab_c && !slabs)
        return fail(CSA_ERR_ARG, "%s: null slab list", who);
    u64 covered = 0;
    for (u32 c = 0; c < slab_c; ++c) {
        const csa_slab& s = slabs[c];
        if (s.size > chunk_cap || s.off > part_sz || s.size > part_sz - s.off)
            return fail(CSA_ERR_ARG, "%s: slab %u covers [%llu, %llu), outside the partition of %llu suffixes or beyond chunk_cap", who, c,
                        (unsigned long long)s.off, (unsigned long long)(s.off + s.size), (unsigned long long)part_sz);
        if (s.size && (!s.key || !s.suf || (need_beta && !s.beta)))
            return fail(CSA_ERR_ARG, "%s: slab %u has a null column", who, c);
        if (s.size && s.off != covered) // the chunks of a partition follow one another (src/GPU_SACA.cu:1396-1400)
            return fail(CSA_ERR_ARG, "%s: slab %u starts at suffix %llu, the slabs before it end at %llu", who, c, (unsigned long long)s.off,
                        (unsigned long long)covered);
        covered += s.size;
    }
    if (covered != part_sz)
        return fail(CSA_ERR_ARG, "%s: the slabs hold %llu suffixes, the partition has %llu", who, (unsigned long long)covered,
                    (unsigned long long)part_sz);
    return CSA_OK;
}

// What both sort steps do once the device step has run: counters to the host, then every slab's share of the ranks,
// the lanes and the outbox (src/GPU_SACA.cu:1305-1331, 1969-1995).
int download_step(const char* who, const SlabArena* a, csa_slab* slabs, u32 slab_c, u32 p, u64 chunk_cap, const csa_step_result& res,
                  u32* h_msg_off, u64* h_active_slot, hipStream_t s)
{
    if (h_msg_off)
        HIP_TRY(hipMemcpyAsync(h_msg_off, a->msg_off, (u64)p * sizeof(u32), hipMemcpyDeviceToHost, s));
    if (h_active_slot)
        *h_active_slot = res.active;
    const u64 outbox_sz = res.messages;
    if (outbox_sz > 2 * chunk_cap * (u64)slab_c)
        return fail(CSA_ERR_ARG, "%s: the outbox of %llu messages does not fit %u slabs of 2 * %llu messages", who,
                    (unsigned long long)outbox_sz, slab_c, (unsigned long long)chunk_cap);
    for (u32 c = 0; c < slab_c; ++c) {
        csa_slab& sl = slabs[c];
        const u64 chunk_off = 2 * (u64)c * chunk_cap;
        const u64 chunk_sz = chunk_off < outbox_sz ? (outbox_sz - chunk_off < 2 * chunk_cap ? outbox_sz - chunk_off : 2 * chunk_cap) : 0;
        sl.outbox_off = (u32)chunk_off;
        sl.outbox_sz = (u32)chunk_sz;
        if (sl.size) {
            HIP_TRY(hipMemcpyAsync(sl.key, a->rank_out + sl.off, sl.size * sizeof(u32), hipMemcpyDeviceToHost, s));
            HIP_TRY(hipMemcpyAsync(sl.suf, a->suf_out + 5 * sl.off, 5 * sl.size, hipMemcpyDeviceToHost, s));
        }
        if (chunk_sz) {
            if (!sl.msg_target || !sl.msg_rank)
                return fail(CSA_ERR_ARG, "%s: slab %u has no room for its %llu outbox messages", who, c, (unsigned long long)chunk_sz);
            HIP_TRY(hipMemcpyAsync(sl.msg_target, a->msg_target + 5 * chunk_off, 5 * chunk_sz, hipMemcpyDeviceToHost, s));
            HIP_TRY(hipMemcpyAsync(sl.msg_rank, a->msg_rank + chunk_off, chunk_sz * sizeof(u32), hipMemcpyDeviceToHost, s));
        }
    }
    HIP_TRY(hipStreamSynchronize(s));
    return CSA_OK;
}

} // namespace

extern "C" {

uint64_t csa_slab_bytes_per_suffix(int key_words)
{
    return 8ull * (u64)(key_words < 1 ? 1 : key_words) + 5 + 4 + 5 + 4 + 4 + 5 + 10 + 8;
}

int csa_sort_init_slabs(csa_handle* h, csa_slab* slabs, uint32_t slab_c, uint64_t part_sz, int key_words, uint32_t p,
                        uint64_t chunk_cap, uint32_t* h_msg_off, uint64_t* h_active_slot, void* stream)
{
    const char* who = "csa_sort_init_slabs";
    if (key_words < 1 || key_words > 4)
        return fail(CSA_ERR_ARG, "%s: key_words = %d is outside [1, 4]", who, key_words);
    if (p < 1 || p > 32768u)
        return fail(CSA_ERR_ARG, "%s: p = %u is outside [1, 32768]", who, p);
    int rc = check_slabs(who, h, slabs, slab_c, part_sz, chunk_cap, true);
    if (rc)
        return rc;
    SlabArena* a = nullptr;
    rc = slab_arena(h, key_words, p, &a);
    if (rc)
        return rc;
    hipStream_t s = (hipStream_t)stream;
    RangeScope range("sort_and_init_rank_and_filter n=%llu", (unsigned long long)part_sz);
    // upload, slab by slab (src/GPU_SACA.cu:1125-1133)
    for (u32 c = 0; c < slab_c; ++c) {
        const csa_slab& sl = slabs[c];
        if (!sl.size)
            continue;
        HIP_TRY(hipMemcpyAsync(a->key + sl.off * (u64)key_words, sl.key, sl.size * 8 * (u64)key_words, hipMemcpyHostToDevice, s));
        HIP_TRY(hipMemcpyAsync(a->suf + 5 * sl.off, sl.suf, 5 * sl.size, hipMemcpyHostToDevice, s));
        HIP_TRY(hipMemcpyAsync(a->beta + sl.off, sl.beta, sl.size * sizeof(u32), hipMemcpyHostToDevice, s));
    }
    csa_step_result res = {0, 0};
    rc = csa_sort_init_dev(h, a->key, key_words, a->suf, a->beta, part_sz, p, a->rank_out, a->suf_out, a->msg_target, a->msg_rank,
                           a->msg_off, stream, &res);
    if (rc)
        return rc;
    return download_step(who, a, slabs, slab_c, p, chunk_cap, res, h_msg_off, h_active_slot, s);
}

int csa_sort_rerank_slabs(csa_handle* h, csa_slab* slabs, uint32_t slab_c, uint64_t part_sz, uint64_t inbox_sz, uint64_t ctx,
                          uint32_t p, uint64_t chunk_cap, uint32_t* h_msg_off, uint64_t* h_active_slot, void* stream)
{
    const char* who = "csa_sort_rerank_slabs";
    if (p < 1 || p > 32768u)
        return fail(CSA_ERR_ARG, "%s: p = %u is outside [1, 32768]", who, p);
    int rc = check_slabs(who, h, slabs, slab_c, part_sz, chunk_cap, true);
    if (rc)
        return rc;
    // a partition cannot receive more messages than it has room for suffixes: one per suffix and generation
    // (src/GPU_SACA.cu:1807-1812)
    if (inbox_sz > h->cap)
        return fail(CSA_ERR_ARG, "%s: an inbox of %llu messages exceeds the handle's capacity %llu", who, (unsigned long long)inbox_sz,
                    (unsigned long long)h->cap);
    u64 delivered = 0;
    for (u32 c = 0; c < slab_c; ++c) {
        const csa_slab& sl = slabs[c];
        if ((u64)sl.inbox_off + sl.inbox_sz > inbox_sz || (sl.inbox_sz && (!sl.msg_target || !sl.msg_rank)))
            return fail(CSA_ERR_ARG, "%s: slab %u carries inbox messages [%u, %u + %u) of %llu, or has no buffer for them", who, c,
                        sl.inbox_off, sl.inbox_off, sl.inbox_sz, (unsigned long long)inbox_sz);
        delivered += sl.inbox_sz;
    }
    if (delivered != inbox_sz)
        return fail(CSA_ERR_ARG, "%s: the slabs carry %llu inbox messages, the inbox has %llu", who, (unsigned long long)delivered,
                    (unsigned long long)inbox_sz);
    SlabArena* a = nullptr;
    rc = slab_arena(h, 1, p, &a);
    if (rc)
        return rc;
    hipStream_t s = (hipStream_t)stream;
    RangeScope range("sort_and_re_rank_and_filter n=%llu ctx=%llu", (unsigned long long)part_sz, (unsigned long long)ctx);
    u32* rank_in = reinterpret_cast<u32*>(a->key);
    // upload: ranks, lanes, routing tags (src/GPU_SACA.cu:1735-1743), then the inbox (:1814-1819)
    for (u32 c = 0; c < slab_c; ++c) {
        const csa_slab& sl = slabs[c];
        if (sl.size) {
            HIP_TRY(hipMemcpyAsync(rank_in + sl.off, sl.key, sl.size * sizeof(u32), hipMemcpyHostToDevice, s));
            HIP_TRY(hipMemcpyAsync(a->suf + 5 * sl.off, sl.suf, 5 * sl.size, hipMemcpyHostToDevice, s));
            HIP_TRY(hipMemcpyAsync(a->beta + sl.off, sl.beta, sl.size * sizeof(u32), hipMemcpyHostToDevice, s));
        }
        if (sl.inbox_sz) {
            HIP_TRY(hipMemcpyAsync(a->inbox_target + 5 * (u64)sl.inbox_off, sl.msg_target, 5 * (u64)sl.inbox_sz, hipMemcpyHostToDevice, s));
            HIP_TRY(hipMemcpyAsync(a->inbox_rank + sl.inbox_off, sl.msg_rank, (u64)sl.inbox_sz * sizeof(u32), hipMemcpyHostToDevice, s));
        }
    }
    csa_step_result res = {0, 0};
    rc = csa_sort_rerank_dev(h, rank_in, a->suf, a->beta, part_sz, a->inbox_target, a->inbox_rank, (u32)inbox_sz, ctx, p, a->rank_out,
                             a->suf_out, a->msg_target, a->msg_rank, a->msg_off, stream, &res);
    if (rc)
        return rc;
    return download_step(who, a, slabs, slab_c, p, chunk_cap, res, h_msg_off, h_active_slot, s);
}

int csa_scatter_slabs(csa_handle* h, csa_slab* slabs, uint32_t slab_c, uint64_t part_sz, uint64_t out_lo, uint64_t chunk_cap,
                      void* stream)
{
    const char* who = "csa_scatter_slabs";
    int rc = check_slabs(who, h, slabs, slab_c, part_sz, chunk_cap, false);
    if (rc)
        return rc;
    if (chunk_cap % 4096 != 0) // the pieces between the edges must be whole disk blocks (include/Direct_File.hpp:27)
        return fail(CSA_ERR_ARG, "%s: chunk_cap = %llu is not a multiple of 4096", who, (unsigned long long)chunk_cap);
    if (part_sz == 0)
        return CSA_OK;
    SlabArena* a = nullptr;
    rc = slab_arena(h, 1, 1, &a);
    if (rc)
        return rc;
    hipStream_t s = (hipStream_t)stream;
    RangeScope range("scatter_to_rank_order n=%llu", (unsigned long long)part_sz);
    u32* rank_in = reinterpret_cast<u32*>(a->key);
    for (u32 c = 0; c < slab_c; ++c) { // src/GPU_SACA.cu:2121-2128
        const csa_slab& sl = slabs[c];
        if (!sl.size)
            continue;
        HIP_TRY(hipMemcpyAsync(a->suf + 5 * sl.off, sl.suf, 5 * sl.size, hipMemcpyHostToDevice, s));
        HIP_TRY(hipMemcpyAsync(rank_in + sl.off, sl.key, sl.size * sizeof(u32), hipMemcpyHostToDevice, s));
    }
    rc = csa_scatter_to_rank_order_dev(h, a->suf, rank_in, part_sz, a->suf_out, stream);
    if (rc)
        return rc;
    // download as cut for the output file: every slab its block-aligned piece, the unaligned edges to the first and the
    // last slab's message-target buffer, the tail one disk block in (src/GPU_SACA.cu:2146-2163)
    const u64 hi = out_lo + 5 * part_sz;
    u64 carried = 0;
    for (u32 c = 0; c < slab_c; ++c) {
        csa_slab& sl = slabs[c];
        u64 cut[6];
        csa_output_cut(out_lo, hi, 5 * chunk_cap, c, slab_c, cut);
        if (cut[1] > cut[0])
            HIP_TRY(hipMemcpyAsync(sl.suf, a->suf_out + (cut[0] - out_lo), cut[1] - cut[0], hipMemcpyDeviceToHost, s));
        if ((cut[3] > cut[2] || cut[5] > cut[4]) && !sl.msg_target)
            return fail(CSA_ERR_ARG, "%s: slab %u carries an edge of the output but has no msg_target buffer", who, c);
        if (cut[3] > cut[2])
            HIP_TRY(hipMemcpyAsync(sl.msg_target, a->suf_out + (cut[2] - out_lo), cut[3] - cut[2], hipMemcpyDeviceToHost, s));
        if (cut[5] > cut[4])
            HIP_TRY(hipMemcpyAsync(sl.msg_target + 4096, a->suf_out + (cut[4] - out_lo), cut[5] - cut[4], hipMemcpyDeviceToHost, s));
        carried += (cut[1] - cut[0]) + (cut[3] - cut[2]) + (cut[5] - cut[4]);
    }
    HIP_TRY(hipStreamSynchronize(s));
    if (carried != 5 * part_sz)
        return fail(CSA_ERR_ARG, "%s: %u chunks of %llu bytes carry %llu of the partition's %llu output bytes (slab_c * chunk_cap "
                    "must reach the partition's size, one chunk more where the partition does not start on a disk block)", who, slab_c,
                    (unsigned long long)(5 * chunk_cap), (unsigned long long)carried, (unsigned long long)(5 * part_sz));
    return CSA_OK;
}

} // extern "C"
