// The three per-partition members of the reference's builder in the form its pipeline calls them: the partition
// arrives as a chain of pinned host slabs, is uploaded slab by slab, goes through the device step, and what the step
// leaves is downloaded slab by slab (reference: src/GPU_SACA.cu:1112-1331, 1715-1995, 2107-2164; slab layout
// include/Staging_Slab.hpp:20-119). The device image of the slabs lives in the handle's block like every other column of
// a step: the uploads go to the places the step's floor plan gives its inputs, the downloads come from the places it
// gives its outputs (step_entries.hpp), so the slab-shaped entries need no memory beyond csa_step_bytes_per_suffix.
// Host code only; included by cascade_hip.hip after step_entries.hpp.
#pragma once

namespace {

// An error found after transfers into the caller's buffers were queued: the stream is drained before the call returns,
// so that nothing is still writing into memory the caller may free or reuse once it sees the failure.
int fail_drained(hipStream_t s, int rc)
{
    (void)hipStreamSynchronize(s);
    return rc;
}

#define SLAB_TRY(expr)                                                                                                  \
    do {                                                                                                                \
        hipError_t e_ = (expr);                                                                                         \
        if (e_ != hipSuccess)                                                                                           \
            return fail_drained(s, fail(CSA_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__)); \
    } while (0)

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
int download_step(const char* who, const StepColumns& col, csa_slab* slabs, u32 slab_c, u32 p, u64 chunk_cap, const csa_step_result& res,
                  u32* h_msg_off, u64* h_active_slot, hipStream_t s)
{
    // everything that can be refused is checked before the first transfer is queued
    const u64 outbox_sz = res.messages;
    if (outbox_sz > 2 * chunk_cap * (u64)slab_c)
        return fail(CSA_ERR_ARG, "%s: the outbox of %llu messages does not fit %u slabs of 2 * %llu messages", who,
                    (unsigned long long)outbox_sz, slab_c, (unsigned long long)chunk_cap);
    for (u32 c = 0; c < slab_c; ++c)
        if (2 * (u64)c * chunk_cap < outbox_sz && (!slabs[c].msg_target || !slabs[c].msg_rank))
            return fail(CSA_ERR_ARG, "%s: slab %u has no room for its share of the %llu outbox messages", who, c,
                        (unsigned long long)outbox_sz);
    if (h_msg_off)
        SLAB_TRY(hipMemcpyAsync(h_msg_off, col.msg_off, (u64)p * sizeof(u32), hipMemcpyDeviceToHost, s));
    if (h_active_slot)
        *h_active_slot = res.active;
    for (u32 c = 0; c < slab_c; ++c) {
        csa_slab& sl = slabs[c];
        const u64 chunk_off = 2 * (u64)c * chunk_cap;
        const u64 chunk_sz = chunk_off < outbox_sz ? (outbox_sz - chunk_off < 2 * chunk_cap ? outbox_sz - chunk_off : 2 * chunk_cap) : 0;
        sl.outbox_off = (u32)chunk_off;
        sl.outbox_sz = (u32)chunk_sz;
        if (sl.size) {
            SLAB_TRY(hipMemcpyAsync(sl.key, col.rank_out + sl.off, sl.size * sizeof(u32), hipMemcpyDeviceToHost, s));
            SLAB_TRY(hipMemcpyAsync(sl.suf, col.suf40_out + 5 * sl.off, 5 * sl.size, hipMemcpyDeviceToHost, s));
        }
        if (chunk_sz) {
            SLAB_TRY(hipMemcpyAsync(sl.msg_target, col.msg_target + 5 * chunk_off, 5 * chunk_sz, hipMemcpyDeviceToHost, s));
            SLAB_TRY(hipMemcpyAsync(sl.msg_rank, col.msg_rank + chunk_off, chunk_sz * sizeof(u32), hipMemcpyDeviceToHost, s));
        }
    }
    SLAB_TRY(hipStreamSynchronize(s));
    return CSA_OK;
}

} // namespace

extern "C" {

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
    hipStream_t s = (hipStream_t)stream;
    RangeScope range("sort_and_init_rank_and_filter n=%llu", (unsigned long long)part_sz);
    h->last_step = csa_step_result{};
    StepPlan pl;
    rc = step_plan(h, who, part_sz, step_plan_init(key_words), &pl);
    if (rc)
        return rc;
    const InitInputs in = init_input_places(pl, key_words);
    StepColumns col; // outputs left null: they stay in the plan's places, from where the download takes them
    col.msg_off = h->msg_off;
    // upload, slab by slab (src/GPU_SACA.cu:1125-1133)
    for (u32 c = 0; c < slab_c; ++c) {
        const csa_slab& sl = slabs[c];
        if (!sl.size)
            continue;
        SLAB_TRY(hipMemcpyAsync(in.keys + sl.off * (u64)key_words, sl.key, sl.size * 8 * (u64)key_words, hipMemcpyHostToDevice, s));
        SLAB_TRY(hipMemcpyAsync(in.suf40 + 5 * sl.off, sl.suf, 5 * sl.size, hipMemcpyHostToDevice, s));
        SLAB_TRY(hipMemcpyAsync(in.beta + sl.off, sl.beta, sl.size * sizeof(u32), hipMemcpyHostToDevice, s));
    }
    col.keys = in.keys;
    col.suf40 = in.suf40;
    col.beta = in.beta;
    csa_step_result res = {};
    if (part_sz) {
        Launch L;
        L.h = h;
        L.stream = s;
        L.flags = 0;
        L.stats = nullptr;
        rc = step_init(L, who, col, pl, key_words, part_sz, p, &res);
    } else {
        SLAB_TRY(hipMemsetAsync(col.msg_off, 0, ((u64)p + 1) * sizeof(u32), s));
    }
    if (!rc)
        rc = download_step(who, col, slabs, slab_c, p, chunk_cap, res, h_msg_off, h_active_slot, s);
    return rc ? fail_drained(s, rc) : CSA_OK;
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
    hipStream_t s = (hipStream_t)stream;
    RangeScope range("sort_and_re_rank_and_filter n=%llu ctx=%llu", (unsigned long long)part_sz, (unsigned long long)ctx);
    h->last_step = csa_step_result{};
    StepPlan pl; // the unit of the plan is the larger of the cohort and its inbox
    rc = step_plan(h, who, part_sz > inbox_sz ? part_sz : inbox_sz, STEP_PLAN_RERANK, &pl);
    if (rc)
        return rc;
    const RerankInputs in = rerank_input_places(pl);
    StepColumns col;
    col.msg_off = h->msg_off;
    // upload: ranks, lanes, routing tags (src/GPU_SACA.cu:1735-1743), then the inbox (:1814-1819)
    for (u32 c = 0; c < slab_c; ++c) {
        const csa_slab& sl = slabs[c];
        if (sl.size) {
            SLAB_TRY(hipMemcpyAsync(in.rank + sl.off, sl.key, sl.size * sizeof(u32), hipMemcpyHostToDevice, s));
            SLAB_TRY(hipMemcpyAsync(in.suf40 + 5 * sl.off, sl.suf, 5 * sl.size, hipMemcpyHostToDevice, s));
            SLAB_TRY(hipMemcpyAsync(in.beta + sl.off, sl.beta, sl.size * sizeof(u32), hipMemcpyHostToDevice, s));
        }
        if (sl.inbox_sz) {
            SLAB_TRY(hipMemcpyAsync(in.inbox_target + 5 * (u64)sl.inbox_off, sl.msg_target, 5 * (u64)sl.inbox_sz, hipMemcpyHostToDevice, s));
            SLAB_TRY(hipMemcpyAsync(in.inbox_rank + sl.inbox_off, sl.msg_rank, (u64)sl.inbox_sz * sizeof(u32), hipMemcpyHostToDevice, s));
        }
    }
    col.rank_in = in.rank;
    col.suf40 = in.suf40;
    col.beta = in.beta;
    col.inbox_target = in.inbox_target;
    col.inbox_rank = in.inbox_rank;
    col.inbox_sz = (u32)inbox_sz;
    csa_step_result res = {};
    if (part_sz) {
        Launch L;
        L.h = h;
        L.stream = s;
        L.flags = 0;
        L.stats = nullptr;
        rc = step_rerank(L, who, col, pl, part_sz, ctx, p, &res);
    } else {
        SLAB_TRY(hipMemsetAsync(col.msg_off, 0, ((u64)p + 1) * sizeof(u32), s));
    }
    if (!rc)
        rc = download_step(who, col, slabs, slab_c, p, chunk_cap, res, h_msg_off, h_active_slot, s);
    return rc ? fail_drained(s, rc) : CSA_OK;
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
    // how Output_File::cut shares the partition's bytes out over the slabs: checked before anything is queued
    const u64 hi = out_lo + 5 * part_sz;
    u64 carried = 0;
    for (u32 c = 0; c < slab_c; ++c) {
        u64 cut[6];
        csa_output_cut(out_lo, hi, 5 * chunk_cap, c, slab_c, cut);
        if ((cut[3] > cut[2] || cut[5] > cut[4]) && !slabs[c].msg_target)
            return fail(CSA_ERR_ARG, "%s: slab %u carries an edge of the output but has no msg_target buffer", who, c);
        if (cut[1] > cut[0] && !slabs[c].suf)
            return fail(CSA_ERR_ARG, "%s: slab %u carries a piece of the output but has no suf buffer", who, c);
        carried += (cut[1] - cut[0]) + (cut[3] - cut[2]) + (cut[5] - cut[4]);
    }
    if (carried != 5 * part_sz)
        return fail(CSA_ERR_ARG, "%s: %u chunks of %llu bytes carry %llu of the partition's %llu output bytes (slab_c * chunk_cap "
                    "must reach the partition's size, one chunk more where the partition does not start on a disk block)", who, slab_c,
                    (unsigned long long)(5 * chunk_cap), (unsigned long long)carried, (unsigned long long)(5 * part_sz));
    hipStream_t s = (hipStream_t)stream;
    RangeScope range("scatter_to_rank_order n=%llu", (unsigned long long)part_sz);
    // 14 bytes per suffix for lanes in, ranks in and lanes out, taken from the top of the block; the scatter itself takes
    // its 24 bytes per suffix of window-pass buffers from the bottom (or scatters directly where they do not fit)
    h->pool.reset();
    u8* d_out = static_cast<u8*>(h->pool.take(5 * part_sz, true));
    u8* d_suf = static_cast<u8*>(h->pool.take(5 * part_sz, true));
    u32* d_rank = static_cast<u32*>(h->pool.take(part_sz * sizeof(u32), true));
    if (!d_out || !d_suf || !d_rank)
        return fail(CSA_ERR_ARG, "%s: no room for 14 bytes per suffix in the handle's block of %llu bytes", who,
                    (unsigned long long)h->pool.bytes());
    for (u32 c = 0; c < slab_c; ++c) { // src/GPU_SACA.cu:2121-2128
        const csa_slab& sl = slabs[c];
        if (!sl.size)
            continue;
        SLAB_TRY(hipMemcpyAsync(d_suf + 5 * sl.off, sl.suf, 5 * sl.size, hipMemcpyHostToDevice, s));
        SLAB_TRY(hipMemcpyAsync(d_rank + sl.off, sl.key, sl.size * sizeof(u32), hipMemcpyHostToDevice, s));
    }
    rc = scatter_to_rank_order(h, who, d_suf, d_rank, part_sz, d_out, s);
    h->last_high_water = h->pool.high_water();
    if (rc)
        return fail_drained(s, rc);
    // download as cut for the output file: every slab its block-aligned piece, the unaligned edges to the first and the
    // last slab's message-target buffer, the tail one disk block in (src/GPU_SACA.cu:2146-2163)
    for (u32 c = 0; c < slab_c; ++c) {
        csa_slab& sl = slabs[c];
        u64 cut[6];
        csa_output_cut(out_lo, hi, 5 * chunk_cap, c, slab_c, cut);
        if (cut[1] > cut[0])
            SLAB_TRY(hipMemcpyAsync(sl.suf, d_out + (cut[0] - out_lo), cut[1] - cut[0], hipMemcpyDeviceToHost, s));
        if (cut[3] > cut[2])
            SLAB_TRY(hipMemcpyAsync(sl.msg_target, d_out + (cut[2] - out_lo), cut[3] - cut[2], hipMemcpyDeviceToHost, s));
        if (cut[5] > cut[4])
            SLAB_TRY(hipMemcpyAsync(sl.msg_target + 4096, d_out + (cut[4] - out_lo), cut[5] - cut[4], hipMemcpyDeviceToHost, s));
    }
    SLAB_TRY(hipStreamSynchronize(s));
    return CSA_OK;
}

} // extern "C"

#undef SLAB_TRY
