// Host side of the two per-generation partition steps (reference: GPU_SACA::sort_and_init_rank_and_filter and
// GPU_SACA::sort_and_re_rank_and_filter, src/GPU_SACA.cu:1112-1331 and 1715-1995) between the upload of a partition and
// its download. Included by cascade_hip.hip after the handle's definition.
//
// Floor plan. A step works inside the handle's block and nowhere else. Every column of a step (input, sort buffer,
// intermediate, output) has a fixed place in the block, given below in bytes per suffix from the block's start, and
// columns whose lives do not overlap share a place: the way the reference reaches its 2 * (key + 8 + 4 + 4) + 1 bytes
// per suffix (the outbox over the sorted buffers, src/GPU_SACA.cu:1268-1270; narrowed ranks and lanes over the key
// buffer, :1292,1301; the inbox over the spare suffix buffer, :1805-1806). Which of the two arrays of a ping-pong pair
// holds a sort's result depends on how many passes ran (passes over a constant digit are skipped); the plans never
// depend on it: what follows a sort takes "the other one" of the pair.
//
// Generation 0, one-word keys (48 bytes per suffix):
//   [ 0, 8) K0   [ 8,16) K1   [16,20) P0   [20,24) P1     sort keys and permutation, two of each
//   [ 0, 5) lanes in, [ 5, 9) routing tags in              until they are packed into the carried records, before the sorts
//   [24,40) carried records (16 bytes: suffix word with its forward tag, routing tags)
//   [40,48) keys in                                         until gathered into K0 after the tag sort
//   sorted suffix words -> the spare K, sorted routing tags -> the spare P (after the key sort)
//   [24,32) ranked keys, [32,40) ranked suffix words (the carried records are dead), ranked tags -> the permutation's place
//   [ 0, 5) outbox targets, [ 5, 9) outbox ranks, [ 9,13) ranks out, [40,45) lanes out
// Generation 0, keys of W = 2..4 words (65 bytes per suffix for W = 2, 8 W + 52 = 76 / 84 for W = 3 / 4):
//   [ 0,24) K0 K1 P0 P1 as above (the sort on word 0)
//   [24,28) places of the tied, [28,36) [36,40) second key array and permutation of the tied suffixes' sort
//           (their first ones are the spare K and the spare P)
//   [40,45) lanes in, [45,49) routing tags in, [ik, ik + 8 W) keys in, ik = 49 (W = 2) or 52
//   sorted word 1 -> the spare K; [24,40) carried records; [40,48) sorted suffix words; sorted tags -> the spare P
//   [24,32) ranked keys, [32,40) ranked suffix words; ranked tags -> the permutation's place (W = 2: the ranking reads
//           words 0 and 1 from the sorted columns) or [48,52) (W >= 3: it reads words 2 and 3 through the permutation)
//   [ 0, 5) outbox targets, [ 5, 9) outbox ranks, [ 9,13) ranks out, [40,45) lanes out
// Generation t >= 1 (47 bytes per unit, the unit being the larger of the cohort and its inbox):
//   [ 0, 4) routing tags in, [ 4, 8) ranks in, [12,17) inbox targets, [17,21) inbox ranks, [42,47) lanes in
//   [21,35) the join table (8-byte slots, up to 1.75 per unit), [35,42) the list places of its slots
//   [ 8,12) what the messages deliver: the rank word received at every list place
//   [24,32) composite keys (the table and the inbox are dead)
//   the sort: keys [24,32) <-> [32,40), permutations in P0 [16,20) and P1 [20,24)
//   sorted suffix words (gathered from the lanes in) -> the other of [24,32) / [32,40); sorted tags -> the spare P
//   [ 0, 8) ranked keys, [ 8,16) ranked suffix words, ranked tags -> the permutation's place
//   [24,34) outbox targets, [34,42) outbox ranks (two messages per suffix), [16,20) ranks out, [42,47) lanes out
// With the caller's own buffers for inputs and outputs (csa_sort_init_dev, csa_sort_rerank_dev) the same plans hold
// and those places stay unused.
#pragma once

namespace {

// A partition on the device as a step sees it: null inputs / outputs are columns of the plan (the slab-shaped entries
// upload into them and download from them), others are the caller's buffers.
struct StepColumns {
    const u64* keys = nullptr;    // generation 0: key_words words per suffix
    const u32* rank_in = nullptr; // later generations: the partition-local ranks kept from the step before
    const u8* suf40 = nullptr;
    const u32* beta = nullptr;
    const u8* inbox_target = nullptr;
    const u32* inbox_rank = nullptr;
    u32 inbox_sz = 0;
    u32* rank_out = nullptr;
    u8* suf40_out = nullptr;
    u8* msg_target = nullptr;
    u32* msg_rank = nullptr;
    u32* msg_off = nullptr; // p + 1 counters
};

// Places of a plan: `off` bytes per suffix from the start of the block, for a unit of `unit` suffixes (the partition's
// size rounded up so that every place starts on a 256-byte boundary).
struct StepPlan {
    unsigned char* base = nullptr;
    u64 unit = 0;
    template <typename T> T* at(u32 off) const { return reinterpret_cast<T*>(base + (u64)off * unit); }
};

constexpr u32 STEP_PLAN_INIT1 = 48, STEP_PLAN_INIT2 = 65, STEP_PLAN_RERANK = 47;
constexpr u32 step_plan_init(int key_words) { return key_words == 1 ? STEP_PLAN_INIT1 : key_words == 2 ? STEP_PLAN_INIT2 : 8u * (u32)key_words + 52u; }

// Lays a plan of `per_suffix` bytes per suffix over the handle's block for `count` suffixes.
int step_plan(csa_handle* h, const char* who, u64 count, u32 per_suffix, StepPlan* plan)
{
    plan->base = h->pool.base();
    plan->unit = (count + 255u) & ~(u64)255u;
    const u64 need = plan->unit * per_suffix;
    if (need > h->pool.bytes())
        return fail(CSA_ERR_ARG, "%s: a step over %llu suffixes needs %llu bytes of the handle's block (%u per suffix), which has %llu: "
                    "create the handle for a larger partition (csa_create_steps holds csa_step_bytes_per_suffix(key_words) per suffix)",
                    who, (unsigned long long)count, (unsigned long long)need, per_suffix, (unsigned long long)h->pool.bytes());
    h->last_high_water = need;
    return CSA_OK;
}

// Places of the slab-shaped entries' uploads (slab_entries.hpp) in the plans above.
struct InitInputs {
    u64* keys;
    u8* suf40;
    u32* beta;
};
InitInputs init_input_places(const StepPlan& pl, int key_words)
{
    if (key_words == 1)
        return {pl.at<u64>(40), pl.at<u8>(0), pl.at<u32>(5)};
    return {pl.at<u64>(key_words == 2 ? 49 : 52), pl.at<u8>(40), pl.at<u32>(45)};
}
struct RerankInputs {
    u32* rank;
    u8* suf40;
    u32* beta;
    u8* inbox_target;
    u32* inbox_rank;
};
RerankInputs rerank_input_places(const StepPlan& pl) { return {pl.at<u32>(4), pl.at<u8>(42), pl.at<u32>(0), pl.at<u8>(12), pl.at<u32>(17)}; }

// Where the tail of a step (ranking, messages, narrowing) puts its columns.
struct TailPlaces {
    u64* key_r;
    u64* words_r;
    u32* beta_r;
    u8* msg_target;
    u32* msg_rank;
    u32* rank_out;
    u8* suf40_out;
};

// Shared tail of the two steps: the list (keys, suffix words, routing tags) sorted by key is ranked and split into
// active / retired, the cohort's messages are emitted, ranks and lanes are narrowed for the caller.
template <bool GEN0>
int finish_partition_step(Launch& L, const char* who, StepColumns& c, const TailPlaces& tp, const u64* sorted_key0, const u64* sorted_key1,
                          const u32* perm, int key_words, const u64* sorted_words, const u32* sorted_beta, u64 m, u64 ctx, u32 p,
                          csa_step_result* res)
{
    csa_handle* h = L.h;
    hipStream_t s = L.stream;
    const RankTables r = rank_tables(h, (u32)m, STEP_TILE);
    unsigned long long* d_active = reinterpret_cast<unsigned long long*>(h->counts + 8);
    StepRankArgs ra;
    ra.key0 = sorted_key0;
    ra.key1 = sorted_key1;
    ra.keys_src = c.keys;
    ra.perm = perm;
    ra.key_words = key_words;
    ra.words = sorted_words;
    ra.beta = sorted_beta;
    ra.m = m;
    ra.key_out = tp.key_r;
    ra.words_out = tp.words_r;
    ra.beta_out = tp.beta_r;
    ra.tile_agg = r.tile_agg;
    ra.tile_splits = r.tile_splits;
    ra.tile_prefix = r.tile_prefix;
    ra.slab_total = r.slab_total;
    ra.slab = r.slab;
    ra.slabs = r.slabs;
    ra.active_out = d_active;
    ra.unserved_out = reinterpret_cast<unsigned long long*>(h->counts + 10);
    ra.pills_out = reinterpret_cast<unsigned long long*>(h->counts + 12);
    ra.incoherent_out = h->counts + 14;
    HIP_TRY(hipMemsetAsync(h->counts + 8, 0, 8 * sizeof(u32), s));
    hipLaunchKernelGGL((step_rank_kernel<GEN0, false>), dim3(r.tiles), dim3(STEP_BLOCK), 0, s, ra);
    hipLaunchKernelGGL(rerank_scan_kernel, dim3(r.slabs), dim3(1024), 0, s, r.tile_agg, r.tile_prefix, r.tiles, r.slab, r.slab_total,
                       r.tile_splits);
    hipLaunchKernelGGL((step_rank_kernel<GEN0, true>), dim3(r.tiles), dim3(STEP_BLOCK), 0, s, ra);
    HIP_TRY(hipGetLastError());
    // the cohort's messages, collated by destination (src/GPU_SACA.cu:1266-1287,1930-1951): at most one per suffix in
    // generation 0, a payload and a forwarded pill later (src/Staging_Slab.cpp:33-34)
    if (!c.msg_target)
        c.msg_target = tp.msg_target;
    if (!c.msg_rank)
        c.msg_rank = tp.msg_rank;
    MessageArgs ma;
    int rc = fill_message_args(ma, who, tp.words_r, tp.key_r, tp.beta_r, m, ctx, GEN0 ? 0 : 1, p);
    if (rc)
        return rc;
    HIP_TRY(hipMemsetAsync(c.msg_off, 0, ((u64)p + 1) * sizeof(u32), s));
    ma.msg_off = c.msg_off;
    const u32 grid = ma.tiles < 4096u ? ma.tiles : 4096u;
    hipLaunchKernelGGL(count_messages_kernel, dim3(grid), dim3(MSG_BLOCK), 0, s, ma);
    hipLaunchKernelGGL(message_offsets_kernel, dim3(1), dim3(1024), 0, s, c.msg_off, p + 1);
    ma.active_sz = d_active;
    ma.msg_target = c.msg_target;
    ma.msg_rank = c.msg_rank;
    const u64 emit_tiles = (m + EMIT_TILE - 1) / EMIT_TILE;
    if (ma.p <= EMIT_FEW_PARTS)
        hipLaunchKernelGGL((emit_messages_kernel<EMIT_FEW_PARTS>), dim3((u32)(emit_tiles < 2048u ? emit_tiles : 2048u)), dim3(EMIT_BLOCK), 0, s, ma);
    else
        hipLaunchKernelGGL((emit_messages_kernel<MSG_LDS_PARTS>), dim3((u32)(emit_tiles < 2048u ? emit_tiles : 2048u)), dim3(EMIT_BLOCK), 0, s, ma);
    HIP_TRY(hipGetLastError());
    // what the caller persists: narrowed ranks and lanes (src/GPU_SACA.cu:1289-1305)
    if (!c.rank_out)
        c.rank_out = tp.rank_out;
    if (!c.suf40_out)
        c.suf40_out = tp.suf40_out;
    hipLaunchKernelGGL(narrow_and_pack_kernel, dim3((u32)((m + 255) / 256)), dim3(256), 0, s, (const u64*)tp.key_r, (const u64*)tp.words_r, m,
                       GEN0 ? 0 : 1, c.rank_out, c.suf40_out);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipMemcpyAsync(h->h_pinned + 8, h->counts + 8, 8 * sizeof(u32), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipMemcpyAsync(h->h_pinned + 16, c.msg_off + (p - 1), sizeof(u32), hipMemcpyDeviceToHost, s));
    rc = read_counts(L, nullptr);
    if (rc)
        return rc;
    const u32* hp = h->h_pinned;
    csa_step_result out;
    out.active = (u64)hp[8] | ((u64)hp[9] << 32);
    out.messages = hp[16];
    out.unserved = GEN0 ? 0 : (u64)hp[10] | ((u64)hp[11] << 32);
    out.pills = GEN0 ? 0 : (u64)hp[12] | ((u64)hp[13] << 32);
    out.incoherent_pills = GEN0 ? 0 : hp[14];
    h->last_step = out;
    if (res)
        *res = out;
    return CSA_OK;
}

int check_step_args(csa_handle* h, const char* who, u64 m, u32 p, const void* a, const void* b, const void* c, const void* d)
{
    if (!h)
        return fail(CSA_ERR_ARG, "%s: null handle", who);
    if (p < 1 || p > 32768u)
        return fail(CSA_ERR_ARG, "%s: p = %u is outside [1, 32768]", who, p);
    if (m > h->cap)
        return fail(CSA_ERR_ARG, "%s: %llu suffixes exceed the handle's capacity %llu", who, (unsigned long long)m,
                    (unsigned long long)h->cap);
    if (m && (!a || !b || !c || !d))
        return fail(CSA_ERR_ARG, "%s: null buffer", who);
    return CSA_OK;
}

// Generation 0 of a partition of m > 0 suffixes, laid out by `pl` (the plans at the top of this file).
int step_init(Launch& L, const char* who, StepColumns& c, const StepPlan& pl, int key_words, u64 m, u32 p, csa_step_result* res)
{
    csa_handle* h = L.h;
    hipStream_t s = L.stream;
    const u32 blocks = (u32)((m + 255) / 256);
    HIP_TRY(hipMemsetAsync(h->counts, 0, 8 * sizeof(u32), s));
    u64* K[2] = {pl.at<u64>(0), pl.at<u64>(8)};
    u32* P[2] = {pl.at<u32>(16), pl.at<u32>(20)};
    uint4* carried = pl.at<uint4>(24);
    int kc = 0, pc = 0; // the arrays that hold the current keys / permutation
    int in_out = 0, passes = 0, rc;
    u64 *sorted_key1 = nullptr, *sorted_words;
    const u32* perm = nullptr;
    TailPlaces tp;
    tp.key_r = pl.at<u64>(24);
    tp.words_r = pl.at<u64>(32);
    tp.msg_target = pl.at<u8>(0);
    tp.msg_rank = pl.at<u32>(5);
    tp.rank_out = pl.at<u32>(9);
    tp.suf40_out = pl.at<u8>(40);
    if (key_words == 1) {
        // lane and routing tags of a suffix side by side in one 16-byte record (a streaming pass), so that the gather by
        // the sort's permutation costs one random line per suffix instead of two; the slabs' lanes and tags lie where
        // the sort buffers are about to be
        hipLaunchKernelGGL(pack_carried_kernel, dim3(blocks), dim3(256), 0, s, c.suf40, c.beta, m, carried);
        // stable LSD sort by (key word, forward tag): the tag first, then the word (src/GPU_SACA.cu:1165-1227), on
        // (64-bit key, permutation) pairs
        hipLaunchKernelGGL(iota_kernel, dim3(blocks), dim3(256), 0, s, P[pc], m);
        hipLaunchKernelGGL(carried_tag_keys_kernel, dim3(blocks), dim3(256), 0, s, (const uint4*)carried, m, K[kc]);
        rc = radix_sort(L, SRC_PAIRS, nullptr, 0, 0, 0, K[kc], P[pc], K[kc ^ 1], P[pc ^ 1], (u32)m, make_plan(0, 16), &in_out, &passes);
        if (rc)
            return rc;
        pc ^= in_out;
        hipLaunchKernelGGL(gather_u64_kernel, dim3(blocks), dim3(256), 0, s, c.keys, (const u32*)P[pc], m, 1u, 0u, K[0]);
        rc = radix_sort(L, SRC_PAIRS, nullptr, 0, 0, 0, K[0], P[pc], K[1], P[pc ^ 1], (u32)m, make_plan(0, 64), &in_out, &passes);
        if (rc)
            return rc;
        kc = in_out;
        pc ^= in_out;
        sorted_words = K[kc ^ 1];
        tp.beta_r = P[pc]; // the permutation is dead once the carried columns are gathered
    } else {
        // Wider keys: the same order, (key words, forward tag), reached from the most significant word. All suffixes are
        // sorted by word 0 alone. Only those that tie with a neighbour on it can still change places, and only inside their
        // run: they are taken out in order, sorted among themselves by (word 0, ..., word W - 1, tag) with the stable LSD
        // passes of the reference (tag, then the words from the last, src/GPU_SACA.cu:1165-1227) and put back, in that
        // order, at the places the tied entries held. Sorting every suffix on every word costs 2 + 8 W passes over the
        // partition; this costs 8, plus 2 + 8 W over the tied ones.
        hipLaunchKernelGGL(iota_kernel, dim3(blocks), dim3(256), 0, s, P[pc], m);
        hipLaunchKernelGGL(gather_u64_kernel, dim3(blocks), dim3(256), 0, s, c.keys, (const u32*)P[pc], m, (u32)key_words, 0u, K[0]);
        rc = radix_sort(L, SRC_PAIRS, nullptr, 0, 0, 0, K[0], P[pc], K[1], P[pc ^ 1], (u32)m, make_plan(0, 64), &in_out, &passes);
        if (rc)
            return rc;
        kc = in_out;
        pc ^= in_out;
        const RankTables r = rank_tables(h, (u32)m, STEP_TILE);
        u32* tied_pos = pl.at<u32>(24);
        TieArgs ta;
        ta.keys = K[kc];
        ta.perm = P[pc];
        ta.m = m;
        ta.pos_out = tied_pos;
        ta.perm_out = P[pc ^ 1]; // the spare permutation array takes the tied suffixes
        ta.tile_agg = r.tile_agg;
        ta.tile_splits = r.tile_splits;
        ta.tile_prefix = r.tile_prefix;
        ta.slab_total = r.slab_total;
        ta.slab = r.slab;
        ta.slabs = r.slabs;
        ta.total_out = reinterpret_cast<unsigned long long*>(h->counts + 6);
        hipLaunchKernelGGL((tie_kernel<false>), dim3(r.tiles), dim3(STEP_BLOCK), 0, s, ta);
        hipLaunchKernelGGL(rerank_scan_kernel, dim3(r.slabs), dim3(1024), 0, s, r.tile_agg, r.tile_prefix, r.tiles, r.slab, r.slab_total,
                           r.tile_splits);
        hipLaunchKernelGGL((tie_kernel<true>), dim3(r.tiles), dim3(STEP_BLOCK), 0, s, ta);
        HIP_TRY(hipGetLastError());
        rc = read_counts(L, nullptr);
        if (rc)
            return rc;
        const u64 tied = h->h_pinned[6];
        if (tied > m)
            return fail(CSA_ERR_INTERNAL, "%s: %llu of %llu suffixes counted as tied", who, (unsigned long long)tied, (unsigned long long)m);
        if (tied > 0) {
            const u32 tblocks = (u32)((tied + 255) / 256);
            u64* SK[2] = {K[kc ^ 1], pl.at<u64>(28)}; // the sorted word 0 stays in K[kc]
            u32* SV[2] = {P[pc ^ 1], pl.at<u32>(36)};
            int sv = 0;
            hipLaunchKernelGGL(gather_tag_keys_kernel, dim3(tblocks), dim3(256), 0, s, c.beta, (const u32*)SV[sv], tied, SK[0]);
            rc = radix_sort(L, SRC_PAIRS, nullptr, 0, 0, 0, SK[0], SV[sv], SK[1], SV[sv ^ 1], (u32)tied, make_plan(0, 16), &in_out, &passes);
            if (rc)
                return rc;
            sv ^= in_out;
            for (int w = key_words - 1; w >= 0; --w) {
                hipLaunchKernelGGL(gather_u64_kernel, dim3(tblocks), dim3(256), 0, s, c.keys, (const u32*)SV[sv], tied, (u32)key_words,
                                   (u32)w, SK[0]);
                rc = radix_sort(L, SRC_PAIRS, nullptr, 0, 0, 0, SK[0], SV[sv], SK[1], SV[sv ^ 1], (u32)tied, make_plan(0, 64), &in_out, &passes);
                if (rc)
                    return rc;
                sv ^= in_out;
            }
            hipLaunchKernelGGL(scatter_u32_kernel, dim3(tblocks), dim3(256), 0, s, (const u32*)SV[sv], (const u32*)tied_pos, tied, m, P[pc],
                               h->counts + 2);
            HIP_TRY(hipGetLastError());
        }
        // sorted: key word 0 in K[kc], the permutation in P[pc]; word 1 follows into the spare key array
        sorted_key1 = K[kc ^ 1];
        hipLaunchKernelGGL(gather_u64_kernel, dim3(blocks), dim3(256), 0, s, c.keys, (const u32*)P[pc], m, (u32)key_words, 1u, sorted_key1);
        hipLaunchKernelGGL(pack_carried_kernel, dim3(blocks), dim3(256), 0, s, c.suf40, c.beta, m, carried);
        sorted_words = pl.at<u64>(40); // (lanes and tags in are dead: the records hold them)
        if (key_words == 2) {
            tp.beta_r = P[pc]; // the ranking compares words 0 and 1 from the sorted columns: the permutation is dead by then
        } else {
            tp.beta_r = pl.at<u32>(48);
            perm = P[pc]; // words 2 and 3 are compared through the permutation where words 0 and 1 tie
        }
    }
    u32* sorted_beta = P[pc ^ 1];
    hipLaunchKernelGGL(gather_carried_kernel, dim3(blocks), dim3(256), 0, s, (const uint4*)carried, (const u32*)P[pc], m, sorted_words,
                       sorted_beta);
    HIP_TRY(hipGetLastError());
    return finish_partition_step<true>(L, who, c, tp, K[kc], sorted_key1, perm, key_words, sorted_words, sorted_beta, m,
                                       4ull * (u64)key_words, p, res);
}

// Generation t >= 1 of a partition's active set of m > 0 suffixes, laid out by `pl`.
int step_rerank(Launch& L, const char* who, StepColumns& c, const StepPlan& pl, u64 m, u64 ctx, u32 p, csa_step_result* res)
{
    csa_handle* h = L.h;
    hipStream_t s = L.stream;
    const u32 blocks = (u32)((m + 255) / 256);
    HIP_TRY(hipMemsetAsync(h->counts, 0, 8 * sizeof(u32), s));
    u32* P[2] = {pl.at<u32>(16), pl.at<u32>(20)};
    // 1. the join (src/GPU_SACA.cu:1769-1835): the cohort stays in the order it came in; its suffixes go into a hash
    //    table, the messages probe it and leave their rank words at the recipients' list places
    u32* sec = pl.at<u32>(8);
    u64* keys = pl.at<u64>(24);
    HIP_TRY(hipMemsetAsync(sec, 0xFF, m * sizeof(u32), s));
    int rc;
    if (c.inbox_sz) {
        unsigned long long* table = pl.at<unsigned long long>(21);
        u32* place_of = pl.at<u32>(35);
        u64 slots = pl.unit + pl.unit / 2 + pl.unit / 4; // 14 bytes per unit of slots, 7 of places
        if (slots > 2 * m + 64)
            slots = 2 * m + 64;
        HIP_TRY(hipMemsetAsync(table, 0xFF, slots * sizeof(unsigned long long), s));
        hipLaunchKernelGGL(join_table_insert_kernel, dim3(blocks), dim3(256), 0, s, c.suf40, m, table, place_of, slots, h->counts + 2);
        hipLaunchKernelGGL(join_table_probe_kernel, dim3((c.inbox_sz + 255u) / 256u), dim3(256), 0, s, c.inbox_target, c.inbox_rank,
                           c.inbox_sz, (const unsigned long long*)table, (const u32*)place_of, slots, sec);
    }
    // 2. composite keys: primary << 31 | received rank, all ones where nothing arrived (src/GPU_SACA.cu:1803-1835)
    hipLaunchKernelGGL(compose_join_keys_kernel, dim3(blocks), dim3(256), 0, s, c.rank_in, (const u32*)sec, m, keys);
    HIP_TRY(hipGetLastError());
    // 3. sort by (primary, secondary): key bits [0, 62) (src/GPU_SACA.cu:1841-1871)
    u64* keys_partner = pl.at<u64>(32);
    hipLaunchKernelGGL(iota_kernel, dim3(blocks), dim3(256), 0, s, P[0], m);
    int in_out = 0, passes = 0;
    rc = radix_sort(L, SRC_PAIRS, nullptr, 0, 0, 0, keys, P[0], keys_partner, P[1], (u32)m, make_plan(0, 62), &in_out, &passes);
    if (rc)
        return rc;
    const u64* sorted_keys = in_out ? keys_partner : keys;
    u64* sorted_words = in_out ? keys : keys_partner;
    const u32* perm = P[in_out];
    u32* sorted_beta = P[in_out ^ 1];
    hipLaunchKernelGGL(gather_lanes_kernel, dim3(blocks), dim3(256), 0, s, c.suf40, perm, m, sorted_words);
    hipLaunchKernelGGL(gather_u32_kernel, dim3(blocks), dim3(256), 0, s, c.beta, perm, m, sorted_beta);
    HIP_TRY(hipGetLastError());
    // 4. refine, split, messages, narrow
    TailPlaces tp;
    tp.key_r = pl.at<u64>(0);
    tp.words_r = pl.at<u64>(8);
    tp.beta_r = P[in_out]; // the permutation is dead once the carried columns are gathered
    tp.msg_target = pl.at<u8>(24);
    tp.msg_rank = pl.at<u32>(34);
    tp.rank_out = pl.at<u32>(16);
    tp.suf40_out = pl.at<u8>(42);
    return finish_partition_step<false>(L, who, c, tp, sorted_keys, nullptr, nullptr, 1, sorted_words, sorted_beta, m, ctx, p, res);
}

} // namespace

extern "C" {

uint64_t csa_step_bytes_per_suffix(int key_words)
{
    const u32 init = step_plan_init(key_words < 1 ? 1 : key_words > 4 ? 4 : key_words);
    return init > STEP_PLAN_RERANK ? init : STEP_PLAN_RERANK;
}

int csa_sort_init_dev(csa_handle* h, const uint64_t* d_keys, int key_words, const uint8_t* d_suf40, const uint32_t* d_beta,
                      uint64_t m, uint32_t p, uint32_t* d_rank_out, uint8_t* d_suf40_out, uint8_t* d_msg_target,
                      uint32_t* d_msg_rank, uint32_t* d_msg_off, void* stream, csa_step_result* res)
{
    const char* who = "csa_sort_init_dev";
    if (key_words < 1 || key_words > 4)
        return fail(CSA_ERR_ARG, "%s: key_words = %d is outside [1, 4]", who, key_words);
    int rc = check_step_args(h, who, m, p, d_keys, d_suf40, d_beta, d_msg_off);
    if (rc)
        return rc;
    h->last_step = csa_step_result{};
    if (res)
        *res = h->last_step;
    if (m == 0) {
        HIP_TRY(hipMemsetAsync(d_msg_off, 0, ((u64)p + 1) * sizeof(u32), (hipStream_t)stream));
        return CSA_OK;
    }
    if (!d_rank_out || !d_suf40_out || !d_msg_target || !d_msg_rank)
        return fail(CSA_ERR_ARG, "%s: null output buffer", who);
    Launch L;
    L.h = h;
    L.stream = (hipStream_t)stream;
    L.flags = 0;
    L.stats = nullptr;
    StepColumns c;
    c.keys = d_keys;
    c.suf40 = d_suf40;
    c.beta = d_beta;
    c.rank_out = d_rank_out;
    c.suf40_out = d_suf40_out;
    c.msg_target = d_msg_target;
    c.msg_rank = d_msg_rank;
    c.msg_off = d_msg_off;
    StepPlan pl;
    rc = step_plan(h, who, m, step_plan_init(key_words), &pl);
    if (rc)
        return rc;
    return step_init(L, who, c, pl, key_words, m, p, res);
}

int csa_sort_rerank_dev(csa_handle* h, const uint32_t* d_rank, const uint8_t* d_suf40, const uint32_t* d_beta, uint64_t m,
                        const uint8_t* d_inbox_target, const uint32_t* d_inbox_rank, uint32_t inbox_sz, uint64_t ctx,
                        uint32_t p, uint32_t* d_rank_out, uint8_t* d_suf40_out, uint8_t* d_msg_target, uint32_t* d_msg_rank,
                        uint32_t* d_msg_off, void* stream, csa_step_result* res)
{
    const char* who = "csa_sort_rerank_dev";
    int rc = check_step_args(h, who, m, p, d_rank, d_suf40, d_beta, d_msg_off);
    if (rc)
        return rc;
    h->last_step = csa_step_result{};
    if (res)
        *res = h->last_step;
    if (m == 0) {
        HIP_TRY(hipMemsetAsync(d_msg_off, 0, ((u64)p + 1) * sizeof(u32), (hipStream_t)stream));
        return CSA_OK;
    }
    if (!d_rank_out || !d_suf40_out || !d_msg_target || !d_msg_rank || (inbox_sz && (!d_inbox_target || !d_inbox_rank)))
        return fail(CSA_ERR_ARG, "%s: null buffer", who);
    Launch L;
    L.h = h;
    L.stream = (hipStream_t)stream;
    L.flags = 0;
    L.stats = nullptr;
    StepColumns c;
    c.rank_in = d_rank;
    c.suf40 = d_suf40;
    c.beta = d_beta;
    c.inbox_target = d_inbox_target;
    c.inbox_rank = d_inbox_rank;
    c.inbox_sz = inbox_sz;
    c.rank_out = d_rank_out;
    c.suf40_out = d_suf40_out;
    c.msg_target = d_msg_target;
    c.msg_rank = d_msg_rank;
    c.msg_off = d_msg_off;
    StepPlan pl;
    rc = step_plan(h, who, m, STEP_PLAN_RERANK, &pl);
    if (rc)
        return rc;
    return step_rerank(L, who, c, pl, m, ctx, p, res);
}

int csa_last_step_result(const csa_handle* h, csa_step_result* out)
{
    if (!h || !out)
        return fail(CSA_ERR_ARG, "csa_last_step_result: null handle or result pointer");
    *out = h->last_step;
    return CSA_OK;
}

uint64_t csa_scratch_high_water(const csa_handle* h) { return h ? h->last_high_water : 0; }

} // extern "C"
