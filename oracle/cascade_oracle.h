/*
 * CPU oracle for the per-partition suffix sort: TEST INFRASTRUCTURE ONLY.
 *
 * Nothing here is part of the product. Only the test suite, the smoke check and the
 * CPU-baseline leg of the benchmark may link or call it, and only as the checker.
 * Every function restates a piece of the reference (saltsystemslab/Cascade) in plain C;
 * the file:line each one follows is given beside its declaration.
 *
 * How each function is pinned (what a plausible mistake would trip over):
 *   orc_cmp_suffixes / orc_build_sa40_u16 : the reference's own known answers and hand cases
 *       (src/test_query.cu:374-392,405-411), closed forms (a^n, increasing, decreasing,
 *       (ab)^k, Fibonacci word), the zero-tail corner case (dataset/make-corner-case.py:37),
 *       and byte-for-byte equality with the reference's compiled build_sa40 where the
 *       _ref library builds.
 *   orc_is_correct_sa_u16 : accepts exactly the SA of build_sa40 and rejects a swapped
 *       pair, an out-of-range entry, a repeated entry and the byte-order SA
 *       (the negative controls of src/test_query.cu:417-454).
 *   orc_pack_word_u16 / orc_pack_prefix_u16 : closed form (4-term shift/or) and the order
 *       invariant key(i) < key(j) <=> T[i..i+4) <lex T[j..j+4).
 *   orc_fwd_tag : closed form, and the tail-order property it exists for.
 *   orc_prefix_doubling_u16 : final order equals orc_build_sa40_u16 on every fixture;
 *       per-generation active counts equal orc_retire_generations (an independent
 *       closed form over SA + LCP, src/sa_structure.cpp:295-306,375) and, where the
 *       reference tree is present, the retirements that the reference's own
 *       src/sa_structure.cpp, compiled into _ref/sa_structure, predicts from the finished
 *       array, for key widths of 1 to 4 words.
 *   orc_sa40_store / orc_sa40_load : round trip (src/test_query.cu:78-96) and explicit bytes;
 *       the file of orc_build_sa40_u16 passes the reference's own tools/sa_convert.cpp
 *       (compiled into _ref/sa_convert: sizes, order spot check, index.meta) and widens
 *       through it to the 64-bit array.
 */
#ifndef CASCADE_ORACLE_H
#define CASCADE_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_SA_WIDTH 5        /* include/sa40.hpp:24 */
#define ORC_SA_PAD_BYTES 128  /* include/sa40.hpp:37 */

/* include/CPU_Reference.hpp:107-123. Order of suffixes i and j of T[0,n), at most max_cmp symbols. */
int orc_cmp_suffixes_u16(const uint16_t* T, uint64_t n, uint64_t i, uint64_t j, uint64_t max_cmp);

/* include/sa40.hpp:72-75 and :46-60 (host branch). */
void orc_sa40_store(uint8_t* SA, uint64_t r, uint64_t v);
uint64_t orc_sa40_load(const uint8_t* SA, uint64_t r);

/* test/query.cpp:42-55. Comparison sort of all suffixes; SA must hold 5*n + ORC_SA_PAD_BYTES bytes
 * (the pad is zero-filled like the reference's). */
void orc_build_sa40_u16(const uint16_t* T, uint64_t n, uint8_t* SA);

/* test/end-to-end.cpp:13-43 and :46-80. sa is 8-byte entries. Returns 1 if correct. */
int orc_is_permutation(const uint64_t* sa, uint64_t n);
int orc_is_correct_sa_u16(const uint64_t* sa, const uint16_t* T, uint64_t n);
/* Same check over 5-byte lanes (test/end-to-end.cpp:99-116 widens them first). */
int orc_is_correct_sa40_u16(const uint8_t* sa40, const uint16_t* T, uint64_t n);

/* include/utility.hpp:147-162: four u16 symbols MSB-first in one word. T must be readable for 4 symbols. */
uint64_t orc_pack_word_u16(const uint16_t* T);
/* include/Packed_Prefix.hpp:91-104 over a text whose tail is padded with zeros (src/GPU_SACA.cu:223-236):
 * words[w] for w in [0,key_words) of suffix j; positions >= n read as 0. */
void orc_pack_prefix_u16(const uint16_t* T, uint64_t n, uint64_t j, int key_words, uint64_t* words);

/* include/bit-layout.hpp:99-100 with a single partition (id == 0): tag of suffix j whose
 * next-generation source is tgt = j + ell. */
uint64_t orc_fwd_tag(uint64_t tgt, uint64_t n, uint64_t ell);

/* The path restated for one partition holding the whole text:
 * gen 0 = sort by (packed key, fwd tag), rank = head offset of the run, active = run length > 1
 * (include/GPU_SACA.cuh:191-208, src/GPU_SACA.cu:1165-1247); generation t >= 1 sorts the active set by
 * (rank(x), rank(x + ell*2^(t-1))) and refines rank += head(key run) - head(primary run)
 * (include/GPU_SACA.cuh:218-280, src/GPU_SACA.cu:1841-1925); loop of src/GPU_SACA.cu:1999-2103;
 * output SA[rank(j)] = j (include/GPU_SACA.cuh:167-182).
 * sa_out: n entries. active_counts[g] = suffixes active entering generation g (g = 0 -> n), up to
 * max_gens entries; returns the number of generations run (including generation 0). */
int orc_prefix_doubling_u16(const uint16_t* T, uint64_t n, int key_words, uint64_t* sa_out,
                            uint64_t* active_counts, int max_gens);

/* src/sa_structure.cpp:295-306,375 with one partition: retirement generation d(j) of every suffix from
 * the finished SA and brute-force LCPs. d_out[j] in [0, 63]. O(n * lcp): small inputs only. */
void orc_retire_generations_u16(const uint16_t* T, uint64_t n, const uint64_t* sa, uint64_t ell, uint8_t* d_out);

/* Stable LSD restatements used to check the device primitives at their boundary
 * (the CUB contracts the reference relies on, src/GPU_SACA.cu:1175-1210,1241-1261). */
void orc_stable_sort_pairs_u64_u32(uint64_t* keys, uint32_t* vals, uint64_t n, int begin_bit, int end_bit);

/* ---- partition ids (the step before the partition sort) ---- */

/* include/Partition_ID_Map.hpp:79 with util::math::bits_for (include/utility.hpp:118-121): bits per map entry. */
uint32_t orc_partition_id_bits(uint32_t p);
/* test/partitioning.cpp:12-39 (= the search of include/GPU_SACA.cuh:52-66) over a zero-padded text: pid[i] = the smallest
 * q with key(i) <= pivots[q] (word-wise, include/Packed_Prefix.hpp:122-135), p - 1 if none; key(i) = `words` packed words
 * of suffix i, positions >= text_len read as 0. psz[q] (p counters, may be NULL) is incremented per suffix
 * (include/GPU_SACA.cuh:69). */
void orc_partition_ids_u16(const uint16_t* T, uint64_t n, uint64_t text_len, const uint64_t* pivots, int words, uint32_t p,
                           uint16_t* pid, uint64_t* psz);
/* include/Partition_ID_Map.hpp:158-177 applied to each group of 64 suffixes as include/GPU_SACA.cuh:82-91 does:
 * group g fills words [g * bits, ...), least significant bits first; a trailing partial group writes
 * ceil(sz * bits / 64) words. `out` must hold ceil(n / 64) * bits words; words not written are left alone. */
void orc_pack_partition_ids(const uint16_t* pid, uint64_t n, uint32_t bits, uint64_t* out);
/* include/Partition_ID_Map.hpp:180-189: the id of suffix i read back from the packed words. */
uint16_t orc_partition_id_map_get(const uint64_t* words, uint32_t bits, uint64_t i);

/* src/GPU_SACA.cu:1674-1691 (GPU_SACA::stage_slab without the spilled-map branch) with include/bit-layout.hpp:99-100,
 * 137-152: keys (generation 0, may be NULL) and routing-tag pairs of `count` suffix lanes. pid[x] and retired[x]
 * (one byte each, 0/1) describe every text position x in [0, n). */
void orc_stage_slab_u16(const uint16_t* T, uint64_t n, const uint8_t* suf40, uint64_t count, int key_words,
                        const uint16_t* pid, const uint8_t* retired, uint64_t ctx, int generation0, uint64_t* keys,
                        uint32_t* beta);

/* ---- rank messages (include/GPU_SACA.cuh:283-389, include/message.hpp:20-52, include/bit-layout.hpp:57,115-152) ---- */

/* The up to two messages of cohort member i: out = {dest, target, rank} of the payload, then of the forwarded pill;
 * dest = 0xFFFFFFFF where there is none (include/GPU_SACA.cuh:334-352). */
void orc_messages_of(uint64_t sa_word, uint64_t key, uint32_t beta, uint64_t i, uint64_t active_sz, uint64_t ctx, int packed,
                     uint64_t out[6]);
/* include/GPU_SACA.cuh:291-308: msg_count[q] += messages to partition q. */
void orc_count_messages(const uint64_t* sa, const uint64_t* keys, const uint32_t* beta, uint64_t n, uint64_t ctx, int packed,
                        uint32_t* msg_count);
/* include/GPU_SACA.cuh:321-353, run sequentially: slot = msg_off[dest]++ in list order (payload before pill). */
void orc_emit_messages(const uint64_t* sa, const uint64_t* keys, const uint32_t* beta, uint64_t n, uint64_t ctx, int packed,
                       uint64_t active_sz, uint8_t* msg_target, uint32_t* msg_rank, uint32_t* msg_off);
/* include/GPU_SACA.cuh:362-389. */
void orc_join_messages(const uint8_t* msg_target, const uint32_t* msg_rank, uint32_t msg_c, const uint64_t* sa,
                       const uint32_t* primary, uint64_t* keys, uint64_t n);

/* ---- after the partition sort ---- */

/* include/GPU_SACA.cuh:167-182 followed by :126-133: out lane[rank[i]] = lane i of suf (5-byte lanes, include/lane.hpp:51-79).
 * Returns 0, or -1 if some rank[i] >= n (the reference traps there under -DTESTS). */
int orc_scatter_to_rank_order(const uint8_t* suf, const uint32_t* rank, uint64_t n, uint8_t* out);
/* src/Output_File.cpp:18-35: how the byte range [lo, hi) of a partition's output is shared out over chunk_c chunks of
 * chunk_bytes so that all but the edges are whole 4 KiB blocks. out = {piece lo, hi, head lo, hi, tail lo, hi}. */
void orc_output_cut(uint64_t lo, uint64_t hi, uint64_t chunk_bytes, uint64_t c, uint64_t chunk_c, uint64_t out[6]);

#ifdef __cplusplus
}
#endif
#endif
