/*
 * cascade_hip.h : C ABI of the MI355X (gfx950) per-partition suffix sort.
 *
 * One partition's suffixes are sorted entirely in HBM by prefix doubling and leave as a
 * suffix array of 5-byte little-endian entries ("sa40"), in the reference's order: numeric
 * symbol order, the shorter suffix first, no sentinel.
 *
 * Every entry point returns 0 on success and a negative csa_status otherwise; nothing here
 * ever exits the process. csa_last_error() describes the last failure of the calling thread.
 * Pointers named d_* are device (HBM) addresses, h_* are host addresses. `stream` is a
 * hipStream_t passed as void* (NULL = the default stream). A handle owns all device scratch
 * memory and serves one call at a time; use one handle per stream for concurrent partitions.
 *
 * Entry points that take a handle, and csa_pack_keys_u16_dev, return after the stream has finished
 * (they read counters back). csa_partition_ids_u16_dev, csa_stage_slab_u16_dev, csa_count_messages_dev,
 * csa_message_offsets_dev, csa_emit_messages_dev and csa_join_messages_dev only enqueue kernels on the
 * stream and allocate nothing.
 */
#ifndef CASCADE_HIP_H
#define CASCADE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CSA_MAX_GENERATIONS 64

/* Largest partition: local ranks are 31-bit (reference: include/bit-layout.hpp:51-68, MAX_PART_SZ). */
#define CSA_MAX_PART_SZ 2147483647ull
/* Largest suffix index a 5-byte lane holds (reference: include/sa40.hpp:24-27, include/bit-layout.hpp:32,47). */
#define CSA_MAX_INDEX (1ull << 40)

typedef enum csa_status {
    CSA_OK = 0,
    CSA_ERR_ARG = -1,       /* null pointer, bad key_words, n beyond the handle's capacity */
    CSA_ERR_TOO_LARGE = -2, /* n > CSA_MAX_PART_SZ or index_base + n > CSA_MAX_INDEX */
    CSA_ERR_HIP = -3,       /* a HIP runtime call failed (out of memory included) */
    CSA_ERR_INTERNAL = -4   /* a device-side invariant failed (look-back spin limit, generation cap) */
} csa_status;

/* Flags of csa_sort_partition_u16_dev. */
#define CSA_FLAG_KERNEL_TIMING 1u /* bracket every radix-pass launch with events (fills the radix_* stats) */

typedef struct csa_stats {
    uint64_t n;
    int32_t key_words;
    int32_t generations;                  /* generations run, generation 0 included */
    uint64_t active[CSA_MAX_GENERATIONS]; /* suffixes active entering generation g; active[0] = n */
    uint64_t groups[CSA_MAX_GENERATIONS]; /* unresolved groups entering generation g (0 for g = 0) */
    uint64_t big[CSA_MAX_GENERATIONS];    /* of active[g], members of groups too large for the in-tile sort */
    int32_t passes[CSA_MAX_GENERATIONS];  /* radix passes run in generation g (over the large groups for g > 0) */
    int32_t rank_update[CSA_MAX_GENERATIONS]; /* how generation g wrote its ranks: 0 scattered from the rank pass,
                                                 1 bucketed by two passes into LDS-sized windows (generation 0),
                                                 2 bucketed by one pass into cache-sized windows */
    int32_t small_only[CSA_MAX_GENERATIONS];  /* 1: generation g held small groups only and ran as two fused kernels
                                                 (in-tile sort + ranking + counting, then apply) without a radix sort */
    int32_t dense[CSA_MAX_GENERATIONS];       /* 1: generation g > 0 sorted the whole partition again by (rank[x], rank[x + h])
                                                 read in text order (most suffixes still active, in long groups) */
    float ms[CSA_MAX_GENERATIONS];        /* device time of generation g */
    float ms_output;                      /* sa40 emission */
    float ms_total;                       /* first kernel to last kernel, on the stream */
    /* with CSA_FLAG_KERNEL_TIMING: the radix-pass kernel, summed over all its launches */
    uint64_t radix_launches;
    uint64_t radix_pairs; /* (key, index) pairs moved, summed over launches */
    double radix_ms;
    uint64_t presorted[CSA_MAX_GENERATIONS]; /* of big[g], members that skipped the radix sort: every large group of the
                                                list was in order of rank[x + h] already (rising or falling along the
                                                list, as in runs of one token and periodic stretches) */
    uint32_t key_symbols;            /* symbols the first sort resolved: 4 (one K-gram word), or up to 64 when the text's
                                        alphabet is small enough for packed codes of 1, 2, 4 or 8 bits */
    uint32_t first_sort_generations; /* generations of the reference that sort stands for: 1, or 1 + j when its keys held
                                        4 * key_words * 2^j symbols. Generations 1 .. j are then reported with the lists
                                        they would have had (active[], groups[]) and with no time or passes of their own */
} csa_stats;

typedef struct csa_handle csa_handle;

/* ---- sizing: what a handle holds on the device ----
 * A handle owns one block of device memory that scales with its capacity, and a workspace that follows the number of
 * tiles (look-back words, per-tile tables, digit counts, the outbox counters). Both are allocated by csa_create /
 * csa_create_steps and nothing is allocated afterwards: every entry point that takes a handle works inside them.
 * Replaces the sizing of the reference's GPU_SACA::partition_size_upper_bound / allocate_device_space / cub_workspace_size
 * (include/GPU_SACA.hpp:209,217,221; src/GPU_SACA.cu:365-380,457-531,535-590), whose floor plan is
 * 2 * (max(8 * key_words, 16) + 8 + 4 + 4) + 1 = 65 / 65 / 81 / 97 bytes per suffix for key_words = 1 / 2 / 3 / 4. */

/* Block bytes per suffix of a handle made by csa_create (text and output excluded): the floor plan of the sort that
 * keeps the partition resident, 60 whatever the key width. Such a handle serves every entry point; the per-generation
 * steps find room in it for partitions of up to capacity * 60 / csa_step_bytes_per_suffix(key_words) suffixes. */
uint64_t csa_bytes_per_suffix(int key_words);

/* Block bytes per suffix of a handle made by csa_create_steps: what the per-generation steps (csa_sort_init_*,
 * csa_sort_rerank_*, csa_scatter_*), their slab-shaped forms included, need for a partition, inputs and outputs on the
 * device included: 48 with one-word keys, 65 with two words, 8 * key_words + 52 = 76 / 84 with three / four.
 * Every column of a step has a fixed place in the block and columns whose lives do not overlap share a place, which is
 * how the reference reaches its own figure (src/GPU_SACA.cu:1268-1270,1292,1301,1805-1806). */
uint64_t csa_step_bytes_per_suffix(int key_words);

/* Bytes of the workspace of a handle for partitions of up to max_part_sz suffixes, rounding slack of the block
 * included (about 0.3 bytes per suffix plus 0.6 MB): what a host adds per handle when it sizes partitions against free
 * device memory, as the reference adds cub's workspace (src/GPU_SACA.cu:385-403). */
uint64_t csa_workspace_bytes(uint64_t max_part_sz);

/* Allocates block and workspace for partitions of up to max_part_sz suffixes on the current device; fails with
 * CSA_ERR_HIP if the device has no room (nothing stays allocated then).
 * key_words: 64-bit words of the generation-0 key, 1 to 4 (4 to 16 uint16 symbols; the reference's
 * PREF_KEY_WORDS, include/Packed_Prefix.hpp:20-24, whose default is 4). The suffix array does not depend on it,
 * only the number of generations and their sizes do; for csa_sort_partition_u16_dev every width costs the same time
 * (wide keys are resolved by doubling steps on one-word keys, which are reported as generation 0).
 * Replaces GPU_SACA::allocate_device_space (src/GPU_SACA.cu:535-590). */
int csa_create(uint64_t max_part_sz, int key_words, csa_handle** out);

/* The same for a host pipeline that drives partitions through the per-generation steps only, one handle per
 * dispatcher thread (STREAM_C of them, include/GPU_SACA.hpp:90-91): the block is csa_step_bytes_per_suffix(key_words)
 * per suffix and csa_sort_partition_u16_dev refuses the handle. Every other entry point works on it. */
int csa_create_steps(uint64_t max_part_sz, int key_words, csa_handle** out);

/* Bytes of the block that the last call on this handle held at its busiest moment (0 for the resident sort, whose
 * carve-up is fixed). For tests and for sizing; the reference prints its device-memory high-water mark the same way
 * (include/utility.cuh:68-131). */
uint64_t csa_scratch_high_water(const csa_handle* h);

/* Declares whether calls on this handle have the device to themselves (exclusive != 0): no other handle, stream or
 * process launches work on it while such a call runs. Only then may the radix passes number their tiles by
 * workgroup index in XCD-sized chunks (about 1.5% faster on the 1B-token workload): that order waits for workgroups
 * which are dispatched later and needs up to 128 workgroups of a pass resident together, which launches that share the
 * device do not guarantee; an unfulfilled wait ends in CSA_ERR_INTERNAL ("look-back wait ran into its spin limit"),
 * not in a hang. The default (0) numbers tiles by arrival and is safe next to any other work, e.g. the three
 * dispatcher threads of the reference (STREAM_C, include/GPU_SACA.hpp:90-91), each with a handle of its own.
 * No counterpart in the reference (CUB's passes always number tiles by arrival). */
int csa_set_device_exclusive(csa_handle* h, int exclusive);

/* Thresholds that choose between equivalent ways of doing a step (the results are the same either way); for tests
 * that want a path taken at small sizes and for measurements. The defaults are the measured best on MI355X.
 *   CSA_TUNE_DEFER_MIN           smallest list whose generation-0 ranks are written through the two-pass bucketed update
 *                                (default 2^23 suffixes)
 *   CSA_TUNE_WINDOW_MIN_CHANGED  fewest changed ranks for the windowed update of later generations (default 2^22;
 *                                0xFFFFFFFF: never)
 *   CSA_TUNE_XCD_CHUNK           tiles (of 8192 pairs) that one XCD takes in a row under csa_set_device_exclusive
 *                                (default 16; 0: the exclusive order is the default order); call before
 *                                csa_set_device_exclusive. 8 chunks of that many workgroups must be resident
 *                                together with room to spare: values above compute units / 16 fail with CSA_ERR_ARG
 *   CSA_TUNE_PACK_SYMBOLS        1 (default): a text whose symbols take at most 256 values (by the values its low and its
 *                                high bytes take) is sorted first on keys of as many packed symbols as 64 bits hold, which
 *                                covers the first generations of the doubling (csa_stats.first_sort_generations); 0: the
 *                                first sort always takes one K-gram word
 *   CSA_TUNE_EXPECT_PRESORTED    0 (default): a generation leaves out the (key, suffix) pairs of its large groups' radix sort
 *                                when every large group of the generation before was in order as it stood (csa_stats.presorted),
 *                                and gathers again with them if this one's are not; 1: every generation starts that way
 *                                (tests of the second gather)
 * No counterpart in the reference. */
enum {
    CSA_TUNE_DEFER_MIN = 0,
    CSA_TUNE_WINDOW_MIN_CHANGED = 1,
    CSA_TUNE_XCD_CHUNK = 2,
    CSA_TUNE_PACK_SYMBOLS = 3,
    CSA_TUNE_EXPECT_PRESORTED = 4
};
int csa_set_tuning(csa_handle* h, int knob, uint32_t value);

/* Frees everything the handle owns (reference: the destructor, src/GPU_SACA.cu:103-120). */
void csa_destroy(csa_handle* h);

/* Sorts the partition d_text[0, n) (uint16 symbols, no padding required) and writes its suffix
 * array as n 5-byte little-endian entries to d_sa40 (5 * n bytes; entry = index_base + position).
 * All generations run in HBM without host round trips of data; the call returns after the
 * stream has finished. Replaces, for a partition resident in HBM, the sequence
 * sort_and_init_rank_and_filter -> sort_and_re_rank_and_filter per generation -> scatter_to_rank_order
 * (include/GPU_SACA.hpp:272,279,288; src/GPU_SACA.cu:1112-1331,1715-1995,1999-2103,2107-2164)
 * and emits the layout of include/lane.hpp:69-79 / include/sa40.hpp:72-75. */
int csa_sort_partition_u16_dev(csa_handle* h, const uint16_t* d_text, uint64_t n, uint64_t index_base,
                               uint8_t* d_sa40, void* stream, uint32_t flags, csa_stats* stats);

/* Convenience for host buffers: creates a handle, copies the text in, sorts, copies the sa40 out
 * (5 * n bytes), destroys the handle. What `cascade <text> <sa>` does for one partition
 * (src/main.cu:12-46 -> GPU_SACA::build_SA, src/GPU_SACA.cu:125-216). */
int csa_sort_partition_u16(const uint16_t* h_text, uint64_t n, int key_words, uint8_t* h_sa40, csa_stats* stats);

/* The same for `count` independent partitions in host memory, pipelined: one handle sized for the largest of them, two
 * sets of device buffers, four streams (one up, one for the sort, two down). While partition k is sorted, the text of partition k + 1 is uploaded and the
 * suffix array of partition k - 1 is downloaded (an upload thread and a download thread beside the calling one), which is
 * how the reference's three dispatcher threads overlap transfers and device work (src/GPU_SACA.cu:1539-1589).
 * h_texts[k]: n[k] symbols; h_sa40[k]: room for 5 * n[k] bytes; index_base (may be NULL = all zero): the suffix index of
 * each partition's first symbol; stats (may be NULL): `count` records. Pinned host buffers (hipHostMalloc) transfer at the
 * link's rate and overlap fully; pageable ones work, staged by the runtime. The call returns when everything is back. */
int csa_sort_partitions_u16(uint32_t count, const uint16_t* const* h_texts, const uint64_t* n, const uint64_t* index_base,
                            int key_words, uint8_t* const* h_sa40, csa_stats* stats);

/* ---- the stages, exposed one by one so each can be checked against its CPU restatement ---- */

/* K-gram key packing: d_keys[j * key_words + w] = symbols [j + 4w, j + 4w + 4) of the zero-padded text,
 * first symbol in the most significant bits (reference: util::pack_word, include/utility.hpp:147-162;
 * Packed_Prefix::pack_prefix, include/Packed_Prefix.hpp:91-104; host loop src/GPU_SACA.cu:1674-1684). */
int csa_pack_keys_u16_dev(const uint16_t* d_text, uint64_t n, int key_words, uint64_t* d_keys, void* stream);

/* Stable LSD radix sort of (64-bit key, 32-bit value) pairs on key bits [begin_bit, end_bit); the sorted
 * pairs are left in d_keys / d_vals. Uses the handle's scratch (n <= its capacity).
 * Replaces cub::DeviceRadixSort::SortPairs (src/GPU_SACA.cu:1175-1181,1203-1210,1783-1789,1849-1855). */
int csa_radix_sort_pairs_dev(csa_handle* h, uint64_t* d_keys, uint32_t* d_vals, uint64_t n, int begin_bit,
                             int end_bit, void* stream);

/* The same sort for callers that cannot allocate (code recorded into a HIP graph, serving loops and harnesses that
 * forbid hipMalloc): no handle, no hipMalloc / hipFree / allocating library routine, no host round trip. The call only
 * enqueues kernels on the stream (no memset or copy nodes) and returns; the sorted pairs are in d_keys / d_vals when the
 * stream has finished. Its scratch (the ping-pong partners of the two arrays, look-back words, digit counts) is a
 * fixed array inside the library's code object, which every device that loads the library holds until the process
 * ends: 8 * CSA_STATIC_SORT_MAX_PAIRS + 4 * CSA_STATIC_SORT_MAX_PAIRS bytes of pairs + 2.3 MB of control words, 14.3 MB
 * in all. n > CSA_STATIC_SORT_MAX_PAIRS fails with CSA_ERR_TOO_LARGE. All calls on one device share that one array:
 * calls that overlap on a device (two streams, two threads) race; serialise them. Every pass of the bit range runs
 * (passes over a constant digit are not skipped: that needs the counts on the host). A failure on the device is not
 * reported by this call: ask csa_radix_sort_pairs_static_status afterwards. The stream's device must be the
 * current one. The first call on a device looks the array's address up (hipGetSymbolAddress); make that call, with
 * n = 0 if need be, before any stream capture begins.
 * No counterpart in the reference (its sorts go through cub's workspace, allocated once by allocate_device_space). */
#ifndef CSA_STATIC_SORT_MAX_PAIRS
#define CSA_STATIC_SORT_MAX_PAIRS (1u << 20)
#endif
int csa_radix_sort_pairs_static_dev(uint64_t* d_keys, uint32_t* d_vals, uint64_t n, int begin_bit, int end_bit, void* stream);

/* csa_radix_sort_pairs_static_dev cannot report a failure on the device (it returns before its kernels run): a
 * look-back wait that runs into its spin limit makes the remaining workgroups leave, and the pairs are then not sorted.
 * This call waits for the stream and returns CSA_ERR_INTERNAL if the last such sort on the current device ended that
 * way, CSA_OK otherwise. It copies one word to the host and allocates nothing; not for use inside a stream capture
 * (ask after the graph's launch has finished). No counterpart in the reference. */
int csa_radix_sort_pairs_static_status(void* stream);

/* O(n) suffix-array check on the device: d_sa40 is a permutation of [index_base, index_base + n) and every
 * adjacent pair is in order (first symbols, then ranks of the successors; a successor past the end sorts
 * first). *ok = 1 if correct. Same rule as the reference's validator (test/end-to-end.cpp:13-80). */
int csa_verify_sa40_dev(csa_handle* h, const uint16_t* d_text, uint64_t n, uint64_t index_base,
                        const uint8_t* d_sa40, void* stream, int* ok);

/* ---- the step before the partition sort: which partition does every suffix belong to ---- */

/* Bits per entry of the packed partition-id map for p partitions: the id's bits, then one retirement flag
 * (reference: Partition_ID_Map::bits_for, include/Partition_ID_Map.hpp:79). */
uint32_t csa_partition_id_bits(uint32_t p);

/* For every suffix i in [0, n) of d_text: id(i) = the smallest q with K-gram(i) <= pivot[q], or p - 1 if there is
 * none, where K-gram(i) is the first 4 * pivot_words symbols of the suffix, zero padded past d_text[text_len).
 * d_pivots: (p - 1) * pivot_words 64-bit words, most significant symbols first, ascending (the reference's Pivot_Key,
 * include/Packed_Prefix.hpp:26-34,88); pivot_words 1..4; p <= 65536.
 * Any of the three outputs may be NULL:
 *   d_pid    : n uint16 ids;
 *   d_packed : the ids bit-packed like Partition_ID_Map::pack (include/Partition_ID_Map.hpp:158-177),
 *              csa_partition_id_bits(p) words per 64 suffixes, ceil(n * bits / 64) words for a trailing partial group;
 *   d_psz    : p counters to which the partition sizes are ADDED (zero them before the first chunk of a text).
 * A chunk in the middle of a text passes text_len = n + 4 * pivot_words - 1 so that its last suffixes see the
 * symbols that follow; n must then be a multiple of 64.
 * Replaces compute_partition_IDs_kernel + pack_partition_IDs_kernel (include/GPU_SACA.cuh:23-91) as launched per
 * chunk by GPU_SACA::compute_partition_IDs (src/GPU_SACA.cu:854-1000); same answers as
 * test::validate_partition_IDs (test/partitioning.cpp:12-39). */
int csa_partition_ids_u16_dev(const uint16_t* d_text, uint64_t n, uint64_t text_len, const uint64_t* d_pivots,
                              int pivot_words, uint32_t p, uint16_t* d_pid, uint64_t* d_packed, uint64_t* d_psz,
                              void* stream);

/* Staging of `count` suffixes of a partition (5-byte lanes d_suf40, any order) on the device, for a text and its packed
 * partition-id map (as csa_partition_ids_u16_dev writes it, retirement flags included) resident in HBM:
 *   generation0 != 0 : d_keys[i * key_words + w] = K-gram word w of suffix i (may be NULL to skip), and
 *                      d_beta[i] = route(j - ell) | forward tag(j + ell) << 16, with ell = 4 * key_words = ctx;
 *   generation0 == 0 : d_beta[i] = route(j - ctx) | route(j - ctx / 2) << 16.
 * route(x) = id of x's partition, bit 15 set if x has retired, 0 if x would lie before the text; forward tag = id + ell, or
 * n + ell - 1 - (j + ell) when j + ell is past the end (include/bit-layout.hpp:99-100,137-152).
 * Replaces the host loop of GPU_SACA::stage_slab (src/GPU_SACA.cu:1674-1691) and the upload of 8 * key_words bytes
 * per suffix that follows it (src/GPU_SACA.cu:1129). */
int csa_stage_slab_u16_dev(const uint16_t* d_text, uint64_t n, const uint8_t* d_suf40, uint64_t count, int key_words,
                           const uint64_t* d_pid_map, uint32_t p, uint64_t ctx, int generation0, uint64_t* d_keys,
                           uint32_t* d_beta, void* stream);

/* ---- rank messages between partitions (for partitions sorted one at a time behind the reference's slab interface) ---- */

/* At the end of a generation that resolved ctx symbols, cohort member i (suffix = low 48 bits of d_sa[i], key d_keys[i],
 * routing tags d_beta[i]) sends its rank to suffix - ctx through the partition in the low half of beta, and forwards a
 * received poison pill to suffix - ctx / 2 through the high half; packed_keys = 0: keys are plain ranks (generation 0),
 * 1: primary << 31 | secondary with the pill receipt in bit 62.
 * d_msg_count[q] += messages bound for partition q, q < p.
 * Replaces count_message_destination_distribution_kernel (include/GPU_SACA.cuh:291-308; src/GPU_SACA.cu:1272-1276). */
int csa_count_messages_dev(const uint64_t* d_sa, const uint64_t* d_keys, const uint32_t* d_beta, uint64_t n, uint64_t ctx,
                           int packed_keys, uint32_t p, uint32_t* d_msg_count, void* stream);

/* In-place exclusive prefix sum of `count` <= 32769 counters: the message counts become the groups' start offsets.
 * Replaces the cub::DeviceScan::ExclusiveSum over p + 1 counters (src/GPU_SACA.cu:1278-1283). */
int csa_message_offsets_dev(uint32_t* d_msg_off, uint32_t count, void* stream);

/* Writes those messages, collated by destination: 5-byte target lanes to d_msg_target and ranks to d_msg_rank (MSB =
 * the sender retired in this generation, i.e. its list index is >= *d_active_sz, or the message is a forwarded pill).
 * d_msg_off[q] must hold the exclusive prefix sum of the counts on entry and holds the exclusive end of q's group on
 * return; the order of messages inside a group is arbitrary.
 * Replaces emit_messages_kernel (include/GPU_SACA.cuh:321-353; src/GPU_SACA.cu:1285-1287,1949-1951). */
int csa_emit_messages_dev(const uint64_t* d_sa, const uint64_t* d_keys, const uint32_t* d_beta, uint64_t n, uint64_t ctx,
                          int packed_keys, const uint64_t* d_active_sz, uint32_t p, uint8_t* d_msg_target,
                          uint32_t* d_msg_rank, uint32_t* d_msg_off, void* stream);

/* Delivers msg_c messages to the cohort d_sa[0, n), which is sorted by suffix: for the position pos of each target,
 * d_keys[pos] = d_primary[pos] << 31 | rank, with bit 62 set for a pill; messages whose target is not in the cohort are
 * dropped (the recipient has retired). Replaces join_messages_kernel (include/GPU_SACA.cuh:362-389; src/GPU_SACA.cu:1826-1833). */
int csa_join_messages_dev(const uint8_t* d_msg_target, const uint32_t* d_msg_rank, uint32_t msg_c, const uint64_t* d_sa,
                          const uint32_t* d_primary, uint64_t* d_keys, uint64_t n, void* stream);

/* The same delivery with the handle's scratch: the inbox is first sorted by target (40-bit LSD radix sort inside the
 * handle, msg_c <= its capacity), so that the searches of neighbouring messages walk neighbouring places of the cohort.
 * Same result as csa_join_messages_dev; the inbox itself is left as it was. The call returns after the stream has
 * finished. No counterpart in the reference (it probes in arrival order). */
int csa_join_messages_sorted_dev(csa_handle* h, const uint8_t* d_msg_target, const uint32_t* d_msg_rank, uint32_t msg_c,
                                 const uint64_t* d_sa, const uint32_t* d_primary, uint64_t* d_keys, uint64_t n, void* stream);

/* ---- per-generation steps of a partition that exchanges ranks through messages ---- */

typedef struct csa_step_result {
    uint64_t active;   /* size of the partition's new active set: entries [0, active) of the outputs */
    uint64_t messages; /* messages in the outbox */
    /* Generations t >= 1, counted on the device in every call (the reference counts and checks them under -DTESTS,
     * include/GPU_SACA.cuh:234-249, src/GPU_SACA.cu:2055-2068): */
    uint64_t unserved; /* cohort members that no message joined: they sorted with an all-ones secondary. The exchange
                          scheme guarantees 0; the reference aborts otherwise ("Active suffixes with no message received") */
    uint64_t pills;    /* cohort members that a poison pill joined (their source's rank is final) */
    uint64_t incoherent_pills; /* neighbours of the sorted cohort with equal (primary, secondary) of which only one carries
                                  a pill receipt (test::validate_coherent_pill_receipts, test/tests.hpp:106-111; the
                                  reference traps). 0 in a coherent exchange */
} csa_step_result;

/* The counters of the last csa_sort_init_* / csa_sort_rerank_* call on the handle (the slab-shaped entries return
 * them this way). */
int csa_last_step_result(const csa_handle* h, csa_step_result* out);

/* Generation 0 of one partition of m suffixes (m <= the handle's capacity), everything resident in HBM:
 *   in : d_keys[i * key_words + w] packed K-gram words (key_words 1 to 4), d_suf40 5-byte lanes, d_beta routing-tag pairs (forward tag in
 *        the high half), in any order: what csa_stage_slab_u16_dev (or the reference's stage_slab) produces;
 *   out: d_rank_out[i] partition-local ranks (offset of the head of the run of equal (key, forward tag)) and
 *        d_suf40_out lanes, the tied ("active") suffixes first, in sorted order, the retired ones after them;
 *        the outbox: 5-byte targets, ranks (MSB = the sender retired), d_msg_off[q] = exclusive END of the group bound
 *        for partition q (p + 1 counters); ctx = 4 * key_words symbols were resolved.
 * The outbox needs room for m messages. The call returns after the stream has finished; res may be NULL.
 * The step works inside the handle's block and allocates nothing (csa_step_bytes_per_suffix covers it with the
 * caller's buffers counted in).
 * Replaces GPU_SACA::sort_and_init_rank_and_filter (include/GPU_SACA.hpp:272, src/GPU_SACA.cu:1112-1331) between the
 * upload of the slabs and their download. */
int csa_sort_init_dev(csa_handle* h, const uint64_t* d_keys, int key_words, const uint8_t* d_suf40, const uint32_t* d_beta,
                      uint64_t m, uint32_t p, uint32_t* d_rank_out, uint8_t* d_suf40_out, uint8_t* d_msg_target,
                      uint32_t* d_msg_rank, uint32_t* d_msg_off, void* stream, csa_step_result* res);

/* Generation t >= 1 (context ctx = ell * 2^t) of one partition's active set:
 *   in : d_rank partition-local ranks, d_suf40 lanes, d_beta routing-tag pairs (route of suffix - ctx | route of
 *        suffix - ctx / 2 << 16), in any order; the inbox (targets, ranks) of the messages sent to this partition at the
 *        end of the previous generation, in any order;
 *   out: as csa_sort_init_dev, ranks refined by (primary, received rank); the outbox needs room for 2 * m messages
 *        (payloads and forwarded pills).
 * A cohort member that received no message sorts with an all-ones secondary, as in the reference (the exchange
 * scheme guarantees there is none; res->unserved counts them).
 * Replaces GPU_SACA::sort_and_re_rank_and_filter (include/GPU_SACA.hpp:279, src/GPU_SACA.cu:1715-1995). */
int csa_sort_rerank_dev(csa_handle* h, const uint32_t* d_rank, const uint8_t* d_suf40, const uint32_t* d_beta, uint64_t m,
                        const uint8_t* d_inbox_target, const uint32_t* d_inbox_rank, uint32_t inbox_sz, uint64_t ctx,
                        uint32_t p, uint32_t* d_rank_out, uint8_t* d_suf40_out, uint8_t* d_msg_target, uint32_t* d_msg_rank,
                        uint32_t* d_msg_off, void* stream, csa_step_result* res);

/* ---- the same three steps in the form the reference's pipeline calls them: a partition as a chain of pinned host slabs ---- */

/* One slab of a partition: the pointers and offsets of the reference's Staging_Slab (include/Staging_Slab.hpp:20-119).
 * The buffers are host memory, pinned for transfers that overlap other work (hipHostMalloc; pageable memory works, more
 * slowly). Capacities as the reference allocates them (src/Staging_Slab.cpp:27-35) for a slab of chunk_cap suffixes:
 * key 8 * key_words * chunk_cap bytes, suf 5 * chunk_cap, beta 4 * chunk_cap, msg_target 5 * 2 * chunk_cap (and at least
 * two disk blocks of 4096 bytes for the scatter's edges), msg_rank 4 * 2 * chunk_cap. */
typedef struct csa_slab {
    void* key;            /* key(): generation 0 in: key_words 64-bit words per suffix; later generations and scatter in:
                             uint32 partition-local ranks; out (sort steps): uint32 ranks */
    uint8_t* suf;         /* suf(): 5-byte lanes in; out: lanes (sort steps), the chunk's block-aligned piece (scatter) */
    uint32_t* beta;       /* beta(): routing-tag pairs in (unused by the scatter) */
    uint8_t* msg_target;  /* msg_target(): the slab's chunk of the inbox in (later generations), of the outbox out;
                             scatter out: the unaligned head of the output at [0, ...), its tail at [4096, ...) */
    uint32_t* msg_rank;   /* msg_rank(): likewise */
    uint64_t off;         /* off(): where the slab's content starts in the partition; the slabs of a list follow one
                           * another (off = the sizes before it summed, src/GPU_SACA.cu:1396-1400) */
    uint64_t size;        /* size(): suffixes in the slab, at most chunk_cap */
    uint32_t inbox_off;   /* inbox_off(), inbox_sz(): the slab's chunk of the partition's inbox (later generations) */
    uint32_t inbox_sz;
    uint32_t outbox_off;  /* written by the sort steps (set_outbox_off_and_size): the slab's chunk of the outbox, */
    uint32_t outbox_sz;   /* messages [2 * c * chunk_cap, ...) for the c-th slab of the list */
} csa_slab;

/* GPU_SACA::sort_and_init_rank_and_filter(p_id, p_assembly, buf_id) (include/GPU_SACA.hpp:272, src/GPU_SACA.cu:1112-1331)
 * as the dispatcher calls it: uploads key(), suf(), beta() of every slab to the slab's off() (:1125-1133), runs
 * csa_sort_init_dev, then downloads into every slab its share of the ranks (over key()) and lanes, active suffixes
 * first, and its chunk of the outbox, split at 2 * chunk_cap messages per slab (:1305-1331).
 * h_msg_off receives the p exclusive END offsets of the destinations' groups (backend_->msg_off(p_id)), *h_active_slot
 * the new active-set size (backend_->active_slot(p_id)); either may be NULL. part_sz = the slabs' sizes summed <= the
 * handle's capacity. The call returns after the stream has finished (the reference's caller synchronises right after,
 * src/GPU_SACA.cu:1582); when it returns an error, nothing is still being copied into the slabs or h_msg_off either.
 * The device image of the slabs lives in the handle's block: no memory is allocated. */
int csa_sort_init_slabs(csa_handle* h, csa_slab* slabs, uint32_t slab_c, uint64_t part_sz, int key_words, uint32_t p,
                        uint64_t chunk_cap, uint32_t* h_msg_off, uint64_t* h_active_slot, void* stream);

/* GPU_SACA::sort_and_re_rank_and_filter (include/GPU_SACA.hpp:279, src/GPU_SACA.cu:1715-1995) likewise: key() carries the
 * uint32 ranks kept from the step before (:1739-1741), msg_target() / msg_rank() the slab's chunk of the partition's inbox at
 * inbox_off() (:1814-1819); inbox_sz = the whole inbox <= the handle's capacity (:1807-1812); ctx = the context this
 * generation resolves to (set_context, src/GPU_SACA.cu:1043-1049). Outputs as csa_sort_init_slabs (:1969-1995). */
int csa_sort_rerank_slabs(csa_handle* h, csa_slab* slabs, uint32_t slab_c, uint64_t part_sz, uint64_t inbox_sz, uint64_t ctx,
                          uint32_t p, uint64_t chunk_cap, uint32_t* h_msg_off, uint64_t* h_active_slot, void* stream);

/* GPU_SACA::scatter_to_rank_order (include/GPU_SACA.hpp:288, src/GPU_SACA.cu:2107-2164): uploads suf() and the ranks in
 * key() of every slab, scatters the lanes to rank order, and downloads the partition's stretch of the output as
 * Output_File::cut shares it out over the slabs (csa_output_cut with chunk_bytes = 5 * chunk_cap): slab c's whole disk
 * blocks into suf(), the unaligned head into the first slab's msg_target(), the unaligned tail into the last slab's
 * msg_target() + 4096. out_lo = byte offset of the partition in the output file (5 * P_off[p_id]). chunk_cap must be
 * a multiple of 4096 and slab_c * chunk_cap must reach part_sz. Returns after the stream has finished. */
int csa_scatter_slabs(csa_handle* h, csa_slab* slabs, uint32_t slab_c, uint64_t part_sz, uint64_t out_lo, uint64_t chunk_cap,
                      void* stream);

/* ---- the step after the partition sort, for partitions that come back as (suffix, local rank) pairs ---- */

/* d_sa40 entry rank[i] = d_suf entry i for i in [0, part_sz): 5-byte little-endian lanes in, lanes in rank order out.
 * d_rank must be a permutation of [0, part_sz); an entry out of range fails the call with CSA_ERR_ARG (checked on the
 * device; the reference traps under -DTESTS). The handle lends its error word only; any capacity will do.
 * Replaces scatter_suffixes_to_rank_kernel + pack_lanes_kernel (include/GPU_SACA.cuh:167-182,126-133) of
 * GPU_SACA::scatter_to_rank_order (src/GPU_SACA.cu:2107-2143). The call returns after the stream has finished. */
int csa_scatter_to_rank_order_dev(csa_handle* h, const uint8_t* d_suf, const uint32_t* d_rank, uint64_t part_sz,
                                  uint8_t* d_sa40, void* stream);

/* The byte ranges of a partition's output that chunk c of chunk_c carries to the output file, so that every write
 * but the first and the last of the file is a whole number of 4 KiB disk blocks: [lo, hi) is the partition's byte
 * range in the file, chunk_bytes the bytes of a full chunk.
 * out[0..1] = the chunk's block-aligned piece, out[2..3] = the range's unaligned head (first chunk only),
 * out[4..5] = its unaligned tail (last chunk only); absent parts are empty intervals.
 * Pure host arithmetic: Output_File::cut (src/Output_File.cpp:18-35; struct at include/Output_File.hpp:29-37). */
void csa_output_cut(uint64_t lo, uint64_t hi, uint64_t chunk_bytes, uint64_t c, uint64_t chunk_c, uint64_t out[6]);

/* Named ranges on a profiler's timeline (roctx; shown by rocprofv3 --marker-trace): one per partition sort, per
 * generation inside it, and per slab-shaped partition step. Off by default; enable != 0 loads the roctx library at run time
 * and fails with CSA_ERR_ARG where there is none. Process-wide.
 * Replaces the NVTX ranges of the reference's -DPROFILE build (include/profile.hpp:19-80; PROFILE_SCOPE_FMT at
 * src/GPU_SACA.cu:1114,1717,2004,2111). */
int csa_enable_profile_ranges(int enable);

/* Message of the calling thread's last failed call ("" if none). */
const char* csa_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
