// Host side of the library: the handle, the radix-sort driver, the generation loop and the C ABI
// declared in include/cascade_hip.h. gfx950 only.
#include "../../include/cascade_hip.h"

#include "device_pool.hpp"
#include "device_utils.hpp"
#include "doubling.hpp"
#include "messages.hpp"
#include "partition_ids.hpp"
#include "pipeline_steps.hpp"
#include "radix_sort.hpp"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <dlfcn.h>
#include <mutex>
#include <vector>

using namespace csa;

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

#define HIP_TRY(expr)                                                                                  \
    do {                                                                                               \
        hipError_t e_ = (expr);                                                                        \
        if (e_ != hipSuccess)                                                                          \
            return fail(CSA_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
    } while (0)

// Named ranges for a profiler's timeline, one per partition step and per generation: the counterpart of the NVTX ranges
// the reference opens under -DPROFILE (include/profile.hpp:19-80; PROFILE_SCOPE_FMT at src/GPU_SACA.cu:1114,1717,2004,2111).
// The roctx library is looked up at run time when csa_enable_profile_ranges(1) asks for it, so the library neither
// links against a profiler nor pays for ranges nobody reads.
#ifndef HIPEMU
struct ProfileRanges {
    std::mutex mu;
    bool tried = false;
    int (*push)(const char*) = nullptr;
    int (*pop)() = nullptr;
    bool enabled = false;
} g_ranges;

int enable_ranges(bool on)
{
    std::lock_guard<std::mutex> lock(g_ranges.mu);
    if (on && !g_ranges.tried) {
        g_ranges.tried = true;
        for (const char* name : {"librocprofiler-sdk-roctx.so", "librocprofiler-sdk-roctx.so.1", "libroctx64.so", "libroctx64.so.4"}) {
            if (void* lib = dlopen(name, RTLD_NOW | RTLD_GLOBAL)) {
                g_ranges.push = reinterpret_cast<int (*)(const char*)>(dlsym(lib, "roctxRangePushA"));
                g_ranges.pop = reinterpret_cast<int (*)()>(dlsym(lib, "roctxRangePop"));
                if (g_ranges.push && g_ranges.pop)
                    break;
                g_ranges.push = nullptr;
                g_ranges.pop = nullptr;
            }
        }
    }
    g_ranges.enabled = on && g_ranges.push && g_ranges.pop;
    return on && !g_ranges.enabled ? 1 : 0;
}
#else
struct ProfileRanges {
    int (*push)(const char*) = nullptr;
    int (*pop)() = nullptr;
    bool enabled = false;
} g_ranges;
int enable_ranges(bool) { return 1; }
#endif

struct RangeScope {
    bool open = false;
    explicit RangeScope(const char* fmt, ...)
    {
        if (!g_ranges.enabled)
            return;
        char name[128];
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(name, sizeof(name), fmt, ap);
        va_end(ap);
        g_ranges.push(name);
        open = true;
    }
    void close()
    {
        if (open)
            g_ranges.pop();
        open = false;
    }
    ~RangeScope() { close(); }
    RangeScope(const RangeScope&) = delete;
    RangeScope& operator=(const RangeScope&) = delete;
};

// tile shape of the radix pass; overridable at build time for tuning runs
#ifndef CSA_SORT_BLOCK
#define CSA_SORT_BLOCK 512
#endif
#ifndef CSA_SORT_ITEMS
#define CSA_SORT_ITEMS 16
#endif
#ifndef CSA_SORT32_ITEMS
#define CSA_SORT32_ITEMS CSA_SORT_ITEMS
#endif
constexpr int SORT_BLOCK = CSA_SORT_BLOCK;
constexpr int SORT_ITEMS = CSA_SORT_ITEMS;
constexpr int SORT32_ITEMS = CSA_SORT32_ITEMS; // pairs per thread when the keys are 32-bit (same LDS bytes at twice the items)
constexpr int SORT_TILE = SORT_BLOCK * SORT_ITEMS;
static_assert(SORT32_ITEMS >= SORT_ITEMS, "the look-back words are sized for tiles of SORT_TILE pairs or more");
// Long passes use workgroups of twice the threads: the runs of a digit a tile writes are twice as long, so fewer of the
// lines it writes are shared with a tile whose L2 is another one. One such workgroup fills a CU's LDS. Measured per
// sort of the 1B-token workload: 125.3 -> 121.4 ms by arrival (the default order, where neighbouring tiles run on
// different XCDs), 119.3 -> 117.4 ms under the chunked order, whose chunks keep their length in pairs (half as many
// of the larger tiles: with the full count the wide workgroups gained nothing there).
#ifndef CSA_SORT_WIDE_BLOCK
#define CSA_SORT_WIDE_BLOCK 1024
#endif
#ifndef CSA_SORT_WIDE_MIN
#define CSA_SORT_WIDE_MIN (1u << 24)
#endif
constexpr int SORT_WIDE_BLOCK = CSA_SORT_WIDE_BLOCK;
constexpr u32 SORT_WIDE_MIN = CSA_SORT_WIDE_MIN; // fewest pairs of a pass that uses the wide workgroups
static_assert(SORT_WIDE_BLOCK >= SORT_BLOCK, "the look-back words are sized for tiles of SORT_TILE pairs or more");
#ifndef CSA_RANK_BLOCK
#define CSA_RANK_BLOCK 256
#endif
#ifndef CSA_RANK_ITEMS
#define CSA_RANK_ITEMS 4
#endif
constexpr int RANK_BLOCK = CSA_RANK_BLOCK;
constexpr int RANK_ITEMS = CSA_RANK_ITEMS;
constexpr int RANK_TILE = RANK_BLOCK * RANK_ITEMS;
// Groups of up to SMALL_MAXG suffixes are sorted inside one tile of the small-group kernel; the larger ones go through
// the radix sort. A list of mostly short groups (at most SMALL_AVG_LIMIT members per group on average: token corpora)
// takes the higher limit SMALL_MAXG_HI, which leaves fewer members to the radix passes (1B-token workload: 117.5 ->
// 115.4 ms per sort). A list of long groups (small alphabets, runs) keeps the lower one: the tile's halo of SMALL_MAXG
// elements on either side and the longer member loops only cost there (4-letter workload sorted from one K-gram word:
// +6 % with the higher limit). The adversarial workload's generation 1 averages 16.5 members per group, most of them in
// groups of 65 to 256: the higher limit takes 37 M members off its radix passes (31.1 -> 29.0 ms), hence 32.
#ifndef CSA_SMALL_MAXG
#define CSA_SMALL_MAXG 64
#endif
#ifndef CSA_SMALL_MAXG_HI
#define CSA_SMALL_MAXG_HI 256
#endif
#ifndef CSA_SMALL_AVG_LIMIT
#define CSA_SMALL_AVG_LIMIT 32
#endif
// tile of the small-group kernel and of the counting / applying kernels behind it (measured per sort of the 1B-token
// workload with 16-byte loads in the applying kernel: 256 x 8 109.4 ms, 256 x 4 106.5, 512 x 4 106.2, 1024 x 4 106.7,
// 512 x 2 106.3, 512 x 8 108.8, 128 x 8 110.4)
#ifndef CSA_SMALL_BLOCK
#define CSA_SMALL_BLOCK 512
#endif
#ifndef CSA_SMALL_ITEMS
#define CSA_SMALL_ITEMS 4
#endif
constexpr int SMALL_BLOCK = CSA_SMALL_BLOCK;
constexpr int SMALL_ITEMS = CSA_SMALL_ITEMS;
constexpr int SMALL_TILE = SMALL_BLOCK * SMALL_ITEMS;
constexpr int SMALL_MAXG = CSA_SMALL_MAXG;
constexpr int SMALL_MAXG_HI = CSA_SMALL_MAXG_HI;
constexpr u32 SMALL_AVG_LIMIT = CSA_SMALL_AVG_LIMIT;
static_assert(SMALL_MAXG_HI >= SMALL_MAXG, "the higher group limit is the higher one");
constexpr u32 TICKET_POOL = 4096;
constexpr u32 PINNED_HIST = 32;        // host mirror: words [0, 16) mirror the device counters, [16, 32) single values, then the histograms
constexpr u32 MSG_OFF_WORDS = 32769;   // p + 1 outbox counters, p <= 32768
constexpr int EVENT_POOL = 2 * CSA_MAX_GENERATIONS * MAX_PASSES * 2;

// Lists of at least this many suffixes update rank[] through two radix passes on the text position instead of
// scattering 4-byte writes over the whole array.
#ifndef CSA_DEFER_MIN
#define CSA_DEFER_MIN (1u << 23)
#endif
// Lists of at least this many suffixes may take the dense form of a later generation (the whole partition sorted again
// by keys read in text order); below it the generation is over before the choice matters. Smaller in test builds.
#ifndef CSA_DENSE_MIN
#define CSA_DENSE_MIN (1u << 16)
#endif
constexpr u32 DENSE_MIN = CSA_DENSE_MIN;
constexpr u32 XCD_CHUNK = 16;
// Windows of rank[] that the last step of generation 0's bucketed update assembles in LDS (1 << 14 positions; twice
// that on the largest partitions, whose two passes cover 16 position bits at most). Smaller in test builds, so that
// short lists go through the passes too.
#ifndef CSA_PLACE_WINDOW_LOG2
#define CSA_PLACE_WINDOW_LOG2 14
#endif
constexpr int PLACE_WINDOW_LOG2 = CSA_PLACE_WINDOW_LOG2;
static_assert(PLACE_WINDOW_LOG2 >= 1 && PLACE_WINDOW_LOG2 <= 14, "the placement kernel holds a window of 1 << 14 or 1 << 15 ranks");
constexpr u32 DEFER_MIN = CSA_DEFER_MIN;
// Later generations: when at least half of the sorted list changes its rank, and at least WINDOW_MIN_CHANGED
// suffixes in all, the rank writes of the generation are bucketed into windows of 1 << WINDOW_LOG2 positions of
// rank[] first. Partitions that fit one window never need it.
#ifndef CSA_WINDOW_LOG2
#define CSA_WINDOW_LOG2 23
#endif
#ifndef CSA_WINDOW_MIN_CHANGED
#define CSA_WINDOW_MIN_CHANGED (1u << 22)
#endif
constexpr int WINDOW_LOG2 = CSA_WINDOW_LOG2;
constexpr u32 WINDOW_MIN_CHANGED = CSA_WINDOW_MIN_CHANGED;
// rank-order scatter of a whole partition: partitions of at least SCATTER_WINDOW_MIN suffixes are first grouped by
// windows of 2^SCATTER_WINDOW_LOG2 ranks (40 MB of output, which the last-level cache holds)
#ifndef CSA_SCATTER_WINDOW_LOG2
#define CSA_SCATTER_WINDOW_LOG2 23
#endif
#ifndef CSA_SCATTER_WINDOW_MIN
#define CSA_SCATTER_WINDOW_MIN (1u << 25)
#endif
constexpr u32 SCATTER_WINDOW_LOG2 = CSA_SCATTER_WINDOW_LOG2;
constexpr u64 SCATTER_WINDOW_MIN = CSA_SCATTER_WINDOW_MIN;
// smallest cohort for which the message join builds a directory over the suffix-ordered cohort first
#ifndef CSA_JOIN_DIR_MIN
#define CSA_JOIN_DIR_MIN 4096u
#endif


int bit_length(u64 v)
{
    int b = 0;
    while (v) {
        ++b;
        v >>= 1;
    }
    return b;
}

} // namespace

// ---- scratch of csa_radix_sort_pairs_static_dev, the one entry point that allocates nothing ----
// One array per device, part of the code object: it exists from the moment the library is loaded until the process
// ends. Host code never uses the name `scratch` as an address (on the host it is a stand-in, not device memory): the
// address on the current device comes from hipGetSymbolAddress, once per device (static_scratch below), and everything
// that needs the memory takes that pointer.
namespace {
constexpr u64 STATIC_SORT_MAX = CSA_STATIC_SORT_MAX_PAIRS;
constexpr u64 STATIC_TILES = (STATIC_SORT_MAX + SORT_TILE - 1) / SORT_TILE;
constexpr u64 STATIC_LB_TILE_WORDS = STATIC_TILES * RADIX_BINS;                                  // per pass
constexpr u64 STATIC_LB_WORDS = STATIC_LB_TILE_WORDS + (STATIC_TILES / LB_GROUP + 1) * RADIX_BINS; // per pass, groups included
constexpr u64 align256(u64 v) { return (v + 255u) & ~(u64)255u; }
// layout: the ping-pong partners of the caller's arrays, then the control words, which every call clears
constexpr u64 STATIC_OFF_KEYS = 0;
constexpr u64 STATIC_OFF_VALS = align256(STATIC_OFF_KEYS + STATIC_SORT_MAX * sizeof(u64));
constexpr u64 STATIC_OFF_CONTROL = align256(STATIC_OFF_VALS + STATIC_SORT_MAX * sizeof(u32));
constexpr u64 STATIC_OFF_LOOKBACK = STATIC_OFF_CONTROL;
constexpr u64 STATIC_OFF_GHIST = align256(STATIC_OFF_LOOKBACK + MAX_PASSES * STATIC_LB_WORDS * sizeof(u64));
constexpr u64 STATIC_OFF_TICKETS = align256(STATIC_OFF_GHIST + MAX_PASSES * RADIX_BINS * sizeof(u32));
constexpr u64 STATIC_OFF_ERR = align256(STATIC_OFF_TICKETS + MAX_PASSES * sizeof(u32));
constexpr u64 STATIC_OFF_DIGIT_BASE = align256(STATIC_OFF_ERR + sizeof(u32)); // written before it is read: not cleared
constexpr u64 STATIC_CONTROL_END = STATIC_OFF_DIGIT_BASE;
constexpr u64 STATIC_SCRATCH_BYTES = align256(STATIC_OFF_DIGIT_BASE + MAX_PASSES * RADIX_BINS * sizeof(u32));
} // namespace

static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

// What a handle was created for (csa_create: everything; csa_create_steps: everything but the resident sort).
constexpr u32 KIND_RESIDENT = 1u;

struct csa_handle {
    int device = 0;
    u64 cap = 0;
    int key_words = 1;
    u32 kinds = 0;
    int cus = 0; // compute units of the device
    // One block of device memory for everything that scales with the partition. The resident sort uses it under a fixed
    // carve-up made at creation (the arrays below); every other entry point takes and returns columns of it as it goes
    // (device_pool.hpp). A handle serves one call at a time, so the two never meet.
    unsigned char* block = nullptr;
    DevicePool pool;
    u64 last_high_water = 0; // of the last call that used the pool
    u64* key[3] = {nullptr, nullptr, nullptr};
    u32* idx[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
    u32* gid = nullptr;
    u32* rank = nullptr;
    u32* gprim[2] = {nullptr, nullptr};
    u32* gstart[2] = {nullptr, nullptr};
    // The workspace: tables whose size follows the number of tiles, and small fixed ones.
    u64* lookback = nullptr;
    u64 lookback_words = 0;
    u64 lookback_tile_words = 0;
    u32* tile_tables = nullptr; // rerank: [rank_tiles_cap][4] tile aggregates, the same of prefixes, [rank_tiles_cap] splits,
                                // [RERANK_SLABS][5] slab totals
    u64 rank_tiles_cap = 0;
    u32* ghist = nullptr;      // [MAX_PASSES][256]
    u32* digit_base = nullptr; // [MAX_PASSES][256]
    u32* tickets = nullptr;    // [TICKET_POOL]
    u32 ticket_next = 0;
    u32* counts = nullptr; // [2] error flag; [3] verifier flag; [4] members of large groups; [6..7] tied entries;
                           // [8..9] active-set size of a step; [10..11] unserved members; [12..13] pill receipts;
                           // [14] incoherent pill receipts
    u32* msg_off = nullptr; // [MSG_OFF_WORDS]: the outbox counters of the slab-shaped steps
    u32* h_pinned = nullptr; // host mirror: [0..15] counts, [16 ..) histogram
    u32 epoch = 0;
    u32 tile_order = TILES_BY_ARRIVAL;           // how the radix passes number their tiles (radix_sort.hpp), in use
    u32 tile_order_exclusive = TILES_BY_ARRIVAL; // the order after csa_set_device_exclusive
    u32 xcd_chunk = XCD_CHUNK;                   // tiles of a radix pass that one XCD takes in a row under TILES_STATIC_CHUNKS
    u32 defer_min = DEFER_MIN; // lists at least this long use the bucketed rank update (csa_set_tuning)
    u32 window_min_changed = WINDOW_MIN_CHANGED; // csa_set_tuning (0xFFFFFFFF: never)
    u32 expect_presorted = 0; // csa_set_tuning: 1 = every generation first runs as if its large groups were in order already
    u32 pack_symbols = 1; // csa_set_tuning: texts over small alphabets start from keys of many symbols (packed_text.hpp)
    csa_step_result last_step = {};              // counters of the last partition step (csa_last_step_result)
    std::vector<hipEvent_t> events;
    hipEvent_t ev_gen[CSA_MAX_GENERATIONS + 2] = {};
    bool ev_gen_ready = false;
};

namespace {

struct Launch {
    csa_handle* h;
    hipStream_t stream;
    u32 flags;
    csa_stats* stats;
    std::vector<std::pair<int, u64>> timed; // (first event index, pairs) of each timed radix launch
    int events_used = 0;
};

int next_ticket(Launch& L, u32** out)
{
    csa_handle* h = L.h;
    if (h->ticket_next == TICKET_POOL) {
        HIP_TRY(hipMemsetAsync(h->tickets, 0, TICKET_POOL * sizeof(u32), L.stream));
        h->ticket_next = 0;
    }
    *out = h->tickets + h->ticket_next++;
    return CSA_OK;
}

u32 next_epoch(csa_handle* h)
{
    h->epoch++;
    if (h->epoch >= (1u << 30)) { // never in practice; stale words would need a clear before reuse
        (void)hipMemset(h->lookback, 0, h->lookback_words * sizeof(u64));
        h->epoch = 1;
    }
    return h->epoch;
}

u32 hist_blocks(u64 items_per_block, u64 n)
{
    u64 blocks = (n + items_per_block - 1) / items_per_block;
    if (blocks > 2048)
        blocks = 2048;
    return (u32)(blocks ? blocks : 1);
}

// How the radix passes of a call number their tiles (radix_sort.hpp).
struct TileOrder {
    u32 order;     // TILES_BY_ARRIVAL or TILES_STATIC_CHUNKS
    u32 xcd_chunk; // tiles of SORT_TILE pairs that one XCD takes in a row under TILES_STATIC_CHUNKS
};

// tile order of a pass over a.n pairs in tiles of `tile` pairs
void set_tile_order(const TileOrder& o, OnesweepArgs& a, u32 tile)
{
    a.tiles = (u32)(((u64)a.n + tile - 1) / tile);
    a.order = o.order;
    // the chunk length is meant in tiles of SORT_TILE pairs: larger tiles, proportionally fewer per chunk
    const u32 chunk = (u32)((u64)o.xcd_chunk * SORT_TILE / tile);
    a.xcd_chunk = chunk ? chunk : 1u;
}

TileOrder tile_order_of(const csa_handle* h) { return TileOrder{h->tile_order, h->xcd_chunk}; }

bool wide_workgroups(const OnesweepArgs& a)
{
    return SORT_WIDE_BLOCK > SORT_BLOCK && a.n >= SORT_WIDE_MIN;
}

template <int SRC, int BLOCK, bool VALS>
void launch_onesweep_shape(const TileOrder& o, OnesweepArgs& a, hipStream_t s)
{
    set_tile_order(o, a, BLOCK * SORT_ITEMS);
    if (a.shift >= 32)
        hipLaunchKernelGGL((onesweep_kernel<u64, BLOCK, SORT_ITEMS, SRC, 1, VALS>), dim3(a.tiles), dim3(BLOCK), 0, s, a);
    else
        hipLaunchKernelGGL((onesweep_kernel<u64, BLOCK, SORT_ITEMS, SRC, 0, VALS>), dim3(a.tiles), dim3(BLOCK), 0, s, a);
}

template <int SRC, bool VALS = true>
void launch_onesweep(const csa_handle* h, OnesweepArgs& a, hipStream_t s)
{
    if (wide_workgroups(a))
        launch_onesweep_shape<SRC, SORT_WIDE_BLOCK, VALS>(tile_order_of(h), a, s);
    else
        launch_onesweep_shape<SRC, SORT_BLOCK, VALS>(tile_order_of(h), a, s);
}

void launch_onesweep32(const csa_handle* hh, OnesweepArgs& a, hipStream_t s)
{
    const TileOrder h = tile_order_of(hh);
    if (wide_workgroups(a)) {
        set_tile_order(h, a, SORT_WIDE_BLOCK * SORT32_ITEMS);
        hipLaunchKernelGGL((onesweep_kernel<u32, SORT_WIDE_BLOCK, SORT32_ITEMS, SRC_PAIRS, 0>), dim3(a.tiles), dim3(SORT_WIDE_BLOCK), 0, s, a);
    } else {
        set_tile_order(h, a, SORT_BLOCK * SORT32_ITEMS);
        hipLaunchKernelGGL((onesweep_kernel<u32, SORT_BLOCK, SORT32_ITEMS, SRC_PAIRS, 0>), dim3(a.tiles), dim3(SORT_BLOCK), 0, s, a);
    }
}

// Sorts n pairs by the digits of `plan`. The first pass that runs takes its input as `src` says
// (pairs kin/vin, or the text); passes alternate between the (kin, vin) and (kout, vout) sets, the
// very first one writing to (kout, vout). *result_in_out = 1 if the sorted pairs ended in (kout, vout).
// Passes whose digit is the same for every pair are skipped (they would be the identity).
// src = SRC_RANKS: pair i is ((rank_src[i], rank_src[i + hop]), i), i < n, built by the first pass that runs; the two
// ranks are combined as rank_pair_key says for `radix`.
// src = SRC_PACKED: the first pass cuts its keys from the code stream `packed` describes; the caller has filled
// ghist already (hist_ready = 2). hist_ready = 1 (SRC_TEXT): the byte histograms of the text are in place.
struct PackedSource {
    const u32* stream;
    u64 words;
    u32 sym_bits, key_bits;
};

int radix_sort(Launch& L, int src, const u16* text, u32 text_n, u32 tail, u32 word, u64* kin, u32* vin, u64* kout,
               u32* vout, u32 n, const PassPlan& plan, int* result_in_out, int* passes_run, const u32* rank_src = nullptr,
               u32 hop = 0, u32 radix = 0, const PackedSource* packed = nullptr, int hist_ready = 0)
{
    csa_handle* h = L.h;
    hipStream_t s = L.stream;
    *result_in_out = 0;
    *passes_run = 0;
    if (n == 0)
        return CSA_OK;
    // ghist[MAX_PASSES][256] followed by the two byte histograms of the text
    if (hist_ready == 0)
        HIP_TRY(hipMemsetAsync(h->ghist, 0, (MAX_PASSES + 2) * RADIX_BINS * sizeof(u32), s));
    if (src == SRC_PACKED) {
        if (!packed || hist_ready != 2)
            return fail(CSA_ERR_INTERNAL, "radix_sort: packed keys come with their histograms");
    } else if (src == SRC_PAIRS || src == SRC_RANKS) {
        HistArgs ha;
        ha.keys = kin;
        ha.vals = vin;
        ha.text = text;
        ha.n = n;
        ha.text_n = text_n;
        ha.word = word;
        ha.plan = plan;
        ha.ghist = h->ghist;
        if (src == SRC_RANKS) {
            ha.rank = rank_src;
            ha.hop = hop;
            ha.radix = radix;
        }
        // the two halves of a (rank[i], rank[i + hop]) key are the same array, one shifted by hop: when the plan takes
        // the same digits from both halves, one histogram of rank[] and one of its first hop entries give them all
        const int half = plan.num_passes / 2;
        bool mirrored = src == SRC_RANKS && radix == 0 && plan.num_passes == 2 * half && half >= 1 && half <= RANK_HIST_PASSES;
        for (int p = 0; mirrored && p < half; ++p)
            mirrored = plan.shift[p] + plan.bits[p] <= 32 && plan.shift[half + p] == 32 + plan.shift[p] && plan.bits[half + p] == plan.bits[p];
        if (mirrored) {
            RankHistArgs ra;
            ra.rank = rank_src;
            ra.num_passes = half;
            for (int p = 0; p < half; ++p) {
                ra.shift[p] = plan.shift[p];
                ra.bits[p] = plan.bits[p];
            }
            const u32 cut = hop < n ? hop : n;
            ra.begin = 0;
            ra.end = n;
            ra.out = h->ghist + half * RADIX_BINS;
            hipLaunchKernelGGL(rank_hist_kernel, dim3(hist_blocks(256 * 16, n)), dim3(256), 0, s, ra);
            if (cut > 0) {
                ra.end = cut;
                ra.out = h->ghist;
                hipLaunchKernelGGL(rank_hist_kernel, dim3(hist_blocks(256 * 16, cut)), dim3(256), 0, s, ra);
            }
            hipLaunchKernelGGL(rank_hist_combine_kernel, dim3(1), dim3(256), 0, s, h->ghist, half, cut);
        } else {
            hipLaunchKernelGGL(radix_hist_kernel, dim3(hist_blocks(256 * 16, n)), dim3(256), 0, s, ha);
        }
    } else {
        // every suffix of the text takes part and the plan is the eight bytes of one key word: the digit
        // histograms follow from the byte histogram of the text, whatever order the pairs are in
        u32* bytehist = h->ghist + MAX_PASSES * RADIX_BINS;
        if (hist_ready == 0)
            hipLaunchKernelGGL(text_byte_hist_kernel, dim3(hist_blocks(256 * 8 * 16, text_n)), dim3(256), 0, s, text, text_n,
                               bytehist);
        hipLaunchKernelGGL(text_hist_expand_kernel, dim3(1), dim3(256), 0, s, text, text_n, word, bytehist, h->ghist);
    }
    hipLaunchKernelGGL(radix_scan_hist_kernel, dim3(1), dim3(256), 0, s, h->ghist, h->digit_base, plan.num_passes);
    HIP_TRY(hipGetLastError());
    u32* h_hist = h->h_pinned + PINNED_HIST;
    HIP_TRY(hipMemcpyAsync(h_hist, h->ghist, plan.num_passes * RADIX_BINS * sizeof(u32), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    bool run[MAX_PASSES];
    int n_run = 0;
    for (int p = 0; p < plan.num_passes; ++p) {
        bool trivial = false;
        for (int d = 0; d < RADIX_BINS; ++d)
            if (h_hist[p * RADIX_BINS + d] == n)
                trivial = true;
        run[p] = !trivial;
        n_run += run[p] ? 1 : 0;
    }
    if (n_run == 0 && src != SRC_PAIRS && plan.num_passes > 0) { // the pairs must still be materialised once
        run[plan.num_passes - 1] = true;
        n_run = 1;
    }
    bool first = true;
    int where = 0; // 0: current data in (kin, vin) (or the text); 1: in (kout, vout)
    for (int p = 0; p < plan.num_passes; ++p) {
        if (!run[p])
            continue;
        OnesweepArgs a;
        a.keys_in = where == 0 ? kin : kout;
        a.vals_in = where == 0 ? vin : vout;
        a.keys_out = where == 0 ? kout : kin;
        a.vals_out = where == 0 ? vout : vin;
        a.text = text;
        a.n = n;
        a.text_n = text_n;
        a.tail = tail;
        a.word = word;
        a.shift = plan.shift[p];
        a.bits = plan.bits[p];
        a.digit_base = h->digit_base + p * RADIX_BINS;
        a.lookback = h->lookback;
        a.lookback_groups = h->lookback + h->lookback_tile_words;
        a.epoch = next_epoch(h);
        a.err = h->counts + 2;
        a.rank = rank_src;
        a.hop = hop;
        a.radix = radix;
        if (packed) {
            a.stream = packed->stream;
            a.stream_words = packed->words;
            a.sym_bits = packed->sym_bits;
            a.key_bits = packed->key_bits;
        }
        int rc = next_ticket(L, &a.ticket);
        if (rc)
            return rc;
        const bool timed = (L.flags & CSA_FLAG_KERNEL_TIMING) && L.events_used + 2 <= (int)h->events.size();
        if (timed)
            HIP_TRY(hipEventRecord(h->events[L.events_used], s));
        const int use_src = first ? src : SRC_PAIRS;
        if (use_src == SRC_PAIRS)
            launch_onesweep<SRC_PAIRS>(h, a, s);
        else if (use_src == SRC_RANKS)
            launch_onesweep<SRC_RANKS>(h, a, s);
        else if (use_src == SRC_PACKED)
            launch_onesweep<SRC_PACKED>(h, a, s);
        else
            launch_onesweep<SRC_TEXT>(h, a, s);
        if (timed) {
            HIP_TRY(hipEventRecord(h->events[L.events_used + 1], s));
            L.timed.push_back({L.events_used, (u64)n});
            L.events_used += 2;
        }
        first = false;
        where ^= 1;
        (*passes_run)++;
    }
    HIP_TRY(hipGetLastError());
    *result_in_out = where;
    return CSA_OK;
}

PassPlan make_plan(int begin_bit, int end_bit)
{
    PassPlan p;
    p.num_passes = 0;
    // digits of up to 8 bits that never straddle bit 32 (a pass reads its digit from one half of the key)
    int s = begin_bit;
    while (s < end_bit && p.num_passes < MAX_PASSES) {
        int bits = end_bit - s < RADIX_BITS ? end_bit - s : RADIX_BITS;
        if (s < 32 && s + bits > 32)
            bits = 32 - s;
        p.shift[p.num_passes] = s;
        p.bits[p.num_passes] = bits;
        p.num_passes++;
        s += bits;
    }
    return p;
}

int ensure_events(csa_handle* h, bool kernel_timing)
{
    if (!h->ev_gen_ready) {
        for (auto& e : h->ev_gen)
            HIP_TRY(hipEventCreate(&e));
        h->ev_gen_ready = true;
    }
    if (kernel_timing && h->events.empty()) {
        h->events.resize(EVENT_POOL);
        for (auto& e : h->events)
            HIP_TRY(hipEventCreate(&e));
    }
    return CSA_OK;
}

// counts: [2] device error flag, [3] verifier flag, [4] members of large groups. Waits for the stream.
int read_counts(Launch& L, u32* big)
{
    csa_handle* h = L.h;
    HIP_TRY(hipMemcpyAsync(h->h_pinned, h->counts, 8 * sizeof(u32), hipMemcpyDeviceToHost, L.stream));
    HIP_TRY(hipStreamSynchronize(L.stream));
    if (h->h_pinned[2]) {
        static const char* const what[] = {"", "a look-back wait ran into its spin limit",
                                           "an active suffix lies outside its group's range (small-group sort)",
                                           "a large-group member was sent outside the active list (place)",
                                           "a rank or suffix index out of range in the sorted active list (rerank)",
                                           "a large group appeared in a list whose groups were all small",
                                           "the join table of a partition step has more members than slots"};
        const u32 code = h->h_pinned[2];
        return fail(CSA_ERR_INTERNAL, "device invariant %u failed: %s", code, code < 7 ? what[code] : "unknown");
    }
    if (big)
        *big = h->h_pinned[4];
    return CSA_OK;
}


struct DeferBuffers {
    u64* recs[2]; // generation 0: [n] (position << 32 | rank) records in sorted-list order, and their ping-pong partner
    u32* vals;    // later generations: [m] new ranks in sorted-list order
    u32* t1_pos;  // ping
    u32* t1_val;
    u32* t2_pos;  // pong
    u32* t2_val;
};

// After a rerank launched with rank_recs = buf.recs[0]: rank[x] = r for each of the n records (x << 32) | r.
// The positions x are a permutation of the text positions [0, n) (the sorted suffixes of generation 0), which makes
// the digit counts of the passes a closed form. The records are sorted on the position bits above the window size
// (windows of at most 1 << 14 positions, 1 << 15 for the largest partitions), then placed window by window.
int deferred_rank_update(Launch& L, const DeferBuffers& buf, u32 n)
{
    csa_handle* h = L.h;
    hipStream_t s = L.stream;
    const int nb = bit_length(n - 1); // <= 31
    int top = nb - PLACE_WINDOW_LOG2; // position bits to sort on
    if (top < 0)
        top = 0;
    if (top > 16)
        top = 16;
    const int window_log2 = nb - top;
    int n_pass = 0, xshift[2] = {0, 0}, xbits[2] = {0, 0};
    if (top > 8) {
        xshift[0] = window_log2;
        xbits[0] = top - 8;
        xshift[1] = window_log2 + top - 8;
        xbits[1] = 8;
        n_pass = 2;
    } else if (top > 0) {
        xshift[0] = window_log2;
        xbits[0] = top;
        n_pass = 1;
    }
    const u64* in_recs = buf.recs[0];
    if (n_pass > 0) {
        u32* h_hist = h->h_pinned + PINNED_HIST;
        for (int p = 0; p < n_pass; ++p) {
            // positions x in [0, n) whose digit (x >> shift) & mask equals d: whole periods plus a clamped remainder
            const u64 unit = 1ull << xshift[p], period = unit << xbits[p];
            const u64 whole = (u64)n / period, rest = (u64)n % period;
            for (u32 d = 0; d < (u32)RADIX_BINS; ++d) {
                u64 c = 0;
                if (d < (1u << xbits[p])) {
                    c = whole * unit;
                    if (rest > d * unit)
                        c += rest - d * unit < unit ? rest - d * unit : unit;
                }
                h_hist[p * RADIX_BINS + d] = (u32)c;
            }
        }
        HIP_TRY(hipMemcpyAsync(h->ghist, h_hist, n_pass * RADIX_BINS * sizeof(u32), hipMemcpyHostToDevice, s));
        hipLaunchKernelGGL(radix_scan_hist_kernel, dim3(1), dim3(256), 0, s, h->ghist, h->digit_base, n_pass);
        for (int p = 0; p < n_pass; ++p) {
            OnesweepArgs a;
            a.keys_in = in_recs;
            a.vals_in = nullptr; // the records travel alone
            a.keys_out = buf.recs[(p + 1) & 1];
            a.vals_out = nullptr;
            a.text = nullptr;
            a.n = n;
            a.text_n = n;
            a.tail = 0;
            a.word = 0;
            a.shift = 32 + xshift[p]; // the position is the high half of a record
            a.bits = xbits[p];
            a.digit_base = h->digit_base + p * RADIX_BINS;
            a.lookback = h->lookback;
            a.lookback_groups = h->lookback + h->lookback_tile_words;
            a.epoch = next_epoch(h);
            a.err = h->counts + 2;
                int rc = next_ticket(L, &a.ticket);
            if (rc)
                return rc;
            launch_onesweep<SRC_PAIRS, false>(h, a, s);
            in_recs = buf.recs[(p + 1) & 1];
        }
    }
    const u32 windows = (u32)((((u64)n - 1) >> window_log2) + 1);
    if (window_log2 <= 14)
        hipLaunchKernelGGL((place_ranks_kernel<14>), dim3(windows), dim3(1024), 0, s, in_recs, n, window_log2, h->rank);
    else
        hipLaunchKernelGGL((place_ranks_kernel<15>), dim3(windows), dim3(1024), 0, s, in_recs, n, window_log2, h->rank);
    HIP_TRY(hipGetLastError());
    return CSA_OK;
}

// Bucketed rank update of a later generation: rank[pos[c]] = vals[c] wherever vals[c] != NO_RANK, c < m.
// One radix pass on the position bits above the window size, then a plain scatter that stays inside one window
// of rank[] at a time.
int windowed_rank_update(Launch& L, const u32* pos, const DeferBuffers& buf, u32 m, u32 n)
{
    csa_handle* h = L.h;
    hipStream_t s = L.stream;
    const int nb = bit_length(n - 1);
    int top = nb - WINDOW_LOG2;
    if (top > 8)
        top = 8;
    const u32* in_pos = pos;
    const u32* in_val = buf.vals;
    if (top > 0) {
        const int shift = nb - top;
        HIP_TRY(hipMemsetAsync(h->ghist, 0, RADIX_BINS * sizeof(u32), s));
        hipLaunchKernelGGL(position_hist_kernel, dim3(hist_blocks(256 * 16, m)), dim3(256), 0, s, pos, m, shift, top, h->ghist);
        hipLaunchKernelGGL(radix_scan_hist_kernel, dim3(1), dim3(256), 0, s, h->ghist, h->digit_base, 1);
        OnesweepArgs a;
        a.keys_in = pos;
        a.vals_in = buf.vals;
        a.keys_out = buf.t1_pos;
        a.vals_out = buf.t1_val;
        a.text = nullptr;
        a.n = m;
        a.text_n = n;
        a.tail = 0;
        a.word = 0;
        a.shift = shift;
        a.bits = top;
        a.digit_base = h->digit_base;
        a.lookback = h->lookback;
        a.lookback_groups = h->lookback + h->lookback_tile_words;
        a.epoch = next_epoch(h);
        a.err = h->counts + 2;
        int rc = next_ticket(L, &a.ticket);
        if (rc)
            return rc;
        launch_onesweep32(h, a, s);
        in_pos = buf.t1_pos;
        in_val = buf.t1_val;
    }
    hipLaunchKernelGGL(scatter_ranks_kernel, dim3((u32)(((u64)m + 1023) / 1024)), dim3(256), 0, s, in_pos, in_val, m, n, h->rank,
                       h->counts + 2);
    HIP_TRY(hipGetLastError());
    return CSA_OK;
}

// Sizes of the rank step's tables for a list of m suffixes cut into tiles of `tile` elements.
struct RankTables {
    u32 tiles, slab, slabs;
    u32 *tile_agg, *tile_prefix, *tile_splits, *slab_total;
};

RankTables rank_tables(csa_handle* h, u32 m, u32 tile)
{
    RankTables r;
    r.tiles = (u32)(((u64)m + tile - 1) / tile);
    r.slab = (r.tiles + RERANK_SLABS - 1) / RERANK_SLABS;
    r.slabs = (r.tiles + r.slab - 1) / r.slab;
    r.tile_agg = h->tile_tables;
    r.tile_prefix = h->tile_tables + (u64)h->rank_tiles_cap * 4;
    r.tile_splits = h->tile_tables + (u64)h->rank_tiles_cap * 8;
    r.slab_total = h->tile_tables + (u64)h->rank_tiles_cap * 9;
    return r;
}

// Scans the per-tile counts, reads the totals back (the one host round trip of the step: the next list's size
// decides the launches that follow) and chooses how the ranks are written: 0 scattered by the applying kernel,
// 1 two-pass bucketed (generation 0 of large partitions), 2 one-pass bucketed (most of a later list changed).
int rank_totals(Launch& L, const RankTables& r, bool gen0, u32 m, u32 n, bool expect_no_big, u32* survivors, u32* groups,
                int* rank_update)
{
    csa_handle* h = L.h;
    hipStream_t s = L.stream;
    hipLaunchKernelGGL(rerank_scan_kernel, dim3(r.slabs), dim3(1024), 0, s, r.tile_agg, r.tile_prefix, r.tiles, r.slab,
                       r.slab_total, r.tile_splits);
    HIP_TRY(hipGetLastError());
    u32* h_slabs = h->h_pinned + PINNED_HIST;
    HIP_TRY(hipMemcpyAsync(h_slabs, r.slab_total, r.slabs * 5 * sizeof(u32), hipMemcpyDeviceToHost, s));
    u32 big_seen = 0;
    int rc = read_counts(L, &big_seen);
    if (rc)
        return rc;
    if (expect_no_big && big_seen != 0) // groups only split; a large group after an all-small generation is a corrupt list
        return fail(CSA_ERR_INTERNAL, "%u members of large groups appeared after a generation without any", big_seen);
    u64 surv = 0, heads = 0, changed = 0;
    for (u32 sl = 0; sl < r.slabs; ++sl) {
        surv += h_slabs[sl * 5 + 2];
        heads += h_slabs[sl * 5 + 3];
        changed += h_slabs[sl * 5 + 4];
    }
    *survivors = (u32)surv;
    *groups = (u32)heads;
    // Generation 0 ranks every suffix of the partition: on large partitions the n scattered writes go through the
    // two-pass bucketed update. Later generations write only the ranks that changed; when those are many and the
    // partition is larger than one window, they go through the one-pass bucketed update.
    const bool defer0 = gen0 && m >= h->defer_min;
    const bool windowed = !gen0 && bit_length(n - 1) > WINDOW_LOG2 && changed >= h->window_min_changed && changed >= m / 2;
    *rank_update = defer0 ? 1 : windowed ? 2 : 0;
    return CSA_OK;
}

// A dense generation: most of the partition is still active and its groups are long (a small alphabet, a periodic
// text), so nearly every member would go through the radix sort anyway; the whole partition is then sorted again by
// keys read in text order. Decided from the size of the active list and the number of its groups alone, so that the
// generation before already knows it (and leaves ordinals in rank[], which such a generation sorts in fewer passes).
bool dense_generation(u32 m, u32 groups, u32 n)
{
    return (u64)m * 5 >= (u64)n * 3 && (u64)m > (u64)groups * SMALL_MAXG_HI && (u64)m >= DENSE_MIN;
}

// Whether, and how, the first sort of a partition takes keys of many packed symbols (packed_text.hpp). From the byte
// histograms of the text: a symbol's code is made of the ranks of its two bytes among the byte values that occur, zero
// (the padding) included; with nhi * nlo <= 256 codes the text qualifies. The key takes the largest context the doubling
// of the caller's key width reaches inside 64 bits: S = 4 W 2^j symbols, which covers j generations after the first.
struct PackedPlan {
    bool enabled;
    SymbolCodes codes;
    u32 skipped; // j
};

PackedPlan plan_packed_text(const u32* bytehist, u32 n, int key_words, u64 room_bytes)
{
    PackedPlan pp;
    memset(&pp, 0, sizeof(pp));
    u32 nlo = 0, nhi = 0;
    for (u32 d = 0; d < 256; ++d) {
        if (d == 0 || bytehist[d] != 0)
            pp.codes.lo[d] = (u8)nlo++;
        if (d == 0 || bytehist[256 + d] != 0)
            pp.codes.hi[d] = (u8)nhi++;
    }
    const u32 codes = nlo * nhi;
    if (codes > 256)
        return pp;
    const u32 b = codes <= 2 ? 1u : codes <= 4 ? 2u : codes <= 16 ? 4u : 8u;
    u32 S = 4u * (u32)key_words;
    if (S * b > 64)
        return pp;
    u32 j = 0;
    while (2 * S * b <= 64) {
        S *= 2;
        ++j;
    }
    const u64 words = ((u64)n * b + 31) / 32 + 4;
    if (words * 4 > room_bytes)
        return pp;
    pp.codes.nlo = nlo;
    pp.codes.bits = b;
    pp.codes.key_syms = S;
    pp.skipped = j;
    pp.enabled = true;
    return pp;
}

// Generation 0: ranks the sorted list described by `ra`: counts per tile, scans the counts, reads the totals back, then
// applies them and brings rank[] up to date, directly from the kernel or through the two-pass bucketed update.
int rerank_step(Launch& L, RerankArgs& ra, const DeferBuffers& buf, u32* survivors, u32* groups, int* rank_update,
                u32* level_counts = nullptr)
{
    csa_handle* h = L.h;
    hipStream_t s = L.stream;
    const RankTables r = rank_tables(h, ra.m, RANK_TILE);
    ra.tile_agg = r.tile_agg;
    ra.tile_prefix = r.tile_prefix;
    ra.tile_splits = r.tile_splits;
    ra.slab_total = r.slab_total;
    ra.slab = r.slab;
    ra.err = h->counts + 2;
    ra.rank_recs = nullptr;
    // the level counts of packed keys ride along: accumulated in the (idle) digit histograms, read back with the totals
    unsigned long long* const h_levels = reinterpret_cast<unsigned long long*>(h->h_pinned + PINNED_HIST + 512);
    if (ra.levels) {
        ra.level_totals = reinterpret_cast<unsigned long long*>(h->ghist);
        HIP_TRY(hipMemsetAsync(ra.level_totals, 0, LEVEL_SLOTS * 8 * sizeof(unsigned long long), s));
    }
    hipLaunchKernelGGL((rerank_count_kernel<RANK_BLOCK, RANK_ITEMS>), dim3(r.tiles), dim3(RANK_BLOCK), 0, s, ra);
    if (ra.levels)
        HIP_TRY(hipMemcpyAsync(h_levels, ra.level_totals, LEVEL_SLOTS * 8 * sizeof(unsigned long long), hipMemcpyDeviceToHost, s));
    int rc = rank_totals(L, r, true, ra.m, ra.n, false, survivors, groups, rank_update);
    if (rc)
        return rc;
    for (u32 i = 0; i < ra.levels && level_counts; ++i) {
        u64 sv = 0, hd = 0;
        for (u32 slot = 0; slot < LEVEL_SLOTS; ++slot) {
            sv += h_levels[slot * 8 + 2 * i];
            hd += h_levels[slot * 8 + 2 * i + 1];
        }
        level_counts[2 * i] = (u32)sv;
        level_counts[2 * i + 1] = (u32)hd;
    }
    // what the list becomes decides what rank[] is to hold: ordinals for a dense generation, ranks otherwise
    ra.ordinals = dense_generation(*survivors, *groups, ra.n) ? 1u : 0u;
    if (*rank_update != 0)
        ra.rank_recs = buf.recs[0];
    hipLaunchKernelGGL((rerank_kernel<RANK_BLOCK, RANK_ITEMS>), dim3(r.tiles), dim3(RANK_BLOCK), 0, s, ra);
    HIP_TRY(hipGetLastError());
    if (*rank_update == 1)
        return deferred_rank_update(L, buf, ra.n);
    return CSA_OK;
}

int sort_partition(Launch& L, const u16* d_text, u64 n64, u64 index_base, u8* d_sa40)
{
    csa_handle* h = L.h;
    hipStream_t s = L.stream;
    csa_stats* st = L.stats;
    const u32 n = (u32)n64;
    // Wide keys are not sorted word by word. A generation 0 that resolves 4 W symbols is what doubling on one-word keys
    // reaches after one or two more generations (4 -> 8 -> 16 symbols; 4 -> 8 -> 12 with the second step looking only 4
    // symbols ahead; the order of suffixes that run off the text is the same: the shorter first). So the sort always
    // starts from one-word keys, steps up to the context of the wide key, reports those generations as its generation 0
    // and doubles from there. Every reported generation then has the context, the ranks and the active set of the wide-key
    // generation it stands for. A 4-word key sorted word by word costs 32 radix passes over all suffixes (316 ms on the
    // 1B-token workload); this way it costs what the one-word key costs.
    const u64 wide_ell = 4ull * (u64)h->key_words;

    RangeScope range_sort("sort_partition n=%u", n);
    HIP_TRY(hipMemsetAsync(h->counts, 0, 4 * sizeof(u32), s));
    HIP_TRY(hipEventRecord(h->ev_gen[0], s));

    // ---- generation 0: sort every suffix by its K-gram key, ties of tail suffixes broken by length ----
    RangeScope range_gen0("generation 0 m=%u", n);
    // The byte histograms of the text come first: they give the digit counts of the passes and tell whether the alphabet
    // is small enough for keys of more than four symbols.
    HIP_TRY(hipMemsetAsync(h->ghist, 0, (MAX_PASSES + 2) * RADIX_BINS * sizeof(u32), s));
    u32* const bytehist = h->ghist + MAX_PASSES * RADIX_BINS;
    hipLaunchKernelGGL(text_byte_hist_kernel, dim3(hist_blocks(256 * 8 * 16, n)), dim3(256), 0, s, d_text, n, bytehist);
    PackedPlan pp;
    memset(&pp, 0, sizeof(pp));
    if (h->pack_symbols) {
        u32* h_bytes = h->h_pinned + PINNED_HIST;
        HIP_TRY(hipMemcpyAsync(h_bytes, bytehist, 2 * RADIX_BINS * sizeof(u32), hipMemcpyDeviceToHost, s));
        HIP_TRY(hipStreamSynchronize(s));
        pp = plan_packed_text(h_bytes, n, h->key_words, (u64)h->cap * sizeof(u32));
    }
    const u32 ell = pp.enabled ? pp.codes.key_syms : 4u; // symbols the first sort resolves
    int folded = 0; // generations after the first that still belong to the reported generation 0
    for (u64 c = ell; c < wide_ell; c += (c < wide_ell - c ? c : wide_ell - c))
        ++folded;
    const u32 tail = n < ell ? n : ell;
    int passes = 0, p1 = 0, in_out = 0;
    u64* K[2] = {h->key[0], h->key[1]};
    u32* V[2] = {h->idx[0], h->idx[1]};
    int cur; // the (K, V) set that holds the sorted pairs
    int rc;
    cur = 0;
    if (pp.enabled) {
        // the code stream lives in rank[], which nothing uses before the sorted list is ranked
        PackedSource ps;
        u32* const stream = h->rank;
        ps.stream = stream;
        ps.sym_bits = pp.codes.bits;
        ps.key_bits = pp.codes.key_syms * pp.codes.bits;
        ps.words = ((u64)n * ps.sym_bits + 31) / 32 + 4;
        u32* const gramhist = bytehist; // (read back already)
        HIP_TRY(hipMemsetAsync(gramhist, 0, RADIX_BINS * sizeof(u32), s));
        const u64 enc_blocks = (ps.words + ENCODE_BLOCK - 1) / ENCODE_BLOCK;
        hipLaunchKernelGGL(encode_text_kernel, dim3((u32)(enc_blocks < 4096 ? enc_blocks : 4096)), dim3(ENCODE_BLOCK), 0, s, d_text, n,
                           pp.codes, stream, ps.words, gramhist);
        const PassPlan plan = make_plan(0, (int)ps.key_bits);
        hipLaunchKernelGGL(packed_hist_expand_kernel, dim3(1), dim3(256), 0, s, ps.stream, n, ps.sym_bits, pp.codes.key_syms,
                           plan.num_passes, gramhist, h->ghist);
        HIP_TRY(hipGetLastError());
        rc = radix_sort(L, SRC_PACKED, d_text, n, tail, 0, K[0], V[0], K[1], V[1], n, plan, &in_out, &p1, nullptr, 0, 0, &ps, 2);
    } else {
        rc = radix_sort(L, SRC_TEXT, d_text, n, tail, 0, K[0], V[0], K[1], V[1], n, make_plan(0, 64), &in_out, &p1, nullptr, 0, 0,
                        nullptr, 1);
    }
    if (rc)
        return rc;
    passes += p1;
    if (in_out)
        cur = 1;
    u64* k_sorted = K[cur];
    u32* sa32 = V[cur]; // from here on the suffix array under construction
    // roles of the remaining arrays in generations t >= 1
    u32* ax = V[cur ^ 1];        // active list: suffixes ...
    u32* agid = h->gid;          // ... and their dense group ids
    u64* key_out = K[cur ^ 1];   // the active list sorted by (group, rank[x + h])
    u32* x_out = h->idx[2];
    u64* bkey[2] = {h->key[2], k_sorted}; // large groups on their way through the radix sort
    u32* bx[2] = {h->idx[3], h->idx[4]};  // (k_sorted is free once generation 0 has been ranked)

    RerankArgs ra;
    memset(&ra, 0, sizeof(ra));
    ra.keys = k_sorted;
    ra.sufs = sa32;
    ra.m = n;
    ra.key_words = 1;
    ra.n = n;
    ra.ell = ell;
    ra.text = d_text;
    ra.rank = h->rank;
    ra.sufs_out = ax;
    ra.gids_out = agid;
    ra.gprim_out = h->gprim[0];
    ra.gstart_out = h->gstart[0];
    // scratch of the bucketed rank update: all free while (and after) a list is being ranked
    // (the records of generation 0 start in the third key array and swap with the sort's other output array; the sorted
    // keys themselves are still being read when the first records are written)
    auto defer_buffers = [&]() { // (by the roles the arrays have when it is asked for: a dense generation swaps two of them)
        return DeferBuffers{{bkey[0], key_out}, bx[0], bx[1], reinterpret_cast<u32*>(bkey[0]), reinterpret_cast<u32*>(bkey[1]),
                            reinterpret_cast<u32*>(bkey[1]) + h->cap};
    };
    u32 m = 0, groups = 0, big = 0;
    // packed keys: what the generations that the first sort covers would have left (contexts 4 W, 8 W, ... symbols)
    u32 level_counts[2 * MAX_LEVELS]; // (survivors, groups) of each
    if (pp.skipped > MAX_LEVELS)
        return fail(CSA_ERR_INTERNAL, "the first sort covers %u generations", pp.skipped);
    ra.levels = pp.skipped;
    for (u32 i = 0; i < pp.skipped; ++i) {
        ra.level_ell[i] = (u32)wide_ell << i;
        ra.level_drop[i] = (ell - ra.level_ell[i]) * pp.codes.bits;
    }
    rc = rerank_step(L, ra, defer_buffers(), &m, &groups, &st->rank_update[0], level_counts);
    range_gen0.close();
    if (rc)
        return rc;
    bool ordinals_in_rank = ra.ordinals != 0; // rank[] holds run ordinals instead of ranks: the coming generation is dense
    st->passes[0] = passes;
    st->active[0] = n;
    st->groups[0] = 0;
    HIP_TRY(hipEventRecord(h->ev_gen[1], s));

    // ---- generations t >= 1 (reference loop: src/GPU_SACA.cu:1999-2103) ----
    int gen = 1;
    int gp = 0; // gprim[gp] / gstart[gp] describe the current groups
    bool all_small = false; // no group of the current list exceeds the limit of the generation that found it so
    bool presorted_before = false; // every large group of the generation before was in order as it stood
    bool high_limit = false; // that generation's limit was SMALL_MAXG_HI (groups only split: the limit stays from there on)
    const int sec_bits = bit_length(n > 1 ? n - 1 : 1);
    u64 ctx = ell; // symbols resolved so far; the next generation looks hop symbols ahead
    while (m > 0) {
        if (gen >= CSA_MAX_GENERATIONS)
            return fail(CSA_ERR_INTERNAL, "generation cap reached with %u suffixes still active", m);
        st->active[gen] = m;
        st->groups[gen] = groups;
        const u32 m_in = m;
        RangeScope range_g("generation %d m=%u groups=%u", gen, m, groups);
        const u64 hop = ctx < wide_ell ? (ctx < wide_ell - ctx ? ctx : wide_ell - ctx) : ctx;
        // A dense generation: most of the partition is still active and its groups are long (a small alphabet, a
        // periodic text), so nearly every member would go through the radix sort anyway. Then the whole partition is sorted
        // again, as in generation 0, by keys that are read in text order: (rank[x], rank[x + hop]) for x = 0, 1, ...,
        // two coalesced streams instead of one random gather per member; the ranks come out of the same run ranking as
        // in generation 0 and go back to rank[] through the bucketed update instead of scattered writes. Suffixes that had
        // retired are alone with their rank: they sort to the place they hold already and keep their rank.
        const bool dense = dense_generation(m_in, groups, n);
        if (dense) {
            // A generation that runs in this form itself, or generation 0, knew that this one would be dense (the same test on
            // the same numbers) and left ordinals in rank[]: the key runs of its sorted list numbered 0, 1, 2, ...; there
            // are as many as it had groups and singletons. Two ordinals make a key of 2 log2(runs) bits: 17 bits after
            // generation 0 of a four-letter text (256 groups and the last four suffixes), three passes where two 31-bit ranks
            // take eight. A generation of the other form leaves ranks, and the list it leaves can still qualify (its many
            // short groups dissolved, a few long ones are left): the key is then the two ranks side by side.
            passes = 0;
            if (ordinals_in_rank) {
                const u64 runs = (u64)groups + ((u64)n - m_in);
                const u32 radix = (u32)runs;
                const PassPlan plan = make_plan(0, runs > 1 ? bit_length(runs * runs - 1) : 1);
                rc = radix_sort(L, SRC_RANKS, nullptr, n, 0, 0, bkey[0], bx[0], bkey[1], bx[1], n, plan, &in_out, &passes, h->rank,
                                (u32)hop, radix);
            } else {
                PassPlan plan; // the digits of the two ranks of a key: bits [0, sec_bits) and [32, 32 + sec_bits)
                plan.num_passes = 0;
                for (int half = 0; half < 2; ++half)
                    for (int b = 0; b < sec_bits; b += RADIX_BITS) {
                        plan.shift[plan.num_passes] = 32 * half + b;
                        plan.bits[plan.num_passes] = sec_bits - b < RADIX_BITS ? sec_bits - b : RADIX_BITS;
                        plan.num_passes++;
                    }
                rc = radix_sort(L, SRC_RANKS, nullptr, n, 0, 0, bkey[0], bx[0], bkey[1], bx[1], n, plan, &in_out, &passes, h->rank,
                                (u32)hop, 0u);
            }
            if (rc)
                return rc;
            RerankArgs rd;
            memset(&rd, 0, sizeof(rd));
            rd.keys = bkey[in_out];
            rd.sufs = bx[in_out];
            rd.m = n;
            rd.key_words = 1;
            rd.n = n;
            rd.ell = 0; // no suffix is set apart for running off the text: the tied ones never do, the others are alone anyway
            rd.text = d_text;
            rd.rank = h->rank;
            rd.sufs_out = ax;
            rd.gids_out = agid;
            rd.gprim_out = h->gprim[gp ^ 1];
            rd.gstart_out = h->gstart[gp ^ 1];
            DeferBuffers db = defer_buffers();
            db.recs[0] = bkey[in_out ^ 1]; // the records of the rank update: the two 8-byte arrays that do not hold the sorted keys
            db.recs[1] = key_out;
            rc = rerank_step(L, rd, db, &m, &groups, &st->rank_update[gen]);
            if (rc)
                return rc;
            ordinals_in_rank = rd.ordinals != 0;
            // the freshly sorted index array is the suffix array under construction from here on; the old one is scratch
            u32* const old_sa32 = sa32;
            sa32 = bx[in_out];
            bx[in_out] = old_sa32;
            big = m_in;
            st->big[gen] = m_in;
            st->passes[gen] = passes;
            st->dense[gen] = 1;
            all_small = false;
            presorted_before = false;
            gp ^= 1;
            HIP_TRY(hipEventRecord(h->ev_gen[gen + 1], s));
            gen++;
            ctx += hop;
            continue;
        }
        if (ordinals_in_rank)
            return fail(CSA_ERR_INTERNAL, "generation %d reads ranks but the one before it left ordinals", gen);
        const RankTables r = rank_tables(h, m_in, SMALL_TILE);
        u32* nr_list = reinterpret_cast<u32*>(key_out); // refined rank at every place of the sorted list
        // 1. gather rank[x + h]; small groups are sorted and ranked inside their tile, members of large groups set aside
        SmallSortArgs sa;
        memset(&sa, 0, sizeof(sa));
        sa.sufs = ax;
        sa.gids = agid;
        sa.gstart = h->gstart[gp];
        sa.gprim = h->gprim[gp];
        sa.rank = h->rank;
        sa.m = m_in;
        sa.n = n;
        sa.h = (u32)hop;
        sa.sec_bits = sec_bits;
        sa.groups = groups;
        sa.err = h->counts + 2;
        sa.sufs_out = x_out;
        sa.nr_out = nr_list;
        sa.big_keys = bkey[0];
        sa.big_sufs = bx[0];
        sa.big_first = reinterpret_cast<const u32*>(bkey[1]); // (free until the radix sort, which starts after the kernel that reads it)
        sa.tile_agg = r.tile_agg;
        sa.tile_splits = r.tile_splits;
        passes = 0;
        if (all_small) {
            // Groups only ever split: once a generation had no large group, none can appear again. The small-group
            // kernel then also counts for the apply step, and nothing else runs before it.
            HIP_TRY(hipMemsetAsync(r.tile_agg, 0, (u64)r.tiles * 4 * sizeof(u32), s));
            HIP_TRY(hipMemsetAsync(r.tile_splits, 0, (u64)r.tiles * sizeof(u32), s));
            if (high_limit)
                hipLaunchKernelGGL((smallsort_kernel<SMALL_BLOCK, SMALL_ITEMS, SMALL_MAXG_HI, true>), dim3(r.tiles), dim3(SMALL_BLOCK), 0,
                                   s, sa);
            else
                hipLaunchKernelGGL((smallsort_kernel<SMALL_BLOCK, SMALL_ITEMS, SMALL_MAXG, true>), dim3(r.tiles), dim3(SMALL_BLOCK), 0, s,
                                   sa);
            HIP_TRY(hipGetLastError());
            st->small_only[gen] = 1;
        } else {
            HIP_TRY(hipMemsetAsync(h->counts + 4, 0, 2 * sizeof(u32), s));
            // marks of the large groups whose gathered ranks are out of order, in the tables the next generation's groups
            // will be written to (free until the apply step)
            sa.big_sec = bx[1];
            sa.not_asc = h->gprim[gp ^ 1];
            sa.not_desc = h->gstart[gp ^ 1];
            high_limit = (u64)m_in <= (u64)groups * SMALL_AVG_LIMIT;
            const u32 maxg = high_limit ? (u32)SMALL_MAXG_HI : (u32)SMALL_MAXG;
            const u32 marks = m_in / maxg + 2u; // one mark index per large group at most
            HIP_TRY(hipMemsetAsync(sa.not_asc, 0, (u64)marks * sizeof(u32), s));
            HIP_TRY(hipMemsetAsync(sa.not_desc, 0, (u64)marks * sizeof(u32), s));
            {
                // where every large group's members start in the list of large-group members, and how many there are
                // (counts[4]): a prefix sum over the group table
                u32* big_first = reinterpret_cast<u32*>(bkey[1]);
                const RankTables gr = rank_tables(h, groups, 1024);
                hipLaunchKernelGGL((big_prefix_kernel<false>), dim3(gr.tiles), dim3(256), 0, s, (const u32*)h->gstart[gp], groups, maxg, big_first,
                                   gr.tile_agg, gr.tile_splits, (const u32*)gr.tile_prefix, (const u32*)gr.slab_total, gr.slab, gr.slabs,
                                   h->counts + 4);
                hipLaunchKernelGGL(rerank_scan_kernel, dim3(gr.slabs), dim3(1024), 0, s, gr.tile_agg, gr.tile_prefix, gr.tiles, gr.slab,
                                   gr.slab_total, gr.tile_splits);
                hipLaunchKernelGGL((big_prefix_kernel<true>), dim3(gr.tiles), dim3(256), 0, s, (const u32*)h->gstart[gp], groups, maxg, big_first,
                                   gr.tile_agg, gr.tile_splits, (const u32*)gr.tile_prefix, (const u32*)gr.slab_total, gr.slab, gr.slabs,
                                   h->counts + 4);
            }
            auto gather_and_sort_small = [&]() {
                if (high_limit)
                    hipLaunchKernelGGL((smallsort_kernel<SMALL_BLOCK, SMALL_ITEMS, SMALL_MAXG_HI, false>), dim3(r.tiles), dim3(SMALL_BLOCK),
                                       0, s, sa);
                else
                    hipLaunchKernelGGL((smallsort_kernel<SMALL_BLOCK, SMALL_ITEMS, SMALL_MAXG, false>), dim3(r.tiles), dim3(SMALL_BLOCK), 0,
                                       s, sa);
            };
            // A list whose large groups were all in order in the generation before (a run, a period: they stay so until
            // they dissolve) is expected to be so again: the (key, suffix) pairs for the radix sort, 12 of the 16 bytes the
            // kernel writes per member of a large group, are then left out, and the kernel runs once more with them in
            // the rare generation in which the marks say otherwise.
            sa.side_list = (presorted_before || h->expect_presorted) ? 0u : 1u;
            gather_and_sort_small();
            hipLaunchKernelGGL(group_order_kernel, dim3((marks + 255u) / 256u), dim3(256), 0, s, (const u32*)sa.not_asc, (const u32*)sa.not_desc,
                               marks, h->counts + 5);
            HIP_TRY(hipGetLastError());
            rc = read_counts(L, &big);
            if (rc)
                return rc;
            all_small = big == 0;
            const u32 unordered = h->h_pinned[5];
            if (big > 0 && unordered != 0 && !sa.side_list) {
                sa.side_list = 1u;
                gather_and_sort_small();
                HIP_TRY(hipGetLastError());
            }
            presorted_before = big > 0 && unordered == 0;
            if (big > 0 && unordered == 0) {
                // 2a. every large group is in order as it stands (runs of one token, periodic stretches: the gathered ranks
                //     rise or fall along the list): no sort, the members are ranked by their runs of equal gathered ranks
                PresortedArgs pa;
                pa.sufs = ax;
                pa.gids = agid;
                pa.big_sec = sa.big_sec;
                pa.gstart = h->gstart[gp];
                pa.gprim = h->gprim[gp];
                pa.big_first = sa.big_first;
                pa.not_asc = sa.not_asc;
                pa.m = m_in;
                pa.n = n;
                pa.groups = groups;
                pa.maxg = maxg;
                pa.sufs_out = x_out;
                pa.nr_out = nr_list;
                pa.err = h->counts + 2;
                // (512 x 4 tiles: 0.8 ms per sort of the adversarial workload ahead of 256 x 4; 8 elements per thread: 8 ms behind)
                constexpr int PRESORTED_BLOCK = 512, PRESORTED_ITEMS = 4;
                const RankTables pr = rank_tables(h, m_in, PRESORTED_BLOCK * PRESORTED_ITEMS);
                pa.tile_agg = pr.tile_agg;
                pa.tile_splits = pr.tile_splits;
                pa.tile_prefix = pr.tile_prefix;
                pa.slab_total = pr.slab_total;
                pa.slab = pr.slab;
                hipLaunchKernelGGL((place_presorted_kernel<PRESORTED_BLOCK, PRESORTED_ITEMS, false>), dim3(pr.tiles), dim3(PRESORTED_BLOCK), 0, s, pa);
                hipLaunchKernelGGL(rerank_scan_kernel, dim3(pr.slabs), dim3(1024), 0, s, pr.tile_agg, pr.tile_prefix, pr.tiles, pr.slab,
                                   pr.slab_total, pr.tile_splits);
                hipLaunchKernelGGL((place_presorted_kernel<PRESORTED_BLOCK, PRESORTED_ITEMS, true>), dim3(pr.tiles), dim3(PRESORTED_BLOCK), 0, s, pa);
                HIP_TRY(hipGetLastError());
                st->presorted[gen] = big;
            }
            // 2. the large groups: radix sort on (group id, rank[x + h]), then back into the list as (suffix, refined rank)
            if (big > 0 && unordered != 0) {
                const int gid_bits = bit_length(groups > 1 ? groups - 1 : 0);
                const PassPlan plan = make_plan(0, sec_bits + gid_bits);
                rc = radix_sort(L, SRC_PAIRS, nullptr, n, 0, 0, bkey[0], bx[0], bkey[1], bx[1], big, plan, &in_out, &passes);
                if (rc)
                    return rc;
                PlaceArgs pa;
                pa.big_keys = bkey[in_out];
                pa.big_sufs = bx[in_out];
                pa.mb = big;
                pa.m = m_in;
                pa.n = n;
                pa.groups = groups;
                pa.sec_bits = sec_bits;
                pa.gstart = h->gstart[gp];
                pa.gprim = h->gprim[gp];
                pa.sufs_out = x_out;
                pa.nr_out = nr_list;
                pa.err = h->counts + 2;
                // (the tile tables are free between the small-group kernel and the counting pass below)
                const RankTables pr = rank_tables(h, big, RANK_TILE);
                pa.tile_agg = pr.tile_agg;
                pa.tile_splits = pr.tile_splits;
                pa.tile_prefix = pr.tile_prefix;
                pa.slab_total = pr.slab_total;
                pa.slab = pr.slab;
                hipLaunchKernelGGL((place_big_kernel<RANK_BLOCK, RANK_ITEMS, false>), dim3(pr.tiles), dim3(RANK_BLOCK), 0, s, pa);
                hipLaunchKernelGGL(rerank_scan_kernel, dim3(pr.slabs), dim3(1024), 0, s, pr.tile_agg, pr.tile_prefix, pr.tiles, pr.slab,
                                   pr.slab_total, pr.tile_splits);
                hipLaunchKernelGGL((place_big_kernel<RANK_BLOCK, RANK_ITEMS, true>), dim3(pr.tiles), dim3(RANK_BLOCK), 0, s, pa);
                HIP_TRY(hipGetLastError());
            }
            // 3. per-tile counts of the sorted list (4 bytes read per member)
            hipLaunchKernelGGL((count_ranks_kernel<SMALL_BLOCK, SMALL_ITEMS>), dim3(r.tiles), dim3(SMALL_BLOCK), 0, s, nr_list, m_in,
                               r.tile_agg, r.tile_splits);
            HIP_TRY(hipGetLastError());
        }
        st->big[gen] = big;
        // 4. scan, totals to the host, apply: retire singletons, compact survivors, write the changed ranks
        rc = rank_totals(L, r, false, m_in, n, all_small && big == 0, &m, &groups, &st->rank_update[gen]);
        if (rc)
            return rc;
        ApplySmallArgs aa;
        aa.sufs = x_out;
        aa.nr = nr_list;
        aa.m = m_in;
        aa.n = n;
        aa.rank = h->rank;
        const DeferBuffers defer_buf = defer_buffers();
        aa.rank_vals = st->rank_update[gen] == 2 ? defer_buf.vals : nullptr;
        aa.sa32 = sa32;
        aa.sufs_out = ax;
        aa.gids_out = agid;
        aa.gprim_out = h->gprim[gp ^ 1];
        aa.gstart_out = h->gstart[gp ^ 1];
        aa.tile_prefix = r.tile_prefix;
        aa.slab_total = r.slab_total;
        aa.slab = r.slab;
        aa.err = h->counts + 2;
        hipLaunchKernelGGL((apply_small_kernel<SMALL_BLOCK, SMALL_ITEMS>), dim3(r.tiles), dim3(SMALL_BLOCK), 0, s, aa);
        HIP_TRY(hipGetLastError());
        if (st->rank_update[gen] == 2) {
            rc = windowed_rank_update(L, x_out, defer_buf, m_in, n);
            if (rc)
                return rc;
        }
        gp ^= 1;
        st->passes[gen] = passes;
        HIP_TRY(hipEventRecord(h->ev_gen[gen + 1], s));
        gen++;
        ctx += hop;
    }
    st->generations = gen;

    // ---- output: 5-byte little-endian entries in rank order ----
    const int aligned4 = ((uintptr_t)d_sa40 & 3u) == 0;
    const u64 quads = ((u64)n + 3) / 4;
    hipLaunchKernelGGL(emit_sa40_kernel, dim3((u32)((quads + 255) / 256)), dim3(256), 0, s, sa32, n, index_base, d_sa40,
                       aligned4);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipEventRecord(h->ev_gen[gen + 1], s));
    rc = read_counts(L, nullptr); // waits for the stream; the last apply pass may still have raised the error word
    if (rc)
        return rc;

    for (int g = 0; g < gen; ++g)
        HIP_TRY(hipEventElapsedTime(&st->ms[g], h->ev_gen[g], h->ev_gen[g + 1]));
    HIP_TRY(hipEventElapsedTime(&st->ms_output, h->ev_gen[gen], h->ev_gen[gen + 1]));
    HIP_TRY(hipEventElapsedTime(&st->ms_total, h->ev_gen[0], h->ev_gen[gen + 1]));
    for (auto& tl : L.timed) {
        float ms = 0;
        HIP_TRY(hipEventElapsedTime(&ms, h->events[tl.first], h->events[tl.first + 1]));
        st->radix_ms += ms;
        st->radix_pairs += tl.second;
        st->radix_launches++;
    }
    // wide keys: the first generations that ran stand for generation 0
    const int merged = folded < gen - 1 ? folded : gen - 1;
    if (merged > 0) {
        for (int g = 1; g <= merged; ++g) {
            st->ms[0] += st->ms[g];
            st->passes[0] += st->passes[g];
        }
        for (int g = 1; g + merged < gen; ++g) {
            st->active[g] = st->active[g + merged];
            st->groups[g] = st->groups[g + merged];
            st->big[g] = st->big[g + merged];
            st->presorted[g] = st->presorted[g + merged];
            st->passes[g] = st->passes[g + merged];
            st->rank_update[g] = st->rank_update[g + merged];
            st->small_only[g] = st->small_only[g + merged];
            st->dense[g] = st->dense[g + merged];
            st->ms[g] = st->ms[g + merged];
        }
        for (int g = gen - merged; g < gen; ++g) {
            st->active[g] = st->groups[g] = st->big[g] = st->presorted[g] = 0;
            st->passes[g] = st->rank_update[g] = st->small_only[g] = st->dense[g] = 0;
            st->ms[g] = 0.0f;
        }
        st->generations = gen - merged;
    }
    // packed keys: the first sort stands for generations 0 .. skipped of the reference; those after the first are reported
    // with the lists they would have had and no time or passes of their own
    st->key_symbols = ell;
    st->first_sort_generations = 1 + pp.skipped;
    if (pp.skipped > 0) {
        const int sk = (int)pp.skipped;
        if (gen + sk > CSA_MAX_GENERATIONS)
            return fail(CSA_ERR_INTERNAL, "%d generations do not fit the statistics", gen + sk);
        for (int g = gen - 1; g >= 1; --g) {
            st->active[g + sk] = st->active[g];
            st->groups[g + sk] = st->groups[g];
            st->big[g + sk] = st->big[g];
            st->presorted[g + sk] = st->presorted[g];
            st->passes[g + sk] = st->passes[g];
            st->rank_update[g + sk] = st->rank_update[g];
            st->small_only[g + sk] = st->small_only[g];
            st->dense[g + sk] = st->dense[g];
            st->ms[g + sk] = st->ms[g];
        }
        for (int g = 1; g <= sk; ++g) {
            st->active[g] = level_counts[2 * (g - 1)];
            st->groups[g] = level_counts[2 * (g - 1) + 1];
            st->big[g] = st->presorted[g] = 0;
            st->passes[g] = st->rank_update[g] = st->small_only[g] = st->dense[g] = 0;
            st->ms[g] = 0.0f;
        }
        st->generations = gen + sk;
        // the reference stops at the first generation that leaves nothing active
        for (int g = 1; g <= sk; ++g)
            if (st->active[g] == 0) {
                st->generations = g;
                break;
            }
    }
    return CSA_OK;
}

} // namespace

extern "C" {

uint32_t csa_partition_id_bits(uint32_t p)
{
    const int id_bits = p <= 1 ? 0 : bit_length((u64)p - 1);
    return (u32)(id_bits < 1 ? 1 : id_bits) + 1u;
}

int csa_partition_ids_u16_dev(const uint16_t* d_text, uint64_t n, uint64_t text_len, const uint64_t* d_pivots,
                              int pivot_words, uint32_t p, uint16_t* d_pid, uint64_t* d_packed, uint64_t* d_psz,
                              void* stream)
{
    if (p < 1 || p > 65536u)
        return fail(CSA_ERR_ARG, "csa_partition_ids_u16_dev: p = %u is outside [1, 65536]", p);
    if (pivot_words < 1 || pivot_words > 4)
        return fail(CSA_ERR_ARG, "csa_partition_ids_u16_dev: pivot_words = %d is outside [1, 4]", pivot_words);
    if (n == 0)
        return CSA_OK;
    if (!d_text || (p > 1 && !d_pivots) || text_len < n)
        return fail(CSA_ERR_ARG, "csa_partition_ids_u16_dev: null text or pivots, or text_len < n");
    const u64 tiles64 = (n + PID_TILE - 1) / PID_TILE;
    if (tiles64 > 0xFFFFFFFFull)
        return fail(CSA_ERR_TOO_LARGE, "csa_partition_ids_u16_dev: %llu suffixes in one call", (unsigned long long)n);
    PartitionIdArgs a;
    a.text = d_text;
    a.n = n;
    a.text_len = text_len;
    a.pivots = d_pivots;
    a.p = p;
    a.bits = csa_partition_id_bits(p);
    a.pid = d_pid;
    a.packed = d_packed;
    a.psz = reinterpret_cast<unsigned long long*>(d_psz);
    a.tiles = (u32)tiles64;
    const u32 grid = a.tiles < 8192u ? a.tiles : 8192u;
    hipStream_t s = (hipStream_t)stream;
    // (the table in LDS is filled up to 2^bits(p - 1) - 1 entries)
    const bool piv_lds = (((u64)1 << bit_length((u64)(p - 1))) - 1) * (u64)pivot_words <= PID_LDS_PIVOT_WORDS;
    const u32 lds = partition_ids_lds_bytes(pivot_words, p, piv_lds, d_psz != nullptr, d_packed != nullptr, a.bits, &a.hist_copies_log2);
#define CSA_LAUNCH_PID(W)                                                                                  \
    do {                                                                                                   \
        if (piv_lds)                                                                                       \
            hipLaunchKernelGGL((partition_ids_kernel<W, true>), dim3(grid), dim3(PID_BLOCK), lds, s, a);  \
        else                                                                                               \
            hipLaunchKernelGGL((partition_ids_kernel<W, false>), dim3(grid), dim3(PID_BLOCK), lds, s, a); \
    } while (0)
    switch (pivot_words) {
    case 1: CSA_LAUNCH_PID(1); break;
    case 2: CSA_LAUNCH_PID(2); break;
    case 3: CSA_LAUNCH_PID(3); break;
    default: CSA_LAUNCH_PID(4); break;
    }
#undef CSA_LAUNCH_PID
    HIP_TRY(hipGetLastError());
    return CSA_OK;
}

namespace {
int fill_message_args(MessageArgs& a, const char* who, const uint64_t* d_sa, const uint64_t* d_keys, const uint32_t* d_beta,
                      uint64_t n, uint64_t ctx, int packed_keys, uint32_t p)
{
    if (p < 1 || p > 32768u)
        return fail(CSA_ERR_ARG, "%s: p = %u is outside [1, 32768]", who, p);
    if (n > CSA_MAX_PART_SZ)
        return fail(CSA_ERR_TOO_LARGE, "%s: %llu suffixes exceed a partition", who, (unsigned long long)n);
    if (n && (!d_sa || !d_keys || !d_beta))
        return fail(CSA_ERR_ARG, "%s: null buffer", who);
    a.sa = d_sa;
    a.keys = d_keys;
    a.beta = d_beta;
    a.n = n;
    a.ctx = ctx;
    a.packed = packed_keys ? 1 : 0;
    a.active_sz = nullptr;
    a.p = p;
    a.msg_target = nullptr;
    a.msg_rank = nullptr;
    a.msg_off = nullptr;
    a.tiles = (u32)((n + MSG_TILE - 1) / MSG_TILE);
    return CSA_OK;
}
} // namespace

int csa_count_messages_dev(const uint64_t* d_sa, const uint64_t* d_keys, const uint32_t* d_beta, uint64_t n, uint64_t ctx,
                           int packed_keys, uint32_t p, uint32_t* d_msg_count, void* stream)
{
    MessageArgs a;
    const int rc = fill_message_args(a, "csa_count_messages_dev", d_sa, d_keys, d_beta, n, ctx, packed_keys, p);
    if (rc || n == 0)
        return rc;
    if (!d_msg_count)
        return fail(CSA_ERR_ARG, "csa_count_messages_dev: null counters");
    a.msg_off = d_msg_count;
    hipLaunchKernelGGL(count_messages_kernel, dim3(a.tiles < 4096u ? a.tiles : 4096u), dim3(MSG_BLOCK), 0, (hipStream_t)stream, a);
    HIP_TRY(hipGetLastError());
    return CSA_OK;
}

int csa_message_offsets_dev(uint32_t* d_msg_off, uint32_t count, void* stream)
{
    if (count == 0)
        return CSA_OK;
    if (!d_msg_off || count > 32769u)
        return fail(CSA_ERR_ARG, "csa_message_offsets_dev: null counters or more than 32769 of them");
    hipLaunchKernelGGL(message_offsets_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, d_msg_off, count);
    HIP_TRY(hipGetLastError());
    return CSA_OK;
}

int csa_emit_messages_dev(const uint64_t* d_sa, const uint64_t* d_keys, const uint32_t* d_beta, uint64_t n, uint64_t ctx,
                          int packed_keys, const uint64_t* d_active_sz, uint32_t p, uint8_t* d_msg_target,
                          uint32_t* d_msg_rank, uint32_t* d_msg_off, void* stream)
{
    MessageArgs a;
    const int rc = fill_message_args(a, "csa_emit_messages_dev", d_sa, d_keys, d_beta, n, ctx, packed_keys, p);
    if (rc || n == 0)
        return rc;
    if (!d_active_sz || !d_msg_target || !d_msg_rank || !d_msg_off)
        return fail(CSA_ERR_ARG, "csa_emit_messages_dev: null buffer");
    a.active_sz = reinterpret_cast<const unsigned long long*>(d_active_sz);
    a.msg_target = d_msg_target;
    a.msg_rank = d_msg_rank;
    a.msg_off = d_msg_off;
    const u64 emit_tiles = (n + EMIT_TILE - 1) / EMIT_TILE;
    if (a.p <= EMIT_FEW_PARTS)
        hipLaunchKernelGGL((emit_messages_kernel<EMIT_FEW_PARTS>), dim3((u32)(emit_tiles < 2048u ? emit_tiles : 2048u)), dim3(EMIT_BLOCK), 0, (hipStream_t)stream, a);
    else
        hipLaunchKernelGGL((emit_messages_kernel<MSG_LDS_PARTS>), dim3((u32)(emit_tiles < 2048u ? emit_tiles : 2048u)), dim3(EMIT_BLOCK), 0, (hipStream_t)stream, a);
    HIP_TRY(hipGetLastError());
    return CSA_OK;
}

extern "C++" {
namespace {
// Builds the join directory of the suffix-ordered cohort d_sa[0, n) in `dir` (room for `room` entries) and returns the
// log2 of its bucket count through *dir_log2; leaves *dir_log2 = 0 and builds nothing when the cohort is small.
int build_join_directory(const u64* d_sa, u64 n, u32* dir, u64 room, hipStream_t s, u32* dir_log2, bool sorted_probes)
{
    *dir_log2 = 0;
    if (n < CSA_JOIN_DIR_MIN || room < 3)
        return CSA_OK;
    // Probes in arrival order: one to two cohort entries per bucket, so that a probe costs the directory's line and one
    // line of the cohort (with at most 2^22 buckets a cohort of 44 M suffixes had 10 per bucket and the join of 268 M
    // messages took 14.5 ms instead of 9.5). Probes sorted by target walk the cohort and the directory in order and find
    // their lines in cache: a coarse directory (two to four entries per bucket, at most 2^22 buckets) is built four
    // times faster and serves them as well.
    u32 lg = (u32)bit_length(n) - (sorted_probes ? 2u : 1u);
    const u32 cap = sorted_probes ? 22u : 26u;
    if (lg > cap)
        lg = cap;
    while (lg && (1ull << lg) + 1 > room)
        --lg;
    if (lg == 0)
        return CSA_OK;
    hipLaunchKernelGGL(join_directory_kernel, dim3((u32)(((1ull << lg) + 256) / 256)), dim3(256), 0, s, d_sa, n, lg, dir);
    HIP_TRY(hipGetLastError());
    *dir_log2 = lg;
    return CSA_OK;
}
} // namespace
} // extern "C++"

int csa_join_messages_dev(const uint8_t* d_msg_target, const uint32_t* d_msg_rank, uint32_t msg_c, const uint64_t* d_sa,
                          const uint32_t* d_primary, uint64_t* d_keys, uint64_t n, void* stream)
{
    if (msg_c == 0)
        return CSA_OK;
    if (!d_msg_target || !d_msg_rank || (n && (!d_sa || !d_primary || !d_keys)))
        return fail(CSA_ERR_ARG, "csa_join_messages_dev: null buffer");
    if (n > CSA_MAX_PART_SZ)
        return fail(CSA_ERR_TOO_LARGE, "csa_join_messages_dev: %llu suffixes exceed a partition", (unsigned long long)n);
    hipLaunchKernelGGL(join_messages_kernel, dim3((msg_c + 255u) / 256u), dim3(256), 0, (hipStream_t)stream, d_msg_target,
                       (const u64*)nullptr, d_msg_rank, msg_c, d_sa, d_primary, d_keys, n, (const u32*)nullptr, 0u);
    HIP_TRY(hipGetLastError());
    return CSA_OK;
}

int csa_join_messages_sorted_dev(csa_handle* h, const uint8_t* d_msg_target, const uint32_t* d_msg_rank, uint32_t msg_c,
                                 const uint64_t* d_sa, const uint32_t* d_primary, uint64_t* d_keys, uint64_t n, void* stream)
{
    if (!h)
        return fail(CSA_ERR_ARG, "csa_join_messages_sorted_dev: null handle");
    if (msg_c == 0)
        return CSA_OK;
    if (!d_msg_target || !d_msg_rank || (n && (!d_sa || !d_primary || !d_keys)))
        return fail(CSA_ERR_ARG, "csa_join_messages_sorted_dev: null buffer");
    if (n > CSA_MAX_PART_SZ)
        return fail(CSA_ERR_TOO_LARGE, "csa_join_messages_sorted_dev: %llu suffixes exceed a partition", (unsigned long long)n);
    if (msg_c > h->cap)
        return fail(CSA_ERR_ARG, "csa_join_messages_sorted_dev: %u messages exceed the handle's capacity %llu", msg_c,
                    (unsigned long long)h->cap);
    Launch L;
    L.h = h;
    L.stream = (hipStream_t)stream;
    L.flags = 0;
    L.stats = nullptr;
    hipStream_t s = L.stream;
    HIP_TRY(hipMemsetAsync(h->counts, 0, 4 * sizeof(u32), s));
    // (target word, rank) pairs in columns of the handle's block, sorted on the 40 target bits
    h->pool.reset();
    u64* K[2];
    u32* V[2];
    for (int i = 0; i < 2; ++i) {
        K[i] = static_cast<u64*>(h->pool.take((u64)msg_c * sizeof(u64)));
        V[i] = static_cast<u32*>(h->pool.take((u64)msg_c * sizeof(u32)));
    }
    if (!K[0] || !V[0] || !K[1] || !V[1])
        return fail(CSA_ERR_ARG, "csa_join_messages_sorted_dev: the handle's block of %llu bytes has no room for 24 bytes per message",
                    (unsigned long long)h->pool.bytes());
    // the directory over the cohort takes what is left, up to an entry per cohort member (a smaller one has longer buckets)
    u64 dir_room = n < 3 ? 3 : n;
    u32* dir = nullptr;
    while (dir_room >= 3 && !(dir = static_cast<u32*>(h->pool.take(dir_room * sizeof(u32)))))
        dir_room /= 2;
    if (!dir)
        dir_room = 0;
    h->last_high_water = h->pool.high_water();
    hipLaunchKernelGGL(unpack_lanes_kernel, dim3((msg_c + 255u) / 256u), dim3(256), 0, s, d_msg_target, (u64)msg_c, K[0]);
    HIP_TRY(hipMemcpyAsync(V[0], d_msg_rank, (u64)msg_c * sizeof(u32), hipMemcpyDeviceToDevice, s));
    int in_out = 0, passes = 0;
    const PassPlan plan = make_plan(0, 40);
    int rc = radix_sort(L, SRC_PAIRS, nullptr, 0, 0, 0, K[0], V[0], K[1], V[1], msg_c, plan, &in_out, &passes);
    if (rc)
        return rc;
    u32 dir_log2 = 0;
    rc = build_join_directory(d_sa, n, dir, dir_room, s, &dir_log2, true);
    if (rc)
        return rc;
    hipLaunchKernelGGL(join_messages_kernel, dim3((msg_c + 255u) / 256u), dim3(256), 0, s, (const u8*)nullptr,
                       (const u64*)K[in_out], (const u32*)V[in_out], msg_c, d_sa, d_primary, d_keys, n,
                       (const u32*)(dir_log2 ? dir : nullptr), dir_log2);
    HIP_TRY(hipGetLastError());
    return read_counts(L, nullptr);
}

int csa_stage_slab_u16_dev(const uint16_t* d_text, uint64_t n, const uint8_t* d_suf40, uint64_t count, int key_words,
                           const uint64_t* d_pid_map, uint32_t p, uint64_t ctx, int generation0, uint64_t* d_keys,
                           uint32_t* d_beta, void* stream)
{
    if (key_words < 1 || key_words > 4)
        return fail(CSA_ERR_ARG, "csa_stage_slab_u16_dev: key_words = %d is outside [1, 4]", key_words);
    if (p < 1 || p > 32768u)
        return fail(CSA_ERR_ARG, "csa_stage_slab_u16_dev: p = %u is outside [1, 32768] (bit 15 of a route is the retirement flag)", p);
    if (generation0 && ctx != 4ull * (u64)key_words)
        return fail(CSA_ERR_ARG, "csa_stage_slab_u16_dev: generation 0 runs at ctx = ell = %d", 4 * key_words);
    if (count == 0)
        return CSA_OK;
    if (!d_text || !d_suf40 || !d_pid_map || !d_beta)
        return fail(CSA_ERR_ARG, "csa_stage_slab_u16_dev: null buffer");
    if (n > CSA_MAX_INDEX)
        return fail(CSA_ERR_TOO_LARGE, "csa_stage_slab_u16_dev: text of %llu symbols", (unsigned long long)n);
    StageArgs a;
    a.text = d_text;
    a.n = n;
    a.suf40 = d_suf40;
    a.count = count;
    a.pid_map = d_pid_map;
    a.bits = csa_partition_id_bits(p);
    a.ctx = ctx;
    a.ell = 4u * (u32)key_words;
    a.gen0 = generation0 ? 1 : 0;
    a.keys = d_keys;
    a.beta = d_beta;
    const u64 blocks = (count + 255) / 256;
    if (blocks > 0x7FFFFFFFull)
        return fail(CSA_ERR_TOO_LARGE, "csa_stage_slab_u16_dev: %llu suffixes in one call", (unsigned long long)count);
    hipStream_t s = (hipStream_t)stream;
    switch (key_words) {
    case 1: hipLaunchKernelGGL(stage_slab_kernel<1>, dim3((u32)blocks), dim3(256), 0, s, a); break;
    case 2: hipLaunchKernelGGL(stage_slab_kernel<2>, dim3((u32)blocks), dim3(256), 0, s, a); break;
    case 3: hipLaunchKernelGGL(stage_slab_kernel<3>, dim3((u32)blocks), dim3(256), 0, s, a); break;
    default: hipLaunchKernelGGL(stage_slab_kernel<4>, dim3((u32)blocks), dim3(256), 0, s, a); break;
    }
    HIP_TRY(hipGetLastError());
    return CSA_OK;
}

extern "C++" {
namespace {
// The scatter behind csa_scatter_to_rank_order_dev and csa_scatter_slabs; takes its columns from the handle's block as
// that block stands (the caller has reset it, or holds columns of its own in it). Waits for the stream.
int scatter_to_rank_order(csa_handle* h, const char* who, const u8* d_suf, const u32* d_rank, u64 part_sz, u8* d_sa40, hipStream_t s)
{
    HIP_TRY(hipMemsetAsync(h->counts, 0, 4 * sizeof(u32), s));
    const u32 blocks = (u32)((part_sz + 255) / 256);
    u64* K[2] = {nullptr, nullptr};
    u32* V[2] = {nullptr, nullptr};
    bool windowed = part_sz >= SCATTER_WINDOW_MIN && part_sz <= h->cap;
    if (windowed) { // (a block without room for the 24 bytes per suffix of the window pass scatters directly)
        for (int i = 0; i < 2; ++i) {
            K[i] = static_cast<u64*>(h->pool.take(part_sz * sizeof(u64)));
            V[i] = static_cast<u32*>(h->pool.take(part_sz * sizeof(u32)));
        }
        windowed = K[0] && V[0] && K[1] && V[1];
    }
    if (windowed) {
        // large partition: group the pairs by the window of the output their rank falls into, then write window by window
        Launch L;
        L.h = h;
        L.stream = s;
        L.flags = 0;
        L.stats = nullptr;
        hipLaunchKernelGGL(scatter_window_keys_kernel, dim3(blocks), dim3(256), 0, s, d_suf, d_rank, part_sz, (int)SCATTER_WINDOW_LOG2,
                           K[0], V[0], h->counts + 3);
        const int window_bits = bit_length((part_sz - 1) >> SCATTER_WINDOW_LOG2);
        int in_out = 0, passes = 0;
        const int rc = radix_sort(L, SRC_PAIRS, nullptr, 0, 0, 0, K[0], V[0], K[1], V[1], (u32)part_sz,
                                  make_plan(40, 40 + window_bits), &in_out, &passes);
        if (rc)
            return rc;
        hipLaunchKernelGGL(scatter_window_lanes_kernel, dim3(blocks), dim3(256), 0, s, (const u64*)K[in_out], (const u32*)V[in_out],
                           part_sz, d_sa40);
    } else {
        hipLaunchKernelGGL(scatter_lanes_kernel, dim3(blocks), dim3(256), 0, s, d_suf, d_rank, part_sz, d_sa40, h->counts + 3);
    }
    HIP_TRY(hipGetLastError());
    for (int i = 0; i < 2; ++i) {
        h->pool.give(K[i]);
        h->pool.give(V[i]);
    }
    Launch R;
    R.h = h;
    R.stream = s;
    R.flags = 0;
    R.stats = nullptr;
    const int rc_counts = read_counts(R, nullptr); // waits for the stream; a failed wait of the bucket pass ends here
    if (h->h_pinned[3])
        return fail(CSA_ERR_ARG, "%s: a rank lies outside [0, %llu)", who, (unsigned long long)part_sz);
    return rc_counts;
}
} // namespace
} // extern "C++"

int csa_scatter_to_rank_order_dev(csa_handle* h, const uint8_t* d_suf, const uint32_t* d_rank, uint64_t part_sz,
                                  uint8_t* d_sa40, void* stream)
{
    if (!h)
        return fail(CSA_ERR_ARG, "csa_scatter_to_rank_order_dev: null handle");
    if (part_sz == 0)
        return CSA_OK;
    if (!d_suf || !d_rank || !d_sa40)
        return fail(CSA_ERR_ARG, "csa_scatter_to_rank_order_dev: null buffer");
    if (part_sz > CSA_MAX_PART_SZ)
        return fail(CSA_ERR_TOO_LARGE, "csa_scatter_to_rank_order_dev: %llu suffixes exceed a partition", (unsigned long long)part_sz);
    h->pool.reset();
    const int rc = scatter_to_rank_order(h, "csa_scatter_to_rank_order_dev", d_suf, d_rank, part_sz, d_sa40, (hipStream_t)stream);
    h->last_high_water = h->pool.high_water();
    return rc;
}

void csa_output_cut(uint64_t lo, uint64_t hi, uint64_t chunk_bytes, uint64_t c, uint64_t chunk_c, uint64_t out[6])
{
    constexpr u64 BLK = 4096; // the O_DIRECT granularity of the output file (include/Direct_File.hpp:27)
    auto clamp = [](u64 v, u64 a, u64 b) { return v < a ? a : (v > b ? b : v); };
    const u64 first_block = lo & ~(BLK - 1);       // chunks are laid out from the block that holds the range's start
    const u64 aligned_lo = (lo + BLK - 1) & ~(BLK - 1);
    u64 aligned_hi = hi & ~(BLK - 1);              // [aligned_lo, aligned_hi): the whole blocks of the range
    if (aligned_hi < aligned_lo)
        aligned_hi = aligned_lo;                   // the range lies inside one block
    // the chunk's piece: its window of chunk_bytes, clipped to the whole blocks
    out[0] = clamp(first_block + c * chunk_bytes, aligned_lo, aligned_hi);
    out[1] = clamp(first_block + (c + 1) * chunk_bytes, out[0], aligned_hi);
    // the first chunk also carries what precedes the whole blocks, the last one what follows them
    out[2] = out[3] = out[4] = out[5] = 0;
    if (c == 0) {
        out[2] = lo;
        out[3] = hi < aligned_lo ? hi : aligned_lo;
    }
    if (c + 1 == chunk_c) {
        out[4] = aligned_hi;
        out[5] = hi > aligned_hi ? hi : aligned_hi;
    }
}

const char* csa_last_error(void) { return g_err; }

uint64_t csa_bytes_per_suffix(int key_words)
{
    (void)key_words;
    // three key arrays (8 B), five index arrays (4 B), group ids, ranks, four half-size group tables
    return 3 * 8 + 5 * 4 + 4 + 4 + 4 * 2;
}

extern "C++" {
namespace {

constexpr u64 BLOCK_SLACK = 64u << 10; // what rounding every column up to DevicePool::ALIGN can cost a call

struct WorkspaceSizes {
    u64 lookback_tile_words, lookback_words, rank_tiles_cap;
    u64 bytes;
};

// The workspace: what a handle holds besides its block. It follows the number of tiles, not the number of suffixes.
WorkspaceSizes workspace_sizes(u64 cap)
{
    WorkspaceSizes w;
    const u64 sort_tiles = (cap + SORT_TILE - 1) / SORT_TILE;
    const u64 rank_tiles = (cap + RANK_TILE - 1) / RANK_TILE;
    w.lookback_tile_words = sort_tiles * RADIX_BINS; // the group words of the radix pass follow the tile words
    w.lookback_words = w.lookback_tile_words + (sort_tiles / LB_GROUP + 1) * RADIX_BINS;
    if (rank_tiles * 4 > w.lookback_words)
        w.lookback_words = rank_tiles * 4;
    w.rank_tiles_cap = rank_tiles + 1;
    w.bytes = w.lookback_words * 8 + (w.rank_tiles_cap * 9 + RERANK_SLABS * 5) * sizeof(u32) + (MAX_PASSES + 2) * RADIX_BINS * 4 +
              MAX_PASSES * RADIX_BINS * 4 + TICKET_POOL * 4 + 16 * 4 + MSG_OFF_WORDS * 4;
    w.bytes += 9 * 4096; // nine allocations, each rounded up by the runtime
    return w;
}

u64 resident_block_bytes(u64 cap)
{
    const u64 A = DevicePool::ALIGN;
    auto up = [&](u64 b) { return (b + A - 1) & ~(A - 1); };
    return 3 * up(cap * 8) + 5 * up(cap * 4) + 2 * up(cap * 4) + 2 * up((cap / 2 + 1) * 4) + 2 * up((cap / 2 + 2) * 4);
}

int create_handle(const char* who, u64 max_part_sz, int key_words, u32 kinds, csa_handle** out)
{
    if (!out)
        return fail(CSA_ERR_ARG, "%s: out is null", who);
    *out = nullptr;
    if (key_words < 1 || key_words > 4)
        return fail(CSA_ERR_ARG, "%s: key_words = %d is outside [1, 4]", who, key_words);
    if (max_part_sz > CSA_MAX_PART_SZ)
        return fail(CSA_ERR_TOO_LARGE, "%s: %llu suffixes exceed the partition limit %llu", who,
                    (unsigned long long)max_part_sz, (unsigned long long)CSA_MAX_PART_SZ);
    csa_handle* h = new csa_handle();
    h->cap = max_part_sz ? max_part_sz : 1;
    h->key_words = key_words;
    h->kinds = kinds;
    const u64 cap = h->cap;
    const WorkspaceSizes ws = workspace_sizes(cap);
    h->lookback_tile_words = ws.lookback_tile_words;
    h->lookback_words = ws.lookback_words;
    hipError_t e = hipGetDevice(&h->device);
    if (e == hipSuccess)
        e = hipDeviceGetAttribute(&h->cus, hipDeviceAttributeMultiprocessorCount, h->device);
    // Tile order of the radix passes: by arrival, unless the caller declares the device its own
    // (csa_set_device_exclusive); the XCD-chunked order then needs 8 * XCD_CHUNK workgroups of a pass resident at once
    // and is offered only on a device with room for twice that many (csa_set_tuning changes the chunk length).
    h->tile_order = TILES_BY_ARRIVAL;
    h->tile_order_exclusive = h->cus >= 2 * 8 * (int)XCD_CHUNK ? TILES_STATIC_CHUNKS : TILES_BY_ARRIVAL;
    h->xcd_chunk = XCD_CHUNK;
    auto alloc = [&](void** p, u64 bytes) {
        if (e == hipSuccess)
            e = hipMalloc(p, bytes ? bytes : 4);
    };
    // the block: the resident sort's floor plan, or what the steps keep alive at their busiest moment
    u64 block_bytes = ((kinds & KIND_RESIDENT) ? resident_block_bytes(cap) : csa_step_bytes_per_suffix(key_words) * cap) + BLOCK_SLACK;
    block_bytes = (block_bytes + DevicePool::ALIGN - 1) & ~(DevicePool::ALIGN - 1);
    alloc((void**)&h->block, block_bytes);
    if (e == hipSuccess) {
        h->pool.attach(h->block, block_bytes);
        if (kinds & KIND_RESIDENT) { // the fixed carve-up of the resident sort
            for (int i = 0; i < 3; ++i)
                h->key[i] = static_cast<u64*>(h->pool.take(cap * 8));
            for (int i = 0; i < 5; ++i)
                h->idx[i] = static_cast<u32*>(h->pool.take(cap * 4));
            h->gid = static_cast<u32*>(h->pool.take(cap * 4));
            h->rank = static_cast<u32*>(h->pool.take(cap * 4));
            for (int i = 0; i < 2; ++i)
                h->gprim[i] = static_cast<u32*>(h->pool.take((cap / 2 + 1) * 4));
            for (int i = 0; i < 2; ++i)
                h->gstart[i] = static_cast<u32*>(h->pool.take((cap / 2 + 2) * 4));
            if (!h->gstart[1])
                e = hipErrorOutOfMemory; // (cannot happen: the block was sized by the same sum)
            h->pool.reset();
        }
    }
    alloc((void**)&h->lookback, h->lookback_words * 8);
    h->rank_tiles_cap = ws.rank_tiles_cap;
    alloc((void**)&h->tile_tables, (h->rank_tiles_cap * 9 + RERANK_SLABS * 5) * sizeof(u32));
    alloc((void**)&h->ghist, (MAX_PASSES + 2) * RADIX_BINS * 4);
    alloc((void**)&h->digit_base, MAX_PASSES * RADIX_BINS * 4);
    alloc((void**)&h->tickets, TICKET_POOL * 4);
    alloc((void**)&h->counts, 16 * 4);
    alloc((void**)&h->msg_off, MSG_OFF_WORDS * 4);
    if (e == hipSuccess)
        e = hipHostMalloc((void**)&h->h_pinned, (PINNED_HIST + MAX_PASSES * RADIX_BINS) * 4, hipHostMallocDefault);
    if (e == hipSuccess)
        e = hipMemset(h->lookback, 0, h->lookback_words * 8);
    if (e == hipSuccess)
        e = hipMemset(h->tickets, 0, TICKET_POOL * 4);
    if (e == hipSuccess)
        e = hipMemset(h->counts, 0, 16 * 4);
    if (e == hipSuccess)
        e = hipDeviceSynchronize();
    if (e != hipSuccess) {
        const int rc = fail(CSA_ERR_HIP, "%s: %s while allocating for %llu suffixes", who, hipGetErrorString(e), (unsigned long long)cap);
        csa_destroy(h);
        return rc;
    }
    *out = h;
    return CSA_OK;
}

} // namespace
} // extern "C++"

uint64_t csa_workspace_bytes(uint64_t max_part_sz) { return workspace_sizes(max_part_sz ? max_part_sz : 1).bytes + BLOCK_SLACK; }

int csa_create(uint64_t max_part_sz, int key_words, csa_handle** out)
{
    return create_handle("csa_create", max_part_sz, key_words, KIND_RESIDENT, out);
}

int csa_create_steps(uint64_t max_part_sz, int key_words, csa_handle** out)
{
    return create_handle("csa_create_steps", max_part_sz, key_words, 0u, out);
}

int csa_set_tuning(csa_handle* h, int knob, uint32_t value)
{
    if (!h)
        return fail(CSA_ERR_ARG, "csa_set_tuning: null handle");
    switch (knob) {
    case CSA_TUNE_DEFER_MIN: h->defer_min = value; break;
    case CSA_TUNE_WINDOW_MIN_CHANGED: h->window_min_changed = value; break;
    case CSA_TUNE_PACK_SYMBOLS: h->pack_symbols = value ? 1u : 0u; break;
    case CSA_TUNE_EXPECT_PRESORTED: h->expect_presorted = value ? 1u : 0u; break;
    case CSA_TUNE_XCD_CHUNK:
        // the chunked order waits for workgroups that are dispatched later: 8 * chunk workgroups of a pass must be able
        // to be resident together, and the device must have room for twice that many (the condition csa_create applies)
        if (value && 2ull * 8ull * value > (u64)(h->cus > 0 ? h->cus : 0))
            return fail(CSA_ERR_ARG, "csa_set_tuning: an XCD chunk of %u tiles needs %llu compute units, the device has %d", value,
                        2ull * 8ull * value, h->cus);
        h->tile_order_exclusive = value ? TILES_STATIC_CHUNKS : TILES_BY_ARRIVAL;
        if (value)
            h->xcd_chunk = value;
        if (h->tile_order != TILES_BY_ARRIVAL) // the handle is in the exclusive order already: follow
            h->tile_order = h->tile_order_exclusive;
        break;
    default: return fail(CSA_ERR_ARG, "csa_set_tuning: unknown knob %d", knob);
    }
    return CSA_OK;
}

int csa_set_device_exclusive(csa_handle* h, int exclusive)
{
    if (!h)
        return fail(CSA_ERR_ARG, "csa_set_device_exclusive: null handle");
    h->tile_order = exclusive ? h->tile_order_exclusive : TILES_BY_ARRIVAL;
    return CSA_OK;
}

void csa_destroy(csa_handle* h)
{
    if (!h)
        return;
    (void)hipFree(h->block);
    (void)hipFree(h->lookback);
    (void)hipFree(h->tile_tables);
    (void)hipFree(h->ghist);
    (void)hipFree(h->digit_base);
    (void)hipFree(h->tickets);
    (void)hipFree(h->counts);
    (void)hipFree(h->msg_off);
    if (h->h_pinned)
        (void)hipHostFree(h->h_pinned);
    for (auto& e : h->events)
        (void)hipEventDestroy(e);
    if (h->ev_gen_ready)
        for (auto& e : h->ev_gen)
            (void)hipEventDestroy(e);
    delete h;
}

int csa_sort_partition_u16_dev(csa_handle* h, const uint16_t* d_text, uint64_t n, uint64_t index_base,
                               uint8_t* d_sa40, void* stream, uint32_t flags, csa_stats* stats)
{
    if (!h)
        return fail(CSA_ERR_ARG, "csa_sort_partition_u16_dev: handle is null");
    if (n > CSA_MAX_PART_SZ)
        return fail(CSA_ERR_TOO_LARGE, "csa_sort_partition_u16_dev: %llu suffixes exceed the partition limit %llu",
                    (unsigned long long)n, (unsigned long long)CSA_MAX_PART_SZ);
    if (index_base > CSA_MAX_INDEX || index_base + n > CSA_MAX_INDEX)
        return fail(CSA_ERR_TOO_LARGE, "csa_sort_partition_u16_dev: suffix indices up to %llu do not fit 40 bits",
                    (unsigned long long)(index_base + n));
    if (!(h->kinds & KIND_RESIDENT))
        return fail(CSA_ERR_ARG, "csa_sort_partition_u16_dev: the handle was created by csa_create_steps, which leaves out the "
                    "resident sort's arrays; use csa_create");
    if (n > h->cap)
        return fail(CSA_ERR_ARG, "csa_sort_partition_u16_dev: %llu suffixes exceed the handle's capacity %llu",
                    (unsigned long long)n, (unsigned long long)h->cap);
    csa_stats local;
    csa_stats* st = stats ? stats : &local;
    memset(st, 0, sizeof(*st));
    st->n = n;
    st->key_words = h->key_words;
    if (n == 0)
        return CSA_OK;
    if (!d_text || !d_sa40)
        return fail(CSA_ERR_ARG, "csa_sort_partition_u16_dev: null text or output pointer");
    int rc = ensure_events(h, flags & CSA_FLAG_KERNEL_TIMING);
    if (rc)
        return rc;
    Launch L;
    L.h = h;
    L.stream = (hipStream_t)stream;
    L.flags = flags;
    L.stats = st;
    return sort_partition(L, d_text, n, index_base, d_sa40);
}

int csa_pack_keys_u16_dev(const uint16_t* d_text, uint64_t n, int key_words, uint64_t* d_keys, void* stream)
{
    if (key_words < 1 || key_words > 4)
        return fail(CSA_ERR_ARG, "csa_pack_keys_u16_dev: key_words = %d is outside [1, 4]", key_words);
    if (n > CSA_MAX_PART_SZ)
        return fail(CSA_ERR_TOO_LARGE, "csa_pack_keys_u16_dev: %llu suffixes exceed the partition limit",
                    (unsigned long long)n);
    if (n == 0)
        return CSA_OK;
    if (!d_text || !d_keys)
        return fail(CSA_ERR_ARG, "csa_pack_keys_u16_dev: null pointer");
    hipLaunchKernelGGL(pack_keys_kernel, dim3((u32)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, d_text, (u32)n,
                       key_words, d_keys);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return CSA_OK;
}

int csa_radix_sort_pairs_dev(csa_handle* h, uint64_t* d_keys, uint32_t* d_vals, uint64_t n, int begin_bit,
                             int end_bit, void* stream)
{
    if (!h)
        return fail(CSA_ERR_ARG, "csa_radix_sort_pairs_dev: handle is null");
    if (begin_bit < 0 || end_bit > 64 || begin_bit > end_bit)
        return fail(CSA_ERR_ARG, "csa_radix_sort_pairs_dev: bad bit range [%d, %d)", begin_bit, end_bit);
    if (n > h->cap)
        return fail(CSA_ERR_ARG, "csa_radix_sort_pairs_dev: %llu pairs exceed the handle's capacity %llu",
                    (unsigned long long)n, (unsigned long long)h->cap);
    if (n == 0 || begin_bit == end_bit)
        return CSA_OK;
    if (!d_keys || !d_vals)
        return fail(CSA_ERR_ARG, "csa_radix_sort_pairs_dev: null pointer");
    Launch L;
    L.h = h;
    L.stream = (hipStream_t)stream;
    L.flags = 0;
    L.stats = nullptr;
    HIP_TRY(hipMemsetAsync(h->counts, 0, 4 * sizeof(u32), L.stream));
    h->pool.reset();
    u64* tmp_keys = static_cast<u64*>(h->pool.take(n * 8));
    u32* tmp_vals = static_cast<u32*>(h->pool.take(n * 4));
    h->last_high_water = h->pool.high_water();
    if (!tmp_keys || !tmp_vals)
        return fail(CSA_ERR_ARG, "csa_radix_sort_pairs_dev: the handle's block of %llu bytes has no room for 12 bytes per pair",
                    (unsigned long long)h->pool.bytes());
    int in_out = 0, passes = 0;
    const PassPlan plan = make_plan(begin_bit, end_bit);
    int rc = radix_sort(L, SRC_PAIRS, nullptr, 0, 0, 0, d_keys, d_vals, tmp_keys, tmp_vals, (u32)n, plan, &in_out, &passes);
    if (rc)
        return rc;
    if (in_out) {
        HIP_TRY(hipMemcpyAsync(d_keys, tmp_keys, n * 8, hipMemcpyDeviceToDevice, L.stream));
        HIP_TRY(hipMemcpyAsync(d_vals, tmp_vals, n * 4, hipMemcpyDeviceToDevice, L.stream));
    }
    return read_counts(L, nullptr);
}

extern "C++" {
namespace {
constexpr int STATIC_MAX_DEVICES = 64;
std::mutex g_static_mutex;
unsigned char* g_static_ptr[STATIC_MAX_DEVICES] = {}; // address of `scratch` on each device, asked for once per device

// The current device's copy of `scratch`.
int static_scratch(unsigned char** out)
{
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= STATIC_MAX_DEVICES)
        return fail(CSA_ERR_ARG, "csa_radix_sort_pairs_static_dev: device %d is beyond the %d devices this entry point keeps a scratch address for",
                    dev, STATIC_MAX_DEVICES);
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (!g_static_ptr[dev]) {
        void* p = nullptr;
        HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p)
            return fail(CSA_ERR_HIP, "csa_radix_sort_pairs_static_dev: no address for the scratch array on device %d", dev);
        g_static_ptr[dev] = static_cast<unsigned char*>(p);
    }
    *out = g_static_ptr[dev];
    return CSA_OK;
}
} // namespace
} // extern "C++"

int csa_radix_sort_pairs_static_dev(uint64_t* d_keys, uint32_t* d_vals, uint64_t n, int begin_bit, int end_bit, void* stream)
{
    if (begin_bit < 0 || end_bit > 64 || begin_bit > end_bit)
        return fail(CSA_ERR_ARG, "csa_radix_sort_pairs_static_dev: bad bit range [%d, %d)", begin_bit, end_bit);
    if (n > STATIC_SORT_MAX)
        return fail(CSA_ERR_TOO_LARGE, "csa_radix_sort_pairs_static_dev: %llu pairs exceed the %llu this entry point's fixed scratch holds "
                    "(use csa_radix_sort_pairs_dev with a handle)", (unsigned long long)n, (unsigned long long)STATIC_SORT_MAX);
    unsigned char* base = nullptr; // the device address of the scratch array: never the array's name from here on
    int rc = static_scratch(&base);
    if (rc)
        return rc;
    if (n == 0 || begin_bit == end_bit)
        return CSA_OK;
    if (!d_keys || !d_vals)
        return fail(CSA_ERR_ARG, "csa_radix_sort_pairs_static_dev: null pointer");
    hipStream_t s = (hipStream_t)stream;
    u64* tmp_keys = reinterpret_cast<u64*>(base + STATIC_OFF_KEYS);
    u32* tmp_vals = reinterpret_cast<u32*>(base + STATIC_OFF_VALS);
    u64* lookback = reinterpret_cast<u64*>(base + STATIC_OFF_LOOKBACK);
    u32* ghist = reinterpret_cast<u32*>(base + STATIC_OFF_GHIST);
    u32* tickets = reinterpret_cast<u32*>(base + STATIC_OFF_TICKETS);
    u32* err = reinterpret_cast<u32*>(base + STATIC_OFF_ERR);
    u32* digit_base = reinterpret_cast<u32*>(base + STATIC_OFF_DIGIT_BASE);
    // The array keeps what the last call left: look-back words, digit counts, tile tickets and the error word start at
    // zero in every call (a fill kernel, not a memset node: the call may be recorded into a graph). With the words
    // cleared the launch epoch can stay the same in every call and replay.
    const u64 control_words = (STATIC_CONTROL_END - STATIC_OFF_CONTROL) / sizeof(u32);
    hipLaunchKernelGGL(fill_u32_kernel, dim3((u32)((control_words + 255) / 256)), dim3(256), 0, s,
                       reinterpret_cast<u32*>(base + STATIC_OFF_CONTROL), control_words, 0u);
    const PassPlan plan = make_plan(begin_bit, end_bit);
    HistArgs ha;
    ha.keys = d_keys;
    ha.vals = d_vals;
    ha.text = nullptr;
    ha.n = (u32)n;
    ha.text_n = 0;
    ha.word = 0;
    ha.plan = plan;
    ha.ghist = ghist;
    hipLaunchKernelGGL(radix_hist_kernel, dim3(hist_blocks(256 * 16, n)), dim3(256), 0, s, ha);
    hipLaunchKernelGGL(radix_scan_hist_kernel, dim3(1), dim3(256), 0, s, ghist, digit_base, plan.num_passes);
    // every pass runs (skipping the passes whose digit is constant would need the counts on the host: a round trip)
    const TileOrder by_arrival = {TILES_BY_ARRIVAL, XCD_CHUNK};
    int where = 0; // 0: the pairs are in the caller's arrays, 1: in the scratch
    for (int p = 0; p < plan.num_passes; ++p) {
        OnesweepArgs a;
        a.keys_in = where == 0 ? d_keys : tmp_keys;
        a.vals_in = where == 0 ? d_vals : tmp_vals;
        a.keys_out = where == 0 ? tmp_keys : d_keys;
        a.vals_out = where == 0 ? tmp_vals : d_vals;
        a.text = nullptr;
        a.n = (u32)n;
        a.text_n = 0;
        a.tail = 0;
        a.word = 0;
        a.shift = plan.shift[p];
        a.bits = plan.bits[p];
        a.digit_base = digit_base + p * RADIX_BINS;
        a.lookback = lookback + (u64)p * STATIC_LB_WORDS;
        a.lookback_groups = a.lookback + STATIC_LB_TILE_WORDS;
        a.ticket = tickets + p;
        a.epoch = 1;
        a.err = err;
        launch_onesweep_shape<SRC_PAIRS, SORT_BLOCK, true>(by_arrival, a, s);
        where ^= 1;
    }
    if (where)
        hipLaunchKernelGGL(copy_pairs_kernel, dim3((u32)((n + 255) / 256)), dim3(256), 0, s, (const u64*)tmp_keys, (const u32*)tmp_vals,
                           (u64)n, d_keys, d_vals);
    HIP_TRY(hipGetLastError());
    return CSA_OK;
}

int csa_radix_sort_pairs_static_status(void* stream)
{
    unsigned char* base = nullptr; // (the device address of the scratch array, as in the sort itself)
    int rc = static_scratch(&base);
    if (rc)
        return rc;
    hipStream_t s = (hipStream_t)stream;
    u32 err = 0; // one word into the caller's stack: no buffer is allocated for it
    HIP_TRY(hipMemcpyAsync(&err, base + STATIC_OFF_ERR, sizeof(u32), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    if (err)
        return fail(CSA_ERR_INTERNAL, "csa_radix_sort_pairs_static_dev: device invariant %u failed in the last sort on this device%s", err,
                    err == DEV_ERR_LOOKBACK_TIMEOUT ? " (a look-back wait ran into its spin limit): the pairs it left are not sorted" : "");
    return CSA_OK;
}

int csa_verify_sa40_dev(csa_handle* h, const uint16_t* d_text, uint64_t n, uint64_t index_base,
                        const uint8_t* d_sa40, void* stream, int* ok)
{
    if (!h || !ok)
        return fail(CSA_ERR_ARG, "csa_verify_sa40_dev: null handle or result pointer");
    *ok = 0;
    if (n > h->cap)
        return fail(CSA_ERR_ARG, "csa_verify_sa40_dev: %llu suffixes exceed the handle's capacity %llu",
                    (unsigned long long)n, (unsigned long long)h->cap);
    if (n == 0) {
        *ok = 1;
        return CSA_OK;
    }
    if (!d_text || !d_sa40)
        return fail(CSA_ERR_ARG, "csa_verify_sa40_dev: null pointer");
    hipStream_t s = (hipStream_t)stream;
    const u32 blocks = (u32)((n + 255) / 256);
    h->pool.reset();
    u32* inverse = static_cast<u32*>(h->pool.take(n * sizeof(u32))); // the inverse suffix array
    h->last_high_water = h->pool.high_water();
    if (!inverse)
        return fail(CSA_ERR_ARG, "csa_verify_sa40_dev: the handle's block of %llu bytes has no room for 4 bytes per suffix",
                    (unsigned long long)h->pool.bytes());
    HIP_TRY(hipMemsetAsync(h->counts + 3, 0, sizeof(u32), s));
    hipLaunchKernelGGL(fill_u32_kernel, dim3(blocks), dim3(256), 0, s, inverse, n, 0xFFFFFFFFu);
    hipLaunchKernelGGL(verify_invert_kernel, dim3(blocks), dim3(256), 0, s, d_sa40, (u32)n, index_base, inverse,
                       h->counts + 3);
    hipLaunchKernelGGL(verify_order_kernel, dim3(blocks), dim3(256), 0, s, d_sa40, d_text, (u32)n, index_base, inverse,
                       h->counts + 3);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipMemcpyAsync(h->h_pinned + 3, h->counts + 3, sizeof(u32), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    *ok = h->h_pinned[3] ? 0 : 1;
    return CSA_OK;
}

int csa_enable_profile_ranges(int enable)
{
    if (enable_ranges(enable != 0))
        return fail(CSA_ERR_ARG, "csa_enable_profile_ranges: no roctx library (librocprofiler-sdk-roctx.so, libroctx64.so) could be loaded");
    return CSA_OK;
}

} // extern "C"

#include "step_entries.hpp"
#include "slab_entries.hpp"
#include "host_pipeline.hpp"
