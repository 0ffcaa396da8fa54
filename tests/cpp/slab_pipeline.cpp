// slab_pipeline <n> <p> <key_words> <chunk_cap> <seed> <sigma> [suffix-array-file|-] [threads] [text-file|-] [budget-bytes]
// A multi-partition suffix-array build driven the way the reference's dispatcher drives its builder class
// (src/GPU_SACA.cu:1354-1600, 2190-2370), through the three per-partition members of include/cascade_gpu_saca.hpp:
// every partition step takes a Partition_Assembly of pinned host slabs (chunks of chunk_cap suffixes, each with its chunk
// of the partition's inbox) and returns ranks, lanes and the outbox in them; partitions exchange ranks only as messages;
// the final permutation comes back cut for the output file. Everything that the reference's backend keeps (partition
// contents, inboxes, the packed partition-id map with its retirement flags) is plain host memory here.
//   threads      dispatcher threads (1 to 3 = STREAM_C), each with its own buffer set and stream, that take the
//                partitions of a generation from a shared counter and call the members concurrently
//                (src/GPU_SACA.cu:1539-1589); default 1
//   text-file    uint16 symbols to build the suffix array of (n = its length; sigma is ignored) instead of the built-in
//                random text with a planted repeat
//   budget-bytes device memory the builder may plan with: the partitions must not exceed partition_size_upper_bound of
//                it, allocate_device_space must take no more than its share, and no step may allocate beyond that
//                (checked with hipMemGetInfo). With n = 0 the text length is that bound itself (use p = 1: one partition
//                of exactly the largest size the floor plan admits)
// The result is compared, byte for byte, with the suffix array of the same text sorted as one resident partition
// (csa_sort_partition_u16); exit status 0 if they agree. The last line also reports what the dispatch phases took and
// moved over the link (host staging and message routing between the phases are not in those times).
// A test program: it is not part of the library.
#include "../../include/cascade_gpu_saca.hpp"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <array>
#include <atomic>
#include <chrono>
#include <cstring>
#include <memory>
#include <random>
#include <thread>

namespace {

using namespace cascade_hip;
using Builder = GPU_SACA<std::uint16_t>;

[[noreturn]] void die(const std::string& what)
{
    std::cerr << "slab_pipeline: " << what << "\n";
    std::exit(2);
}

void hip_check(hipError_t e, const char* what)
{
    if (e != hipSuccess)
        die(std::string(what) + ": " + hipGetErrorString(e));
}

void csa_check(int rc, const char* what)
{
    if (rc != CSA_OK)
        die(std::string(what) + ": " + csa_last_error());
}

template <typename T> T* dev_alloc(std::size_t count)
{
    T* p = nullptr;
    hip_check(hipMalloc(reinterpret_cast<void**>(&p), (count ? count : 1) * sizeof(T)), "hipMalloc");
    return p;
}

template <typename T> T* pinned_alloc(std::size_t count)
{
    T* p = nullptr;
    hip_check(hipHostMalloc(reinterpret_cast<void**>(&p), (count ? count : 1) * sizeof(T), hipHostMallocDefault), "hipHostMalloc");
    return p;
}

std::size_t device_free_bytes()
{
    std::size_t free_b = 0, total_b = 0;
    hip_check(hipMemGetInfo(&free_b, &total_b), "hipMemGetInfo");
    return free_b;
}

void put_lane(std::uint8_t* lanes, std::size_t i, std::uint64_t v)
{
    for (int b = 0; b < 5; ++b)
        lanes[5 * i + b] = static_cast<std::uint8_t>(v >> (8 * b));
}

std::uint64_t get_lane(const std::uint8_t* lanes, std::size_t i)
{
    std::uint64_t v = 0;
    for (int b = 0; b < 5; ++b)
        v |= static_cast<std::uint64_t>(lanes[5 * i + b]) << (8 * b);
    return v;
}

// One pinned slab with the reference's capacities for chunk_cap suffixes (src/Staging_Slab.cpp:27-35).
struct Slab_Buffers {
    Staging_Slab slab;
    Slab_Buffers(idx_t chunk_cap, int key_words)
    {
        csa_slab& raw = slab; // the fields behind the reference's accessors
        raw.key = pinned_alloc<std::uint64_t>(chunk_cap * key_words);
        raw.suf = pinned_alloc<std::uint8_t>(5 * chunk_cap);
        raw.beta = pinned_alloc<std::uint32_t>(chunk_cap);
        raw.msg_target = pinned_alloc<std::uint8_t>(std::max<idx_t>(10 * chunk_cap, 2 * 4096));
        raw.msg_rank = pinned_alloc<std::uint32_t>(2 * chunk_cap);
    }
};

struct Partition {
    std::vector<std::uint64_t> suf; // its suffixes, active ones first
    std::vector<p_sz_t> rank;       // their partition-local ranks
    idx_t active = 0;
    std::vector<std::unique_ptr<Slab_Buffers>> slabs; // the partition's own slabs, kept over the generations
    Partition_Assembly assembly;                      // the chain handed to the members in this phase
    Staging_Slab& slab_of(std::size_t c, idx_t chunk_cap, int key_words)
    {
        while (slabs.size() <= c)
            slabs.push_back(std::make_unique<Slab_Buffers>(chunk_cap, key_words));
        return slabs[c]->slab;
    }
};

struct Inbox {
    std::vector<std::uint64_t> target;
    std::vector<p_sz_t> rank;
};

// Runs job(q, buf_id) for every listed partition on `threads` dispatcher threads, buffer set = thread index; returns
// the seconds the phase took.
template <typename Job> double dispatch(const std::vector<std::uint32_t>& todo, unsigned threads, Job job)
{
    const auto t0 = std::chrono::steady_clock::now();
    if (threads <= 1) {
        for (const std::uint32_t q : todo)
            job(q, 0);
    } else {
        std::atomic<std::size_t> next{0};
        std::vector<std::thread> pool;
        for (unsigned b = 0; b < threads; ++b)
            pool.emplace_back([&, b] {
                for (std::size_t i = next.fetch_add(1); i < todo.size(); i = next.fetch_add(1))
                    job(todo[i], b);
            });
        for (auto& t : pool)
            t.join();
    }
    return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

} // namespace

int main(int argc, char** argv)
{
    if (argc < 7)
        die("usage: slab_pipeline <n> <p> <key_words> <chunk_cap> <seed> <sigma> [suffix-array-file|-] [threads] [text-file|-] [budget-bytes]");
    idx_t n = std::strtoull(argv[1], nullptr, 10);
    const std::uint32_t p = static_cast<std::uint32_t>(std::strtoul(argv[2], nullptr, 10));
    const int key_words = std::atoi(argv[3]);
    const idx_t chunk_cap = std::strtoull(argv[4], nullptr, 10);
    const std::uint64_t seed = std::strtoull(argv[5], nullptr, 10);
    const std::uint32_t sigma = static_cast<std::uint32_t>(std::strtoul(argv[6], nullptr, 10));
    const std::string sa_path = argc > 7 && std::string(argv[7]) != "-" ? argv[7] : "";
    const unsigned threads = argc > 8 ? static_cast<unsigned>(std::atoi(argv[8])) : 1u;
    const std::string text_path = argc > 9 && std::string(argv[9]) != "-" ? argv[9] : "";
    const std::size_t budget = argc > 10 ? std::strtoull(argv[10], nullptr, 10) : 0;
    if (p < 1 || p > 32768 || key_words < 1 || key_words > 4 || chunk_cap % 4096 != 0 || chunk_cap == 0 || sigma < 1 || threads < 1 ||
        threads > Builder::STREAM_C)
        die("bad arguments");
    const idx_t ell = 4 * static_cast<idx_t>(key_words);
    if (budget && n == 0) // one partition of exactly the size the floor plan admits for this budget
        n = Builder(1, static_cast<p_id_t>(p), key_words, chunk_cap).partition_size_upper_bound(budget);

    // ---- the text: a file, or random symbols with a long repeat (many generations, pills in flight) and a zero tail ----
    std::mt19937_64 rng(seed);
    std::vector<std::uint16_t> text;
    if (!text_path.empty()) {
        std::ifstream in(text_path, std::ios::binary | std::ios::ate);
        if (!in)
            die("cannot open " + text_path);
        n = static_cast<idx_t>(in.tellg()) / 2;
        text.resize(n);
        in.seekg(0);
        in.read(reinterpret_cast<char*>(text.data()), static_cast<std::streamsize>(2 * n));
    } else {
        if (n < 16)
            die("bad arguments: n < 16");
        text.resize(n);
        for (auto& s : text)
            s = static_cast<std::uint16_t>(rng() % sigma);
        std::copy(text.begin(), text.begin() + n / 3, text.begin() + n / 2);
        for (idx_t i = n - 9; i < n; ++i)
            text[i] = 0;
    }
    if (n < 16)
        die("the text is shorter than 16 symbols");
    std::uint16_t* d_text = dev_alloc<std::uint16_t>(n);
    hip_check(hipMemcpy(d_text, text.data(), n * 2, hipMemcpyHostToDevice), "text upload");

    // ---- partition ids, packed map, partition sizes (src/GPU_SACA.cu:854-1000) ----
    const int pivot_words = 2;
    std::vector<std::uint64_t> pivots;
    {
        std::vector<std::array<std::uint64_t, 2>> piv(p - 1);
        for (auto& k : piv) {
            const idx_t at = rng() % n;
            for (int w = 0; w < pivot_words; ++w) {
                std::uint64_t word = 0;
                for (int q = 0; q < 4; ++q) {
                    const idx_t pos = at + 4 * w + q;
                    word = (word << 16) | (pos < n ? text[pos] : 0);
                }
                k[w] = word;
            }
        }
        std::sort(piv.begin(), piv.end());
        for (const auto& k : piv)
            pivots.insert(pivots.end(), k.begin(), k.end());
    }
    const std::uint32_t bits = csa_partition_id_bits(p);
    const std::size_t map_words = ((n + 63) / 64) * bits + 1;
    std::uint64_t* d_piv = dev_alloc<std::uint64_t>(pivots.size());
    std::uint16_t* d_pid = dev_alloc<std::uint16_t>(n);
    std::uint64_t* d_map = dev_alloc<std::uint64_t>(map_words);
    std::uint64_t* d_psz = dev_alloc<std::uint64_t>(p);
    hip_check(hipMemcpy(d_piv, pivots.data(), pivots.size() * 8, hipMemcpyHostToDevice), "pivot upload");
    hip_check(hipMemset(d_map, 0, map_words * 8), "memset");
    hip_check(hipMemset(d_psz, 0, p * 8), "memset");
    csa_check(csa_partition_ids_u16_dev(d_text, n, n, p > 1 ? d_piv : nullptr, pivot_words, p, d_pid, d_map, d_psz, nullptr), "partition ids");
    hip_check(hipDeviceSynchronize(), "sync");
    std::vector<std::uint16_t> pid(n);
    std::vector<std::uint64_t> map(map_words), psz(p);
    hip_check(hipMemcpy(pid.data(), d_pid, n * 2, hipMemcpyDeviceToHost), "pid download");
    hip_check(hipMemcpy(map.data(), d_map, map_words * 8, hipMemcpyDeviceToHost), "map download");
    hip_check(hipMemcpy(psz.data(), d_psz, p * 8, hipMemcpyDeviceToHost), "sizes download");
    hip_check(hipFree(d_pid), "free");
    hip_check(hipFree(d_piv), "free");
    hip_check(hipFree(d_psz), "free");
    std::vector<idx_t> P_off(p + 1, 0);
    idx_t max_part = 1;
    for (std::uint32_t q = 0; q < p; ++q) {
        P_off[q + 1] = P_off[q] + psz[q];
        max_part = std::max<idx_t>(max_part, psz[q]);
    }
    if (P_off[p] != n)
        die("the partition sizes do not add up to n");

    std::vector<Partition> part(p);
    for (std::uint32_t q = 0; q < p; ++q)
        part[q].suf.reserve(psz[q]);
    for (idx_t j = 0; j < n; ++j)
        part[pid[j]].suf.push_back(j);
    for (std::uint32_t q = 0; q < p; ++q) {
        std::shuffle(part[q].suf.begin(), part[q].suf.end(), rng); // a partition's suffixes arrive in no particular order
        part[q].rank.assign(part[q].suf.size(), 0);
        part[q].active = part[q].suf.size();
    }
    std::uint8_t* d_lanes = dev_alloc<std::uint8_t>(5 * max_part);
    std::uint64_t* d_keys = dev_alloc<std::uint64_t>(max_part * key_words);
    std::uint32_t* d_beta = dev_alloc<std::uint32_t>(max_part);
    std::vector<std::uint8_t> lanes(5 * max_part);
    std::vector<std::uint64_t> keys(max_part * key_words);
    std::vector<std::uint32_t> beta(max_part);

    // ---- the builder: sized by its own bound when a budget is given; everything it will ever hold is allocated here ----
    Builder saca(max_part, static_cast<p_id_t>(p), key_words, chunk_cap);
    if (budget && max_part > saca.partition_size_upper_bound(budget))
        die("the largest partition (" + std::to_string(max_part) + ") exceeds partition_size_upper_bound(" + std::to_string(budget) +
            ") = " + std::to_string(saca.partition_size_upper_bound(budget)));
    const std::size_t free_before = device_free_bytes();
    if (!saca.allocate_device_space())
        die("no device space");
    const std::size_t free_after = device_free_bytes();
    const std::size_t taken = free_before - free_after;
    if (budget && taken > static_cast<std::size_t>(static_cast<double>(budget) * (1.0 - Builder::MEM_SAFETY_MARGIN)))
        die("allocate_device_space took " + std::to_string(taken) + " bytes, more than the budget's share");
    if (taken > saca.device_bytes_required(max_part) + (64u << 20))
        die("allocate_device_space took " + std::to_string(taken) + " bytes, the floor plan says " +
            std::to_string(saca.device_bytes_required(max_part)));
    hipStream_t streams[Builder::STREAM_C] = {};
    for (unsigned b = 0; b < threads; ++b) {
        hip_check(hipStreamCreateWithFlags(&streams[b], hipStreamNonBlocking), "stream");
        saca.set_stream(b, streams[b]);
    }
    // No step may take device memory of its own. The level is read after the streams exist (the runtime keeps a few MB
    // per stream), and what the runtime sets up on a stream's first use is allowed for below; a column of a partition
    // would be far more.
    const std::size_t free_ready = device_free_bytes();
    std::size_t free_lowest = free_ready;

    double dispatch_s = 0, gen0_s = 0;
    std::uint64_t link_bytes = 0, gen0_bytes = 0;
    std::vector<Inbox> inbox(p);
    idx_t gen = 0, ctx = ell;
    for (;; ++gen, ctx *= 2) {
        std::vector<std::uint32_t> todo;
        for (std::uint32_t q = 0; q < p; ++q)
            if (part[q].active > 0)
                todo.push_back(q);
        if (todo.empty())
            break;
        if (gen >= 64)
            die("64 generations and still active suffixes");
        saca.set_context(ctx, gen);
        hip_check(hipMemcpy(d_map, map.data(), map_words * 8, hipMemcpyHostToDevice), "map upload");
        // ---- phase 1, host (the reference's readers and stagers, src/GPU_SACA.cu:1412-1500, 1611-1692): every
        //      partition and its inbox cut into chunks of chunk_cap (:1396-1400), keys at generation 0, routing tags ----
        std::uint64_t bytes_up = 0;
        for (const std::uint32_t q : todo) {
            Partition& pt = part[q];
            const idx_t a = pt.active;
            for (idx_t i = 0; i < a; ++i)
                put_lane(lanes.data(), i, pt.suf[i]);
            hip_check(hipMemcpy(d_lanes, lanes.data(), 5 * a, hipMemcpyHostToDevice), "lane upload");
            csa_check(csa_stage_slab_u16_dev(d_text, n, d_lanes, a, key_words, d_map, p, ctx, gen == 0 ? 1 : 0, gen == 0 ? d_keys : nullptr,
                                             d_beta, nullptr),
                      "stage slab");
            hip_check(hipDeviceSynchronize(), "sync");
            hip_check(hipMemcpy(beta.data(), d_beta, a * 4, hipMemcpyDeviceToHost), "beta download");
            if (gen == 0)
                hip_check(hipMemcpy(keys.data(), d_keys, a * key_words * 8, hipMemcpyDeviceToHost), "key download");
            const Inbox& in = inbox[q];
            const idx_t inbox_sz = gen == 0 ? 0 : in.target.size();
            const std::size_t chunk_c = std::max<std::size_t>(1, std::max((a + chunk_cap - 1) / chunk_cap, (inbox_sz + chunk_cap - 1) / chunk_cap));
            pt.assembly.slab.clear();
            for (std::size_t c = 0; c < chunk_c; ++c) {
                Staging_Slab& s = pt.slab_of(c, chunk_cap, key_words);
                const idx_t off = c * chunk_cap;
                const idx_t sz = off < a ? std::min(chunk_cap, a - off) : 0;
                const idx_t msg_sz = off < inbox_sz ? std::min(chunk_cap, inbox_sz - off) : 0;
                s.assign(sz ? off : a, sz, static_cast<p_sz_t>(msg_sz ? off : 0), static_cast<p_sz_t>(msg_sz));
                if (gen == 0)
                    std::memcpy(s.key(), keys.data() + off * key_words, sz * key_words * 8);
                else
                    std::memcpy(s.key(), pt.rank.data() + off, sz * 4);
                std::memcpy(s.suf(), lanes.data() + 5 * off, 5 * sz);
                std::memcpy(s.beta(), beta.data() + off, sz * 4);
                for (idx_t i = 0; i < msg_sz; ++i)
                    put_lane(s.msg_target(), i, in.target[off + i]);
                if (msg_sz)
                    std::memcpy(s.msg_rank(), in.rank.data() + off, msg_sz * 4);
                pt.assembly.slab.push_back(&s);
            }
            bytes_up += a * (gen == 0 ? 8 * key_words + 9 : 13) + inbox_sz * 9;
        }
        // ---- phase 2, the dispatchers (src/GPU_SACA.cu:1539-1589): the members, concurrently, one buffer set each ----
        const double secs = dispatch(todo, threads, [&](std::uint32_t q, unsigned buf_id) {
            if (gen == 0)
                saca.sort_and_init_rank_and_filter(static_cast<p_id_t>(q), part[q].assembly, buf_id);
            else
                saca.sort_and_re_rank_and_filter(static_cast<p_id_t>(q), part[q].assembly, buf_id);
        });
        free_lowest = std::min(free_lowest, device_free_bytes());
        // ---- phase 3, host (the reference's writers, src/GPU_SACA.cu:1305-1331, 1503-1530, 1695-1711): ranks over
        //      key(), lanes, the outbox split by destination, retirement flags ----
        std::vector<Inbox> next(p);
        std::vector<std::uint64_t> retired_now;
        std::uint64_t bytes_down = 0;
        for (const std::uint32_t q : todo) {
            Partition& pt = part[q];
            const idx_t a = pt.active;
            const idx_t a_new = *saca.active_slot(static_cast<p_id_t>(q));
            const p_sz_t* end = saca.msg_off(static_cast<p_id_t>(q));
            const idx_t total = end[p - 1];
            if (a_new > a)
                die("more active suffixes after a step than before");
            std::vector<std::uint64_t> m_target(total);
            std::vector<p_sz_t> m_rank(total);
            for (std::size_t c = 0; c < pt.assembly.slab.size(); ++c) {
                const Staging_Slab& s = *pt.assembly.slab[c];
                for (idx_t i = 0; i < s.size(); ++i) {
                    pt.suf[s.off() + i] = get_lane(s.suf(), i);
                    pt.rank[s.off() + i] = reinterpret_cast<const p_sz_t*>(s.key())[i];
                }
                const idx_t want_off = 2 * c * chunk_cap, want_sz = want_off < total ? std::min(2 * chunk_cap, total - want_off) : 0;
                if (s.outbox_off() != want_off || s.outbox_sz() != want_sz) // src/GPU_SACA.cu:1318-1320
                    die("a slab's outbox chunk is not where the split at 2 * chunk_cap puts it");
                for (idx_t i = 0; i < s.outbox_sz(); ++i) {
                    m_target[s.outbox_off() + i] = get_lane(s.msg_target(), i);
                    m_rank[s.outbox_off() + i] = s.msg_rank()[i];
                }
            }
            idx_t start = 0;
            for (std::uint32_t dest = 0; dest < p; ++dest) { // src/Partition_Backend.cpp:516-554
                for (idx_t i = start; i < end[dest]; ++i) {
                    if (pid[m_target[i]] != dest)
                        die("a message sits in the group of a partition its target does not belong to");
                    next[dest].target.push_back(m_target[i]);
                    next[dest].rank.push_back(m_rank[i]);
                }
                start = end[dest];
            }
            for (idx_t i = a_new; i < a; ++i)
                retired_now.push_back(pt.suf[i]);
            pt.active = a_new;
            bytes_down += a * 9 + total * 9;
        }
        for (const std::uint64_t j : retired_now) {
            const std::uint64_t bit = j * bits + (bits - 1);
            map[bit / 64] |= std::uint64_t(1) << (bit % 64);
        }
        inbox.swap(next);
        dispatch_s += secs;
        link_bytes += bytes_up + bytes_down;
        if (gen == 0) {
            gen0_s = secs;
            gen0_bytes = bytes_up + bytes_down;
        }
    }

    // ---- every partition to rank order, as cut for the output file (src/GPU_SACA.cu:2107-2164, 2337-2365) ----
    std::vector<std::uint8_t> file(5 * n, 0xEE);
    std::vector<std::uint32_t> todo;
    for (std::uint32_t q = 0; q < p; ++q) {
        Partition& pt = part[q];
        const idx_t m = pt.suf.size();
        if (m == 0)
            continue;
        todo.push_back(q);
        const std::size_t chunk_c = (m + chunk_cap - 1) / chunk_cap + 1; // one more: the partition need not start on a disk block
        pt.assembly.slab.clear();
        for (std::size_t c = 0; c < chunk_c; ++c) {
            Staging_Slab& s = pt.slab_of(c, chunk_cap, key_words);
            const idx_t off = c * chunk_cap;
            const idx_t sz = off < m ? std::min(chunk_cap, m - off) : 0;
            s.assign(sz ? off : m, sz, 0, 0);
            for (idx_t i = 0; i < sz; ++i)
                put_lane(s.suf(), i, pt.suf[off + i]);
            std::memcpy(s.key(), pt.rank.data() + off, sz * 4);
            pt.assembly.slab.push_back(&s);
        }
    }
    const double scatter_s = dispatch(todo, threads, [&](std::uint32_t q, unsigned buf_id) {
        saca.scatter_to_rank_order(static_cast<p_id_t>(q), part[q].assembly, buf_id, 5 * P_off[q]);
    });
    free_lowest = std::min(free_lowest, device_free_bytes());
    for (const std::uint32_t q : todo) {
        const Partition& pt = part[q];
        const idx_t m = pt.suf.size(), lo = 5 * P_off[q];
        const std::size_t chunk_c = pt.assembly.slab.size();
        for (std::size_t c = 0; c < chunk_c; ++c) {
            std::uint64_t cut[6];
            csa_output_cut(lo, lo + 5 * m, 5 * chunk_cap, static_cast<std::uint32_t>(c), static_cast<std::uint32_t>(chunk_c), cut);
            const Staging_Slab& s = *pt.assembly.slab[c];
            std::memcpy(file.data() + cut[0], s.suf(), cut[1] - cut[0]);
            std::memcpy(file.data() + cut[2], s.msg_target(), cut[3] - cut[2]);
            std::memcpy(file.data() + cut[4], s.msg_target() + 4096, cut[5] - cut[4]);
        }
    }
    if (free_lowest + (32u << 20) < free_ready)
        die("a step took device memory of its own: " + std::to_string(free_ready - free_lowest) + " bytes below the level after allocate_device_space");

    if (!sa_path.empty()) {
        std::ofstream out(sa_path, std::ios::binary | std::ios::trunc);
        out.write(reinterpret_cast<const char*>(file.data()), static_cast<std::streamsize>(file.size()));
        if (text_path.empty()) {
            std::ofstream txt(sa_path + ".text", std::ios::binary | std::ios::trunc);
            txt.write(reinterpret_cast<const char*>(text.data()), static_cast<std::streamsize>(2 * n));
        }
    }
    // ---- the same text as one resident partition ----
    std::vector<std::uint8_t> want(5 * n);
    csa_stats st{};
    csa_check(csa_sort_partition_u16(text.data(), n, key_words, want.data(), &st), "resident sort");
    if (file != want) {
        idx_t at = 0;
        while (at < 5 * n && file[at] == want[at])
            ++at;
        std::cout << "MISMATCH at entry " << at / 5 << " after " << gen << " generations\n";
        return 1;
    }
    std::cout << "OK n=" << n << " p=" << p << " key_words=" << key_words << " generations=" << gen << " (resident sort: " << st.generations
              << ") threads=" << threads << " max_part=" << max_part << " device_bytes=" << taken << " gen0_ms=" << gen0_s * 1e3
              << " gen0_link_bytes=" << gen0_bytes << " dispatch_ms=" << dispatch_s * 1e3 << " link_bytes=" << link_bytes
              << " scatter_ms=" << scatter_s * 1e3 << " scatter_link_bytes=" << 14 * n << "\n";
    return 0;
}
