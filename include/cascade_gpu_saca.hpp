// cascade_gpu_saca.hpp : the reference's builder surface over the C ABI of cascade_hip.h, header only, plain C++17
// (no HIP header: device pointers and streams travel as plain pointers, as in the C ABI).
//
// Names, argument meaning and error behaviour follow gpu_saca::GPU_SACA<T_sym_> (reference: include/GPU_SACA.hpp:39-310):
//   GPU_SACA(ip_path, op_path) / build_SA()        include/GPU_SACA.hpp:304-310, src/main.cu:27-30
//   partition_size_upper_bound()                   include/GPU_SACA.hpp:209
//   allocate_device_space()                        include/GPU_SACA.hpp:221
//   set_context(ctx, gen)                          include/GPU_SACA.hpp:236
//   sort_and_init_rank_and_filter(p_id, ., buf_id) include/GPU_SACA.hpp:272
//   sort_and_re_rank_and_filter(p_id, ., buf_id)   include/GPU_SACA.hpp:279
//   scatter_to_rank_order(p_id, ., buf_id)         include/GPU_SACA.hpp:288
// The three per-partition members take what the reference's take: a Partition_Assembly, the chain of pinned host slabs
// (include/Staging_Slab.hpp:20-119) that holds the partition before and after; upload, device step and download happen
// inside, as in src/GPU_SACA.cu:1125-1133,1305-1331. Overloads that take a Device_Partition (the same columns, already in
// HBM) serve callers that keep partitions on the device.
// A failure prints the library's message and ends the process, as CUDA_CHECK does (include/utility.cuh:19-29); code
// that wants the status instead calls the C ABI directly.
#ifndef CASCADE_GPU_SACA_HPP
#define CASCADE_GPU_SACA_HPP

#include "cascade_hip.h"

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <string>
#include <vector>

namespace cascade_hip {

using idx_t = std::uint64_t;  // text positions, sizes (reference: include/types.hpp:12-16)
using p_id_t = std::uint16_t; // partition ids
using p_sz_t = std::uint32_t; // partition-local ranks
using beta_t = std::uint32_t; // pair of routing tags

// A slab of a partition in pinned host memory: the reference's Staging_Slab (include/Staging_Slab.hpp:20-119) with the
// same accessors, laid out as the C ABI's csa_slab. The buffers belong to the caller (the reference's slab pool).
struct Staging_Slab : csa_slab {
    Staging_Slab() : csa_slab{} {}
    auto key() const { return csa_slab::key; }
    auto suf() const { return csa_slab::suf; }
    auto beta() const { return csa_slab::beta; }
    auto msg_target() const { return csa_slab::msg_target; }
    auto msg_rank() const { return csa_slab::msg_rank; }
    auto off() const { return csa_slab::off; }
    auto size() const { return csa_slab::size; }
    auto inbox_off() const { return csa_slab::inbox_off; }
    auto inbox_sz() const { return csa_slab::inbox_sz; }
    auto outbox_off() const { return csa_slab::outbox_off; }
    auto outbox_sz() const { return csa_slab::outbox_sz; }
    void set_outbox_off_and_size(idx_t off, idx_t sz) { csa_slab::outbox_off = static_cast<std::uint32_t>(off), csa_slab::outbox_sz = static_cast<std::uint32_t>(sz); }
    // Tags the slab with the chunk it carries (src/Staging_Slab.cpp:38-41).
    void assign(idx_t off, idx_t sz, p_sz_t msg_off, p_sz_t inbox_sz)
    {
        csa_slab::off = off, csa_slab::size = sz, csa_slab::inbox_off = msg_off, csa_slab::inbox_sz = inbox_sz;
        csa_slab::outbox_off = csa_slab::outbox_sz = 0;
    }
};

// The chain of slabs that makes up a partition (include/Staging_Slab.hpp:122-126).
struct Partition_Assembly {
    std::vector<Staging_Slab*> slab;
};

// One partition's columns on the device, before and after a step (the device-side image of a Partition_Assembly).
struct Device_Partition {
    idx_t sz = 0;                         // suffixes in the cohort handed to the step
    const std::uint64_t* key = nullptr;   // generation 0: packed K-gram words, key_words per suffix (Staging_Slab::key())
    const p_sz_t* rank = nullptr;         // later generations: the partition-local ranks kept from the step before
    const std::uint8_t* suf = nullptr;    // 5-byte lanes (Staging_Slab::suf())
    const beta_t* beta = nullptr;         // routing tags (Staging_Slab::beta())
    const std::uint8_t* inbox_target = nullptr; // later generations: the messages delivered to this partition
    const p_sz_t* inbox_rank = nullptr;
    std::uint32_t inbox_sz = 0;
    p_sz_t* rank_out = nullptr;           // outputs: ranks and lanes, active suffixes first
    std::uint8_t* suf_out = nullptr;
    std::uint8_t* msg_target = nullptr;   // outbox, grouped by destination partition
    p_sz_t* msg_rank = nullptr;
    p_sz_t* msg_off = nullptr;            // p + 1 counters: exclusive end of every destination's group
    idx_t active_sz = 0;                  // filled by the step: the new active-set size (active_set_sz[p_id])
    idx_t msg_c = 0;                      // filled by the step: messages in the outbox
};

template <typename T_sym_> class GPU_SACA {
    static_assert(sizeof(T_sym_) == 2, "the partition sort is built for uint16 symbols");

public:
    static constexpr idx_t STREAM_C = 3; // buffer sets, one dispatcher thread each (include/GPU_SACA.hpp:90)

    // The reference's command-line use: the text at ip_path is one partition, its suffix array goes to op_path.
    GPU_SACA(const std::string& ip_path, const std::string& op_path, int key_words = 1)
        : ip_path_(ip_path), op_path_(op_path), key_words_(key_words)
    {
    }

    // For a pipeline that drives partitions itself: p partitions of at most max_part_sz suffixes, staged through slabs
    // of chunk_cap suffixes (a multiple of 4096, as the reference's slab_capacity gives).
    GPU_SACA(idx_t max_part_sz, p_id_t p, int key_words = 1, idx_t chunk_cap = idx_t(1) << 21)
        : key_words_(key_words), p_(p), max_part_sz_(max_part_sz), chunk_cap_(chunk_cap), msg_off_(p, std::vector<p_sz_t>(p, 0)),
          active_sz_(p, 0)
    {
    }

    GPU_SACA(const GPU_SACA&) = delete;
    GPU_SACA& operator=(const GPU_SACA&) = delete;

    ~GPU_SACA()
    {
        for (idx_t b = 0; b < STREAM_C; ++b)
            if (csa_[b])
                csa_destroy(csa_[b]);
        for (idx_t b = 0; b < STREAM_C; ++b)
            if (resident_[b])
                csa_destroy(resident_[b]);
    }

    static constexpr double MEM_SAFETY_MARGIN = 0.1;        // spared for the runtime (include/GPU_SACA.hpp:44)
    static constexpr double PART_SZ_IMBALANCE_SLACK = 1.20; // partitions may come out larger than planned (include/GPU_SACA.hpp:61)

    // Largest partition such that STREAM_C handles of the steps' floor plan, workspaces included, fit into
    // free_device_bytes with the reference's margins (src/GPU_SACA.cu:365-403): a host that creates its partitions no
    // larger than this finds that allocate_device_space() succeeds and that no step runs out of device memory, because
    // the steps allocate nothing.
    idx_t partition_size_upper_bound(std::size_t free_device_bytes) const
    {
        const double budget_f = static_cast<double>(free_device_bytes) * (1.0 - MEM_SAFETY_MARGIN) / PART_SZ_IMBALANCE_SLACK;
        const std::size_t budget = static_cast<std::size_t>(budget_f);
        const std::size_t per_suffix = csa_step_bytes_per_suffix(key_words_);
        idx_t p_sz_max = budget / (STREAM_C * per_suffix);
        if (p_sz_max > CSA_MAX_PART_SZ)
            p_sz_max = CSA_MAX_PART_SZ;
        // the workspace follows the partition size: shrink until block and workspace fit together
        while (p_sz_max > 0 && STREAM_C * (p_sz_max * per_suffix + csa_workspace_bytes(p_sz_max)) > budget) {
            const std::size_t ws = STREAM_C * csa_workspace_bytes(p_sz_max);
            const idx_t next = ws >= budget ? 0 : (budget - ws) / (STREAM_C * per_suffix);
            p_sz_max = next < p_sz_max ? next : p_sz_max - 1;
        }
        return p_sz_max;
    }

    // What allocate_device_space() takes from the device for partitions of up to part_sz suffixes.
    std::size_t device_bytes_required(idx_t part_sz) const
    {
        return STREAM_C * (part_sz * csa_step_bytes_per_suffix(key_words_) + csa_workspace_bytes(part_sz));
    }

    // One handle per buffer set, each with everything the three members will ever use; false if the device has no
    // room (the reference returns the same way, src/GPU_SACA.cu:550-560).
    bool allocate_device_space()
    {
        for (idx_t b = 0; b < STREAM_C; ++b)
            if (!csa_[b] && csa_create_steps(max_part_sz_, key_words_, &csa_[b]) != CSA_OK) {
                std::cerr << csa_last_error() << "\n";
                return false;
            }
        return true;
    }

    // The stream (a hipStream_t) of a buffer set; the default stream otherwise.
    void set_stream(idx_t buf_id, void* stream) { stream_[buf_id] = stream; }

    // Context the coming generation resolves to, and its index (src/GPU_SACA.cu:1043-1049).
    void set_context(idx_t ctx, idx_t gen)
    {
        ctx_ = ctx;
        gen_ = gen;
    }

    // What the reference's backend holds per partition and the members fill: the exclusive END offset of every
    // destination's group in the partition's outbox (backend_->msg_off(p_id)) and the new active-set size
    // (backend_->active_slot(p_id)).
    p_sz_t* msg_off(p_id_t p_id) { return msg_off_[p_id].data(); }
    idx_t* active_slot(p_id_t p_id) { return &active_sz_[p_id]; }
    idx_t chunk_cap() const { return chunk_cap_; }

    // The partition's slabs in, its ranks, lanes and outbox back in the slabs (src/GPU_SACA.cu:1112-1331).
    void sort_and_init_rank_and_filter(p_id_t p_id, Partition_Assembly& p_assembly, idx_t buf_id)
    {
        std::vector<csa_slab> slabs = gather(p_assembly);
        check(csa_sort_init_slabs(csa_[buf_id], slabs.data(), static_cast<std::uint32_t>(slabs.size()), total(slabs), key_words_, p_,
                                  chunk_cap_, msg_off(p_id), active_slot(p_id), stream_[buf_id]));
        spread(slabs, p_assembly);
    }

    // The same for a later generation; every slab also carries its chunk of the partition's inbox (src/GPU_SACA.cu:1715-1995).
    void sort_and_re_rank_and_filter(p_id_t p_id, Partition_Assembly& p_assembly, idx_t buf_id)
    {
        std::vector<csa_slab> slabs = gather(p_assembly);
        idx_t inbox_sz = 0;
        for (const auto& s : slabs)
            inbox_sz += s.inbox_sz;
        check(csa_sort_rerank_slabs(csa_[buf_id], slabs.data(), static_cast<std::uint32_t>(slabs.size()), total(slabs), inbox_sz, ctx_,
                                    p_, chunk_cap_, msg_off(p_id), active_slot(p_id), stream_[buf_id]));
        spread(slabs, p_assembly);
#ifdef TESTS
        // what the reference checks after a generation under -DTESTS (src/GPU_SACA.cu:2055-2063; the device trap of
        // include/GPU_SACA.cuh:246-249)
        csa_step_result r{};
        check(csa_last_step_result(csa_[buf_id], &r));
        if (r.unserved > 0)
            fail("Active suffixes with no message received: " + std::to_string(r.unserved));
        if (r.incoherent_pills > 0)
            fail("Incoherent poison-pill receipts: " + std::to_string(r.incoherent_pills));
#endif
    }

    // Lanes and final ranks in the slabs -> the partition's stretch of the output, cut for the output file whose
    // byte range for this partition starts at out_lo = 5 * P_off[p_id] (src/GPU_SACA.cu:2107-2164).
    void scatter_to_rank_order(p_id_t /*p_id*/, Partition_Assembly& p_assembly, idx_t buf_id, idx_t out_lo)
    {
        std::vector<csa_slab> slabs = gather(p_assembly);
        check(csa_scatter_slabs(csa_[buf_id], slabs.data(), static_cast<std::uint32_t>(slabs.size()), total(slabs), out_lo, chunk_cap_,
                                stream_[buf_id]));
    }

    void sort_and_init_rank_and_filter(p_id_t /*p_id*/, Device_Partition& part, idx_t buf_id)
    {
        csa_step_result r{};
        check(csa_sort_init_dev(csa_[buf_id], part.key, key_words_, part.suf, part.beta, part.sz, p_, part.rank_out, part.suf_out,
                                part.msg_target, part.msg_rank, part.msg_off, stream_[buf_id], &r));
        part.active_sz = r.active;
        part.msg_c = r.messages;
    }

    void sort_and_re_rank_and_filter(p_id_t /*p_id*/, Device_Partition& part, idx_t buf_id)
    {
        csa_step_result r{};
        check(csa_sort_rerank_dev(csa_[buf_id], part.rank, part.suf, part.beta, part.sz, part.inbox_target, part.inbox_rank,
                                  part.inbox_sz, ctx_, p_, part.rank_out, part.suf_out, part.msg_target, part.msg_rank,
                                  part.msg_off, stream_[buf_id], &r));
        part.active_sz = r.active;
        part.msg_c = r.messages;
    }

    // part_sz suffixes (lanes) with their final partition-local ranks -> the partition's stretch of the suffix array.
    void scatter_to_rank_order(p_id_t /*p_id*/, const std::uint8_t* suf, const p_sz_t* rank, idx_t part_sz, std::uint8_t* sa40,
                               idx_t buf_id)
    {
        check(csa_scatter_to_rank_order_dev(csa_[buf_id], suf, rank, part_sz, sa40, stream_[buf_id]));
    }

    // A partition whose symbols are a window of the text resident in HBM: every generation inside one call. The handles
    // of allocate_device_space() are made for the steps; this member keeps handles of its own (csa_create), made on
    // first use.
    void sort_partition(const T_sym_* d_text, idx_t part_sz, idx_t index_base, std::uint8_t* d_sa40, idx_t buf_id,
                        csa_stats* stats = nullptr)
    {
        if (!resident_[buf_id])
            check(csa_create(max_part_sz_, key_words_, &resident_[buf_id]));
        check(csa_sort_partition_u16_dev(resident_[buf_id], reinterpret_cast<const std::uint16_t*>(d_text), part_sz, index_base, d_sa40,
                                         stream_[buf_id], 0, stats));
    }

    // Builds the suffix array of the text file as one partition and writes it as 5-byte entries (src/main.cu:27-30).
    void build_SA()
    {
        std::ifstream in(ip_path_, std::ios::binary | std::ios::ate);
        if (!in)
            fail("cannot open " + ip_path_);
        const std::streamoff bytes = in.tellg();
        if (bytes % 2 != 0)
            fail(ip_path_ + " does not hold whole 16-bit symbols");
        std::vector<std::uint16_t> text(static_cast<std::size_t>(bytes / 2));
        in.seekg(0);
        in.read(reinterpret_cast<char*>(text.data()), bytes);
        if (!in && bytes)
            fail("cannot read " + ip_path_);
        std::vector<std::uint8_t> sa40(5 * text.size());
        check(csa_sort_partition_u16(text.data(), text.size(), key_words_, sa40.data(), &stats_));
        std::ofstream out(op_path_, std::ios::binary | std::ios::trunc);
        out.write(reinterpret_cast<const char*>(sa40.data()), static_cast<std::streamsize>(sa40.size()));
        if (!out)
            fail("cannot write " + op_path_);
    }

    const csa_stats& stats() const { return stats_; } // generations and their sizes of the last build_SA()

private:
    static std::vector<csa_slab> gather(const Partition_Assembly& a)
    {
        std::vector<csa_slab> slabs;
        slabs.reserve(a.slab.size());
        for (const auto* s : a.slab)
            slabs.push_back(*s);
        return slabs;
    }
    static void spread(const std::vector<csa_slab>& slabs, Partition_Assembly& a)
    {
        for (std::size_t c = 0; c < slabs.size(); ++c)
            a.slab[c]->set_outbox_off_and_size(slabs[c].outbox_off, slabs[c].outbox_sz);
    }
    static idx_t total(const std::vector<csa_slab>& slabs)
    {
        idx_t sz = 0;
        for (const auto& s : slabs)
            sz += s.size;
        return sz;
    }

    [[noreturn]] static void fail(const std::string& what)
    {
        std::cerr << what << ". Aborting.\n";
        std::exit(EXIT_FAILURE);
    }
    static void check(int status)
    {
        if (status != CSA_OK)
            fail(csa_last_error());
    }

    std::string ip_path_, op_path_;
    int key_words_ = 1;
    p_id_t p_ = 1;
    idx_t max_part_sz_ = 0;
    idx_t chunk_cap_ = idx_t(1) << 21; // the reference's CHUNK_CAP (include/GPU_SACA.hpp:99)
    std::vector<std::vector<p_sz_t>> msg_off_;
    std::vector<idx_t> active_sz_;
    idx_t ctx_ = 0, gen_ = 0;
    csa_handle* csa_[STREAM_C] = {};
    csa_handle* resident_[STREAM_C] = {};
    void* stream_[STREAM_C] = {};
    csa_stats stats_{};
};

} // namespace cascade_hip

#endif
