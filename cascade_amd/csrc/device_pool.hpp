// The handle's device memory as one block that every call carves up for itself. Host code only.
//
// The reference allocates each stream's buffers once (GPU_SACA::allocate_device_space, src/GPU_SACA.cu:535-590) and
// reaches its floor plan of 2 * (key + 8 + 4 + 4) + 1 bytes per suffix by reusing them under other names inside a
// step: the outbox over the sorted buffers (src/GPU_SACA.cu:1268-1270), narrowed ranks and packed lanes over the key
// buffer (:1292,1301), the inbox over the spare suffix buffer (:1805-1806). Here the reuse is explicit: a step takes a
// column from the block when it first writes it and gives it back after its last read, so what a handle must hold is
// the largest sum of columns alive at one time, not the sum of all of them. Nothing is allocated after csa_create.
#pragma once

#include <cstdint>
#include <vector>

namespace csa {

class DevicePool {
public:
    static constexpr uint64_t ALIGN = 256;

    void attach(unsigned char* base, uint64_t bytes)
    {
        base_ = base;
        bytes_ = bytes & ~(ALIGN - 1);
        reset();
    }
    unsigned char* base() const { return base_; }
    uint64_t bytes() const { return bytes_; }
    // Forgets every column: the state at the start of a call.
    void reset()
    {
        free_.clear();
        used_.clear();
        if (bytes_)
            free_.push_back({0, bytes_});
        in_use_ = high_water_ = 0;
    }
    // Bytes taken at the busiest moment since the last reset.
    uint64_t high_water() const { return high_water_; }
    uint64_t in_use() const { return in_use_; }

    // A column of `bytes` bytes, or nullptr if no free stretch is long enough. Columns that live to the end of a call
    // (a step's inputs while they wait, its outputs) are taken from the top of the block, the short-lived ones from
    // the bottom, so that neither kind cuts the other's free space in pieces.
    void* take(uint64_t bytes, bool from_top = false)
    {
        const uint64_t len = (bytes + ALIGN - 1) & ~(ALIGN - 1);
        if (len == 0)
            return base_; // an empty column: any address will do, nothing is recorded
        if (!from_top) {
            for (size_t i = 0; i < free_.size(); ++i)
                if (free_[i].len >= len)
                    return carve(i, free_[i].off, len);
        } else {
            for (size_t i = free_.size(); i-- > 0;)
                if (free_[i].len >= len)
                    return carve(i, free_[i].off + free_[i].len - len, len);
        }
        return nullptr;
    }

    // Gives a column back; pointers that are not columns of the pool (a caller's own buffer, nullptr) are ignored.
    void give(const void* p)
    {
        if (!p || !base_)
            return;
        const unsigned char* q = static_cast<const unsigned char*>(p);
        if (q < base_ || q >= base_ + bytes_)
            return;
        const uint64_t off = (uint64_t)(q - base_);
        for (size_t u = 0; u < used_.size(); ++u) {
            if (used_[u].off != off)
                continue;
            const Span s = used_[u];
            used_.erase(used_.begin() + (long)u);
            in_use_ -= s.len;
            size_t i = 0;
            while (i < free_.size() && free_[i].off < s.off)
                ++i;
            free_.insert(free_.begin() + (long)i, s);
            if (i + 1 < free_.size() && free_[i].off + free_[i].len == free_[i + 1].off) {
                free_[i].len += free_[i + 1].len;
                free_.erase(free_.begin() + (long)i + 1);
            }
            if (i > 0 && free_[i - 1].off + free_[i - 1].len == free_[i].off) {
                free_[i - 1].len += free_[i].len;
                free_.erase(free_.begin() + (long)i);
            }
            return;
        }
    }

private:
    struct Span {
        uint64_t off, len;
    };
    void* carve(size_t i, uint64_t off, uint64_t len)
    {
        const Span f = free_[i];
        free_.erase(free_.begin() + (long)i);
        if (off + len < f.off + f.len)
            free_.insert(free_.begin() + (long)i, Span{off + len, f.off + f.len - (off + len)});
        if (off > f.off)
            free_.insert(free_.begin() + (long)i, Span{f.off, off - f.off});
        used_.push_back(Span{off, len});
        in_use_ += len;
        if (in_use_ > high_water_)
            high_water_ = in_use_;
        return base_ + off;
    }

    unsigned char* base_ = nullptr;
    uint64_t bytes_ = 0;
    std::vector<Span> free_; // ascending by offset, neighbours merged
    std::vector<Span> used_;
    uint64_t in_use_ = 0, high_water_ = 0;
};

} // namespace csa
