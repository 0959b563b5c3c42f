// Sub-allocator over one reserved range of device memory (the role cnmem plays in the reference:
// network.cu:47-53 reserves, layer.cu:989-1011 and the drivers carve tensors out of it).
// Host-only bookkeeping: it never touches the memory it manages, so the same class serves a real
// hipMalloc'd range and the virtual range of a plan-only context.
#pragma once
#include <cstddef>
#include <cstdint>
#include <map>
#include <unordered_map>

namespace vdnn {

class Pool {
public:
    static constexpr size_t kGranularity = 512; // cnmem's allocation granularity

    void   init(uintptr_t base, size_t bytes);
    void   clear();
    bool   initialised() const { return total_ != 0; }
    // best fit; returns 0 on out-of-memory (no block fits, or the cap would be exceeded)
    uintptr_t allocate(size_t bytes);
    // false if ptr is not a live block
    bool   release(uintptr_t ptr);
    size_t total() const { return total_; }
    size_t in_use() const { return in_use_; }
    size_t peak_in_use() const { return peak_in_use_; }
    size_t peak_extent() const { return peak_extent_; }
    size_t live_blocks() const { return used_.size(); }
    size_t largest_free() const;
    void   reset_peak() { peak_in_use_ = in_use_; peak_extent_ = extent(); }
    void   set_cap(size_t cap) { cap_ = cap; }
    size_t cap() const { return cap_; }
    uintptr_t base() const { return base_; }

private:
    size_t extent() const;
    uintptr_t base_ = 0;
    size_t total_ = 0, in_use_ = 0, peak_in_use_ = 0, peak_extent_ = 0, cap_ = 0;
    std::map<size_t, size_t> free_by_off_;             // offset -> size
    std::multimap<size_t, size_t> free_by_size_;       // size -> offset
    std::unordered_map<size_t, size_t> used_;          // offset -> size
    void erase_free(std::map<size_t, size_t>::iterator it);
    void insert_free(size_t off, size_t size);
};

} // namespace vdnn
