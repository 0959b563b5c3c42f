#include "pool.h"

namespace vdnn {

static size_t round_up(size_t v, size_t g) { return (v + g - 1) / g * g; }

void Pool::init(uintptr_t base, size_t bytes) {
    clear();
    base_ = base;
    total_ = bytes / kGranularity * kGranularity;
    if (total_) insert_free(0, total_);
}

void Pool::clear() {
    free_by_off_.clear(); free_by_size_.clear(); used_.clear();
    base_ = 0; total_ = in_use_ = peak_in_use_ = peak_extent_ = 0;
}

void Pool::insert_free(size_t off, size_t size) {
    free_by_off_[off] = size;
    free_by_size_.emplace(size, off);
}

void Pool::erase_free(std::map<size_t, size_t>::iterator it) {
    auto range = free_by_size_.equal_range(it->second);
    for (auto s = range.first; s != range.second; ++s)
        if (s->second == it->first) { free_by_size_.erase(s); break; }
    free_by_off_.erase(it);
}

size_t Pool::extent() const {
    size_t e = 0;
    for (const auto& u : used_) if (u.first + u.second > e) e = u.first + u.second;
    return e;
}

size_t Pool::largest_free() const { return free_by_size_.empty() ? 0 : free_by_size_.rbegin()->first; }

uintptr_t Pool::allocate(size_t bytes) {
    if (!total_) return 0;
    const size_t need = round_up(bytes ? bytes : 1, kGranularity);
    if (cap_ && in_use_ + need > cap_) return 0;
    // best fit; among equal sizes the multimap keeps insertion order, take the lowest offset
    auto s = free_by_size_.lower_bound(need);
    if (s == free_by_size_.end()) return 0;
    size_t best_off = s->second;
    for (auto t = s; t != free_by_size_.end() && t->first == s->first; ++t)
        if (t->second < best_off) best_off = t->second;
    auto it = free_by_off_.find(best_off);
    const size_t off = it->first, size = it->second;
    erase_free(it);
    if (size > need) insert_free(off + need, size - need);
    used_[off] = need;
    in_use_ += need;
    if (in_use_ > peak_in_use_) peak_in_use_ = in_use_;
    if (off + need > peak_extent_) peak_extent_ = off + need;
    return base_ + off;
}

bool Pool::release(uintptr_t ptr) {
    if (ptr < base_) return false;
    size_t off = ptr - base_;
    auto u = used_.find(off);
    if (u == used_.end()) return false;
    size_t size = u->second;
    used_.erase(u);
    in_use_ -= size;
    // coalesce with the neighbours
    auto next = free_by_off_.lower_bound(off);
    if (next != free_by_off_.end() && next->first == off + size) {
        size += next->second;
        erase_free(next);
    }
    auto prev = free_by_off_.lower_bound(off);
    if (prev != free_by_off_.begin()) {
        --prev;
        if (prev->first + prev->second == off) {
            off = prev->first;
            size += prev->second;
            erase_free(prev);
        }
    }
    insert_free(off, size);
    return true;
}

} // namespace vdnn
