// Host-side bookkeeping for sub-allocating one contiguous address range (in
// practice: one block carved from the hipMalloc'd device arena).  First fit with
// coalescing of freed neighbours.  It never dereferences the addresses it hands
// out, so it works the same over device memory and, in the unit tests, over a
// made-up base address.
#pragma once

#include <stddef.h>
#include <stdint.h>

#include <map>

namespace fastconv {

class RangeAllocator {
   public:
    RangeAllocator(void *base, size_t bytes, size_t align = 256)
        : base_((uintptr_t)base), bytes_(bytes), align_(align ? align : 1), used_(0), peak_(0) {
        if (bytes_ > 0) free_[0] = bytes_;
    }

    // NULL when no free block is large enough (or bytes == 0).
    void *Allocate(size_t bytes) {
        if (bytes == 0) return NULL;
        const size_t need = (bytes + align_ - 1) / align_ * align_;
        for (std::map<size_t, size_t>::iterator it = free_.begin(); it != free_.end(); ++it) {
            if (it->second < need) continue;
            const size_t off = it->first, len = it->second;
            free_.erase(it);
            if (len > need) free_[off + need] = len - need;
            live_[off] = need;
            used_ += need;
            if (used_ > peak_) peak_ = used_;
            return (void *)(base_ + off);
        }
        return NULL;
    }

    // false when p was not handed out by Allocate (or was freed already).
    bool Free(void *p) {
        const size_t off = (uintptr_t)p - base_;
        std::map<size_t, size_t>::iterator it = live_.find(off);
        if (p == NULL || it == live_.end()) return false;
        size_t len = it->second;
        size_t start = off;
        live_.erase(it);
        used_ -= len;
        std::map<size_t, size_t>::iterator next = free_.lower_bound(start);
        if (next != free_.end() && next->first == start + len) {
            len += next->second;
            free_.erase(next);
        }
        std::map<size_t, size_t>::iterator prev = free_.lower_bound(start);
        if (prev != free_.begin()) {
            --prev;
            if (prev->first + prev->second == start) {
                start = prev->first;
                len += prev->second;
                free_.erase(prev);
            }
        }
        free_[start] = len;
        return true;
    }

    bool Owns(const void *p) const { return live_.count((uintptr_t)p - base_) != 0; }
    size_t SizeOf(const void *p) const {
        std::map<size_t, size_t>::const_iterator it = live_.find((uintptr_t)p - base_);
        return it == live_.end() ? 0 : it->second;
    }
    size_t capacity() const { return bytes_; }
    size_t used() const { return used_; }
    size_t peak() const { return peak_; }
    size_t live_blocks() const { return live_.size(); }
    size_t free_blocks() const { return free_.size(); }
    size_t largest_free() const {
        size_t m = 0;
        for (std::map<size_t, size_t>::const_iterator it = free_.begin(); it != free_.end(); ++it)
            if (it->second > m) m = it->second;
        return m;
    }

   private:
    uintptr_t base_;
    size_t bytes_, align_, used_, peak_;
    std::map<size_t, size_t> free_;   // offset -> length
    std::map<size_t, size_t> live_;   // offset -> length
};

}  // namespace fastconv
