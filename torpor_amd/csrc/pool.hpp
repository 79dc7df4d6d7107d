// Pooled HBM allocator: one arena cut into fixed slabs, extents of whole slabs
// handed out best-fit with coalescing on release.
//
// Takes the place of the reference's BuddyBasedBlockManager / Block
// (include/server/block_manager.hpp:23-125, 260-418): there, budget/128 MiB
// physical blocks are cudaMalloc'ed up front and carved into 2 MiB or 16 MiB
// slots by a first-fit bitmap scan.  Here the arena is one allocation (sized
// for a 288 GB part), a model occupies two extents (weight image, activation
// arena), and all bookkeeping is offset arithmetic, so the class is pure host
// logic and runs without a device.
//
// Two policies, as the reference has two managers chosen by BLOCK_MANAGER (memory_manager.hpp:46-52):
//   kBestFit    the default described above.
//   kFixedSize  FixedSizeBlockManager (block_manager.hpp:188-258): a released extent is kept, whole, in an
//               idle list of its exact size and the next request of that size takes the one released last;
//               a size with no idle extent is carved from the free part of the arena, and when that fails
//               idle extents are given back -- largest size first (the reference's idle map is ordered by
//               std::greater, types.hpp:31), the one released last first -- until it fits.  The reference keeps a byte budget over raw cudaMalloc / cudaFree and allocates beyond
//               it when nothing is left to free (block_manager.hpp:222-234); here the arena is the budget
//               and that case is "no fit".  Served models come in a few sizes, so a swap-in usually gets the
//               extents a model of its kind left behind without any search or coalescing.
#pragma once
#include <cstdint>
#include <iterator>
#include <map>
#include <set>
#include <utility>
#include <vector>

namespace tp {

class SlabPool {
public:
    static constexpr uint64_t kSlab = 2ull << 20;  // 2 MiB, the reference's regular slot (block_manager.hpp:28)

    enum Policy : int { kBestFit = 0, kFixedSize = 1 };

    SlabPool() = default;
    void reset(uint64_t capacity_bytes, int policy = -1) {
        if (policy == kBestFit || policy == kFixedSize) policy_ = policy;
        capacity_ = (capacity_bytes / kSlab) * kSlab;
        free_.clear();
        by_size_.clear();
        used_.clear();
        idle_.clear();
        if (capacity_) add_free(0, capacity_);
        used_bytes_ = cached_bytes_ = 0;
        idle_count_ = 0;
    }
    int policy() const { return policy_; }
    static uint64_t round_up(uint64_t bytes) { return ((bytes + kSlab - 1) / kSlab) * kSlab; }

    // Returns the arena offset of a contiguous extent, or UINT64_MAX.
    uint64_t alloc(uint64_t bytes) {
        if (bytes == 0) bytes = 1;
        if (bytes > capacity_) return UINT64_MAX;  // also keeps round_up from wrapping
        const uint64_t need = round_up(bytes);
        if (policy_ == kFixedSize) {
            auto it = idle_.find(need);
            if (it != idle_.end() && !it->second.empty()) {  // block_manager.hpp:193-198: the one released last
                const uint64_t off = it->second.back();
                it->second.pop_back();
                --idle_count_;
                cached_bytes_ -= need;
                used_[off] = need;
                used_bytes_ += need;
                return off;
            }
            uint64_t off = carve(need);
            // block_manager.hpp:205-221: give idle extents back, largest size first, until the request fits
            // (they coalesce with their free neighbours, which the reference's cudaFree leaves to the driver)
            while (off == UINT64_MAX && trim_one()) off = carve(need);
            return off;
        }
        return carve(need);
    }

    // Returns false when `off` is not the start of a live extent.
    bool release(uint64_t off) {
        auto u = used_.find(off);
        if (u == used_.end()) return false;
        const uint64_t len = u->second;
        used_.erase(u);
        used_bytes_ -= len;
        if (policy_ == kFixedSize) {  // block_manager.hpp:243-252 with free_flag == false
            idle_[len].push_back(off);
            ++idle_count_;
            cached_bytes_ += len;
            return true;
        }
        give_back(off, len);
        return true;
    }

    // kFixedSize: gives every idle extent back to the free part of the arena; returns how many there were.
    size_t trim() {
        size_t n = 0;
        while (trim_one()) ++n;
        return n;
    }

    uint64_t capacity() const { return capacity_; }
    uint64_t used_bytes() const { return used_bytes_; }
    uint64_t cached_bytes() const { return cached_bytes_; }   // idle extents of the fixed-size policy
    size_t idle_extents() const { return idle_count_; }
    uint64_t free_bytes() const { return capacity_ - used_bytes_; }
    // the largest request that fits without giving an idle extent back
    uint64_t largest_free() const { return by_size_.empty() ? 0 : by_size_.rbegin()->first; }
    size_t live_extents() const { return used_.size(); }
    size_t free_extents() const { return free_.size(); }
    uint64_t extent_size(uint64_t off) const {
        auto u = used_.find(off);
        return u == used_.end() ? 0 : u->second;
    }
    const std::map<uint64_t, uint64_t>& used() const { return used_; }
    const std::map<uint64_t, uint64_t>& free_map() const { return free_; }
    const std::map<uint64_t, std::vector<uint64_t>>& idle_map() const { return idle_; }

private:
    uint64_t carve(uint64_t need) {
        // best fit: the smallest free extent that holds `need`, the lowest address among equals.  The
        // size-ordered index makes this a tree search; with tens of thousands of free extents (a
        // 288 GB arena of small models) a scan of the address-ordered map would cost milliseconds.
        auto best = by_size_.lower_bound(std::make_pair(need, (uint64_t)0));
        if (best == by_size_.end()) return UINT64_MAX;
        const uint64_t len = best->first, off = best->second;
        drop_free(off, len);
        if (len > need) add_free(off + need, len - need);
        used_[off] = need;
        used_bytes_ += need;
        return off;
    }

    // A freed extent joins its free neighbours.
    void give_back(uint64_t off, uint64_t len) {
        auto next = free_.lower_bound(off);
        if (next != free_.end() && off + len == next->first) {
            const uint64_t noff = next->first, nlen = next->second;
            len += nlen;
            drop_free(noff, nlen);
        }
        next = free_.lower_bound(off);
        if (next != free_.begin()) {
            auto prev = std::prev(next);
            if (prev->first + prev->second == off) {
                const uint64_t poff = prev->first, plen = prev->second;
                drop_free(poff, plen);
                add_free(poff, plen + len);
                return;
            }
        }
        add_free(off, len);
    }
    bool trim_one() {
        while (!idle_.empty()) {
            auto it = std::prev(idle_.end());  // largest size
            if (it->second.empty()) {
                idle_.erase(it);
                continue;
            }
            const uint64_t off = it->second.back();
            it->second.pop_back();
            --idle_count_;
            cached_bytes_ -= it->first;
            give_back(off, it->first);
            return true;
        }
        return false;
    }
    void add_free(uint64_t off, uint64_t len) {
        free_[off] = len;
        by_size_.emplace(len, off);
    }
    void drop_free(uint64_t off, uint64_t len) {
        free_.erase(off);
        by_size_.erase(std::make_pair(len, off));
    }

    int policy_ = kBestFit;
    uint64_t capacity_ = 0;
    uint64_t used_bytes_ = 0, cached_bytes_ = 0;
    size_t idle_count_ = 0;
    std::map<uint64_t, std::vector<uint64_t>> idle_;  // kFixedSize: extent size -> offsets, released last at the back
    std::map<uint64_t, uint64_t> free_;  // offset -> length, address ordered, never adjacent
    std::set<std::pair<uint64_t, uint64_t>> by_size_;  // (length, offset) of the same extents
    std::map<uint64_t, uint64_t> used_;  // offset -> length
};

}  // namespace tp
