// LRU eviction policy over whole models on one GPU.
//
// Same decisions as the reference's LRUEvictor
// (include/server/evictor.hpp:190-264): a hit moves the model to the front and
// evicts nothing; a miss evicts from the tail, skipping locked entries, while
// cur + size >= budget, then inserts at the front.  One deliberate difference:
// the reference spins forever when every remaining entry is locked or the list
// is empty (evictor.hpp:211-224); here the loop stops and the caller sees
// `over_budget` so it can refuse the request.
#pragma once
#include <cstdint>
#include <list>
#include <set>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

namespace tp {

class LruEvictor {
public:
    explicit LruEvictor(uint64_t budget = 0) : budget_(budget) {}
    void set_budget(uint64_t b) { budget_ = b; }
    uint64_t budget() const { return budget_; }
    uint64_t cur_size() const { return cur_; }

    // evictor.hpp:200-235
    std::vector<std::string> check_and_add(const std::string& func, uint64_t sz, bool* over_budget = nullptr) {
        if (over_budget) *over_budget = false;
        auto hit = index_.find(func);
        if (hit != index_.end()) {
            items_.splice(items_.begin(), items_, hit->second);
            return {};
        }
        std::vector<std::string> victims;
        while (cur_ + sz >= budget_) {
            bool found = false;
            for (auto it = items_.rbegin(); it != items_.rend(); ++it) {
                if (locked_.count(it->first)) continue;
                victims.push_back(it->first);
                cur_ -= it->second;
                index_.erase(it->first);
                items_.erase(std::next(it).base());
                found = true;
                break;
            }
            if (!found) {
                if (over_budget) *over_budget = true;
                break;
            }
        }
        items_.emplace_front(func, sz);
        index_[func] = items_.begin();
        cur_ += sz;
        return victims;
    }

    // evictor.hpp:237-247 ; returns false when the model was not tracked
    bool force_evict(const std::string& func) {
        auto it = index_.find(func);
        if (it == index_.end()) return false;
        cur_ -= it->second->second;
        items_.erase(it->second);
        index_.erase(it);
        return true;
    }

    // Next eviction candidate (tail-most unlocked entry other than `keep`), without removing it.
    bool peek_victim(const std::string& keep, std::string* out) const {
        for (auto it = items_.rbegin(); it != items_.rend(); ++it) {
            if (locked_.count(it->first) || it->first == keep) continue;
            *out = it->first;
            return true;
        }
        return false;
    }

    void lock(const std::string& func) {  // evictor.hpp:249-254
        if (index_.count(func)) locked_.insert(func);
    }
    void unlock(const std::string& func) { locked_.erase(func); }  // evictor.hpp:256-260
    bool contains(const std::string& func) const { return index_.count(func) != 0; }
    size_t size() const { return items_.size(); }
    std::vector<std::string> order() const {  // most recent first
        std::vector<std::string> v;
        for (auto& kv : items_) v.push_back(kv.first);
        return v;
    }

private:
    uint64_t budget_;
    uint64_t cur_ = 0;
    std::list<std::pair<std::string, uint64_t>> items_;
    std::unordered_map<std::string, std::list<std::pair<std::string, uint64_t>>::iterator> index_;
    std::set<std::string> locked_;
};

}  // namespace tp
