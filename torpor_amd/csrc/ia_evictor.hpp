// Interference-aware eviction policy: a two-class LRU per GPU.
//
// Same decisions as the reference's InterferenceAwareEvictor
// (include/server/evictor.hpp:28-188).  A model of level Median or Heavy that
// is resident on exactly one GPU is "protected" there (the reference's first
// class): losing it means a swap over the host link next time, so it is
// evicted only after every unprotected entry (light models, and models that
// another GPU also holds and could serve or hand over a peer link) is gone.
// When a second copy appears the first one loses its protection, and when an
// eviction leaves a single copy that copy gains it.
//
// Layout differs from the reference's four list/index vectors: each GPU keeps
// one name -> {stamp, size, class} table plus, per class, a stamp-ordered map;
// "move to front" is "take a new stamp".  One deliberate difference in
// behaviour: the reference loops forever when the protected class holds no
// unlocked entry (evictor.hpp:85-97); here the search stops and the caller
// sees `over_budget`.
#pragma once
#include <cstdint>
#include <map>
#include <set>
#include <string>
#include <unordered_map>
#include <vector>

namespace tp {

enum ModelLevel : int { LEVEL_LIGHT = 0, LEVEL_MEDIAN = 1, LEVEL_HEAVY = 2 };  // evictor.hpp:10-12

class IaEvictor {
public:
    IaEvictor(int gpu_count = 1, uint64_t budget = 0) : budget_(budget), gpus_((size_t)(gpu_count > 0 ? gpu_count : 1)) {}
    void set_budget(uint64_t b) { budget_ = b; }
    uint64_t budget() const { return budget_; }
    int gpu_count() const { return (int)gpus_.size(); }
    uint64_t cur_size(int gpu = 0) const { return ok(gpu) ? gpus_[(size_t)gpu].used : 0; }
    size_t size(int gpu = 0) const { return ok(gpu) ? gpus_[(size_t)gpu].entries.size() : 0; }

    // controller.hpp:142-152 keeps the level per function; a victim's level is looked up at eviction time.
    void set_level(const std::string& func, int level) { level_[func] = level; }
    int level(const std::string& func) const {
        auto it = level_.find(func);
        return it == level_.end() ? (int)LEVEL_LIGHT : it->second;  // map default, as operator[] gives in the reference
    }

    // evictor.hpp:41-147
    std::vector<std::string> check_and_add(int gpu, const std::string& func, uint64_t sz, bool* over_budget = nullptr) {
        if (over_budget) *over_budget = false;
        if (!ok(gpu)) return {};
        Gpu& g = gpus_[(size_t)gpu];
        auto where = holders_.find(func);
        if (where != holders_.end() && where->second.count(gpu)) {  // hit: refresh within its class
            auto e = g.entries.find(func);
            if (e != g.entries.end()) restamp(g, e->second, e->second.prot, func);
            return {};
        }
        std::vector<std::string> victims;
        for (int cls = 0; cls < 2; ++cls) {  // unprotected entries first, then protected ones
            while (g.used + sz >= budget_) {
                auto& order = g.order[cls];
                auto v = order.begin();
                while (v != order.end() && g.locked.count(v->second)) ++v;
                if (v == order.end()) break;
                const std::string name = v->second;
                g.used -= g.entries[name].size;
                g.entries.erase(name);
                order.erase(v);
                victims.push_back(name);
            }
        }
        if (g.used + sz >= budget_ && over_budget) *over_budget = true;

        const bool weighty = level(func) >= LEVEL_MEDIAN;
        std::set<int>& mine = holders_[func];
        const bool protect = weighty && mine.empty();
        Entry e;
        e.size = sz;
        e.prot = protect;
        e.stamp = ++clock_;
        g.entries[func] = e;
        g.order[protect ? 1 : 0][e.stamp] = func;
        if (weighty && !mine.empty()) {  // a second copy exists now: the others lose their protection
            for (int other : mine) {
                Gpu& og = gpus_[(size_t)other];
                auto oe = og.entries.find(func);
                if (oe != og.entries.end() && oe->second.prot) restamp(og, oe->second, false, func);
            }
        }
        mine.insert(gpu);
        g.used += sz;

        for (const auto& mod : victims) {  // evictor.hpp:126-144
            std::set<int>& left = holders_[mod];
            left.erase(gpu);
            if (level(mod) >= LEVEL_MEDIAN && left.size() == 1) {
                Gpu& og = gpus_[(size_t)*left.begin()];
                auto oe = og.entries.find(mod);
                if (oe != og.entries.end() && !oe->second.prot) restamp(og, oe->second, true, mod);
            }
        }
        return victims;
    }

    // evictor.hpp:149-170 ; the surviving copy of a model is not re-classified here, as in the reference
    bool force_evict(int gpu, const std::string& func) {
        if (!ok(gpu)) return false;
        Gpu& g = gpus_[(size_t)gpu];
        bool tracked = false;
        auto e = g.entries.find(func);
        if (e != g.entries.end()) {
            g.used -= e->second.size;
            g.order[e->second.prot ? 1 : 0].erase(e->second.stamp);
            g.entries.erase(e);
            tracked = true;
        }
        auto h = holders_.find(func);
        if (h != holders_.end()) h->second.erase(gpu);
        return tracked;
    }

    // Next eviction candidate on `gpu` other than `keep`, in the order check_and_add would take them.
    bool peek_victim(int gpu, const std::string& keep, std::string* out) const {
        if (!ok(gpu)) return false;
        const Gpu& g = gpus_[(size_t)gpu];
        for (int cls = 0; cls < 2; ++cls)
            for (const auto& kv : g.order[cls]) {
                if (kv.second == keep || g.locked.count(kv.second)) continue;
                *out = kv.second;
                return true;
            }
        return false;
    }

    void lock(int gpu, const std::string& func) {  // evictor.hpp:172-174
        if (ok(gpu)) gpus_[(size_t)gpu].locked.insert(func);
    }
    void unlock(int gpu, const std::string& func) {  // evictor.hpp:176-180
        if (ok(gpu)) gpus_[(size_t)gpu].locked.erase(func);
    }
    bool contains(int gpu, const std::string& func) const { return ok(gpu) && gpus_[(size_t)gpu].entries.count(func) != 0; }
    bool is_protected(int gpu, const std::string& func) const {
        if (!ok(gpu)) return false;
        auto e = gpus_[(size_t)gpu].entries.find(func);
        return e != gpus_[(size_t)gpu].entries.end() && e->second.prot;
    }
    // Eviction order on one GPU, first victim first.
    std::vector<std::string> order(int gpu) const {
        std::vector<std::string> v;
        if (!ok(gpu)) return v;
        for (int cls = 0; cls < 2; ++cls)
            for (const auto& kv : gpus_[(size_t)gpu].order[cls]) v.push_back(kv.second);
        return v;
    }

private:
    struct Entry {
        uint64_t stamp = 0;
        uint64_t size = 0;
        bool prot = false;
    };
    struct Gpu {
        std::unordered_map<std::string, Entry> entries;
        std::map<uint64_t, std::string> order[2];  // [0] unprotected, [1] protected; smallest stamp = least recent
        std::set<std::string> locked;
        uint64_t used = 0;
    };
    bool ok(int gpu) const { return gpu >= 0 && (size_t)gpu < gpus_.size(); }
    void restamp(Gpu& g, Entry& e, bool prot, const std::string& name) {
        g.order[e.prot ? 1 : 0].erase(e.stamp);
        e.prot = prot;
        e.stamp = ++clock_;
        g.order[prot ? 1 : 0][e.stamp] = name;
    }

    uint64_t budget_;
    uint64_t clock_ = 0;
    std::vector<Gpu> gpus_;
    std::map<std::string, std::set<int>> holders_;  // function -> GPUs that hold it
    std::unordered_map<std::string, int> level_;
};

}  // namespace tp
