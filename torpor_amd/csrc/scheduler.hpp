// Placement and scheduling decisions of the controller for a node with several GPUs.
//
// Pure decision logic, no device calls: which GPU runs a request and where its
// weights come from, given which executors are idle and which GPUs hold the
// model.  Restates include/server/controller.hpp:271-389.  On one GPU every
// decision degenerates to "GPU 0 if idle"; the engine's own request queue
// (controller.hpp:218-263) covers that case, so this object is used by tests
// and by a multi-GPU controller, not by the single-GPU engine.
//
// Topology: the reference hard-codes a 4-GPU machine (PCIe switch pairs
// {1,0,3,2} and an NVLink table with 1 = slow and 2 = fast links,
// controller.hpp:117-118).  Here both tables are inputs; the default is an
// MI355X node: eight GPUs, every pair joined by one xGMI link (all fast), and
// host-link siblings paired (0,1) (2,3) (4,5) (6,7).
#pragma once
#include <cstdint>
#include <cstdlib>
#include <map>
#include <set>
#include <string>
#include <vector>

namespace tp {

// controller.hpp:18-24
enum ExecStatus : int {
    XS_AVAIL = -1,
    XS_RUN_LOCAL = 0,
    XS_RUN_PEER = 1,
    XS_RUN_HOST_LIGHT = 2,
    XS_RUN_HOST_MEDIAN = 3,
    XS_RUN_HOST_HEAVY = 4,
    XS_RUN_COLD_START = 5,
};

// controller.hpp:26-32
inline int level_to_exec_status(int level) { return (level >= 0 && level <= 2) ? level + XS_RUN_HOST_LIGHT : XS_RUN_HOST_MEDIAN; }

struct ScheduleDecision {  // controller.hpp:40-44
    int dst_gpu = -1;
    int src_gpu = -1;  // >= 0: swap from that GPU over a peer link
    int status = -1;
};

class Scheduler {
public:
    explicit Scheduler(int gpu_count = 8) { reset(gpu_count); }

    void reset(int gpu_count) {
        n_ = gpu_count > 0 ? gpu_count : 1;
        status_.assign((size_t)n_, XS_AVAIL);
        sibling_.resize((size_t)n_);
        for (int i = 0; i < n_; ++i) sibling_[(size_t)i] = (i ^ 1) < n_ ? (i ^ 1) : i;
        link_.assign((size_t)n_ * (size_t)n_, 2);
        for (int i = 0; i < n_; ++i) link_[(size_t)i * (size_t)n_ + (size_t)i] = 0;
        holders_.clear();
        level_.clear();
        rr_ = 0;
    }
    int gpu_count() const { return n_; }

    bool set_sibling(int gpu, int other) {
        if (!ok(gpu) || !ok(other)) return false;
        sibling_[(size_t)gpu] = other;
        return true;
    }
    // -1: host link only; 0: self; 1: slow peer link; 2: fast peer link
    bool set_link(int a, int b, int kind) {
        if (!ok(a) || !ok(b)) return false;
        link_[(size_t)a * (size_t)n_ + (size_t)b] = kind;
        return true;
    }
    bool set_status(int gpu, int status) {
        if (!ok(gpu)) return false;
        status_[(size_t)gpu] = status;
        return true;
    }
    int status(int gpu) const { return ok(gpu) ? status_[(size_t)gpu] : (int)XS_AVAIL; }
    void set_level(const std::string& func, int level) { level_[func] = level; }
    // model_repo.hpp's model_active_device_map_: the GPUs on which the model is resident
    void set_resident(const std::string& func, int gpu, bool resident) {
        if (!ok(gpu)) return;
        if (resident) holders_[func].insert(gpu);
        else {
            auto it = holders_.find(func);
            if (it != holders_.end()) it->second.erase(gpu);
        }
    }

    // controller.hpp:271-294: round-robin over idle executors, else the first idle one, else -1
    int placement() {
        if (status_[(size_t)rr_] == XS_AVAIL) {
            const int g = rr_;
            rr_ = (rr_ + 1) % n_;
            return g;
        }
        for (int i = 0; i < n_; ++i)
            if (status_[(size_t)i] == XS_AVAIL) return i;
        return -1;
    }

    // controller.hpp:296-319.  `pick` chooses among the idle GPUs when the model is resident on no
    // idle one (the reference calls rand()); it receives the count and returns an index below it.
    template <class Pick>
    ScheduleDecision random_schedule(const std::string& func, Pick pick) const {
        const std::vector<int> idle = idle_gpus();
        if (idle.empty()) return {};
        if (const std::set<int>* h = holders(func))
            for (int g : *h)
                if (status_[(size_t)g] == XS_AVAIL) return {g, -1, XS_RUN_LOCAL};
        const int g = idle[(size_t)pick((int)idle.size()) % idle.size()];
        return {g, -1, level_to_exec_status(level(func))};
    }
    ScheduleDecision random_schedule(const std::string& func) const {
        return random_schedule(func, [](int n) { return std::rand() % n; });
    }

    // controller.hpp:321-389
    ScheduleDecision interference_aware_schedule(const std::string& func) const {
        const std::vector<int> idle = idle_gpus();
        if (idle.empty()) return {};
        const std::set<int>* h = holders(func);
        if (h && !h->empty()) {
            for (int g : *h)
                if (status_[(size_t)g] == XS_AVAIL) return {g, -1, XS_RUN_LOCAL};  // resident and idle: no swap
            // Resident only on busy GPUs: copy from one of them over a peer link.  As in the reference
            // the pair taken is the one found for the LAST idle GPU that has a fast link to a holder
            // (its inner loop stops at the first such holder, the outer loop keeps going); without any
            // fast link it is (first idle GPU, lowest-numbered holder).
            int dst = idle[0], src = *h->begin();
            for (int i : idle)
                for (int j : *h)
                    if (link_[(size_t)i * (size_t)n_ + (size_t)j] == 2) {
                        dst = i;
                        src = j;
                        break;
                    }
            return {dst, src, XS_RUN_PEER};
        }
        // Not resident anywhere: swap from host memory on the idle GPU whose host-link sibling is least
        // busy (statuses are ordered by how hard they use the link; idle = -1 is best).
        int best = idle[0], best_status = status_[(size_t)sibling_[(size_t)idle[0]]];
        for (int g : idle) {
            const int s = status_[(size_t)sibling_[(size_t)g]];
            if (s < best_status) {
                best_status = s;
                best = g;
            }
        }
        return {best, -1, level_to_exec_status(level(func))};
    }

private:
    bool ok(int g) const { return g >= 0 && g < n_; }
    std::vector<int> idle_gpus() const {
        std::vector<int> v;
        for (int i = 0; i < n_; ++i)
            if (status_[(size_t)i] == XS_AVAIL) v.push_back(i);
        return v;
    }
    const std::set<int>* holders(const std::string& func) const {
        auto it = holders_.find(func);
        return it == holders_.end() ? nullptr : &it->second;
    }
    int level(const std::string& func) const {
        auto it = level_.find(func);
        return it == level_.end() ? 0 : it->second;
    }

    int n_ = 1;
    int rr_ = 0;
    std::vector<int> status_, sibling_, link_;
    std::map<std::string, std::set<int>> holders_;
    std::map<std::string, int> level_;
};

}  // namespace tp
