// Shared by the engine's translation units (engine.cpp: set-up, memory ops, introspection;
// engine_swap.cpp: weight image, transfer format, swap-in / swap-out; engine_request.cpp: the controller's
// signal loop; engine_exec.cpp: compute ops, recording and replay).  Not part of the C-ABI.
#pragma once
#include "engine.hpp"
#include "weight_pack.hpp"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "kernels/kernels.hpp"

namespace tp {

using Clock = std::chrono::steady_clock;
inline double us_since(Clock::time_point t0) {
    return std::chrono::duration<double, std::micro>(Clock::now() - t0).count();
}
inline uint64_t align_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

#define HIPCHK(expr)                         \
    do {                                     \
        hipError_t _e = (expr);              \
        if (_e != hipSuccess) return (int)_e; \
    } while (0)

inline uint64_t env_u64(const char* name, uint64_t dflt) {
    const char* v = std::getenv(name);
    if (!v || !*v) return dflt;
    char* end = nullptr;
    unsigned long long x = std::strtoull(v, &end, 10);
    if (end == v) return dflt;
    return (uint64_t)x;
}

// Algorithmic work of one op (engine_exec.cpp).
void op_work(const Op& op, double* flops, double* bytes, const char** name);

// Runs f(0) .. f(n-1) on up to TORPOR_HOST_THREADS (default 8) threads, the caller's included; tasks are
// handed out one at a time.  Returns false if a task threw (the others still ran).
template <class F>
bool parallel_for(size_t n, F&& f) {
    static const size_t cap = [] {
        const uint64_t hw = std::thread::hardware_concurrency();
        const uint64_t want = env_u64("TORPOR_HOST_THREADS", 8);
        return (size_t)std::max<uint64_t>(1, std::min<uint64_t>(want, hw ? hw : 1));
    }();
    std::atomic<size_t> next{0};
    std::atomic<bool> ok{true};
    auto work = [&] {
        for (;;) {
            const size_t i = next.fetch_add(1);
            if (i >= n) return;
            try {
                f(i);
            } catch (...) {
                ok.store(false);
            }
        }
    };
    std::vector<std::thread> helpers;
    const size_t want = std::min(cap, n);
    try {
        helpers.reserve(want);
        for (size_t t = 1; t < want; ++t) helpers.emplace_back(work);
    } catch (...) {  // no more threads to be had: go on with those that started
    }
    work();
    for (auto& t : helpers) t.join();
    return ok.load();
}

}  // namespace tp
