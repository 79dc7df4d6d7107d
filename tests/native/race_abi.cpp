// Three threads on one host-only engine through the C-ABI, for ThreadSanitizer: a controller issuing
// signals, an executor issuing data-plane calls for whichever function is active, and an observer
// reading statistics.  The reference shares its controller / executor / repository state between
// threads without synchronisation (model_repo.hpp:180-185, memory_manager.hpp:494-495,529); here
// every entry point must be safe to call from any thread.  Return codes are not the subject (most
// calls are refused: wrong client, wrong mode); what is checked is that nothing races and that the
// pool and the evictor stay consistent.  CPU only.
#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <random>
#include <string>
#include <thread>
#include <vector>

#include "../../include/torpor_amd.h"

namespace {

std::atomic<bool> stop{false};
std::atomic<long> n_signals{0}, n_ops{0}, n_reads{0};
std::atomic<int> failures{0};
constexpr int kFuncs = 6;

void controller(tp_server* s) {
    std::mt19937 rng(1);
    while (!stop.load()) {
        const int id = (int)(rng() % kFuncs);
        const std::string fn = std::to_string(id);
        int32_t ack = 0, resp = 0, dfr = 0;
        switch (rng() % 8) {
            case 0: (void)tp_signal(s, TP_REQ_EXECUTE_AFTER_LOAD, fn.c_str(), "1", &ack, &resp, &dfr); break;
            case 1: case 2: case 3: (void)tp_signal(s, TP_REQ_EXECUTE, fn.c_str(), "", &ack, &resp, &dfr); break;
            case 4: case 5: (void)tp_signal(s, TP_REQ_LOAD, fn.c_str(), "", &ack, &resp, &dfr); break;
            default: (void)tp_signal(s, TP_REQ_UNLOAD, fn.c_str(), "", &ack, &resp, &dfr); break;
        }
        while (tp_take_deferred_ack(s, &ack, &resp) == 1) {
        }
        (void)tp_poll(s);
        n_signals.fetch_add(1);
    }
}

void executor(tp_server* s) {
    std::mt19937 rng(2);
    std::vector<float> host(4096, 1.0f), out(4096);
    uint64_t va[kFuncs] = {0};
    while (!stop.load()) {
        const int id = (int)(rng() % kFuncs);
        switch (rng() % 8) {
            case 0: {  // registration steps: allocate + upload a weight, end the loading phase
                uint64_t w = 0;
                if (tp_malloc(s, id, 16384, &w) == 0) {
                    (void)tp_memcpy_h2d(s, id, w, host.data(), 16384);
                    va[id] = w;
                }
                (void)tp_device_synchronize(s, id);
                break;
            }
            case 1: {
                uint64_t a = 0;
                if (tp_malloc(s, id, 16384, &a) == 0) {
                    const uint64_t p[2] = {va[id] ? va[id] : a, a};
                    const int64_t n[1] = {4096};
                    (void)tp_launch(s, id, TP_OP_RELU, p, 2, n, 1, nullptr, 0);
                    (void)tp_memcpy_d2h_async(s, id, out.data(), a, 16384);  // ends the request
                }
                break;
            }
            case 2: (void)tp_stream_synchronize(s, id); break;
            case 3: (void)tp_replay(s, id, host.data(), 16384, out.data(), 16384); break;
            case 4: (void)tp_memset_async(s, id, va[id], 0, 64); break;
            case 5: (void)tp_memcpy_d2h(s, id, out.data(), va[id], 64); break;
            case 6: (void)tp_free(s, id, va[id]); break;
            default: (void)tp_memcpy_d2d(s, id, va[id], va[id], 64); break;
        }
        n_ops.fetch_add(1);
    }
}

void observer(tp_server* s) {
    std::mt19937 rng(3);
    while (!stop.load()) {
        tp_pool_stats ps;
        std::memset(&ps, 0, sizeof ps);
        if (tp_get_pool_stats(s, &ps) == 0 && ps.used > ps.capacity) failures.fetch_add(1);
        const int id = (int)(rng() % kFuncs);
        tp_model_info mi;
        (void)tp_get_model_info(s, id, &mi);
        (void)tp_model_resident(s, id);
        tp_swap_stats ss;
        (void)tp_get_swap_stats(s, id, &ss);
        const void* p = nullptr;
        uint64_t n = 0;
        (void)tp_host_weights(s, id, &p, &n);
        n_reads.fetch_add(1);
    }
}

}  // namespace

int main() {
    tp_config cfg;
    std::memset(&cfg, 0, sizeof cfg);
    cfg.struct_size = sizeof cfg;
    cfg.flags = TP_FLAG_HOST_ONLY;
    cfg.mem_limit_bytes = 1ull << 20;  // a few models fit: evictions all the time
    cfg.pool_bytes = 4ull << 20;
    cfg.request_timeout_ms = 2;        // abandoned requests time out quickly, so the state machine keeps moving
    tp_server* s = nullptr;
    if (tp_server_create(&cfg, &s) != 0) return 2;
    std::thread a(controller, s), b(executor, s), c(observer, s);
    std::this_thread::sleep_for(std::chrono::milliseconds(1500));
    stop.store(true);
    a.join();
    b.join();
    c.join();
    tp_pool_stats ps;
    std::memset(&ps, 0, sizeof ps);
    const int r = tp_get_pool_stats(s, &ps);
    tp_server_destroy(s);
    if (r != 0 || ps.used > ps.capacity || failures.load()) return 3;
    if (ps.swap_ins == 0 || ps.evictions == 0) return 4;  // the run never got past registration: it tested nothing
    std::printf("race ok: %ld signals, %ld data-plane calls, %ld reads, %llu swap-ins, %llu evictions\n", n_signals.load(),
                n_ops.load(), n_reads.load(), (unsigned long long)ps.swap_ins, (unsigned long long)ps.evictions);
    return 0;
}
