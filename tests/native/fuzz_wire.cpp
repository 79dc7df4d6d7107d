// Host-side robustness check, built with AddressSanitizer + UndefinedBehaviorSanitizer on the host pass
// (tests/test_sanitize_host.py): the wire front end's message handlers are fed (a) well-formed
// request sequences, (b) the same bytes with random mutations, (c) random bytes, against an engine
// created with TP_FLAG_HOST_ONLY (no device is touched).  Nothing may crash, leak or trip a
// sanitizer; malformed input must come back as error codes.
#include <sys/socket.h>

#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <random>
#include <string>

#define main torpor_server_main   // the front end's handlers live in an anonymous namespace of its one file
#include "../../torpor_amd/csrc/wire/server_main.cpp"
#undef main

namespace {

std::string query(int type, const std::string& body, int client) {
    pb::Writer q;
    q.i32(1, type);
    q.message(2, body);
    q.i32(3, client);
    pb::Writer l;
    l.message(1, q.out);
    return l.out;
}
std::string signal_msg(int type, const char* fn, const char* payload) {
    pb::Writer w;
    w.i32(1, type);
    w.str(2, fn);
    w.str(3, payload);
    return w.out;
}

}  // namespace

int main() {
    tp_config cfg;
    std::memset(&cfg, 0, sizeof cfg);
    cfg.struct_size = sizeof cfg;
    cfg.flags = TP_FLAG_HOST_ONLY;
    cfg.mem_limit_bytes = 64ull << 20;
    cfg.pool_bytes = 96ull << 20;
    Server S;
    if (tp_server_create(&cfg, &S.eng) != 0) {
        std::fprintf(stderr, "tp_server_create failed\n");
        return 2;
    }
    std::mt19937_64 rng(12345);
    std::vector<std::string> corpus;

    // a well-formed registration: ExecuteAfterLoad, malloc, upload, device synchronise
    bool dfr = false;
    corpus.push_back(signal_msg(TP_REQ_EXECUTE_AFTER_LOAD, "3", "1"));
    uint64_t ticket = 0;
    (void)handle_signal(S, corpus.back(), &dfr, &ticket);
    {
        pb::Writer m;
        m.u64(1, 4096);
        corpus.push_back(query(Q_MALLOC, m.out, 3));
        pb::Writer c;  // a convolution descriptor with every field present
        c.u64(4, 1);
        c.u64(6, 2);
        c.u64(13, 3);
        for (int f = 20; f <= 33; ++f) c.i32(f, 3);
        c.u64(35, 8);
        c.u64(36, 8);
        corpus.push_back(query(Q_CONV, c.out, 3));
        pb::Writer l;
        l.i32(20, TP_OP_LAYERNORM);
        corpus.push_back(query(Q_LAUNCH, l.out, 3));
        pb::Writer g;
        for (int f = 1; f <= 20; ++f) g.u64(f, 1 + f);
        corpus.push_back(query(Q_GEMM, g.out, 3));
        corpus.push_back(query(Q_SGEMM, g.out, 3));
        corpus.push_back(query(Q_SGEMM_BATCHED, g.out, 3));
        corpus.push_back(query(Q_BN, g.out, 3));
        corpus.push_back(query(Q_MEMCPY, g.out, 3));
        corpus.push_back(query(Q_MEMCPY_ASYNC, g.out, 3));
        corpus.push_back(query(Q_MEMSET_ASYNC, g.out, 3));
        corpus.push_back(query(Q_REPLAY, g.out, 3));
        corpus.push_back(query(Q_FREE, g.out, 3));
        corpus.push_back(query(Q_STREAM_SYNC, "", 3));
        corpus.push_back(query(Q_DEVICE_SYNC, "", 3));
    }
    for (const auto& m : corpus) handle_query_list(S, m);
    {
        // device-to-host copies whose count the engine cannot vouch for (4 GiB, 2^64 - 1, a source that is
        // no address) must be refused before the front end sets that much memory aside
        const uint64_t counts[3] = {1ull << 32, ~0ull, 1ull << 31};
        for (uint64_t cnt : counts)
            for (int qt : {(int)Q_MEMCPY, (int)Q_MEMCPY_ASYNC}) {
                pb::Writer c;
                c.u64(1, KIND_D2H);
                c.u64(2, 0x1234);
                c.u64(3, 0x5678);
                c.u64(4, cnt);
                handle_query_list(S, query(qt, c.out, 3));
            }
        if (!S.staged[3].empty()) return 20;
    }
    {
        // A peer that never reads: the writer gives up after its time budget (TORPOR_SEND_TIMEOUT_MS) and
        // marks the connection failed instead of blocking the only server thread for ever.
        setenv("TORPOR_SEND_TIMEOUT_MS", "200", 1);
        int sv[2];
        if (::socketpair(AF_UNIX, SOCK_STREAM, 0, sv) != 0) return 21;
        int small = 4096;
        (void)::setsockopt(sv[0], SOL_SOCKET, SO_SNDBUF, &small, sizeof small);
        zmtp::Conn c(sv[0], zmtp::PUSH);
        const auto t0 = std::chrono::steady_clock::now();
        const bool sent = c.send({std::string(8u << 20, 'x')});
        const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        ::close(sv[1]);
        if (sent || !c.failed() || ms > 5000.0) return 22;
        // and a frame header that announces more than any legitimate message is refused at once
        int sv2[2];
        if (::socketpair(AF_UNIX, SOCK_STREAM, 0, sv2) != 0) return 23;
        zmtp::Conn d(sv2[0], zmtp::PULL);
        std::string hello = zmtp::greeting() + zmtp::ready_command(zmtp::PUSH);
        hello.push_back(2);  // long frame
        for (int sh = 56; sh >= 0; sh -= 8) hello.push_back((char)((zmtp::kMaxFrame + 1) >> sh));
        if (::send(sv2[1], hello.data(), hello.size(), 0) != (ssize_t)hello.size()) return 24;
        (void)d.pump();
        ::close(sv2[1]);
        if (!d.failed()) return 25;
    }

    long handled = 0;
    for (int it = 0; it < 20000; ++it) {
        std::string m;
        const int mode = (int)(rng() % 3);
        if (mode == 0) {
            m.resize(rng() % 96);
            for (auto& ch : m) ch = (char)rng();
        } else {
            m = corpus[rng() % corpus.size()];
            const int flips = 1 + (int)(rng() % 4);
            for (int k = 0; k < flips && !m.empty(); ++k) {
                const size_t pos = rng() % m.size();
                if (mode == 1)
                    m[pos] = (char)rng();
                else
                    m.erase(pos, 1 + rng() % 3);
            }
        }
        if (rng() % 5 == 0) {
            bool d = false;
            uint64_t tk = 0;
            (void)handle_signal(S, m, &d, &tk);
            if (d && rng() % 2) (void)tp_cancel_deferred(S.eng, tk);  // the peer went away while queued
            if (rng() % 16 == 0) (void)tp_cancel_deferred(S.eng, rng() % 64);
        } else {
            handle_query_list(S, m);
        }
        int32_t ack, resp;
        uint64_t tk2 = 0;
        while ((rng() % 2 ? tp_take_deferred_ack(S.eng, &ack, &resp) : tp_take_deferred_ack_ticket(S.eng, &ack, &resp, &tk2)) == 1) {
        }
        (void)tp_poll(S.eng);
        ++handled;
    }
    tp_server_destroy(S.eng);

    // the slab pool and the LRU evictor through their stand-alone handles: random alloc / release and
    // add / lock / evict sequences, including stale offsets and unknown names
    tp_pool* pool = tp_pool_create(64ull << 20);
    std::vector<uint64_t> live;
    for (int it = 0; it < 20000; ++it) {
        const int op = (int)(rng() % 4);
        if (op < 2) {
            const uint64_t off = tp_pool_alloc(pool, 1 + rng() % (6ull << 20));
            if (off != UINT64_MAX) live.push_back(off);
        } else if (op == 2 && !live.empty()) {
            const size_t k = rng() % live.size();
            if (tp_pool_release(pool, live[k]) != 0) return 3;
            live.erase(live.begin() + (long)k);
        } else {
            (void)tp_pool_release(pool, rng() % (64ull << 20));   // mostly not a live extent: must be refused
            live.clear();                                          // (a hit frees one of ours; stop tracking)
            tp_pool_destroy(pool);
            pool = tp_pool_create(64ull << 20);
        }
    }
    tp_pool_destroy(pool);
    tp_lru* lru = tp_lru_create(1000);
    char victims[256];
    for (int it = 0; it < 20000; ++it) {
        char name[8];
        std::snprintf(name, sizeof name, "%d", (int)(rng() % 24));
        int32_t nv = 0, over = 0;
        switch (rng() % 5) {
            case 0: case 1: (void)tp_lru_check_and_add(lru, name, 1 + rng() % 400, victims, sizeof victims, &nv, &over); break;
            case 2: (void)tp_lru_lock(lru, name); break;
            case 3: (void)tp_lru_unlock(lru, name); break;
            default: (void)tp_lru_force_evict(lru, name); break;
        }
    }
    tp_lru_destroy(lru);

    // the multi-GPU policy objects: random traces with out-of-range GPUs and unknown names mixed in
    for (int policy = 0; policy < 2; ++policy) {
        tp_evictor* ev = tp_evictor_create(policy, 4, 1000);
        if (!ev) return 4;
        for (int it = 0; it < 20000; ++it) {
            char name[8];
            std::snprintf(name, sizeof name, "%d", (int)(rng() % 24));
            const int gpu = (int)(rng() % 6) - 1;   // -1 and 4 are invalid
            int32_t nv = 0, over = 0;
            switch (rng() % 8) {
                case 0: case 1: case 2:
                    (void)tp_evictor_check_and_add(ev, gpu, name, 1 + rng() % 400, victims, sizeof victims, &nv, &over);
                    break;
                case 3: (void)tp_evictor_lock(ev, gpu, name); break;
                case 4: (void)tp_evictor_unlock(ev, gpu, name); break;
                case 5: (void)tp_evictor_force_evict(ev, gpu, name); break;
                case 6: (void)tp_evictor_set_level(ev, name, (int32_t)(rng() % 5) - 1); break;
                default: (void)tp_evictor_order(ev, gpu, victims, 1 + rng() % sizeof victims); (void)tp_evictor_is_protected(ev, gpu, name); break;
            }
            uint64_t sum = 0;
            for (int g = 0; g < 4; ++g) sum += tp_evictor_used(ev, g);
            if (sum > 4ull * 24 * 400) return 5;
        }
        tp_evictor_destroy(ev);
    }
    tp_sched* sc = tp_sched_create(8);
    if (!sc) return 6;
    for (int it = 0; it < 20000; ++it) {
        char name[8];
        std::snprintf(name, sizeof name, "%d", (int)(rng() % 12));
        const int gpu = (int)(rng() % 10) - 1;
        int32_t d = 0, sr = 0, st = 0;
        switch (rng() % 7) {
            case 0: (void)tp_sched_set_status(sc, gpu, (int32_t)(rng() % 9) - 2); break;
            case 1: (void)tp_sched_set_resident(sc, name, gpu, (int32_t)(rng() % 2)); break;
            case 2: (void)tp_sched_set_level(sc, name, (int32_t)(rng() % 5) - 1); break;
            case 3: (void)tp_sched_set_sibling(sc, gpu, (int32_t)(rng() % 10) - 1); break;
            case 4: (void)tp_sched_set_link(sc, gpu, (int32_t)(rng() % 10) - 1, (int32_t)(rng() % 6) - 2); break;
            case 5: { const int g = tp_sched_placement(sc); if (g < -1 || g > 7) return 7; break; }
            default:
                if (tp_sched_decide(sc, (int32_t)(rng() % 2), name, (uint32_t)rng(), &d, &sr, &st) != 0) return 8;
                if (d < -1 || d > 7 || sr < -1 || sr > 7) return 9;
                break;
        }
    }
    tp_sched_destroy(sc);

    // the packed transfer format: exactly sized buffers, every length, weight-like and arbitrary words
    for (int it = 0; it < 3000; ++it) {
        const uint64_t n = it < 2990 ? rng() % 300 : 2040 + rng() % 4200;
        std::vector<uint32_t> w(n), back(n, 0xDEADBEEFu), tab((size_t)tp_pack_blocks(n));
        const int kind = (int)(rng() % 3);
        for (auto& v : w)
            v = kind == 0 ? (uint32_t)rng()
                          : (uint32_t)(((rng() % 2) << 31) | ((uint64_t)(120 + rng() % (kind == 1 ? 6 : 40)) << 23) | (rng() & 0x7FFFFF));
        std::vector<uint8_t> payload((size_t)tp_pack_bound(n)), ext(n);
        int32_t base = -1;
        uint64_t ne = 0;
        uint8_t dummy = 0;
        uint32_t dummy32 = 0;
        if (tp_pack_words(w.data(), n, payload.empty() ? &dummy : payload.data(), &base, ext.data(), n, &ne,
                          tab.empty() ? &dummy32 : tab.data()) != 0)
            return 10;
        if (tp_unpack_words(payload.empty() ? &dummy : payload.data(), n, base, ext.data(), ne, back.data()) != 0) return 11;
        if (w != back) return 12;
        if (ne && tp_unpack_words(payload.data(), n, base, ext.data(), ne - 1, back.data()) == 0) return 13;  // short stream
    }
    std::printf("fuzz ok: %ld messages\n", handled);
    return 0;
}
