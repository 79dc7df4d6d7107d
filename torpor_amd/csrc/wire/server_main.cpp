// torpor_server: the request-flow front end of the engine.
//
// Binds the reference's endpoints (common/include/socket_helper.hpp:10-20; the directory
// defaults to /cuda and can be moved with TORPOR_IPC_DIR):
//   REP  ipc://<dir>/signal_0   one SignalRequest -> one SignalAck   (controller.hpp:77,131-216)
//   PULL ipc://<dir>/server_0   QueryList of WapperQuery             (cuda_server.hpp:53,199-209)
// and connects a PUSH to ipc://<dir>/client_<id> for the reply of every synchronous query
// (cuda_server.hpp:1314-1318).  Everything below the sockets goes through the C-ABI of
// include/torpor_amd.h and nothing else, i.e. this file is what a maintainer of the reference
// would write to put its wire layer on top of this engine.
//
// The reference spins two threads at 100 % CPU on poll(0) (controller.hpp:129,
// cuda_server.hpp:121); here one thread sleeps in poll(2) on all sockets.
#include <signal.h>

#include <cstdio>
#include <cstdlib>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "../../../include/torpor_amd.h"
#include "proto.hpp"
#include "zmtp.hpp"

namespace {

volatile sig_atomic_t g_stop = 0;
void on_signal(int) { g_stop = 1; }

enum QueryType : int {
    Q_DEVICE_SYNC = 14,
    Q_STREAM_SYNC = 23,
    Q_MALLOC = 30,
    Q_FREE = 31,
    Q_MEMCPY = 32,
    Q_MEMCPY_ASYNC = 33,
    Q_MEMSET_ASYNC = 34,
    Q_LAUNCH = 50,
    Q_SGEMM = 104,
    Q_SGEMM_BATCHED = 105,
    Q_CONV = 211,
    Q_BN = 212,
    Q_GEMM = 300,
    Q_REPLAY = 301,
};
enum { KIND_H2D = 1, KIND_D2H = 2, KIND_D2D = 3 };  // cudaMemcpyKind values

struct StagedD2H {
    uint64_t client_ptr;
    std::vector<uint8_t> data;
};

struct Server {
    tp_server* eng = nullptr;
    std::string dir;
    int sig_listen = -1, srv_listen = -1;
    std::vector<std::unique_ptr<zmtp::Conn>> rep_conns, pull_conns;
    std::map<int, std::unique_ptr<zmtp::Conn>> pushers;  // client id -> PUSH connection
    std::map<int, std::vector<StagedD2H>> staged;        // client id -> D2H copies awaiting the next sync
    // REP peers whose signal was queued, by the engine's ticket for it.  Acks are matched to peers by
    // ticket and peers are named by a tag that is never reused (a freed Conn's address can be).
    struct Waiting {
        uint64_t ticket, conn_tag;
    };
    std::vector<Waiting> waiting_ack;
    uint64_t next_tag = 1;
    bool verbose = false;
    // Replay results are received in pinned memory of the engine (tp_host_alloc): the device writes
    // them there itself, and the reply message is built from it.  Grown on demand, freed with the engine.
    uint8_t* reply_buf = nullptr;
    uint64_t reply_cap = 0;
    uint8_t* reply_room(uint64_t bytes) {
        if (bytes <= reply_cap) return reply_buf;
        if (reply_buf) (void)tp_host_free(eng, reply_buf);
        reply_buf = nullptr;
        reply_cap = 0;
        void* p = nullptr;
        uint64_t cap = 1ull << 20;
        while (cap < bytes) cap *= 2;
        if (tp_host_alloc(eng, cap, &p) != 0) return nullptr;
        reply_buf = static_cast<uint8_t*>(p);
        reply_cap = cap;
        return reply_buf;
    }
};

std::string generic_response(int err) {
    pb::Writer w;
    w.i32(1, err);
    return w.out;
}

void parse_epilogue(const pb::View& v, tp_epilogue* e) {
    pb::Reader r(v);
    int f, wt;
    while (r.next(&f, &wt)) {
        uint64_t u = 0;
        switch (f) {
            case 1: if (wt == pb::WT_FIXED32) e->alpha = r.f32(); else r.skip(wt); break;
            case 2: if (wt == pb::WT_FIXED32) e->beta = r.f32(); else r.skip(wt); break;
            case 3: if (r.read_u64(wt, &u)) e->bias = u; break;
            case 4: if (r.read_u64(wt, &u)) e->bn_scale = u; break;
            case 5: if (r.read_u64(wt, &u)) e->bn_bias = u; break;
            case 6: if (r.read_u64(wt, &u)) e->bn_mean = u; break;
            case 7: if (r.read_u64(wt, &u)) e->bn_var = u; break;
            case 8: if (wt == pb::WT_FIXED32) e->bn_eps = r.f32(); else r.skip(wt); break;
            case 9: if (r.read_u64(wt, &u)) e->act = (int32_t)u; break;
            case 10: if (r.read_u64(wt, &u)) e->residual = u; break;
            case 11: if (r.read_u64(wt, &u)) e->ldr = (int64_t)u; break;
            default: r.skip(wt);
        }
    }
}

// Runs one query; returns true and fills `reply` when the query type is synchronous.
bool handle_query(Server& S, int type, const pb::View& q, int client, std::string* reply) {
    pb::Reader r(q);
    int f, wt;
    uint64_t u = 0;
    switch (type) {
        case Q_MALLOC: {
            uint64_t size = 0, ptr = 0;
            while (r.next(&f, &wt)) {
                if (f == 1 && r.read_u64(wt, &u)) size = u;
                else if (f != 1) r.skip(wt);
            }
            const int err = tp_malloc(S.eng, client, size, &ptr);
            pb::Writer w;
            w.i32(1, err);
            w.u64(2, ptr);
            *reply = w.out;
            return true;
        }
        case Q_FREE: {
            uint64_t ptr = 0;
            while (r.next(&f, &wt)) {
                if (f == 1 && r.read_u64(wt, &u)) ptr = u;
                else if (f != 1) r.skip(wt);
            }
            *reply = generic_response(tp_free(S.eng, client, ptr));
            return true;
        }
        case Q_MEMCPY:
        case Q_MEMCPY_ASYNC: {
            int kind = 0;
            uint64_t src = 0, dst = 0, count = 0;
            pb::View payload;
            while (r.next(&f, &wt)) {
                switch (f) {
                    case 1: if (r.read_u64(wt, &u)) kind = (int)u; break;
                    case 2: if (r.read_u64(wt, &u)) src = u; break;
                    case 3: if (r.read_u64(wt, &u)) dst = u; break;
                    case 4: if (r.read_u64(wt, &u)) count = u; break;
                    case 5: if (wt == pb::WT_LEN) payload = r.bytes(); else r.skip(wt); break;
                    default: r.skip(wt);
                }
            }
            int err = 0;
            std::vector<uint8_t> back;
            if (kind == KIND_H2D) {
                err = tp_memcpy_h2d(S.eng, client, dst, payload.p, payload.n);  // cuda_server.hpp:1000-1004,1031-1036
            } else if (kind == KIND_D2D) {
                err = tp_memcpy_d2d(S.eng, client, dst, src, count);
            } else if (kind == KIND_D2H) {
                // the engine vouches for source and count before this process sets `count` bytes aside
                if (count > (1ull << 32)) {
                    err = TP_EINVAL;
                } else if ((err = tp_check_address(S.eng, client, src, count)) != 0) {
                } else if (type == Q_MEMCPY) {
                    back.resize(count);
                    err = tp_memcpy_d2h(S.eng, client, back.data(), src, count);
                } else {
                    // staged; returned by the next StreamSynchronize (cuda_server.hpp:1038-1045,1139-1147)
                    auto& list = S.staged[client];
                    list.push_back({dst, std::vector<uint8_t>(count)});
                    err = tp_memcpy_d2h_async(S.eng, client, list.back().data.data(), src, count);
                    if (err) list.pop_back();
                }
            } else {
                err = TP_EINVAL;
            }
            if (type == Q_MEMCPY) {
                pb::Writer w;
                w.i32(1, err);
                if (!err) w.bytes(2, back.data(), back.size());
                *reply = w.out;
                return true;
            }
            return false;
        }
        case Q_MEMSET_ASYNC: {
            uint64_t ptr = 0, count = 0;
            int value = 0;
            while (r.next(&f, &wt)) {
                switch (f) {
                    case 1: if (r.read_u64(wt, &u)) ptr = u; break;
                    case 2: if (r.read_u64(wt, &u)) value = (int)u; break;
                    case 3: if (r.read_u64(wt, &u)) count = u; break;
                    default: r.skip(wt);
                }
            }
            (void)tp_memset_async(S.eng, client, ptr, value, count);
            return false;
        }
        case Q_SGEMM:
        case Q_SGEMM_BATCHED: {
            int ta = 0, tb = 0, m = 0, n = 0, k = 0, lda = 0, ldb = 0, ldc = 0, count = 1;
            float alpha = 0.f, beta = 0.f;
            uint64_t a = 0, b = 0, c = 0;
            int64_t sa = 0, sb = 0, sc = 0;
            while (r.next(&f, &wt)) {
                switch (f) {
                    case 2: if (r.read_u64(wt, &u)) ta = (int)u; break;
                    case 3: if (r.read_u64(wt, &u)) tb = (int)u; break;
                    case 4: if (r.read_u64(wt, &u)) m = (int)u; break;
                    case 5: if (r.read_u64(wt, &u)) n = (int)u; break;
                    case 6: if (r.read_u64(wt, &u)) k = (int)u; break;
                    case 7: if (wt == pb::WT_FIXED32) alpha = r.f32(); else r.skip(wt); break;
                    case 8: if (r.read_u64(wt, &u)) a = u; break;
                    case 9: if (r.read_u64(wt, &u)) lda = (int)u; break;
                    case 10: if (r.read_u64(wt, &u)) b = u; break;
                    case 11: if (r.read_u64(wt, &u)) ldb = (int)u; break;
                    case 12: if (wt == pb::WT_FIXED32) beta = r.f32(); else r.skip(wt); break;
                    case 13: if (r.read_u64(wt, &u)) c = u; break;
                    case 14: if (r.read_u64(wt, &u)) ldc = (int)u; break;
                    case 15: if (r.read_u64(wt, &u)) sa = (int64_t)u; break;
                    case 16: if (r.read_u64(wt, &u)) sb = (int64_t)u; break;
                    case 17: if (r.read_u64(wt, &u)) sc = (int64_t)u; break;
                    case 18: if (r.read_u64(wt, &u)) count = (int)u; break;
                    default: r.skip(wt);
                }
            }
            // the reference passes cublasOperation_t values: 0 = N, 1 = T
            if (type == Q_SGEMM)
                (void)tp_sgemm(S.eng, client, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
            else
                (void)tp_sgemm_strided_batched(S.eng, client, ta, tb, m, n, k, alpha, a, lda, sa, b, ldb, sb, beta, c,
                                               ldc, sc, count);
            return false;
        }
        case Q_GEMM: {
            tp_gemm_desc d;
            std::memset(&d, 0, sizeof(d));
            d.xs_k = d.ys_k = 1;
            d.nb0 = d.nb1 = 1;
            d.ep.alpha = 1.f;
            while (r.next(&f, &wt)) {
                if (f == 20 && wt == pb::WT_LEN) {
                    parse_epilogue(r.bytes(), &d.ep);
                    continue;
                }
                if (!r.read_u64(wt, &u)) continue;
                switch (f) {
                    case 1: d.x = u; break;
                    case 2: d.y = u; break;
                    case 3: d.c = u; break;
                    case 4: d.m = (int64_t)u; break;
                    case 5: d.n = (int64_t)u; break;
                    case 6: d.k = (int64_t)u; break;
                    case 7: d.xs_r = (int64_t)u; break;
                    case 8: d.xs_k = (int64_t)u; break;
                    case 9: d.ys_c = (int64_t)u; break;
                    case 10: d.ys_k = (int64_t)u; break;
                    case 11: d.ldc = (int64_t)u; break;
                    case 12: d.nb0 = (int32_t)u; break;
                    case 13: d.nb1 = (int32_t)u; break;
                    case 14: d.xb0 = (int64_t)u; break;
                    case 15: d.xb1 = (int64_t)u; break;
                    case 16: d.yb0 = (int64_t)u; break;
                    case 17: d.yb1 = (int64_t)u; break;
                    case 18: d.cb0 = (int64_t)u; break;
                    case 19: d.cb1 = (int64_t)u; break;
                    default: break;
                }
            }
            (void)tp_gemm(S.eng, client, &d);
            return false;
        }
        case Q_CONV: {
            tp_conv_desc d;
            std::memset(&d, 0, sizeof(d));
            d.groups = 1;
            d.ep.alpha = 1.f;
            float alpha = 1.f, beta = 0.f;
            bool has_alpha = false, has_beta = false;
            while (r.next(&f, &wt)) {
                if (f == 2 && wt == pb::WT_FIXED32) { alpha = r.f32(); has_alpha = true; continue; }
                if (f == 11 && wt == pb::WT_FIXED32) { beta = r.f32(); has_beta = true; continue; }
                if (f == 34 && wt == pb::WT_LEN) { parse_epilogue(r.bytes(), &d.ep); continue; }
                if (!r.read_u64(wt, &u)) continue;
                switch (f) {
                    case 4: d.x = u; break;
                    case 6: d.w = u; break;
                    case 13: d.y = u; break;
                    case 20: d.n = (int32_t)u; break;
                    case 21: d.h = (int32_t)u; break;
                    case 22: d.w_in = (int32_t)u; break;
                    case 23: d.cin = (int32_t)u; break;
                    case 24: d.cout = (int32_t)u; break;
                    case 25: d.kh = (int32_t)u; break;
                    case 26: d.kw = (int32_t)u; break;
                    case 27: d.stride_h = (int32_t)u; break;
                    case 28: d.stride_w = (int32_t)u; break;
                    case 29: d.pad_h = (int32_t)u; break;
                    case 30: d.pad_w = (int32_t)u; break;
                    case 31: d.groups = (int32_t)u; break;
                    case 32: d.x_layout = (int32_t)u; break;
                    case 33: d.y_layout = (int32_t)u; break;
                    case 35: d.x_pitch = (int64_t)u; break;
                    case 36: d.y_pitch = (int64_t)u; break;
                    default: break;
                }
            }
            if (has_alpha) d.ep.alpha = alpha;
            if (has_beta) d.ep.beta = beta;
            (void)tp_conv_forward(S.eng, client, &d);
            return false;
        }
        case Q_BN: {
            uint64_t x = 0, y = 0, g = 0, b = 0, mu = 0, var = 0;
            double eps = 0.0;
            int64_t rows = 0, hw = 1, x_pitch = 0;
            int channels = 0, layout = 0, relu = 0;
            while (r.next(&f, &wt)) {
                if (f == 14 && wt == pb::WT_FIXED64) { eps = r.f64(); continue; }
                if (!r.read_u64(wt, &u)) continue;
                switch (f) {
                    case 6: x = u; break;
                    case 8: y = u; break;
                    case 10: g = u; break;
                    case 11: b = u; break;
                    case 12: mu = u; break;
                    case 13: var = u; break;
                    case 20: rows = (int64_t)u; break;
                    case 21: channels = (int)u; break;
                    case 22: hw = (int64_t)u; break;
                    case 23: layout = (int)u; break;
                    case 24: relu = (int)u; break;
                    case 25: x_pitch = (int64_t)u; break;
                    default: break;
                }
            }
            (void)tp_bn_inference_pitched(S.eng, client, x, y, g, b, mu, var, eps, rows, channels, hw, layout, relu,
                                          x_pitch);
            return false;
        }
        case Q_LAUNCH: {
            int op_id = 0;
            std::vector<uint64_t> ptrs, ints_u;
            std::vector<float> floats;
            while (r.next(&f, &wt)) {
                switch (f) {
                    case 20: if (r.read_u64(wt, &u)) op_id = (int)u; break;
                    case 21: r.read_rep_varint(wt, &ptrs); break;
                    case 22: r.read_rep_varint(wt, &ints_u); break;
                    case 23: r.read_rep_f32(wt, &floats); break;
                    default: r.skip(wt);
                }
            }
            std::vector<int64_t> ints(ints_u.begin(), ints_u.end());
            (void)tp_launch(S.eng, client, op_id, ptrs.data(), (int)ptrs.size(), ints.data(), (int)ints.size(),
                            floats.data(), (int)floats.size());
            return false;
        }
        case Q_STREAM_SYNC: {
            const int err = tp_stream_synchronize(S.eng, client);
            pb::Writer w;
            w.i32(1, err);
            auto it = S.staged.find(client);
            if (it != S.staged.end()) {
                for (auto& sd : it->second) {
                    pb::Writer e;
                    e.u64(1, sd.client_ptr);
                    if (!err) e.bytes(2, sd.data.data(), sd.data.size());
                    w.message(2, e.out);
                }
                S.staged.erase(it);
            }
            *reply = w.out;
            return true;
        }
        case Q_DEVICE_SYNC:
            *reply = generic_response(tp_device_synchronize(S.eng, client));
            return true;
        case Q_REPLAY: {  // the whole request in one message: input bytes in, output bytes back
            pb::View payload;
            uint64_t out_bytes = 0;
            while (r.next(&f, &wt)) {
                if (f == 1 && wt == pb::WT_LEN) payload = r.bytes();
                else if (f == 2 && r.read_u64(wt, &u)) out_bytes = u;
                else if (f != 2) r.skip(wt);
            }
            int err = out_bytes > (1ull << 32) ? TP_EINVAL : 0;
            uint8_t* out = nullptr;
            if (!err) {
                out = S.reply_room(out_bytes ? out_bytes : 1);
                err = out ? tp_replay(S.eng, client, payload.p, payload.n, out, out_bytes) : TP_ENOMEM;
            }
            pb::Writer w;
            w.i32(1, err);
            if (!err) w.bytes(2, out, out_bytes);
            *reply = w.out;
            return true;
        }
        default:
            // unknown / unsupported query: synchronous callers still get an answer
            *reply = generic_response(TP_EUNSUPPORTED);
            return true;
    }
}

zmtp::Conn* pusher_for(Server& S, int client) {
    auto it = S.pushers.find(client);
    if (it != S.pushers.end() && !it->second->failed()) return it->second.get();
    const int fd = zmtp::connect_ipc("ipc://" + S.dir + "/client_" + std::to_string(client));
    if (fd < 0) return nullptr;
    auto c = std::make_unique<zmtp::Conn>(fd, zmtp::PUSH);
    for (int i = 0; i < 2000 && !c->ready() && !c->failed(); ++i) {  // wait for the peer's READY
        struct pollfd p = {c->fd(), POLLIN, 0};
        ::poll(&p, 1, 1);
        c->pump();
    }
    if (!c->ready()) return nullptr;
    zmtp::Conn* raw = c.get();
    S.pushers[client] = std::move(c);
    return raw;
}

void handle_query_list(Server& S, const std::string& body) {
    pb::Reader r(body.data(), body.size());
    int f, wt;
    while (r.next(&f, &wt)) {
        if (f != 1 || wt != pb::WT_LEN) {
            r.skip(wt);
            continue;
        }
        pb::Reader q(r.bytes());
        int type = 0, client = 0;
        bool need_sync = false;
        pb::View query;
        int qf, qwt;
        uint64_t u;
        while (q.next(&qf, &qwt)) {
            switch (qf) {
                case 1: if (q.read_u64(qwt, &u)) type = (int)u; break;
                case 2: if (qwt == pb::WT_LEN) query = q.bytes(); else q.skip(qwt); break;
                case 3: if (q.read_u64(qwt, &u)) client = (int)u; break;
                case 4: if (q.read_u64(qwt, &u)) need_sync = u != 0; break;
                default: q.skip(qwt);
            }
        }
        (void)need_sync;  // the reply policy follows the query type, like cuda_common.hpp:80-106
        std::string reply;
        if (handle_query(S, type, query, client, &reply)) {
            zmtp::Conn* p = pusher_for(S, client);
            if (p)
                p->send({reply});
            else if (S.verbose)
                std::fprintf(stderr, "torpor_server: cannot reach client %d\n", client);
        }
    }
}

std::string handle_signal(Server& S, const std::string& body, bool* deferred, uint64_t* ticket) {
    pb::Reader r(body.data(), body.size());
    int f, wt, type = 0;
    uint64_t u;
    std::string function, payload;
    while (r.next(&f, &wt)) {
        switch (f) {
            case 1: if (r.read_u64(wt, &u)) type = (int)u; break;
            case 2: if (wt == pb::WT_LEN) function = r.bytes().str(); else r.skip(wt); break;
            case 3: if (wt == pb::WT_LEN) payload = r.bytes().str(); else r.skip(wt); break;
            default: r.skip(wt);
        }
    }
    int32_t ack = TP_ACK_INAVAIL, resp = -1, dfr = 0;
    const int rc = tp_signal_ticket(S.eng, type, function.c_str(), payload.c_str(), &ack, &resp, &dfr, ticket);
    if (rc != 0) {
        ack = TP_ACK_INAVAIL;
        resp = -1;
        dfr = 0;
    }
    *deferred = dfr != 0;
    pb::Writer w;
    w.i32(1, ack);
    w.i32(2, resp);
    return w.out;
}

void accept_all(Server& S, int lfd, zmtp::SockType t, std::vector<std::unique_ptr<zmtp::Conn>>& into) {
    for (;;) {
        const int fd = ::accept(lfd, nullptr, nullptr);
        if (fd < 0) break;
        into.push_back(std::make_unique<zmtp::Conn>(fd, t));
        into.back()->tag = S.next_tag++;
    }
}

uint64_t env_u64(const char* name, uint64_t dflt) {
    const char* v = std::getenv(name);
    return (v && *v) ? std::strtoull(v, nullptr, 10) : dflt;
}

}  // namespace

int main() {
    Server S;
    const char* dir = std::getenv("TORPOR_IPC_DIR");
    S.dir = (dir && *dir) ? dir : "/cuda";
    S.verbose = std::getenv("TORPOR_VERBOSE") != nullptr;
    ::mkdir(S.dir.c_str(), 0777);

    tp_config cfg;
    std::memset(&cfg, 0, sizeof(cfg));
    cfg.struct_size = sizeof(cfg);
    cfg.device = (int32_t)env_u64("TORPOR_DEVICE", 0);
    cfg.mem_limit_bytes = env_u64("TORPOR_MEM_LIMIT_BYTES", 0);  // else MEM_LIMIT_IN_GB (controller.hpp:83-93)
    cfg.pool_bytes = env_u64("TORPOR_POOL_BYTES", 0);
    cfg.request_timeout_ms = (int32_t)env_u64("TORPOR_REQUEST_TIMEOUT_MS", 0);
    if (env_u64("TORPOR_HOST_ONLY", 0)) cfg.flags |= TP_FLAG_HOST_ONLY;
    const int rc = tp_server_create(&cfg, &S.eng);
    if (rc != 0) {
        std::fprintf(stderr, "torpor_server: engine start failed: %s (%d)\n", tp_strerror(rc), rc);
        return 1;
    }
    S.sig_listen = zmtp::listen_ipc("ipc://" + S.dir + "/signal_0");
    S.srv_listen = zmtp::listen_ipc("ipc://" + S.dir + "/server_0");
    if (S.sig_listen < 0 || S.srv_listen < 0) {
        std::fprintf(stderr, "torpor_server: cannot bind under %s\n", S.dir.c_str());
        tp_server_destroy(S.eng);
        return 1;
    }
    struct sigaction sa;
    std::memset(&sa, 0, sizeof(sa));
    sa.sa_handler = on_signal;
    sigaction(SIGINT, &sa, nullptr);
    sigaction(SIGTERM, &sa, nullptr);
    signal(SIGPIPE, SIG_IGN);
    std::printf("torpor_server: %s listening on ipc://%s/{signal_0,server_0}\n", tp_version(), S.dir.c_str());
    std::fflush(stdout);

    while (!g_stop) {
        std::vector<struct pollfd> pfds;
        pfds.push_back({S.sig_listen, POLLIN, 0});
        pfds.push_back({S.srv_listen, POLLIN, 0});
        for (auto& c : S.rep_conns) pfds.push_back({c->fd(), POLLIN, 0});
        for (auto& c : S.pull_conns) pfds.push_back({c->fd(), POLLIN, 0});
        ::poll(pfds.data(), pfds.size(), S.waiting_ack.empty() ? 50 : 1);
        if (pfds[0].revents & POLLIN) accept_all(S, S.sig_listen, zmtp::REP, S.rep_conns);
        if (pfds[1].revents & POLLIN) accept_all(S, S.srv_listen, zmtp::PULL, S.pull_conns);

        for (auto& c : S.pull_conns) {
            c->pump();
            while (!c->inbox().empty()) {
                zmtp::Message m = std::move(c->inbox().front());
                c->inbox().pop_front();
                for (auto& frame : m) handle_query_list(S, frame);
            }
        }
        for (auto& c : S.rep_conns) {
            c->pump();
            while (!c->inbox().empty()) {
                zmtp::Message m = std::move(c->inbox().front());
                c->inbox().pop_front();
                if (m.empty()) continue;
                bool deferred = false;
                uint64_t ticket = 0;
                const std::string ack = handle_signal(S, m.back(), &deferred, &ticket);
                if (deferred) {
                    S.waiting_ack.push_back({ticket, c->tag});  // answered when the active request completes
                } else {
                    zmtp::Message reply(m.begin(), m.end() - 1);  // envelope (empty delimiter) first
                    reply.push_back(ack);
                    c->send(reply);
                }
            }
        }
        (void)tp_poll(S.eng);  // request timeout (cuda_server.hpp:257-264)
        auto prune = [&](std::vector<std::unique_ptr<zmtp::Conn>>& v) {
            for (size_t i = 0; i < v.size();) {
                if (v[i]->failed() && v[i]->inbox().empty()) {
                    // A peer that waited for a deferred ack is gone: its queued signal is withdrawn, so
                    // that the engine neither starts a request nobody will drive nor produces an ack
                    // that another peer could be handed.
                    for (size_t k = 0; k < S.waiting_ack.size();)
                        if (S.waiting_ack[k].conn_tag == v[i]->tag) {
                            (void)tp_cancel_deferred(S.eng, S.waiting_ack[k].ticket);
                            S.waiting_ack.erase(S.waiting_ack.begin() + (long)k);
                        } else {
                            ++k;
                        }
                    v.erase(v.begin() + (long)i);
                } else {
                    ++i;
                }
            }
        };
        // Failed connections go first, their tickets with them: an ack is only taken for a peer that is
        // still there.  Should the peer vanish between this check and the send, or the send fail, the
        // request the ack belongs to has been started for nobody: it is withdrawn (tp_cancel_deferred
        // also takes back an ack that has been handed out, while its request is the active one).
        prune(S.rep_conns);
        int32_t ack = 0, resp = 0;
        uint64_t ticket = 0;
        while (tp_take_deferred_ack_ticket(S.eng, &ack, &resp, &ticket) == 1) {
            pb::Writer w;
            w.i32(1, ack);
            w.i32(2, resp);
            uint64_t tag = 0;
            for (size_t k = 0; k < S.waiting_ack.size(); ++k)
                if (S.waiting_ack[k].ticket == ticket) {
                    tag = S.waiting_ack[k].conn_tag;
                    S.waiting_ack.erase(S.waiting_ack.begin() + (long)k);
                    break;
                }
            bool delivered = false;
            for (auto& rc2 : S.rep_conns)
                if (tag && rc2->tag == tag && !rc2->failed()) delivered = rc2->send({std::string(), w.out});
            if (!delivered) (void)tp_cancel_deferred(S.eng, ticket);
        }
        prune(S.rep_conns);
        prune(S.pull_conns);
    }
    S.pushers.clear();
    S.rep_conns.clear();
    S.pull_conns.clear();
    ::close(S.sig_listen);
    ::close(S.srv_listen);
    ::unlink((S.dir + "/signal_0").c_str());
    ::unlink((S.dir + "/server_0").c_str());
    tp_server_destroy(S.eng);
    return 0;
}
