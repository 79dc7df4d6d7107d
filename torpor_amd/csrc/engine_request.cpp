#include "engine_internal.hpp"

namespace tp {

// ------------------------------------------------------------------ controller
// Everything a model holds, given back: its place in the eviction order, a copy that may still be
// running, pool extents (the weight image, the activation arena, and the per-allocation extents of a
// registration that never reached its layout step), the host store, events and a captured graph.  The
// one teardown path of a replaced registration, an abandoned one and the engine's own end; the caller
// erases the entry.
void Engine::destroy_model(Model& m) {
    lru_.force_evict(std::to_string(m.id));
    wait_copy_idle(m);
    if (!host_only() && m.touch_seq > synced_seq_ && hipStreamSynchronize(compute_) == hipSuccess)
        synced_seq_ = work_seq_;  // its last kernels may still run
    for (auto& kv : m.ablocks) {
        if (kv.second.pool_off != UINT64_MAX) pool_.release(kv.second.pool_off);
        kv.second.pool_off = UINT64_MAX;
    }
    if (m.w_pool_off != UINT64_MAX) pool_.release(m.w_pool_off);
    if (m.a_pool_off != UINT64_MAX) pool_.release(m.a_pool_off);
    m.w_pool_off = m.a_pool_off = UINT64_MAX;
    m.w_dev = m.a_dev = nullptr;
    m.resident = m.fully_loaded = false;
    m.copy_state.store(CS_IDLE);
    free_host_store(m);
    if (!host_only()) {
        for (auto ev : m.dma_ev) (void)hipEventDestroy(ev);
        for (auto ev : m.chunk_ev) (void)hipEventDestroy(ev);
        m.dma_ev.clear();
        m.chunk_ev.clear();
        if (m.t0) (void)hipEventDestroy(m.t0);
        if (m.t1) (void)hipEventDestroy(m.t1);
        m.t0 = m.t1 = nullptr;
        drop_graph(m);
    }
}

void Engine::start_cold(int id, int level) {
    // controller.hpp:402-413 + cuda_server.hpp:223-228 (Startup): a re-registration replaces
    // the previous model of that id
    Model* old = find(id);
    if (old) {
        destroy_model(*old);
        models_.erase(id);
    }
    auto m = std::make_unique<Model>();
    m->id = id;
    m->level = level;
    models_[id] = std::move(m);
    active_ = id;
    mode_ = MODE_LOAD;
    exec_status_ = ES_COLD;
}

int Engine::start_execute(int id) {
    Model* m = find(id);
    if (!m || m->state != MS_READY) return TP_ENOENT;
    const bool was_resident = m->resident;
    // controller.hpp:420-427 send_load_req: eviction check, then the Load signal
    check_eviction(*m);
    int r = swap_in(*m);
    if (r) {
        lru_.force_evict(std::to_string(id));
        return r;
    }
    // controller.hpp:414-417 + cuda_server.hpp:229-239
    active_ = id;
    mode_ = MODE_EXEC;
    // A Load for another model may arrive while this one runs (controller.hpp:208-215 has no busy
    // test): the running model is not a candidate for its eviction.
    lru_.lock(std::to_string(id));
    m->stats.gate_waits = 0;
    m->stats.host_gathers = 0;
    req_start_ = Clock::now();
    if (Roctx::get().available()) {
        char name[64];
        std::snprintf(name, sizeof name, "request of model %d (%s)", id, was_resident ? "resident" : "swapped out");
        req_range_ = Roctx::get().start(name);
    }
    if (was_resident)
        exec_status_ = ES_LOCAL;
    else
        exec_status_ = (m->level == 0) ? ES_PCIE_LIGHT : (m->level == 2 ? ES_PCIE_HEAVY : ES_PCIE_MEDIAN);
    return 0;
}

// cuda_server.hpp:287-299 send_complete_signal + controller.hpp:218-263
void Engine::complete_request() {
    if (active_ < 0) return;
    Model* m = find(active_);
    if (m && mode_ == MODE_TRACK) {
        int r = finish_tracking(*m);
        if (r && !m->async_error) m->async_error = r;
    }
    const int status = exec_status_;
    Roctx::get().stop(req_range_);
    req_range_ = 0;
    if (mode_ == MODE_EXEC)  // cuda_server.hpp:294-295
        log_.write(ExecLog::INFO, "Request of model %d completed in %.3f ms (%s)", active_, us_since(req_start_) / 1000.0,
                   status == ES_LOCAL ? "resident" : "swapped in");
    lru_.unlock(std::to_string(active_));
    active_ = -1;
    mode_ = MODE_NONE;
    if (m && m->state == MS_READY) {
        if (status == ES_COLD) check_eviction(*m);  // controller.hpp:223-227
    }
    exec_status_ = ES_AVAIL;
    start_next_queued();
}

// controller.hpp:242-262: the executor is free; the oldest queued signal gets it and its ack is produced
void Engine::start_next_queued() {
    while (exec_status_ == ES_AVAIL && !req_queue_.empty()) {
        Queued q = req_queue_.front();
        req_queue_.pop_front();
        if (q.cold) {
            start_cold(q.id, q.level);
            deferred_acks_.push_back({TP_ACK_OK, 0, q.ticket, q.id});
        } else {
            int r = start_execute(q.id);
            deferred_acks_.push_back({r ? TP_ACK_INAVAIL : TP_ACK_OK, 0, q.ticket, q.id});
        }
    }
}

bool Engine::poll_timeout_locked() {
    // cuda_server.hpp:257-264
    if (active_ >= 0 && mode_ == MODE_EXEC) {
        const double ms = us_since(req_start_) / 1000.0;
        if (ms > (double)cfg_.request_timeout_ms) {
            if (!host_only()) (void)hipStreamSynchronize(compute_);
            complete_request();
            return true;
        }
    }
    return false;
}

int Engine::poll() {
    std::lock_guard<std::mutex> lk(mu_);
    return poll_timeout_locked() ? 1 : 0;
}

int Engine::take_deferred_ack(int* ack, int* resp, uint64_t* ticket) {
    std::lock_guard<std::mutex> lk(mu_);
    if (deferred_acks_.empty()) return 0;
    if (ack) *ack = deferred_acks_.front().ack;
    if (resp) *resp = deferred_acks_.front().resp;
    if (ticket) *ticket = deferred_acks_.front().ticket;
    // Remembered while the request it started is the active one: a front end that then fails to deliver the
    // ack can still withdraw the request (cancel_deferred).
    while (!taken_acks_.empty() && taken_acks_.front().id != active_) taken_acks_.pop_front();
    if (deferred_acks_.front().ack == TP_ACK_OK && deferred_acks_.front().id == active_)
        taken_acks_.push_back(deferred_acks_.front());
    deferred_acks_.pop_front();
    return 1;
}

// The peer that sent a queued signal is gone.  Still queued: the entry is dropped and no ack will
// appear for it (1).  Already started -- its ack not yet taken, or taken by a front end that could not
// deliver it -- the ack is dropped and the request, which nobody will drive, is completed at once instead
// of holding the executor until the request timeout (or, for a registration, for good) (2).  Unknown, or
// the request it started is no longer the active one: 0.
int Engine::cancel_deferred(uint64_t ticket) {
    std::lock_guard<std::mutex> lk(mu_);
    for (auto it = req_queue_.begin(); it != req_queue_.end(); ++it)
        if (it->ticket == ticket) {
            req_queue_.erase(it);
            return 1;
        }
    for (auto it = taken_acks_.begin(); it != taken_acks_.end(); ++it)
        if (it->ticket == ticket) {
            if (it->id != active_) {  // that request is over
                taken_acks_.erase(it);
                return 0;
            }
            deferred_acks_.push_front(*it);  // handled below like an ack that was never taken
            taken_acks_.erase(it);
            break;
        }
    for (auto it = deferred_acks_.begin(); it != deferred_acks_.end(); ++it)
        if (it->ticket == ticket) {
            const int id = it->id;
            const bool started = it->ack == TP_ACK_OK;
            deferred_acks_.erase(it);
            if (started && active_ == id) {
                if (mode_ == MODE_LOAD || mode_ == MODE_TRACK) {
                    // a registration nobody finishes: forget the half-built model
                    Model* m = find(id);
                    if (!host_only()) (void)hipStreamSynchronize(compute_);  // its tracked kernels may still run
                    if (m) {
                        destroy_model(*m);
                        models_.erase(id);
                    }
                    active_ = -1;
                    mode_ = MODE_NONE;
                    exec_status_ = ES_AVAIL;
                    start_next_queued();
                } else {
                    if (!host_only()) (void)hipStreamSynchronize(compute_);
                    complete_request();
                }
            }
            return 2;
        }
    return 0;
}

// Does [va, va + bytes) lie inside one block the active function `client` may address right now?
// No side effects (no access-order rank, no gate wait): a front end asks before it sets aside
// `bytes` of its own memory for a copy.
int Engine::check_address(int client, uint64_t va, uint64_t bytes) {
    std::lock_guard<std::mutex> lk(mu_);
    if (active_ < 0 || mode_ == MODE_NONE) return TP_ESTATE;
    if (client != active_) return TP_ENOTACTIVE;
    Model* m = find(active_);
    if (!m) return TP_ENOENT;
    Xlat x;
    return translate(*m, va, bytes, &x);
}

static bool parse_int(const char* s, int* out) {
    if (!s || !*s) return false;
    char* end = nullptr;
    long v = std::strtol(s, &end, 10);
    if (*end != '\0') return false;
    *out = (int)v;
    return true;
}

int Engine::signal(int type, const char* function, const char* payload, int* ack, int* resp, int* deferred,
                   uint64_t* ticket) {
    std::lock_guard<std::mutex> lk(mu_);
    if (ack) *ack = TP_ACK_OK;
    if (resp) *resp = -1;
    if (deferred) *deferred = 0;
    if (ticket) *ticket = 0;
    int id = -1;
    if (!parse_int(function, &id) || id < 0) return TP_EINVAL;  // cuda_server.hpp:221 stoi(func)
    if (id > kMaxClient) return TP_ERANGE;  // the id is part of every address handed to the function
    poll_timeout_locked();
    const bool busy = exec_status_ != ES_AVAIL;
    switch (type) {
        case TP_REQ_EXECUTE_AFTER_LOAD: {  // controller.hpp:141-162
            int level = 1;
            int lv = 0;
            if (payload && *payload && parse_int(payload, &lv) && lv >= 0 && lv <= 2) level = lv;
            if (busy) {
                if (active_ == id) {
                    if (ack) *ack = TP_ACK_INAVAIL;
                    return 0;
                }
                req_queue_.push_back({id, true, level, ++ticket_seq_});
                if (deferred) *deferred = 1;
                if (ticket) *ticket = ticket_seq_;
                return 0;
            }
            start_cold(id, level);
            if (resp) *resp = 0;
            return 0;
        }
        case TP_REQ_EXECUTE: {  // controller.hpp:163-186
            if (busy) {
                req_queue_.push_back({id, false, 1, ++ticket_seq_});
                if (deferred) *deferred = 1;
                if (ticket) *ticket = ticket_seq_;
                return 0;
            }
            int r = start_execute(id);
            if (r) {
                if (ack) *ack = TP_ACK_INAVAIL;
                return 0;
            }
            if (resp) *resp = 0;
            return 0;
        }
        case TP_REQ_UNLOAD: {  // controller.hpp:187-207
            Model* m = find(id);
            if (active_ == id) {
                if (ack) *ack = TP_ACK_INAVAIL;
                return 0;
            }
            if (m && m->resident && m->state == MS_READY) {
                lru_.force_evict(std::to_string(id));
                evict_model(*m);
            }
            return 0;  // ack OK, resp -1
        }
        case TP_REQ_LOAD: {  // controller.hpp:208-215
            Model* m = find(id);
            if (!m || m->state != MS_READY || active_ == id) {
                if (ack) *ack = TP_ACK_INAVAIL;
                return 0;
            }
            check_eviction(*m);
            int r = swap_in(*m);
            if (r) {
                lru_.force_evict(std::to_string(id));
                if (ack) *ack = TP_ACK_INAVAIL;
            }
            return 0;
        }
        default:  // ExecuteForRecord / Replay are refused like in cuda_server.hpp:188-195
            if (ack) *ack = TP_ACK_INAVAIL;
            return 0;
    }
}
}  // namespace tp
