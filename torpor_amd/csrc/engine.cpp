#include "engine.hpp"
#include "weight_pack.hpp"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "kernels/kernels.hpp"

namespace tp {

using Clock = std::chrono::steady_clock;
static inline double us_since(Clock::time_point t0) {
    return std::chrono::duration<double, std::micro>(Clock::now() - t0).count();
}
static inline uint64_t align_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

#define HIPCHK(expr)                         \
    do {                                     \
        hipError_t _e = (expr);              \
        if (_e != hipSuccess) return (int)_e; \
    } while (0)

static uint64_t env_u64(const char* name, uint64_t dflt) {
    const char* v = std::getenv(name);
    if (!v || !*v) return dflt;
    char* end = nullptr;
    unsigned long long x = std::strtoull(v, &end, 10);
    if (end == v) return dflt;
    return (uint64_t)x;
}

static void op_work(const Op& op, double* flops, double* bytes, const char** name);

// Runs f(0) .. f(n-1) on up to TORPOR_HOST_THREADS (default 8) threads, the caller's included; tasks are
// handed out one at a time.  Returns false if a task threw (the others still ran).
template <class F>
static bool parallel_for(size_t n, F&& f) {
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

// The four streams of an engine outlive it: a later engine of the same process on the same device takes
// them over instead of creating new ones.  A process has few hardware queues (four by default) and streams
// are bound to them as they are created; the streams of a second engine, created after the first one's
// were destroyed, ended up sharing queues (the expansion stream with the compute stream), and every kernel
// of a cold request then waited behind the other stream's (ResNet-152 batch 1 cold 3.8 -> 4.6 ms).
namespace {
struct StreamSet {
    int device;
    hipStream_t s[4];
};
std::mutex g_streams_mu;
std::vector<StreamSet> g_idle_streams;

int acquire_streams(int device, hipStream_t out[4]) {
    {
        std::lock_guard<std::mutex> lk(g_streams_mu);
        for (size_t i = 0; i < g_idle_streams.size(); ++i)
            if (g_idle_streams[i].device == device) {
                for (int k = 0; k < 4; ++k) out[k] = g_idle_streams[i].s[k];
                g_idle_streams.erase(g_idle_streams.begin() + (long)i);
                return 0;
            }
    }
    for (int k = 0; k < 4; ++k) {
        hipError_t e = hipStreamCreateWithFlags(&out[k], hipStreamNonBlocking);
        if (e != hipSuccess) {
            for (int j = 0; j < k; ++j) (void)hipStreamDestroy(out[j]);
            for (int j = 0; j < 4; ++j) out[j] = nullptr;
            return (int)e;
        }
    }
    return 0;
}

void release_streams(int device, hipStream_t in[4]) {  // the caller has drained them
    StreamSet set;
    set.device = device;
    for (int k = 0; k < 4; ++k) set.s[k] = in[k];
    std::lock_guard<std::mutex> lk(g_streams_mu);
    try {
        g_idle_streams.push_back(set);
    } catch (...) {
        for (int k = 0; k < 4; ++k) (void)hipStreamDestroy(in[k]);
    }
}
}  // namespace

Engine::Engine(const tp_config& cfg) : cfg_(cfg) {}

int Engine::init() {
    // controller.hpp:83-93: MEM_LIMIT_IN_GB; the reference caps it below 25 GB for 32 GB parts,
    // here any positive value up to the device size is accepted.
    if (cfg_.mem_limit_bytes == 0) cfg_.mem_limit_bytes = env_u64("MEM_LIMIT_IN_GB", 24) << 30;
    if (cfg_.chunk_bytes == 0) cfg_.chunk_bytes = env_u64("BUFFER_SIZE", 2ull << 20);  // memory_manager.hpp:22
    per_tensor_groups_ = cfg_.chunk_bytes < kTensorAlign;                              // BUFFER_SIZE=1 ablation
    if (cfg_.chunk_bytes < kTensorAlign) cfg_.chunk_bytes = kTensorAlign;
    chunk_max_auto_ = cfg_.chunk_max_bytes == 0;
    if (cfg_.chunk_max_bytes == 0) cfg_.chunk_max_bytes = 8ull << 20;
    if (cfg_.chunk_max_bytes < cfg_.chunk_bytes) cfg_.chunk_max_bytes = cfg_.chunk_bytes;
    if (cfg_.workspace_bytes == 0) cfg_.workspace_bytes = 64ull << 20;
    if (cfg_.request_timeout_ms <= 0) cfg_.request_timeout_ms = 5000;  // cuda_server.hpp:29
    // memory_manager.hpp:42-44 adds 5 GiB of slack above the eviction budget; 1 GiB is enough
    // here because allocations are whole-model extents, not per-tensor blocks.
    if (cfg_.pool_bytes == 0) cfg_.pool_bytes = cfg_.mem_limit_bytes + (1ull << 30);
    {
        const char* pol = std::getenv("EVICT_POLICY");  // controller.hpp:103-109
        lru_.two_class = !((cfg_.flags & TP_FLAG_EVICT_LRU) || (pol && std::string(pol) == "LRU"));
    }
    lru_.set_budget(cfg_.mem_limit_bytes);
    {
        const char* bm = std::getenv("BLOCK_MANAGER");  // memory_manager.hpp:46-52
        const bool fixed = (cfg_.flags & TP_FLAG_POOL_FIXED) || (bm && std::string(bm) == "Fixed");
        pool_.reset(cfg_.pool_bytes, fixed ? SlabPool::kFixedSize : SlabPool::kBestFit);
    }
    log_.open(cfg_.device);
    log_.write(ExecLog::INFO, "Executor %d started: budget %llu MiB, pool %llu MiB, first transfer group %llu KiB, %s eviction",
               cfg_.device, (unsigned long long)(cfg_.mem_limit_bytes >> 20), (unsigned long long)(pool_.capacity() >> 20),
               (unsigned long long)(cfg_.chunk_bytes >> 10), lru_.two_class ? "two-class" : "LRU");

    if (host_only()) {
        arena_ = reinterpret_cast<uint8_t*>(0x100000000000ull);
        return 0;
    }
    HIPCHK(hipSetDevice(cfg_.device));
    tpk::kernels_init(cfg_.device);
    HIPCHK(hipMalloc(reinterpret_cast<void**>(&arena_), pool_.capacity()));
    HIPCHK(hipMalloc(reinterpret_cast<void**>(&workspace_), cfg_.workspace_bytes));
    HIPCHK(hipMemset(workspace_, 0, cfg_.workspace_bytes));  // split-K tile counters start at zero
    {
        hipStream_t st[4] = {nullptr, nullptr, nullptr, nullptr};
        int r = acquire_streams(cfg_.device, st);
        if (r) return r;
        compute_ = st[0];
        copy_ = st[1];
        copy2_ = st[2];
        decode_ = st[3];
    }
    copy_streams_cfg_ = (int)env_u64("TORPOR_COPY_STREAMS", (uint64_t)cfg_.copy_streams);  // 0 = per model
    plan_trials_ = (int)env_u64("TORPOR_PLAN_TRIALS", 2);
    graph_min_ops_ = (int)env_u64("TORPOR_GRAPH_MIN_OPS", 0);
    pack_ = !(cfg_.flags & TP_FLAG_NO_PACK) && env_u64("TORPOR_PACK", 1) != 0;
    slim_host_ = !(cfg_.flags & TP_FLAG_KEEP_HOST_IMAGE) && env_u64("TORPOR_SLIM_HOST", 1) != 0;
    HIPCHK(hipEventCreateWithFlags(&stage_free_ev_, hipEventDisableTiming));
    d2h_kernel_ = (int)env_u64("TORPOR_D2H_KERNEL", 2);  // 0 never, 1 always, 2 small copies and while a swap-in is running
    small_copy_bytes_ = env_u64("TORPOR_SMALL_COPY_BYTES", 1ull << 20);
    host_gather_ = !(cfg_.flags & TP_FLAG_NO_HOST_GATHER) && env_u64("TORPOR_HOST_GATHER", 1) != 0;
    HIPCHK(hipHostMalloc(reinterpret_cast<void**>(&h2d_stage_), 16ull << 20, hipHostMallocDefault));
    h2d_cap_ = 16ull << 20;
    HIPCHK(hipHostMalloc(reinterpret_cast<void**>(&d2h_stage_), 8ull << 20, hipHostMallocDefault));
    d2h_cap_ = 8ull << 20;
    {  // first use of the copy kernel and of device writes into the pinned buffer, off the request path
        void* stage_dev = nullptr;
        if (hipHostGetDevicePointer(&stage_dev, d2h_stage_, 0) == hipSuccess && stage_dev) {
            (void)tpk::launch_copy(workspace_, stage_dev, 4096, compute_);
            HIPCHK(hipStreamSynchronize(compute_));
        } else {
            (void)hipGetLastError();
            d2h_kernel_ = 0;
        }
    }
    {
        // First use of the copy streams (queue and copy-engine set-up, about 6 ms) happens here
        // rather than inside the first swap-in: a few copies on both streams, issued as a swap-in
        // issues them, into the upper half of the workspace.
        uint8_t* ws = reinterpret_cast<uint8_t*>(workspace_);
        const uint64_t half = cfg_.workspace_bytes / 2;
        const uint64_t n = std::min<uint64_t>(std::min<uint64_t>(half / 2, h2d_cap_ / 2), 8ull << 20) & ~uint64_t(255);
        if (n) {
            // The second half of the burst is timed: both streams taking turns, as a swap-in of a link-bound
            // model drives them, is the rate the swap-in plans are made with until tp_measure_h2d is asked
            // for the single-copy figure.
            hipEvent_t ev_a = nullptr, ev_b = nullptr, ev_2 = nullptr;
            (void)hipEventCreate(&ev_a);
            (void)hipEventCreate(&ev_b);
            (void)hipEventCreateWithFlags(&ev_2, hipEventDisableTiming);
            constexpr int kBurst = 24, kTimedFrom = 12;
            for (int rep = 0; rep < kBurst; ++rep) {
                if (rep == kTimedFrom && ev_a && ev_2) {
                    (void)hipEventRecord(ev_2, copy2_);
                    (void)hipStreamWaitEvent(copy_, ev_2, 0);  // both streams start the timed half together
                    (void)hipEventRecord(ev_a, copy_);
                    (void)hipStreamWaitEvent(copy2_, ev_a, 0);
                }
                HIPCHK(hipMemcpyAsync(ws + half, h2d_stage_, n, hipMemcpyHostToDevice, copy_));
                HIPCHK(hipMemcpyAsync(ws + half + n, h2d_stage_ + n, n, hipMemcpyHostToDevice, copy2_));
            }
            if (ev_a && ev_b && ev_2) {
                (void)hipEventRecord(ev_2, copy2_);
                (void)hipStreamWaitEvent(copy_, ev_2, 0);
                (void)hipEventRecord(ev_b, copy_);
            }
            (void)tpk::launch_copy(ws + half, ws + half + n, 4096, decode_);
            HIPCHK(hipStreamSynchronize(copy_));
            HIPCHK(hipStreamSynchronize(copy2_));
            HIPCHK(hipStreamSynchronize(decode_));
            float burst_ms = 0.f;
            if (ev_a && ev_b && hipEventElapsedTime(&burst_ms, ev_a, ev_b) == hipSuccess && burst_ms > 0.f) {
                const double gbps = 2.0 * (kBurst - kTimedFrom) * (double)n / (burst_ms * 1e-3) / 1e9 / 0.99;
                if (gbps > 1.0 && gbps < 1000.0) link_gbps_ = gbps;
            } else {
                (void)hipGetLastError();
            }
            if (ev_a) (void)hipEventDestroy(ev_a);
            if (ev_b) (void)hipEventDestroy(ev_b);
            if (ev_2) (void)hipEventDestroy(ev_2);
            log_.write(ExecLog::INFO, "Host link measured at %.1f GB/s", link_gbps_);
            // One swap-in in the first few dozen of a process used to take 6.5 ms longer: a single
            // hipMemcpyAsync call of one of its first groups blocked that long on the host (timed per call,
            // tp_swap_stats.max_call_*), whatever the model.  It is a one-time set-up inside the runtime that
            // a copy triggers when it is submitted while the copy engines used so far are busy; two streams
            // taking turns reach that state only now and then.  Copies in flight on several more streams at
            // once reach it here: 3 of 8 fresh processes showed the stall within 160 swap-ins without this
            // burst, none of 8 with it.  (TORPOR_INIT_STREAMS=0 leaves it out.)
            const int extra = (int)env_u64("TORPOR_INIT_STREAMS", 6);
            if (extra > 0) {
                std::vector<hipStream_t> tmp((size_t)extra, nullptr);
                for (auto& t : tmp) (void)hipStreamCreateWithFlags(&t, hipStreamNonBlocking);
                const uint64_t piece = (n / (uint64_t)(extra + 2)) & ~uint64_t(255);
                for (int rep = 0; rep < 4 && piece; ++rep) {
                    int k = 0;
                    (void)hipMemcpyAsync(ws + half + piece * k, h2d_stage_ + piece * k, piece, hipMemcpyHostToDevice, copy_);
                    ++k;
                    (void)hipMemcpyAsync(ws + half + piece * k, h2d_stage_ + piece * k, piece, hipMemcpyHostToDevice, copy2_);
                    ++k;
                    for (auto& t : tmp)
                        if (t) {
                            (void)hipMemcpyAsync(ws + half + piece * k, h2d_stage_ + piece * k, piece, hipMemcpyHostToDevice, t);
                            ++k;
                        }
                }
                (void)hipStreamSynchronize(copy_);
                (void)hipStreamSynchronize(copy2_);
                for (auto& t : tmp)
                    if (t) {
                        (void)hipStreamSynchronize(t);
                        (void)hipStreamDestroy(t);
                    }
            }
            HIPCHK(hipMemset(ws + half, 0, 2 * n));  // the workspace is handed to the kernels zeroed
        }
    }
    copy_thread_ = std::thread(&Engine::copy_main, this);
    return 0;
}

Engine::~Engine() {
    {
        std::lock_guard<std::mutex> lk(cmu_);
        stop_ = true;
    }
    ccv_.notify_all();
    if (copy_thread_.joinable()) copy_thread_.join();
    if (!host_only()) {
        (void)hipSetDevice(cfg_.device);
        (void)hipDeviceSynchronize();
    }
    for (auto& kv : models_) {
        kv.second->copy_state.store(CS_IDLE);  // the copy thread is gone: a job it never took is not waited for
        destroy_model(*kv.second);
    }
    models_.clear();
    for (auto& kv : user_pinned_) host_free(reinterpret_cast<void*>(kv.first));
    user_pinned_.clear();
    if (!host_only()) {
        for (auto e : prof_events_) (void)hipEventDestroy(e);
        if (h2d_stage_) (void)hipHostFree(h2d_stage_);
        if (d2h_stage_) (void)hipHostFree(d2h_stage_);
        if (workspace_) (void)hipFree(workspace_);
        if (arena_) (void)hipFree(arena_);
        if (xfer_stage_) (void)hipFree(xfer_stage_);
        if (stage_free_ev_) (void)hipEventDestroy(stage_free_ev_);
        if (compute_ && copy_ && copy2_ && decode_) {  // drained by the device synchronisation above
            hipStream_t st[4] = {compute_, copy_, copy2_, decode_};
            release_streams(cfg_.device, st);
        }
    }
}

void* Engine::host_alloc(uint64_t bytes) {
    if (bytes == 0) bytes = 1;
    if (host_only()) return std::malloc(bytes);
    void* p = nullptr;
    // The host weight store is pinned once, at registration, so a swap-in is a straight DMA.
    // The reference keeps it pageable (model_repo.hpp:173-177) and stages through pinned
    // buffers on every swap-in (memory_manager.hpp:311-329,354-370).
    if (hipHostMalloc(&p, bytes, hipHostMallocDefault) != hipSuccess) return nullptr;
    return p;
}
void Engine::host_free(void* p) {
    if (!p) return;
    if (host_only())
        std::free(p);
    else
        (void)hipHostFree(p);
}

Model* Engine::find(int id) {
    auto it = models_.find(id);
    return it == models_.end() ? nullptr : it->second.get();
}

Model* Engine::active_model(int client, int* err) {
    if (active_ < 0 || mode_ == MODE_NONE) {
        *err = TP_ESTATE;
        return nullptr;
    }
    if (client != active_) {
        *err = TP_ENOTACTIVE;
        return nullptr;
    }
    Model* m = find(active_);
    if (!m)
        *err = TP_ENOENT;
    else
        m->touch_seq = ++work_seq_;
    return m;
}

// ------------------------------------------------------------------ address translation
// memory_manager.hpp:261-271 (get_cuda_addr), 527-568 (check_param_readiness, get_phy_address):
// the reference walks several hash maps per pointer; here a weight address is one binary
// search in the tensor table plus an add, an activation address one map lookup plus an add.
int Engine::translate(Model& m, uint64_t va, uint64_t span, Xlat* out) {
    if ((va & kVaTagMask) != kVaTag) return TP_EFAULT;
    if ((int)((va >> kVaClientShift) & kVaClientMask) != m.id) return TP_EFAULT;
    const uint64_t off = va & kVaOffMask;
    if (va & kVaActBit) {
        auto it = m.ablocks.upper_bound(off);
        if (it == m.ablocks.begin()) return TP_EFAULT;
        --it;
        ABlock& b = it->second;
        // (off - b.voff) < b.size here, so neither side of the comparison can wrap
        if (off >= b.voff + b.size || span > b.size - (off - b.voff)) return TP_EFAULT;
        // Once the arena is frozen every block keeps its place for good and later requests repeat
        // the tracked op stream without re-issuing its malloc/free calls, so liveness is only
        // enforced while the first inference is being tracked.
        if (!m.act_frozen && !b.live) return TP_EFAULT;
        if (m.act_frozen) {
            if (!m.resident) return TP_EFAULT;
            out->p = m.a_dev + off;
        } else {
            if (b.pool_off == UINT64_MAX) return TP_EFAULT;
            out->p = arena_ + b.pool_off + (off - b.voff);
        }
        out->weight = false;
        out->param = nullptr;
        return 0;
    }
    // weight region
    auto it = std::upper_bound(m.params.begin(), m.params.end(), off,
                               [](uint64_t o, const Param& p) { return o < p.voff; });
    if (it == m.params.begin()) return TP_EFAULT;
    --it;
    if (off >= it->voff + it->size || span > it->size - (off - it->voff)) return TP_EFAULT;
    if (m.state == MS_LOADING || !m.resident) return TP_EFAULT;
    out->p = m.w_dev + it->image_off + (off - it->voff);
    out->weight = true;
    out->image_end = it->image_off + it->size;
    out->param = &*it;
    return 0;
}

// memory_manager.hpp:527-533: the reference blocks the executor thread on a host queue until
// the tensor's transfer group has been host-synchronised.  Here the executor only makes the
// compute stream wait for the group's event; the host never waits for data.
int Engine::gate(Model& m, const Xlat& x) {
    if (!x.weight || m.fully_loaded || host_only()) return 0;
    if (m.copy_state.load(std::memory_order_acquire) == CS_IDLE) return 0;  // resident from registration
    auto it = std::lower_bound(m.chunk_end.begin(), m.chunk_end.end(), x.image_end);
    if (it == m.chunk_end.end()) return TP_EFAULT;
    const uint32_t idx = (uint32_t)(it - m.chunk_end.begin());
    if (idx < m.gated_upto) return 0;
    // the event must have been recorded by the copy thread before the stream may wait on it
    while (m.issued.load(std::memory_order_acquire) <= idx) {
        if (m.copy_error.load()) return m.copy_error.load();
        if (m.copy_state.load(std::memory_order_acquire) != CS_RUNNING && m.issued.load() <= idx) return TP_ESTATE;
#if defined(__x86_64__)
        __builtin_ia32_pause();
#endif
    }
    HIPCHK(hipStreamWaitEvent(compute_, m.chunk_ev[idx], 0));
    // groups alternate between two copy streams: the previous group travels on the other one
    if (m.ncopy == 2 && idx > 0 && idx - 1 >= m.gated_upto) HIPCHK(hipStreamWaitEvent(compute_, m.chunk_ev[idx - 1], 0));
    m.gated_upto = idx + 1;
    m.stats.gate_waits++;
    return 0;
}

// Has transfer group `idx` of the running swap-in arrived?  Never blocks.
bool Engine::landed(Model& m, uint32_t idx) {
    if (idx < m.gated_upto) return true;
    if (m.issued.load(std::memory_order_acquire) <= idx) return false;
    if (hipEventQuery(m.chunk_ev[idx]) != hipSuccess) return false;
    return !(m.ncopy == 2 && idx > 0 && idx - 1 >= m.gated_upto && hipEventQuery(m.chunk_ev[idx - 1]) != hipSuccess);
}

// `gather`: the kernel looks rows of this operand up by index instead of streaming it.
int Engine::resolve(Model& m, uint64_t va, uint64_t span, bool optional, void** out, bool gather) {
    *out = nullptr;
    if (va == 0) return optional ? 0 : TP_EFAULT;
    Xlat x;
    int r = translate(m, va, span, &x);
    if (r) return r;
    if (x.weight) {
        // memory_manager.hpp:273-284 / model_repo.hpp:102-109: first-access order, tracked run only
        if (mode_ == MODE_TRACK) {
            if (x.param->access_rank < 0) x.param->access_rank = m.next_rank++;
            if (gather) x.param->gathered = true;
        }
        // A table whose transfer group has not arrived is read where it lies in the pinned host
        // store: the few rows a request needs cross the link at once, the table itself follows
        // after every tensor the forward pass streams through.
        if (gather && host_gather_ && x.param->gathered && (m.host_image_dev || m.gather_dev) && !m.fully_loaded &&
            !host_only() && m.copy_state.load(std::memory_order_acquire) != CS_IDLE) {
            auto it = std::lower_bound(m.chunk_end.begin(), m.chunk_end.end(), x.image_end);
            if (it == m.chunk_end.end()) return TP_EFAULT;
            if (!landed(m, (uint32_t)(it - m.chunk_end.begin()))) {
                if (m.copy_error.load()) return m.copy_error.load();
                const uint64_t ioff = (uint64_t)(static_cast<uint8_t*>(x.p) - m.w_dev);
                if (m.host_image_dev) {
                    *out = m.host_image_dev + ioff;
                } else {
                    if (ioff < m.gather_off || x.image_end > m.gather_off + m.gather_bytes) return TP_EFAULT;
                    *out = m.gather_dev + (ioff - m.gather_off);
                }
                m.stats.host_gathers++;
                return 0;
            }
        }
        r = gate(m, x);
        if (r) return r;
    }
    *out = x.p;
    return 0;
}

// ------------------------------------------------------------------ memory ops
int Engine::op_malloc(int client, uint64_t bytes, uint64_t* va) {
    std::lock_guard<std::mutex> lk(mu_);
    if (!va) return TP_EINVAL;
    int err = 0;
    Model* m = active_model(client, &err);
    if (!m) return err;
    if (bytes == 0) bytes = 1;
    if (bytes > kVaOffMask) return TP_ENOMEM;  // larger than a function's address region: nothing below may wrap
    const uint64_t base = kVaTag | ((uint64_t)m->id << kVaClientShift);
    if (mode_ == MODE_LOAD) {  // weight block: cuda_server.hpp:969-970 with load flag set
        const uint64_t off = m->wbump;
        if (off + bytes > kVaOffMask) return TP_ENOMEM;
        const uint64_t bump = align_up(off + bytes, kTensorAlign);
        if (!m->staging.resize(bump)) return TP_ENOMEM;  // nothing recorded for a block that has no room
        m->wbump = bump;
        m->wblocks.push_back({off, bytes});
        *va = base | off;
        return 0;
    }
    // activation block
    auto fr = m->afree.find(bytes);
    if (fr != m->afree.end()) {
        ABlock& b = m->ablocks[fr->second];
        m->afree.erase(fr);
        b.live = true;
        *va = base | kVaActBit | b.voff;
        return 0;
    }
    if (m->act_frozen) return TP_ENOMEM;  // arena is sized by the first (tracked) inference
    if (m->abump + bytes > kVaOffMask) return TP_ENOMEM;
    ABlock b;
    b.voff = m->abump;
    b.size = bytes;
    b.live = true;
    b.pool_off = pool_.alloc(bytes);
    if (b.pool_off == UINT64_MAX) return TP_ENOMEM;
    m->abump = align_up(m->abump + bytes, kTensorAlign);
    m->ablocks[b.voff] = b;
    *va = base | kVaActBit | b.voff;
    return 0;
}

int Engine::op_free(int client, uint64_t va) {
    std::lock_guard<std::mutex> lk(mu_);
    int err = 0;
    Model* m = active_model(client, &err);
    if (!m) return err;
    if ((va & kVaTagMask) != kVaTag || (int)((va >> kVaClientShift) & kVaClientMask) != m->id) return TP_EFAULT;
    if (!(va & kVaActBit)) return TP_EINVAL;  // memory_manager.hpp:99-101: freeing a model block is refused
    auto it = m->ablocks.find(va & kVaOffMask);
    if (it == m->ablocks.end() || !it->second.live) return TP_EFAULT;
    it->second.live = false;
    m->afree.emplace(it->second.size, it->second.voff);
    return 0;
}

int Engine::ensure_stage(uint8_t** buf, uint64_t* cap, uint64_t need) {
    if (need <= *cap) return 0;
    uint64_t ncap = *cap ? *cap : (1ull << 20);
    while (ncap < need) ncap *= 2;
    HIPCHK(hipStreamSynchronize(compute_));
    uint8_t* nb = nullptr;
    HIPCHK(hipHostMalloc(reinterpret_cast<void**>(&nb), ncap, hipHostMallocDefault));
    if (*buf) (void)hipHostFree(*buf);
    *buf = nb;
    *cap = ncap;
    return 0;
}

// A request's input or result, by a copy kernel or by the copy engines?  During a swap-in -- this model's or
// anybody's -- always by kernel (see do_h2d); otherwise by kernel up to small_copy_bytes_: a hipMemcpyAsync
// carries about 15 us of fixed cost, a kernel launch behind the previous one 2-3 us, and the link moves 1 MiB in
// 18 us either way (ResNet-50 batch 1, 602 KB of input: warm 0.551 -> 0.538 ms; ResNet-152 batch 8, 4.8 MB:
// 2.95 ms either way).  TORPOR_D2H_KERNEL: 0 never, 1 always, 2 by this rule.
bool Engine::copy_by_kernel(const Model& m, uint64_t bytes) {
    if (d2h_kernel_ == 1) return true;
    if (d2h_kernel_ != 2) return false;
    return bytes <= small_copy_bytes_ || !m.fully_loaded || swap_in_flight();
}

int Engine::do_h2d(Model& m, uint64_t dst, const void* src, uint64_t bytes) {
    if (bytes == 0) return 0;
    if (!src || bytes > kVaOffMask) return TP_EINVAL;
    if (mode_ == MODE_LOAD) {
        // memory_manager.hpp:124-142 + model_repo.hpp:151-168: capture into the host weight store
        if ((dst & kVaTagMask) != kVaTag || (int)((dst >> kVaClientShift) & kVaClientMask) != m.id ||
            (dst & kVaActBit))
            return TP_EFAULT;
        const uint64_t off = dst & kVaOffMask;
        bool inside = false;
        for (const WBlock& b : m.wblocks)
            if (off >= b.voff && off - b.voff < b.size && bytes <= b.size - (off - b.voff)) {
                inside = true;
                break;
            }
        if (!inside) return TP_EFAULT;
        std::memcpy(m.staging.data() + off, src, bytes);
        // a tensor is what one upload covers; a repeated upload to the same start replaces it
        for (Param& p : m.params)
            if (p.voff == off) {
                if (p.size != bytes) return TP_EINVAL;
                return 0;
            }
        Param p;
        p.voff = off;
        p.size = bytes;
        m.params.push_back(p);
        return 0;
    }
    if (!(dst & kVaActBit)) return TP_ESTATE;  // the host copy of the weights is authoritative
    Xlat x;
    int r = translate(m, dst, bytes, &x);
    if (r) return r;
    if (host_only()) return 0;
    // A source inside a pinned buffer handed out by user_host_alloc needs no staging copy: the device reads it
    // where it lies (the caller leaves it alone until the request's next synchronising call, as with any
    // asynchronous copy from pinned memory).  ResNet-152 batch 8, 4.8 MB of input: the staging memcpy was
    // 0.1 ms of a 2.9 ms request.
    {
        const uintptr_t sp = reinterpret_cast<uintptr_t>(src);
        auto ub = user_pinned_.upper_bound(sp);
        if (ub != user_pinned_.begin()) {
            --ub;
            if (sp >= ub->first && sp - ub->first + bytes <= ub->second) {
                void* src_dev = nullptr;
                if (copy_by_kernel(m, bytes) &&
                    hipHostGetDevicePointer(&src_dev, const_cast<void*>(src), 0) == hipSuccess && src_dev) {
                    int kr = tpk::launch_copy(static_cast<const uint8_t*>(src_dev), x.p, bytes, compute_);
                    if (kr) return kr;
                } else {
                    HIPCHK(hipMemcpyAsync(x.p, src, bytes, hipMemcpyHostToDevice, compute_));
                }
                return 0;
            }
        }
    }
    if (h2d_pos_ + bytes > h2d_cap_) {
        HIPCHK(hipStreamSynchronize(compute_));
        h2d_pos_ = 0;
        r = ensure_stage(&h2d_stage_, &h2d_cap_, bytes);
        if (r) return r;
    }
    // During a swap-in -- this model's or, when requests of resident models are served while another
    // model streams in, anybody's -- the copy engines belong to the weight stream: a request input handed
    // to them queues among its transfer groups and disturbs how they alternate over the engines.  A copy
    // kernel reads the pinned buffer instead (alignment of the destination permitting).
    void* stage_dev = nullptr;
    const bool by_kernel = copy_by_kernel(m, bytes) &&
                           hipHostGetDevicePointer(&stage_dev, h2d_stage_, 0) == hipSuccess && stage_dev;
    // A large input goes through the staging buffer in pieces of 1 MiB: the host copies the next piece while
    // the link moves the one before.
    const uint64_t piece = bytes > (2ull << 20) ? (1ull << 20) : bytes;
    for (uint64_t off = 0; off < bytes; off += piece) {
        const uint64_t n = std::min(piece, bytes - off);
        std::memcpy(h2d_stage_ + h2d_pos_ + off, static_cast<const uint8_t*>(src) + off, n);
        if (by_kernel) {
            int kr = tpk::launch_copy(static_cast<uint8_t*>(stage_dev) + h2d_pos_ + off, x.p + off, n, compute_);
            if (kr) return kr;
        } else {
            HIPCHK(hipMemcpyAsync(x.p + off, h2d_stage_ + h2d_pos_ + off, n, hipMemcpyHostToDevice, compute_));
        }
    }
    h2d_pos_ = align_up(h2d_pos_ + bytes, 256);
    return 0;
}

int Engine::op_h2d(int client, uint64_t dst, const void* src, uint64_t bytes) {
    std::lock_guard<std::mutex> lk(mu_);
    int err = 0;
    Model* m = active_model(client, &err);
    if (!m) return err;
    int r = do_h2d(*m, dst, src, bytes);
    if (r == 0 && mode_ == MODE_TRACK) {
        Op op;
        op.kind = OPK_H2D;
        op.p[0] = dst;
        op.i[0] = (int64_t)bytes;
        m->program.push_back(op);
    }
    if (r && !m->async_error) m->async_error = r;
    return r;
}

int Engine::do_d2h_async(Model& m, void* dst, uint64_t src, uint64_t bytes) {
    if ((!dst && bytes) || bytes > kVaOffMask) return TP_EINVAL;
    void* p = nullptr;
    int r = resolve(m, src, bytes, false, &p);
    if (r) return r;
    if (!host_only() && bytes) {
        // a destination inside a pinned result buffer of ours is written by the device itself
        auto ub = user_pinned_.upper_bound(reinterpret_cast<uintptr_t>(dst));
        if (ub != user_pinned_.begin()) {
            --ub;
            const uintptr_t d = reinterpret_cast<uintptr_t>(dst);
            if (d >= ub->first && d - ub->first + bytes <= ub->second) {
                void* dst_dev = nullptr;
                if (copy_by_kernel(m, bytes) &&
                    hipHostGetDevicePointer(&dst_dev, dst, 0) == hipSuccess && dst_dev) {
                    int kr = tpk::launch_copy(p, dst_dev, bytes, compute_);
                    if (kr) return kr;
                } else {
                    HIPCHK(hipMemcpyAsync(dst, p, bytes, hipMemcpyDeviceToHost, compute_));
                }
                d2h_seen_ = true;
                return 0;
            }
        }
        if (d2h_pos_ + bytes > d2h_cap_) {
            if (!pending_d2h_.empty()) {
                // pending copies still point into the old buffer: deliver them first
                HIPCHK(hipStreamSynchronize(compute_));
                for (auto& pd : pending_d2h_) std::memcpy(pd.dst, d2h_stage_ + pd.stage_off, pd.bytes);
                pending_d2h_.clear();
            }
            d2h_pos_ = 0;
            r = ensure_stage(&d2h_stage_, &d2h_cap_, bytes);
            if (r) return r;
        }
        // While a swap-in is running the copy engines hold its queued transfer groups, and a
        // device-to-host copy handed to them would wait for all of those; a copy kernel writing
        // into the pinned buffer goes the other way over the link without queueing behind them.
        void* stage_dev = nullptr;
        if (copy_by_kernel(m, bytes) &&
            hipHostGetDevicePointer(&stage_dev, d2h_stage_, 0) == hipSuccess && stage_dev) {
            int kr = tpk::launch_copy(p, static_cast<uint8_t*>(stage_dev) + d2h_pos_, bytes, compute_);
            if (kr) return kr;
        } else {
            HIPCHK(hipMemcpyAsync(d2h_stage_ + d2h_pos_, p, bytes, hipMemcpyDeviceToHost, compute_));
        }
        pending_d2h_.push_back({dst, d2h_pos_, bytes});
        d2h_pos_ = align_up(d2h_pos_ + bytes, 256);
    }
    d2h_seen_ = true;
    return 0;
}

int Engine::user_host_alloc(uint64_t bytes, void** ptr) {
    std::lock_guard<std::mutex> lk(mu_);
    if (!ptr || bytes == 0) return TP_EINVAL;
    void* p = host_alloc(bytes);
    if (!p) return TP_ENOMEM;
    user_pinned_[reinterpret_cast<uintptr_t>(p)] = bytes;
    *ptr = p;
    return 0;
}

int Engine::user_host_free(void* ptr) {
    std::lock_guard<std::mutex> lk(mu_);
    auto it = user_pinned_.find(reinterpret_cast<uintptr_t>(ptr));
    if (it == user_pinned_.end()) return TP_EINVAL;
    if (!host_only()) (void)hipStreamSynchronize(compute_);  // a result may still be on its way into it
    host_free(ptr);
    user_pinned_.erase(it);
    return 0;
}

// Test hook: the expansion kernel of a packed swap-in on caller-supplied input.  Words outside
// [w_from, w_to) come back as 0xA5A5A5A5.
int Engine::unpack_on_device(const uint8_t* payload, uint64_t n_words, int32_t base, const uint8_t* ext, uint64_t n_ext,
                             const uint32_t* block_tab, uint64_t w_from, uint64_t w_to, uint32_t* words) {
    std::lock_guard<std::mutex> lk(mu_);
    if (host_only()) return TP_ENODEV;
    if (n_words == 0) return 0;
    if (active_ >= 0) return TP_EBUSY;  // the workspace belongs to the running request
    const uint64_t pb = align_up(packed_bytes(n_words), 256), eb = align_up(n_ext + 1, 256),
                   tb = align_up(packed_blocks(n_words) * 4, 256), wb = align_up(n_words * 4 + 4, 256);
    // behind the zero page and the ticket counters at the head of the workspace
    if (cfg_.workspace_bytes < 16384 || pb + eb + tb + wb > cfg_.workspace_bytes - 8192) return TP_EINVAL;
    uint8_t* d_payload = reinterpret_cast<uint8_t*>(workspace_) + 8192;
    uint8_t* d_ext = d_payload + pb;
    uint8_t* d_tab = d_ext + eb;
    uint8_t* d_words = d_tab + tb;
    HIPCHK(hipStreamSynchronize(compute_));
    HIPCHK(hipMemcpy(d_payload, payload, packed_bytes(n_words), hipMemcpyHostToDevice));
    if (n_ext) HIPCHK(hipMemcpy(d_ext, ext, n_ext, hipMemcpyHostToDevice));
    HIPCHK(hipMemcpy(d_tab, block_tab, packed_blocks(n_words) * 4, hipMemcpyHostToDevice));
    HIPCHK(hipMemset(d_words, 0xA5, wb));
    tpk::UnpackArgs a;
    a.n = 1;
    a.piece[0].src = d_payload;
    a.piece[0].dst = d_words;
    a.piece[0].bytes = 0;
    a.piece[0].w_from = w_from;
    a.piece[0].w_to = w_to;
    a.piece[0].w_zero_to = 0;
    a.piece[0].ext = d_ext;
    a.piece[0].tab = reinterpret_cast<const uint32_t*>(d_tab);
    a.piece[0].base = base;
    a.piece[0].first_block = 0;
    int r = tpk::launch_unpack(a, compute_);
    if (r) return r;
    HIPCHK(hipStreamSynchronize(compute_));
    HIPCHK(hipMemcpy(words, d_words, n_words * 4, hipMemcpyDeviceToHost));
    uint32_t guard = 0;  // the word past the end must be untouched (the last group is written word by word)
    HIPCHK(hipMemcpy(&guard, d_words + n_words * 4, 4, hipMemcpyDeviceToHost));
    HIPCHK(hipMemset(reinterpret_cast<uint8_t*>(workspace_) + 8192, 0, pb + eb + tb + wb));
    return guard == 0xA5A5A5A5u ? 0 : TP_EFAULT;
}

int Engine::op_d2h_async(int client, void* dst, uint64_t src, uint64_t bytes) {
    std::lock_guard<std::mutex> lk(mu_);
    int err = 0;
    Model* m = active_model(client, &err);
    if (!m) return err;
    if (mode_ == MODE_LOAD) return TP_ESTATE;
    int r = do_d2h_async(*m, dst, src, bytes);
    if (r) {
        if (!m->async_error) m->async_error = r;
        return r;
    }
    if (mode_ == MODE_TRACK) {
        Op op;
        op.kind = OPK_D2H;
        op.p[0] = src;
        op.i[0] = (int64_t)bytes;
        m->program.push_back(op);
    }
    // cuda_server.hpp:1044: the asynchronous D2H copy is the "request finished" marker
    complete_request();
    return 0;
}

int Engine::op_d2h(int client, void* dst, uint64_t src, uint64_t bytes) {
    std::lock_guard<std::mutex> lk(mu_);
    int err = 0;
    Model* m = active_model(client, &err);
    if (!m) return err;
    if ((!dst && bytes) || bytes > kVaOffMask) return TP_EINVAL;
    void* p = nullptr;
    int r = resolve(*m, src, bytes, false, &p);
    if (r) return r;
    if (host_only()) return TP_ENODEV;
    HIPCHK(hipStreamSynchronize(compute_));
    HIPCHK(hipMemcpy(dst, p, bytes, hipMemcpyDeviceToHost));
    return 0;
}

int Engine::op_d2d(int client, uint64_t dst, uint64_t src, uint64_t bytes) {
    std::lock_guard<std::mutex> lk(mu_);
    int err = 0;
    Model* m = active_model(client, &err);
    if (!m) return err;
    if (bytes > kVaOffMask) return TP_EINVAL;  // before the count is narrowed into the recorded op
    Op op;
    op.kind = OPK_D2D;
    op.p[0] = dst;
    op.p[1] = src;
    op.i[0] = (int64_t)bytes;
    int r = exec_op(*m, op, nullptr, true);
    if (r == 0 && mode_ == MODE_TRACK) m->program.push_back(op);
    if (r && !m->async_error) m->async_error = r;
    return r;
}

int Engine::op_memset(int client, uint64_t dst, int value, uint64_t bytes) {
    std::lock_guard<std::mutex> lk(mu_);
    int err = 0;
    Model* m = active_model(client, &err);
    if (!m) return err;
    if (bytes > kVaOffMask) return TP_EINVAL;
    Op op;
    op.kind = OPK_MEMSET;
    op.p[0] = dst;
    op.i[0] = (int64_t)bytes;
    op.i[1] = value;
    int r = exec_op(*m, op, nullptr, true);
    if (r == 0 && mode_ == MODE_TRACK) m->program.push_back(op);
    if (r && !m->async_error) m->async_error = r;
    return r;
}

int Engine::do_stream_sync(Model* m) {
    int ret = 0;
    if (!host_only()) {
        hipError_t e = hipStreamSynchronize(compute_);
        if (e != hipSuccess) ret = (int)e;
        else synced_seq_ = work_seq_;
        for (auto& pd : pending_d2h_)
            if (!ret) std::memcpy(pd.dst, d2h_stage_ + pd.stage_off, pd.bytes);
    } else if (d2h_seen_) {
        ret = TP_ENODEV;  // no device: there is no data to deliver
    }
    pending_d2h_.clear();
    d2h_pos_ = 0;
    h2d_pos_ = 0;
    d2h_seen_ = false;
    if (m) {
        if (!ret && m->async_error) ret = m->async_error;
        m->async_error = 0;
        if (!host_only() && m->resident && !m->fully_loaded && m->copy_state.load() == CS_ISSUED && m->t1 &&
            hipEventQuery(m->t1) == hipSuccess) {
            m->fully_loaded = true;
            log_transfer(*m);
        }
    }
    return ret;
}

int Engine::op_stream_sync(int client) {
    std::lock_guard<std::mutex> lk(mu_);
    Model* m = find(client);
    return do_stream_sync(m);
}

int Engine::op_device_sync(int client) {
    std::lock_guard<std::mutex> lk(mu_);
    Model* m = find(client);
    int ret = 0;
    if (!host_only()) {
        hipError_t e = hipStreamSynchronize(compute_);
        if (e != hipSuccess) ret = (int)e;
        else synced_seq_ = work_seq_;
    }
    // cuda_server.hpp:959-961: the first device synchronisation after the uploads ends the
    // weight-loading phase; what is allocated from now on is not model memory.
    if (m && client == active_ && mode_ == MODE_LOAD) {
        int r = finish_loading(*m);
        if (r) return r;
        mode_ = MODE_TRACK;
    }
    if (m && !ret && m->async_error) {
        ret = m->async_error;
        m->async_error = 0;
    }
    return ret;
}

// ------------------------------------------------------------------ image layout
// The weight image holds every uploaded tensor, 256 B aligned, in first-access order (tensors
// never touched by the tracked run follow in address order).  The same offsets are used in the
// pinned host store and in HBM, so a swap-in is a sequential copy and a weight address
// translates with one add.  (Reference: per-tensor host allocations and a per-tensor
// virtual->physical map rebuilt on every swap-in, memory_manager.hpp:451-507.)
int Engine::build_image(Model& m, bool by_access) {
    std::vector<size_t> order(m.params.size());
    for (size_t i = 0; i < order.size(); ++i) order[i] = i;
    if (by_access) {
        std::stable_sort(order.begin(), order.end(), [&](size_t a, size_t b) {
            const int ra = m.params[a].access_rank, rb = m.params[b].access_rank;
            if ((ra >= 0) != (rb >= 0)) return ra >= 0;
            // index-looked-up tables after everything the forward pass streams through
            if (m.params[a].gathered != m.params[b].gathered) return !m.params[a].gathered;
            if (ra >= 0 && ra != rb) return ra < rb;
            return m.params[a].voff < m.params[b].voff;
        });
    }
    std::vector<uint64_t> new_off(m.params.size());
    uint64_t off = 0;
    bool same = (m.host_image != nullptr);
    for (size_t k = 0; k < order.size(); ++k) {
        const Param& p = m.params[order[k]];
        new_off[order[k]] = off;
        if (p.image_off != off) same = false;
        off = align_up(off + p.size, kTensorAlign);
    }
    if (same && m.image_bytes == off) return 0;
    uint8_t* img = static_cast<uint8_t*>(host_alloc(off));
    if (!img) return TP_ENOMEM;
    if (off == 0) img[0] = 0;
    parallel_for(m.params.size(), [&](size_t i) {
        const Param& p = m.params[i];
        const uint8_t* src = m.host_image ? m.host_image + p.image_off : m.staging.data() + p.voff;
        std::memcpy(img + new_off[i], src, p.size);
        const uint64_t end = new_off[i] + p.size;  // the alignment gap behind the tensor reads as zeros
        std::memset(img + end, 0, align_up(end, kTensorAlign) - end);
    });
    for (size_t i = 0; i < m.params.size(); ++i) m.params[i].image_off = new_off[i];
    host_free(m.host_image);
    m.host_image = img;
    m.host_image_dev = nullptr;
    if (!host_only()) {
        void* dp = nullptr;
        if (hipHostGetDevicePointer(&dp, img, 0) == hipSuccess) m.host_image_dev = static_cast<uint8_t*>(dp);
        else (void)hipGetLastError();
    }
    m.image_bytes = off;
    return 1;  // image changed
}

// ------------------------------------------------------------------ transfer image
void Engine::free_host_store(Model& m) {
    host_free(m.host_image);
    host_free(m.timg);
    host_free(m.gather_image);
    m.host_image = m.host_image_dev = m.timg = m.gather_image = m.gather_dev = nullptr;
    m.timg_bytes = m.gather_off = m.gather_bytes = 0;
}

void Engine::free_transfer(Model& m) {
    host_free(m.timg);
    m.timg = nullptr;
    m.timg_bytes = 0;
    for (auto& p : m.params) {
        p.pack_base = -1;
        p.t_off = p.tab_off = p.ext_off = 0;
    }
}

// Builds what a swap-in sends over the link (weight_pack.hpp) once the image has its final order.
// Tensors whose words compress go in the packed format, the rest as they are; a model that would
// save under 3 % keeps sending its image directly.
int Engine::build_transfer(Model& m) {
    free_transfer(m);
    m.image_order.resize(m.params.size());
    for (size_t i = 0; i < m.image_order.size(); ++i) m.image_order[i] = (uint32_t)i;
    std::sort(m.image_order.begin(), m.image_order.end(),
              [&](uint32_t a, uint32_t b) { return m.params[a].image_off < m.params[b].image_off; });
    if (!pack_ || host_only() || m.image_bytes == 0 || m.image_bytes >= (16ull << 30)) return 0;
    // A model whose forward pass outlasts its swap-in hides the copy behind compute as it is; the
    // expansion kernels would only compete with its own (measured on MobileNetV2, EfficientNet-B0,
    // DenseNet-169/201: cold equal or up to 0.04 ms slower with the format than without).
    if (m.warm_us > 0 && (double)m.image_bytes / stream_rate_bytes_per_us(1, 32ull << 20) < 0.8 * m.warm_us) return 0;
    std::vector<int32_t> base(m.params.size(), -1);
    std::vector<uint64_t> n_ext(m.params.size(), 0), tab_off(m.params.size(), 0), ext_off(m.params.size(), 0);
    std::vector<uint64_t> t_off(m.params.size(), 0);
    uint64_t off = 0;
    // one histogram pass per tensor picks its window; tensors are independent of each other
    std::vector<uint32_t> win(m.params.size(), 0);
    std::vector<uint64_t> win_out(m.params.size(), 0);
    parallel_for(m.params.size(), [&](size_t i) {
        const Param& p = m.params[i];
        if (p.size % 4 == 0 && p.size >= 4096)
            choose_window(reinterpret_cast<const uint32_t*>(m.host_image + p.image_off), p.size / 4, &win[i], &win_out[i]);
    });
    for (uint32_t idx : m.image_order) {
        const Param& p = m.params[idx];
        t_off[idx] = off;
        if (p.size % 4 == 0 && p.size >= 4096) {
            const uint32_t b = win[idx];
            const uint64_t outside = win_out[idx];
            const uint64_t nw = p.size / 4;
            if (packed_bytes(nw) + packed_blocks(nw) * 4 + outside <= p.size - p.size / 20) {
                // a packed tensor's region: block table, extension stream, payload -- the first two
                // arrive with the tensor's first bytes, whichever transfer group carries them
                base[idx] = (int32_t)b;
                n_ext[idx] = outside;
                tab_off[idx] = off;
                ext_off[idx] = off + packed_blocks(nw) * 4;
                t_off[idx] = align_up(ext_off[idx] + outside, kTensorAlign);
            }
        }
        off = align_up(t_off[idx] + (base[idx] >= 0 ? packed_bytes(p.size / 4) : p.size), kTensorAlign);
    }
    if (off > m.image_bytes - m.image_bytes / 32) return 0;
    if (off > xfer_stage_cap_) {  // registration time: no swap-in may be using the area while it is replaced
        for (auto& kv : models_)
            while (kv.second->copy_state.load(std::memory_order_acquire) == CS_RUNNING) std::this_thread::yield();
        (void)hipStreamSynchronize(copy_);
        (void)hipStreamSynchronize(copy2_);
        (void)hipStreamSynchronize(decode_);
        if (xfer_stage_) (void)hipFree(xfer_stage_);
        xfer_stage_ = nullptr;
        xfer_stage_cap_ = 0;
        const uint64_t cap = align_up(off, 2ull << 20);
        if (hipMalloc(reinterpret_cast<void**>(&xfer_stage_), cap) != hipSuccess) {
            (void)hipGetLastError();
            xfer_stage_ = nullptr;
            return 0;  // no room for a staging area: the image travels as it is
        }
        xfer_stage_cap_ = cap;
    }
    uint8_t* t = static_cast<uint8_t*>(host_alloc(off));
    if (!t) return 0;
    for (uint32_t idx : m.image_order) {
        Param& p = m.params[idx];
        p.t_off = t_off[idx];
        p.pack_base = base[idx];
        p.tab_off = tab_off[idx];
        p.ext_off = ext_off[idx];
    }
    // every tensor fills its own region of the transfer image; whatever lies between regions is zero
    std::atomic<bool> agree{true};
    const bool ran = parallel_for(m.image_order.size(), [&](size_t k) {
        const uint32_t idx = m.image_order[k];
        const Param& p = m.params[idx];
        const uint8_t* src = m.host_image + p.image_off;
        const uint64_t region_beg = p.pack_base >= 0 ? p.tab_off : p.t_off;
        const uint64_t region_end = k + 1 < m.image_order.size()
                                        ? (m.params[m.image_order[k + 1]].pack_base >= 0 ? m.params[m.image_order[k + 1]].tab_off
                                                                                         : m.params[m.image_order[k + 1]].t_off)
                                        : off;
        uint64_t filled_to = region_beg;
        auto zero_to = [&](uint64_t upto) {
            if (upto > filled_to) std::memset(t + filled_to, 0, upto - filled_to);
        };
        if (p.pack_base >= 0) {
            std::vector<uint8_t> ext;
            const uint64_t nw = p.size / 4;
            pack_words(reinterpret_cast<const uint32_t*>(src), nw, (uint32_t)p.pack_base, t + p.t_off, &ext,
                       reinterpret_cast<uint32_t*>(t + p.tab_off));
            if (ext.size() != n_ext[idx]) {  // the two passes disagree: never send a stream that does not decode
                agree.store(false);
                return;
            }
            if (!ext.empty()) std::memcpy(t + p.ext_off, ext.data(), ext.size());
            filled_to = p.ext_off + ext.size();
            zero_to(p.t_off);
            filled_to = p.t_off + packed_bytes(nw);
        } else {
            std::memcpy(t + p.t_off, src, p.size);
            filled_to = p.t_off + p.size;
        }
        zero_to(region_end);
    });
    if (!ran || !agree.load()) {
        host_free(t);
        free_transfer(m);
        return 0;
    }
    m.timg = t;
    m.timg_bytes = off;
    return 1;
}

// Expands the transfer image on the host: every tensor to its place in image_out (image_bytes, zero-filled by
// the caller: the gaps between tensors are zero in the image), or, with image_out == nullptr, compares the
// expansion with `expect` without storing it.  Packed tensors are cut into runs of whole blocks, which expand
// independently of each other (the block table gives each block's place in the extension stream).
bool Engine::decode_transfer(const Model& m, uint8_t* image_out, const uint8_t* expect) {
    if (!m.timg) return false;
    struct Run {
        uint32_t idx;
        uint64_t w0, w1;  // words [w0, w1) of the tensor
    };
    constexpr uint64_t kRunWords = 256 * kPackBlockWords;  // 2 MiB of tensor per work item
    std::vector<Run> runs;
    for (uint32_t idx : m.image_order) {
        const Param& p = m.params[idx];
        const uint64_t nw = p.pack_base >= 0 ? p.size / 4 : 0;
        if (p.pack_base < 0) {
            runs.push_back({idx, 0, 0});
            continue;
        }
        for (uint64_t w = 0; w < nw; w += kRunWords) runs.push_back({idx, w, std::min(nw, w + kRunWords)});
    }
    std::atomic<bool> ok{true};
    const bool ran = parallel_for(runs.size(), [&](size_t k) {
        const Run& r = runs[k];
        const Param& p = m.params[r.idx];
        if (p.pack_base < 0) {
            if (image_out) std::memcpy(image_out + p.image_off, m.timg + p.t_off, p.size);
            else if (std::memcmp(expect + p.image_off, m.timg + p.t_off, p.size) != 0) ok.store(false);
            return;
        }
        const uint32_t* tab = reinterpret_cast<const uint32_t*>(m.timg + p.tab_off);
        const uint64_t ext_total = p.t_off - p.ext_off;  // stream length rounded up to the tensor alignment
        const uint64_t ext_at = tab[r.w0 / kPackBlockWords];
        if (ext_at > ext_total) {
            ok.store(false);
            return;
        }
        const uint64_t n = r.w1 - r.w0;
        const uint8_t* payload = m.timg + p.t_off + (r.w0 / kPackUnitWords) * kPackUnitBytes;
        std::vector<uint32_t> tmp;
        uint32_t* dst;
        if (image_out) {
            dst = reinterpret_cast<uint32_t*>(image_out + p.image_off) + r.w0;
        } else {
            tmp.resize(n);
            dst = tmp.data();
        }
        const uint64_t used = unpack_words(payload, n, (uint32_t)p.pack_base, m.timg + p.ext_off + ext_at,
                                           ext_total - ext_at, dst);
        if (used == UINT64_MAX) {
            ok.store(false);
            return;
        }
        if (!image_out && std::memcmp(expect + p.image_off + r.w0 * 4, dst, n * 4) != 0) ok.store(false);
    });
    return ran && ok.load();
}

// The transfer image becomes the host store.  It is first expanded on the host and compared with the image,
// word for word; only then is the image released (a mismatch keeps the image and drops the transfer image:
// the model then travels as it is).  The tables that lookups read in place while a swap-in is under way keep
// a raw pinned copy.  Pinned host memory per packed model: 0.85x the image (+ its tables) instead of 1.85x.
int Engine::slim_host_store(Model& m) {
    if (!m.timg || !m.host_image) return 0;
    if (!decode_transfer(m, nullptr, m.host_image)) {
        log_.write(ExecLog::ERR, "Register model %d: the transfer image does not decode back to the image; sent as it is", m.id);
        free_transfer(m);
        return 0;
    }
    uint64_t table_off = UINT64_MAX;
    for (const Param& p : m.params)
        if (p.gathered) table_off = std::min(table_off, p.image_off);
    if (host_gather_ && table_off != UINT64_MAX) {
        const uint64_t n = m.image_bytes - table_off;
        uint8_t* g = static_cast<uint8_t*>(host_alloc(n));
        if (!g) return 0;  // keep the image
        std::memcpy(g, m.host_image + table_off, n);
        void* dp = nullptr;
        if (hipHostGetDevicePointer(&dp, g, 0) != hipSuccess) {
            (void)hipGetLastError();
            host_free(g);
            return 0;
        }
        m.gather_image = g;
        m.gather_dev = static_cast<uint8_t*>(dp);
        m.gather_off = table_off;
        m.gather_bytes = n;
    }
    host_free(m.host_image);
    m.host_image = nullptr;
    m.host_image_dev = nullptr;
    return 1;
}

// Where image offset d (a multiple of the tensor alignment) lies in the transfer image.
uint64_t Engine::xfer_off(const Model& m, uint64_t d) const {
    size_t lo = 0, hi = m.image_order.size();
    while (lo < hi) {
        const size_t mid = (lo + hi) / 2;
        if (m.params[m.image_order[mid]].image_off <= d) lo = mid + 1;
        else hi = mid;
    }
    if (lo == 0) return 0;
    const Param& p = m.params[m.image_order[lo - 1]];
    const uint64_t rel = d - p.image_off;
    auto region = [](const Param& q) { return q.pack_base >= 0 ? q.tab_off : q.t_off; };
    if (rel >= p.size) return lo < m.image_order.size() ? region(m.params[m.image_order[lo]]) : m.timg_bytes;
    if (rel == 0) return region(p);
    return p.t_off + (p.pack_base >= 0 ? rel / 256 * kPackUnitBytes : rel);
}

// The copy thread times every runtime call of a swap-in's hand-over and keeps the slowest: the link paces
// a swap-in unless one of these calls stalls on the host (tp_swap_stats.max_call_*).
namespace {
thread_local Model* t_timed = nullptr;
enum : uint32_t { CALL_COPY = 0, CALL_RECORD = 1, CALL_WAIT = 2, CALL_EXPAND = 3 };
template <class F>
inline auto timed_call(uint32_t group, uint32_t kind, F&& f) -> decltype(f()) {
    if (!t_timed) return f();
    const auto t0 = Clock::now();
    const auto r = f();
    const double us = us_since(t0);
    if (us > t_timed->max_call_us) {
        t_timed->max_call_us = us;
        t_timed->max_call_group = group;
        t_timed->max_call_kind = kind;
    }
    return r;
}
}  // namespace

// One transfer group of a packed swap-in: DMA into the staging area, then, on the expansion stream,
// every tensor run of the group into its place, the out-of-window words patched, the group published.
int Engine::copy_chunk_packed(Model& m, size_t i, uint64_t beg, uint64_t end, hipStream_t cs, bool do_dma,
                              bool do_expand) {
    if (do_dma) {
        const uint64_t tb = i == 0 ? 0 : xfer_off(m, beg);
        const uint64_t te = end >= m.image_bytes ? m.timg_bytes : xfer_off(m, end);
        if (te < tb || te > xfer_stage_cap_) return TP_EFAULT;
        hipError_t e = hipSuccess;
        if (te > tb)
            e = timed_call((uint32_t)i, CALL_COPY,
                           [&] { return hipMemcpyAsync(xfer_stage_ + tb, m.timg + tb, te - tb, hipMemcpyHostToDevice, cs); });
        if (e == hipSuccess) e = timed_call((uint32_t)i, CALL_RECORD, [&] { return hipEventRecord(m.dma_ev[i], cs); });
        if (e != hipSuccess) return (int)e;
    }
    if (!do_expand) return 0;
    hipError_t e = timed_call((uint32_t)i, CALL_WAIT, [&] { return hipStreamWaitEvent(decode_, m.dma_ev[i], 0); });
    if (e != hipSuccess) return (int)e;
    size_t lo = 0, hi = m.image_order.size();
    while (lo < hi) {
        const size_t mid = (lo + hi) / 2;
        if (m.params[m.image_order[mid]].image_off <= beg) lo = mid + 1;
        else hi = mid;
    }
    tpk::UnpackArgs a;
    int r = 0;
    for (size_t k = lo ? lo - 1 : 0; k < m.image_order.size() && !r; ++k) {
        const Param& p = m.params[m.image_order[k]];
        if (p.image_off >= end) break;
        const uint64_t from = std::max(beg, p.image_off), to = std::min(end, p.image_off + p.size);
        if (to <= from) continue;
        tpk::UnpackPiece& pc = a.piece[a.n++];
        pc.base = p.pack_base;
        pc.first_block = 0;
        if (p.pack_base >= 0) {
            pc.src = xfer_stage_ + p.t_off;
            pc.dst = m.w_dev + p.image_off;
            pc.bytes = 0;
            pc.w_from = (from - p.image_off) / 4;
            pc.w_to = (to - p.image_off) / 4;
            // The image keeps every tensor 256 B aligned and the host copy holds zeros in the gaps; the
            // pool memory a swap-in lands in holds whatever its previous tenant left.  The run that
            // delivers a tensor's last word clears the gap behind it, so that the device image equals the
            // host image byte for byte wherever it is placed.
            pc.w_zero_to = (to == p.image_off + p.size) ? align_up(p.size, kTensorAlign) / 4 : 0;
            if (pc.w_zero_to == pc.w_to) pc.w_zero_to = 0;
            pc.ext = xfer_stage_ + p.ext_off;
            pc.tab = reinterpret_cast<const uint32_t*>(xfer_stage_ + p.tab_off);
        } else {
            pc.src = xfer_stage_ + p.t_off + (from - p.image_off);
            pc.dst = m.w_dev + from;
            // a run that ends the tensor takes the zeros behind it along (the transfer image holds zeros
            // up to the next tensor's region, which starts no earlier than the aligned end)
            pc.bytes = (to == p.image_off + p.size ? align_up(p.image_off + p.size, kTensorAlign) : to) - from;
            pc.w_from = pc.w_to = 0;
            pc.w_zero_to = 0;
            pc.ext = nullptr;
            pc.tab = nullptr;
        }
        if (a.n == tpk::kUnpackMaxPieces) {
            r = timed_call((uint32_t)i, CALL_EXPAND, [&] { return tpk::launch_unpack(a, decode_); });
            a.n = 0;
        }
    }
    if (!r && a.n) r = timed_call((uint32_t)i, CALL_EXPAND, [&] { return tpk::launch_unpack(a, decode_); });
    if (r) return r;
    return (int)timed_call((uint32_t)i, CALL_RECORD, [&] { return hipEventRecord(m.chunk_ev[i], decode_); });
}

// One copy stream or two.  Measured on MI355X: a single stream loses ~15 us of DMA set-up per
// hipMemcpyAsync (51 GB/s at 8 MiB groups, 55 GB/s at 32 MiB, of a 57 GB/s link); alternating
// the groups over two streams hides that (56-57 GB/s at any group size) but every compute
// kernel dispatched while DMA queues are active starts ~1.2 us later per active queue.  So a
// model whose forward pass takes about as long as its swap-in is better off with one stream and
// large groups, and a link-bound model with two streams.  The forward time is the best warm
// replay seen so far, or an estimate from the recorded op stream before the first one.
void Engine::choose_copy_plan(Model& m) {
    double compute_us = m.warm_us;
    double kernels = 0;
    double est = 0;
    for (const Op& op : m.program) {
        if (op.kind != OPK_GEMM && op.kind != OPK_CONV && op.kind != OPK_BN && op.kind != OPK_LAUNCH) continue;
        double flops, bytes;
        const char* name;
        op_work(op, &flops, &bytes, &name);
        // only used before the first timed forward pass exists (an engine without a device): 50 TFLOP/s, 2 TB/s, 6 us floor
        est += std::max(6.0, std::max(flops / 5.0e7, bytes / 2.0e6));
        kernels += (op.kind == OPK_GEMM || op.kind == OPK_CONV) ? 1.5 : 1.0;
    }
    if (compute_us <= 0) compute_us = est;
    const double bytes = (double)(m.timg ? m.timg_bytes : m.image_bytes);  // what crosses the link
    // Rates follow the link this engine measured (init, tp_measure_h2d), not a figure of the box they were
    // tuned on: two streams hide each copy's fixed cost and deliver about 99 % of it; one stream pays the fixed
    // cost once per group (its groups grow to 32 MiB).
    const double t1 = std::max(bytes / stream_rate_bytes_per_us(1, 32ull << 20), compute_us + kernels * 1.2);
    // (measured on ResNet-152 batch 8: kernels that share the device with two copy streams run
    // about 15 % longer, on top of the per-launch cost)
    const double t2 = std::max(bytes / stream_rate_bytes_per_us(2, 16ull << 20), compute_us * 1.15 + kernels * 2.4);
    m.ncopy = (t2 <= t1) ? 2 : 1;
    // The estimate's constants (what a busy copy queue costs a launch, how much slower kernels run beside two of
    // them) were fitted to the kernels of their day and were off by 5 % in opposite directions for ResNet-152
    // batch 8 once its forward pass had become faster (estimated 3.68 / 3.96 ms for one / two streams, measured
    // 3.98 / 3.82).  Where the two estimates are within a quarter of each other the model's own cold requests
    // decide instead: the first plan_trials_ of them run under the estimated plan, the next plan_trials_ under
    // the other one, and from then on the plan whose best request was shorter is kept.
    if (plan_trials_ > 0 && std::max(t1, t2) < 1.25 * std::min(t1, t2)) {
        const int a = m.ncopy, b = 3 - a;
        if (m.cold_n[a] >= plan_trials_) {
            if (m.cold_n[b] < plan_trials_) m.ncopy = b;
            else if (m.cold_us[b] < 0.99 * m.cold_us[a]) m.ncopy = b;
        }
    }
    if (copy_streams_cfg_ == 1 || copy_streams_cfg_ == 2) m.ncopy = copy_streams_cfg_;
    m.chunk_max = cfg_.chunk_max_bytes;
    if (chunk_max_auto_ && m.ncopy == 1) m.chunk_max = std::max<uint64_t>(cfg_.chunk_max_bytes, 32ull << 20);
    // Two streams: 16 MiB.  Groups of 8 MiB left a whole swap-in of BERT-large in one of two modes from one
    // process to the next (56.1 or 55.2 GB/s, cold 18.84 or 19.09 ms); with 16 MiB all of 5 fresh processes ran
    // 56.3 GB/s and 18.66-18.69 ms.  The size in the middle of the image costs a link-bound request nothing,
    // since the groups shrink again towards the end (build_chunks); 32 MiB was no faster and worse for ResNet-50.
    if (chunk_max_auto_ && m.ncopy == 2) m.chunk_max = std::max<uint64_t>(cfg_.chunk_max_bytes, 16ull << 20);
}

// Sustained swap-in rate, in bytes per microsecond, of `streams` copy streams moving groups of `group`
// bytes over the measured link.  Every hipMemcpyAsync carries a fixed cost (kCopyFixedUs, measured: 51 GB/s
// at 8 MiB and 55 GB/s at 32 MiB groups on one stream of a 57 GB/s link); one stream pays it per group,
// two streams overlap it with the other stream's transfer and lose about 1 %.
double Engine::stream_rate_bytes_per_us(int streams, uint64_t group) const {
    const double link = link_gbps_ * 1.0e3;  // bytes per microsecond
    if (streams >= 2) return 0.99 * link;
    const double g = (double)group;
    return g / (g / link + kCopyFixedUs);
}

// Transfer groups: the first is chunk_bytes, each next one doubles up to chunk_max_bytes, so the
// first layers can start after a short copy while the bulk moves in DMA-efficient pieces.
// (Reference: fixed >= BUFFER_SIZE groups, memory_manager.hpp:399-409.)
void Engine::build_chunks(Model& m) {
    choose_copy_plan(m);
    m.chunk_end.clear();
    uint64_t sz = cfg_.chunk_bytes, pos = 0;
    if (per_tensor_groups_) {
        // memory_manager.hpp:399-409 with BUFFER_SIZE=1: a group closes behind every tensor
        std::vector<uint64_t> ends;
        ends.reserve(m.params.size());
        for (const Param& p : m.params) ends.push_back(align_up(p.image_off + p.size, kTensorAlign));
        std::sort(ends.begin(), ends.end());
        for (uint64_t e : ends)
            if (e > pos) {
                m.chunk_end.push_back(e);
                pos = e;
            }
        if (pos < m.image_bytes) m.chunk_end.push_back(m.image_bytes);
        pos = m.image_bytes;
    }
    // Where the part of the image ends that a request streams through (tables looked up by index lie behind it).
    uint64_t table_off = UINT64_MAX;
    for (const Param& p : m.params)
        if (p.gathered) table_off = std::min(table_off, p.image_off);
    const uint64_t streamed_end = (host_gather_ && table_off != UINT64_MAX) ? table_off : m.image_bytes;
    // The last layers cannot start before their group has landed whole, so the time the last group spends on
    // the link is added to a cold request that the link paces.  With two copy streams (the link-bound models)
    // the groups therefore shrink again towards the end of the streamed part: none is larger than half of what
    // is left, down to the first group's size (BERT-base batch 1 cold 5.35 -> 5.30 ms, BERT-large 18.95 ->
    // 18.89 ms).  With one stream every extra copy costs link time and the request ends 0.07 ms after the last
    // byte anyway (ResNet-152 batch 8: 3.98 -> 4.01 ms tapered), so those keep full groups.  TORPOR_TAPER=0 /
    // =2: never / always.
    static const uint64_t taper_mode = env_u64("TORPOR_TAPER", 1);
    const bool taper = taper_mode == 2 || (taper_mode == 1 && m.ncopy == 2);
    const uint64_t cmin = align_up(std::max<uint64_t>(cfg_.chunk_bytes, kTensorAlign), kTensorAlign);
    while (pos < m.image_bytes) {
        uint64_t g = align_up(sz, kTensorAlign);
        uint64_t limit = m.image_bytes;
        if (taper && !per_tensor_groups_ && pos < streamed_end) {
            g = std::min(g, std::max(cmin, align_up((streamed_end - pos) / 2, kTensorAlign)));
            limit = streamed_end;
        }
        uint64_t end = (g > limit - pos) ? limit : pos + g;
        m.chunk_end.push_back(end);
        pos = end;
        if (sz < m.chunk_max) sz = std::min(sz * 2, m.chunk_max);
    }
    // first group that holds nothing but tables looked up by index (they are last in the image)
    m.defer_from = UINT32_MAX;
    if (host_gather_ && table_off != UINT64_MAX)
        for (size_t i = 0; i < m.chunk_end.size(); ++i)
            if ((i ? m.chunk_end[i - 1] : 0) >= table_off) {
                m.defer_from = (uint32_t)i;
                break;
            }
    if (!host_only()) {
        while (m.chunk_ev.size() < m.chunk_end.size()) {
            hipEvent_t ev = nullptr;
            if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) break;
            m.chunk_ev.push_back(ev);
        }
        while (m.timg && m.dma_ev.size() < m.chunk_end.size()) {
            hipEvent_t ev = nullptr;
            if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) break;
            m.dma_ev.push_back(ev);
        }
        if (!m.t0) (void)hipEventCreate(&m.t0);
        if (!m.t1) (void)hipEventCreate(&m.t1);
    }
}

int Engine::finish_loading(Model& m) {
    std::sort(m.params.begin(), m.params.end(), [](const Param& a, const Param& b) { return a.voff < b.voff; });
    for (size_t i = 1; i < m.params.size(); ++i)
        if (m.params[i - 1].voff + m.params[i - 1].size > m.params[i].voff) return TP_EINVAL;  // overlapping uploads
    m.param_bytes = 0;
    for (auto& p : m.params) m.param_bytes += p.size;
    int r = build_image(m, false);
    if (r < 0) return r;
    m.staging.release();
    // cold start leaves the weights on the device (memory_manager.hpp:141), so the tracked
    // inference runs with a resident model
    m.w_pool_off = pool_.alloc(m.image_bytes);
    if (m.w_pool_off == UINT64_MAX) return TP_ENOMEM;
    m.w_dev = arena_ + m.w_pool_off;
    if (!host_only() && m.image_bytes) HIPCHK(hipMemcpy(m.w_dev, m.host_image, m.image_bytes, hipMemcpyHostToDevice));
    m.resident = true;
    m.fully_loaded = true;
    m.state = MS_TRACKING;
    return 0;
}

int Engine::finish_tracking(Model& m) {
    TraceRange trace("register: lay out and pack model", m.id);
    auto t_phase = Clock::now();
    auto phase = [&](const char* what) {  // debug level: where a registration's time goes
        log_.write(ExecLog::DEBUG, "Register model %d: %s elasped %.0f us", m.id, what, us_since(t_phase));
        t_phase = Clock::now();
    };
    // memory_manager.hpp:73-80 unset_track_model_memory + the layout step described above
    int r = build_image(m, true);
    if (r < 0) return r;
    phase("image in access order");
    if (r == 1 && !host_only() && m.image_bytes)
        HIPCHK(hipMemcpy(m.w_dev, m.host_image, m.image_bytes, hipMemcpyHostToDevice));
    phase("upload of the re-ordered image");
    build_chunks(m);
    // fold the per-allocation activation extents of the tracked run into one arena
    if (!host_only()) HIPCHK(hipStreamSynchronize(compute_));
    for (auto& kv : m.ablocks) {
        if (kv.second.pool_off != UINT64_MAX) pool_.release(kv.second.pool_off);
        kv.second.pool_off = UINT64_MAX;
    }
    m.act_bytes = m.abump;
    m.act_frozen = true;
    m.a_pool_off = pool_.alloc(m.act_bytes);
    if (m.a_pool_off == UINT64_MAX) return TP_ENOMEM;
    m.a_dev = arena_ + m.a_pool_off;
    m.state = MS_READY;
    // Forward-pass time for the swap-in plan: re-issue the recorded compute ops (not the copies)
    // on whatever the arena holds and time the second pass.  Activations only; weights untouched.
    if (!host_only()) {
        const int saved_mode = mode_;
        mode_ = MODE_EXEC;
        for (int pass = 0; pass < 2; ++pass) {
            const auto t0 = Clock::now();
            for (const Op& op : m.program)
                if (op.kind == OPK_GEMM || op.kind == OPK_CONV || op.kind == OPK_BN || op.kind == OPK_LAUNCH)
                    (void)exec_compute_impl(m, op, true);
            (void)hipStreamSynchronize(compute_);
            if (pass == 1) m.warm_us = us_since(t0);
        }
        mode_ = saved_mode;
        phase("two timed forward passes");
        r = build_transfer(m);  // needs the forward time: only a link-bound model gains from fewer bytes
        if (r < 0) return r;
        phase("transfer image");
        if (r == 1 && slim_host_) {
            r = slim_host_store(m);
            if (r < 0) return r;
            phase("transfer image decoded and compared, raw image released");
        }
        build_chunks(m);
    }
    return 0;
}

// ------------------------------------------------------------------ swap engine
void Engine::copy_main() {
    (void)hipSetDevice(cfg_.device);
    for (;;) {
        Model* m = nullptr;
        {
            std::unique_lock<std::mutex> lk(cmu_);
            ccv_.wait(lk, [&] { return stop_ || !jobs_.empty(); });
            if (stop_) return;
            m = jobs_.front();
            jobs_.pop_front();
        }
        // memory_manager.hpp:378-409: walk the tensors in access order, one DMA per group, and
        // publish each group.  Publishing is an event record, not a host synchronisation.
        int err = 0;
        TraceRange trace("swap-in: issue copies of model", m->id);
        const auto t_issue = Clock::now();
        m->max_call_us = 0;
        m->max_call_group = m->max_call_kind = 0;
        t_timed = m;  // every runtime call of the hand-over is timed (timed_call)
        if (!m->cancel.load()) {
            if (m->timg && stage_used_) {  // the staging area is shared: the previous expansion must be done with it
                (void)hipStreamWaitEvent(copy_, stage_free_ev_, 0);
                (void)hipStreamWaitEvent(copy2_, stage_free_ev_, 0);
            }
            hipError_t e = hipEventRecord(m->t0, copy_);
            if (e != hipSuccess) err = (int)e;
            // A group is handed over in two steps: its DMA (and, sent as it is, its event), then --
            // for a packed transfer -- its expansion and event on the expansion stream.
            auto dma = [&](size_t i, uint64_t beg, uint64_t end) -> int {
                // alternate streams so that one group's DMA set-up hides behind the other's transfer
                hipStream_t cs = (m->ncopy == 2 && (i & 1)) ? copy2_ : copy_;
                // The link is not shared evenly between two streams and one may run several groups
                // ahead.  Its first group of deferred tables waits for the other stream's last group
                // of streamed tensors, so that the stream that lags gets the whole link for those.
                if (m->ncopy == 2 && (i == m->defer_from || i == m->defer_from + 1) && i >= 2)
                    (void)hipStreamWaitEvent(cs, (m->timg ? m->dma_ev : m->chunk_ev)[i == m->defer_from ? i - 1 : i - 2], 0);
                if (m->timg) return copy_chunk_packed(*m, i, beg, end, cs, /*dma=*/true, /*expand=*/false);
                hipError_t e = timed_call((uint32_t)i, CALL_COPY, [&] {
                    return hipMemcpyAsync(m->w_dev + beg, m->host_image + beg, end - beg, hipMemcpyHostToDevice, cs);
                });
                if (e == hipSuccess) e = timed_call((uint32_t)i, CALL_RECORD, [&] { return hipEventRecord(m->chunk_ev[i], cs); });
                return (int)e;
            };
            auto publish = [&](size_t i, uint64_t beg, uint64_t end) -> int {
                int r = m->timg ? copy_chunk_packed(*m, i, beg, end, nullptr, false, true) : 0;
                if (!r) m->issued.store((uint32_t)i + 1, std::memory_order_release);
                return r;
            };
            const size_t n_groups = m->chunk_end.size();
            size_t i = 0;
            uint64_t beg = 0;
            // With two streams the first two DMAs go out back to back, before anything else is
            // submitted.  Measured: when the second stream's first copy is submitted while the first
            // stream's is already moving (25 us later), the whole swap-in runs at 52.5 GB/s instead of
            // 56.5 GB/s; submitted together, both streams settle into the faster pattern.
            if (m->ncopy == 2 && n_groups >= 2 && !err && !m->cancel.load()) {
                const uint64_t e0 = m->chunk_end[0], e1 = m->chunk_end[1];
                err = dma(0, 0, e0);
                if (!err) err = dma(1, e0, e1);
                if (!err) err = publish(0, 0, e0);
                if (!err) err = publish(1, e0, e1);
                i = 2;
                beg = e1;
            }
            for (; i < n_groups && !err; ++i) {
                if (m->cancel.load()) break;
                const uint64_t end = m->chunk_end[i];
                err = dma(i, beg, end);
                if (!err) err = publish(i, beg, end);
                beg = end;
            }
            if (m->timg) {
                (void)hipEventRecord(stage_free_ev_, decode_);
                stage_used_ = true;
                if (!err) (void)hipEventRecord(m->t1, decode_);  // the expansions follow the groups in order
            } else if (!err) {
                const size_t n = m->chunk_end.size();
                if (m->ncopy == 2 && n >= 2) {  // t1 = both streams drained
                    const size_t last_odd = (n - 1) & 1 ? n - 1 : n - 2;
                    (void)hipStreamWaitEvent(copy_, m->chunk_ev[last_odd], 0);
                }
                (void)hipEventRecord(m->t1, copy_);
            }
        }
        t_timed = nullptr;
        m->issue_ms = us_since(t_issue) / 1000.0;
        if (err) m->copy_error.store(err);
        m->copy_state.store(CS_ISSUED, std::memory_order_release);
    }
}

// memory_manager.hpp:425-431: one line per finished swap-in, written when the engine first learns that
// the last group has landed (a later synchronisation of the model, or its swap-out).
void Engine::log_transfer(Model& m) {
    if (!log_.on(ExecLog::INFO) || m.transfer_logged || host_only() || !m.timing_valid || !m.t0 || !m.t1) return;
    if (m.cancel.load() || m.copy_error.load() || m.copy_state.load(std::memory_order_acquire) != CS_ISSUED) return;
    if (hipEventQuery(m.t1) != hipSuccess) return;
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, m.t0, m.t1) != hipSuccess) return;
    m.transfer_logged = true;
    log_.write(ExecLog::INFO, "Transfer model %d: %llu bytes over the link in %u groups on %d streams, overall elasped %.0f us",
               m.id, (unsigned long long)m.stats.bytes, m.stats.chunks, m.ncopy, ms * 1e3);
}

// Waits until nothing of this model's swap-in is on its way any more: a hand-over still running is
// cancelled, and the groups that were handed to the streams are waited for by their own events.  Copies
// of other models are left alone: an eviction during another model's swap-in (a Load signal while requests
// run, a request that finds the budget full) must not stall the executor for the rest of that swap-in.
void Engine::wait_copy_idle(Model& m) {
    if (host_only()) return;
    const int st0 = m.copy_state.load(std::memory_order_acquire);
    if (st0 == CS_IDLE) {  // resident since registration: no copy of it was ever queued
        if (last_swap_ == &m) last_swap_ = nullptr;
        return;
    }
    if (st0 == CS_RUNNING) {
        m.cancel.store(true);
        while (m.copy_state.load(std::memory_order_acquire) == CS_RUNNING) std::this_thread::yield();
    }
    const uint32_t n = m.issued.load(std::memory_order_acquire);
    bool ok = true;
    // transfer groups publish in order on the expansion stream (packed) or alternate over the copy streams
    for (uint32_t back = 1; back <= 2 && back <= n && ok; ++back)
        if (n - back < m.chunk_ev.size()) ok = hipEventSynchronize(m.chunk_ev[n - back]) == hipSuccess;
    // a packed group's DMA precedes its expansion; one that was handed over but not yet expanded cannot exist
    // (the copy thread hands over DMA and expansion of a group together), and a cancelled hand-over stops
    // between groups.  Anything unexpected: fall back to draining the streams.
    if (!ok || m.copy_error.load()) {
        (void)hipGetLastError();
        (void)hipStreamSynchronize(copy_);
        (void)hipStreamSynchronize(copy2_);
        (void)hipStreamSynchronize(decode_);
    }
    if (last_swap_ == &m) last_swap_ = nullptr;
}

// Is a swap-in (of any model) still using the copy engines?  Asked without waiting.  Swap-ins are handed to
// the streams one after the other, so the one started last finishes last.
bool Engine::swap_in_flight() {
    Model* m = last_swap_;
    if (!m || host_only()) return false;
    const int st = m->copy_state.load(std::memory_order_acquire);
    if (st == CS_RUNNING) return true;
    if (st == CS_ISSUED && !m->cancel.load() && !m->copy_error.load() && m->t1 && hipEventQuery(m->t1) == hipErrorNotReady)
        return true;
    (void)hipGetLastError();
    last_swap_ = nullptr;
    return false;
}

// memory_manager.hpp:213-227 sig_trans_thread + 451-507 check_and_malloc_model
int Engine::swap_in(Model& m) {
    if (m.resident) return 0;
    TraceRange trace("swap-in: allocate model", m.id);
    const auto t0 = Clock::now();
    m.swap_t0 = t0;
    auto try_alloc = [&]() -> bool {
        m.w_pool_off = pool_.alloc(m.image_bytes);
        if (m.w_pool_off == UINT64_MAX) return false;
        m.a_pool_off = pool_.alloc(m.act_bytes);
        if (m.a_pool_off == UINT64_MAX) {
            pool_.release(m.w_pool_off);
            m.w_pool_off = UINT64_MAX;
            return false;
        }
        return true;
    };
    while (!try_alloc()) {
        // The budget test passed but no contiguous extent fits: keep evicting in LRU order.
        // (The reference exits the process here, block_manager.hpp:345-351.)
        std::string victim;
        if (!lru_.peek_victim(std::to_string(m.id), &victim)) return TP_ENOMEM;
        lru_.force_evict(victim);
        Model* v = find(std::atoi(victim.c_str()));
        if (v) evict_model(*v);
        ++frag_evictions_;
    }
    m.w_dev = arena_ + m.w_pool_off;
    m.a_dev = arena_ + m.a_pool_off;
    drop_graph(m);  // the captured launches hold the old addresses
    build_chunks(m);  // the plan follows the latest forward-time figure
    m.resident = true;
    m.fully_loaded = false;
    m.gated_upto = 0;
    m.issued.store(0);
    m.cancel.store(false);
    m.copy_error.store(0);
    m.transfer_logged = false;
    m.stats.alloc_us = us_since(t0);
    m.stats.bytes = m.timg ? m.timg_bytes : m.image_bytes;
    m.stats.deferred_bytes = 0;
    if (m.defer_from != UINT32_MAX && m.defer_from > 0 && m.defer_from < m.chunk_end.size()) {
        const uint64_t from = m.chunk_end[m.defer_from - 1];
        m.stats.deferred_bytes = m.timg ? m.timg_bytes - xfer_off(m, from) : m.image_bytes - from;
    }
    m.stats.chunks = (uint32_t)m.chunk_end.size();
    m.stats.copy_streams = (uint32_t)m.ncopy;
    ++swap_ins_;
    log_.write(ExecLog::INFO, "CheckMalloc model %d elasped %.0f us (%llu weight + %llu activation bytes)", m.id,
               m.stats.alloc_us, (unsigned long long)m.image_bytes, (unsigned long long)m.act_bytes);
    if (host_only() || m.image_bytes == 0) {
        m.fully_loaded = true;
        return 0;
    }
    m.timing_valid = true;
    m.copy_state.store(CS_RUNNING, std::memory_order_release);
    last_swap_ = &m;
    {
        std::lock_guard<std::mutex> lk(cmu_);
        jobs_.push_back(&m);
    }
    ccv_.notify_one();
    return 0;
}

// memory_manager.hpp:240-259: metadata only, the host copy stays authoritative.
void Engine::evict_model(Model& m) {
    if (!m.resident) return;
    TraceRange trace("swap-out model", m.id);
    const auto t0 = Clock::now();
    const bool was_running = m.copy_state.load(std::memory_order_acquire) == CS_RUNNING;
    wait_copy_idle(m);
    if (!was_running) log_transfer(m);
    // A request counts as finished once its result copy is queued (cuda_server.hpp:1044), so the
    // model's last kernels may still be running: its memory is not handed on before they are done.
    if (!host_only() && m.touch_seq > synced_seq_ && hipStreamSynchronize(compute_) == hipSuccess)
        synced_seq_ = work_seq_;
    if (m.w_pool_off != UINT64_MAX) pool_.release(m.w_pool_off);
    if (m.a_pool_off != UINT64_MAX) pool_.release(m.a_pool_off);
    m.w_pool_off = m.a_pool_off = UINT64_MAX;
    m.w_dev = m.a_dev = nullptr;
    drop_graph(m);
    m.resident = false;
    m.fully_loaded = false;
    m.copy_state.store(CS_IDLE);
    m.stats.evict_us = us_since(t0);
    ++evictions_;
    log_.write(ExecLog::INFO, "Evict model %d elasped %.0f us", m.id, m.stats.evict_us);
}

// controller.hpp:392-400
bool Engine::check_eviction(Model& m) {
    bool over = false;
    auto victims = lru_.check_and_add(std::to_string(m.id), m.total_bytes(), m.level, &over);
    for (auto& v : victims) {
        Model* vm = find(std::atoi(v.c_str()));
        if (vm) evict_model(*vm);
    }
    return !over;
}

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

// ------------------------------------------------------------------ compute ops
static tpk::EpilogueArgs ep_from(const Op& op, void* const* q, int pbase, int fbase, int ibase) {
    tpk::EpilogueArgs e;
    e.alpha = op.f[fbase + 0];
    e.beta = op.f[fbase + 1];
    e.bn_eps = op.f[fbase + 2];
    e.bias = static_cast<const float*>(q[pbase + 0]);
    e.bn_scale = static_cast<const float*>(q[pbase + 1]);
    e.bn_bias = static_cast<const float*>(q[pbase + 2]);
    e.bn_mean = static_cast<const float*>(q[pbase + 3]);
    e.bn_var = static_cast<const float*>(q[pbase + 4]);
    e.residual = static_cast<const float*>(q[pbase + 5]);
    e.ldr = op.i[ibase + 0];
    e.act = (int)op.i[ibase + 1];
    return e;
}

// Layout of Op for the compute kinds (filled by the C-ABI layer):
//  GEMM  p: x y c bias bns bnb bnm bnv res   i: m n k xs_r xs_k ys_c ys_k ldc nb0 nb1 xb0 xb1 yb0 yb1 cb0 cb1 ldr act
//        f: alpha beta eps
//  CONV  p: x w y bias bns bnb bnm bnv res   i: n h w cin cout kh kw sh sw ph pw xl yl ldr act   f: alpha beta eps
//  BN    p: x y g b mean var                 i: rows C hw layout relu   f: eps
//  LAUNCH p/i/f per op id (see torpor_amd.h)
int Engine::exec_compute_impl(Model& m, const Op& op, bool launch) {
    void* q[12] = {nullptr};
    // The scratch allocation: 256 bytes that stay zero for good (padding source of the 3x3
    // convolution), the ticket counters of split K ranges (zero between launches), then the partial
    // sums.  No device workspace in host-only mode (nothing is launched there).
    constexpr size_t kHead = 256 + tpk::kSplitTickets * sizeof(unsigned);
    const tpk::Workspace ws = workspace_ ? tpk::Workspace{workspace_ + kHead / 4, (size_t)cfg_.workspace_bytes - kHead, workspace_,
                                                           reinterpret_cast<unsigned*>(workspace_ + 64)}
                                        : tpk::Workspace{};
    // Every operand is translated together with the byte span the kernel will touch, so an op
    // whose shapes do not fit its buffers is refused on the host instead of faulting the GPU.
    // Spans are computed in 128-bit integers from arguments that have been range-checked first
    // (anything a launcher narrows to int: at most INT32_MAX; counts, strides and pitches: at most
    // the size of an address region), so that no product can wrap into a span that passes.
    using i128 = __int128;
    constexpr int64_t kIntMax = 0x7fffffff;
    constexpr int64_t kLongMax = (int64_t)kVaOffMask;
    auto R = [&](int idx, bool optional, i128 elems, int elem_size = 4) -> int {
        if (elems < 1) elems = 1;
        if (elems > (i128)kLongMax) return TP_EFAULT;  // no block is that large
        return resolve(m, op.p[idx], (uint64_t)elems * (uint64_t)elem_size, optional, &q[idx]);
    };
    i128 I[20];
    for (int k = 0; k < 20; ++k) I[k] = k < op.ni ? (i128)op.i[k] : (i128)0;
    // arguments whose bit is set in long_mask may be as large as an address region, the others fit an int
    auto ranges_ok = [&](uint32_t long_mask) {
        for (int k = 0; k < op.ni && k < 20; ++k) {
            if (op.i[k] < 0) return false;
            if (op.i[k] > (((long_mask >> k) & 1u) ? kLongMax : kIntMax)) return false;
        }
        return true;
    };
    static const uint32_t kLaunchLong[] = {
        /* 0 */ 0,
        /* RELU */ 1u << 0, /* ADD */ 1u << 0, /* BIAS_ACT */ 1u << 0, /* GELU */ 1u << 0,
        /* MAXPOOL */ 1u << 8, /* AVGPOOL */ 0, /* LAYERNORM */ 1u << 0, /* SOFTMAX */ (1u << 0) | (1u << 2),
        /* EMBEDDING */ (1u << 0) | (1u << 3), /* NCHW_TO_NHWC */ 0, /* NHWC_TO_NCHW */ 0, /* SUM */ 1u << 0,
        /* FILL */ 1u << 0, /* ATTENTION */ 0xF0u, /* AVGPOOL2D */ 1u << 7, /* COPY2D */ (1u << 0) | (1u << 2) | (1u << 3),
        /* SCALE_CHANNELS */ 1u << 1};
    {
        uint32_t long_mask = 0;
        switch (op.kind) {
            case OPK_GEMM: long_mask = 0xF8u | 0xFC00u | (1u << 16); break;  // strides, ldc, batch strides, ldr
            case OPK_CONV: long_mask = (1u << 13) | (1u << 15) | (1u << 16); break;  // ldr, x / y pitch
            case OPK_BN: long_mask = (1u << 0) | (1u << 2) | (1u << 5); break;  // rows, hw, x pitch
            case OPK_LAUNCH:
                if (op.op_id > 0 && op.op_id < (int)(sizeof(kLaunchLong) / sizeof(kLaunchLong[0])))
                    long_mask = kLaunchLong[op.op_id];
                break;
            default: break;
        }
        if (!ranges_ok(long_mask)) return TP_EINVAL;
    }
    int r = 0;
    switch (op.kind) {
        case OPK_GEMM: {
            const i128 M = I[0], N = I[1], K = I[2];
            const i128 nb0 = I[8], nb1 = I[9];
            if (M < 1 || N < 1 || nb0 < 1 || nb1 < 1) return TP_EINVAL;
            if (nb0 * nb1 > 65535) return TP_EUNSUPPORTED;  // batches are the grid's z dimension
            const i128 kx = K > 0 ? K - 1 : 0;
            const i128 xs = (M - 1) * I[3] + kx * I[4] + (nb0 - 1) * I[10] + (nb1 - 1) * I[11] + 1;
            const i128 ys = (N - 1) * I[5] + kx * I[6] + (nb0 - 1) * I[12] + (nb1 - 1) * I[13] + 1;
            const i128 cs = (M - 1) * I[7] + N + (nb0 - 1) * I[14] + (nb1 - 1) * I[15];
            if (I[7] < N) return TP_EINVAL;
            const i128 ldr = I[16] ? I[16] : I[7];
            if (op.p[8] && (nb0 * nb1 != 1 || ldr < N)) return TP_EUNSUPPORTED;
            if ((r = R(0, false, xs)) || (r = R(1, false, ys)) || (r = R(2, false, cs))) return r;
            for (int k = 3; k < 8 && !r; ++k) r = R(k, true, N);
            if (!r) r = R(8, true, (M - 1) * ldr + N);
            if (r) return r;
            if ((q[4] != nullptr) != (q[5] != nullptr) || (q[4] != nullptr) != (q[6] != nullptr) ||
                (q[4] != nullptr) != (q[7] != nullptr))
                return TP_EINVAL;
            tpk::GemmArgs g;
            g.X = static_cast<const float*>(q[0]);
            g.Y = static_cast<const float*>(q[1]);
            g.C = static_cast<float*>(q[2]);
            g.M = (long)M;
            g.N = (long)N;
            g.K = (long)K;
            g.xs_r = (long)I[3];
            g.xs_k = (long)I[4];
            g.ys_c = (long)I[5];
            g.ys_k = (long)I[6];
            g.ldc = (long)I[7];
            g.nb0 = (int)nb0;
            g.nb1 = (int)nb1;
            g.xb0 = (long)I[10];
            g.xb1 = (long)I[11];
            g.yb0 = (long)I[12];
            g.yb1 = (long)I[13];
            g.cb0 = (long)I[14];
            g.cb1 = (long)I[15];
            g.ep = ep_from(op, q, 3, 0, 16);
            g.ep.ldr = (long)ldr;
            if (!launch) return 0;
            return tpk::launch_gemm(g, ws, compute_);
        }
        case OPK_CONV: {
            const i128 N = I[0], H = I[1], W = I[2], Cin = I[3], Cout = I[4], KH = I[5], KW = I[6];
            const i128 sh = I[7], sw = I[8], ph = I[9], pw = I[10];
            if (N < 1 || H < 1 || W < 1 || Cin < 1 || Cout < 1 || KH < 1 || KW < 1 || sh < 1 || sw < 1)
                return TP_EINVAL;
            const i128 Ho = (H + 2 * ph - KH) / sh + 1, Wo = (W + 2 * pw - KW) / sw + 1;
            if (H + 2 * ph < KH || W + 2 * pw < KW || Ho < 1 || Wo < 1) return TP_EINVAL;
            const i128 xpitch = op.ni > 15 ? I[15] : 0, ypitch = op.ni > 16 ? I[16] : 0;
            const i128 groups = (op.ni > 17 && I[17] > 0) ? I[17] : 1;
            const bool x_nhwc = I[11] != 0, y_nhwc = I[12] != 0;
            if ((xpitch && (!x_nhwc || xpitch < Cin)) || (ypitch && (!y_nhwc || ypitch < Cout))) return TP_EINVAL;
            if (groups != 1 && (Cin % groups != 0 || Cout % groups != 0)) return TP_EINVAL;
            // grouped but not depthwise: one launch per group over channel slices, NHWC only
            if (groups != 1 && (groups != Cin || Cin != Cout) && (!x_nhwc || !y_nhwc)) return TP_EUNSUPPORTED;
            const i128 ys = ypitch ? (N * Ho * Wo - 1) * ypitch + Cout : N * Ho * Wo * Cout;
            const i128 xs = xpitch ? (N * H * W - 1) * xpitch + Cin : N * H * W * Cin;
            if ((r = R(0, false, xs)) || (r = R(1, false, Cout * (Cin / groups) * KH * KW)) || (r = R(2, false, ys)))
                return r;
            for (int k = 3; k < 8 && !r; ++k) r = R(k, true, Cout);
            if (!r) r = R(8, true, N * Ho * Wo * Cout);  // residual: dense unless ldr says otherwise
            if (r) return r;
            if ((q[4] != nullptr) != (q[5] != nullptr) || (q[4] != nullptr) != (q[6] != nullptr) ||
                (q[4] != nullptr) != (q[7] != nullptr))
                return TP_EINVAL;
            tpk::ConvArgs c;
            c.x = static_cast<const float*>(q[0]);
            c.w = static_cast<const float*>(q[1]);
            c.y = static_cast<float*>(q[2]);
            c.N = (int)N;
            c.H = (int)H;
            c.W = (int)W;
            c.Cin = (int)Cin;
            c.Cout = (int)Cout;
            c.KH = (int)KH;
            c.KW = (int)KW;
            c.sh = (int)sh;
            c.sw = (int)sw;
            c.ph = (int)ph;
            c.pw = (int)pw;
            c.x_nhwc = (int)I[11];
            c.y_nhwc = (int)I[12];
            c.x_pitch = (long)xpitch;
            c.y_pitch = (long)ypitch;
            c.groups = (int)groups;
            c.ep = ep_from(op, q, 3, 0, 13);
            c.ep.ldr = 0;  // residual shares the layout and pitch of y
            if (!launch) return 0;
            return tpk::launch_conv2d(c, ws, compute_);
        }
        case OPK_BN: {
            const i128 rows = I[0], C = I[1];
            const i128 xpitch = op.ni > 5 ? I[5] : 0;
            if (C < 1 || (xpitch && xpitch < C)) return TP_EINVAL;
            const i128 xspan = (xpitch && rows > 0) ? (rows - 1) * xpitch + C : rows * C;
            if ((r = R(0, false, xspan)) || (r = R(1, false, rows * C))) return r;
            for (int k = 2; k < 6 && !r; ++k) r = R(k, false, C);
            if (r) return r;
            if (!I[3] && I[2] < 1) return TP_EINVAL;
            if (!launch) return 0;
            return tpk::launch_bn_inference(static_cast<const float*>(q[0]), static_cast<float*>(q[1]),
                                            static_cast<const float*>(q[2]), static_cast<const float*>(q[3]),
                                            static_cast<const float*>(q[4]), static_cast<const float*>(q[5]), op.f[0],
                                            rows, (int)C, (int)I[3], I[2], (int)I[4], xpitch, compute_);
        }
        case OPK_LAUNCH:
            break;
        default:
            return TP_EINVAL;
    }
    // generic launch by op id
    auto need = [&](int np, int ni, int nf) { return op.np >= np && op.ni >= ni && op.nf >= nf; };
    auto F = [&](int k) { return static_cast<const float*>(q[k]); };
    auto Fm = [&](int k) { return static_cast<float*>(q[k]); };
    switch (op.op_id) {
        case TP_OP_RELU:
        case TP_OP_GELU:
            if (!need(2, 1, 0)) return TP_EINVAL;
            if ((r = R(0, false, I[0])) || (r = R(1, false, I[0]))) return r;
            if (!launch) return 0;
            return op.op_id == TP_OP_RELU ? tpk::launch_relu(F(0), Fm(1), I[0], compute_)
                                          : tpk::launch_gelu(F(0), Fm(1), I[0], compute_);
        case TP_OP_ADD:
            if (!need(3, 2, 0)) return TP_EINVAL;
            if ((r = R(0, false, I[0])) || (r = R(1, false, I[0])) || (r = R(2, false, I[0]))) return r;
            if (!launch) return 0;
            return tpk::launch_add(F(0), F(1), Fm(2), I[0], (int)I[1], compute_);
        case TP_OP_BIAS_ACT:
            if (!need(3, 3, 0) || I[1] < 1) return TP_EINVAL;
            if ((r = R(0, false, I[0] * I[1])) || (r = R(1, false, I[1])) || (r = R(2, false, I[0] * I[1]))) return r;
            if (!launch) return 0;
            return tpk::launch_bias_act(F(0), F(1), Fm(2), I[0], (int)I[1], (int)I[2], compute_);
        case TP_OP_MAXPOOL: {
            if (!need(2, 8, 0)) return TP_EINVAL;
            const i128 N = I[0], H = I[1], W = I[2], C = I[3], k = I[4], st = I[5], pad = I[6];
            if (N < 1 || H < 1 || W < 1 || C < 1 || k < 1 || st < 1 || H + 2 * pad < k || W + 2 * pad < k)
                return TP_EINVAL;
            const i128 Ho = (H + 2 * pad - k) / st + 1, Wo = (W + 2 * pad - k) / st + 1;
            const i128 yp = (op.ni > 8 && I[8]) ? I[8] : C;   // NHWC: elements between output pixels
            if (yp < C || (yp != C && !I[7])) return TP_EINVAL;
            if ((r = R(0, false, N * H * W * C)) || (r = R(1, false, (N * Ho * Wo - 1) * yp + C))) return r;
            if (!launch) return 0;
            return tpk::launch_maxpool2d(F(0), Fm(1), (int)N, (int)H, (int)W, (int)C, (int)k, (int)st, (int)pad,
                                         (int)I[7], yp, compute_);
        }
        case TP_OP_AVGPOOL:
            if (!need(2, 4, 0)) return TP_EINVAL;
            if ((r = R(0, false, I[0] * I[1] * I[2])) || (r = R(1, false, I[0] * I[2]))) return r;
            if (!launch) return 0;
            return tpk::launch_global_avgpool(F(0), Fm(1), (int)I[0], (int)I[1], (int)I[2], (int)I[3], ws, compute_);
        case TP_OP_LAYERNORM:
            if (!need(5, 2, 1)) return TP_EINVAL;
            if ((r = R(0, false, I[0] * I[1])) || (r = R(1, true, I[0] * I[1])) || (r = R(2, false, I[1])) ||
                (r = R(3, false, I[1])) || (r = R(4, false, I[0] * I[1])))
                return r;
            if (!launch) return 0;
            return tpk::launch_layernorm(F(0), F(1), F(2), F(3), Fm(4), I[0], (int)I[1], op.f[0], compute_);
        case TP_OP_SOFTMAX: {
            if (!need(3, 3, 1)) return TP_EINVAL;
            const i128 rpm = I[2] > 0 ? I[2] : 1;
            if ((r = R(0, false, I[0] * I[1])) || (r = R(1, true, ((I[0] + rpm - 1) / rpm) * I[1])) ||
                (r = R(2, false, I[0] * I[1])))
                return r;
            if (!launch) return 0;
            return tpk::launch_softmax(F(0), F(1), Fm(2), I[0], (int)I[1], op.f[0], rpm, compute_);
        }
        case TP_OP_EMBEDDING:
            if (!need(6, 5, 0)) return TP_EINVAL;
            if (I[1] < 1 || I[2] < 1 || I[3] < 1 || I[4] < 1) return TP_EINVAL;
            if ((r = R(0, false, I[0], 8)) || (r = R(1, true, I[0], 8)) ||
                (r = resolve(m, op.p[2], (uint64_t)(I[3] * I[2]) * 4, false, &q[2], /*gather=*/true)) ||
                (r = R(3, true, I[1] * I[2])) || (r = R(4, true, I[4] * I[2])) || (r = R(5, false, I[0] * I[2])))
                return r;
            if (!launch) return 0;
            return tpk::launch_embedding(static_cast<const int64_t*>(q[0]), static_cast<const int64_t*>(q[1]), F(2),
                                         F(3), F(4), Fm(5), I[0], (int)I[1], (int)I[2], I[3], (int)I[4], compute_);
        case TP_OP_NCHW_TO_NHWC:
        case TP_OP_NHWC_TO_NCHW: {
            if (!need(2, 4, 0)) return TP_EINVAL;
            const i128 n = I[0] * I[1] * I[2] * I[3];
            if ((r = R(0, false, n)) || (r = R(1, false, n))) return r;
            if (!launch) return 0;
            return op.op_id == TP_OP_NCHW_TO_NHWC
                       ? tpk::launch_nchw_to_nhwc(F(0), Fm(1), (int)I[0], (int)I[1], (int)I[2], (int)I[3], compute_)
                       : tpk::launch_nhwc_to_nchw(F(0), Fm(1), (int)I[0], (int)I[1], (int)I[2], (int)I[3], compute_);
        }
        case TP_OP_SUM:
            if (!need(2, 1, 0)) return TP_EINVAL;
            if ((r = R(0, false, I[0])) || (r = R(1, false, 1))) return r;
            if (!launch) return 0;
            return tpk::launch_sum(F(0), Fm(1), I[0], compute_);
        case TP_OP_AVGPOOL2D: {
            if (!need(2, 8, 0)) return TP_EINVAL;
            const i128 N = I[0], H = I[1], W = I[2], C = I[3], k = I[4], st = I[5], pad = I[6];
            if (N < 1 || H < 1 || W < 1 || C < 1 || k < 1 || st < 1 || H + 2 * pad < k || W + 2 * pad < k)
                return TP_EINVAL;
            const i128 yp = I[7] ? I[7] : C;
            if (yp < C) return TP_EINVAL;
            const i128 Ho = (H + 2 * pad - k) / st + 1, Wo = (W + 2 * pad - k) / st + 1;
            if ((r = R(0, false, N * H * W * C)) || (r = R(1, false, (N * Ho * Wo - 1) * yp + C))) return r;
            if (!launch) return 0;
            return tpk::launch_avgpool2d(F(0), Fm(1), (int)N, (int)H, (int)W, (int)C, (int)k, (int)st, (int)pad, yp,
                                         compute_);
        }
        case TP_OP_COPY2D: {
            if (!need(2, 4, 0)) return TP_EINVAL;
            const i128 rows = I[0], width = I[1], sp = I[2], dp = I[3];
            if (rows < 1 || width < 1 || sp < width || dp < width) return TP_EINVAL;
            if ((r = R(0, false, (rows - 1) * sp + width)) || (r = R(1, false, (rows - 1) * dp + width))) return r;
            if (!launch) return 0;
            return tpk::launch_copy2d(F(0), Fm(1), rows, (int)width, sp, dp, compute_);
        }
        case TP_OP_SCALE_CHANNELS: {
            if (!need(3, 3, 0)) return TP_EINVAL;
            const i128 N = I[0], HW = I[1], C = I[2];
            if (N < 1 || HW < 1 || C < 1 || N > 0x7fffffff || C > 0x7fffffff) return TP_EINVAL;
            if ((r = R(0, false, N * HW * C)) || (r = R(1, false, N * C)) || (r = R(2, false, N * HW * C))) return r;
            if (!launch) return 0;
            return tpk::launch_scale_channels(F(0), F(1), Fm(2), (int)N, HW, (int)C, compute_);
        }
        case TP_OP_ATTENTION: {
            if (!need(5, 8, 1)) return TP_EINVAL;
            const i128 B = I[0], A = I[1], S = I[2], dh = I[3];
            if (B < 1 || A < 1 || S < 1 || dh < 1 || B * S > 0x7fffffff || A * dh > 0x7fffffff) return TP_EINVAL;
            for (int k = 4; k < 8; ++k)
                if (I[k] < A * dh) return TP_EINVAL;
            // span of a strided [B*S][A*dh] view: last row start + one row
            auto span = [&](int64_t ld) { return (B * S - 1) * ld + A * dh; };
            if ((r = R(0, false, span(I[4]))) || (r = R(1, false, span(I[5]))) || (r = R(2, false, span(I[6]))) ||
                (r = R(3, true, B * S)) || (r = R(4, false, span(I[7]))))
                return r;
            if (!launch) return 0;
            return tpk::launch_attention(F(0), F(1), F(2), F(3), Fm(4), (int)B, (int)A, (int)S, (int)dh, I[4], I[5],
                                         I[6], I[7], op.f[0], compute_);
        }
        case TP_OP_FILL:
            if (!need(1, 1, 1)) return TP_EINVAL;
            if ((r = R(0, false, I[0]))) return r;
            if (!launch) return 0;
            return tpk::launch_fill(Fm(0), op.f[0], I[0], compute_);
        default:
            return TP_EUNSUPPORTED;
    }
}

// Algorithmic work of one op: floating-point operations and bytes that have to move at least
// once (each operand read once, each result written once).
static void op_work(const Op& op, double* flops, double* bytes, const char** name) {
    const int64_t* I = op.i;
    *flops = 0;
    *bytes = 0;
    *name = "op";
    switch (op.kind) {
        case OPK_GEMM: {
            const double M = (double)I[0], N = (double)I[1], K = (double)I[2], nb = (double)(I[8] * I[9]);
            *flops = 2.0 * M * N * K * nb;
            *bytes = 4.0 * (M * K + N * K + M * N) * nb;
            *name = "gemm";
            break;
        }
        case OPK_CONV: {
            const double Ho = (double)((I[1] + 2 * I[9] - I[5]) / I[7] + 1), Wo = (double)((I[2] + 2 * I[10] - I[6]) / I[8] + 1);
            const double groups = (op.ni > 17 && I[17] > 0) ? (double)I[17] : 1.0;
            const double M = (double)I[0] * Ho * Wo, kk = (double)(I[3] * I[5] * I[6]) / groups;
            *flops = 2.0 * M * (double)I[4] * kk;
            *bytes = 4.0 * ((double)(I[0] * I[1] * I[2] * I[3]) + (double)I[4] * kk + M * (double)I[4] * (op.p[8] ? 2.0 : 1.0));
            *name = "conv";
            break;
        }
        case OPK_BN:
            *bytes = 8.0 * (double)(I[0] * I[1]);
            *name = "bn_inference";
            break;
        case OPK_LAUNCH:
            switch (op.op_id) {
                case TP_OP_RELU: *bytes = 8.0 * (double)I[0]; *name = "relu"; break;
                case TP_OP_GELU: *bytes = 8.0 * (double)I[0]; *name = "gelu"; break;
                case TP_OP_ADD: *bytes = 12.0 * (double)I[0]; *name = "add"; break;
                case TP_OP_BIAS_ACT: *bytes = 8.0 * (double)(I[0] * I[1]); *name = "bias_act"; break;
                case TP_OP_MAXPOOL: {
                    const double Ho = (double)((I[1] + 2 * I[6] - I[4]) / I[5] + 1), Wo = (double)((I[2] + 2 * I[6] - I[4]) / I[5] + 1);
                    *bytes = 4.0 * ((double)(I[0] * I[1] * I[2] * I[3]) + (double)(I[0] * I[3]) * Ho * Wo);
                    *name = "maxpool";
                    break;
                }
                case TP_OP_AVGPOOL: *bytes = 4.0 * (double)(I[0] * I[1] * I[2] + I[0] * I[2]); *name = "avgpool"; break;
                case TP_OP_LAYERNORM: *bytes = 4.0 * (double)(I[0] * I[1]) * (op.p[1] ? 3.0 : 2.0); *name = "layernorm"; break;
                case TP_OP_SOFTMAX: *bytes = 8.0 * (double)(I[0] * I[1]); *name = "softmax"; break;
                case TP_OP_EMBEDDING: *bytes = 8.0 * (double)(I[0] * I[2]); *name = "embedding"; break;
                case TP_OP_NCHW_TO_NHWC:
                case TP_OP_NHWC_TO_NCHW: *bytes = 8.0 * (double)(I[0] * I[1] * I[2] * I[3]); *name = "layout"; break;
                case TP_OP_SUM: *bytes = 4.0 * (double)I[0]; *name = "sum"; break;
                case TP_OP_FILL: *bytes = 4.0 * (double)I[0]; *name = "fill"; break;
                case TP_OP_AVGPOOL2D: *bytes = 4.0 * (double)(I[0] * I[1] * I[2] * I[3]) * 1.25; *name = "avgpool2d"; break;
                case TP_OP_COPY2D: *bytes = 8.0 * (double)(I[0] * I[1]); *name = "copy2d"; break;
                case TP_OP_SCALE_CHANNELS: *bytes = 8.0 * (double)(I[0] * I[1] * I[2]); *name = "scale_channels"; break;
                case TP_OP_ATTENTION:
                    *flops = 4.0 * (double)(I[0] * I[1]) * (double)(I[2] * I[2]) * (double)I[3];
                    *bytes = 16.0 * (double)(I[0] * I[2]) * (double)(I[1] * I[3]);
                    *name = "attention";
                    break;
                default: break;
            }
            break;
        default:
            break;
    }
}

int Engine::exec_compute(Model& m, const Op& op, bool launch) {
    if (!profiling_ || !launch || host_only()) return exec_compute_impl(m, op, launch);
    while (prof_events_.size() < prof_next_ + 2) {
        hipEvent_t e = nullptr;
        HIPCHK(hipEventCreate(&e));
        prof_events_.push_back(e);
    }
    hipEvent_t a = prof_events_[prof_next_], b = prof_events_[prof_next_ + 1];
    prof_next_ += 2;
    double flops, bytes;
    const char* name;
    op_work(op, &flops, &bytes, &name);
    tpk::set_last_kernel(name);  // the MFMA launchers overwrite this with the variant they pick
    HIPCHK(hipEventRecord(a, compute_));
    const int r = exec_compute_impl(m, op, true);
    HIPCHK(hipEventRecord(b, compute_));
    // GEMM and convolution launches are accounted per shape: the same kernel runs at very different
    // fractions of the matrix peak on different shapes
    std::string label = tpk::last_kernel_name();
    char shape[48] = "";
    if (op.kind == OPK_GEMM) {
        if (op.i[8] * op.i[9] > 1)
            std::snprintf(shape, sizeof shape, "[%lldx%lldx%lld b%lld]", (long long)op.i[0], (long long)op.i[1],
                          (long long)op.i[2], (long long)(op.i[8] * op.i[9]));
        else
            std::snprintf(shape, sizeof shape, "[%lldx%lldx%lld]", (long long)op.i[0], (long long)op.i[1], (long long)op.i[2]);
    } else if (op.kind == OPK_CONV) {
        std::snprintf(shape, sizeof shape, "[%lldx%lldx%lldx%lld>%lld k%lldx%lld s%lld]", (long long)op.i[0], (long long)op.i[1],
                      (long long)op.i[2], (long long)op.i[3], (long long)op.i[4], (long long)op.i[5], (long long)op.i[6],
                      (long long)op.i[7]);
    }
    label += shape;
    prof_records_.push_back({prof_label(label), a, b, flops, bytes});
    return r;
}

// Labels live as long as the engine: records and statistics hold pointers to them.
const char* Engine::prof_label(const std::string& s) { return prof_labels_.insert(s).first->c_str(); }

int Engine::profile_begin() {
    std::lock_guard<std::mutex> lk(mu_);
    if (host_only()) return TP_ENODEV;
    profiling_ = true;
    prof_next_ = 0;
    prof_records_.clear();
    prof_stats_.clear();
    return 0;
}

int Engine::profile_end() {
    std::lock_guard<std::mutex> lk(mu_);
    if (host_only()) return TP_ENODEV;
    if (!profiling_) return TP_ESTATE;
    profiling_ = false;
    HIPCHK(hipStreamSynchronize(compute_));
    prof_stats_.clear();
    for (auto& r : prof_records_) {
        float ms = 0.f;
        HIPCHK(hipEventElapsedTime(&ms, r.a, r.b));
        tp_kernel_stat* st = nullptr;
        for (auto& s : prof_stats_)
            if (std::strncmp(s.name, r.name, sizeof(s.name) - 1) == 0) st = &s;
        if (!st) {
            tp_kernel_stat ns;
            std::memset(&ns, 0, sizeof(ns));
            std::strncpy(ns.name, r.name, sizeof(ns.name) - 1);
            prof_stats_.push_back(ns);
            st = &prof_stats_.back();
        }
        st->launches++;
        st->total_us += (double)ms * 1000.0;
        st->flops += r.flops;
        st->bytes += r.bytes;
    }
    // event overhead: median duration of an empty bracket
    while (prof_events_.size() < 2) {
        hipEvent_t e = nullptr;
        HIPCHK(hipEventCreate(&e));
        prof_events_.push_back(e);
    }
    std::vector<float> empt;
    for (int i = 0; i < 21; ++i) {
        HIPCHK(hipEventRecord(prof_events_[0], compute_));
        HIPCHK(hipEventRecord(prof_events_[1], compute_));
        HIPCHK(hipEventSynchronize(prof_events_[1]));
        float ms = 0.f;
        HIPCHK(hipEventElapsedTime(&ms, prof_events_[0], prof_events_[1]));
        empt.push_back(ms);
    }
    std::sort(empt.begin(), empt.end());
    tp_kernel_stat es;
    std::memset(&es, 0, sizeof(es));
    std::strncpy(es.name, "__empty_bracket__", sizeof(es.name) - 1);
    es.launches = 1;
    es.total_us = (double)empt[empt.size() / 2] * 1000.0;
    prof_stats_.push_back(es);
    prof_records_.clear();
    return 0;
}

int Engine::profile_read(int index, tp_kernel_stat* out) {
    std::lock_guard<std::mutex> lk(mu_);
    if (!out) return TP_EINVAL;
    if (index < 0 || index >= (int)prof_stats_.size()) return TP_ENOENT;
    *out = prof_stats_[index];
    return 0;
}

int Engine::exec_op(Model& m, const Op& op, ReplayCtx* rc, bool launch) {
    const bool run = launch && !host_only();
    switch (op.kind) {
        case OPK_GEMM:
        case OPK_CONV:
        case OPK_BN:
        case OPK_LAUNCH:
            return exec_compute(m, op, run);
        case OPK_H2D: {
            const uint64_t bytes = (uint64_t)op.i[0];
            if (!rc) return TP_EINVAL;
            if (rc->in_pos + bytes > rc->in_bytes) return TP_EINVAL;
            int r = do_h2d(m, op.p[0], rc->in + rc->in_pos, bytes);
            rc->in_pos += bytes;
            return r;
        }
        case OPK_D2H: {
            const uint64_t bytes = (uint64_t)op.i[0];
            if (!rc) return TP_EINVAL;
            if (rc->out_pos + bytes > rc->out_bytes) return TP_EINVAL;
            int r = do_d2h_async(m, rc->out + rc->out_pos, op.p[0], bytes);
            rc->out_pos += bytes;
            return r;
        }
        case OPK_D2D: {
            void *d = nullptr, *s = nullptr;
            const uint64_t bytes = (uint64_t)op.i[0];
            int r = resolve(m, op.p[0], bytes, false, &d);
            if (!r) r = resolve(m, op.p[1], bytes, false, &s);
            if (r) return r;
            if (!run || bytes == 0) return 0;
            return tpk::launch_copy(s, d, bytes, compute_);
        }
        case OPK_MEMSET: {
            void* d = nullptr;
            const uint64_t bytes = (uint64_t)op.i[0];
            int r = resolve(m, op.p[0], bytes, false, &d);
            if (r) return r;
            if (!(op.p[0] & kVaActBit)) return TP_ESTATE;
            if (!run || bytes == 0) return 0;
            HIPCHK(hipMemsetAsync(d, (int)op.i[1], bytes, compute_));
            return 0;
        }
        default:
            return TP_EINVAL;
    }
}

int Engine::op_compute(int client, const Op& op) {
    std::lock_guard<std::mutex> lk(mu_);
    int err = 0;
    Model* m = active_model(client, &err);
    if (!m) return err;
    if (mode_ == MODE_LOAD) return TP_ESTATE;
    int r = exec_op(*m, op, nullptr, true);
    if (r) {
        if (!m->async_error) m->async_error = r;
        return r;
    }
    if (mode_ == MODE_TRACK) m->program.push_back(op);
    return 0;
}

void Engine::drop_graph(Model& m) {
    if (m.graph_exec) (void)hipGraphExecDestroy(m.graph_exec);
    m.graph_exec = nullptr;
    m.graph_begin = m.graph_end = -1;
    m.graph_state = 0;
    m.warm_streak = 0;
}

// Captures the longest run of compute ops of the recorded program on the compute stream.  The
// model is fully loaded (no gate waits), the run holds no copy from or to the host and no memset
// (memset nodes are kept out of graphs on purpose), and capture is thread-local: the copy thread
// may be issuing another model's transfers meanwhile.
int Engine::build_graph(Model& m) {
    auto graphable = [](const Op& op) {
        return op.kind == OPK_GEMM || op.kind == OPK_CONV || op.kind == OPK_BN || op.kind == OPK_LAUNCH || op.kind == OPK_D2D;
    };
    int best_b = -1, best_e = -1;
    const int n = (int)m.program.size();
    for (int i = 0; i < n;) {
        if (!graphable(m.program[(size_t)i])) {
            ++i;
            continue;
        }
        int j = i;
        while (j < n && graphable(m.program[(size_t)j])) ++j;
        if (j - i > best_e - best_b) best_b = i, best_e = j;
        i = j;
    }
    m.graph_state = -1;
    if (best_b < 0 || best_e - best_b < graph_min_ops_) return 0;
    if (hipStreamBeginCapture(compute_, hipStreamCaptureModeThreadLocal) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    int r = 0;
    for (int i = best_b; i < best_e && !r; ++i) r = exec_op(m, m.program[(size_t)i], nullptr, true);
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(compute_, &g);
    if (r || e != hipSuccess || !g) {
        if (std::getenv("TORPOR_GRAPH_DEBUG")) std::fprintf(stderr, "graph: capture failed r=%d e=%d\n", r, (int)e);
        if (g) (void)hipGraphDestroy(g);
        (void)hipGetLastError();
        return r ? r : (int)e;
    }
    hipGraphExec_t ge = nullptr;
    e = hipGraphInstantiate(&ge, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess || !ge) {
        (void)hipGetLastError();
        return (int)e;
    }
    m.graph_exec = ge;
    m.graph_begin = best_b;
    m.graph_end = best_e;
    m.graph_state = 1;
    if (std::getenv("TORPOR_GRAPH_DEBUG")) std::fprintf(stderr, "graph: model %d ops [%d, %d)\n", m.id, best_b, best_e);
    return 0;
}

int Engine::replay(int client, const void* in, uint64_t in_bytes, void* out, uint64_t out_bytes) {
    std::lock_guard<std::mutex> lk(mu_);
    int err = 0;
    Model* m = active_model(client, &err);
    if (!m) return err;
    if (mode_ != MODE_EXEC) return TP_ESTATE;
    if (m->program.empty()) return TP_ENOENT;
    TraceRange trace("replay of model", m->id);
    const bool warm = m->fully_loaded;
    const auto t_start = Clock::now();
    ReplayCtx rc;
    rc.in = static_cast<const uint8_t*>(in);
    rc.in_bytes = in_bytes;
    rc.out = static_cast<uint8_t*>(out);
    rc.out_bytes = out_bytes;
    int ret = 0;
    bool completed = false;
    // Warm requests at an unchanged placement launch the compute part of the program as one HIP
    // graph (captured on the second such request); everything else goes op by op.
    bool graphed = false;
    if (warm && graph_min_ops_ > 0 && !profiling_ && !host_only()) {
        if (m->graph_state == 0 && ++m->warm_streak >= 2) (void)build_graph(*m);
        graphed = m->graph_state == 1;
    }
    const int n_ops = (int)m->program.size();
    for (int i = 0; i < n_ops; ++i) {
        if (graphed && i == m->graph_begin) {
            hipError_t e = hipGraphLaunch(m->graph_exec, compute_);
            if (e != hipSuccess) {
                ret = (int)e;
                break;
            }
            i = m->graph_end - 1;
            continue;
        }
        const Op& op = m->program[(size_t)i];
        int r = exec_op(*m, op, &rc, true);
        if (r && !ret) ret = r;
        if (r) break;
        if (op.kind == OPK_D2H) completed = true;
    }
    const double issue_us = us_since(t_start);
    int sr = do_stream_sync(m);
    if (!ret) ret = sr;
    static const bool dbg_timing = std::getenv("TORPOR_REPLAY_TIMING") != nullptr;
    if (dbg_timing)
        std::fprintf(stderr, "replay of %d (%s, %d ops): issued in %.1f us, done after %.1f us\n", m->id,
                     warm ? "warm" : "cold", n_ops, issue_us, us_since(t_start));
    if (warm && !ret && !profiling_) {
        const double us = us_since(t_start);
        if (m->warm_us <= 0 || us < m->warm_us) m->warm_us = us;
    }
    if (!warm && !ret && !profiling_ && !host_only() && m->ncopy >= 1 && m->ncopy <= 2) {
        // A sample for choose_copy_plan: the swap-in this request ran beside, from its start to the request's end
        // -- provided the request followed its swap-in at once.  One that was started later (a prefetch, a
        // dispatcher that serves other requests meanwhile) ends when its own schedule says, not the copy plan's.
        const double us = us_since(m->swap_t0);
        const double delay = std::chrono::duration<double, std::micro>(t_start - m->swap_t0).count();
        if (delay <= 0.1 * us) {
            double& best = m->cold_us[m->ncopy];
            if (m->cold_n[m->ncopy] == 0 || us < best) best = us;
            ++m->cold_n[m->ncopy];
        }
    }
    (void)completed;
    complete_request();
    return ret;
}

// ------------------------------------------------------------------ introspection
int Engine::model_resident(int client) {
    std::lock_guard<std::mutex> lk(mu_);
    Model* m = find(client);
    if (!m) return TP_ENOENT;
    return m->resident ? 1 : 0;
}

// 1 when every transfer group of the resident model is in place (asked of the device without waiting), 0 while
// a swap-in is on its way or the model is swapped out.
int Engine::model_loaded(int client) {
    std::lock_guard<std::mutex> lk(mu_);
    Model* m = find(client);
    if (!m) return TP_ENOENT;
    if (!m->resident || m->state != MS_READY) return 0;
    if (m->fully_loaded || host_only() || m->chunk_end.empty()) return 1;
    if (m->copy_error.load() || m->cancel.load()) return 0;
    return landed(*m, (uint32_t)m->chunk_end.size() - 1) ? 1 : 0;
}

// How long the host link is busy with the part of a swap-in that a request has to wait for, and the
// forward pass alone (timed at registration, the best warm request since).
int Engine::load_estimate(int client, double* swap_ms, double* forward_ms) {
    std::lock_guard<std::mutex> lk(mu_);
    Model* m = find(client);
    if (!m) return TP_ENOENT;
    if (m->state != MS_READY) return TP_ESTATE;
    if (m->chunk_end.empty()) build_chunks(*m);
    uint64_t bytes = m->timg ? m->timg_bytes : m->image_bytes;
    if (m->defer_from != UINT32_MAX && m->defer_from > 0 && m->defer_from < m->chunk_end.size()) {
        const uint64_t from = m->chunk_end[m->defer_from - 1];
        bytes = m->timg ? xfer_off(*m, from) : from;
    }
    if (swap_ms) *swap_ms = (double)bytes / stream_rate_bytes_per_us(m->ncopy, m->chunk_max ? m->chunk_max : (16ull << 20)) / 1000.0;
    if (forward_ms) {
        // the forward pass as it runs beside its own swap-in: every launch starts later while copy queues are
        // active, and two copy streams slow the kernels themselves (the figures of choose_copy_plan)
        double kernels = 0;
        for (const Op& op : m->program)
            if (op.kind == OPK_GEMM || op.kind == OPK_CONV) kernels += 1.5;
            else if (op.kind == OPK_BN || op.kind == OPK_LAUNCH) kernels += 1.0;
        const double us = m->ncopy == 2 ? m->warm_us * 1.15 + kernels * 2.4 : m->warm_us + kernels * 1.2;
        *forward_ms = us / 1000.0;
    }
    return 0;
}

int Engine::model_info(int client, tp_model_info* out) {
    std::lock_guard<std::mutex> lk(mu_);
    if (!out) return TP_EINVAL;
    Model* m = find(client);
    if (!m) return TP_ENOENT;
    std::memset(out, 0, sizeof(*out));
    out->registered = m->state == MS_READY;
    out->resident = m->resident;
    out->level = m->level;
    out->n_params = (int)m->params.size();
    out->n_chunks = (int)m->chunk_end.size();
    out->n_ops = (int)m->program.size();
    out->image_bytes = m->image_bytes;
    out->param_bytes = m->param_bytes;
    out->act_bytes = m->act_bytes;
    out->total_bytes = m->total_bytes();
    out->weight_off = m->w_pool_off;
    out->act_off = m->a_pool_off;
    return 0;
}

int Engine::pool_stats(tp_pool_stats* out) {
    std::lock_guard<std::mutex> lk(mu_);
    if (!out) return TP_EINVAL;
    out->capacity = pool_.capacity();
    out->used = pool_.used_bytes();
    out->largest_free = pool_.largest_free();
    out->live_extents = pool_.live_extents();
    out->free_extents = pool_.free_extents();
    out->lru_budget = lru_.budget();
    out->lru_used = lru_.cur_size();
    out->lru_models = lru_.size();
    out->evictions = evictions_;
    out->swap_ins = swap_ins_;
    out->fragmentation_evictions = frag_evictions_;
    out->host_image_bytes = out->host_transfer_bytes = 0;
    for (auto& kv : models_) {
        if (kv.second->host_image) out->host_image_bytes += kv.second->image_bytes;
        if (kv.second->gather_image) out->host_image_bytes += kv.second->gather_bytes;
        if (kv.second->timg) out->host_transfer_bytes += kv.second->timg_bytes;
    }
    out->host_staging_bytes = h2d_cap_ + d2h_cap_;
    for (auto& kv : user_pinned_) out->host_staging_bytes += kv.second;
    out->device_staging_bytes = xfer_stage_cap_;
    out->device_workspace_bytes = host_only() ? 0 : cfg_.workspace_bytes;
    out->pool_cached_bytes = pool_.cached_bytes();
    out->pool_idle_extents = pool_.idle_extents();
    return 0;
}

int Engine::swap_stats(int client, tp_swap_stats* out) {
    std::lock_guard<std::mutex> lk(mu_);
    if (!out) return TP_EINVAL;
    Model* m = find(client);
    if (!m) return TP_ENOENT;
    // the copy thread may still be handing the last groups to the streams (it never takes mu_)
    while (!host_only() && m->timing_valid && m->copy_state.load(std::memory_order_acquire) == CS_RUNNING)
        std::this_thread::yield();
    if (!host_only() && m->timing_valid && m->copy_state.load() == CS_ISSUED && !m->cancel.load()) {
        if (hipEventSynchronize(m->t1) == hipSuccess) {
            float ms = 0.f;
            if (hipEventElapsedTime(&ms, m->t0, m->t1) == hipSuccess) m->stats.copy_ms = ms;
        }
    }
    if (m->copy_state.load(std::memory_order_acquire) == CS_ISSUED) {
        m->stats.issue_ms = m->issue_ms;
        m->stats.max_call_us = m->max_call_us;
        m->stats.max_call_group = m->max_call_group;
        m->stats.max_call_kind = m->max_call_kind;
    }
    *out = m->stats;
    return 0;
}

int Engine::readback_weights(int client, void* dst, uint64_t bytes) {
    std::lock_guard<std::mutex> lk(mu_);
    Model* m = find(client);
    if (!m) return TP_ENOENT;
    if (!m->resident) return TP_ESTATE;
    if (!dst || bytes != m->image_bytes) return TP_EINVAL;
    if (host_only()) return TP_ENODEV;
    while (m->copy_state.load(std::memory_order_acquire) == CS_RUNNING) std::this_thread::yield();
    HIPCHK(hipStreamSynchronize(copy_));
    HIPCHK(hipStreamSynchronize(copy2_));
    HIPCHK(hipStreamSynchronize(decode_));
    HIPCHK(hipStreamSynchronize(compute_));
    HIPCHK(hipMemcpy(dst, m->w_dev, bytes, hipMemcpyDeviceToHost));
    return 0;
}

int Engine::host_weights(int client, const void** ptr, uint64_t* bytes) {
    std::lock_guard<std::mutex> lk(mu_);
    Model* m = find(client);
    if (!m) return TP_ENOENT;
    if (m->host_image) {
        if (ptr) *ptr = m->host_image;
        if (bytes) *bytes = m->image_bytes;
        return 0;
    }
    if (!m->timg) return TP_ESTATE;
    // the host store is the transfer image: decode it into the engine's one view buffer
    if (ptr) {
        host_view_.assign(m->image_bytes, 0);
        if (!decode_transfer(*m, host_view_.data(), nullptr)) return TP_ESTATE;  // cannot happen: it decoded at registration
        *ptr = host_view_.data();
    }
    if (bytes) *bytes = m->image_bytes;
    return 0;
}

int Engine::weight_offset(int client, uint64_t va, uint64_t* off) {
    std::lock_guard<std::mutex> lk(mu_);
    Model* m = find(client);
    if (!m) return TP_ENOENT;
    if ((va & kVaTagMask) != kVaTag || (va & kVaActBit)) return TP_EFAULT;
    const uint64_t o = va & kVaOffMask;
    for (auto& p : m->params)
        if (o >= p.voff && o < p.voff + p.size) {
            if (off) *off = p.image_off + (o - p.voff);
            return 0;
        }
    return TP_EFAULT;
}

int Engine::measure_h2d(uint64_t bytes, int iters, double* gbps) {
    std::lock_guard<std::mutex> lk(mu_);
    if (host_only()) return TP_ENODEV;
    if (!gbps || bytes == 0 || iters <= 0) return TP_EINVAL;
    if (bytes > pool_.largest_free()) return TP_ENOMEM;
    const uint64_t off = pool_.alloc(bytes);
    if (off == UINT64_MAX) return TP_ENOMEM;
    uint8_t* h = nullptr;
    int ret = 0;
    hipEvent_t a = nullptr, b = nullptr;
    std::vector<float> ms;
    if (hipHostMalloc(reinterpret_cast<void**>(&h), bytes, hipHostMallocDefault) != hipSuccess) {
        pool_.release(off);
        return TP_ENOMEM;
    }
    std::memset(h, 0x5a, bytes);
    (void)hipEventCreate(&a);
    (void)hipEventCreate(&b);
    for (int i = 0; i < iters + 1 && !ret; ++i) {
        hipError_t e = hipEventRecord(a, copy_);
        if (e == hipSuccess) e = hipMemcpyAsync(arena_ + off, h, bytes, hipMemcpyHostToDevice, copy_);
        if (e == hipSuccess) e = hipEventRecord(b, copy_);
        if (e == hipSuccess) e = hipEventSynchronize(b);
        float t = 0.f;
        if (e == hipSuccess) e = hipEventElapsedTime(&t, a, b);
        if (e != hipSuccess) ret = (int)e;
        if (i > 0) ms.push_back(t);  // first one warms the path
    }
    if (!ret) {
        std::sort(ms.begin(), ms.end());
        const double med = ms[ms.size() / 2];
        *gbps = (double)bytes / (med * 1e-3) / 1e9;
        if (bytes >= (64ull << 20) && *gbps > 1.0) link_gbps_ = *gbps;  // a copy long enough to show the link itself
    }
    (void)hipEventDestroy(a);
    (void)hipEventDestroy(b);
    (void)hipHostFree(h);
    pool_.release(off);
    return ret;
}

int Engine::time_op(int client, int op_index, int iters, double* mean_us) {
    std::lock_guard<std::mutex> lk(mu_);
    if (host_only()) return TP_ENODEV;
    Model* m = find(client);
    if (!m) return TP_ENOENT;
    if (!mean_us || iters <= 0) return TP_EINVAL;
    if (!m->resident || m->state != MS_READY) return TP_ESTATE;
    if (active_ >= 0) return TP_EBUSY;
    if (op_index < 0) op_index = (int)m->program.size() - 1;
    if (op_index < 0 || op_index >= (int)m->program.size()) return TP_EINVAL;
    const Op& op = m->program[op_index];
    if (op.kind != OPK_GEMM && op.kind != OPK_CONV && op.kind != OPK_BN && op.kind != OPK_LAUNCH) return TP_EINVAL;
    while (m->copy_state.load(std::memory_order_acquire) == CS_RUNNING) std::this_thread::yield();
    HIPCHK(hipStreamSynchronize(copy_));
    HIPCHK(hipStreamSynchronize(copy2_));
    m->fully_loaded = true;
    hipEvent_t a = nullptr, b = nullptr;
    HIPCHK(hipEventCreate(&a));
    HIPCHK(hipEventCreate(&b));
    int ret = 0;
    for (int i = 0; i < 3 && !ret; ++i) ret = exec_compute(*m, op, true);  // warm-up
    if (!ret) {
        (void)hipEventRecord(a, compute_);
        for (int i = 0; i < iters && !ret; ++i) ret = exec_compute(*m, op, true);
        (void)hipEventRecord(b, compute_);
        hipError_t e = hipEventSynchronize(b);
        float ms = 0.f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, a, b);
        if (e != hipSuccess && !ret) ret = (int)e;
        *mean_us = (double)ms * 1000.0 / iters;
    }
    (void)hipEventDestroy(a);
    (void)hipEventDestroy(b);
    return ret;
}

}  // namespace tp
