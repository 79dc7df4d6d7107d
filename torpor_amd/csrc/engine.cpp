#include "engine_internal.hpp"

namespace tp {

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
