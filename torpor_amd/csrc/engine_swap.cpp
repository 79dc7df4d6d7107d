#include "engine_internal.hpp"

namespace tp {

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
}  // namespace tp
