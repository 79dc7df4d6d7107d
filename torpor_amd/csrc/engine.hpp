// Engine: executor + memory manager + controller of one GPU.
//
// Reference counterparts (paths relative to the reference tree):
//   Controller        include/server/controller.hpp      -> Engine::signal / complete_request
//   CUDAExecutor      include/server/cuda_server.hpp     -> Engine op entry points / exec_op
//   MemoryManager     include/server/memory_manager.hpp  -> translate / gate / swap engine
//   ModelRepo         include/server/model_repo.hpp      -> Model (host weight store, tables)
// The reference shares these objects between a controller thread, an executor
// thread and a transfer thread through unsynchronised singletons; here all
// engine state is owned by one mutex, and the copy thread only touches the
// per-model atomics and the immutable chunk table of the job it was handed.
#pragma once
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdlib>
#include <deque>
#include <map>
#include <memory>
#include <mutex>
#include <set>
#include <string>
#include <thread>
#include <unordered_map>
#include <vector>

#include "../../include/torpor_amd.h"
#include "ia_evictor.hpp"
#include "lru.hpp"
#include "pool.hpp"
#include "trace.hpp"

namespace tp {

constexpr uint64_t kTensorAlign = 256;
constexpr uint64_t kVaTag = 0x7Aull << 56;
constexpr uint64_t kVaTagMask = 0xFFull << 56;
// tag (8 bits) | function id (16 bits) | region bit | offset (39 bits: 512 GiB per region, above the
// 288 GB of the part).  The reference takes any integer as a function id (cuda_server.hpp:221-224);
// here ids above kMaxClient are refused with TP_ERANGE.
constexpr int kVaClientShift = 40;
constexpr uint64_t kVaClientMask = 0xFFFFull;
constexpr uint64_t kVaActBit = 1ull << 39;
constexpr uint64_t kVaOffMask = (1ull << 39) - 1;
constexpr int kMaxClient = 65535;

enum OpKind : int { OPK_GEMM = 1, OPK_CONV, OPK_BN, OPK_LAUNCH, OPK_H2D, OPK_D2H, OPK_D2D, OPK_MEMSET };

// One recorded data-plane call, addresses still virtual.
struct Op {
    int kind = 0;
    int op_id = 0;
    int np = 0, ni = 0, nf = 0;
    uint64_t p[12] = {0};
    int64_t i[20] = {0};
    float f[4] = {0};
};

struct Param {  // one uploaded weight tensor (model_repo.hpp:31-36 ModelParamInfo)
    uint64_t voff = 0;       // offset in the function's weight address region
    uint64_t size = 0;
    uint64_t image_off = 0;  // offset in the weight image (host store and device copy alike)
    int access_rank = -1;    // first-access position in the tracked run, -1 = never touched
    // Rows of this tensor are looked up by index (an embedding table).  Such a tensor travels
    // last in the weight image, and while its transfer group is still on its way a lookup reads
    // the rows it needs straight from the pinned host store.
    bool gathered = false;
    // place in the transfer image: as it is (pack_base < 0) or packed with that window base, its block
    // table and extension stream right before its payload
    uint64_t t_off = 0;
    uint64_t tab_off = 0, ext_off = 0;
    int32_t pack_base = -1;
};
struct WBlock {
    uint64_t voff, size;
};
struct ABlock {  // activation allocation
    uint64_t voff = 0, size = 0;
    bool live = false;
    uint64_t pool_off = UINT64_MAX;  // own extent while tracking, else inside the model's arena
};

// Bytes of a model's uploads until its weight image is laid out.  Grows with realloc: for blocks of this
// size the C library moves pages instead of copying them, and nothing is filled in (only bytes that an
// upload has written are ever read back).
class UploadBuffer {
public:
    UploadBuffer() = default;
    UploadBuffer(const UploadBuffer&) = delete;
    UploadBuffer& operator=(const UploadBuffer&) = delete;
    ~UploadBuffer() { release(); }
    bool resize(uint64_t n) {
        if (n > cap_) {
            const uint64_t want = std::max<uint64_t>(n, cap_ + cap_ / 2);
            void* q = std::realloc(p_, (size_t)want);
            if (!q) return false;
            p_ = static_cast<uint8_t*>(q);
            cap_ = want;
        }
        size_ = n;
        return true;
    }
    void release() {
        std::free(p_);
        p_ = nullptr;
        size_ = cap_ = 0;
    }
    uint8_t* data() { return p_; }
    uint64_t size() const { return size_; }

private:
    uint8_t* p_ = nullptr;
    uint64_t size_ = 0, cap_ = 0;
};

enum ModelState : int { MS_LOADING = 0, MS_TRACKING = 1, MS_READY = 2 };
enum CopyState : int { CS_IDLE = 0, CS_RUNNING = 1, CS_ISSUED = 2 };

struct Model {
    int id = -1;
    int level = 1;
    int state = MS_LOADING;
    // weight address region and host store
    uint64_t wbump = 0;
    std::vector<WBlock> wblocks;
    std::vector<Param> params;  // sorted by voff
    UploadBuffer staging;
    uint8_t* host_image = nullptr;
    uint8_t* host_image_dev = nullptr;  // the same memory as kernels address it, null if not mapped
    uint64_t image_bytes = 0, param_bytes = 0;
    // What a swap-in sends when the weights compress: the tensors in image order, each as it is or as
    // [block table][extension stream][payload].  Null when the image travels as it is.
    uint8_t* timg = nullptr;
    uint64_t timg_bytes = 0;
    // Once the transfer image exists and has been decoded back to the image bit for bit, the image itself is
    // given up (host_image == nullptr): the host store of such a model is its transfer image, plus a raw copy
    // of the tables looked up by index -- image bytes [gather_off, image_bytes) -- that lookups read in place
    // during a swap-in.
    uint8_t* gather_image = nullptr;
    uint8_t* gather_dev = nullptr;
    uint64_t gather_off = 0, gather_bytes = 0;
    std::vector<uint32_t> image_order; // params[] indices by image_off
    std::vector<hipEvent_t> dma_ev;    // transfer group arrived in the staging area (packed transfers)
    int next_rank = 0;
    std::vector<uint64_t> chunk_end;
    std::vector<hipEvent_t> chunk_ev;
    // activation region
    uint64_t abump = 0;
    std::map<uint64_t, ABlock> ablocks;
    std::multimap<uint64_t, uint64_t> afree;  // size -> voff
    uint64_t act_bytes = 0;
    bool act_frozen = false;
    // residency
    bool resident = false;
    bool fully_loaded = false;
    uint64_t w_pool_off = UINT64_MAX, a_pool_off = UINT64_MAX;
    uint8_t* w_dev = nullptr;
    uint8_t* a_dev = nullptr;
    std::atomic<uint32_t> issued{0};
    std::atomic<int> copy_state{CS_IDLE};
    std::atomic<bool> cancel{false};
    std::atomic<int> copy_error{0};
    // written by the copy thread before it publishes CS_ISSUED, read by the engine after that
    double issue_ms = 0, max_call_us = 0;
    uint32_t max_call_group = 0, max_call_kind = 0;
    uint32_t gated_upto = 0;
    uint64_t touch_seq = 0;   // Engine::work_seq_ at this model's last data-plane call
    uint32_t defer_from = UINT32_MAX;  // first transfer group made of deferred tables only
    int ncopy = 2;            // copy streams used by the current swap-in plan
    uint64_t chunk_max = 0;   // largest transfer group of the current plan
    double warm_us = 0;       // best warm replay so far (host wall clock), 0 = none yet
    // Cold requests seen under each copy plan (index = number of copy streams): the shortest time from the start
    // of a swap-in to the end of the request that ran beside it, and how many there were (choose_copy_plan).
    double cold_us[3] = {0, 0, 0};
    int cold_n[3] = {0, 0, 0};
    std::chrono::steady_clock::time_point swap_t0;
    // captured compute segment of the recorded program (warm replays at an unchanged placement)
    hipGraphExec_t graph_exec = nullptr;
    int graph_begin = -1, graph_end = -1;  // program[graph_begin, graph_end) is what the graph launches
    int graph_state = 0;                   // 0 none yet, 1 ready, -1 not usable for this model
    int warm_streak = 0;                   // warm replays since the placement last changed
    hipEvent_t t0 = nullptr, t1 = nullptr;
    bool timing_valid = false;
    bool transfer_logged = false;  // the executor log has this swap-in's Transfer line
    // recorded program
    std::vector<Op> program;
    int async_error = 0;
    tp_swap_stats stats{};

    uint64_t total_bytes() const { return SlabPool::round_up(image_bytes) + SlabPool::round_up(act_bytes); }
};

struct PendingD2H {
    void* dst;
    uint64_t stage_off;
    uint64_t bytes;
};

struct ReplayCtx {
    const uint8_t* in = nullptr;
    uint64_t in_bytes = 0, in_pos = 0;
    uint8_t* out = nullptr;
    uint64_t out_bytes = 0, out_pos = 0;
};

class Engine {
public:
    explicit Engine(const tp_config& cfg);
    ~Engine();
    int init();

    int signal(int type, const char* function, const char* payload, int* ack, int* resp, int* deferred,
               uint64_t* ticket = nullptr);
    int take_deferred_ack(int* ack, int* resp, uint64_t* ticket = nullptr);
    int cancel_deferred(uint64_t ticket);
    int check_address(int client, uint64_t va, uint64_t bytes);
    int poll();

    int op_malloc(int client, uint64_t bytes, uint64_t* va);
    int op_free(int client, uint64_t va);
    int op_h2d(int client, uint64_t dst, const void* src, uint64_t bytes);
    int op_d2h_async(int client, void* dst, uint64_t src, uint64_t bytes);
    int user_host_alloc(uint64_t bytes, void** ptr);
    int user_host_free(void* ptr);
    int unpack_on_device(const uint8_t* payload, uint64_t n_words, int32_t base, const uint8_t* ext, uint64_t n_ext,
                         const uint32_t* block_tab, uint64_t w_from, uint64_t w_to, uint32_t* words);
    int op_d2h(int client, void* dst, uint64_t src, uint64_t bytes);
    int op_d2d(int client, uint64_t dst, uint64_t src, uint64_t bytes);
    int op_memset(int client, uint64_t dst, int value, uint64_t bytes);
    int op_device_sync(int client);
    int op_stream_sync(int client);
    int op_compute(int client, const Op& op);  // GEMM / CONV / BN / LAUNCH
    int replay(int client, const void* in, uint64_t in_bytes, void* out, uint64_t out_bytes);

    int model_resident(int client);
    int model_loaded(int client);
    int load_estimate(int client, double* swap_ms, double* forward_ms);
    int model_info(int client, tp_model_info* out);
    int pool_stats(tp_pool_stats* out);
    int swap_stats(int client, tp_swap_stats* out);
    int readback_weights(int client, void* dst, uint64_t bytes);
    int host_weights(int client, const void** ptr, uint64_t* bytes);
    int weight_offset(int client, uint64_t va, uint64_t* off);
    int measure_h2d(uint64_t bytes, int iters, double* gbps);
    int time_op(int client, int op_index, int iters, double* mean_us);
    int profile_begin();
    int profile_end();
    int profile_read(int index, tp_kernel_stat* out);

private:
    enum Mode : int { MODE_NONE = 0, MODE_LOAD = 1, MODE_TRACK = 2, MODE_EXEC = 3 };
    // controller.hpp:17-23
    enum ExecStatus : int { ES_AVAIL = -1, ES_LOCAL = 0, ES_PCIE_LIGHT = 2, ES_PCIE_MEDIAN = 3, ES_PCIE_HEAVY = 4, ES_COLD = 5 };
    struct Queued {
        int id;
        bool cold;
        int level;
        uint64_t ticket;
    };
    struct DeferredAck {
        int ack, resp;
        uint64_t ticket;
        int id;  // the function whose request this ack started
    };
    struct Xlat {
        uint8_t* p = nullptr;
        bool weight = false;
        uint64_t image_end = 0;
        Param* param = nullptr;
    };

    bool host_only() const { return (cfg_.flags & TP_FLAG_HOST_ONLY) != 0; }
    Model* find(int id);
    Model* active_model(int client, int* err);
    int translate(Model& m, uint64_t va, uint64_t span, Xlat* out);
    int gate(Model& m, const Xlat& x);
    int resolve(Model& m, uint64_t va, uint64_t span, bool optional, void** out, bool gather = false);
    bool landed(Model& m, uint32_t idx);
    int build_transfer(Model& m);
    int slim_host_store(Model& m);
    bool decode_transfer(const Model& m, uint8_t* image_out, const uint8_t* expect);
    void free_host_store(Model& m);
    uint64_t xfer_off(const Model& m, uint64_t image_off) const;
    void free_transfer(Model& m);
    int copy_chunk_packed(Model& m, size_t i, uint64_t beg, uint64_t end, hipStream_t cs, bool do_dma, bool do_expand);
    int exec_op(Model& m, const Op& op, ReplayCtx* rc, bool launch);
    int exec_compute(Model& m, const Op& op, bool launch);
    int exec_compute_impl(Model& m, const Op& op, bool launch);
    int do_h2d(Model& m, uint64_t dst, const void* src, uint64_t bytes);
    int do_d2h_async(Model& m, void* dst, uint64_t src, uint64_t bytes);
    int do_stream_sync(Model* m);

    void start_cold(int id, int level);
    int start_execute(int id);
    int swap_in(Model& m);
    void evict_model(Model& m);
    void destroy_model(Model& m);
    bool check_eviction(Model& m);
    void complete_request();
    void start_next_queued();
    int finish_loading(Model& m);
    int finish_tracking(Model& m);
    int build_image(Model& m, bool by_access);
    void build_chunks(Model& m);
    void choose_copy_plan(Model& m);
    double stream_rate_bytes_per_us(int streams, uint64_t group) const;
    void drop_graph(Model& m);
    int build_graph(Model& m);
    void wait_copy_idle(Model& m);
    bool swap_in_flight();
    bool copy_by_kernel(const Model& m, uint64_t bytes);
    void log_transfer(Model& m);
    void copy_main();
    int ensure_stage(uint8_t** buf, uint64_t* cap, uint64_t need);
    void* host_alloc(uint64_t bytes);
    void host_free(void* p);
    bool poll_timeout_locked();

    tp_config cfg_;
    std::mutex mu_;
    SlabPool pool_;
    // controller.hpp:103-109: EVICT_POLICY=LRU selects the plain LRU, anything else the two-class policy.
    // With one GPU and every model at the default level (Median) both make the same decisions.
    struct EvictPolicy {
        bool two_class = true;
        LruEvictor lru;
        IaEvictor ia{1, 0};
        void set_budget(uint64_t b) { lru.set_budget(b); ia.set_budget(b); }
        uint64_t budget() const { return two_class ? ia.budget() : lru.budget(); }
        uint64_t cur_size() const { return two_class ? ia.cur_size(0) : lru.cur_size(); }
        size_t size() const { return two_class ? ia.size(0) : lru.size(); }
        std::vector<std::string> check_and_add(const std::string& f, uint64_t sz, int level, bool* over) {
            if (!two_class) return lru.check_and_add(f, sz, over);
            ia.set_level(f, level);
            return ia.check_and_add(0, f, sz, over);
        }
        bool force_evict(const std::string& f) { return two_class ? ia.force_evict(0, f) : lru.force_evict(f); }
        bool peek_victim(const std::string& keep, std::string* out) const {
            return two_class ? ia.peek_victim(0, keep, out) : lru.peek_victim(keep, out);
        }
        void lock(const std::string& f) { two_class ? ia.lock(0, f) : lru.lock(f); }
        void unlock(const std::string& f) { two_class ? ia.unlock(0, f) : lru.unlock(f); }
    } lru_;
    uint8_t* arena_ = nullptr;
    float* workspace_ = nullptr;
    hipStream_t compute_ = nullptr, copy_ = nullptr, copy2_ = nullptr;
    // packed transfers land in a staging area and are expanded into place on their own stream
    hipStream_t decode_ = nullptr;
    uint8_t* xfer_stage_ = nullptr;
    uint64_t xfer_stage_cap_ = 0;
    hipEvent_t stage_free_ev_ = nullptr;  // the last expansion that read the staging area
    bool stage_used_ = false;
    bool pack_ = true;
    bool slim_host_ = true;  // give up the raw image of a model whose transfer image decodes back to it
    std::vector<uint8_t> host_view_;  // where tp_host_weights decodes such a model's image to (one at a time)
    int copy_streams_cfg_ = 0;
    // Pinned-host -> HBM rate of this box's link in GB/s: timed on the copy streams when the engine starts,
    // replaced by tp_measure_h2d's figure when a caller asks for one.  Swap-in plans and load estimates use it.
    double link_gbps_ = kNominalLinkGbps;
    static constexpr double kNominalLinkGbps = 56.0;  // until measured (an engine without a device keeps it)
    static constexpr double kCopyFixedUs = 15.0;      // fixed cost of one hipMemcpyAsync on a copy stream
    bool chunk_max_auto_ = true;
    int plan_trials_ = 2;  // cold requests per copy plan before the measured choice is made (TORPOR_PLAN_TRIALS; 0 = estimate only)
    bool per_tensor_groups_ = false;  // BUFFER_SIZE=1: a transfer group closes behind every tensor
    int d2h_kernel_ = 0;
    uint64_t small_copy_bytes_ = 1ull << 20;  // request copies up to this size go by copy kernel (TORPOR_SMALL_COPY_BYTES)
    bool host_gather_ = true;  // lookups may read a table in place from the host store during a swap-in
    int graph_min_ops_ = 0;  // 0: warm replays launch op by op; n: capture compute runs of at least n ops
    std::unordered_map<int, std::unique_ptr<Model>> models_;

    int active_ = -1;
    int mode_ = MODE_NONE;
    int exec_status_ = ES_AVAIL;
    std::chrono::steady_clock::time_point req_start_;
    std::deque<Queued> req_queue_;
    std::deque<DeferredAck> deferred_acks_;
    std::deque<DeferredAck> taken_acks_;  // acks handed out for the request that is still active
    uint64_t ticket_seq_ = 0;  // queued signals are numbered from 1 in the order they were queued
    bool d2h_seen_ = false;
    // Data-plane calls are numbered; synced_seq_ is the number reached when the host last waited for
    // the compute stream.  A model whose touch_seq is above it may still have work on the device.
    uint64_t work_seq_ = 0, synced_seq_ = 0;

    uint8_t* h2d_stage_ = nullptr;
    uint64_t h2d_cap_ = 0, h2d_pos_ = 0;
    std::map<uintptr_t, uint64_t> user_pinned_;  // result buffers handed out by user_host_alloc: base -> bytes
    uint8_t* d2h_stage_ = nullptr;
    uint64_t d2h_cap_ = 0, d2h_pos_ = 0;
    std::vector<PendingD2H> pending_d2h_;

    uint64_t evictions_ = 0, swap_ins_ = 0, frag_evictions_ = 0;

    struct ProfRecord {
        const char* name;
        hipEvent_t a, b;
        double flops, bytes;
    };
    bool profiling_ = false;
    std::vector<hipEvent_t> prof_events_;
    size_t prof_next_ = 0;
    std::vector<ProfRecord> prof_records_;
    std::vector<tp_kernel_stat> prof_stats_;
    std::set<std::string> prof_labels_;
    const char* prof_label(const std::string& s);

    ExecLog log_;
    uint64_t req_range_ = 0;  // open "request" range of the marker trace, 0 = none

    std::thread copy_thread_;
    std::mutex cmu_;
    std::condition_variable ccv_;
    std::deque<Model*> jobs_;
    Model* last_swap_ = nullptr;  // the model whose swap-in was started last, until it is seen to have landed
    bool stop_ = false;
};

}  // namespace tp
