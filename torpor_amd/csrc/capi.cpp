// extern "C" surface of the engine (include/torpor_amd.h).  Nothing here throws across the
// boundary: allocation failures and engine errors come back as integer codes.
#include <algorithm>
#include <cstring>
#include <new>

#include "engine.hpp"
#include "scheduler.hpp"
#include "weight_pack.hpp"
#include "kernels/kernels.hpp"

struct tp_server {
    tp::Engine* engine;
};

#define TP_GUARD_BEGIN try {
#define TP_GUARD_END                 \
    }                                \
    catch (const std::bad_alloc&) {  \
        return TP_ENOMEM;            \
    }                                \
    catch (...) {                    \
        return TP_EINVAL;            \
    }

extern "C" {

const char* tp_version(void) { return "torpor_amd 0.1 (gfx950)"; }

const char* tp_strerror(int code) {
    switch (code) {
        case TP_OK: return "ok";
        case TP_EINVAL: return "invalid argument or shape";
        case TP_ENOMEM: return "out of pool or host memory";
        case TP_ENOENT: return "unknown function or address";
        case TP_EBUSY: return "executor busy";
        case TP_ENODEV: return "host-only engine: no device";
        case TP_ESTATE: return "call not valid in the current executor mode";
        case TP_ENOTACTIVE: return "client is not the active function";
        case TP_EUNSUPPORTED: return "not supported";
        case TP_EFAULT: return "virtual address does not translate";
        case TP_ERANGE: return "function id out of range (0..65535)";
        case TP_ESCRATCH: return "needs more scratch memory than the fixed buffer of the no-allocation entry point";
        default: break;
    }
    if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
    return "unknown error";
}

int tp_server_create(const tp_config* cfg, tp_server** out) {
    TP_GUARD_BEGIN
    if (!out) return TP_EINVAL;
    *out = nullptr;
    tp_config c;
    std::memset(&c, 0, sizeof(c));
    if (cfg) {
        size_t n = cfg->struct_size ? cfg->struct_size : sizeof(tp_config);
        if (n > sizeof(tp_config)) n = sizeof(tp_config);
        std::memcpy(&c, cfg, n);
    }
    auto* e = new tp::Engine(c);
    int r = e->init();
    if (r) {
        delete e;
        return r;
    }
    *out = new tp_server{e};
    return 0;
    TP_GUARD_END
}

void tp_server_destroy(tp_server* s) {
    if (!s) return;
    try {
        delete s->engine;
    } catch (...) {
    }
    delete s;
}

#define ENG(s)                  \
    if (!(s) || !(s)->engine) return TP_EINVAL; \
    tp::Engine& E = *(s)->engine

int tp_signal(tp_server* s, int32_t type, const char* function, const char* payload, int32_t* ack, int32_t* resp,
              int32_t* deferred) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.signal(type, function, payload, ack, resp, deferred);
    TP_GUARD_END
}
int tp_take_deferred_ack(tp_server* s, int32_t* ack, int32_t* resp) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.take_deferred_ack(ack, resp);
    TP_GUARD_END
}
int tp_signal_ticket(tp_server* s, int32_t type, const char* function, const char* payload, int32_t* ack,
                     int32_t* resp, int32_t* deferred, uint64_t* ticket) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.signal(type, function, payload, ack, resp, deferred, ticket);
    TP_GUARD_END
}
int tp_take_deferred_ack_ticket(tp_server* s, int32_t* ack, int32_t* resp, uint64_t* ticket) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.take_deferred_ack(ack, resp, ticket);
    TP_GUARD_END
}
int tp_cancel_deferred(tp_server* s, uint64_t ticket) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.cancel_deferred(ticket);
    TP_GUARD_END
}
int tp_check_address(tp_server* s, int32_t client, uint64_t vaddr, uint64_t bytes) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.check_address(client, vaddr, bytes);
    TP_GUARD_END
}
int tp_poll(tp_server* s) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.poll();
    TP_GUARD_END
}

int tp_malloc(tp_server* s, int32_t client, uint64_t bytes, uint64_t* vaddr) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.op_malloc(client, bytes, vaddr);
    TP_GUARD_END
}
int tp_free(tp_server* s, int32_t client, uint64_t vaddr) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.op_free(client, vaddr);
    TP_GUARD_END
}
int tp_memcpy_h2d(tp_server* s, int32_t client, uint64_t dst, const void* src, uint64_t bytes) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.op_h2d(client, dst, src, bytes);
    TP_GUARD_END
}
int tp_memcpy_d2h_async(tp_server* s, int32_t client, void* dst, uint64_t src, uint64_t bytes) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.op_d2h_async(client, dst, src, bytes);
    TP_GUARD_END
}
int tp_memcpy_d2h(tp_server* s, int32_t client, void* dst, uint64_t src, uint64_t bytes) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.op_d2h(client, dst, src, bytes);
    TP_GUARD_END
}
int tp_memcpy_d2d(tp_server* s, int32_t client, uint64_t dst, uint64_t src, uint64_t bytes) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.op_d2d(client, dst, src, bytes);
    TP_GUARD_END
}
int tp_memset_async(tp_server* s, int32_t client, uint64_t dst, int32_t value, uint64_t bytes) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.op_memset(client, dst, value, bytes);
    TP_GUARD_END
}
int tp_device_synchronize(tp_server* s, int32_t client) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.op_device_sync(client);
    TP_GUARD_END
}
int tp_stream_synchronize(tp_server* s, int32_t client) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.op_stream_sync(client);
    TP_GUARD_END
}

static void fill_epilogue(tp::Op& op, const tp_epilogue& e, int pbase, int ibase) {
    op.p[pbase + 0] = e.bias;
    op.p[pbase + 1] = e.bn_scale;
    op.p[pbase + 2] = e.bn_bias;
    op.p[pbase + 3] = e.bn_mean;
    op.p[pbase + 4] = e.bn_var;
    op.p[pbase + 5] = e.residual;
    op.f[0] = e.alpha;
    op.f[1] = e.beta;
    op.f[2] = e.bn_eps;
    op.nf = 3;
    op.i[ibase + 0] = e.ldr;
    op.i[ibase + 1] = e.act;
}

int tp_gemm(tp_server* s, int32_t client, const tp_gemm_desc* d) {
    TP_GUARD_BEGIN
    ENG(s);
    if (!d) return TP_EINVAL;
    tp::Op op;
    op.kind = tp::OPK_GEMM;
    op.p[0] = d->x;
    op.p[1] = d->y;
    op.p[2] = d->c;
    const int64_t iv[16] = {d->m,   d->n,   d->k,   d->xs_r, d->xs_k, d->ys_c, d->ys_k, d->ldc,
                            d->nb0, d->nb1, d->xb0, d->xb1,  d->yb0,  d->yb1,  d->cb0,  d->cb1};
    for (int k = 0; k < 16; ++k) op.i[k] = iv[k];
    fill_epilogue(op, d->ep, 3, 16);
    op.np = 9;
    op.ni = 18;
    return E.op_compute(client, op);
    TP_GUARD_END
}

// Column-major C(m x n) = alpha*op(A)*op(B) + beta*C is the row-major product
// C'[j][i] = sum_k X(j,k) * Y(i,k) with X(j,k) = op(B)(k,j) and Y(i,k) = op(A)(i,k).
static int sgemm_common(tp_server* s, int32_t client, int transa, int transb, int m, int n, int k, float alpha,
                        uint64_t a, int lda, int64_t stride_a, uint64_t b, int ldb, int64_t stride_b, float beta,
                        uint64_t c, int ldc, int64_t stride_c, int count) {
    if (!s || !s->engine) return TP_EINVAL;
    if (m < 0 || n < 0 || k < 0 || count < 1) return TP_EINVAL;
    if (m == 0 || n == 0) return 0;
    tp_gemm_desc d;
    std::memset(&d, 0, sizeof(d));
    d.x = b;
    d.y = a;
    d.c = c;
    d.m = n;
    d.n = m;
    d.k = k;
    if (transb == 0) {  // B is k x n, element (k,j) at k + j*ldb
        d.xs_r = ldb;
        d.xs_k = 1;
    } else {  // B is n x k, element (j,k) at j + k*ldb
        d.xs_r = 1;
        d.xs_k = ldb;
    }
    if (transa == 0) {  // A is m x k, element (i,k) at i + k*lda
        d.ys_c = 1;
        d.ys_k = lda;
    } else {  // A is k x m, element (k,i) at k + i*lda
        d.ys_c = lda;
        d.ys_k = 1;
    }
    d.ldc = ldc;
    d.nb0 = 1;
    d.nb1 = count;
    d.xb1 = stride_b;
    d.yb1 = stride_a;
    d.cb1 = stride_c;
    d.ep.alpha = alpha;
    d.ep.beta = beta;
    d.ep.bn_eps = 0.f;
    return tp_gemm(s, client, &d);
}

int tp_sgemm(tp_server* s, int32_t client, int32_t transa, int32_t transb, int32_t m, int32_t n, int32_t k,
             float alpha, uint64_t a, int32_t lda, uint64_t b, int32_t ldb, float beta, uint64_t c, int32_t ldc) {
    TP_GUARD_BEGIN
    return sgemm_common(s, client, transa, transb, m, n, k, alpha, a, lda, 0, b, ldb, 0, beta, c, ldc, 0, 1);
    TP_GUARD_END
}
int tp_sgemm_strided_batched(tp_server* s, int32_t client, int32_t transa, int32_t transb, int32_t m, int32_t n,
                             int32_t k, float alpha, uint64_t a, int32_t lda, int64_t stride_a, uint64_t b,
                             int32_t ldb, int64_t stride_b, float beta, uint64_t c, int32_t ldc, int64_t stride_c,
                             int32_t count) {
    TP_GUARD_BEGIN
    return sgemm_common(s, client, transa, transb, m, n, k, alpha, a, lda, stride_a, b, ldb, stride_b, beta, c, ldc,
                        stride_c, count);
    TP_GUARD_END
}

int tp_conv_forward(tp_server* s, int32_t client, const tp_conv_desc* d) {
    TP_GUARD_BEGIN
    ENG(s);
    if (!d) return TP_EINVAL;
    if (d->groups < 0) return TP_EINVAL;
    tp::Op op;
    op.kind = tp::OPK_CONV;
    op.p[0] = d->x;
    op.p[1] = d->w;
    op.p[2] = d->y;
    const int64_t iv[13] = {d->n,        d->h,     d->w_in,  d->cin,      d->cout,    d->kh, d->kw, d->stride_h,
                            d->stride_w, d->pad_h, d->pad_w, d->x_layout, d->y_layout};
    for (int k = 0; k < 13; ++k) op.i[k] = iv[k];
    fill_epilogue(op, d->ep, 3, 13);
    op.i[15] = d->x_pitch;
    op.i[16] = d->y_pitch;
    op.i[17] = d->groups > 0 ? d->groups : 1;
    op.np = 9;
    op.ni = 18;
    return E.op_compute(client, op);
    TP_GUARD_END
}

int tp_bn_inference(tp_server* s, int32_t client, uint64_t x, uint64_t y, uint64_t scale, uint64_t bias,
                    uint64_t mean, uint64_t var, double eps, int64_t rows, int32_t channels, int64_t hw,
                    int32_t layout, int32_t relu) {
    TP_GUARD_BEGIN
    ENG(s);
    tp::Op op;
    op.kind = tp::OPK_BN;
    op.p[0] = x;
    op.p[1] = y;
    op.p[2] = scale;
    op.p[3] = bias;
    op.p[4] = mean;
    op.p[5] = var;
    op.np = 6;
    op.i[0] = rows;
    op.i[1] = channels;
    op.i[2] = hw;
    op.i[3] = layout;
    op.i[4] = relu;
    op.ni = 5;
    op.f[0] = (float)eps;
    op.nf = 1;
    return E.op_compute(client, op);
    TP_GUARD_END
}

int tp_bn_inference_pitched(tp_server* s, int32_t client, uint64_t x, uint64_t y, uint64_t scale, uint64_t bias,
                    uint64_t mean, uint64_t var, double eps, int64_t rows, int32_t channels, int64_t hw,
                    int32_t layout, int32_t relu, int64_t x_pitch) {
    TP_GUARD_BEGIN
    ENG(s);
    tp::Op op;
    op.kind = tp::OPK_BN;
    op.p[0] = x;
    op.p[1] = y;
    op.p[2] = scale;
    op.p[3] = bias;
    op.p[4] = mean;
    op.p[5] = var;
    op.np = 6;
    op.i[0] = rows;
    op.i[1] = channels;
    op.i[2] = hw;
    op.i[3] = layout;
    op.i[4] = relu;
    op.i[5] = x_pitch;
    op.ni = 6;
    op.f[0] = (float)eps;
    op.nf = 1;
    return E.op_compute(client, op);
    TP_GUARD_END
}

int tp_launch(tp_server* s, int32_t client, int32_t op_id, const uint64_t* ptrs, int32_t n_ptrs,
              const int64_t* ints, int32_t n_ints, const float* floats, int32_t n_floats) {
    TP_GUARD_BEGIN
    ENG(s);
    if (n_ptrs < 0 || n_ptrs > 12 || n_ints < 0 || n_ints > 20 || n_floats < 0 || n_floats > 4) return TP_EINVAL;
    if ((n_ptrs && !ptrs) || (n_ints && !ints) || (n_floats && !floats)) return TP_EINVAL;
    tp::Op op;
    op.kind = tp::OPK_LAUNCH;
    op.op_id = op_id;
    op.np = n_ptrs;
    op.ni = n_ints;
    op.nf = n_floats;
    for (int k = 0; k < n_ptrs; ++k) op.p[k] = ptrs[k];
    for (int k = 0; k < n_ints; ++k) op.i[k] = ints[k];
    for (int k = 0; k < n_floats; ++k) op.f[k] = floats[k];
    return E.op_compute(client, op);
    TP_GUARD_END
}

int tp_replay(tp_server* s, int32_t client, const void* input, uint64_t input_bytes, void* output,
              uint64_t output_bytes) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.replay(client, input, input_bytes, output, output_bytes);
    TP_GUARD_END
}

int tp_host_alloc(tp_server* s, uint64_t bytes, void** ptr) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.user_host_alloc(bytes, ptr);
    TP_GUARD_END
}
int tp_host_free(tp_server* s, void* ptr) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.user_host_free(ptr);
    TP_GUARD_END
}

int tp_model_resident(tp_server* s, int32_t client) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.model_resident(client);
    TP_GUARD_END
}
int tp_model_loaded(tp_server* s, int32_t client) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.model_loaded(client);
    TP_GUARD_END
}
int tp_get_load_estimate(tp_server* s, int32_t client, double* swap_ms, double* forward_ms) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.load_estimate(client, swap_ms, forward_ms);
    TP_GUARD_END
}
int tp_get_model_info(tp_server* s, int32_t client, tp_model_info* out) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.model_info(client, out);
    TP_GUARD_END
}
int tp_get_pool_stats(tp_server* s, tp_pool_stats* out) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.pool_stats(out);
    TP_GUARD_END
}
int tp_get_swap_stats(tp_server* s, int32_t client, tp_swap_stats* out) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.swap_stats(client, out);
    TP_GUARD_END
}
int tp_readback_weights(tp_server* s, int32_t client, void* dst, uint64_t bytes) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.readback_weights(client, dst, bytes);
    TP_GUARD_END
}
int tp_host_weights(tp_server* s, int32_t client, const void** ptr, uint64_t* bytes) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.host_weights(client, ptr, bytes);
    TP_GUARD_END
}
int tp_weight_offset(tp_server* s, int32_t client, uint64_t vaddr, uint64_t* image_off) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.weight_offset(client, vaddr, image_off);
    TP_GUARD_END
}
const char* tp_last_kernel(void) { return tpk::last_kernel_name(); }
int tp_measure_h2d(tp_server* s, uint64_t bytes, int32_t iters, double* gbps) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.measure_h2d(bytes, iters, gbps);
    TP_GUARD_END
}
int tp_time_op(tp_server* s, int32_t client, int32_t op_index, int32_t iters, double* mean_us) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.time_op(client, op_index, iters, mean_us);
    TP_GUARD_END
}

int tp_profile_begin(tp_server* s) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.profile_begin();
    TP_GUARD_END
}
int tp_profile_end(tp_server* s) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.profile_end();
    TP_GUARD_END
}
int tp_profile_read(tp_server* s, int32_t index, tp_kernel_stat* out) {
    TP_GUARD_BEGIN
    ENG(s);
    return E.profile_read(index, out);
    TP_GUARD_END
}

struct tp_pool {
    tp::SlabPool pool;
};
struct tp_lru {
    tp::LruEvictor lru;
};

tp_pool* tp_pool_create(uint64_t capacity_bytes) {
    try {
        auto* p = new tp_pool;
        p->pool.reset(capacity_bytes);
        return p;
    } catch (...) {
        return nullptr;
    }
}
tp_pool* tp_pool_create_policy(uint64_t capacity_bytes, int32_t policy) {
    if (policy != TP_POOL_BEST_FIT && policy != TP_POOL_FIXED_SIZE) return nullptr;
    try {
        auto* p = new tp_pool;
        p->pool.reset(capacity_bytes, policy);
        return p;
    } catch (...) {
        return nullptr;
    }
}
int tp_pool_cached(tp_pool* p, uint64_t* cached_bytes, uint64_t* idle_extents) {
    if (!p) return TP_EINVAL;
    if (cached_bytes) *cached_bytes = p->pool.cached_bytes();
    if (idle_extents) *idle_extents = p->pool.idle_extents();
    return 0;
}
int tp_pool_trim(tp_pool* p) {
    TP_GUARD_BEGIN
    if (!p) return TP_EINVAL;
    return (int)p->pool.trim();
    TP_GUARD_END
}
void tp_pool_destroy(tp_pool* p) { delete p; }
uint64_t tp_pool_alloc(tp_pool* p, uint64_t bytes) {
    if (!p) return UINT64_MAX;
    try {
        return p->pool.alloc(bytes);
    } catch (...) {
        return UINT64_MAX;
    }
}
int tp_pool_release(tp_pool* p, uint64_t offset) {
    TP_GUARD_BEGIN
    if (!p) return TP_EINVAL;
    return p->pool.release(offset) ? 0 : TP_ENOENT;
    TP_GUARD_END
}
int tp_pool_query(tp_pool* p, uint64_t* capacity, uint64_t* used, uint64_t* largest_free, uint64_t* live_extents,
                  uint64_t* free_extents) {
    if (!p) return TP_EINVAL;
    if (capacity) *capacity = p->pool.capacity();
    if (used) *used = p->pool.used_bytes();
    if (largest_free) *largest_free = p->pool.largest_free();
    if (live_extents) *live_extents = p->pool.live_extents();
    if (free_extents) *free_extents = p->pool.free_extents();
    return 0;
}
tp_lru* tp_lru_create(uint64_t budget_bytes) {
    try {
        auto* l = new tp_lru;
        l->lru.set_budget(budget_bytes);
        return l;
    } catch (...) {
        return nullptr;
    }
}
void tp_lru_destroy(tp_lru* l) { delete l; }
int tp_lru_check_and_add(tp_lru* l, const char* function, uint64_t size, char* victims, uint64_t cap,
                         int32_t* n_victims, int32_t* over_budget) {
    TP_GUARD_BEGIN
    if (!l || !function) return TP_EINVAL;
    bool over = false;
    auto v = l->lru.check_and_add(function, size, &over);
    if (n_victims) *n_victims = (int32_t)v.size();
    if (over_budget) *over_budget = over ? 1 : 0;
    if (victims && cap) {
        std::string joined;
        for (size_t i = 0; i < v.size(); ++i) {
            if (i) joined += '\n';
            joined += v[i];
        }
        std::strncpy(victims, joined.c_str(), cap - 1);
        victims[cap - 1] = '\0';
    }
    return 0;
    TP_GUARD_END
}
int tp_lru_force_evict(tp_lru* l, const char* function) {
    TP_GUARD_BEGIN
    if (!l || !function) return TP_EINVAL;
    return l->lru.force_evict(function) ? 1 : 0;
    TP_GUARD_END
}
int tp_lru_lock(tp_lru* l, const char* function) {
    TP_GUARD_BEGIN
    if (!l || !function) return TP_EINVAL;
    l->lru.lock(function);
    return 0;
    TP_GUARD_END
}
int tp_lru_unlock(tp_lru* l, const char* function) {
    TP_GUARD_BEGIN
    if (!l || !function) return TP_EINVAL;
    l->lru.unlock(function);
    return 0;
    TP_GUARD_END
}
uint64_t tp_lru_used(tp_lru* l) { return l ? l->lru.cur_size() : 0; }

static void join_names(const std::vector<std::string>& v, char* out, uint64_t cap) {
    if (!out || !cap) return;
    std::string joined;
    for (size_t i = 0; i < v.size(); ++i) {
        if (i) joined += '\n';
        joined += v[i];
    }
    std::strncpy(out, joined.c_str(), cap - 1);
    out[cap - 1] = '\0';
}

struct tp_evictor {
    int policy = TP_EVICT_IA;
    tp::IaEvictor ia;
    std::vector<tp::LruEvictor> lru;  // evictor.hpp:190-264 keeps one list per GPU
    bool ok(int gpu) const { return gpu >= 0 && gpu < ia.gpu_count(); }
};
tp_evictor* tp_evictor_create(int32_t policy, int32_t gpu_count, uint64_t budget_bytes) {
    if ((policy != TP_EVICT_LRU && policy != TP_EVICT_IA) || gpu_count < 1 || gpu_count > 64) return nullptr;
    try {
        auto* e = new tp_evictor;
        e->policy = policy;
        e->ia = tp::IaEvictor(gpu_count, budget_bytes);
        e->lru.assign((size_t)gpu_count, tp::LruEvictor(budget_bytes));
        return e;
    } catch (...) {
        return nullptr;
    }
}
void tp_evictor_destroy(tp_evictor* e) { delete e; }
int tp_evictor_set_level(tp_evictor* e, const char* function, int32_t level) {
    TP_GUARD_BEGIN
    if (!e || !function) return TP_EINVAL;
    e->ia.set_level(function, level);
    return 0;
    TP_GUARD_END
}
int tp_evictor_check_and_add(tp_evictor* e, int32_t gpu, const char* function, uint64_t size, char* victims,
                             uint64_t cap, int32_t* n_victims, int32_t* over_budget) {
    TP_GUARD_BEGIN
    if (!e || !function || !e->ok(gpu)) return TP_EINVAL;
    bool over = false;
    auto v = e->policy == TP_EVICT_IA ? e->ia.check_and_add(gpu, function, size, &over)
                                      : e->lru[(size_t)gpu].check_and_add(function, size, &over);
    if (n_victims) *n_victims = (int32_t)v.size();
    if (over_budget) *over_budget = over ? 1 : 0;
    join_names(v, victims, cap);
    return 0;
    TP_GUARD_END
}
int tp_evictor_force_evict(tp_evictor* e, int32_t gpu, const char* function) {
    TP_GUARD_BEGIN
    if (!e || !function || !e->ok(gpu)) return TP_EINVAL;
    return (e->policy == TP_EVICT_IA ? e->ia.force_evict(gpu, function) : e->lru[(size_t)gpu].force_evict(function)) ? 1 : 0;
    TP_GUARD_END
}
int tp_evictor_lock(tp_evictor* e, int32_t gpu, const char* function) {
    TP_GUARD_BEGIN
    if (!e || !function || !e->ok(gpu)) return TP_EINVAL;
    if (e->policy == TP_EVICT_IA) e->ia.lock(gpu, function);
    else e->lru[(size_t)gpu].lock(function);
    return 0;
    TP_GUARD_END
}
int tp_evictor_unlock(tp_evictor* e, int32_t gpu, const char* function) {
    TP_GUARD_BEGIN
    if (!e || !function || !e->ok(gpu)) return TP_EINVAL;
    if (e->policy == TP_EVICT_IA) e->ia.unlock(gpu, function);
    else e->lru[(size_t)gpu].unlock(function);
    return 0;
    TP_GUARD_END
}
uint64_t tp_evictor_used(tp_evictor* e, int32_t gpu) {
    if (!e || !e->ok(gpu)) return 0;
    return e->policy == TP_EVICT_IA ? e->ia.cur_size(gpu) : e->lru[(size_t)gpu].cur_size();
}
int tp_evictor_is_protected(tp_evictor* e, int32_t gpu, const char* function) {
    TP_GUARD_BEGIN
    if (!e || !function || !e->ok(gpu)) return TP_EINVAL;
    return e->policy == TP_EVICT_IA && e->ia.is_protected(gpu, function) ? 1 : 0;
    TP_GUARD_END
}
int tp_evictor_order(tp_evictor* e, int32_t gpu, char* out, uint64_t cap) {
    TP_GUARD_BEGIN
    if (!e || !e->ok(gpu)) return TP_EINVAL;
    std::vector<std::string> v;
    if (e->policy == TP_EVICT_IA) v = e->ia.order(gpu);
    else {
        v = e->lru[(size_t)gpu].order();  // most recent first
        std::reverse(v.begin(), v.end());
    }
    join_names(v, out, cap);
    return (int)v.size();
    TP_GUARD_END
}

struct tp_sched {
    tp::Scheduler s;
};
tp_sched* tp_sched_create(int32_t gpu_count) {
    if (gpu_count < 1 || gpu_count > 64) return nullptr;
    try {
        auto* s = new tp_sched;
        s->s.reset(gpu_count);
        return s;
    } catch (...) {
        return nullptr;
    }
}
void tp_sched_destroy(tp_sched* s) { delete s; }
int tp_sched_set_sibling(tp_sched* s, int32_t gpu, int32_t other) {
    return s && s->s.set_sibling(gpu, other) ? 0 : TP_EINVAL;
}
int tp_sched_set_link(tp_sched* s, int32_t a, int32_t b, int32_t kind) {
    return s && kind >= -1 && kind <= 2 && s->s.set_link(a, b, kind) ? 0 : TP_EINVAL;
}
int tp_sched_set_status(tp_sched* s, int32_t gpu, int32_t status) {
    return s && status >= -1 && status <= 5 && s->s.set_status(gpu, status) ? 0 : TP_EINVAL;
}
int tp_sched_set_level(tp_sched* s, const char* function, int32_t level) {
    TP_GUARD_BEGIN
    if (!s || !function) return TP_EINVAL;
    s->s.set_level(function, level);
    return 0;
    TP_GUARD_END
}
int tp_sched_set_resident(tp_sched* s, const char* function, int32_t gpu, int32_t resident) {
    TP_GUARD_BEGIN
    if (!s || !function || gpu < 0 || gpu >= s->s.gpu_count()) return TP_EINVAL;
    s->s.set_resident(function, gpu, resident != 0);
    return 0;
    TP_GUARD_END
}
int tp_sched_placement(tp_sched* s) { return s ? s->s.placement() : TP_EINVAL; }
int tp_sched_decide(tp_sched* s, int32_t policy, const char* function, uint32_t draw, int32_t* dst_gpu,
                    int32_t* src_gpu, int32_t* status) {
    TP_GUARD_BEGIN
    if (!s || !function || (policy != TP_SCHED_RANDOM && policy != TP_SCHED_IA)) return TP_EINVAL;
    const tp::ScheduleDecision d = policy == TP_SCHED_IA
                                       ? s->s.interference_aware_schedule(function)
                                       : s->s.random_schedule(function, [draw](int n) { return (int)(draw % (uint32_t)n); });
    if (dst_gpu) *dst_gpu = d.dst_gpu;
    if (src_gpu) *src_gpu = d.src_gpu;
    if (status) *status = d.status;
    return 0;
    TP_GUARD_END
}

// ------------------------------------------------------------------ transfer format
uint64_t tp_pack_bound(uint64_t n_words) { return tp::packed_bytes(n_words); }
uint64_t tp_pack_blocks(uint64_t n_words) { return tp::packed_blocks(n_words); }

int tp_pack_words(const uint32_t* words, uint64_t n_words, uint8_t* payload, int32_t* base, uint8_t* ext,
                  uint64_t ext_cap, uint64_t* n_ext, uint32_t* block_tab) {
    TP_GUARD_BEGIN
    if ((!words && n_words) || !payload || !base || (!ext && ext_cap) || (!block_tab && n_words)) return TP_EINVAL;
    uint32_t b = 0;
    uint64_t outside = 0;
    tp::choose_window(words, n_words, &b, &outside);
    std::memset(payload, 0, tp::packed_bytes(n_words));
    std::vector<uint8_t> e;
    tp::pack_words(words, n_words, b, payload, &e, block_tab);
    *base = (int32_t)b;
    if (n_ext) *n_ext = e.size();
    if (e.size() > ext_cap) return TP_ENOMEM;
    if (!e.empty()) std::memcpy(ext, e.data(), e.size());
    return 0;
    TP_GUARD_END
}

int tp_unpack_words(const uint8_t* payload, uint64_t n_words, int32_t base, const uint8_t* ext, uint64_t n_ext,
                    uint32_t* words) {
    TP_GUARD_BEGIN
    if (!payload || (!words && n_words) || base < 0 || base > 255 || (!ext && n_ext)) return TP_EINVAL;
    return tp::unpack_words(payload, n_words, (uint32_t)base, ext, n_ext, words) == UINT64_MAX ? TP_EINVAL : 0;
    TP_GUARD_END
}

int tp_unpack_words_device(tp_server* s, const uint8_t* payload, uint64_t n_words, int32_t base, const uint8_t* ext,
                           uint64_t n_ext, const uint32_t* block_tab, uint64_t w_from, uint64_t w_to,
                           uint32_t* words) {
    TP_GUARD_BEGIN
    ENG(s);
    if (!payload || (!words && n_words) || base < 0 || base > 255 || (!ext && n_ext) || (!block_tab && n_words))
        return TP_EINVAL;
    if (w_from > w_to || w_to > n_words || (w_from & 63) || ((w_to & 63) && w_to != n_words)) return TP_EINVAL;
    {  // the stream must hold what the codes ask for: expand on the host first
        std::vector<uint32_t> probe(n_words);
        if (tp::unpack_words(payload, n_words, (uint32_t)base, ext, n_ext, probe.data()) == UINT64_MAX) return TP_EINVAL;
    }
    return E.unpack_on_device(payload, n_words, base, ext, n_ext, block_tab, w_from, w_to, words);
    TP_GUARD_END
}

}  // extern "C"
