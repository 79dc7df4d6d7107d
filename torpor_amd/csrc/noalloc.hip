// tp_gemm_noalloc: the GEMM of tp_gemm for callers that must not allocate (code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc).  It takes raw device addresses
// instead of an engine's virtual ones, runs on the caller's stream and keeps the only scratch memory
// the GEMM kernels use -- the partial sums of a K range split over workgroups -- in a fixed array
// in device memory that the library's code object carries, one copy per GPU.
//
// Every call on a GPU shares that GPU's array: two calls that overlap on one GPU (different
// streams or threads) race on it.  The array keeps the previous call's partial sums: a split GEMM
// writes every partial sum it later reads.  Its first 4 KiB are the ticket counters by which the
// workgroups of a split tile find out which of them finishes last; they start at zero (the array is
// zero-initialised with the code object) and the last workgroup of every tile sets its counter back.
#include <hip/hip_runtime.h>

#include <mutex>

#include "../../include/torpor_amd.h"
#include "kernels/kernels.hpp"

namespace {

constexpr size_t kScratchBytes = TP_NOALLOC_SCRATCH_BYTES;
constexpr int kMaxDevices = 64;

}  // namespace

static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {

std::mutex g_mu;
void* g_scratch_ptr[kMaxDevices] = {nullptr};

// Address of the current device's copy of `scratch`; looked up once per device.  In host code the
// array's name is only a handle for this lookup, never an address a kernel could use.
int scratch_of_current_device(float** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return TP_EINVAL;
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return TP_EFAULT;
        tpk::kernels_init(dev);
        g_scratch_ptr[dev] = p;
    }
    *out = static_cast<float*>(g_scratch_ptr[dev]);
    return 0;
}

inline const float* dev_ptr(uint64_t a) { return reinterpret_cast<const float*>(static_cast<uintptr_t>(a)); }

}  // namespace

extern "C" int tp_gemm_noalloc(const tp_gemm_desc* d, void* stream) {
    if (!d) return TP_EINVAL;
    if (d->m < 1 || d->n < 1 || d->k < 0 || d->nb0 < 1 || d->nb1 < 1 || d->ldc < d->n) return TP_EINVAL;
    constexpr int64_t kDimMax = 1ll << 31;
    if (d->m >= kDimMax || d->n >= kDimMax || d->k >= kDimMax) return TP_EINVAL;
    if (!d->x || !d->y || !d->c) return TP_EINVAL;
    const tp_epilogue& e = d->ep;
    const bool any_bn = e.bn_scale || e.bn_bias || e.bn_mean || e.bn_var;
    if (any_bn && !(e.bn_scale && e.bn_bias && e.bn_mean && e.bn_var)) return TP_EINVAL;
    const int64_t ldr = e.ldr ? e.ldr : d->ldc;
    if (e.residual && ((int64_t)d->nb0 * d->nb1 != 1 || ldr < d->n)) return TP_EUNSUPPORTED;

    tpk::GemmArgs g;
    g.X = dev_ptr(d->x);
    g.Y = dev_ptr(d->y);
    g.C = const_cast<float*>(dev_ptr(d->c));
    g.M = d->m;
    g.N = d->n;
    g.K = d->k;
    g.xs_r = d->xs_r;
    g.xs_k = d->xs_k;
    g.ys_c = d->ys_c;
    g.ys_k = d->ys_k;
    g.ldc = d->ldc;
    g.nb0 = d->nb0;
    g.nb1 = d->nb1;
    g.xb0 = d->xb0;
    g.xb1 = d->xb1;
    g.yb0 = d->yb0;
    g.yb1 = d->yb1;
    g.cb0 = d->cb0;
    g.cb1 = d->cb1;
    g.ep.alpha = e.alpha;
    g.ep.beta = e.beta;
    g.ep.bias = dev_ptr(e.bias);
    g.ep.bn_scale = dev_ptr(e.bn_scale);
    g.ep.bn_bias = dev_ptr(e.bn_bias);
    g.ep.bn_mean = dev_ptr(e.bn_mean);
    g.ep.bn_var = dev_ptr(e.bn_var);
    g.ep.bn_eps = e.bn_eps;
    g.ep.residual = dev_ptr(e.residual);
    g.ep.ldr = ldr;
    g.ep.act = e.act;

    float* ptr = nullptr;
    int r = scratch_of_current_device(&ptr);
    if (r) return r;
    // The split of K is the one tp_gemm picks when its workspace holds every partial sum; a shape
    // whose partial sums do not fit the fixed array is refused rather than split differently, so
    // that both entry points keep computing the same bits.
    const long need = tpk::gemm_workspace_need(g);
    if (need < 0) return (int)need;
    constexpr size_t kTicketBytes = tpk::kSplitTickets * sizeof(unsigned);
    if ((size_t)need > kScratchBytes - kTicketBytes) return TP_ESCRATCH;
    // head of the array: the ticket counters of split K ranges.  They are zero when the code object is
    // loaded and every launch leaves them zero, so nothing has to be cleared between calls.
    const tpk::Workspace ws{ptr + kTicketBytes / 4, kScratchBytes - kTicketBytes, nullptr, reinterpret_cast<unsigned*>(ptr)};
    return tpk::launch_gemm(g, ws, static_cast<hipStream_t>(stream));
}
