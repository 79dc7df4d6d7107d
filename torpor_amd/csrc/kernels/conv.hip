// Implicit-GEMM fp32 convolution on MFMA for gfx950.
//
// Replaces the cudnnConvolutionForward call site of the reference executor
// (include/server/cuda_server.hpp:708-735): y = alpha*conv2d(x, w) + beta*y,
// fp32, groups = 1, weights in the framework's native [Cout][Cin][KH][KW]
// order (the swapped-in bytes are used as they are; nothing is re-laid-out).
// The GEMM view is rows = output pixels (n, ho, wo), cols = Cout,
// K = Cin*KH*KW; the fused epilogue adds bias / inference batch-norm /
// residual / activation.
//
//   1x1, NHWC, Cin%4==0, pad 0      -> the dense GEMM kernel with a row gather
//   3x3, 1x7, 7x1, 1x3, 3x1; NHWC, Cin%8==0 -> conv_taps_kernel (K-block = 8 or 16 channels x taps)
//   everything else (7x7 stem, NCHW) -> conv_generic_kernel (scalar gathers)
#include "kernels.hpp"
#include "mfma_tile.hpp"

namespace tpk {

void set_last_kernel(const char* n);
int num_cu();
Epilogue make_epilogue(const EpilogueArgs& a, long ldc);
int launch_splitk_reduce(const float* ws, int splits, long M, long N, float* C, const Epilogue& e, hipStream_t s);
int choose_splits(long tiles, long K, int bk, long tile_floats, size_t ws_bytes, long* kper_out, int max_splits = 32, bool pairs = true,
                  int balance = -1);
unsigned* split_tickets(const Workspace& ws, long tiles, int splits);
int launch_conv3x3_winograd(const ConvArgs& a, const Workspace& ws, hipStream_t s);  // winograd.hip

struct ConvDev {
    const float* x;
    const float* w;
    float* y;
    int N, H, W, Cin, Cout, KH, KW, Ho, Wo, sh, sw, ph, pw;
    long xs_n, xs_h, xs_w, xs_c;
    long M;     // N*Ho*Wo
    long K;     // Cin*KH*KW
    int splits;
    long kper;  // K (generic) or channels (3x3 fast) per split
    float* ws;
    unsigned* tickets;  // non-null: a split is summed inside the launch (finish_split)
    const float* zeros;
    int tiles_m, tiles_n;
    Epilogue ep;
};

__device__ __forceinline__ void fetch_now(const ConvDev& p) {
    fetch_now(p.x);
    fetch_now(p.w);
    fetch_now(p.y);
    fetch_now(p.H);
    fetch_now(p.W);
    fetch_now(p.Cin);
    fetch_now(p.Cout);
    fetch_now(p.Ho);
    fetch_now(p.Wo);
    fetch_now(p.sh);
    fetch_now(p.sw);
    fetch_now(p.ph);
    fetch_now(p.pw);
    fetch_now(p.xs_n);
    fetch_now(p.xs_h);
    fetch_now(p.xs_w);
    fetch_now(p.M);
    fetch_now(p.splits);
    fetch_now(p.kper);
    fetch_now(p.ws);
    fetch_now(p.tickets);
    fetch_now(p.zeros);
    fetch_now(p.tiles_m);
    fetch_now(p.tiles_n);
    fetch_now(p.ep);
}

__device__ __forceinline__ int remap_xcd_c(int bid, int n) {
    const int q = n >> 3, rem = n & 7;
    const int xcd = bid & 7, local = bid >> 3;
    return xcd * q + (xcd < rem ? xcd : rem) + local;
}

// KH x KW taps (T = KH*KW; 3x3, and the 1x7 / 7x1 / 1x3 / 3x1 shapes of Inception), NHWC,
// Cin % 8 == 0.  K-block = CB input channels x T taps (CB = BK / T: 8, or 16 for the nine-wavefront
// 3x3 tile), ordered k_local = tap*CB + c in LDS.
// Activation side: for (pixel, tap) the CB channels are 4*CB contiguous bytes of
// the NHWC input (CB/4 dwordx4 loads by neighbouring threads).  Weight side:
// for one output channel the CB x T block is CB*T contiguous floats of the
// [Cout][Cin][KH][KW] tensor; each thread loads 4T of them (4 channels x T taps)
// with dwordx4 and transposes in registers to the tap-major LDS order.
//
// WGK > 1 (3 or 9 for 3x3: the nine k-groups of a K-block split evenly) lets extra wavefronts
// share one output tile; with few output tiles this replaces a split over workgroups, whose
// partial sums go through memory and a reduction launch.
//
// STAGES = 2 keeps two K-blocks in LDS: the block fetched during the previous iteration is
// written to the idle stage before the MFMAs of the current one are issued, so LDS writes and
// matrix work overlap and an iteration has one barrier instead of two.
template <class C, int KH, int KW, int STAGES = 2>
__global__ __launch_bounds__(C::THREADS, (C::THREADS > 512 ? 1 : 2)) void conv_taps_kernel(const ConvDev p) {
    fetch_now(p);
    constexpr int T = KH * KW;
    constexpr int CB = C::BK / T;  // input channels per K-block
    constexpr int Q = CB / 4;      // 128-bit pieces of a pixel's channel block
    static_assert(C::BK == CB * T && (CB == 8 || CB == 16), "K-block = 8 or 16 channels x taps");
    static_assert(C::BN * Q <= C::THREADS, "Q threads fetch the weights of one output channel");
    __shared__ __attribute__((aligned(16))) float lds[cmax(STAGES * C::LDS_FLOATS, red_floats<C>() + stage_floats<C>() + 4)];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wk = wave / (C::WGM * C::WGN), wsp = wave - wk * (C::WGM * C::WGN);
    const int wm = wsp / C::WGN, wn = wsp % C::WGN;
    const int t = remap_xcd_c(blockIdx.x, p.tiles_m * p.tiles_n);
    const int tm = t / p.tiles_n, tn = t - tm * p.tiles_n;
    const long m0 = (long)tm * C::BM, n0 = (long)tn * C::BN;
    const int split = blockIdx.z;
    const int cbeg = split * (int)p.kper;
    const int cend = (cbeg + (int)p.kper < p.Cin) ? cbeg + (int)p.kper : p.Cin;

    // Branch-free operand fetch: rows past the last pixel are clamped to it (computed, then
    // dropped at the store) and taps that fall into the padding read from a page of zeros with
    // a zero channel step, so every load in the loop is unconditional.
    constexpr int NVA = (C::BM * Q * T + C::THREADS - 1) / C::THREADS;
    const float* pa[NVA];
    int stepA[NVA];
#pragma unroll
    for (int i = 0; i < NVA; ++i) {
        int idx = i * C::THREADS + tid;
        if (idx > C::BM * Q * T - 1) idx = C::BM * Q * T - 1;
        const int row = idx / (Q * T), t2 = idx - row * (Q * T);
        const int tap = t2 / Q, cq = t2 % Q;
        long grow = m0 + row;
        if (grow > p.M - 1) grow = p.M - 1;
        const int wo = (int)(grow % p.Wo);
        const long tt = grow / p.Wo;
        const int ho = (int)(tt % p.Ho);
        const long n = tt / p.Ho;
        const int hi = ho * p.sh - p.ph + tap / KW;
        const int wi = wo * p.sw - p.pw + tap % KW;
        const bool inside = hi >= 0 && hi < p.H && wi >= 0 && wi < p.W;
        pa[i] = inside ? p.x + n * p.xs_n + (long)hi * p.xs_h + (long)wi * p.xs_w + cq * 4 : p.zeros;
        stepA[i] = inside ? 1 : 0;
    }
    // weight assignment: thread -> (col = tid / Q, cq = tid % Q)
    const int wcol = tid / Q, wcq = tid % Q;
    long wc = n0 + wcol;
    if (wc > p.Cout - 1) wc = p.Cout - 1;
    const float* __restrict__ wbase = p.w + (wc * (long)p.Cin + wcq * 4) * T;

    f32x16 acc[C::TM][C::TN];
    zero_acc<C>(acc);
    f32x4 ra[NVA];
    f32x4 rw[T];
    ColConsts<C::TN> cc;  // bias / batch-norm vectors of this wavefront's columns: requested now, used at the end
    if (wk == 0) cols_issue<C>(cc, p.ep, p.y, n0, wn, lane, (long)p.Cout);

    auto load_regs = [&](int c0) {
        if (c0 > cend - CB) c0 = cend - CB;  // look-ahead past the end re-reads the last block
#pragma unroll
        for (int i = 0; i < NVA; ++i) ra[i] = *reinterpret_cast<const f32x4*>(pa[i] + c0 * stepA[i]);
        if (tid < C::BN * Q) {
#pragma unroll
            for (int j = 0; j < T; ++j) rw[j] = *reinterpret_cast<const f32x4*>(wbase + (long)c0 * T + j * 4);
        }
    };
    auto store_lds = [&](int stage) {
        float* As = lds + stage * C::LDS_FLOATS;
        float* Bs = As + C::BM * C::LDK;
#pragma unroll
        for (int i = 0; i < NVA; ++i) {
            const int idx = i * C::THREADS + tid;
            const int row = idx / (Q * T), t2 = idx - row * (Q * T);
            if (idx < C::BM * Q * T) *reinterpret_cast<f32x4*>(As + row * C::LDK + t2 * 4) = ra[i];
        }
        if (tid < C::BN * Q) {
            // rw holds w[c][tap] for c = 0..3 (this thread's channel quad), flat index c*T + tap
#pragma unroll
            for (int tap = 0; tap < T; ++tap) {
                f32x4 v;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int f = c * T + tap;
                    v[c] = rw[f >> 2][f & 3];
                }
                *reinterpret_cast<f32x4*>(Bs + wcol * C::LDK + tap * CB + wcq * 4) = v;
            }
        }
    };

    load_regs(cbeg);
    if (wk == 0) cols_fold<C>(cc, p.ep);
    if (STAGES == 2) {
        store_lds(0);
        load_regs(cbeg + CB);
        __syncthreads();
        int cur = 0;
        for (int c0 = cbeg; c0 < cend; c0 += CB) {
            // the other stage was last read before the barrier that ended the previous iteration
            store_lds(cur ^ 1);
            load_regs(c0 + 2 * CB);
            const float* As = lds + cur * C::LDS_FLOATS;
            mma_block<C>(As, As + C::BM * C::LDK, acc, wm, wn, lane, wk);
            __syncthreads();
            cur ^= 1;
        }
    } else {
        for (int c0 = cbeg; c0 < cend; c0 += CB) {
            store_lds(0);
            __syncthreads();
            load_regs(c0 + CB);
            mma_block<C>(lds, lds + C::BM * C::LDK, acc, wm, wn, lane, wk);
            __syncthreads();
        }
    }
    if (!reduce_k_slices<C>(acc, lds, wk, wsp, lane)) return;
    float* partial = nullptr;
    if (p.splits > 1) {
        if (p.tickets) {
            if (!finish_split<C>(acc, p.ws, p.tickets, p.splits, t, split, wsp, lane,
                                 reinterpret_cast<unsigned*>(lds + red_floats<C>() + stage_floats<C>())))
                return;
        } else {
            partial = p.ws + (long)split * p.M * p.Cout;
        }
    }
    store_tile<C>(acc, wm, wn, lane, m0, n0, p.M, (long)p.Cout, p.y, p.ep, partial,
                  lds + red_floats<C>() + wsp * STAGE_BLOCK, &cc);
}

// Any kernel size / stride / padding / input layout; K ordered (c, kh, kw) as
// the weights are stored.  One wavefront gathers one k for 64 pixels at a time,
// so the k -> (c, kh, kw) decode is wavefront-uniform.
using ConvGenCfg = TileCfg<64, 64, 16, 2, 2>;

__global__ __launch_bounds__(ConvGenCfg::THREADS, 2) void conv_generic_kernel(const ConvDev p) {
    using C = ConvGenCfg;
    __shared__ __attribute__((aligned(16))) float lds[cmax(C::LDS_FLOATS, stage_floats<C>() + 4)];
    float* As = lds;
    float* Bs = lds + C::BM * C::LDK;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / C::WGN, wn = wave % C::WGN;
    const int t = blockIdx.x;
    const int tm = t / p.tiles_n, tn = t - tm * p.tiles_n;
    const long m0 = (long)tm * C::BM, n0 = (long)tn * C::BN;
    const int split = blockIdx.z;
    const long kbeg = (long)split * p.kper;
    const long kend = (kbeg + p.kper < p.K) ? kbeg + p.kper : p.K;

    // activation gather: thread -> pixel row (tid % 64), k slots wave + 4*i
    const int arow = tid & 63;
    const long grow = m0 + arow;
    const bool rvalid = grow < p.M;
    int hi0 = 0, wi0 = 0;
    long nbase = 0;
    if (rvalid) {
        const int wo = (int)(grow % p.Wo);
        const long tt = grow / p.Wo;
        const int ho = (int)(tt % p.Ho);
        const long n = tt / p.Ho;
        hi0 = ho * p.sh - p.ph;
        wi0 = wo * p.sw - p.pw;
        nbase = n * p.xs_n;
    }
    // weight loads: thread -> (k = tid % 16, col = tid/16 + 16*i)
    const int wk = tid & 15, wc0 = tid >> 4;
    const int khw = p.KH * p.KW;

    f32x16 acc[C::TM][C::TN];
    zero_acc<C>(acc);
    float ra[4], rb[4];
    auto load_regs = [&](long k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const long k = k0 + wave + 4 * i;
            float v = 0.f;
            if (rvalid && k < kend) {
                const int c = (int)(k / khw);
                const int rr = (int)(k - (long)c * khw);
                const int kh = rr / p.KW, kw = rr - kh * p.KW;
                const int hi = hi0 + kh, wi = wi0 + kw;
                if (hi >= 0 && hi < p.H && wi >= 0 && wi < p.W)
                    v = p.x[nbase + (long)c * p.xs_c + (long)hi * p.xs_h + (long)wi * p.xs_w];
            }
            ra[i] = v;
            const long col = n0 + wc0 + 16 * i;
            const long kk = k0 + wk;
            rb[i] = (col < p.Cout && kk < kend) ? p.w[col * p.K + kk] : 0.f;
        }
    };
    load_regs(kbeg);
    for (long k0 = kbeg; k0 < kend; k0 += C::BK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            As[arow * C::LDK + wave + 4 * i] = ra[i];
            Bs[(wc0 + 16 * i) * C::LDK + wk] = rb[i];
        }
        __syncthreads();
        if (k0 + C::BK < kend) load_regs(k0 + C::BK);
        mma_block<C>(As, Bs, acc, wm, wn, lane);
        __syncthreads();
    }
    float* partial = nullptr;
    if (p.splits > 1) {
        if (p.tickets) {
            if (!finish_split<C>(acc, p.ws, p.tickets, p.splits, t, split, wave, lane,
                                 reinterpret_cast<unsigned*>(lds + stage_floats<C>())))
                return;
        } else {
            partial = p.ws + (long)split * p.M * p.Cout;
        }
    }
    store_tile<C>(acc, wm, wn, lane, m0, n0, p.M, (long)p.Cout, p.y, p.ep, partial, lds + wave * STAGE_BLOCK);
}

using Conv3L = TileCfg<128, 128, 72, 2, 2>;
using Conv3M = TileCfg<64, 64, 72, 2, 2>;
using Conv3S = TileCfg<64, 64, 72, 2, 2, 3>;  // 12 wavefronts: 2x2 over the tile, 3 K slices
using Conv3T = TileCfg<32, 32, 72, 1, 1, 9>;  // 9 wavefronts, one k-group each
using Conv3U = TileCfg<32, 32, 72, 1, 1, 3>;  // 3 wavefronts
using Conv3T16 = TileCfg<32, 32, 144, 1, 1, 9>;  // as Conv3T with 16 input channels per K-block

// Depthwise convolution (groups == Cin == Cout), NHWC, weights [C][1][KH][KW]: HBM-bound, one
// thread per output pixel and channel quad, taps accumulated in registers, same fused epilogue
// as the MFMA kernels (folded batch-norm / bias, residual, activation).
struct DwDev {
    const float* x;
    const float* w;
    float* y;
    int H, W, C, KH, KW, Ho, Wo, sh, sw, ph, pw;
    long xp, yp;
    long total;  // N*Ho*Wo*(C/4)
    Epilogue ep;
};
__global__ __launch_bounds__(256) void depthwise_kernel(const DwDev p) {
    const long st = (long)gridDim.x * blockDim.x;
    const int C4 = p.C >> 2;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < p.total; i += st) {
        const int c = (int)(i % C4) * 4;
        long t = i / C4;
        const long row = t;  // output pixel index (n, ho, wo)
        const int wo = (int)(t % p.Wo);
        t /= p.Wo;
        const int ho = (int)(t % p.Ho);
        const long n = t / p.Ho;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        const float* wc = p.w + (long)c * p.KH * p.KW;
        const int kk = p.KH * p.KW;
        for (int kh = 0; kh < p.KH; ++kh) {
            const int hi = ho * p.sh - p.ph + kh;
            if (hi < 0 || hi >= p.H) continue;
            for (int kw = 0; kw < p.KW; ++kw) {
                const int wi = wo * p.sw - p.pw + kw;
                if (wi < 0 || wi >= p.W) continue;
                const f32x4 xv = *reinterpret_cast<const f32x4*>(p.x + ((n * p.H + hi) * p.W + wi) * p.xp + c);
                const int tap = kh * p.KW + kw;
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[j] += xv[j] * wc[j * kk + tap];
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float cs, ct;
            epilogue_column(p.ep, c + j, cs, ct);
            epilogue_store(p.ep, p.y, row, c + j, acc[j], cs, ct);
        }
    }
}

// The same for fixed K x K taps (3x3, 5x5), weights 16-byte aligned, row-major output with aligned
// rows and no beta term: the 4*K*K weights of the channel quad are fetched up front as vectors,
// every tap's load is unconditional (out-of-range taps read a clamped address and are zeroed by
// a select), so all K*K loads of a thread are in flight together, and the result leaves as one
// 128-bit store.
template <int KS>
__global__ __launch_bounds__(256) void depthwise_taps_kernel(const DwDev p) {
    constexpr int T = KS * KS;
    const long st = (long)gridDim.x * blockDim.x;
    const int C4 = p.C >> 2;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < p.total; i += st) {
        const int c = (int)(i % C4) * 4;
        long t = i / C4;
        const long row = t;
        const int wo = (int)(t % p.Wo);
        t /= p.Wo;
        const int ho = (int)(t % p.Ho);
        const long n = t / p.Ho;
        f32x4 wv[T];  // flat [channel j][tap]: element j*T + tap
        const f32x4* wq = reinterpret_cast<const f32x4*>(p.w + (long)c * T);
#pragma unroll
        for (int q = 0; q < T; ++q) wv[q] = wq[q];
        f32x4 xv[T];
        bool ok[T];
        const int hi0 = ho * p.sh - p.ph, wi0 = wo * p.sw - p.pw;
#pragma unroll
        for (int kh = 0; kh < KS; ++kh)
#pragma unroll
            for (int kw = 0; kw < KS; ++kw) {
                const int hi = hi0 + kh, wi = wi0 + kw;
                const int tap = kh * KS + kw;
                ok[tap] = hi >= 0 && hi < p.H && wi >= 0 && wi < p.W;
                const int hc = hi < 0 ? 0 : (hi >= p.H ? p.H - 1 : hi);
                const int wc = wi < 0 ? 0 : (wi >= p.W ? p.W - 1 : wi);
                xv[tap] = *reinterpret_cast<const f32x4*>(p.x + ((n * p.H + hc) * p.W + wc) * p.xp + c);
            }
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int tap = 0; tap < T; ++tap) {  // same order of additions as the general kernel
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int f = j * T + tap;
                const float xw = xv[tap][j] * wv[f >> 2][f & 3];
                acc[j] += ok[tap] ? xw : 0.f;
            }
        }
        f32x4 res = {0.f, 0.f, 0.f, 0.f};
        if (p.ep.residual) res = *reinterpret_cast<const f32x4*>(p.ep.residual + row * p.ep.ldr + c);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float cs, ct;
            epilogue_column(p.ep, c + j, cs, ct);
            float v = acc[j] * p.ep.alpha;
            v = v * cs + ct;
            if (p.ep.residual) v += res[j];
            acc[j] = apply_act(v, p.ep.act);
        }
        *reinterpret_cast<f32x4*>(p.y + row * p.ep.ldc + c) = acc;
    }
}

static int launch_depthwise(const ConvArgs& a, int Ho, int Wo, long xp, long yp, hipStream_t s) {
    if (a.groups != a.Cin || a.Cin != a.Cout) return K_EUNSUPPORTED;  // only groups == channels
    if (!a.x_nhwc || !a.y_nhwc || a.Cin % 4 != 0 || xp % 4 != 0) return K_EUNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(a.x) & 15) != 0) return K_EUNSUPPORTED;
    DwDev p;
    p.x = a.x;
    p.w = a.w;
    p.y = a.y;
    p.H = a.H;
    p.W = a.W;
    p.C = a.Cin;
    p.KH = a.KH;
    p.KW = a.KW;
    p.Ho = Ho;
    p.Wo = Wo;
    p.sh = a.sh;
    p.sw = a.sw;
    p.ph = a.ph;
    p.pw = a.pw;
    p.xp = xp;
    p.yp = yp;
    p.total = (long)a.N * Ho * Wo * (a.Cin / 4);
    EpilogueArgs ea = a.ep;
    if (ea.residual && ea.ldr == 0) ea.ldr = a.Cout;
    p.ep = make_epilogue(ea, yp);
    long blocks = (p.total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    const bool vec = a.KH == a.KW && (a.KH == 3 || a.KH == 5) && p.ep.beta == 0.f && (yp & 3) == 0 &&
                     (reinterpret_cast<uintptr_t>(a.w) & 15) == 0 && (reinterpret_cast<uintptr_t>(a.y) & 15) == 0 &&
                     (!p.ep.residual || ((p.ep.ldr & 3) == 0 && (reinterpret_cast<uintptr_t>(p.ep.residual) & 15) == 0));
    if (vec && a.KH == 3) {
        hipLaunchKernelGGL(depthwise_taps_kernel<3>, dim3((unsigned)blocks), dim3(256), 0, s, p);
        set_last_kernel("depthwise_3x3");
    } else if (vec) {
        hipLaunchKernelGGL(depthwise_taps_kernel<5>, dim3((unsigned)blocks), dim3(256), 0, s, p);
        set_last_kernel("depthwise_5x5");
    } else {
        hipLaunchKernelGGL(depthwise_kernel, dim3((unsigned)blocks), dim3(256), 0, s, p);
        set_last_kernel("depthwise_nhwc");
    }
    return (int)hipGetLastError();
}

static inline bool aligned16c(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// ---------------------------------------------------------------- 7x7 stride-2 stem (3 input channels)
// The first layer of the ResNets and DenseNets: 7x7, stride 2, padding 3, 3 -> Cout channels (Cout % 64 == 0).
// With 3 input channels the taps kernels' channel blocks do not apply and the general kernel spends its time on
// gather addresses (1x224x224: 16 us).  Here a workgroup owns 2 output rows x 32 output columns x 64 output
// channels: the input patch they read (3 channels x 10 rows x 69 columns) and the 64 filters, as they lie in
// memory, are put into LDS once, and every MFMA operand is then one LDS word at a compile-time offset from a
// per-lane base.
//
// K order.  v_mfma_f32_32x32x2_f32 takes k = 0 from lanes 0-31 and k = 1 from lanes 32-63.  The 7 filter rows are
// split 4 + 3 between the lane halves: step (c, j, kw) multiplies filter row kh = 4*half + j, so the two halves read
// patch and filter 4 rows apart -- constants that fold into the lanes' base addresses -- and 3 * 4 * 7 = 84 steps
// cover the 147 products.  Filter row 7 does not exist: in the 21 steps with j = 3 both operands of the upper half
// are replaced by zero (what the filter side reads instead is the next channel's first row, or the 8 floats of
// padding behind the last filter; the input side would read a row below the receptive field, whose Inf or NaN
// times zero must not reach the sum).
struct StemCfg {  // what store_tile needs to know: one 32x32 accumulator per wavefront, 2 x 2 wavefronts
    static constexpr int BM = 64, BN = 64, WGM = 2, WGN = 2, WGK = 1, THREADS = 256;
    static constexpr int WTM = 32, WTN = 32, TM = 1, TN = 1;
};
constexpr int kStemRows = 10, kStemCols = 69, kStemPitch = 72;  // patch rows 2*ty + kh (kh 0..7), columns 2*tx + kw
constexpr int kStemPatch = 3 * kStemRows * kStemPitch;          // floats
constexpr int kStemFilters = 64 * 147;
constexpr int kStemLds = kStemPatch + kStemFilters + 8;
static_assert(kStemFilters + 8 >= 4 * STAGE_BLOCK, "the filter area doubles as the write-out staging blocks");

__global__ __launch_bounds__(256, 2) void conv_stem7_kernel(const ConvDev p) {
    __shared__ __attribute__((aligned(16))) float lds[kStemLds];
    float* P = lds;
    float* Wt = lds + kStemPatch;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int r = lane & 31, h = lane >> 5;
    // workgroup -> (image, pair of output rows, block of 32 output columns, block of 64 output channels)
    const int tiles_x = (p.Wo + 31) >> 5, tiles_y = (p.Ho + 1) >> 1;
    int t = (int)blockIdx.x;
    const int tx0 = t % tiles_x;
    t /= tiles_x;
    const int ty0 = t % tiles_y;
    const int n = t / tiles_y;
    const int ho0 = ty0 * 2, wo0 = tx0 * 32;
    const int n0 = (int)blockIdx.y * 64;
    const int hi0 = ho0 * 2 - 3, wi0 = wo0 * 2 - 3;

    ColConsts<1> cc;
    cols_issue<StemCfg>(cc, p.ep, p.y, n0, wn, lane, (long)p.Cout);

    // the 64 filters: 64 * 147 contiguous floats, copied as they are (16-byte aligned: checked by the launcher)
    const f32x4* wsrc = reinterpret_cast<const f32x4*>(p.w + (long)n0 * 147);
    constexpr int NW4 = kStemFilters / 4;  // 2352
    f32x4 wv[(NW4 + 255) / 256];
#pragma unroll
    for (int it = 0; it < (NW4 + 255) / 256; ++it) {
        const int i = it * 256 + tid;
        wv[it] = wsrc[i < NW4 ? i : NW4 - 1];
    }
    // the input patch, zero outside the image (the padding): a wavefront per (channel, row) line of 69 columns
    const float* xn = p.x + (long)n * p.xs_n;
    float pv[8][2];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const int line = wave + 4 * q;  // 0..31, 30 lines exist
        const int c = line / kStemRows, row = line - c * kStemRows;
        const int hi = hi0 + row;
        const bool line_ok = line < 3 * kStemRows && hi >= 0 && hi < p.H;
        const float* src = xn + (long)(line_ok ? c : 0) * p.xs_c + (long)(line_ok ? hi : 0) * p.xs_h;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int col = lane + 64 * u;
            const int wi = wi0 + col;
            const bool ok = line_ok && col < kStemCols && wi >= 0 && wi < p.W;
            const float v = src[(long)(ok ? wi : 0) * p.xs_w];  // always a valid address: element (n, c, 0 or hi, 0 or wi)
            pv[q][u] = ok ? v : 0.f;
        }
    }
    cols_fold<StemCfg>(cc, p.ep);
#pragma unroll
    for (int it = 0; it < (NW4 + 255) / 256; ++it) {
        const int i = it * 256 + tid;
        if (i < NW4) *reinterpret_cast<f32x4*>(Wt + 4 * i) = wv[it];
    }
    if (tid < 8) Wt[kStemFilters + tid] = 0.f;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const int line = wave + 4 * q;
        if (line < 3 * kStemRows) {
            P[line * kStemPitch + lane] = pv[q][0];
            if (lane + 64 < kStemPitch) P[line * kStemPitch + lane + 64] = pv[q][1];
        }
    }
    __syncthreads();

    f32x16 acc[1][1];
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[0][0][v] = 0.f;
    const float* ap = P + (2 * wm + 4 * h) * kStemPitch + 2 * r;
    const float* bp = Wt + (wn * 32 + r) * 147 + h * 28;
#pragma unroll
    for (int c = 0; c < 3; ++c)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int kw = 0; kw < 7; ++kw) {
                float a = ap[(c * kStemRows + j) * kStemPitch + kw];
                float b = bp[c * 49 + j * 7 + kw];
                if (j == 3) {  // filter row 7: both operands, so that an Inf or NaN in the input row it would meet stays out
                    a = h ? 0.f : a;
                    b = h ? 0.f : b;
                }
                acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[0][0], 0, 0, 0);
            }
    __syncthreads();  // the operands are no longer read: the filter area becomes the write-out staging blocks

    // rows of this wavefront's block = 32 consecutive pixels of output row ho0 + wm; those past the end of the
    // row (or a row past the image) are cut off through the row bound
    const int ho = ho0 + wm;
    const long m0 = ((long)n * p.Ho + ho) * p.Wo + wo0;
    int valid = p.Wo - wo0;
    if (valid > 32) valid = 32;
    if (ho >= p.Ho) valid = 0;
    store_tile<StemCfg>(acc, 0, wn, lane, m0, (long)n0, m0 + valid, (long)p.Cout, p.y, p.ep, nullptr,
                        Wt + wave * STAGE_BLOCK, &cc);
}

int launch_conv2d(const ConvArgs& a, const Workspace& ws, hipStream_t s) {
    if (!a.x || !a.w || !a.y) return K_EINVAL;
    if (a.N <= 0 || a.H <= 0 || a.W <= 0 || a.Cin <= 0 || a.Cout <= 0 || a.KH <= 0 || a.KW <= 0) return K_EINVAL;
    if (a.sh <= 0 || a.sw <= 0 || a.ph < 0 || a.pw < 0) return K_EINVAL;
    const int Ho = (a.H + 2 * a.ph - a.KH) / a.sh + 1;
    const int Wo = (a.W + 2 * a.pw - a.KW) / a.sw + 1;
    if (Ho <= 0 || Wo <= 0) return K_EINVAL;
    const long M = (long)a.N * Ho * Wo;

    if ((a.x_pitch && (!a.x_nhwc || a.x_pitch < a.Cin)) || (a.y_pitch && (!a.y_nhwc || a.y_pitch < a.Cout)))
        return K_EINVAL;
    const long xp = a.x_pitch ? a.x_pitch : a.Cin;   // floats between pixels (NHWC)
    const long yp = a.y_pitch ? a.y_pitch : a.Cout;
    if (a.groups != 1 && a.groups == a.Cin && a.Cin == a.Cout) {
        const int r = launch_depthwise(a, Ho, Wo, xp, yp, s);
        if (r != K_EUNSUPPORTED) return r;  // else: as a grouped convolution, below
    }
    if (a.groups != 1) {
        // General grouped convolution (cudnnSetConvolutionGroupCount, cuda_server.hpp:671): group g maps input
        // channels [g*Cin/G, (g+1)*Cin/G) to output channels [g*Cout/G, (g+1)*Cout/G) with its own block of
        // the [Cout][Cin/G][KH][KW] filter.  In NHWC each group is a convolution over a channel slice of x
        // written into a channel slice of y, which the kernels serve through their pixel pitches; one launch
        // per group.
        if (a.groups < 1 || a.Cin % a.groups || a.Cout % a.groups) return K_EINVAL;
        if (!a.x_nhwc || !a.y_nhwc) return K_EUNSUPPORTED;
        const int cig = a.Cin / a.groups, cog = a.Cout / a.groups;
        for (int g = 0; g < a.groups; ++g) {
            ConvArgs b = a;
            b.groups = 1;
            b.Cin = cig;
            b.Cout = cog;
            b.x = a.x + (long)g * cig;
            b.y = a.y + (long)g * cog;
            b.w = a.w + (long)g * cog * cig * a.KH * a.KW;
            b.x_pitch = xp;
            b.y_pitch = yp;
            if (b.ep.bias) b.ep.bias += (long)g * cog;
            if (b.ep.bn_scale) {
                b.ep.bn_scale += (long)g * cog;
                b.ep.bn_bias += (long)g * cog;
                b.ep.bn_mean += (long)g * cog;
                b.ep.bn_var += (long)g * cog;
            }
            if (b.ep.residual) {
                if (b.ep.ldr == 0) b.ep.ldr = a.Cout;
                b.ep.residual += (long)g * cog;
            }
            const int r = launch_conv2d(b, ws, s);
            if (r) return r;
        }
        return 0;
    }

    // 1x1 over NHWC is a dense GEMM, with a row gather when strided.
    if (a.KH == 1 && a.KW == 1 && a.ph == 0 && a.pw == 0 && a.x_nhwc && a.y_nhwc) {
        GemmArgs g;
        g.X = a.x;
        g.Y = a.w;
        g.C = a.y;
        g.M = M;
        g.N = a.Cout;
        g.K = a.Cin;
        g.xs_r = xp;
        g.xs_k = 1;
        g.ys_c = a.Cin;
        g.ys_k = 1;
        g.ldc = yp;
        if (a.sh != 1 || a.sw != 1) {
            g.gather = 1;
            g.Ho = Ho;
            g.Wo = Wo;
            g.H = a.H;
            g.W = a.W;
            g.sh = a.sh;
            g.sw = a.sw;
        }
        g.ep = a.ep;
        if (g.ep.residual && g.ep.ldr == 0) g.ep.ldr = a.Cout;
        return launch_gemm(g, ws, s);
    }

    ConvDev p;
    p.x = a.x;
    p.w = a.w;
    p.y = a.y;
    p.N = a.N;
    p.H = a.H;
    p.W = a.W;
    p.Cin = a.Cin;
    p.Cout = a.Cout;
    p.KH = a.KH;
    p.KW = a.KW;
    p.Ho = Ho;
    p.Wo = Wo;
    p.sh = a.sh;
    p.sw = a.sw;
    p.ph = a.ph;
    p.pw = a.pw;
    if (a.x_nhwc) {
        p.xs_c = 1;
        p.xs_w = xp;
        p.xs_h = (long)a.W * xp;
        p.xs_n = (long)a.H * a.W * xp;
    } else {
        p.xs_w = 1;
        p.xs_h = a.W;
        p.xs_c = (long)a.H * a.W;
        p.xs_n = (long)a.Cin * a.H * a.W;
    }
    p.M = M;
    p.K = (long)a.Cin * a.KH * a.KW;
    p.ws = ws.ptr;
    p.tickets = nullptr;  // set below once the tile grid is known
    p.zeros = ws.zeros;
    EpilogueArgs ea = a.ep;
    if (ea.residual && ea.ldr == 0) ea.ldr = a.Cout;
    p.ep = make_epilogue(ea, yp);
    if (!a.y_nhwc) {
        p.ep.out_nchw = 1;
        p.ep.howo = (long)Ho * Wo;
        p.ep.ncols = a.Cout;
    }

    const bool taps_ok = a.x_nhwc && (a.Cin % 8 == 0) && (xp % 4 == 0) && aligned16c(a.x) && aligned16c(a.w) &&
                         ws.zeros != nullptr;
    const bool fast3 = a.KH == 3 && a.KW == 3 && taps_ok;
    const int other_taps = !taps_ok ? 0 : (a.KH == 1 && a.KW == 7) ? 1 : (a.KH == 7 && a.KW == 1) ? 2
                           : (a.KH == 1 && a.KW == 3) ? 3 : (a.KH == 3 && a.KW == 1) ? 4 : 0;
    // TORPOR_CONV_STEM=0: the general kernel for the 7x7 stem, as before
    static const bool stem_on = getenv("TORPOR_CONV_STEM") == nullptr || atoi(getenv("TORPOR_CONV_STEM")) != 0;
    const bool stem7 = stem_on && a.KH == 7 && a.KW == 7 && a.sh == 2 && a.sw == 2 && a.ph == 3 && a.pw == 3 &&
                       a.Cin == 3 && a.Cout % 64 == 0 && a.Cout / 64 <= 65535 && aligned16c(a.w) &&
                       (long)a.N * ((Ho + 1) / 2) * ((Wo + 31) / 32) < (1L << 31);
    if (other_taps) {
        // the asymmetric shapes (Inception): one 64x64 tile shape, split over channel blocks.  (5x5 stays on
        // the general kernel: a 200-wide K-block leaves one workgroup per CU and measured 2x slower.)
        const int T = a.KH * a.KW;
        // Few 64x64 tiles (Inception's 17x17 and 8x8 maps at batch 1: 10 to 15 of them, whose K then had to be
        // cut 16 to 25 ways and summed by a second launch): 32x32 tiles with one wavefront per tap, as for the
        // 3x3 shapes, split so that every workgroup still has a CU to itself.  TORPOR_CONV_TAPS_SMALL=0: as before.
        static const bool small_on = getenv("TORPOR_CONV_TAPS_SMALL") == nullptr || atoi(getenv("TORPOR_CONV_TAPS_SMALL")) != 0;
        const long t64 = ((M + 63) / 64) * ((a.Cout + 63) / 64);
        const long t32 = ((M + 31) / 32) * ((a.Cout + 31) / 32);
        if (small_on && t64 < num_cu() / 2 && t32 <= kSplitTickets && a.Cin >= 32) {
            p.tiles_m = (int)((M + 31) / 32);
            p.tiles_n = (a.Cout + 31) / 32;
            const bool cb16 = a.Cin % 16 == 0;
            int cap = (int)(num_cu() / t32);
            if (cap > 8) cap = 8;
            long kper_k = p.K;
            p.splits = cap >= 2 ? choose_splits(t32, p.K, (cb16 ? 16 : 8) * T, 32 * 32, ws.ptr ? ws.bytes : 0, &kper_k, cap, true, 0) : 1;
            p.kper = kper_k / T;
            p.tickets = split_tickets(ws, t32, p.splits);
            dim3 grid((unsigned)t32, 1, p.splits);
            static const char* const nms[5] = {"", "conv_taps_1x7_32x32_k7", "conv_taps_7x1_32x32_k7", "conv_taps_1x3_32x32_k3",
                                               "conv_taps_3x1_32x32_k3"};
            using T7 = TileCfg<32, 32, 56, 1, 1, 7>;
            using T7w = TileCfg<32, 32, 112, 1, 1, 7>;
            using T3 = TileCfg<32, 32, 24, 1, 1, 3>;
            using T3w = TileCfg<32, 32, 48, 1, 1, 3>;
            switch (other_taps * 2 + (cb16 ? 1 : 0)) {
                case 2: hipLaunchKernelGGL((conv_taps_kernel<T7, 1, 7, 1>), grid, dim3(T7::THREADS), 0, s, p); break;
                case 3: hipLaunchKernelGGL((conv_taps_kernel<T7w, 1, 7, 1>), grid, dim3(T7w::THREADS), 0, s, p); break;
                case 4: hipLaunchKernelGGL((conv_taps_kernel<T7, 7, 1, 1>), grid, dim3(T7::THREADS), 0, s, p); break;
                case 5: hipLaunchKernelGGL((conv_taps_kernel<T7w, 7, 1, 1>), grid, dim3(T7w::THREADS), 0, s, p); break;
                case 6: hipLaunchKernelGGL((conv_taps_kernel<T3, 1, 3, 1>), grid, dim3(T3::THREADS), 0, s, p); break;
                case 7: hipLaunchKernelGGL((conv_taps_kernel<T3w, 1, 3, 1>), grid, dim3(T3w::THREADS), 0, s, p); break;
                case 8: hipLaunchKernelGGL((conv_taps_kernel<T3, 3, 1, 1>), grid, dim3(T3::THREADS), 0, s, p); break;
                default: hipLaunchKernelGGL((conv_taps_kernel<T3w, 3, 1, 1>), grid, dim3(T3w::THREADS), 0, s, p); break;
            }
            set_last_kernel(nms[other_taps]);
            int err = (int)hipGetLastError();
            if (err) return err;
            if (p.splits > 1 && !p.tickets) return launch_splitk_reduce(ws.ptr, p.splits, M, a.Cout, a.y, p.ep, s);
            return 0;
        }
        p.tiles_m = (int)((M + 63) / 64);
        p.tiles_n = (a.Cout + 63) / 64;
        long kper_k = p.K;
        p.splits = choose_splits((long)p.tiles_m * p.tiles_n, p.K, 8 * T, 64 * 64, ws.ptr ? ws.bytes : 0, &kper_k);
        p.kper = kper_k / T;
        p.tickets = split_tickets(ws, (long)p.tiles_m * p.tiles_n, p.splits);
        dim3 grid(p.tiles_m * p.tiles_n, 1, p.splits);
        switch (other_taps) {
            case 1: hipLaunchKernelGGL((conv_taps_kernel<TileCfg<64, 64, 56, 2, 2>, 1, 7>), grid, dim3(256), 0, s, p); break;
            case 2: hipLaunchKernelGGL((conv_taps_kernel<TileCfg<64, 64, 56, 2, 2>, 7, 1>), grid, dim3(256), 0, s, p); break;
            case 3: hipLaunchKernelGGL((conv_taps_kernel<TileCfg<64, 64, 24, 2, 2>, 1, 3>), grid, dim3(256), 0, s, p); break;
            default: hipLaunchKernelGGL((conv_taps_kernel<TileCfg<64, 64, 24, 2, 2>, 3, 1>), grid, dim3(256), 0, s, p); break;
        }
        static const char* const nm[5] = {"", "conv_taps_1x7_64x64", "conv_taps_7x1_64x64", "conv_taps_1x3_64x64",
                                          "conv_taps_3x1_64x64"};
        set_last_kernel(nm[other_taps]);
    } else if (fast3) {
        // Stride 1: Winograd F(2x2, 3x3), 2.25 times fewer multiplications (winograd.hip).  TORPOR_WINOGRAD=0: the
        // direct kernels below for every 3x3.
        // (read per call, so that one process can compare the two paths)
        const char* wino_env = getenv("TORPOR_WINOGRAD");
        const bool wino_on = wino_env == nullptr || atoi(wino_env) != 0;
        if (wino_on && a.sh == 1 && a.sw == 1 && a.ph == 1 && a.pw == 1) {
            const int r = launch_conv3x3_winograd(a, ws, s);
            if (r != K_EUNSUPPORTED) return r;
        }
        const long tl = ((M + 127) / 128) * ((a.Cout + 127) / 128);
        const long t64 = ((M + 63) / 64) * ((a.Cout + 63) / 64);
        static const int forced = getenv("TORPOR_CONV3_CFG") ? atoi(getenv("TORPOR_CONV3_CFG")) : -1;
        // 0: 128x128, 1: 64x64, 2: 64x64 with 3 K slices, 3: 32x32 with 9 K slices, 4: 32x32 with 3
        // Measured on MI355X (ResNet shapes, 1.85 GFLOP each): with between half a tile and one
        // tile per CU, three K slices per 64x64 tile beat a 2-3 way split over workgroups
        // (8x28x28x128: 38.8 -> 32.9 us); a short K with many pixels runs best as 32x32 tiles
        // with nine K slices (1x56x56x64: 13.5 -> 9.0 us); elsewhere 64x64 tiles, split over
        // workgroups when there are fewer tiles than CUs.
        const long t32 = ((M + 31) / 32) * ((a.Cout + 31) / 32);
        int cfg = tl >= 2L * num_cu() ? 0 : 1;
        if (cfg == 1 && t64 >= num_cu() / 2 && t64 < num_cu()) cfg = 2;
        if (cfg == 1 && t64 < num_cu() / 4 && t32 >= num_cu() / 2 && a.Cin <= 128) cfg = 3;
        // Few 64x64 tiles (batch 1): 32x32 tiles with nine K slices, split over channel blocks as well
        // when even those leave CUs idle -- up to eight slots, summed inside the launch.  Its workgroups
        // are short-lived, where a 64x64 tile with a deep split pays a long serial chain per wavefront
        // and a reduction launch.  TORPOR_CONV3_SMALL=0 restores the old rule, =n moves the bound to
        // t64 < n.
        static const int small_bound = getenv("TORPOR_CONV3_SMALL") ? atoi(getenv("TORPOR_CONV3_SMALL")) : num_cu() / 4;
        // (only where the launch is bound by latency, not by matrix work: ResNet-152 batch 8, 392 pixels x 512
        // channels, 1.85 GFLOP, runs 56 us this way against 30 us as 64x64 tiles)
        const bool small = cfg == 1 && t64 < small_bound && 2.0 * (double)M * a.Cout * (double)p.K < 6.0e8;
        if (small) cfg = 3;
        if (forced >= 0 && forced <= 4) cfg = forced;
        const int bm = cfg == 0 ? 128 : cfg <= 2 ? 64 : 32;
        p.tiles_m = (int)((M + bm - 1) / bm);
        p.tiles_n = (a.Cout + bm - 1) / bm;
        const long tiles = (long)p.tiles_m * p.tiles_n;
        // split over channel blocks of 8 (one K-block each)
        long kper_k = p.K;
        p.splits = 1;
        bool cb16 = false;
        static const bool pairs = getenv("TORPOR_CONV_PAIRS") != nullptr;
        if (cfg <= 1) p.splits = choose_splits(tiles, p.K, 72, (long)bm * bm, ws.ptr ? ws.bytes : 0, &kper_k, 32, pairs);
        if (cfg == 3) {
            // Nine-wavefront workgroups do not share a CU well: two of them on one CU take 2.4x as long per
            // K-block as one alone, so the split stops where every workgroup still has a CU to itself
            // (1x14x14x256>256, 56 tiles: 4 slots 9.8 us, 8 slots 11.4 us; 1x56x56x64>64, 196 tiles: unsplit
            // 7.1 us, 2 slots 10.1 us).  TORPOR_CONV_PAIRS=1 keeps the earlier rule (two workgroups per CU).
            int cap = pairs ? 8 : (int)(num_cu() / tiles);
            if (cap > 8) cap = 8;
            // K-blocks of 16 input channels where the channel count allows: a wavefront then issues 8 MFMAs between
            // two barriers instead of 4 (ResNet-50 batch 1: 10.6 -> 9.9 us per launch; TORPOR_CONV3_CB16=0: always 8)
            static const bool cb16_on = getenv("TORPOR_CONV3_CB16") == nullptr || atoi(getenv("TORPOR_CONV3_CB16")) != 0;
            cb16 = cb16_on && a.Cin % 16 == 0;
            p.splits = cap >= 2 ? choose_splits(tiles, p.K, cb16 ? 144 : 72, 32 * 32, ws.ptr ? ws.bytes : 0, &kper_k, cap, true, 0) : 1;
            // ... but not where the coarser blocks cost parallelism: a split keeps at least four K-blocks per slot,
            // so few channels in blocks of 16 allow half as many slots (DenseNet's 128 -> 32 layers, 7 tiles: 2
            // slots of 4 blocks of 16 run 8.8 us, 4 slots of 4 blocks of 8 run 6.9 us)
            if (cb16 && cap >= 2) {
                long kper8 = p.K;
                const int splits8 = choose_splits(tiles, p.K, 72, 32 * 32, ws.ptr ? ws.bytes : 0, &kper8, cap, true, 0);
                if (splits8 > p.splits) {
                    cb16 = false;
                    p.splits = splits8;
                    kper_k = kper8;
                }
            }
        }
        p.kper = kper_k / 9;  // channels per split (multiple of 8)
        p.tickets = split_tickets(ws, (long)p.tiles_m * p.tiles_n, p.splits);
        dim3 grid(p.tiles_m * p.tiles_n, 1, p.splits);
        switch (cfg) {
            case 0:
                hipLaunchKernelGGL((conv_taps_kernel<Conv3L, 3, 3, 1>), grid, dim3(Conv3L::THREADS), 0, s, p);
                set_last_kernel("conv3x3_fast_128x128");
                break;
            case 1:
                // two LDS stages halve the workgroups a CU can hold: only when all of them still fit at once
                if (tiles * p.splits <= 2L * num_cu())
                    hipLaunchKernelGGL((conv_taps_kernel<Conv3M, 3, 3, 2>), grid, dim3(Conv3M::THREADS), 0, s, p);
                else
                    hipLaunchKernelGGL((conv_taps_kernel<Conv3M, 3, 3, 1>), grid, dim3(Conv3M::THREADS), 0, s, p);
                set_last_kernel("conv3x3_fast_64x64");
                break;
            case 2:
                hipLaunchKernelGGL((conv_taps_kernel<Conv3S, 3, 3>), grid, dim3(Conv3S::THREADS), 0, s, p);
                set_last_kernel("conv3x3_fast_64x64_k3");
                break;
            case 3:
                if (cb16) {
                    hipLaunchKernelGGL((conv_taps_kernel<Conv3T16, 3, 3, 1>), grid, dim3(Conv3T16::THREADS), 0, s, p);
                    set_last_kernel("conv3x3_fast_32x32_k9");
                } else {
                    hipLaunchKernelGGL((conv_taps_kernel<Conv3T, 3, 3, 1>), grid, dim3(Conv3T::THREADS), 0, s, p);
                    set_last_kernel("conv3x3_fast_32x32_k9");
                }
                break;
            default:
                hipLaunchKernelGGL((conv_taps_kernel<Conv3U, 3, 3, 1>), grid, dim3(Conv3U::THREADS), 0, s, p);
                set_last_kernel("conv3x3_fast_32x32_k3");
                break;
        }
    } else if (stem7) {
        const long wgs = (long)a.N * ((Ho + 1) / 2) * ((Wo + 31) / 32);
        p.splits = 1;
        hipLaunchKernelGGL(conv_stem7_kernel, dim3((unsigned)wgs, (unsigned)(a.Cout / 64)), dim3(256), 0, s, p);
        set_last_kernel("conv_stem7x7_s2");
    } else {
        p.tiles_m = (int)((M + 63) / 64);
        p.tiles_n = (a.Cout + 63) / 64;
        const long tiles = (long)p.tiles_m * p.tiles_n;
        p.splits = choose_splits(tiles, p.K, 16, 64 * 64, ws.ptr ? ws.bytes : 0, &p.kper);
        p.tickets = split_tickets(ws, (long)p.tiles_m * p.tiles_n, p.splits);
        dim3 grid(p.tiles_m * p.tiles_n, 1, p.splits);
        hipLaunchKernelGGL(conv_generic_kernel, grid, dim3(256), 0, s, p);
        set_last_kernel("conv_generic_64x64");
    }
    int err = (int)hipGetLastError();
    if (err) return err;
    if (p.splits > 1 && !p.tickets) return launch_splitk_reduce(ws.ptr, p.splits, M, a.Cout, a.y, p.ep, s);
    return 0;
}

}  // namespace tpk
