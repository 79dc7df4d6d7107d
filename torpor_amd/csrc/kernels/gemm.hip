// Dense / strided-batched fp32 GEMM on MFMA for gfx950.
//
// Replaces the cublasSgemm and cublasSgemmStridedBatched call sites of the
// reference executor (include/server/cuda_server.hpp:502-550).  The operation is
// expressed row-major as C[r][c] = sum_k X(r,k) * Y(c,k); the C-ABI layer maps
// the column-major (transa, transb) convention onto the four stride combos.
//
//   gemm_fast_kernel<Cfg, YKC>  X rows K-contiguous, loaded with dwordx4;
//                               Y either K-contiguous (YKC) or c-contiguous.
//   gemm_generic_kernel         any strides / alignment, scalar loads.
//   splitk_reduce_kernel        deterministic reduction of split-K partials
//                               with the fused epilogue.
#include "kernels.hpp"
#include "mfma_tile.hpp"

#include <cstdlib>

// Cycle stamps for kernel-phase measurements: an experiment harness that includes this file defines
// TP_CLK before it; in the library the hooks are empty.
#ifndef TP_CLK
#define TP_CLK(n)
#endif

namespace tpk {

static int g_num_cu = 256;
static thread_local const char* g_last_kernel = "";

void kernels_init(int device) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess && prop.multiProcessorCount > 0)
        g_num_cu = prop.multiProcessorCount;
}
const char* last_kernel_name() { return g_last_kernel; }
void set_last_kernel(const char* n) { g_last_kernel = n; }
int num_cu() { return g_num_cu; }

struct GemmDev {
    const float* X;
    const float* Y;
    float* C;
    long M, N, K;
    long xs_r, xs_k, ys_c, ys_k;
    int nb1;
    long xb0, xb1, yb0, yb1, cb0, cb1;
    int gather, Ho, Wo, H, W, sh, sw;
    int splits;
    long kper;
    float* ws;
    unsigned* tickets;  // non-null: the split is summed inside the launch (finish_split)
    int tiles_m, tiles_n;
    int xr, xc;  // the 8 XCDs form an xr x xc grid over the tile grid (xr*xc == 8), 0 = linear mapping
    // the rectangle of each XCD (first tile row / column, width, height), worked out on the host: in the
    // kernel the same arithmetic is four 64-bit divisions, about two thousand cycles before the first load
    struct Rect {
        unsigned short r0, c0, w, h;
    } rect[8];
    Epilogue ep;
    // batch-norm (+ ReLU) of the X operand per K index (gemm_clean_kernel<..., APRE = true> only)
    const float* pre_gamma;
    const float* pre_beta;
    const float* pre_mean;
    const float* pre_var;
    float pre_eps;
    int pre_relu;
};

// Workgroups are handed to the 8 XCDs round-robin by linear id; remap so that
// each XCD (own L2) works on a contiguous run of tiles.
__device__ __forceinline__ int remap_xcd(int bid, int n) {
    const int q = n >> 3, rem = n & 7;
    const int xcd = bid & 7, local = bid >> 3;
    return xcd * q + (xcd < rem ? xcd : rem) + local;
}

// Workgroup -> tile with a 2-D partition over the XCDs.  XCD x = bid % 8 owns the rectangle
// (x / xc, x % xc) of an xr x xc split of the tile grid, so that its private L2 sees only
// 1/xr of the X rows and 1/xc of the Y rows.  The grid is padded to 8 * (largest rectangle);
// workgroups beyond their XCD's rectangle return false and exit.
__device__ __forceinline__ bool tile_of(const GemmDev& p, int bid, int* tm, int* tn, int* t) {
    if (p.xr <= 0) {
        const int n = p.tiles_m * p.tiles_n;
        if (bid >= n) return false;
        *t = p.xr == 0 ? remap_xcd(bid, n) : bid;
        *tm = *t / p.tiles_n;
        *tn = *t - *tm * p.tiles_n;
        return true;
    }
    const int xcd = bid & 7;
    const unsigned local = (unsigned)bid >> 3;
    const unsigned w = p.rect[xcd].w, h = p.rect[xcd].h;
    if (local >= w * h) return false;
    const unsigned lr = local / w;
    *tm = (int)(p.rect[xcd].r0 + lr);
    *tn = (int)(p.rect[xcd].c0 + (local - lr * w));
    *t = *tm * p.tiles_n + *tn;
    return true;
}

__device__ __forceinline__ void fetch_now(const GemmDev& p) {
    fetch_now(p.X);
    fetch_now(p.Y);
    fetch_now(p.C);
    fetch_now(p.M);
    fetch_now(p.N);
    fetch_now(p.K);
    fetch_now(p.xs_r);
    fetch_now(p.ys_c);
    fetch_now(p.ys_k);
    fetch_now(p.nb1);
    fetch_now(p.gather);
    fetch_now(p.splits);
    fetch_now(p.kper);
    fetch_now(p.ws);
    fetch_now(p.tickets);
    fetch_now(p.tiles_m);
    fetch_now(p.tiles_n);
    fetch_now(p.xr);
    fetch_now(p.ep);
}

__device__ __forceinline__ long gather_row(const GemmDev& p, long grow) {
    if (!p.gather) return grow;
    const long wo = grow % p.Wo;
    const long t = grow / p.Wo;
    const long ho = t % p.Ho;
    const long n = t / p.Ho;
    return (n * p.H + ho * p.sh) * p.W + wo * p.sw;
}

template <class C, bool YKC>
__global__ __launch_bounds__(C::THREADS, (C::TM * C::TN >= 4 ? 1 : 2)) void gemm_fast_kernel(const GemmDev p) {
    fetch_now(p);
    // two LDS stages: while the MFMAs read one, the next K-block is written to the other, so
    // the loop needs a single barrier per K-block
    __shared__ __attribute__((aligned(16))) float lds[cmax(2 * C::LDS_FLOATS, stage_floats<C>() + 4)];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / C::WGN, wn = wave % C::WGN;
    int tm, tn, t;
    if (!tile_of(p, blockIdx.x, &tm, &tn, &t)) return;
    const long m0 = (long)tm * C::BM, n0 = (long)tn * C::BN;

    int split = 0, batch = blockIdx.z;
    if (p.splits > 1) {
        split = blockIdx.z;
        batch = 0;
    }
    const int b0 = batch / p.nb1, b1 = batch - b0 * p.nb1;
    const float* __restrict__ X = p.X + b0 * p.xb0 + b1 * p.xb1;
    const float* __restrict__ Y = p.Y + b0 * p.yb0 + b1 * p.yb1;
    float* __restrict__ Cc = p.C + b0 * p.cb0 + b1 * p.cb1;
    const long kbeg = (long)split * p.kper;
    const long kend = (kbeg + p.kper < p.K) ? kbeg + p.kper : p.K;

    constexpr int KV = C::BK / 4;
    constexpr int NVA = (C::BM * KV + C::THREADS - 1) / C::THREADS;
    constexpr int NVB_KC = (C::BN * KV + C::THREADS - 1) / C::THREADS;
    constexpr int CV = C::BN / 4;
    constexpr int NVB_CC = (C::BK * CV + C::THREADS - 1) / C::THREADS;
    constexpr int NVB = YKC ? NVB_KC : NVB_CC;

    long offA[NVA];
#pragma unroll
    for (int i = 0; i < NVA; ++i) {
        const int idx = i * C::THREADS + tid;
        const int row = idx / KV, kq = idx - row * KV;
        offA[i] = -1;
        if (idx < C::BM * KV && m0 + row < p.M) offA[i] = gather_row(p, m0 + row) * p.xs_r + kq * 4;
    }
    long offB[NVB];
#pragma unroll
    for (int i = 0; i < NVB; ++i) {
        const int idx = i * C::THREADS + tid;
        offB[i] = -1;
        if (YKC) {
            const int col = idx / KV, kq = idx - col * KV;
            if (idx < C::BN * KV && n0 + col < p.N) offB[i] = (n0 + col) * p.ys_c + kq * 4;
        } else {
            const int cq = idx % CV;
            if (idx < C::BK * CV && n0 + cq * 4 < p.N) offB[i] = n0 + cq * 4;
        }
    }

    f32x16 acc[C::TM][C::TN];
    zero_acc<C>(acc);
    // two register sets: the global loads run two K-blocks ahead of the MFMAs
    f32x4 ra0[NVA], rb0[NVB], ra1[NVA], rb1[NVB];

    auto load_regs = [&](f32x4 (&ra)[NVA], f32x4 (&rb)[NVB], long k0) {
#pragma unroll
        for (int i = 0; i < NVA; ++i) {
            const int idx = i * C::THREADS + tid;
            const int kq = idx % KV;
            f32x4 v = {0.f, 0.f, 0.f, 0.f};
            if (offA[i] >= 0 && k0 + kq * 4 < kend) v = *reinterpret_cast<const f32x4*>(X + offA[i] + k0);
            ra[i] = v;
        }
#pragma unroll
        for (int i = 0; i < NVB; ++i) {
            const int idx = i * C::THREADS + tid;
            f32x4 v = {0.f, 0.f, 0.f, 0.f};
            if (YKC) {
                const int kq = idx % KV;
                if (offB[i] >= 0 && k0 + kq * 4 < kend) v = *reinterpret_cast<const f32x4*>(Y + offB[i] + k0);
            } else {
                const int kk = idx / CV;
                const long k = k0 + kk;
                if (offB[i] >= 0 && k < kend) {
                    const float* src = Y + k * p.ys_k + offB[i];
                    if (offB[i] + 3 < p.N) {
                        v = *reinterpret_cast<const f32x4*>(src);
                    } else {
                        v[0] = src[0];
                        if (offB[i] + 1 < p.N) v[1] = src[1];
                        if (offB[i] + 2 < p.N) v[2] = src[2];
                    }
                }
            }
            rb[i] = v;
        }
    };
    auto store_lds = [&](const f32x4 (&ra)[NVA], const f32x4 (&rb)[NVB], int stage) {
        float* As = lds + stage * C::LDS_FLOATS;
        float* Bs = As + C::BM * C::LDK;
#pragma unroll
        for (int i = 0; i < NVA; ++i) {
            const int idx = i * C::THREADS + tid;
            const int row = idx / KV, kq = idx - row * KV;
            if (idx < C::BM * KV) *reinterpret_cast<f32x4*>(As + row * C::LDK + kq * 4) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < NVB; ++i) {
            const int idx = i * C::THREADS + tid;
            if (YKC) {
                const int col = idx / KV, kq = idx - col * KV;
                if (idx < C::BN * KV) *reinterpret_cast<f32x4*>(Bs + col * C::LDK + kq * 4) = rb[i];
            } else {
                const int kk = idx / CV, cq = idx - kk * CV;
                if (idx < C::BK * CV) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) Bs[(cq * 4 + j) * C::LDK + kk] = rb[i][j];
                }
            }
        }
    };

    // K-block i lives in LDS stage i&1 and travels through register set i&1.  While block i is
    // multiplied, block i+2 is requested from memory and block i+1 (requested one iteration ago)
    // moves from registers to the other LDS stage; one barrier per K-block.  Loads past the end
    // of K are predicated off and yield zeros, so the tail needs no special casing.
    const float* As0 = lds;
    const float* As1 = lds + C::LDS_FLOATS;
    load_regs(ra0, rb0, kbeg);
    load_regs(ra1, rb1, kbeg + C::BK);
    store_lds(ra0, rb0, 0);
    __syncthreads();
    for (long k0 = kbeg; k0 < kend; k0 += 2 * C::BK) {
        load_regs(ra0, rb0, k0 + 2 * C::BK);
        mma_block<C>(As0, As0 + C::BM * C::LDK, acc, wm, wn, lane);
        store_lds(ra1, rb1, 1);
        __syncthreads();
        // no early exit between the halves: with an odd number of K-blocks the second half
        // multiplies a block of zeros, which is cheaper than the accumulator shuffling a
        // mid-loop exit costs on every iteration
        load_regs(ra1, rb1, k0 + 3 * C::BK);
        mma_block<C>(As1, As1 + C::BM * C::LDK, acc, wm, wn, lane);
        store_lds(ra0, rb0, 0);
        __syncthreads();
    }
    float* partial = nullptr;
    if (p.splits > 1) {
        if (p.tickets) {
            if (!finish_split<C>(acc, p.ws, p.tickets, p.splits, t, split, wave, lane,
                                 reinterpret_cast<unsigned*>(lds + stage_floats<C>())))
                return;
        } else {
            partial = p.ws + (long)split * p.M * p.N;
        }
    }
    store_tile<C>(acc, wm, wn, lane, m0, n0, p.M, p.N, Cc, p.ep, partial, lds + wave * STAGE_BLOCK);
}

// Branch-free variant of gemm_fast_kernel for the common case: K covered by an even number of
// whole K-blocks per split.  Rows / columns past the edge are clamped to the last valid one
// (their products are computed and thrown away at the store) and the look-ahead loads past the
// end of K are clamped to the last K-block, so the loop body has no predication and no control
// flow: loads, LDS traffic and MFMAs can be interleaved freely by the scheduler.
//
// APRE: inference batch-norm (+ ReLU) of the X operand per K index, for pre-activation networks.  The
// workgroup folds the four vectors of its K range to scale and shift once, into LDS, while its first operand
// loads are in flight; every 128-bit slice of X is then transformed in registers on its way into the LDS
// tile (a thread's slices all share one K offset within the block, so that is two LDS reads and eight vector
// instructions per K-block and slice).  The weights and the MFMA loop are untouched.
template <class C, bool YKC, int STAGES, bool APRE = false>
#ifndef TP_CLEAN_OCC
#define TP_CLEAN_OCC (C::TM * C::TN >= 4 ? 1 : 2)
#endif
__global__ __launch_bounds__(C::THREADS, TP_CLEAN_OCC) void gemm_clean_kernel(const GemmDev p) {
    fetch_now(p);
    constexpr int RED_FLOATS = red_floats<C>();  // K-slice reduction area, then the epilogue staging blocks
    __shared__ __attribute__((aligned(16))) float lds[cmax(STAGES * C::LDS_FLOATS, RED_FLOATS + stage_floats<C>() + 4)];
    __shared__ __attribute__((aligned(16))) float pre_sb[APRE ? 2 * kPreBnMaxK : 4];  // folded scale, then shift (unused and dropped without APRE)
    TP_CLK(0);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wk = wave / (C::WGM * C::WGN), wsp = wave - wk * (C::WGM * C::WGN);
    const int wm = wsp / C::WGN, wn = wsp % C::WGN;
    int tm, tn, t;
    if (!tile_of(p, blockIdx.x, &tm, &tn, &t)) return;
    const long m0 = (long)tm * C::BM, n0 = (long)tn * C::BN;
    int split = 0, batch = blockIdx.z;
    if (p.splits > 1) {
        split = blockIdx.z;
        batch = 0;
    }
    const int b0 = batch / p.nb1, b1 = batch - b0 * p.nb1;
    const float* __restrict__ X = p.X + b0 * p.xb0 + b1 * p.xb1;
    const float* __restrict__ Y = p.Y + b0 * p.yb0 + b1 * p.yb1;
    float* __restrict__ Cc = p.C + b0 * p.cb0 + b1 * p.cb1;
    const long kbeg = (long)split * p.kper;
    const long kend = (kbeg + p.kper < p.K) ? kbeg + p.kper : p.K;
    const long klast = kend - C::BK;
    ColConsts<C::TN> cc;  // bias / batch-norm vectors of this wavefront's columns: requested now, used at the end
    if (wk == 0) cols_issue<C>(cc, p.ep, Cc, n0, wn, lane, p.N);
    // APRE: the four batch-norm vectors of this workgroup's K range, requested before anything else needs the
    // memory pipe (at most kPreBnMaxK values of each: PRE_STEPS 128-bit loads per thread and vector)
    constexpr int PRE_STEPS = APRE ? (int)((kPreBnMaxK / 4 + C::THREADS - 1) / C::THREADS) : 1;
    f32x4 pre_g[PRE_STEPS], pre_b[PRE_STEPS], pre_m[PRE_STEPS], pre_v[PRE_STEPS];
    if (APRE) {
#pragma unroll
        for (int j = 0; j < PRE_STEPS; ++j) {
            const long k = kbeg + ((long)j * C::THREADS + tid) * 4;
            if (k < kend) {
                pre_g[j] = *reinterpret_cast<const f32x4*>(p.pre_gamma + k);
                if (p.pre_var) {  // (uniform: all three or none; none = a plain per-K scale)
                    pre_b[j] = *reinterpret_cast<const f32x4*>(p.pre_beta + k);
                    pre_m[j] = *reinterpret_cast<const f32x4*>(p.pre_mean + k);
                    pre_v[j] = *reinterpret_cast<const f32x4*>(p.pre_var + k);
                }
            }
        }
    }

    constexpr int KV = C::BK / 4;
    constexpr int CV = C::BN / 4;
    constexpr int NVA = C::BM * KV / C::THREADS;
    constexpr int NVB = (YKC ? C::BN * KV : C::BK * CV) / C::THREADS;
    static_assert(C::BM * KV % C::THREADS == 0 && C::BN * KV % C::THREADS == 0 && C::BK * CV % C::THREADS == 0,
                  "tile must split evenly over the workgroup");

    const float* pa[NVA];
    const float* pb[NVB];
    int sa[NVA], sb[NVB];  // LDS offsets
#pragma unroll
    for (int i = 0; i < NVA; ++i) {
        const int idx = i * C::THREADS + tid;
        const int row = idx / KV, kq = idx - row * KV;
        long grow = m0 + row;
        if (grow > p.M - 1) grow = p.M - 1;
        pa[i] = X + gather_row(p, grow) * p.xs_r + kq * 4;
        sa[i] = row * C::LDK + kq * 4;
    }
#pragma unroll
    for (int i = 0; i < NVB; ++i) {
        const int idx = i * C::THREADS + tid;
        if (YKC) {
            const int col = idx / KV, kq = idx - col * KV;
            long gcol = n0 + col;
            if (gcol > p.N - 1) gcol = p.N - 1;
            pb[i] = Y + gcol * p.ys_c + kq * 4;
            sb[i] = col * C::LDK + kq * 4;
        } else {
            const int kk = idx / CV, cq = idx - kk * CV;
            long gcol = n0 + cq * 4;
            if (gcol > p.N - 4) gcol = p.N - 4;
            pb[i] = Y + kk * p.ys_k + gcol;
            sb[i] = (cq * 4) * C::LDK + kk;
        }
    }
    const long ystep = YKC ? 1 : p.ys_k;

    f32x16 acc[C::TM][C::TN];
    zero_acc<C>(acc);
    f32x4 ra0[NVA], rb0[NVB], ra1[NVA], rb1[NVB];

    static_assert(!APRE || C::THREADS % KV == 0, "a thread's X slices must share their K offset within the block");
    const int pre_kq = (tid % KV) * 4;  // APRE: this thread's K offset within a block
    const float pre_lo = (APRE && !p.pre_relu) ? -__builtin_huge_valf() : 0.f;
    long kreg[2] = {0, 0}, kwant[2] = {0, 0};  // APRE: the K position each register set was loaded from / stands for
    auto load_regs = [&](f32x4 (&ra)[NVA], f32x4 (&rb)[NVB], long k0, int set = 0) {
        const long k = k0 < klast ? k0 : klast;
        if (APRE) {
            kreg[set] = k;
            kwant[set] = k0;
        }
#pragma unroll
        for (int i = 0; i < NVA; ++i) ra[i] = *reinterpret_cast<const f32x4*>(pa[i] + k);
#pragma unroll
        for (int i = 0; i < NVB; ++i) rb[i] = *reinterpret_cast<const f32x4*>(pb[i] + k * ystep);
    };
    auto store_lds = [&](const f32x4 (&ra)[NVA], const f32x4 (&rb)[NVB], int stage, int set = 0) {
        float* As = lds + stage * C::LDS_FLOATS;
        float* Bs = As + C::BM * C::LDK;
        if (APRE) {
            int at = (int)(kreg[set] - kbeg) + pre_kq;
            // a slice in front of the position the block stands for (the half block at the end of K, or a
            // look-ahead block past it, which nobody multiplies) is written as zeros
            const bool dead = kreg[set] + pre_kq < kwant[set];
            if (at < 0) at = 0;
            const f32x4 sc = *reinterpret_cast<const f32x4*>(pre_sb + at);
            const f32x4 sh = *reinterpret_cast<const f32x4*>(pre_sb + kPreBnMaxK + at);
#pragma unroll
            for (int i = 0; i < NVA; ++i) {
                f32x4 v = ra[i];
#pragma unroll
                for (int c = 0; c < 4; ++c) v[c] = dead ? 0.f : fmaxf(v[c] * sc[c] + sh[c], pre_lo);
                *reinterpret_cast<f32x4*>(As + sa[i]) = v;
            }
        } else {
#pragma unroll
            for (int i = 0; i < NVA; ++i) *reinterpret_cast<f32x4*>(As + sa[i]) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < NVB; ++i) {
            if (YKC) {
                *reinterpret_cast<f32x4*>(Bs + sb[i]) = rb[i];
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) Bs[sb[i] + j * C::LDK] = rb[i][j];
            }
        }
    };

    TP_CLK(1);
    const float* As0 = lds;
    // APRE only: K may end with half a K-block.  That block is loaded from the last whole block's position (the
    // look-ahead clamp below does that by itself) and the part of X that belongs to the block before is zeroed
    // on its way into LDS, so the weights it meets contribute nothing.  kendv = end of K rounded up to blocks.
    const long kendv = APRE ? kbeg + (kend - kbeg + C::BK - 1) / C::BK * C::BK : kend;
    const long kpairs = kbeg + (kendv - kbeg) / (2 * C::BK) * (2 * C::BK);  // end of the whole pairs of K-blocks
    // APRE: fold this workgroup's K range of the four batch-norm vectors to scale and shift (same arithmetic as
    // epilogue_column), 128 bits per thread and step; called once the first operand loads are on their way
    auto fold_pre = [&]() {
#pragma unroll
        for (int j = 0; j < PRE_STEPS; ++j) {
            const long k = kbeg + ((long)j * C::THREADS + tid) * 4;
            if (k < kend) {
                f32x4 sc = pre_g[j], sh = {0.f, 0.f, 0.f, 0.f};
                if (p.pre_var) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const float inv = 1.0f / sqrtf(pre_v[j][c] + p.pre_eps);
                        sc[c] = pre_g[j][c] * inv;
                        sh[c] = pre_b[j][c] - pre_m[j][c] * sc[c];
                    }
                }
                *reinterpret_cast<f32x4*>(pre_sb + (k - kbeg)) = sc;
                *reinterpret_cast<f32x4*>(pre_sb + kPreBnMaxK + (k - kbeg)) = sh;
            }
        }
        __syncthreads();
    };
    if (STAGES == 2) {
        const float* As1 = lds + C::LDS_FLOATS;
        load_regs(ra0, rb0, kbeg, 0);
        load_regs(ra1, rb1, kbeg + C::BK, 1);
        if (APRE) fold_pre();
        if (wk == 0) cols_fold<C>(cc, p.ep);
        store_lds(ra0, rb0, 0, 0);
        __syncthreads();
        for (long k0 = kbeg; k0 < kpairs; k0 += 2 * C::BK) {
            load_regs(ra0, rb0, k0 + 2 * C::BK, 0);
            mma_block<C>(As0, As0 + C::BM * C::LDK, acc, wm, wn, lane, wk);
            store_lds(ra1, rb1, 1, 1);
            __syncthreads();
            load_regs(ra1, rb1, k0 + 3 * C::BK, 1);
            mma_block<C>(As1, As1 + C::BM * C::LDK, acc, wm, wn, lane, wk);
            store_lds(ra0, rb0, 0, 0);
            __syncthreads();
        }
        // an odd last K-block is in stage 0 by now (kept out of the loop: a branch there costs 10 %)
        if (kpairs < kendv) mma_block<C>(As0, As0 + C::BM * C::LDK, acc, wm, wn, lane, wk);
    } else {
        // one LDS stage, two barriers per K-block: half the LDS footprint, so twice as many
        // workgroups stay resident and hide each other's barrier and memory latency
        static_assert(!APRE || STAGES == 2, "the operand transform is built into the two-stage loop only");
        load_regs(ra0, rb0, kbeg);
        load_regs(ra1, rb1, kbeg + C::BK);
        if (wk == 0) cols_fold<C>(cc, p.ep);
        for (long k0 = kbeg; k0 < kpairs; k0 += 2 * C::BK) {
            store_lds(ra0, rb0, 0);
            __syncthreads();
            load_regs(ra0, rb0, k0 + 2 * C::BK);
            mma_block<C>(As0, As0 + C::BM * C::LDK, acc, wm, wn, lane, wk);
            __syncthreads();
            store_lds(ra1, rb1, 0);
            __syncthreads();
            load_regs(ra1, rb1, k0 + 3 * C::BK);
            mma_block<C>(As0, As0 + C::BM * C::LDK, acc, wm, wn, lane, wk);
            __syncthreads();
        }
        if (kpairs < kend) {  // odd last K-block: it is in the first register set
            store_lds(ra0, rb0, 0);
            __syncthreads();
            mma_block<C>(As0, As0 + C::BM * C::LDK, acc, wm, wn, lane, wk);
            __syncthreads();
        }
    }
    TP_CLK(2);
    if (!reduce_k_slices<C>(acc, lds, wk, wsp, lane)) return;
    TP_CLK(3);
    float* partial = nullptr;
    if (p.splits > 1) {
        if (p.tickets) {
            if (!finish_split<C>(acc, p.ws, p.tickets, p.splits, t, split, wsp, lane,
                                 reinterpret_cast<unsigned*>(lds + RED_FLOATS + stage_floats<C>())))
                return;
        } else {
            partial = p.ws + (long)split * p.M * p.N;
        }
    }
    store_tile<C>(acc, wm, wn, lane, m0, n0, p.M, p.N, Cc, p.ep, partial, lds + RED_FLOATS + wsp * STAGE_BLOCK, &cc);
    TP_CLK(4);
}

// Any strides, any alignment.  64x64x16 tile, scalar loads.
using GenCfg = TileCfg<64, 64, 16, 2, 2>;

__global__ __launch_bounds__(GenCfg::THREADS, 2) void gemm_generic_kernel(const GemmDev p) {
    using C = GenCfg;
    __shared__ __attribute__((aligned(16))) float lds[cmax(C::LDS_FLOATS, stage_floats<C>() + 4)];
    float* As = lds;
    float* Bs = lds + C::BM * C::LDK;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / C::WGN, wn = wave % C::WGN;
    const int t = blockIdx.x;
    const int tm = t / p.tiles_n, tn = t - tm * p.tiles_n;
    const long m0 = (long)tm * C::BM, n0 = (long)tn * C::BN;
    int split = 0, batch = blockIdx.z;
    if (p.splits > 1) {
        split = blockIdx.z;
        batch = 0;
    }
    const int b0 = batch / p.nb1, b1 = batch - b0 * p.nb1;
    const float* __restrict__ X = p.X + b0 * p.xb0 + b1 * p.xb1;
    const float* __restrict__ Y = p.Y + b0 * p.yb0 + b1 * p.yb1;
    float* __restrict__ Cc = p.C + b0 * p.cb0 + b1 * p.cb1;
    const long kbeg = (long)split * p.kper;
    const long kend = (kbeg + p.kper < p.K) ? kbeg + p.kper : p.K;

    constexpr int NE = C::BM * C::BK / C::THREADS;  // 4 (BM == BN)
    const bool xk = (p.xs_k == 1), yk = (p.ys_k == 1);
    int rowA[NE], kA[NE], rowB[NE], kB[NE];
    long offA[NE], offB[NE];
#pragma unroll
    for (int i = 0; i < NE; ++i) {
        const int idx = i * C::THREADS + tid;
        if (xk) {
            kA[i] = idx % C::BK;
            rowA[i] = idx / C::BK;
        } else {
            rowA[i] = idx % C::BM;
            kA[i] = idx / C::BM;
        }
        if (yk) {
            kB[i] = idx % C::BK;
            rowB[i] = idx / C::BK;
        } else {
            rowB[i] = idx % C::BN;
            kB[i] = idx / C::BN;
        }
        offA[i] = (m0 + rowA[i] < p.M) ? gather_row(p, m0 + rowA[i]) * p.xs_r : -1;
        offB[i] = (n0 + rowB[i] < p.N) ? (n0 + rowB[i]) * p.ys_c : -1;
    }
    f32x16 acc[C::TM][C::TN];
    zero_acc<C>(acc);
    float ra[NE], rb[NE];
    auto load_regs = [&](long k0) {
#pragma unroll
        for (int i = 0; i < NE; ++i) {
            const long ka = k0 + kA[i], kb = k0 + kB[i];
            ra[i] = (offA[i] >= 0 && ka < kend) ? X[offA[i] + ka * p.xs_k] : 0.f;
            rb[i] = (offB[i] >= 0 && kb < kend) ? Y[offB[i] + kb * p.ys_k] : 0.f;
        }
    };
    load_regs(kbeg);
    for (long k0 = kbeg; k0 < kend; k0 += C::BK) {
#pragma unroll
        for (int i = 0; i < NE; ++i) {
            As[rowA[i] * C::LDK + kA[i]] = ra[i];
            Bs[rowB[i] * C::LDK + kB[i]] = rb[i];
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
            partial = p.ws + (long)split * p.M * p.N;
        }
    }
    store_tile<C>(acc, wm, wn, lane, m0, n0, p.M, p.N, Cc, p.ep, partial, lds + wave * STAGE_BLOCK);
}

__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws, int splits, long M, long N,
                                                            float* __restrict__ Cout, const Epilogue e) {
    const long total = M * N;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        float s = 0.f;
        for (int z = 0; z < splits; ++z) s += ws[(long)z * total + i];
        const long row = i / N, col = i - row * N;
        float cs, ct;
        epilogue_column(e, col, cs, ct);
        epilogue_store(e, Cout, row, col, s, cs, ct);
    }
}

Epilogue make_epilogue(const EpilogueArgs& a, long ldc);

// A GEMM of at most eight rows (the classifier of a convolutional network, BERT's pooler, the two small
// layers of a squeeze-and-excitation block at batch 1..8) is a matrix-vector product: a 32x32 MFMA tile
// would spend 75-97 % of its multiplications on rows that do not exist, and what bounds the launch is
// reading the weights once.  One wavefront per output column: its lanes walk the column's K-contiguous
// weights 128 bits at a time (1 KB per step and wavefront), multiply them with the same slice of every
// row of X (read through the L1, shared by the workgroup's four columns), and a butterfly over the lanes
// finishes the sums -- a fixed order, so repeated launches agree bit for bit.  Lane m applies the epilogue
// to row m.  MR = rows held in registers (1, 2, 4 or 8; rows past M repeat the last one and are not stored).
struct GemvDev {
    const float* X;
    const float* Y;
    float* C;
    int M;
    long N, K, xs_r, ys_c;
    Epilogue ep;
};

template <int MR>
__global__ __launch_bounds__(256) void gemv_rows_kernel(const GemvDev p) {
    const int lane = threadIdx.x & 63;
    const long col = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (col >= p.N) return;  // whole wavefronts leave; the kernel has no barrier
    const float* __restrict__ w = p.Y + col * p.ys_c;
    const float* xr[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) xr[m] = p.X + (long)(m < p.M ? m : p.M - 1) * p.xs_r;
    float acc[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[m] = 0.f;
#pragma unroll 4
    for (long k = lane * 4; k < p.K; k += 256) {
        const f32x4 wv = *reinterpret_cast<const f32x4*>(w + k);
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            const f32x4 xv = *reinterpret_cast<const f32x4*>(xr[m] + k);
            acc[m] += wv[0] * xv[0] + wv[1] * xv[1] + wv[2] * xv[2] + wv[3] * xv[3];
        }
    }
    float mine = 0.f;
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        float v = acc[m];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
        if (lane == m) mine = v;
    }
    if (lane < p.M && lane < MR) {
        float cs, ct;
        epilogue_column(p.ep, col, cs, ct);
        epilogue_store(p.ep, p.C, lane, col, mine, cs, ct);
    }
}

// Does this call take the matrix-vector path?  (No workspace, no split, any N and K.)
static bool gemv_applies(const GemmArgs& a) {
    static const bool on = getenv("TORPOR_GEMV") == nullptr || atoi(getenv("TORPOR_GEMV")) != 0;
    return on && !a.pre_gamma && a.M >= 1 && a.M <= 8 && a.nb0 * a.nb1 == 1 && !a.gather && a.xs_k == 1 && a.ys_k == 1 && a.K >= 4 &&
           a.K % 4 == 0 && a.xs_r % 4 == 0 && a.ys_c % 4 == 0 && (reinterpret_cast<uintptr_t>(a.X) & 15) == 0 &&
           (reinterpret_cast<uintptr_t>(a.Y) & 15) == 0 && a.N <= (1L << 31);
}

static int launch_gemv(const GemmArgs& a, hipStream_t s) {
    GemvDev p;
    p.X = a.X;
    p.Y = a.Y;
    p.C = a.C;
    p.M = (int)a.M;
    p.N = a.N;
    p.K = a.K;
    p.xs_r = a.xs_r;
    p.ys_c = a.ys_c;
    p.ep = make_epilogue(a.ep, a.ldc);
    const dim3 grid((unsigned)((a.N + 3) / 4)), block(256);
    if (a.M == 1)
        hipLaunchKernelGGL(gemv_rows_kernel<1>, grid, block, 0, s, p);
    else if (a.M == 2)
        hipLaunchKernelGGL(gemv_rows_kernel<2>, grid, block, 0, s, p);
    else if (a.M <= 4)
        hipLaunchKernelGGL(gemv_rows_kernel<4>, grid, block, 0, s, p);
    else
        hipLaunchKernelGGL(gemv_rows_kernel<8>, grid, block, 0, s, p);
    g_last_kernel = "gemv_rows_kc";
    return (int)hipGetLastError();
}

Epilogue make_epilogue(const EpilogueArgs& a, long ldc) {
    Epilogue e;
    e.alpha = a.alpha;
    e.beta = a.beta;
    e.bias = a.bias;
    e.bn_scale = a.bn_scale;
    e.bn_bias = a.bn_bias;
    e.bn_mean = a.bn_mean;
    e.bn_var = a.bn_var;
    e.bn_eps = a.bn_eps;
    e.residual = a.residual;
    e.ldr = a.ldr;
    e.act = a.act;
    e.ldc = ldc;
    e.out_nchw = 0;
    e.howo = 1;
    e.ncols = 0;
    return e;
}

int launch_splitk_reduce(const float* ws, int splits, long M, long N, float* C, const Epilogue& e, hipStream_t s) {
    long total = M * N;
    int blocks = (int)((total + 255) / 256);
    if (blocks > g_num_cu * 8) blocks = g_num_cu * 8;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3(blocks), dim3(256), 0, s, ws, splits, M, N, C, e);
    return (int)hipGetLastError();
}

// XCD partition of the tile grid: X is re-fetched once per column group and Y once per row
// group, so pick the split of 8 that moves the fewest bytes; returns the padded grid.x.
static int plan_xcd_grid(GemmDev& p, long M, long N) {
    const int cand[4][2] = {{1, 8}, {2, 4}, {4, 2}, {8, 1}};
    double best = 1e300;
    p.xr = 0;
    p.xc = 0;
    static const int dbg_xcd = getenv("TORPOR_GEMM_XCD") ? atoi(getenv("TORPOR_GEMM_XCD")) : 1;
    if (dbg_xcd <= 0) {
        p.xr = dbg_xcd;  // 0: linear + remap, -1: identity
        return p.tiles_m * p.tiles_n;
    }
    for (auto& c : cand) {
        if (c[0] > p.tiles_m || c[1] > p.tiles_n) continue;
        const double cost = (double)M * c[1] + (double)N * c[0];
        if (cost < best) {
            best = cost;
            p.xr = c[0];
            p.xc = c[1];
        }
    }
    if (p.xr == 0) return p.tiles_m * p.tiles_n;  // fewer tiles than a split needs: linear mapping
    if (p.tiles_m > 65535 || p.tiles_n > 65535) {  // beyond the rectangle table's range: linear mapping
        p.xr = p.xc = 0;
        return p.tiles_m * p.tiles_n;
    }
    int biggest = 0;
    for (int br = 0; br < p.xr; ++br)
        for (int bc = 0; bc < p.xc; ++bc) {
            const int r0 = (int)((long)p.tiles_m * br / p.xr), r1 = (int)((long)p.tiles_m * (br + 1) / p.xr);
            const int c0 = (int)((long)p.tiles_n * bc / p.xc), c1 = (int)((long)p.tiles_n * (bc + 1) / p.xc);
            const int h = r1 - r0, w = c1 - c0;
            GemmDev::Rect& q = p.rect[br * p.xc + bc];
            q.r0 = (unsigned short)r0;
            q.c0 = (unsigned short)c0;
            q.w = (unsigned short)w;
            q.h = (unsigned short)h;
            if (h * w > biggest) biggest = h * w;
        }
    return 8 * biggest;
}

using CfgL = TileCfg<128, 128, 32, 2, 2>;  // 2x2 accumulators per wavefront
using CfgW = TileCfg<128, 64, 32, 2, 2>;   // 2x1
using CfgM = TileCfg<64, 64, 32, 2, 2>;    // 1x1
using CfgS = TileCfg<64, 32, 64, 2, 1, 2>; // 1x1, two wavefronts per output tile split each K-block
using CfgT = TileCfg<32, 32, 64, 1, 1, 4>; // one 32x32 tile, its four wavefronts split each K-block

// Returns 0 = predicated kernel, 1 = branch-free with one LDS stage, 2 = branch-free with two.
template <class C>
static int launch_fast(const GemmDev& p, bool y_kc, bool clean, dim3 grid, hipStream_t s) {
    // With many tiles per CU a single LDS stage wins (twice the resident workgroups hide each
    // other's latencies: 99 vs 94 TFLOP/s on 1536x4096x1024); with one or two tiles per CU the
    // two-stage loop with its single barrier per K-block does (83 vs 79 on 1536x1024x4096).
    const long tiles = (long)p.tiles_m * p.tiles_n * grid.z;
    static const int dbg_st = getenv("TORPOR_GEMM_STAGES") ? atoi(getenv("TORPOR_GEMM_STAGES")) : 0;
    const bool one_stage = dbg_st ? dbg_st == 1 : tiles >= 5L * g_num_cu;
    if (clean && one_stage) {
        if (y_kc)
            hipLaunchKernelGGL((gemm_clean_kernel<C, true, 1>), grid, dim3(C::THREADS), 0, s, p);
        else
            hipLaunchKernelGGL((gemm_clean_kernel<C, false, 1>), grid, dim3(C::THREADS), 0, s, p);
        return 1;
    } else if (clean) {
        if (y_kc)
            hipLaunchKernelGGL((gemm_clean_kernel<C, true, 2>), grid, dim3(C::THREADS), 0, s, p);
        else
            hipLaunchKernelGGL((gemm_clean_kernel<C, false, 2>), grid, dim3(C::THREADS), 0, s, p);
        return 2;
    } else {
        if (y_kc)
            hipLaunchKernelGGL((gemm_fast_kernel<C, true>), grid, dim3(C::THREADS), 0, s, p);
        else
            hipLaunchKernelGGL((gemm_fast_kernel<C, false>), grid, dim3(C::THREADS), 0, s, p);
    }
    return 0;
}

// Tiles that exist only as the branch-free kernel (the caller has checked its preconditions).
template <class C>
static int launch_clean_only(const GemmDev& p, bool y_kc, dim3 grid, hipStream_t s) {
    static const int dbg_st = getenv("TORPOR_GEMM_STAGES") ? atoi(getenv("TORPOR_GEMM_STAGES")) : 0;
    if (dbg_st == 1) {
        if (y_kc)
            hipLaunchKernelGGL((gemm_clean_kernel<C, true, 1>), grid, dim3(C::THREADS), 0, s, p);
        else
            hipLaunchKernelGGL((gemm_clean_kernel<C, false, 1>), grid, dim3(C::THREADS), 0, s, p);
        return 1;
    }
    if (y_kc)
        hipLaunchKernelGGL((gemm_clean_kernel<C, true, 2>), grid, dim3(C::THREADS), 0, s, p);
    else
        hipLaunchKernelGGL((gemm_clean_kernel<C, false, 2>), grid, dim3(C::THREADS), 0, s, p);
    return 2;
}

// Tile shape.  Measured on MI355X over the served shapes (BERT-large 1536 x {1024,4096} x
// {1024,4096}, ResNet 1x1 convolutions from 25088x256x64 to 392x2048x512), the 64x64 tile is
// the fastest everywhere: it keeps the most workgroups resident per CU, and for fp32 MFMA
// (2 k per instruction) occupancy hides more latency than larger register tiles save in LDS
// traffic.  The 128x128 / 128x64 variants are kept for very large grids and for experiments
// (TORPOR_GEMM_CFG=0/1/2 forces one).
static int choose_tile(long M, long N, long K, int batch, bool y_kc, bool half_ok = false) {
    static const int forced = [] {
        const char* e = getenv("TORPOR_GEMM_CFG");
        return e ? atoi(e) : -1;
    }();
    if (forced >= 0 && forced <= 4) return forced;
    const long tiles_w = ((M + 127) / 128) * ((N + 63) / 64) * batch;
    if (tiles_w >= 64L * g_num_cu) return 1;  // enough 128x64 tiles to keep every CU full for long
    // Tile quantisation: with t tiles on n CUs the slowest CU works ceil(t/n) tiles.  When
    // halving the tile (64x32, K split over wavefront pairs) evens that out, take it: 384 tiles
    // of 64x64 on 256 CUs are two rounds, 768 of 64x32 are three rounds of half the work
    // (1536x1024x4096: 140 -> 114 us).  Only for long K and few rounds, where it was measured
    // to win; the [K][N] weight layout and short K lose with it.
    const long t64 = ((M + 63) / 64) * ((N + 63) / 64) * batch;
    const long t32 = ((M + 63) / 64) * ((N + 31) / 32) * batch;
    if (y_kc && K >= 512 && K % 128 == 0 && t64 >= g_num_cu && t64 < 3L * g_num_cu) {
        const double r64 = (double)((t64 + g_num_cu - 1) / g_num_cu);
        const double r32 = 0.5 * (double)((t32 + g_num_cu - 1) / g_num_cu);
        if (r32 <= 0.8 * r64) return 3;
    }
    // Fewer 64x64 tiles than CUs: quarter the tile and split each K-block over its four wavefronts
    // (1568x256x1024: 22.4 -> 16.0 us against a split over workgroups).  A long K with few of these small
    // tiles is split over workgroups as well (plan_gemm): up to eight slots are summed inside the launch, and
    // a workgroup of this shape is short-lived -- 128x768x3072 runs 96 tiles x 6 slots instead of 24 tiles of
    // 64x64 x 16 slots and a reduction launch.  TORPOR_GEMM_SMALL=0 restores the old rule for comparison.
    static const bool small_split = getenv("TORPOR_GEMM_SMALL") == nullptr || atoi(getenv("TORPOR_GEMM_SMALL")) != 0;
    const long t3232 = ((M + 31) / 32) * ((N + 31) / 32) * batch;
    // (whole 64-wide K-blocks, an odd count is fine; half_ok: the kernel with the operand transform also takes
    // half a block at the end)
    if (batch == 1 && K >= 256 && K % (half_ok ? 32 : 64) == 0 && t64 < g_num_cu) {
        if (small_split) return 4;
        if (t3232 >= 3 * g_num_cu / 8 && (t3232 >= g_num_cu || K <= 1024)) return 4;
    }
    return 2;
}

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Pick the split-K factor: fill the chip when the tile count alone cannot.
// The ticket counters of a workspace, if the in-launch summation of split K ranges is to be used for a
// grid of `tiles` output tiles split `splits` ways.  Measured on MI355X: with up to 8 slots the workgroup
// that finishes a tile last sums them as fast as a reduction launch would or faster (ResNet-152 batch 8,
// 3x3 convolutions of 100 tiles x 6: 29.1 against 30.2 us, and the cold request, whose launches queue behind
// the swap-in's copies, 4.11 against 4.23 ms); with 16 to 32 slots its serial read of them loses to the
// reduction kernel's whole-chip pass (1x1000x2048, 32 slots: 13.6 against 11.3 us).
// TORPOR_SPLITK_FUSED=0 forces the two-launch form, =2 the in-launch form for any split count.
unsigned* split_tickets(const Workspace& ws, long tiles, int splits) {
    static const int mode = getenv("TORPOR_SPLITK_FUSED") ? atoi(getenv("TORPOR_SPLITK_FUSED")) : 1;
    if (mode == 0 || tiles > kSplitTickets || splits < 2) return nullptr;
    return (mode == 2 || splits <= 8) ? ws.tickets : nullptr;
}

// One split's partial sums are `tiles` whole output tiles of tile_floats each (the in-launch summation
// keeps them per tile and per wavefront; the two-launch form needs no more than that).
int choose_splits(long tiles, long K, int bk, long tile_floats, size_t ws_bytes, long* kper_out, int max_splits = 32, bool pairs = true,
                  int balance = -1) {
    int splits = 1;
    const long kblocks = (K + bk - 1) / bk;
    const size_t per = (size_t)tiles * (size_t)tile_floats * sizeof(float);
    static const int forced = getenv("TORPOR_SPLITS") ? atoi(getenv("TORPOR_SPLITS")) : 0;
    if (forced > 0 && kblocks >= 2L * forced && (size_t)forced * per <= ws_bytes) {
        splits = forced;
    } else if (tiles < g_num_cu && kblocks >= 8) {
        long want = (2L * g_num_cu + tiles - 1) / tiles;
        long maxs = kblocks / 4;  // keep at least 4 K-blocks per split
        if (want > maxs) want = maxs;
        if (want > max_splits) want = max_splits;
        while (want > 1 && (size_t)want * per > ws_bytes) --want;
        if (want > 1) splits = (int)want;
        if ((balance < 0 ? !pairs : balance != 0) && want > 1) {
            // Kernels that take any number of K-blocks per split: weigh the candidates by what the
            // fullest CU has to work through.  With s splits of b = ceil(kblocks / s) blocks the
            // tiles * s workgroups land ceil(tiles * s / CUs) deep on some CU; a CU that holds a single
            // workgroup hides no latency (about 1.3x per block), and every slot costs its tile's last
            // workgroup a quarter of a block to read back.  8x14x14x256>256 (100 tiles, 32 blocks): 5
            // splits of 7 (two deep, 14 blocks) run 29.0 us, the 6 of 6 (three deep, 18) 30.9 us.
            double best = 1e30;
            for (long s = 2; s <= want + 2 && s <= maxs && s <= max_splits && (size_t)s * per <= ws_bytes; ++s) {
                long b = (kblocks + s - 1) / s;
                if (pairs && (b & 1)) ++b;
                const long s_eff = (kblocks + b - 1) / b;
                const long deep = (tiles * s_eff + g_num_cu - 1) / g_num_cu;
                const double cost = (double)deep * (double)b * (deep == 1 ? 1.3 : 1.0) + 0.25 * (double)s_eff;
                if (cost < best) {
                    best = cost;
                    splits = (int)s_eff;
                }
            }
        }
    }
    long per_blocks = (kblocks + splits - 1) / splits;
    if (pairs && splits > 1 && (per_blocks & 1)) ++per_blocks;  // whole pairs of K-blocks per split
    splits = (int)((kblocks + per_blocks - 1) / per_blocks);
    *kper_out = per_blocks * bk;
    return splits;
}

// 32x32 GEMM tiles: the split is weighed by the depth of the fullest CU as well (128x768x3072, 96 tiles of 48
// K-blocks: 8 slots of 6 blocks, three deep, 11.6 us; the 6 slots of 8 that "two workgroups per CU" gives, also three
// deep, 13.0 us).  TORPOR_GEMM_BALANCE=0 restores the plain rule.
static const int g_small_balance = getenv("TORPOR_GEMM_BALANCE") ? atoi(getenv("TORPOR_GEMM_BALANCE")) : 1;

// What launch_gemm decides from the shape alone: kernel family, tile and split of K over workgroups.
struct GemmPlan {
    bool fast = false, y_kc = false;
    int cfg = 2, bm = 64, bn = 64;
    int tiles_m = 0, tiles_n = 0;
    int splits = 1;
    long kper = 0;
};

static GemmPlan plan_gemm(const GemmArgs& a, size_t ws_bytes) {
    GemmPlan g;
    const int batch = a.nb0 * a.nb1;
    const bool x_fast = a.xs_k == 1 && (a.xs_r % 4 == 0) && (a.K % 4 == 0) && aligned16(a.X) && (a.xb0 % 4 == 0) &&
                        (a.xb1 % 4 == 0);
    g.y_kc = a.ys_k == 1 && (a.ys_c % 4 == 0) && (a.K % 4 == 0);
    const bool y_cc = a.ys_c == 1 && a.ys_k != 1 && (a.ys_k % 4 == 0);
    const bool y_fast = (g.y_kc || y_cc) && aligned16(a.Y) && (a.yb0 % 4 == 0) && (a.yb1 % 4 == 0);
    g.fast = x_fast && y_fast;
    if (g.fast) {
        const bool half_ok = a.pre_gamma != nullptr && g.y_kc;
        int cfg = choose_tile(a.M, a.N, a.K, batch, g.y_kc, half_ok);
        if (cfg >= 3 && !(a.K >= 128 && a.K % (cfg == 4 ? (half_ok ? 32 : 64) : 128) == 0 && (g.y_kc || a.N % 4 == 0))) cfg = 2;  // branch-free only
        if (a.pre_gamma && cfg != 2 && cfg != 4) cfg = 2;  // the operand transform exists for the 64x64 and 32x32 tiles
        g.cfg = cfg;
        g.bm = cfg == 4 ? 32 : cfg >= 2 ? 64 : 128;
        g.bn = cfg == 0 ? 128 : cfg >= 3 ? 32 : 64;
        g.tiles_m = (int)((a.M + g.bm - 1) / g.bm);
        g.tiles_n = (int)((a.N + g.bn - 1) / g.bn);
        long tiles = (long)g.tiles_m * g.tiles_n * batch;
        g.kper = ((a.K + 31) / 32) * 32;
        // A long K with one to three 64x64 tiles per CU: instead of halving the tile (cfg 3) halve K -- two
        // workgroups per 64x64 tile, summed inside the launch.  Same number of workgroups, a third less operand
        // traffic into LDS per multiplication (1536x1024x4096: 135.7 -> 126.9 us bracketed, 95 -> 101.5 TFLOP/s;
        // at K = 1024 the two are equal and the tile stays halved).  Only where the partial sums stay within
        // what every caller's scratch memory holds (kSplitPairBytes), so that all entry points split alike.
        static const bool pair_split = getenv("TORPOR_GEMM_PAIR") == nullptr || atoi(getenv("TORPOR_GEMM_PAIR")) != 0;
        constexpr size_t kSplitPairBytes = (16u << 20) - 4096;
        const size_t pair_bytes = 2 * (size_t)a.M * (size_t)a.N * sizeof(float);
        if (pair_split && cfg == 3 && batch == 1 && a.K >= 2048 && a.K % 128 == 0 && pair_bytes <= kSplitPairBytes &&
            pair_bytes <= ws_bytes && (long)((a.M + 63) / 64) * ((a.N + 63) / 64) <= kSplitTickets) {
            cfg = g.cfg = 2;
            g.bm = g.bn = 64;
            g.tiles_m = (int)((a.M + 63) / 64);
            g.tiles_n = (int)((a.N + 63) / 64);
            tiles = (long)g.tiles_m * g.tiles_n;
            g.splits = 2;
            g.kper = a.K / 2;
        } else if (batch == 1 && cfg < 3) {
            g.splits = choose_splits(tiles, a.K, 32, (long)g.bm * g.bn, ws_bytes, &g.kper);
        }
        // (with more than half a tile per CU the split does not pay: 196x1024x512, 224 tiles, 8.5 against 7.4 us)
        if (batch == 1 && cfg == 4 && tiles <= g_num_cu / 2)
            g.splits = choose_splits(tiles, a.K, 64, 32 * 32, ws_bytes, &g.kper, /*max_splits=*/8, true, g_small_balance);
    } else {
        g.tiles_m = (int)((a.M + 63) / 64);
        g.tiles_n = (int)((a.N + 63) / 64);
        const long tiles = (long)g.tiles_m * g.tiles_n * batch;
        g.kper = ((a.K + 15) / 16) * 16;
        if (batch == 1) g.splits = choose_splits(tiles, a.K, 16, 64 * 64, ws_bytes, &g.kper);
    }
    return g;
}

static bool gemm_args_ok(const GemmArgs& a) {
    if (a.M <= 0 || a.N <= 0 || a.K < 0 || !a.X || !a.Y || !a.C) return false;
    if (a.nb0 < 1 || a.nb1 < 1) return false;
    if (!((a.xs_k == 1) || (a.xs_r == 1)) || !((a.ys_k == 1) || (a.ys_c == 1))) return false;
    if (a.gather && (a.Ho <= 0 || a.Wo <= 0 || a.H <= 0 || a.W <= 0)) return false;
    return true;
}

// Bytes of split-K partial sums launch_gemm would write for this call if the workspace were unbounded.
long gemm_workspace_need(const GemmArgs& a) {
    if (!gemm_args_ok(a)) return K_EINVAL;
    if (gemv_applies(a)) return 0;
    const GemmPlan g = plan_gemm(a, ~(size_t)0);
    return g.splits > 1 ? (long)g.splits * g.tiles_m * g.tiles_n * g.bm * g.bn * (long)sizeof(float) : 0;
}

int launch_gemm(const GemmArgs& a, const Workspace& ws, hipStream_t s) {
    if (!gemm_args_ok(a)) return K_EINVAL;
    if (gemv_applies(a)) return launch_gemv(a, s);
    const int batch = a.nb0 * a.nb1;
    const GemmPlan g = plan_gemm(a, ws.ptr ? ws.bytes : 0);
    GemmDev p;
    p.X = a.X;
    p.Y = a.Y;
    p.C = a.C;
    p.M = a.M;
    p.N = a.N;
    p.K = a.K;
    p.xs_r = a.xs_r;
    p.xs_k = a.xs_k;
    p.ys_c = a.ys_c;
    p.ys_k = a.ys_k;
    p.nb1 = a.nb1;
    p.xb0 = a.xb0;
    p.xb1 = a.xb1;
    p.yb0 = a.yb0;
    p.yb1 = a.yb1;
    p.cb0 = a.cb0;
    p.cb1 = a.cb1;
    p.gather = a.gather;
    p.Ho = a.Ho;
    p.Wo = a.Wo;
    p.H = a.H;
    p.W = a.W;
    p.sh = a.sh;
    p.sw = a.sw;
    p.ws = ws.ptr;
    p.ep = make_epilogue(a.ep, a.ldc);
    p.pre_gamma = a.pre_gamma;
    p.pre_beta = a.pre_beta;
    p.pre_mean = a.pre_mean;
    p.pre_var = a.pre_var;
    p.pre_eps = a.pre_eps;
    p.pre_relu = a.pre_relu;
    p.tickets = split_tickets(ws, (long)g.tiles_m * g.tiles_n, g.splits);

    p.tiles_m = g.tiles_m;
    p.tiles_n = g.tiles_n;
    p.splits = g.splits;
    p.kper = g.kper;
    const bool y_kc = g.y_kc;

    if (g.fast) {
        const int cfg = g.cfg;
        dim3 grid(plan_xcd_grid(p, a.M, a.N), 1, p.splits > 1 ? p.splits : batch);
        static const bool allow_clean = getenv("TORPOR_GEMM_NOCLEAN") == nullptr;
        // whole K-blocks; the 32-wide tiles take them in pairs, an odd last one is handled in the loop
        const long kq = cfg >= 3 ? 64 : 32;
        const long kq_mult = (a.pre_gamma && cfg == 4) ? 32 : kq;  // the operand-transform kernel masks half a block
        const bool clean = allow_clean && a.K >= kq && a.K % kq_mult == 0 && (p.splits == 1 || p.kper % 64 == 0) &&
                           (y_kc || (a.N % 4 == 0 && a.N >= 4));
        // kernel variant names: <tile>_<kc|cc>[_s1|_s2]; _s1 / _s2 = branch-free kernel with one /
        // two LDS stages (gemm_clean_kernel<..., 1|2>), no suffix = predicated gemm_fast_kernel
        static const char* const names[5][2][3] = {
            {{"gemm_fast_128x128_cc", "gemm_fast_128x128_cc_s1", "gemm_fast_128x128_cc_s2"},
             {"gemm_fast_128x128_kc", "gemm_fast_128x128_kc_s1", "gemm_fast_128x128_kc_s2"}},
            {{"gemm_fast_128x64_cc", "gemm_fast_128x64_cc_s1", "gemm_fast_128x64_cc_s2"},
             {"gemm_fast_128x64_kc", "gemm_fast_128x64_kc_s1", "gemm_fast_128x64_kc_s2"}},
            {{"gemm_fast_64x64_cc", "gemm_fast_64x64_cc_s1", "gemm_fast_64x64_cc_s2"},
             {"gemm_fast_64x64_kc", "gemm_fast_64x64_kc_s1", "gemm_fast_64x64_kc_s2"}},
            {{"gemm_fast_64x32_cc", "gemm_fast_64x32_cc_s1", "gemm_fast_64x32_cc_s2"},
             {"gemm_fast_64x32_kc", "gemm_fast_64x32_kc_s1", "gemm_fast_64x32_kc_s2"}},
            {{"gemm_fast_32x32_cc", "gemm_fast_32x32_cc_s1", "gemm_fast_32x32_cc_s2"},
             {"gemm_fast_32x32_kc", "gemm_fast_32x32_kc_s1", "gemm_fast_32x32_kc_s2"}}};
        if (a.pre_gamma) {
            // batch-norm (+ ReLU) of the X operand: the branch-free two-stage kernel of the two small tiles carries it
            const long range = p.splits > 1 ? p.kper : a.K;
            const bool all3 = a.pre_beta && a.pre_mean && a.pre_var, none3 = !a.pre_beta && !a.pre_mean && !a.pre_var;
            if (!(clean && y_kc && (cfg == 2 || cfg == 4) && range <= kPreBnMaxK && (all3 || none3) &&
                  aligned16(a.pre_gamma) && aligned16(a.pre_beta) && aligned16(a.pre_mean) && aligned16(a.pre_var)))
                return K_EUNSUPPORTED;
            if (cfg == 4) {
                hipLaunchKernelGGL((gemm_clean_kernel<CfgT, true, 2, true>), grid, dim3(CfgT::THREADS), 0, s, p);
                g_last_kernel = "gemm_prebn_32x32_kc_s2";
            } else {
                hipLaunchKernelGGL((gemm_clean_kernel<CfgM, true, 2, true>), grid, dim3(CfgM::THREADS), 0, s, p);
                g_last_kernel = "gemm_prebn_64x64_kc_s2";
            }
            int err = (int)hipGetLastError();
            if (err) return err;
            if (p.splits > 1 && !p.tickets) return launch_splitk_reduce(ws.ptr, p.splits, a.M, a.N, a.C, p.ep, s);
            return 0;
        }
        int variant;
        if (cfg == 0)
            variant = launch_fast<CfgL>(p, y_kc, clean, grid, s);
        else if (cfg == 1)
            variant = launch_fast<CfgW>(p, y_kc, clean, grid, s);
        else if (cfg == 3)
            variant = launch_clean_only<CfgS>(p, y_kc, grid, s);
        else if (cfg == 4)
            variant = launch_clean_only<CfgT>(p, y_kc, grid, s);
        else
            variant = launch_fast<CfgM>(p, y_kc, clean, grid, s);
        g_last_kernel = names[cfg][y_kc ? 1 : 0][variant];
    } else {
        if (a.pre_gamma) return K_EUNSUPPORTED;
        p.xr = p.xc = 0;
        dim3 grid(p.tiles_m * p.tiles_n, 1, p.splits > 1 ? p.splits : batch);
        hipLaunchKernelGGL(gemm_generic_kernel, grid, dim3(256), 0, s, p);
        g_last_kernel = "gemm_generic_64x64";
    }
    int err = (int)hipGetLastError();
    if (err) return err;
    if (p.splits > 1 && !p.tickets) return launch_splitk_reduce(ws.ptr, p.splits, a.M, a.N, a.C, p.ep, s);
    return 0;
}

}  // namespace tpk
