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
    int tiles_m, tiles_n;
    Epilogue ep;
};

// Workgroups are handed to the 8 XCDs round-robin by linear id; remap so that
// each XCD (own L2) works on a contiguous run of tiles.
__device__ __forceinline__ int remap_xcd(int bid, int n) {
    const int q = n >> 3, rem = n & 7;
    const int xcd = bid & 7, local = bid >> 3;
    return xcd * q + (xcd < rem ? xcd : rem) + local;
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
__global__ __launch_bounds__(C::THREADS, 2) void gemm_fast_kernel(const GemmDev p) {
    __shared__ __attribute__((aligned(16))) float lds[C::LDS_FLOATS];
    float* As = lds;
    float* Bs = lds + C::BM * C::LDK;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / C::WGN, wn = wave % C::WGN;
    const int t = remap_xcd(blockIdx.x, p.tiles_m * p.tiles_n);
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
    f32x4 ra[NVA], rb[NVB];

    auto load_regs = [&](long k0) {
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
    auto store_lds = [&]() {
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

    load_regs(kbeg);
    for (long k0 = kbeg; k0 < kend; k0 += C::BK) {
        store_lds();
        __syncthreads();
        if (k0 + C::BK < kend) load_regs(k0 + C::BK);
        mma_block<C>(As, Bs, acc, wm, wn, lane);
        __syncthreads();
    }
    float* partial = nullptr;
    if (p.splits > 1) partial = p.ws + (long)split * p.M * p.N;
    store_tile<C>(acc, wm, wn, lane, m0, n0, p.M, p.N, Cc, p.ep, partial);
}

// Any strides, any alignment.  64x64x16 tile, scalar loads.
using GenCfg = TileCfg<64, 64, 16, 2, 2>;

__global__ __launch_bounds__(GenCfg::THREADS, 2) void gemm_generic_kernel(const GemmDev p) {
    using C = GenCfg;
    __shared__ __attribute__((aligned(16))) float lds[C::LDS_FLOATS];
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
    if (p.splits > 1) partial = p.ws + (long)split * p.M * p.N;
    store_tile<C>(acc, wm, wn, lane, m0, n0, p.M, p.N, Cc, p.ep, partial);
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

using CfgL = TileCfg<128, 128, 32, 2, 2>;
using CfgM = TileCfg<64, 64, 32, 2, 2>;

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Pick the split-K factor: fill the chip when the tile count alone cannot.
int choose_splits(long tiles, long K, int bk, long M, long N, size_t ws_bytes, long* kper_out) {
    int splits = 1;
    const long kblocks = (K + bk - 1) / bk;
    if (tiles < g_num_cu && kblocks >= 8) {
        long want = (2L * g_num_cu + tiles - 1) / tiles;
        long maxs = kblocks / 4;  // keep at least 4 K-blocks per split
        if (want > maxs) want = maxs;
        if (want > 32) want = 32;
        const size_t per = (size_t)M * (size_t)N * sizeof(float);
        while (want > 1 && (size_t)want * per > ws_bytes) --want;
        if (want > 1) splits = (int)want;
    }
    long per_blocks = (kblocks + splits - 1) / splits;
    splits = (int)((kblocks + per_blocks - 1) / per_blocks);
    *kper_out = per_blocks * bk;
    return splits;
}

int launch_gemm(const GemmArgs& a, const Workspace& ws, hipStream_t s) {
    if (a.M <= 0 || a.N <= 0 || a.K < 0 || !a.X || !a.Y || !a.C) return K_EINVAL;
    if (a.nb0 < 1 || a.nb1 < 1) return K_EINVAL;
    if (!((a.xs_k == 1) || (a.xs_r == 1)) || !((a.ys_k == 1) || (a.ys_c == 1))) return K_EINVAL;
    if (a.gather && (a.Ho <= 0 || a.Wo <= 0 || a.H <= 0 || a.W <= 0)) return K_EINVAL;
    const int batch = a.nb0 * a.nb1;

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

    const bool x_fast = a.xs_k == 1 && (a.xs_r % 4 == 0) && (a.K % 4 == 0) && aligned16(a.X) && (a.xb0 % 4 == 0) &&
                        (a.xb1 % 4 == 0);
    const bool y_kc = a.ys_k == 1 && (a.ys_c % 4 == 0) && (a.K % 4 == 0);
    const bool y_cc = a.ys_c == 1 && a.ys_k != 1 && (a.ys_k % 4 == 0);
    const bool y_fast = (y_kc || y_cc) && aligned16(a.Y) && (a.yb0 % 4 == 0) && (a.yb1 % 4 == 0);

    if (x_fast && y_fast) {
        const long tl = ((a.M + 127) / 128) * ((a.N + 127) / 128) * batch;
        const bool big = tl >= 2L * g_num_cu;
        const int bm = big ? 128 : 64;
        p.tiles_m = (int)((a.M + bm - 1) / bm);
        p.tiles_n = (int)((a.N + bm - 1) / bm);
        const long tiles = (long)p.tiles_m * p.tiles_n * batch;
        p.splits = 1;
        p.kper = ((a.K + 31) / 32) * 32;
        if (batch == 1) p.splits = choose_splits(tiles, a.K, 32, a.M, a.N, ws.ptr ? ws.bytes : 0, &p.kper);
        dim3 grid(p.tiles_m * p.tiles_n, 1, p.splits > 1 ? p.splits : batch);
        if (big) {
            if (y_kc) {
                hipLaunchKernelGGL((gemm_fast_kernel<CfgL, true>), grid, dim3(256), 0, s, p);
                g_last_kernel = "gemm_fast_128x128_kc";
            } else {
                hipLaunchKernelGGL((gemm_fast_kernel<CfgL, false>), grid, dim3(256), 0, s, p);
                g_last_kernel = "gemm_fast_128x128_cc";
            }
        } else {
            if (y_kc) {
                hipLaunchKernelGGL((gemm_fast_kernel<CfgM, true>), grid, dim3(256), 0, s, p);
                g_last_kernel = "gemm_fast_64x64_kc";
            } else {
                hipLaunchKernelGGL((gemm_fast_kernel<CfgM, false>), grid, dim3(256), 0, s, p);
                g_last_kernel = "gemm_fast_64x64_cc";
            }
        }
    } else {
        p.tiles_m = (int)((a.M + 63) / 64);
        p.tiles_n = (int)((a.N + 63) / 64);
        const long tiles = (long)p.tiles_m * p.tiles_n * batch;
        p.splits = 1;
        p.kper = ((a.K + 15) / 16) * 16;
        if (batch == 1) p.splits = choose_splits(tiles, a.K, 16, a.M, a.N, ws.ptr ? ws.bytes : 0, &p.kper);
        dim3 grid(p.tiles_m * p.tiles_n, 1, p.splits > 1 ? p.splits : batch);
        hipLaunchKernelGGL(gemm_generic_kernel, grid, dim3(256), 0, s, p);
        g_last_kernel = "gemm_generic_64x64";
    }
    int err = (int)hipGetLastError();
    if (err) return err;
    if (p.splits > 1) return launch_splitk_reduce(ws.ptr, p.splits, a.M, a.N, a.C, p.ep, s);
    return 0;
}

}  // namespace tpk
