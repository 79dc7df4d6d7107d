// fp32 MFMA block-tile machinery shared by the dense GEMM and implicit-GEMM
// convolution kernels (gfx950 / CDNA4, 64-wide wavefronts).
//
// A workgroup is 256 threads = 4 wavefronts laid out WGM x WGN over a BM x BN
// output tile.  Each wavefront owns TM x TN accumulators of 32x32, fed by
// v_mfma_f32_32x32x2_f32.  Both operand tiles live in LDS as [row][k] with a
// padded row pitch so that one ds_read_b128 per lane fetches four consecutive
// k values of that lane's row; lane half h (lane/32) takes k = 8g+4h .. 8g+4h+3
// of every group of eight, and MFMA step s multiplies k = 8g+s (half 0) with
// k = 8g+4+s (half 1).  The sum over k is order-free, so A and B only have to
// agree on this permutation, which they do because both use the same lane math.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tpk {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

enum Act : int { ACT_NONE = 0, ACT_RELU = 1, ACT_GELU = 2, ACT_TANH = 3, ACT_RELU6 = 4, ACT_SILU = 5, ACT_SIGMOID = 6 };

// Kernel arguments live in memory and the compiler fetches each one where it is first used; in a
// prologue full of dependent branches that is a chain of a dozen scalar-load round trips of a few
// hundred cycles each before the first operand load goes out.  fetch_now pins a value into a scalar
// register at the point of the call, so a run of calls at the top of a kernel turns the chain into
// one batch of loads and one wait.
template <class T>
__device__ __forceinline__ void fetch_now(const T& v) {
    asm volatile("" ::"s"(v));
}

// out = act( bn( alpha*acc + beta*C_old + bias[n] ) + residual )
struct Epilogue {
    float alpha;
    float beta;
    const float* bias;      // [N] or nullptr
    const float* bn_scale;  // gamma[N] or nullptr (all four bn_* set together)
    const float* bn_bias;   // beta[N]
    const float* bn_mean;   // running mean[N]
    const float* bn_var;    // running var[N]
    float bn_eps;
    const float* residual;  // [M][ldr] or nullptr (same mapping as C when out_nchw)
    long ldr;
    int act;
    // output mapping: element (row, col) lives at row*ldc + col, or, for an
    // NCHW convolution output with row = n*howo + p, at (n*ncols + col)*howo + p.
    long ldc;
    int out_nchw;
    long howo;
    long ncols;
};

__device__ __forceinline__ void fetch_now(const Epilogue& e) {
    fetch_now(e.alpha);
    fetch_now(e.beta);
    fetch_now(e.bias);
    fetch_now(e.bn_scale);
    fetch_now(e.bn_bias);
    fetch_now(e.bn_mean);
    fetch_now(e.bn_var);
    fetch_now(e.bn_eps);
    fetch_now(e.residual);
    fetch_now(e.ldr);
    fetch_now(e.act);
    fetch_now(e.ldc);
    fetch_now(e.out_nchw);
}

__device__ __forceinline__ float apply_act(float v, int act) {
    if (act == ACT_RELU) return v > 0.f ? v : 0.f;
    if (act == ACT_GELU) return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f));
    if (act == ACT_TANH) return tanhf(v);
    if (act == ACT_RELU6) return fminf(fmaxf(v, 0.f), 6.f);
    if (act == ACT_SILU) return v / (1.0f + expf(-v));
    if (act == ACT_SIGMOID) return 1.0f / (1.0f + expf(-v));
    return v;
}

__device__ __forceinline__ long out_index(const Epilogue& e, long row, long col, long pitch) {
    if (e.out_nchw) {
        const long n = row / e.howo;
        const long p = row - n * e.howo;
        return (n * e.ncols + col) * e.howo + p;
    }
    return row * pitch + col;
}

// Full epilogue for one element given its folded column constants.
__device__ __forceinline__ void epilogue_store(const Epilogue& e, float* __restrict__ Cout, long row, long col,
                                               float x, float cs, float ct) {
    const long ci = out_index(e, row, col, e.ldc);
    x *= e.alpha;
    if (e.beta != 0.f) x += e.beta * Cout[ci];
    x = x * cs + ct;
    if (e.residual) x += e.residual[out_index(e, row, col, e.ldr)];
    Cout[ci] = apply_act(x, e.act);
}

// Per-column constants of the epilogue folded to v*cs + ct.
__device__ __forceinline__ void epilogue_column(const Epilogue& e, long col, float& cs, float& ct) {
    float b = e.bias ? e.bias[col] : 0.f;
    cs = 1.f;
    ct = b;
    if (e.bn_scale) {
        float inv = 1.0f / sqrtf(e.bn_var[col] + e.bn_eps);
        float g = e.bn_scale[col] * inv;
        cs = g;
        ct = (b - e.bn_mean[col]) * g + e.bn_bias[col];
    }
}

// WGM x WGN wavefronts tile the BM x BN output; WGK > 1 adds wavefronts that share an output
// tile and each multiply a 1/WGK slice of every K-block (their sums are combined through LDS
// when the K loop ends), which keeps four wavefronts busy on tiles as small as 64x32.
template <int BM_, int BN_, int BK_, int WGM_, int WGN_, int WGK_ = 1>
struct TileCfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WGM = WGM_, WGN = WGN_, WGK = WGK_;
    static constexpr int THREADS = 64 * WGM * WGN * WGK;
    static constexpr int WTM = BM / WGM, WTN = BN / WGN;  // per-wavefront tile
    static constexpr int TM = WTM / 32, TN = WTN / 32;    // 32x32 MFMA tiles per wavefront
    static constexpr int LDK = BK + 4;                    // LDS row pitch in floats
    static constexpr int LDS_FLOATS = (BM + BN) * LDK;
    static_assert(BK % (8 * WGK) == 0, "each K slice must be a multiple of 8");
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be 32-aligned");
};

template <class C>
__device__ __forceinline__ void zero_acc(f32x16 (&acc)[C::TM][C::TN]) {
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
}

// Multiply the LDS-resident BM x BK and BN x BK tiles into the accumulators.  The operand
// fragments of k-group g+1 are fetched from LDS before the MFMAs of group g are issued, so the
// LDS latency hides behind matrix work instead of stalling every eighth MFMA.
template <class C>
__device__ __forceinline__ void mma_block(const float* __restrict__ As, const float* __restrict__ Bs,
                                          f32x16 (&acc)[C::TM][C::TN], int wm, int wn, int lane, int wk = 0) {
    const int r = lane & 31;
    const int h = lane >> 5;
    constexpr int G = C::BK / 8 / C::WGK;  // k-groups of 8 in this wavefront's slice
    const float* ap = As + (wm * C::WTM + r) * C::LDK + 4 * h + wk * (G * 8);
    const float* bp = Bs + (wn * C::WTN + r) * C::LDK + 4 * h + wk * (G * 8);
    f32x4 a[2][C::TM], b[2][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; ++i) a[0][i] = *reinterpret_cast<const f32x4*>(ap + i * 32 * C::LDK);
#pragma unroll
    for (int j = 0; j < C::TN; ++j) b[0][j] = *reinterpret_cast<const f32x4*>(bp + j * 32 * C::LDK);
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int cur = g & 1, nxt = cur ^ 1;
        if (g + 1 < G) {
#pragma unroll
            for (int i = 0; i < C::TM; ++i)
                a[nxt][i] = *reinterpret_cast<const f32x4*>(ap + i * 32 * C::LDK + (g + 1) * 8);
#pragma unroll
            for (int j = 0; j < C::TN; ++j)
                b[nxt][j] = *reinterpret_cast<const f32x4*>(bp + j * 32 * C::LDK + (g + 1) * 8);
        }
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int i = 0; i < C::TM; ++i)
#pragma unroll
                for (int j = 0; j < C::TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][i][s], b[cur][j][s], acc[i][j], 0, 0, 0);
    }
}

// LDS traffic inside one wavefront needs no hardware barrier (the LDS serves a wavefront's
// instructions in order); this only keeps the compiler from moving accesses across it.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// LDS floats store_tile needs: one 32x32 staging block per wavefront.
constexpr int STAGE_BLOCK = 32 * 32;
template <class C>
constexpr int stage_floats() {
    return C::WGM * C::WGN * STAGE_BLOCK;
}
constexpr int cmax(int a, int b) { return a > b ? a : b; }

// LDS floats reduce_k_slices needs.
template <class C>
constexpr int red_floats() {
    return (C::WGK - 1) * C::WGM * C::WGN * C::TM * C::TN * 16 * 64;
}

// WGK > 1: the wavefronts of K slices 1.. hand their sums to slice 0 through `red`
// (red_floats<C>() floats of LDS that no wavefront still reads operands from: call it after the
// K loop's last barrier).  Returns false for the wavefronts that are done (slices 1..); the
// slice-0 wavefronts return true with the complete sums in acc.  wsp = wavefront index within
// its slice (wm * WGN + wn).
template <class C>
__device__ __forceinline__ bool reduce_k_slices(f32x16 (&acc)[C::TM][C::TN], float* __restrict__ red, int wk, int wsp,
                                                int lane) {
    if (C::WGK == 1) return true;
    constexpr int PER_WAVE = C::TM * C::TN * 16 * 64;
    if (wk > 0) {
        float* dst = red + ((wk - 1) * C::WGM * C::WGN + wsp) * PER_WAVE + lane;
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
#pragma unroll
            for (int j = 0; j < C::TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) dst[((i * C::TN + j) * 16 + v) * 64] = acc[i][j][v];
    }
    __syncthreads();
    if (wk > 0) return false;
#pragma unroll 1
    for (int z = 1; z < C::WGK; ++z) {
        const float* src = red + ((z - 1) * C::WGM * C::WGN + wsp) * PER_WAVE + lane;
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
#pragma unroll
            for (int j = 0; j < C::TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] += src[((i * C::TN + j) * 16 + v) * 64];
    }
    return true;
}

// A K range split over `splits` workgroups, summed inside the launch.  Every workgroup of a tile writes
// its accumulators, register by register and lane-major (so each store instruction covers 256 contiguous
// bytes), to slot `split` of the tile's block in `part`, then draws a ticket; the workgroup that draws the
// last one reads all slots back in slot order -- a fixed order of summation, whichever workgroup it is --
// and returns true with the complete sums in acc; the others return false and are done.
//
// The 8 XCDs have private L2s that are not coherent with each other for ordinary accesses, and an
// agent-scope fence writes back / invalidates a whole L2.  So partial sums and tickets are moved with
// relaxed agent-scope atomic accesses instead (write-through stores, loads that bypass the L2, a
// read-modify-write at the memory side): coherent per access, nothing to flush.  The wait for the stores
// before the ticket is explicit, since a workgroup barrier alone does not wait for global stores.
// tickets[tile] is zero at entry and zero again when the last workgroup leaves.
// Call it from every wavefront that holds sums (the K-slice-0 wavefronts) after the K loop's last
// barrier; `flag` is one word of LDS that nobody uses meanwhile.
template <class C>
__device__ __forceinline__ bool finish_split(f32x16 (&acc)[C::TM][C::TN], float* __restrict__ part,
                                             unsigned* __restrict__ tickets, int splits, int tile, int split, int wsp,
                                             int lane, unsigned* flag) {
    constexpr int PER_WAVE = C::TM * C::TN * 16 * 64;
    constexpr long TILE_FLOATS = (long)C::WGM * C::WGN * PER_WAVE;
    float* mine = part + ((long)tile * splits + split) * TILE_FLOATS + wsp * PER_WAVE + lane;
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v)
                __hip_atomic_store(mine + ((i * C::TN + j) * 16 + v) * 64, acc[i][j][v], __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's partial sums have reached memory
    __syncthreads();
    if (threadIdx.x == 0)
        *flag = __hip_atomic_fetch_add(tickets + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*flag != (unsigned)(splits - 1)) return false;
    if (threadIdx.x == 0) __hip_atomic_store(tickets + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const float* src = part + (long)tile * splits * TILE_FLOATS + wsp * PER_WAVE + lane;
    // four slots are fetched together (their loads are all in flight before the first is used) and
    // then added in slot order
    constexpr int NR = C::TM * C::TN * 16;
    constexpr int ZU = NR <= 16 ? 4 : 2;
#pragma unroll 1
    for (int z = 0; z < splits; z += ZU) {
        float x[ZU][NR];
#pragma unroll
        for (int u = 0; u < ZU; ++u) {
            const int zz = z + u < splits ? z + u : splits - 1;  // past the end: re-read the last slot, unused
#pragma unroll
            for (int r = 0; r < NR; ++r)
                x[u][r] = __hip_atomic_load(src + (long)zz * TILE_FLOATS + r * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int u = 0; u < ZU; ++u) {
            if (z + u < splits) {
#pragma unroll
                for (int i = 0; i < C::TM; ++i)
#pragma unroll
                    for (int j = 0; j < C::TN; ++j)
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const float y = x[u][(i * C::TN + j) * 16 + v];
                            acc[i][j][v] = (z + u == 0) ? y : acc[i][j][v] + y;
                        }
            }
        }
    }
    return true;
}

__device__ __forceinline__ bool aligned16_dev(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Activation with the kind fixed at compile time: the write-out loops are instantiated per kind and
// entered through one switch, instead of testing the kind for every element (a taken branch costs a
// wavefront that is alone on its SIMD tens of cycles, and there were six per element).
template <int ACT>
__device__ __forceinline__ float act_fixed(float v) {
    if (ACT == ACT_RELU) return v > 0.f ? v : 0.f;
    if (ACT == ACT_GELU) return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f));
    if (ACT == ACT_TANH) return tanhf(v);
    if (ACT == ACT_RELU6) return fminf(fmaxf(v, 0.f), 6.f);
    if (ACT == ACT_SILU) return v / (1.0f + expf(-v));
    if (ACT == ACT_SIGMOID) return 1.0f / (1.0f + expf(-v));
    return v;
}

// The per-column constants of a wavefront's TN column blocks for the vector write-out, folded to
// x * cs + ct.  A kernel issues the loads when it starts (cols_issue) and folds them once its first
// operand loads are on their way (cols_fold), so that their latency is not paid at the end, where
// nothing else is left to hide it.  ok = the wavefront qualifies for the vector write-out.
template <int TN>
struct ColConsts {
    f32x4 cs[TN], ct[TN];   // after cols_issue: ct = bias, cs = gamma
    f32x4 vr[TN], mu[TN], bb[TN];
    bool ok = false, bn = false;
};

template <class C>
__device__ __forceinline__ bool vec_store_ok(const Epilogue& e, const float* Cout, long n0, int wn, long N) {
    return n0 + (wn + 1) * C::WTN <= N && !e.out_nchw && e.beta == 0.f && (e.ldc & 3) == 0 && aligned16_dev(Cout) &&
           (!e.bias || aligned16_dev(e.bias)) &&
           (!e.bn_scale || (aligned16_dev(e.bn_scale) && aligned16_dev(e.bn_var) && aligned16_dev(e.bn_mean) &&
                            aligned16_dev(e.bn_bias))) &&
           (!e.residual || ((e.ldr & 3) == 0 && aligned16_dev(e.residual)));
}

template <class C>
__device__ __forceinline__ void cols_issue(ColConsts<C::TN>& cc, const Epilogue& e, const float* Cout, long n0, int wn,
                                           int lane, long N) {
    cc.ok = vec_store_ok<C>(e, Cout, n0, wn, N);
    cc.bn = e.bn_scale != nullptr;
    if (!cc.ok) return;
#pragma unroll
    for (int j = 0; j < C::TN; ++j) {
        const long col = n0 + wn * C::WTN + j * 32 + (lane & 7) * 4;
        cc.ct[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        cc.cs[j] = f32x4{1.f, 1.f, 1.f, 1.f};
        if (e.bias) cc.ct[j] = *reinterpret_cast<const f32x4*>(e.bias + col);
        if (cc.bn) {
            cc.cs[j] = *reinterpret_cast<const f32x4*>(e.bn_scale + col);
            cc.vr[j] = *reinterpret_cast<const f32x4*>(e.bn_var + col);
            cc.mu[j] = *reinterpret_cast<const f32x4*>(e.bn_mean + col);
            cc.bb[j] = *reinterpret_cast<const f32x4*>(e.bn_bias + col);
        }
    }
}

template <class C>
__device__ __forceinline__ void cols_fold(ColConsts<C::TN>& cc, const Epilogue& e) {
    if (!cc.ok || !cc.bn) return;
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
        for (int c = 0; c < 4; ++c) {  // same arithmetic as epilogue_column
            const float inv = 1.0f / sqrtf(cc.vr[j][c] + e.bn_eps);
            const float gg = cc.cs[j][c] * inv;
            const float b = cc.ct[j][c];
            cc.cs[j][c] = gg;
            cc.ct[j][c] = (b - cc.mu[j][c]) * gg + cc.bb[j][c];
        }
}

// Vector form of the accumulator write-out for the common case: row-major output with 16-byte
// aligned rows, no beta term, whole 32-column blocks in range.  Each 32x32 block goes through the
// wavefront's LDS staging block and comes back transposed to "four consecutive columns per
// lane", so one step writes eight rows with 128-bit stores (4 steps per block instead of 16 with
// 32-bit stores).  The four steps are straight-line code with the activation fixed at compile time:
// no load sits under a branch (that makes the compiler wait for every outstanding memory operation
// at the join, stores included) and no branch is taken per element.  RES: add a residual tensor
// (rows clamped for the load, the store is predicated).  RAW: split-K partial sums, no epilogue.
template <class C, bool RES, bool RAW, int ACT>
__device__ __forceinline__ void store_tile_rows(f32x16 (&acc)[C::TM][C::TN], int wm, int wn, int lane, long m0, long n0,
                                                long M, float* __restrict__ out, long pitch, const Epilogue& e,
                                                float* __restrict__ stage, const ColConsts<C::TN>& cc) {
    const int r = lane & 31;
    const int h = lane >> 5;
    const int cq = (lane & 7) * 4;  // this lane's four columns within the block
    const int rq = lane >> 3;       // and its row within each group of eight
#pragma unroll
    for (int j = 0; j < C::TN; ++j) {
        const long col = n0 + wn * C::WTN + j * 32 + cq;
#pragma unroll
        for (int i = 0; i < C::TM; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) stage[((v >> 2) * 8 + h * 4 + (v & 3)) * 32 + r] = acc[i][j][v];
            wave_lds_sync();
            const long row0 = m0 + wm * C::WTM + i * 32 + rq;
            f32x4 x[4], res[4];
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                x[it] = *reinterpret_cast<const f32x4*>(stage + (it * 8 + rq) * 32 + cq);
                if (RES) {
                    const long row = row0 + it * 8;
                    const long rr = row < M ? row : M - 1;
                    res[it] = *reinterpret_cast<const f32x4*>(e.residual + rr * e.ldr + col);
                }
            }
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const long row = row0 + it * 8;
                if (!RAW) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        float y = x[it][c] * e.alpha;
                        y = y * cc.cs[j][c] + cc.ct[j][c];
                        if (RES) y += res[it][c];
                        x[it][c] = act_fixed<ACT>(y);
                    }
                }
                if (row < M) *reinterpret_cast<f32x4*>(out + row * pitch + col) = x[it];
            }
            wave_lds_sync();
        }
    }
}

template <class C, bool RES, bool RAW>
__device__ __forceinline__ void store_tile_vec(f32x16 (&acc)[C::TM][C::TN], int wm, int wn, int lane, long m0, long n0,
                                               long M, float* __restrict__ out, long pitch, const Epilogue& e,
                                               float* __restrict__ stage, const ColConsts<C::TN>& cc) {
    if (RAW) {
        store_tile_rows<C, false, true, ACT_NONE>(acc, wm, wn, lane, m0, n0, M, out, pitch, e, stage, cc);
        return;
    }
    switch (e.act) {
        case ACT_RELU: store_tile_rows<C, RES, false, ACT_RELU>(acc, wm, wn, lane, m0, n0, M, out, pitch, e, stage, cc); break;
        case ACT_GELU: store_tile_rows<C, RES, false, ACT_GELU>(acc, wm, wn, lane, m0, n0, M, out, pitch, e, stage, cc); break;
        case ACT_TANH: store_tile_rows<C, RES, false, ACT_TANH>(acc, wm, wn, lane, m0, n0, M, out, pitch, e, stage, cc); break;
        case ACT_RELU6: store_tile_rows<C, RES, false, ACT_RELU6>(acc, wm, wn, lane, m0, n0, M, out, pitch, e, stage, cc); break;
        case ACT_SILU: store_tile_rows<C, RES, false, ACT_SILU>(acc, wm, wn, lane, m0, n0, M, out, pitch, e, stage, cc); break;
        case ACT_SIGMOID: store_tile_rows<C, RES, false, ACT_SIGMOID>(acc, wm, wn, lane, m0, n0, M, out, pitch, e, stage, cc); break;
        default: store_tile_rows<C, RES, false, ACT_NONE>(acc, wm, wn, lane, m0, n0, M, out, pitch, e, stage, cc); break;
    }
}

// Write the accumulators.  `partial` != nullptr: raw sums go to the split-K workspace slice
// [M][N]; otherwise the epilogue is applied and C is written.
//
// Each 32x32 accumulator block first goes to `stage` (1024 floats of LDS private to this
// wavefront; the caller guarantees that every wavefront has finished reading the operand
// tiles).  Wavefronts whose columns are all in range and whose output rows are 16-byte aligned
// take store_tile_vec; the rest (NCHW outputs, a beta term, ragged right edge, odd pitches) a
// rolled 16-step loop that writes two rows per step.  Rolled or short loops keep one copy of the
// epilogue in the program instead of one per accumulator register: the unrolled form was tens of
// thousands of instructions, whose fetch alone cost up to a third of a GEMM.
template <class C>
__device__ __forceinline__ void store_tile(f32x16 (&acc)[C::TM][C::TN], int wm, int wn, int lane, long m0, long n0,
                                           long M, long N, float* __restrict__ Cout, const Epilogue& e,
                                           float* __restrict__ partial, float* __restrict__ stage,
                                           const ColConsts<C::TN>* pre = nullptr) {
    const int r = lane & 31;
    const int h = lane >> 5;
    if (n0 + (wn + 1) * C::WTN <= N) {  // the same for every lane of the wavefront
        if (partial) {
            if ((N & 3) == 0 && aligned16_dev(partial)) {
                ColConsts<C::TN> none;
                store_tile_vec<C, false, true>(acc, wm, wn, lane, m0, n0, M, partial, N, e, stage, none);
                return;
            }
        } else if (pre ? pre->ok : vec_store_ok<C>(e, Cout, n0, wn, N)) {
            ColConsts<C::TN> own;
            if (!pre) {  // the kernel did not fetch them ahead: fetch and fold here
                cols_issue<C>(own, e, Cout, n0, wn, lane, N);
                cols_fold<C>(own, e);
                pre = &own;
            }
            if (!e.residual)
                store_tile_vec<C, false, false>(acc, wm, wn, lane, m0, n0, M, Cout, e.ldc, e, stage, *pre);
            else
                store_tile_vec<C, true, false>(acc, wm, wn, lane, m0, n0, M, Cout, e.ldc, e, stage, *pre);
            return;
        }
    }
#pragma unroll
    for (int j = 0; j < C::TN; ++j) {
        const long col = n0 + wn * C::WTN + j * 32 + r;
        const bool col_ok = col < N;
        float cs = 1.f, ct = 0.f;
        if (!partial && col_ok) epilogue_column(e, col, cs, ct);
#pragma unroll
        for (int i = 0; i < C::TM; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) stage[((v >> 2) * 8 + h * 4 + (v & 3)) * 32 + r] = acc[i][j][v];
            wave_lds_sync();
            const long row0 = m0 + wm * C::WTM + i * 32 + h;
#pragma unroll 1
            for (int it = 0; it < 16; ++it) {
                const long row = row0 + 2 * it;
                const float x = stage[(2 * it + h) * 32 + r];
                if (row < M && col_ok) {
                    if (partial)
                        partial[row * N + col] = x;
                    else
                        epilogue_store(e, Cout, row, col, x, cs, ct);
                }
            }
            wave_lds_sync();
        }
    }
}

}  // namespace tpk
