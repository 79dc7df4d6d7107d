// 3x3 stride-1 convolution as Winograd F(2x2, 3x3) on fp32 MFMA for gfx950.
//
// One of the paths behind the cudnnConvolutionForward call site of the reference executor
// (include/server/cuda_server.hpp:708-735; its traces show cuDNN picking Winograd kernels for these
// layers too, misc/tools/resnet_all.txt:34-48).  The output is cut into 2x2 tiles; with
//   U = G g G^T   (the 3x3 filter of one (cout, cin) pair -> 4x4)
//   V = B^T d B   (the 4x4 input patch of one (tile, cin) pair -> 4x4)
// the tile's outputs are Y = A^T [ sum_cin U .* V ] A: sixteen independent products
// M[xi] = V[xi] (tiles x cin) . U[xi]^T (cin x cout), xi = 4i + j, with 2.25 times fewer multiplications
// than the direct form.  Nothing is precomputed or stored: the filter bytes stay as they were uploaded
// (they are swapped in and out byte for byte) and U is formed on the fly -- a few dozen additions per
// filter, repeated by every workgroup that needs it, against thousands of matrix-core cycles.
//
// A workgroup owns 32 tiles x 32 output channels x all sixteen xi for a slice of the input channels, in
// K-blocks of 16 input channels.  Patches are fetched by thread = tile x channel quad (sixteen 128-bit loads)
// and filters by thread = output channel x channel quad (36 contiguous floats), transformed in registers and
// written as [xi][row][16 channels] operand blocks into LDS, XOR-swizzled in 16-byte chunks so that the
// 128-bit fragment reads of the MFMA loop are conflict-free without padding.  The fragment layout and K
// permutation are those of mma_block (mfma_tile.hpp).  How the work is spread over the wavefronts is
// described at the kernel.
//
// After the K loop each multiplying wavefront folds its row over j (T[i][b] = sum_j M[i][j] A^T[b][j]), the
// four rows are exchanged through LDS, and wavefront (a, b) ends up with output pixel (a, b) of every tile as
// one 32x32 block (tiles x channels) in the usual accumulator layout.  A split over input channels is summed
// inside the launch by finish_split, in slot order.
#include "kernels.hpp"
#include "mfma_tile.hpp"

#include <cstdlib>

namespace tpk {

void set_last_kernel(const char* n);
int num_cu();
Epilogue make_epilogue(const EpilogueArgs& a, long ldc);
unsigned* split_tickets(const Workspace& ws, long tiles, int splits);

namespace {

constexpr int kKC = 16;                        // input channels per K-block
constexpr int kOperandFloats = 16 * 32 * kKC;  // V (or U of 32 output channels) of one K-block: [xi][row][channel]
// Blocks of 32 output channels per workgroup.  The multiply, exchange and write-out code is written for any count;
// the fetch and transform jobs of the kernel and the launcher's grid are laid out for one (two was measured
// slower, see the launcher).
constexpr int kNB = 1;

struct WinoDev {
    const float* x;
    const float* w;
    float* y;
    int H, W, Cin, Cout;   // stride 1, padding 1: the output is H x W as well
    long xp, yp;           // floats between pixels of x / y
    unsigned xbytes, wbytes;  // extent of x and of w in bytes (both below 2^31)
    int tiles_h, tiles_w;  // 2x2 output tiles per image
    long ntiles;           // N * tiles_h * tiles_w
    int mt, nt;            // blocks of 32 tiles / of 32 output channels
    int splits, cper;      // input-channel slices and channels per slice (a multiple of kKC)
    float* ws;
    unsigned* tickets;
    Epilogue ep;
};

// what finish_split and the write-out need to know: four wavefronts with kNB 32x32 accumulator blocks each
struct WinoOutCfg {
    static constexpr int TM = 1, TN = kNB, WGM = 2, WGN = 2;
    static constexpr int WTN = 32 * kNB;  // columns of one wavefront's block of the output tile
};

__device__ __forceinline__ void fetch_args(const WinoDev& p) {
    fetch_now(p.x);
    fetch_now(p.w);
    fetch_now(p.y);
    fetch_now(p.H);
    fetch_now(p.W);
    fetch_now(p.Cin);
    fetch_now(p.xp);
    fetch_now(p.yp);
    fetch_now(p.xbytes);
    fetch_now(p.wbytes);
    fetch_now(p.tiles_h);
    fetch_now(p.tiles_w);
    fetch_now(p.ntiles);
    fetch_now(p.mt);
    fetch_now(p.nt);
    fetch_now(p.splits);
    fetch_now(p.cper);
    fetch_now(p.ws);
    fetch_now(p.tickets);
    fetch_now(p.ep);
}

__device__ __forceinline__ int remap_xcd_w(int bid, int n) {
    const int q = n >> 3, rem = n & 7;
    const int xcd = bid & 7, local = bid >> 3;
    return xcd * q + (xcd < rem ? xcd : rem) + local;
}

// Float offset of 16-byte chunk `chunk` (0..3) inside row `row` (16 floats = 64 bytes = half of the LDS's 32
// banks) of an operand block.  A 128-bit access is served eight lanes at a time: eight consecutive rows are four
// even ones on banks 0-15 and four odd ones on banks 16-31, and rows two apart get different chunks.
__device__ __forceinline__ int swz(int row, int chunk) { return (chunk ^ ((row >> 1) & 3)) << 2; }

// V = B^T d B of one 4x4 patch, for the two or four channels of a vector at a time, in place: first down the
// rows of every column, then along the columns of every row (d0 - d2, d1 + d2, d2 - d1, d1 - d3 each time);
// d[4i + j] = pixel (i, j), zeros where the patch reaches into the padding.  dst = this thread's channels of row
// `tile` in block xi = 0.
template <class V>
__device__ __forceinline__ void transform_patch(V (&d)[16], float* __restrict__ dst) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const V d1 = d[1 * 4 + j];
        d[0 * 4 + j] -= d[2 * 4 + j];
        d[1 * 4 + j] = d1 + d[2 * 4 + j];
        d[2 * 4 + j] -= d1;
        d[3 * 4 + j] = d1 - d[3 * 4 + j];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const V d1 = d[i * 4 + 1];
        const V v0 = d[i * 4 + 0] - d[i * 4 + 2];
        const V v1 = d1 + d[i * 4 + 2];
        const V v2 = d[i * 4 + 2] - d1;
        const V v3 = d1 - d[i * 4 + 3];
        *reinterpret_cast<V*>(dst + (i * 4 + 0) * 32 * kKC) = v0;
        *reinterpret_cast<V*>(dst + (i * 4 + 1) * 32 * kKC) = v1;
        *reinterpret_cast<V*>(dst + (i * 4 + 2) * 32 * kKC) = v2;
        *reinterpret_cast<V*>(dst + (i * 4 + 3) * 32 * kKC) = v3;
    }
}

// U = G g G^T for four input channels of one output channel; raw[0..8] = the 36 floats g[ci][kh][kw].
// dst = this thread's chunk of row `channel` in block xi = 0 of a [xi][ROWS][16] operand.
template <int ROWS, int NRAW>
__device__ __forceinline__ void transform_filter(const f32x4 (&raw)[NRAW], float* __restrict__ dst) {
    float a[4][4][3];  // [ci][i][kw] = (G g) of channel ci
#pragma unroll
    for (int ci = 0; ci < 4; ++ci) {
        float g[9];
#pragma unroll
        for (int k = 0; k < 9; ++k) {
            const int f = ci * 9 + k;
            g[k] = raw[f >> 2][f & 3];
        }
#pragma unroll
        for (int kw = 0; kw < 3; ++kw) {
            a[ci][0][kw] = g[0 * 3 + kw];
            a[ci][1][kw] = 0.5f * ((g[0 * 3 + kw] + g[1 * 3 + kw]) + g[2 * 3 + kw]);
            a[ci][2][kw] = 0.5f * ((g[0 * 3 + kw] - g[1 * 3 + kw]) + g[2 * 3 + kw]);
            a[ci][3][kw] = g[2 * 3 + kw];
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f32x4 u0, u1, u2, u3;
#pragma unroll
        for (int ci = 0; ci < 4; ++ci) {
            u0[ci] = a[ci][i][0];
            u1[ci] = 0.5f * ((a[ci][i][0] + a[ci][i][1]) + a[ci][i][2]);
            u2[ci] = 0.5f * ((a[ci][i][0] - a[ci][i][1]) + a[ci][i][2]);
            u3[ci] = a[ci][i][2];
        }
        *reinterpret_cast<f32x4*>(dst + (i * 4 + 0) * ROWS * kKC) = u0;
        *reinterpret_cast<f32x4*>(dst + (i * 4 + 1) * ROWS * kKC) = u1;
        *reinterpret_cast<f32x4*>(dst + (i * 4 + 2) * ROWS * kKC) = u2;
        *reinterpret_cast<f32x4*>(dst + (i * 4 + 3) * ROWS * kKC) = u3;
    }
}

// Write-out of one wavefront's kNB 32x32 blocks (rows = tiles, columns = output channels) for its output pixel
// (oa, ob) of every tile, in the form the GEMM tiles use: each block goes through the wavefront's LDS staging
// block and comes back as four consecutive columns per lane, so one step writes eight rows with 128-bit stores.
// Straight-line code with the activation fixed at compile time: a load under a branch (the residual, say) makes
// the compiler wait for every outstanding memory operation at the join, the stores of the previous step included
// -- the element-wise form of this write-out took 3.4 us of a 24 us launch that way.
template <bool RES, int ACT>
__device__ __forceinline__ void store_rows(f32x16 (&out)[1][kNB], int lane, long n0, const WinoDev& p, int pixoff, int oa,
                                           int ob, float* __restrict__ stage_blk, const int* rowpix, const int* rowok,
                                           const ColConsts<kNB>& cc) {
    const Epilogue& e = p.ep;
    const int r = lane & 31, h = lane >> 5;
    const int cq = (lane & 7) * 4;  // this lane's four columns within a block
    const int rq = lane >> 3;       // and its row within each group of eight
    long o[4];
    bool live[4];
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int pix = rowpix[it * 8 + rq];
        const int ok = rowok[it * 8 + rq];
        live[it] = pix >= 0 && (!oa || (ok & 1)) && (!ob || (ok & 2));
        o[it] = live[it] ? (long)(pix + pixoff) : 0;  // rows that are not written read the residual of pixel 0
    }
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
        const long col = n0 + nb * 32 + cq;
#pragma unroll
        for (int v = 0; v < 16; ++v) stage_blk[((v >> 2) * 8 + h * 4 + (v & 3)) * 32 + r] = out[0][nb][v];
        wave_lds_sync();
        f32x4 x[4], res[4];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            x[it] = *reinterpret_cast<const f32x4*>(stage_blk + (it * 8 + rq) * 32 + cq);
            if (RES) res[it] = *reinterpret_cast<const f32x4*>(e.residual + o[it] * e.ldr + col);
        }
#pragma unroll
        for (int it = 0; it < 4; ++it) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                float y = x[it][c] * e.alpha;
                y = y * cc.cs[nb][c] + cc.ct[nb][c];
                if (RES) y += res[it][c];
                x[it][c] = act_fixed<ACT>(y);
            }
            if (live[it]) *reinterpret_cast<f32x4*>(p.y + o[it] * p.yp + col) = x[it];
        }
        wave_lds_sync();
    }
}

template <bool RES>
__device__ __forceinline__ void store_rows_any_act(f32x16 (&out)[1][kNB], int lane, long n0, const WinoDev& p, int pixoff,
                                                   int oa, int ob, float* __restrict__ stage_blk, const int* rowpix,
                                                   const int* rowok, const ColConsts<kNB>& cc) {
    switch (p.ep.act) {
        case ACT_RELU: store_rows<RES, ACT_RELU>(out, lane, n0, p, pixoff, oa, ob, stage_blk, rowpix, rowok, cc); break;
        case ACT_GELU: store_rows<RES, ACT_GELU>(out, lane, n0, p, pixoff, oa, ob, stage_blk, rowpix, rowok, cc); break;
        case ACT_TANH: store_rows<RES, ACT_TANH>(out, lane, n0, p, pixoff, oa, ob, stage_blk, rowpix, rowok, cc); break;
        case ACT_RELU6: store_rows<RES, ACT_RELU6>(out, lane, n0, p, pixoff, oa, ob, stage_blk, rowpix, rowok, cc); break;
        case ACT_SILU: store_rows<RES, ACT_SILU>(out, lane, n0, p, pixoff, oa, ob, stage_blk, rowpix, rowok, cc); break;
        case ACT_SIGMOID: store_rows<RES, ACT_SIGMOID>(out, lane, n0, p, pixoff, oa, ob, stage_blk, rowpix, rowok, cc); break;
        default: store_rows<RES, ACT_NONE>(out, lane, n0, p, pixoff, oa, ob, stage_blk, rowpix, rowok, cc); break;
    }
}

constexpr unsigned kBeyond = 0x80000000u;  // a byte offset no tensor of this path reaches: such a load returns zeros

// A buffer descriptor that sits in scalar registers: say so in terms the compiler cannot overlook, or every
// load becomes a loop over the distinct descriptors of the wavefront's lanes.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t uniform_rsrc(const float* base, unsigned bytes) {
    const unsigned long long bits = reinterpret_cast<unsigned long long>(base);
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)bits);
    const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(bits >> 32));
    const unsigned extent = __builtin_amdgcn_readfirstlane(bytes);
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(((unsigned long long)hi << 32) | lo), 0, (int)extent,
                                             0x00020000);
}

// Byte offsets of the sixteen pixels of tile `tile_in_block`'s 4x4 input patch, pixel (i, j) = entry 4i + j, for
// the channels that start `chan` floats into the pixel; kBeyond where the patch reaches into the padding and
// for tiles past the last one.  32-bit arithmetic throughout (the launcher checks that every offset fits): a
// 64-bit division costs some hundred instructions and this is on every workgroup's way to its first load.
__device__ __forceinline__ void patch_offsets(const WinoDev& p, int tm, int tile_in_block, int chan, unsigned (&off)[16]) {
    const unsigned gt = (unsigned)tm * 32u + (unsigned)tile_in_block;
    const bool real = gt < (unsigned)p.ntiles;
    const unsigned q = gt / (unsigned)p.tiles_w;
    const int tw = (int)(gt - q * (unsigned)p.tiles_w);
    const unsigned n = q / (unsigned)p.tiles_h;
    const int th = (int)(q - n * (unsigned)p.tiles_h);
    const int hi0 = 2 * th - 1, wi0 = 2 * tw - 1;
    const int xp = (int)p.xp;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int hi = hi0 + i;
        const int rowoff = (((int)n * p.H + hi) * p.W) * xp + chan;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int wi = wi0 + j;
            const bool inside = real && hi >= 0 && hi < p.H && wi >= 0 && wi < p.W;
            off[i * 4 + j] = inside ? (unsigned)(rowoff + wi * xp) * 4u : kBeyond;
        }
    }
}

// Where each tile of the block writes: (n*H + 2*th)*W + 2*tw, -1 past the last tile; bit 0 of rowok: the tile's
// second output row exists, bit 1: its second column.
__device__ __forceinline__ void tile_rows(const WinoDev& p, int tm, int tid, int* rowpix, int* rowok) {
    if (tid < 32) {
        const unsigned gt = (unsigned)tm * 32u + (unsigned)tid;
        int pix = -1, ok = 0;
        if (gt < (unsigned)p.ntiles) {
            const unsigned q = gt / (unsigned)p.tiles_w;
            const int tw = (int)(gt - q * (unsigned)p.tiles_w);
            const unsigned n = q / (unsigned)p.tiles_h;
            const int th = (int)(q - n * (unsigned)p.tiles_h);
            pix = ((int)n * p.H + 2 * th) * p.W + 2 * tw;
            ok = (2 * th + 1 < p.H ? 1 : 0) | (2 * tw + 1 < p.W ? 2 : 0);
        }
        rowpix[tid] = pix;
        rowok[tid] = ok;
    }
}

// One K-block of the sixteen products: wavefront `wave` owns xi = 4*wave + j, j = 0..3, for kNB blocks of 32
// output channels.  Eight (k-group, xi) steps of 1 + kNB fragment reads and 4 * kNB MFMAs; the fragments of step
// n+1 are requested before the MFMAs of step n are issued, so the LDS latency hides behind matrix work.  Each
// step also calls prefetch(n), which issues that step's share of the next K-block's global loads: issued in one
// go after the barrier they held the wavefront for about a thousand cycles in which its SIMD did nothing else
// (measured with one workgroup per CU); between MFMAs the matrix pipeline is busy meanwhile.
// V is [xi][32 rows][16 channels], U is [xi][32*kNB rows][16 channels]; lane (r, h) reads row r, chunk 2g + h.
template <class Prefetch>
__device__ __forceinline__ void multiply_block(f32x16 (&acc)[4][kNB], const float* Vs, const float* Us, int wave, int r,
                                               int h, Prefetch prefetch) {
    const int vfrag0 = (wave * 4 * 32 + r) * kKC + swz(r, h);
    const int vfrag1 = (wave * 4 * 32 + r) * kKC + swz(r, 2 + h);
    const int ufrag0 = (wave * 4 * 32 * kNB + r) * kKC + swz(r, h);
    const int ufrag1 = (wave * 4 * 32 * kNB + r) * kKC + swz(r, 2 + h);
    f32x4 a[2], b[2][kNB];
    a[0] = *reinterpret_cast<const f32x4*>(Vs + vfrag0);
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) b[0][nb] = *reinterpret_cast<const f32x4*>(Us + ufrag0 + nb * 32 * kKC);
#pragma unroll
    for (int n = 0; n < 8; ++n) {
        const int cur = n & 1, nxt = cur ^ 1;
        if (n + 1 < 8) {
            const int g = (n + 1) >> 2, j = (n + 1) & 3;
            a[nxt] = *reinterpret_cast<const f32x4*>(Vs + (g ? vfrag1 : vfrag0) + j * 32 * kKC);
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb)
                b[nxt][nb] = *reinterpret_cast<const f32x4*>(Us + (g ? ufrag1 : ufrag0) + (j * kNB + nb) * 32 * kKC);
        }
        const int j = n & 3;
        acc[j][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][0], b[cur][0][0], acc[j][0], 0, 0, 0);
        prefetch(n);
#pragma unroll
        for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
            for (int s = (nb == 0 ? 1 : 0); s < 4; ++s)
                acc[j][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][s], b[cur][nb][s], acc[j][nb], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);  // or the scheduler gathers the loads at the end of the block again
    }
}

// After the K loop: output transform, sum over the input-channel slices, write-out.  The wavefront holds row
// i = wave of M; it folds the row over j, the four rows are exchanged through LDS (the operand blocks are no
// longer read: the caller's last barrier), and wavefront (oa, ob) ends up with output pixel (oa, ob) of every
// tile.  Returns early in every workgroup but the one that finishes a split tile last.
__device__ __forceinline__ void transform_and_store(f32x16 (&acc)[4][kNB], const WinoDev& p, float* lds, const int* rowpix,
                                                    const int* rowok, unsigned* flag, int wave, int lane, int t, int split,
                                                    int tn, ColConsts<kNB>& cc) {
    const int r = lane & 31, h = lane >> 5;
    float* ex = lds;  // [((i*2 + b)*kNB + nb)*16 + v][lane]
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            ex[(((wave * 2 + 0) * kNB + nb) * 16 + v) * 64 + lane] = (acc[0][nb][v] + acc[1][nb][v]) + acc[2][nb][v];
            ex[(((wave * 2 + 1) * kNB + nb) * 16 + v) * 64 + lane] = (acc[1][nb][v] - acc[2][nb][v]) - acc[3][nb][v];
        }
    __syncthreads();
    const int oa = wave >> 1, ob = wave & 1;
    f32x16 out[1][kNB];
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const float t1 = ex[(((1 * 2 + ob) * kNB + nb) * 16 + v) * 64 + lane];
            const float t2 = ex[(((2 * 2 + ob) * kNB + nb) * 16 + v) * 64 + lane];
            const float t03 = ex[((((oa ? 3 : 0) * 2 + ob) * kNB + nb) * 16 + v) * 64 + lane];
            out[0][nb][v] = oa ? (t1 - t2) - t03 : (t03 + t1) + t2;
        }
    if (p.splits > 1) {
        if (!finish_split<WinoOutCfg>(out, p.ws, p.tickets, p.splits, t, split, wave, lane, flag)) return;
    }

    // write-out: row of the block = tile, column = output channel
    const Epilogue& e = p.ep;
    const long n0 = (long)tn * 32 * kNB;
    const int pixoff = oa * p.W + ob;
    if (cc.ok) {
        cols_fold<WinoOutCfg>(cc, e);
        // beyond the exchange area (other wavefronts may still be reading theirs): 1024 floats per wavefront
        float* const stage_blk = lds + 8 * kNB * 1024 + wave * 1024;
        if (!e.residual) store_rows_any_act<false>(out, lane, n0, p, pixoff, oa, ob, stage_blk, rowpix, rowok, cc);
        else store_rows_any_act<true>(out, lane, n0, p, pixoff, oa, ob, stage_blk, rowpix, rowok, cc);
        return;
    }
    // odd pitches or unaligned tensors: one element at a time
#pragma unroll 1
    for (int nb = 0; nb < kNB; ++nb) {
        const long col = n0 + nb * 32 + r;
        float cs, ct;
        epilogue_column(e, col, cs, ct);
#pragma unroll 1
        for (int v = 0; v < 16; ++v) {
            const int row = (v >> 2) * 8 + h * 4 + (v & 3);
            const int pix = rowpix[row];
            const int ok = rowok[row];
            if (pix < 0 || (oa && !(ok & 1)) || (ob && !(ok & 2))) continue;
            const long o = (long)(pix + pixoff);
            float xv = out[0][nb][v] * e.alpha;
            xv = xv * cs + ct;
            if (e.residual) xv += e.residual[o * e.ldr + col];
            p.y[o * p.yp + col] = apply_act(xv, e.act);
        }
    }
}

// 32 tiles x 32 output channels per workgroup, 64 KiB of LDS, two workgroups per CU.  Four wavefronts; all of
// them multiply (multiply_block).  Before that, per K-block, wavefronts 0-1 fetch and transform the 4x4 patch
// of tile `row` for four input channels (pixel (i, j) = load 4i + j) and wavefronts 2-3 the filter of output
// channel `row` for four input channels (36 contiguous floats = loads 0..8); the loads of the next K-block are
// in flight while this one is multiplied.  All loads are buffer loads of 16 bytes: one descriptor per wavefront
// (x or w), a per-lane byte offset that never changes, and the K-block's offset in a scalar register -- no
// address arithmetic in the loop.  A load whose offset lies beyond the descriptor's extent returns zeros without
// touching memory: that is how the padding around the image, the tiles past the last one and a filter thread's
// loads 9..15 are expressed, so that every thread issues the same sixteen loads and none of them sits under a
// branch (two role branches that each end in a load get their tails merged by the compiler through a pointer in
// scratch memory, and a scratch access in the loop turns every wait into a wait for all loads in flight).
// Measured on MI355X: fp32 MFMAs and fp32 vector instructions share the SIMD's lanes -- n independent v_add_f32
// between two dependent MFMAs add 4.6 cycles each to the 64 of the MFMA, whatever n -- so a SIMD's time per
// K-block is its 2048 MFMA cycles plus its transform job, and wavefronts of their own for the transforms
// (built and measured) change nothing.
__global__ __launch_bounds__(256, 2) void conv_wino_kernel(const WinoDev p) {
    fetch_args(p);
    __shared__ __attribute__((aligned(16))) float lds[2 * kOperandFloats];  // [V | U] of one K-block
    __shared__ int rowpix[32];
    __shared__ int rowok[32];
    __shared__ unsigned flag;
    float* const Vs = lds;
    float* const Us = lds + kOperandFloats;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // the same for the whole wavefront: role branches are scalar
    const int t = remap_xcd_w((int)blockIdx.x, p.mt * p.nt);
    const int tm = t / p.nt, tn = t - tm * p.nt;
    const int split = (int)blockIdx.z;
    const int cbeg = split * p.cper;
    const int cend = cbeg + p.cper < p.Cin ? cbeg + p.cper : p.Cin;
    const int nblocks = (cend - cbeg) / kKC;

    const bool patches = wave < 2;
    const int q4 = (tid & 3) * 4;      // channel quad within the K-block
    const int row = (tid & 127) >> 2;  // tile / output channel within the block
    unsigned off[16];
    if (patches) {
        patch_offsets(p, tm, row, q4, off);
    } else {
        const unsigned fv = (unsigned)((tn * 32 + row) * p.Cin + q4) * 36u;  // whole blocks only: in range
#pragma unroll
        for (int k = 0; k < 16; ++k) off[k] = k < 9 ? fv + 16u * k : kBeyond;
    }
    const __amdgpu_buffer_rsrc_t rsrc = uniform_rsrc(patches ? p.x : p.w, patches ? p.xbytes : p.wbytes);
    const int chan_bytes = patches ? 4 : 36;  // from one input channel to the next
    f32x4 raw[16];
    auto load_one = [&](int k, int soff) {
        raw[k] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off[k], soff, 0));
    };

    // per-column constants of the epilogue, asked for now and folded at the very end
    ColConsts<kNB> cc;
    cols_issue<WinoOutCfg>(cc, p.ep, p.y, (long)tn * 32, 0, lane, p.Cout);
    tile_rows(p, tm, tid, rowpix, rowok);

    f32x16 acc[4][1];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[j][0][v] = 0.f;

#pragma unroll
    for (int k = 0; k < 16; ++k) load_one(k, cbeg * chan_bytes);
    for (int n = 0; n < nblocks; ++n) {
        if (patches) transform_patch(raw, Vs + row * kKC + swz(row, tid & 3));
        else transform_filter<32>(raw, Us + row * kKC + swz(row, tid & 3));
        __syncthreads();
        int c0 = cbeg + (n + 1) * kKC;
        if (c0 > cend - kKC) c0 = cend - kKC;  // the look-ahead past the end reads the last block again
        const int soff = c0 * chan_bytes;
        multiply_block(acc, Vs, Us, wave, lane & 31, lane >> 5, [&](int step) {
            load_one(2 * step, soff);
            load_one(2 * step + 1, soff);
        });
        __syncthreads();
    }
    transform_and_store(acc, p, lds, rowpix, rowok, &flag, wave, lane, t, split, tn, cc);
}

inline bool aligned16w(const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; }

}  // namespace

// Returns K_EUNSUPPORTED when the shape is not one this path takes (the caller then uses the direct
// kernels).  Taken: 3x3, stride 1, padding 1, NHWC in and out, Cin a multiple of 16, Cout a multiple of 32,
// no beta term.
int launch_conv3x3_winograd(const ConvArgs& a, const Workspace& ws, hipStream_t s) {
    if (a.KH != 3 || a.KW != 3 || a.sh != 1 || a.sw != 1 || a.ph != 1 || a.pw != 1) return K_EUNSUPPORTED;
    if (!a.x_nhwc || !a.y_nhwc || a.groups != 1 || a.ep.beta != 0.f) return K_EUNSUPPORTED;
    if (a.Cin % kKC != 0 || a.Cout % 32 != 0) return K_EUNSUPPORTED;
    const long xp = a.x_pitch ? a.x_pitch : a.Cin, yp = a.y_pitch ? a.y_pitch : a.Cout;
    if (xp % 4 != 0 || !aligned16w(a.x) || !aligned16w(a.w)) return K_EUNSUPPORTED;
    // Small launches are bound by the length of one workgroup's chain (fetch, transform, multiply, exchange, sum),
    // which is longer here than in the direct kernels' nine-wavefront tiles: batch-1 ResNet layers ran 11-16 us
    // this way against 8-11 us.  TORPOR_WINO_MIN_GFLOP moves the bound (direct-form FLOP of the layer).
    const char* min_env = getenv("TORPOR_WINO_MIN_GFLOP");  // read per call: tests send small shapes down this path
    const double min_gflop = min_env ? atof(min_env) : 0.8;
    if (2.0 * a.N * a.H * a.W * (double)a.Cout * a.Cin * 9.0 < min_gflop * 1e9) return K_EUNSUPPORTED;
    const long pixels = (long)a.N * a.H * a.W;
    // byte offsets are 32-bit in the kernel and 2^31 marks "beyond the tensor"
    if (pixels * xp >= (1L << 29) || pixels * yp >= (1L << 31) || (long)a.Cout * a.Cin * 36 >= (1L << 31)) return K_EUNSUPPORTED;

    WinoDev p;
    p.x = a.x;
    p.w = a.w;
    p.y = a.y;
    p.H = a.H;
    p.W = a.W;
    p.Cin = a.Cin;
    p.Cout = a.Cout;
    p.xp = xp;
    p.yp = yp;
    p.xbytes = (unsigned)(((pixels - 1) * xp + a.Cin) * 4);
    p.wbytes = (unsigned)((long)a.Cout * a.Cin * 36);
    p.tiles_h = (a.H + 1) / 2;
    p.tiles_w = (a.W + 1) / 2;
    p.ntiles = (long)a.N * p.tiles_h * p.tiles_w;
    const long mt = (p.ntiles + 31) / 32;
    if (mt * (a.Cout / 32) >= (1L << 31) / 8) return K_EUNSUPPORTED;
    p.mt = (int)mt;
    const int kblocks = a.Cin / kKC;

    p.nt = a.Cout / 32;
    const long base = mt * p.nt;

    // Split over input channels when the blocks alone leave CUs idle.  The kernel is bound by what a SIMD
    // issues (transforms and MFMAs add up), so two workgroups on a CU take twice as long as one: the candidates
    // are weighed by the K-blocks the fullest CU works through, with a slight preference for a CU that holds two
    // workgroups (they fill each other's barrier waits), two K-blocks' worth for reading a split back and
    // summing it, and a little per slot.  Measured on MI355X (us): 8x14x14x256>256 1/2/4/8 slots 27.8 / 18.8 /
    // 17.9 / 22.6; 8x28x28x128>128 16.5 / 18.2 / 22.6 / 29.6; 8x7x7x512>512 52.5 / 31.1 / 19.9 / 20.4.
    // (A workgroup of 64 output channels -- one patch transform for two filter transforms, 25 loads per thread
    // and K-block instead of 2 x 16 -- was built and measured: 12 % less time per K-block and unit of work, but
    // half as many workgroups for grids that fill the chip barely once; 22.4 / 21.0 / 18.2 / 26.7 us on the four
    // ResNet-152 batch 8 layers against 17.8 / 16.7 / 16.1 / 19.6.  It is not kept.)
    const char* forced_env = getenv("TORPOR_WINO_SPLITS");  // read per call: tests compare split depths in one process
    const int forced = forced_env ? atoi(forced_env) : 0;
    const size_t per_split = (size_t)base * 4096 * sizeof(float);
    int splits = 1;
    if (ws.ptr && ws.tickets && base <= kSplitTickets) {
        double best = 1e30;
        for (int sp = 1; sp <= 8 && sp <= kblocks; ++sp) {
            if (sp > 1 && (size_t)sp * per_split > ws.bytes) break;
            const int kb = (kblocks + sp - 1) / sp;
            const int eff = (kblocks + kb - 1) / kb;
            if (eff != sp) continue;
            const long deep = (base * sp + num_cu() - 1) / num_cu();
            const double cost = (double)deep * kb * (deep == 1 ? 1.1 : 1.0) + (sp > 1 ? 2.0 : 0.0) + 0.05 * sp;
            if (cost < best) {
                best = cost;
                splits = sp;
            }
        }
        if (forced > 0 && forced <= 8 && forced <= kblocks && (size_t)forced * per_split <= ws.bytes) splits = forced;
    }
    int kb = (kblocks + splits - 1) / splits;
    p.cper = kb * kKC;
    p.splits = (a.Cin + p.cper - 1) / p.cper;
    p.ws = ws.ptr;
    p.tickets = p.splits > 1 ? split_tickets(ws, base, p.splits) : nullptr;
    if (p.splits > 1 && !p.tickets) {  // in-launch summation switched off: one slice
        p.splits = 1;
        p.cper = a.Cin;
    }
    EpilogueArgs ea = a.ep;
    if (ea.residual && ea.ldr == 0) ea.ldr = a.Cout;  // the residual is dense unless its pitch is given
    p.ep = make_epilogue(ea, yp);
    hipLaunchKernelGGL(conv_wino_kernel, dim3((unsigned)base, 1, (unsigned)p.splits), dim3(256), 0, s, p);
    set_last_kernel("conv3x3_wino_f2x2");
    return (int)hipGetLastError();
}

}  // namespace tpk
