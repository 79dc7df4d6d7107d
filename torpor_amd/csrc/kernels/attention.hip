// Fused scaled-dot-product attention, fp32 MFMA, gfx950.
//
//   out[b, q, a, :] = softmax_k( scale * Q[b,q,a,:] . K[b,k,a,:] + mask[b,k] ) . V[b,k,a,:]
//
// stands in for the three calls the reference forwards for one BERT attention layer
// (cublasSgemmStridedBatched, the libtorch softmax launch, cublasSgemmStridedBatched again:
// include/server/cuda_server.hpp:524-550,1226-1310) without ever writing the [S, S] score
// matrix to memory.
//
// One workgroup = one head and 32 query rows; its four wavefronts take every fourth block of
// 32 keys and merge their partial results at the end, so the main loop has no workgroup
// barrier.  Per key block a wavefront computes the TRANSPOSED scores S^T = K . Q^T with
// v_mfma_f32_32x32x2_f32.  In the MFMA result layout a lane then owns one query (its column)
// and sixteen keys, so the running row maximum / sum of the online softmax are per-lane
// scalars, and the sixteen probabilities a lane holds are exactly the B-operand values the
// next product O^T += V^T . P^T wants from it (result row 8j+4h+i of lane half h is k index
// 8j+4h+i of the k-permuted operand layout described in mfma_tile.hpp).  The probabilities
// therefore never leave registers.  K and V blocks pass through a wavefront-private LDS buffer
// (coalesced global reads in, operand fragments out).
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "kernels.hpp"
#include "mfma_tile.hpp"

namespace tpk {

namespace {

constexpr int DH = 64;            // head width this kernel is built for
constexpr int LDB = DH + 4;       // LDS row pitch of a K / V block (conflict-free 128-bit reads)
constexpr int BLK = 32 * LDB;     // floats per wavefront buffer
constexpr int OLD = 65;           // pitch of the merge area: one row per accumulator register
constexpr int MERGE = 4 * 32 * OLD + 256;
constexpr int LDS_FLOATS = (4 * BLK > MERGE) ? 4 * BLK : MERGE;

struct AttnDev {
    const float* q;
    const float* k;
    const float* v;
    const float* mask;  // [B][S] additive, or nullptr
    float* out;
    int B, A, S;
    long ldq, ldk, ldv, ldo;
    float scale;
    int qblocks;  // ceil(S / 32)
    int xcd_remap;
};

__global__ __launch_bounds__(256, 3) void attention_kernel(const AttnDev p) {
    __shared__ __attribute__((aligned(16))) float lds[LDS_FLOATS];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int r = lane & 31, h = lane >> 5;

    // workgroup -> (head, query block); with a head count divisible by 8 every XCD (workgroup id
    // mod 8) keeps whole heads, so a head's K and V are fetched into one L2 only
    int head, qb;
    if (p.xcd_remap) {
        const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
        const int hl = local / p.qblocks;
        qb = local - hl * p.qblocks;
        head = xcd * ((p.B * p.A) >> 3) + hl;
    } else {
        head = blockIdx.x / p.qblocks;
        qb = blockIdx.x - head * p.qblocks;
    }
    const int b = head / p.A, a = head - b * p.A;
    const int q0 = qb * 32;
    const int nkb = p.qblocks;  // key blocks of 32

    const float* Qb = p.q + (long)b * p.S * p.ldq + a * DH;
    const float* Kb = p.k + (long)b * p.S * p.ldk + a * DH;
    const float* Vb = p.v + (long)b * p.S * p.ldv + a * DH;

    // Q^T operand fragments for this lane's query, pre-multiplied by the softmax scale
    f32x4 qf[8];
    {
        const int qrow = (q0 + r < p.S) ? q0 + r : p.S - 1;
        const float* qp = Qb + (long)qrow * p.ldq + 4 * h;
#pragma unroll
        for (int g = 0; g < 8; ++g) qf[g] = *reinterpret_cast<const f32x4*>(qp + 8 * g) * p.scale;
    }

    float* buf = lds + w * BLK;
    const int srow = lane >> 4, scol = (lane & 15) * 4;  // staging: 4 rows x 16 float4 per instruction
    f32x4 st[8];
    auto load_block = [&](const float* base, long ld, int kb) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int key = kb * 32 + srow + 4 * i;
            if (key > p.S - 1) key = p.S - 1;  // padded keys read a valid row; their scores are masked
            st[i] = *reinterpret_cast<const f32x4*>(base + (long)key * ld + scol);
        }
    };
    auto store_block = [&]() {
#pragma unroll
        for (int i = 0; i < 8; ++i) *reinterpret_cast<f32x4*>(buf + (srow + 4 * i) * LDB + scol) = st[i];
    };

    float m = -INFINITY, l = 0.f;
    f32x16 o[2];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        o[0][v] = 0.f;
        o[1][v] = 0.f;
    }

    int kb = w;
    if (kb < nkb) load_block(Kb, p.ldk, kb);
    for (; kb < nkb; kb += 4) {
        store_block();  // K block
        wave_lds_sync();
        load_block(Vb, p.ldv, kb);  // in flight during the score product

        f32x16 s;
#pragma unroll
        for (int v = 0; v < 16; ++v) s[v] = 0.f;
        const float* kp = buf + r * LDB + 4 * h;
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            const f32x4 kf = *reinterpret_cast<const f32x4*>(kp + 8 * g);
#pragma unroll
            for (int t = 0; t < 4; ++t) s = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[t], qf[g][t], s, 0, 0, 0);
        }

        // online softmax for this lane's query over the 16 keys it holds (+ the other lane half)
        float mb = -INFINITY;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int key0 = kb * 32 + 8 * j + 4 * h;
            f32x4 mk = {0.f, 0.f, 0.f, 0.f};
            // S % 4 == 0 whenever a mask is given (checked on the host), so a group of four keys
            // is inside the row or entirely past its end
            if (p.mask && key0 < p.S) mk = *reinterpret_cast<const f32x4*>(p.mask + (long)b * p.S + key0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float x = s[4 * j + i] + mk[i];
                if (key0 + i >= p.S) x = -INFINITY;
                s[4 * j + i] = x;
                mb = fmaxf(mb, x);
            }
        }
        mb = fmaxf(mb, __shfl_xor(mb, 32));
        const float m_new = fmaxf(m, mb);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = __expf(m - m_use);
        float ls = 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const float e = __expf(s[v] - m_use);
            s[v] = e;
            ls += e;
        }
        l = l * alpha + ls;
        m = m_new;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            o[0][v] *= alpha;
            o[1][v] *= alpha;
        }

        store_block();  // V block replaces K (every K fragment has been consumed by the MFMAs above)
        wave_lds_sync();
        if (kb + 4 < nkb) load_block(Kb, p.ldk, kb + 4);  // in flight during the value product

        // O^T[d][query] += V^T[d][key] . P^T[key][query]
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            const float* vp = buf + (4 * h) * LDB + 32 * blk + r;
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    o[blk] = __builtin_amdgcn_mfma_f32_32x32x2f32(vp[(8 * g + t) * LDB], s[4 * g + t], o[blk], 0, 0, 0);
        }
        wave_lds_sync();
    }
    l += __shfl_xor(l, 32);  // the two lane halves summed disjoint keys

    // merge the four wavefronts' partial results
    __syncthreads();  // every wavefront is done with its K / V buffer
    float* mo = lds;                 // [wave][register 0..31][OLD]: O^T partials, lane-major
    float* mm = lds + 4 * 32 * OLD;  // [wave][query]
    float* ml = mm + 128;
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int v = 0; v < 16; ++v) mo[(w * 32 + 16 * blk + v) * OLD + lane] = o[blk][v];
    if (h == 0) {
        mm[w * 32 + r] = m;
        ml[w * 32 + r] = l;
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        const int c = tid & 15;                  // float4 column of the 64-wide head
        const int q = (tid >> 4) + 16 * pass;    // query row in the block
        float mw[4], f[4];
        float mt = -INFINITY;
#pragma unroll
        for (int z = 0; z < 4; ++z) {
            mw[z] = mm[z * 32 + q];
            mt = fmaxf(mt, mw[z]);
        }
        float L = 0.f;
#pragma unroll
        for (int z = 0; z < 4; ++z) {
            f[z] = (mw[z] == -INFINITY) ? 0.f : __expf(mw[z] - mt);
            L += ml[z * 32 + q] * f[z];
        }
        const float inv = L > 0.f ? 1.0f / L : 0.f;  // a row with every key masked by -inf gives 0
        const int blk = c >> 3, j = (c & 7) >> 1, hh = c & 1;
        f32x4 res;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int reg = 16 * blk + 4 * j + i;
            float acc = 0.f;
#pragma unroll
            for (int z = 0; z < 4; ++z) acc += f[z] * mo[(z * 32 + reg) * OLD + q + 32 * hh];
            res[i] = acc * inv;
        }
        if (q0 + q < p.S)
            *reinterpret_cast<f32x4*>(p.out + ((long)b * p.S + q0 + q) * p.ldo + a * DH + 4 * c) = res;
    }
}

}  // namespace

int launch_attention(const float* q, const float* k, const float* v, const float* mask, float* out, int B, int A, int S,
                     int dh, long ldq, long ldk, long ldv, long ldo, float scale, hipStream_t s) {
    if (!q || !k || !v || !out || B < 1 || A < 1 || S < 1) return K_EINVAL;
    if (dh != DH) return K_EUNSUPPORTED;
    const auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    if ((ldq | ldk | ldv | ldo) & 3) return K_EUNSUPPORTED;
    if (!al16(q) || !al16(k) || !al16(v) || !al16(out) || (mask && !al16(mask))) return K_EUNSUPPORTED;
    if (mask && (S & 3)) return K_EUNSUPPORTED;  // 128-bit mask reads assume 16 B aligned rows
    const long width = (long)A * DH;
    if (ldq < width || ldk < width || ldv < width || ldo < width) return K_EINVAL;
    AttnDev p;
    p.q = q;
    p.k = k;
    p.v = v;
    p.mask = mask;
    p.out = out;
    p.B = B;
    p.A = A;
    p.S = S;
    p.ldq = ldq;
    p.ldk = ldk;
    p.ldv = ldv;
    p.ldo = ldo;
    p.scale = scale;
    p.qblocks = (S + 31) / 32;
    const long heads = (long)B * A;
    p.xcd_remap = (heads % 8 == 0) ? 1 : 0;
    const long grid = heads * p.qblocks;
    if (grid > 0x7fffffffL) return K_EINVAL;
    hipLaunchKernelGGL(attention_kernel, dim3((unsigned)grid), dim3(256), 0, s, p);
    set_last_kernel("attention_32q_dh64");
    return (int)hipGetLastError();
}

}  // namespace tpk
