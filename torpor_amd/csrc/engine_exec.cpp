#include "engine_internal.hpp"

namespace tp {

// ------------------------------------------------------------------ compute ops
static tpk::EpilogueArgs ep_from(const Op& op, void* const* q, int pbase, int fbase, int ibase) {
    tpk::EpilogueArgs e;
    e.alpha = op.f[fbase + 0];
    e.beta = op.f[fbase + 1];
    e.bn_eps = op.f[fbase + 2];
    e.bias = static_cast<const float*>(q[pbase + 0]);
    e.bn_scale = static_cast<const float*>(q[pbase + 1]);
    e.bn_bias = static_cast<const float*>(q[pbase + 2]);
    e.bn_mean = static_cast<const float*>(q[pbase + 3]);
    e.bn_var = static_cast<const float*>(q[pbase + 4]);
    e.residual = static_cast<const float*>(q[pbase + 5]);
    e.ldr = op.i[ibase + 0];
    e.act = (int)op.i[ibase + 1];
    return e;
}

// Layout of Op for the compute kinds (filled by the C-ABI layer):
//  GEMM  p: x y c bias bns bnb bnm bnv res   i: m n k xs_r xs_k ys_c ys_k ldc nb0 nb1 xb0 xb1 yb0 yb1 cb0 cb1 ldr act
//        f: alpha beta eps
//  CONV  p: x w y bias bns bnb bnm bnv res   i: n h w cin cout kh kw sh sw ph pw xl yl ldr act   f: alpha beta eps
//  BN    p: x y g b mean var                 i: rows C hw layout relu   f: eps
//  LAUNCH p/i/f per op id (see torpor_amd.h)
int Engine::exec_compute_impl(Model& m, const Op& op, bool launch) {
    void* q[12] = {nullptr};
    // The scratch allocation: 256 bytes that stay zero for good (padding source of the 3x3
    // convolution), the ticket counters of split K ranges (zero between launches), then the partial
    // sums.  No device workspace in host-only mode (nothing is launched there).
    constexpr size_t kHead = 256 + tpk::kSplitTickets * sizeof(unsigned);
    const tpk::Workspace ws = workspace_ ? tpk::Workspace{workspace_ + kHead / 4, (size_t)cfg_.workspace_bytes - kHead, workspace_,
                                                           reinterpret_cast<unsigned*>(workspace_ + 64)}
                                        : tpk::Workspace{};
    // Every operand is translated together with the byte span the kernel will touch, so an op
    // whose shapes do not fit its buffers is refused on the host instead of faulting the GPU.
    // Spans are computed in 128-bit integers from arguments that have been range-checked first
    // (anything a launcher narrows to int: at most INT32_MAX; counts, strides and pitches: at most
    // the size of an address region), so that no product can wrap into a span that passes.
    using i128 = __int128;
    constexpr int64_t kIntMax = 0x7fffffff;
    constexpr int64_t kLongMax = (int64_t)kVaOffMask;
    auto R = [&](int idx, bool optional, i128 elems, int elem_size = 4) -> int {
        if (elems < 1) elems = 1;
        if (elems > (i128)kLongMax) return TP_EFAULT;  // no block is that large
        return resolve(m, op.p[idx], (uint64_t)elems * (uint64_t)elem_size, optional, &q[idx]);
    };
    i128 I[20];
    for (int k = 0; k < 20; ++k) I[k] = k < op.ni ? (i128)op.i[k] : (i128)0;
    // arguments whose bit is set in long_mask may be as large as an address region, the others fit an int
    auto ranges_ok = [&](uint32_t long_mask) {
        for (int k = 0; k < op.ni && k < 20; ++k) {
            if (op.i[k] < 0) return false;
            if (op.i[k] > (((long_mask >> k) & 1u) ? kLongMax : kIntMax)) return false;
        }
        return true;
    };
    static const uint32_t kLaunchLong[] = {
        /* 0 */ 0,
        /* RELU */ 1u << 0, /* ADD */ 1u << 0, /* BIAS_ACT */ 1u << 0, /* GELU */ 1u << 0,
        /* MAXPOOL */ 1u << 8, /* AVGPOOL */ 0, /* LAYERNORM */ 1u << 0, /* SOFTMAX */ (1u << 0) | (1u << 2),
        /* EMBEDDING */ (1u << 0) | (1u << 3), /* NCHW_TO_NHWC */ 0, /* NHWC_TO_NCHW */ 0, /* SUM */ 1u << 0,
        /* FILL */ 1u << 0, /* ATTENTION */ 0xF0u, /* AVGPOOL2D */ 1u << 7, /* COPY2D */ (1u << 0) | (1u << 2) | (1u << 3),
        /* SCALE_CHANNELS */ 1u << 1, /* BN_CONV1X1 */ (1u << 0) | (1u << 3) | (1u << 4)};
    {
        uint32_t long_mask = 0;
        switch (op.kind) {
            case OPK_GEMM: long_mask = 0xF8u | 0xFC00u | (1u << 16); break;  // strides, ldc, batch strides, ldr
            case OPK_CONV: long_mask = (1u << 13) | (1u << 15) | (1u << 16); break;  // ldr, x / y pitch
            case OPK_BN: long_mask = (1u << 0) | (1u << 2) | (1u << 5); break;  // rows, hw, x pitch
            case OPK_LAUNCH:
                if (op.op_id > 0 && op.op_id < (int)(sizeof(kLaunchLong) / sizeof(kLaunchLong[0])))
                    long_mask = kLaunchLong[op.op_id];
                break;
            default: break;
        }
        if (!ranges_ok(long_mask)) return TP_EINVAL;
    }
    int r = 0;
    switch (op.kind) {
        case OPK_GEMM: {
            const i128 M = I[0], N = I[1], K = I[2];
            const i128 nb0 = I[8], nb1 = I[9];
            if (M < 1 || N < 1 || nb0 < 1 || nb1 < 1) return TP_EINVAL;
            if (nb0 * nb1 > 65535) return TP_EUNSUPPORTED;  // batches are the grid's z dimension
            const i128 kx = K > 0 ? K - 1 : 0;
            const i128 xs = (M - 1) * I[3] + kx * I[4] + (nb0 - 1) * I[10] + (nb1 - 1) * I[11] + 1;
            const i128 ys = (N - 1) * I[5] + kx * I[6] + (nb0 - 1) * I[12] + (nb1 - 1) * I[13] + 1;
            const i128 cs = (M - 1) * I[7] + N + (nb0 - 1) * I[14] + (nb1 - 1) * I[15];
            if (I[7] < N) return TP_EINVAL;
            const i128 ldr = I[16] ? I[16] : I[7];
            if (op.p[8] && (nb0 * nb1 != 1 || ldr < N)) return TP_EUNSUPPORTED;
            if ((r = R(0, false, xs)) || (r = R(1, false, ys)) || (r = R(2, false, cs))) return r;
            for (int k = 3; k < 8 && !r; ++k) r = R(k, true, N);
            if (!r) r = R(8, true, (M - 1) * ldr + N);
            if (r) return r;
            if ((q[4] != nullptr) != (q[5] != nullptr) || (q[4] != nullptr) != (q[6] != nullptr) ||
                (q[4] != nullptr) != (q[7] != nullptr))
                return TP_EINVAL;
            tpk::GemmArgs g;
            g.X = static_cast<const float*>(q[0]);
            g.Y = static_cast<const float*>(q[1]);
            g.C = static_cast<float*>(q[2]);
            g.M = (long)M;
            g.N = (long)N;
            g.K = (long)K;
            g.xs_r = (long)I[3];
            g.xs_k = (long)I[4];
            g.ys_c = (long)I[5];
            g.ys_k = (long)I[6];
            g.ldc = (long)I[7];
            g.nb0 = (int)nb0;
            g.nb1 = (int)nb1;
            g.xb0 = (long)I[10];
            g.xb1 = (long)I[11];
            g.yb0 = (long)I[12];
            g.yb1 = (long)I[13];
            g.cb0 = (long)I[14];
            g.cb1 = (long)I[15];
            g.ep = ep_from(op, q, 3, 0, 16);
            g.ep.ldr = (long)ldr;
            if (!launch) return 0;
            return tpk::launch_gemm(g, ws, compute_);
        }
        case OPK_CONV: {
            const i128 N = I[0], H = I[1], W = I[2], Cin = I[3], Cout = I[4], KH = I[5], KW = I[6];
            const i128 sh = I[7], sw = I[8], ph = I[9], pw = I[10];
            if (N < 1 || H < 1 || W < 1 || Cin < 1 || Cout < 1 || KH < 1 || KW < 1 || sh < 1 || sw < 1)
                return TP_EINVAL;
            const i128 Ho = (H + 2 * ph - KH) / sh + 1, Wo = (W + 2 * pw - KW) / sw + 1;
            if (H + 2 * ph < KH || W + 2 * pw < KW || Ho < 1 || Wo < 1) return TP_EINVAL;
            const i128 xpitch = op.ni > 15 ? I[15] : 0, ypitch = op.ni > 16 ? I[16] : 0;
            const i128 groups = (op.ni > 17 && I[17] > 0) ? I[17] : 1;
            const bool x_nhwc = I[11] != 0, y_nhwc = I[12] != 0;
            if ((xpitch && (!x_nhwc || xpitch < Cin)) || (ypitch && (!y_nhwc || ypitch < Cout))) return TP_EINVAL;
            if (groups != 1 && (Cin % groups != 0 || Cout % groups != 0)) return TP_EINVAL;
            // grouped but not depthwise: one launch per group over channel slices, NHWC only
            if (groups != 1 && (groups != Cin || Cin != Cout) && (!x_nhwc || !y_nhwc)) return TP_EUNSUPPORTED;
            const i128 ys = ypitch ? (N * Ho * Wo - 1) * ypitch + Cout : N * Ho * Wo * Cout;
            const i128 xs = xpitch ? (N * H * W - 1) * xpitch + Cin : N * H * W * Cin;
            if ((r = R(0, false, xs)) || (r = R(1, false, Cout * (Cin / groups) * KH * KW)) || (r = R(2, false, ys)))
                return r;
            for (int k = 3; k < 8 && !r; ++k) r = R(k, true, Cout);
            if (!r) r = R(8, true, N * Ho * Wo * Cout);  // residual: dense unless ldr says otherwise
            if (r) return r;
            if ((q[4] != nullptr) != (q[5] != nullptr) || (q[4] != nullptr) != (q[6] != nullptr) ||
                (q[4] != nullptr) != (q[7] != nullptr))
                return TP_EINVAL;
            tpk::ConvArgs c;
            c.x = static_cast<const float*>(q[0]);
            c.w = static_cast<const float*>(q[1]);
            c.y = static_cast<float*>(q[2]);
            c.N = (int)N;
            c.H = (int)H;
            c.W = (int)W;
            c.Cin = (int)Cin;
            c.Cout = (int)Cout;
            c.KH = (int)KH;
            c.KW = (int)KW;
            c.sh = (int)sh;
            c.sw = (int)sw;
            c.ph = (int)ph;
            c.pw = (int)pw;
            c.x_nhwc = (int)I[11];
            c.y_nhwc = (int)I[12];
            c.x_pitch = (long)xpitch;
            c.y_pitch = (long)ypitch;
            c.groups = (int)groups;
            c.ep = ep_from(op, q, 3, 0, 13);
            c.ep.ldr = 0;  // residual shares the layout and pitch of y
            if (!launch) return 0;
            return tpk::launch_conv2d(c, ws, compute_);
        }
        case OPK_BN: {
            const i128 rows = I[0], C = I[1];
            const i128 xpitch = op.ni > 5 ? I[5] : 0;
            if (C < 1 || (xpitch && xpitch < C)) return TP_EINVAL;
            const i128 xspan = (xpitch && rows > 0) ? (rows - 1) * xpitch + C : rows * C;
            if ((r = R(0, false, xspan)) || (r = R(1, false, rows * C))) return r;
            for (int k = 2; k < 6 && !r; ++k) r = R(k, false, C);
            if (r) return r;
            if (!I[3] && I[2] < 1) return TP_EINVAL;
            if (!launch) return 0;
            return tpk::launch_bn_inference(static_cast<const float*>(q[0]), static_cast<float*>(q[1]),
                                            static_cast<const float*>(q[2]), static_cast<const float*>(q[3]),
                                            static_cast<const float*>(q[4]), static_cast<const float*>(q[5]), op.f[0],
                                            rows, (int)C, (int)I[3], I[2], (int)I[4], xpitch, compute_);
        }
        case OPK_LAUNCH:
            break;
        default:
            return TP_EINVAL;
    }
    // generic launch by op id
    auto need = [&](int np, int ni, int nf) { return op.np >= np && op.ni >= ni && op.nf >= nf; };
    auto F = [&](int k) { return static_cast<const float*>(q[k]); };
    auto Fm = [&](int k) { return static_cast<float*>(q[k]); };
    switch (op.op_id) {
        case TP_OP_RELU:
        case TP_OP_GELU:
            if (!need(2, 1, 0)) return TP_EINVAL;
            if ((r = R(0, false, I[0])) || (r = R(1, false, I[0]))) return r;
            if (!launch) return 0;
            return op.op_id == TP_OP_RELU ? tpk::launch_relu(F(0), Fm(1), I[0], compute_)
                                          : tpk::launch_gelu(F(0), Fm(1), I[0], compute_);
        case TP_OP_ADD:
            if (!need(3, 2, 0)) return TP_EINVAL;
            if ((r = R(0, false, I[0])) || (r = R(1, false, I[0])) || (r = R(2, false, I[0]))) return r;
            if (!launch) return 0;
            return tpk::launch_add(F(0), F(1), Fm(2), I[0], (int)I[1], compute_);
        case TP_OP_BIAS_ACT:
            if (!need(3, 3, 0) || I[1] < 1) return TP_EINVAL;
            if ((r = R(0, false, I[0] * I[1])) || (r = R(1, false, I[1])) || (r = R(2, false, I[0] * I[1]))) return r;
            if (!launch) return 0;
            return tpk::launch_bias_act(F(0), F(1), Fm(2), I[0], (int)I[1], (int)I[2], compute_);
        case TP_OP_MAXPOOL: {
            if (!need(2, 8, 0)) return TP_EINVAL;
            const i128 N = I[0], H = I[1], W = I[2], C = I[3], k = I[4], st = I[5], pad = I[6];
            if (N < 1 || H < 1 || W < 1 || C < 1 || k < 1 || st < 1 || H + 2 * pad < k || W + 2 * pad < k)
                return TP_EINVAL;
            const i128 Ho = (H + 2 * pad - k) / st + 1, Wo = (W + 2 * pad - k) / st + 1;
            const i128 yp = (op.ni > 8 && I[8]) ? I[8] : C;   // NHWC: elements between output pixels
            if (yp < C || (yp != C && !I[7])) return TP_EINVAL;
            if ((r = R(0, false, N * H * W * C)) || (r = R(1, false, (N * Ho * Wo - 1) * yp + C))) return r;
            if (!launch) return 0;
            return tpk::launch_maxpool2d(F(0), Fm(1), (int)N, (int)H, (int)W, (int)C, (int)k, (int)st, (int)pad,
                                         (int)I[7], yp, compute_);
        }
        case TP_OP_AVGPOOL:
            if (!need(2, 4, 0)) return TP_EINVAL;
            if ((r = R(0, false, I[0] * I[1] * I[2])) || (r = R(1, false, I[0] * I[2]))) return r;
            if (!launch) return 0;
            return tpk::launch_global_avgpool(F(0), Fm(1), (int)I[0], (int)I[1], (int)I[2], (int)I[3], ws, compute_);
        case TP_OP_LAYERNORM:
            if (!need(5, 2, 1)) return TP_EINVAL;
            if ((r = R(0, false, I[0] * I[1])) || (r = R(1, true, I[0] * I[1])) || (r = R(2, false, I[1])) ||
                (r = R(3, false, I[1])) || (r = R(4, false, I[0] * I[1])))
                return r;
            if (!launch) return 0;
            return tpk::launch_layernorm(F(0), F(1), F(2), F(3), Fm(4), I[0], (int)I[1], op.f[0], compute_);
        case TP_OP_SOFTMAX: {
            if (!need(3, 3, 1)) return TP_EINVAL;
            const i128 rpm = I[2] > 0 ? I[2] : 1;
            if ((r = R(0, false, I[0] * I[1])) || (r = R(1, true, ((I[0] + rpm - 1) / rpm) * I[1])) ||
                (r = R(2, false, I[0] * I[1])))
                return r;
            if (!launch) return 0;
            return tpk::launch_softmax(F(0), F(1), Fm(2), I[0], (int)I[1], op.f[0], rpm, compute_);
        }
        case TP_OP_EMBEDDING:
            if (!need(6, 5, 0)) return TP_EINVAL;
            if (I[1] < 1 || I[2] < 1 || I[3] < 1 || I[4] < 1) return TP_EINVAL;
            if ((r = R(0, false, I[0], 8)) || (r = R(1, true, I[0], 8)) ||
                (r = resolve(m, op.p[2], (uint64_t)(I[3] * I[2]) * 4, false, &q[2], /*gather=*/true)) ||
                (r = R(3, true, I[1] * I[2])) || (r = R(4, true, I[4] * I[2])) || (r = R(5, false, I[0] * I[2])))
                return r;
            if (!launch) return 0;
            return tpk::launch_embedding(static_cast<const int64_t*>(q[0]), static_cast<const int64_t*>(q[1]), F(2),
                                         F(3), F(4), Fm(5), I[0], (int)I[1], (int)I[2], I[3], (int)I[4], compute_);
        case TP_OP_NCHW_TO_NHWC:
        case TP_OP_NHWC_TO_NCHW: {
            if (!need(2, 4, 0)) return TP_EINVAL;
            const i128 n = I[0] * I[1] * I[2] * I[3];
            if ((r = R(0, false, n)) || (r = R(1, false, n))) return r;
            if (!launch) return 0;
            return op.op_id == TP_OP_NCHW_TO_NHWC
                       ? tpk::launch_nchw_to_nhwc(F(0), Fm(1), (int)I[0], (int)I[1], (int)I[2], (int)I[3], compute_)
                       : tpk::launch_nhwc_to_nchw(F(0), Fm(1), (int)I[0], (int)I[1], (int)I[2], (int)I[3], compute_);
        }
        case TP_OP_SUM:
            if (!need(2, 1, 0)) return TP_EINVAL;
            if ((r = R(0, false, I[0])) || (r = R(1, false, 1))) return r;
            if (!launch) return 0;
            return tpk::launch_sum(F(0), Fm(1), I[0], compute_);
        case TP_OP_AVGPOOL2D: {
            if (!need(2, 8, 0)) return TP_EINVAL;
            const i128 N = I[0], H = I[1], W = I[2], C = I[3], k = I[4], st = I[5], pad = I[6];
            if (N < 1 || H < 1 || W < 1 || C < 1 || k < 1 || st < 1 || H + 2 * pad < k || W + 2 * pad < k)
                return TP_EINVAL;
            const i128 yp = I[7] ? I[7] : C;
            if (yp < C) return TP_EINVAL;
            const i128 Ho = (H + 2 * pad - k) / st + 1, Wo = (W + 2 * pad - k) / st + 1;
            if ((r = R(0, false, N * H * W * C)) || (r = R(1, false, (N * Ho * Wo - 1) * yp + C))) return r;
            if (!launch) return 0;
            return tpk::launch_avgpool2d(F(0), Fm(1), (int)N, (int)H, (int)W, (int)C, (int)k, (int)st, (int)pad, yp,
                                         compute_);
        }
        case TP_OP_COPY2D: {
            if (!need(2, 4, 0)) return TP_EINVAL;
            const i128 rows = I[0], width = I[1], sp = I[2], dp = I[3];
            if (rows < 1 || width < 1 || sp < width || dp < width) return TP_EINVAL;
            if ((r = R(0, false, (rows - 1) * sp + width)) || (r = R(1, false, (rows - 1) * dp + width))) return r;
            if (!launch) return 0;
            return tpk::launch_copy2d(F(0), Fm(1), rows, (int)width, sp, dp, compute_);
        }
        case TP_OP_SCALE_CHANNELS: {
            if (!need(3, 3, 0)) return TP_EINVAL;
            const i128 N = I[0], HW = I[1], C = I[2];
            if (N < 1 || HW < 1 || C < 1 || N > 0x7fffffff || C > 0x7fffffff) return TP_EINVAL;
            if ((r = R(0, false, N * HW * C)) || (r = R(1, false, N * C)) || (r = R(2, false, N * HW * C))) return r;
            if (!launch) return 0;
            return tpk::launch_scale_channels(F(0), F(1), Fm(2), (int)N, HW, (int)C, compute_);
        }
        case TP_OP_BN_CONV1X1: {
            if (!need(11, 7, 2)) return TP_EINVAL;
            const i128 rows = I[0], cin = I[1], cout = I[2];
            const i128 xp = I[3] ? I[3] : cin, yp = I[4] ? I[4] : cout;
            if (rows < 1 || cin < 1 || cout < 1 || xp < cin || yp < cout || I[6] > 16) return TP_EINVAL;
            if ((r = R(0, false, (rows - 1) * xp + cin)) || (r = R(5, false, cout * cin)) ||
                (r = R(6, false, (rows - 1) * yp + cout)) || (r = R(1, false, cin)))
                return r;
            for (int k = 2; k < 5 && !r; ++k) r = R(k, true, cin);
            for (int k = 7; k < 11 && !r; ++k) r = R(k, true, cout);
            if (!r && op.np > 11) r = R(11, true, (rows - 1) * yp + cout);  // residual, laid out like y
            if (r) return r;
            if ((q[7] != nullptr) != (q[8] != nullptr) || (q[7] != nullptr) != (q[9] != nullptr) ||
                (q[7] != nullptr) != (q[10] != nullptr))
                return TP_EINVAL;
            if ((q[2] != nullptr) != (q[3] != nullptr) || (q[2] != nullptr) != (q[4] != nullptr)) return TP_EINVAL;
            tpk::GemmArgs g;
            g.X = F(0);
            g.Y = F(5);
            g.C = Fm(6);
            g.M = (long)rows;
            g.N = (long)cout;
            g.K = (long)cin;
            g.xs_r = (long)xp;
            g.ys_c = (long)cin;
            g.ldc = (long)yp;
            g.pre_gamma = F(1);
            g.pre_beta = F(2);
            g.pre_mean = F(3);
            g.pre_var = F(4);
            g.pre_eps = op.f[0];
            g.pre_relu = I[5] != 0;
            g.ep.bn_scale = F(7);
            g.ep.bn_bias = F(8);
            g.ep.bn_mean = F(9);
            g.ep.bn_var = F(10);
            g.ep.bn_eps = op.f[1];
            g.ep.act = (int)I[6];
            g.ep.residual = op.np > 11 ? F(11) : nullptr;
            g.ep.ldr = (long)yp;
            if (!launch) return 0;
            return tpk::launch_gemm(g, ws, compute_);
        }
        case TP_OP_ATTENTION: {
            if (!need(5, 8, 1)) return TP_EINVAL;
            const i128 B = I[0], A = I[1], S = I[2], dh = I[3];
            if (B < 1 || A < 1 || S < 1 || dh < 1 || B * S > 0x7fffffff || A * dh > 0x7fffffff) return TP_EINVAL;
            for (int k = 4; k < 8; ++k)
                if (I[k] < A * dh) return TP_EINVAL;
            // span of a strided [B*S][A*dh] view: last row start + one row
            auto span = [&](int64_t ld) { return (B * S - 1) * ld + A * dh; };
            if ((r = R(0, false, span(I[4]))) || (r = R(1, false, span(I[5]))) || (r = R(2, false, span(I[6]))) ||
                (r = R(3, true, B * S)) || (r = R(4, false, span(I[7]))))
                return r;
            if (!launch) return 0;
            return tpk::launch_attention(F(0), F(1), F(2), F(3), Fm(4), (int)B, (int)A, (int)S, (int)dh, I[4], I[5],
                                         I[6], I[7], op.f[0], compute_);
        }
        case TP_OP_FILL:
            if (!need(1, 1, 1)) return TP_EINVAL;
            if ((r = R(0, false, I[0]))) return r;
            if (!launch) return 0;
            return tpk::launch_fill(Fm(0), op.f[0], I[0], compute_);
        default:
            return TP_EUNSUPPORTED;
    }
}

// Algorithmic work of one op: floating-point operations and bytes that have to move at least
// once (each operand read once, each result written once).
void op_work(const Op& op, double* flops, double* bytes, const char** name) {
    const int64_t* I = op.i;
    *flops = 0;
    *bytes = 0;
    *name = "op";
    switch (op.kind) {
        case OPK_GEMM: {
            const double M = (double)I[0], N = (double)I[1], K = (double)I[2], nb = (double)(I[8] * I[9]);
            *flops = 2.0 * M * N * K * nb;
            *bytes = 4.0 * (M * K + N * K + M * N) * nb;
            *name = "gemm";
            break;
        }
        case OPK_CONV: {
            const double Ho = (double)((I[1] + 2 * I[9] - I[5]) / I[7] + 1), Wo = (double)((I[2] + 2 * I[10] - I[6]) / I[8] + 1);
            const double groups = (op.ni > 17 && I[17] > 0) ? (double)I[17] : 1.0;
            const double M = (double)I[0] * Ho * Wo, kk = (double)(I[3] * I[5] * I[6]) / groups;
            *flops = 2.0 * M * (double)I[4] * kk;
            *bytes = 4.0 * ((double)(I[0] * I[1] * I[2] * I[3]) + (double)I[4] * kk + M * (double)I[4] * (op.p[8] ? 2.0 : 1.0));
            *name = "conv";
            break;
        }
        case OPK_BN:
            *bytes = 8.0 * (double)(I[0] * I[1]);
            *name = "bn_inference";
            break;
        case OPK_LAUNCH:
            switch (op.op_id) {
                case TP_OP_RELU: *bytes = 8.0 * (double)I[0]; *name = "relu"; break;
                case TP_OP_GELU: *bytes = 8.0 * (double)I[0]; *name = "gelu"; break;
                case TP_OP_ADD: *bytes = 12.0 * (double)I[0]; *name = "add"; break;
                case TP_OP_BIAS_ACT: *bytes = 8.0 * (double)(I[0] * I[1]); *name = "bias_act"; break;
                case TP_OP_MAXPOOL: {
                    const double Ho = (double)((I[1] + 2 * I[6] - I[4]) / I[5] + 1), Wo = (double)((I[2] + 2 * I[6] - I[4]) / I[5] + 1);
                    *bytes = 4.0 * ((double)(I[0] * I[1] * I[2] * I[3]) + (double)(I[0] * I[3]) * Ho * Wo);
                    *name = "maxpool";
                    break;
                }
                case TP_OP_AVGPOOL: *bytes = 4.0 * (double)(I[0] * I[1] * I[2] + I[0] * I[2]); *name = "avgpool"; break;
                case TP_OP_LAYERNORM: *bytes = 4.0 * (double)(I[0] * I[1]) * (op.p[1] ? 3.0 : 2.0); *name = "layernorm"; break;
                case TP_OP_SOFTMAX: *bytes = 8.0 * (double)(I[0] * I[1]); *name = "softmax"; break;
                case TP_OP_EMBEDDING: *bytes = 8.0 * (double)(I[0] * I[2]); *name = "embedding"; break;
                case TP_OP_NCHW_TO_NHWC:
                case TP_OP_NHWC_TO_NCHW: *bytes = 8.0 * (double)(I[0] * I[1] * I[2] * I[3]); *name = "layout"; break;
                case TP_OP_SUM: *bytes = 4.0 * (double)I[0]; *name = "sum"; break;
                case TP_OP_FILL: *bytes = 4.0 * (double)I[0]; *name = "fill"; break;
                case TP_OP_AVGPOOL2D: *bytes = 4.0 * (double)(I[0] * I[1] * I[2] * I[3]) * 1.25; *name = "avgpool2d"; break;
                case TP_OP_COPY2D: *bytes = 8.0 * (double)(I[0] * I[1]); *name = "copy2d"; break;
                case TP_OP_SCALE_CHANNELS: *bytes = 8.0 * (double)(I[0] * I[1] * I[2]); *name = "scale_channels"; break;
                case TP_OP_BN_CONV1X1:
                    *flops = 2.0 * (double)I[0] * (double)I[1] * (double)I[2];
                    *bytes = 4.0 * ((double)I[0] * (double)I[1] + (double)I[1] * (double)I[2] + (double)I[0] * (double)I[2]);
                    *name = "bn_conv1x1";
                    break;
                case TP_OP_ATTENTION:
                    *flops = 4.0 * (double)(I[0] * I[1]) * (double)(I[2] * I[2]) * (double)I[3];
                    *bytes = 16.0 * (double)(I[0] * I[2]) * (double)(I[1] * I[3]);
                    *name = "attention";
                    break;
                default: break;
            }
            break;
        default:
            break;
    }
}

int Engine::exec_compute(Model& m, const Op& op, bool launch) {
    if (!profiling_ || !launch || host_only()) return exec_compute_impl(m, op, launch);
    while (prof_events_.size() < prof_next_ + 2) {
        hipEvent_t e = nullptr;
        HIPCHK(hipEventCreate(&e));
        prof_events_.push_back(e);
    }
    hipEvent_t a = prof_events_[prof_next_], b = prof_events_[prof_next_ + 1];
    prof_next_ += 2;
    double flops, bytes;
    const char* name;
    op_work(op, &flops, &bytes, &name);
    tpk::set_last_kernel(name);  // the MFMA launchers overwrite this with the variant they pick
    HIPCHK(hipEventRecord(a, compute_));
    const int r = exec_compute_impl(m, op, true);
    HIPCHK(hipEventRecord(b, compute_));
    // GEMM and convolution launches are accounted per shape: the same kernel runs at very different
    // fractions of the matrix peak on different shapes
    std::string label = tpk::last_kernel_name();
    char shape[48] = "";
    if (op.kind == OPK_GEMM) {
        if (op.i[8] * op.i[9] > 1)
            std::snprintf(shape, sizeof shape, "[%lldx%lldx%lld b%lld]", (long long)op.i[0], (long long)op.i[1],
                          (long long)op.i[2], (long long)(op.i[8] * op.i[9]));
        else
            std::snprintf(shape, sizeof shape, "[%lldx%lldx%lld]", (long long)op.i[0], (long long)op.i[1], (long long)op.i[2]);
    } else if (op.kind == OPK_CONV) {
        std::snprintf(shape, sizeof shape, "[%lldx%lldx%lldx%lld>%lld k%lldx%lld s%lld]", (long long)op.i[0], (long long)op.i[1],
                      (long long)op.i[2], (long long)op.i[3], (long long)op.i[4], (long long)op.i[5], (long long)op.i[6],
                      (long long)op.i[7]);
    }
    label += shape;
    prof_records_.push_back({prof_label(label), a, b, flops, bytes});
    return r;
}

// Labels live as long as the engine: records and statistics hold pointers to them.
const char* Engine::prof_label(const std::string& s) { return prof_labels_.insert(s).first->c_str(); }

int Engine::profile_begin() {
    std::lock_guard<std::mutex> lk(mu_);
    if (host_only()) return TP_ENODEV;
    profiling_ = true;
    prof_next_ = 0;
    prof_records_.clear();
    prof_stats_.clear();
    return 0;
}

int Engine::profile_end() {
    std::lock_guard<std::mutex> lk(mu_);
    if (host_only()) return TP_ENODEV;
    if (!profiling_) return TP_ESTATE;
    profiling_ = false;
    HIPCHK(hipStreamSynchronize(compute_));
    prof_stats_.clear();
    for (auto& r : prof_records_) {
        float ms = 0.f;
        HIPCHK(hipEventElapsedTime(&ms, r.a, r.b));
        tp_kernel_stat* st = nullptr;
        for (auto& s : prof_stats_)
            if (std::strncmp(s.name, r.name, sizeof(s.name) - 1) == 0) st = &s;
        if (!st) {
            tp_kernel_stat ns;
            std::memset(&ns, 0, sizeof(ns));
            std::strncpy(ns.name, r.name, sizeof(ns.name) - 1);
            prof_stats_.push_back(ns);
            st = &prof_stats_.back();
        }
        st->launches++;
        st->total_us += (double)ms * 1000.0;
        st->flops += r.flops;
        st->bytes += r.bytes;
    }
    // event overhead: median duration of an empty bracket
    while (prof_events_.size() < 2) {
        hipEvent_t e = nullptr;
        HIPCHK(hipEventCreate(&e));
        prof_events_.push_back(e);
    }
    std::vector<float> empt;
    for (int i = 0; i < 21; ++i) {
        HIPCHK(hipEventRecord(prof_events_[0], compute_));
        HIPCHK(hipEventRecord(prof_events_[1], compute_));
        HIPCHK(hipEventSynchronize(prof_events_[1]));
        float ms = 0.f;
        HIPCHK(hipEventElapsedTime(&ms, prof_events_[0], prof_events_[1]));
        empt.push_back(ms);
    }
    std::sort(empt.begin(), empt.end());
    tp_kernel_stat es;
    std::memset(&es, 0, sizeof(es));
    std::strncpy(es.name, "__empty_bracket__", sizeof(es.name) - 1);
    es.launches = 1;
    es.total_us = (double)empt[empt.size() / 2] * 1000.0;
    prof_stats_.push_back(es);
    prof_records_.clear();
    return 0;
}

int Engine::profile_read(int index, tp_kernel_stat* out) {
    std::lock_guard<std::mutex> lk(mu_);
    if (!out) return TP_EINVAL;
    if (index < 0 || index >= (int)prof_stats_.size()) return TP_ENOENT;
    *out = prof_stats_[index];
    return 0;
}

int Engine::exec_op(Model& m, const Op& op, ReplayCtx* rc, bool launch) {
    const bool run = launch && !host_only();
    switch (op.kind) {
        case OPK_GEMM:
        case OPK_CONV:
        case OPK_BN:
        case OPK_LAUNCH:
            return exec_compute(m, op, run);
        case OPK_H2D: {
            const uint64_t bytes = (uint64_t)op.i[0];
            if (!rc) return TP_EINVAL;
            if (rc->in_pos + bytes > rc->in_bytes) return TP_EINVAL;
            int r = do_h2d(m, op.p[0], rc->in + rc->in_pos, bytes);
            rc->in_pos += bytes;
            return r;
        }
        case OPK_D2H: {
            const uint64_t bytes = (uint64_t)op.i[0];
            if (!rc) return TP_EINVAL;
            if (rc->out_pos + bytes > rc->out_bytes) return TP_EINVAL;
            int r = do_d2h_async(m, rc->out + rc->out_pos, op.p[0], bytes);
            rc->out_pos += bytes;
            return r;
        }
        case OPK_D2D: {
            void *d = nullptr, *s = nullptr;
            const uint64_t bytes = (uint64_t)op.i[0];
            int r = resolve(m, op.p[0], bytes, false, &d);
            if (!r) r = resolve(m, op.p[1], bytes, false, &s);
            if (r) return r;
            if (!run || bytes == 0) return 0;
            return tpk::launch_copy(s, d, bytes, compute_);
        }
        case OPK_MEMSET: {
            void* d = nullptr;
            const uint64_t bytes = (uint64_t)op.i[0];
            int r = resolve(m, op.p[0], bytes, false, &d);
            if (r) return r;
            if (!(op.p[0] & kVaActBit)) return TP_ESTATE;
            if (!run || bytes == 0) return 0;
            HIPCHK(hipMemsetAsync(d, (int)op.i[1], bytes, compute_));
            return 0;
        }
        default:
            return TP_EINVAL;
    }
}

int Engine::op_compute(int client, const Op& op) {
    std::lock_guard<std::mutex> lk(mu_);
    int err = 0;
    Model* m = active_model(client, &err);
    if (!m) return err;
    if (mode_ == MODE_LOAD) return TP_ESTATE;
    int r = exec_op(*m, op, nullptr, true);
    if (r) {
        if (!m->async_error) m->async_error = r;
        return r;
    }
    if (mode_ == MODE_TRACK) m->program.push_back(op);
    return 0;
}

void Engine::drop_graph(Model& m) {
    if (m.graph_exec) (void)hipGraphExecDestroy(m.graph_exec);
    m.graph_exec = nullptr;
    m.graph_begin = m.graph_end = -1;
    m.graph_state = 0;
    m.warm_streak = 0;
}

// Captures the longest run of compute ops of the recorded program on the compute stream.  The
// model is fully loaded (no gate waits), the run holds no copy from or to the host and no memset
// (memset nodes are kept out of graphs on purpose), and capture is thread-local: the copy thread
// may be issuing another model's transfers meanwhile.
int Engine::build_graph(Model& m) {
    auto graphable = [](const Op& op) {
        return op.kind == OPK_GEMM || op.kind == OPK_CONV || op.kind == OPK_BN || op.kind == OPK_LAUNCH || op.kind == OPK_D2D;
    };
    int best_b = -1, best_e = -1;
    const int n = (int)m.program.size();
    for (int i = 0; i < n;) {
        if (!graphable(m.program[(size_t)i])) {
            ++i;
            continue;
        }
        int j = i;
        while (j < n && graphable(m.program[(size_t)j])) ++j;
        if (j - i > best_e - best_b) best_b = i, best_e = j;
        i = j;
    }
    m.graph_state = -1;
    if (best_b < 0 || best_e - best_b < graph_min_ops_) return 0;
    if (hipStreamBeginCapture(compute_, hipStreamCaptureModeThreadLocal) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    int r = 0;
    for (int i = best_b; i < best_e && !r; ++i) r = exec_op(m, m.program[(size_t)i], nullptr, true);
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(compute_, &g);
    if (r || e != hipSuccess || !g) {
        if (std::getenv("TORPOR_GRAPH_DEBUG")) std::fprintf(stderr, "graph: capture failed r=%d e=%d\n", r, (int)e);
        if (g) (void)hipGraphDestroy(g);
        (void)hipGetLastError();
        return r ? r : (int)e;
    }
    hipGraphExec_t ge = nullptr;
    e = hipGraphInstantiate(&ge, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess || !ge) {
        (void)hipGetLastError();
        return (int)e;
    }
    m.graph_exec = ge;
    m.graph_begin = best_b;
    m.graph_end = best_e;
    m.graph_state = 1;
    if (std::getenv("TORPOR_GRAPH_DEBUG")) std::fprintf(stderr, "graph: model %d ops [%d, %d)\n", m.id, best_b, best_e);
    return 0;
}

int Engine::replay(int client, const void* in, uint64_t in_bytes, void* out, uint64_t out_bytes) {
    std::lock_guard<std::mutex> lk(mu_);
    int err = 0;
    Model* m = active_model(client, &err);
    if (!m) return err;
    if (mode_ != MODE_EXEC) return TP_ESTATE;
    if (m->program.empty()) return TP_ENOENT;
    TraceRange trace("replay of model", m->id);
    const bool warm = m->fully_loaded;
    const auto t_start = Clock::now();
    ReplayCtx rc;
    rc.in = static_cast<const uint8_t*>(in);
    rc.in_bytes = in_bytes;
    rc.out = static_cast<uint8_t*>(out);
    rc.out_bytes = out_bytes;
    int ret = 0;
    bool completed = false;
    // Warm requests at an unchanged placement launch the compute part of the program as one HIP
    // graph (captured on the second such request); everything else goes op by op.
    bool graphed = false;
    if (warm && graph_min_ops_ > 0 && !profiling_ && !host_only()) {
        if (m->graph_state == 0 && ++m->warm_streak >= 2) (void)build_graph(*m);
        graphed = m->graph_state == 1;
    }
    const int n_ops = (int)m->program.size();
    for (int i = 0; i < n_ops; ++i) {
        if (graphed && i == m->graph_begin) {
            hipError_t e = hipGraphLaunch(m->graph_exec, compute_);
            if (e != hipSuccess) {
                ret = (int)e;
                break;
            }
            i = m->graph_end - 1;
            continue;
        }
        const Op& op = m->program[(size_t)i];
        int r = exec_op(*m, op, &rc, true);
        if (r && !ret) ret = r;
        if (r) break;
        if (op.kind == OPK_D2H) completed = true;
    }
    const double issue_us = us_since(t_start);
    int sr = do_stream_sync(m);
    if (!ret) ret = sr;
    static const bool dbg_timing = std::getenv("TORPOR_REPLAY_TIMING") != nullptr;
    if (dbg_timing)
        std::fprintf(stderr, "replay of %d (%s, %d ops): issued in %.1f us, done after %.1f us\n", m->id,
                     warm ? "warm" : "cold", n_ops, issue_us, us_since(t_start));
    if (warm && !ret && !profiling_) {
        const double us = us_since(t_start);
        if (m->warm_us <= 0 || us < m->warm_us) m->warm_us = us;
    }
    if (!warm && !ret && !profiling_ && !host_only() && m->ncopy >= 1 && m->ncopy <= 2) {
        // A sample for choose_copy_plan: the swap-in this request ran beside, from its start to the request's end
        // -- provided the request followed its swap-in at once.  One that was started later (a prefetch, a
        // dispatcher that serves other requests meanwhile) ends when its own schedule says, not the copy plan's.
        const double us = us_since(m->swap_t0);
        const double delay = std::chrono::duration<double, std::micro>(t_start - m->swap_t0).count();
        if (delay <= 0.1 * us) {
            double& best = m->cold_us[m->ncopy];
            if (m->cold_n[m->ncopy] == 0 || us < best) best = us;
            ++m->cold_n[m->ncopy];
        }
    }
    (void)completed;
    complete_request();
    return ret;
}
}  // namespace tp
