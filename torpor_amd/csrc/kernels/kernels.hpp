// Host-side launch interface of the hand-written gfx950 kernels.  Every
// launcher validates shapes on the host, enqueues on the given stream and
// returns a hipError_t-compatible int (0 = ok) or a negative TP_E* code.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace tpk {

enum : int { K_OK = 0, K_EINVAL = -22, K_EUNSUPPORTED = -38 };

struct EpilogueArgs {
    float alpha = 1.f;
    float beta = 0.f;
    const float* bias = nullptr;
    const float* bn_scale = nullptr;
    const float* bn_bias = nullptr;
    const float* bn_mean = nullptr;
    const float* bn_var = nullptr;
    float bn_eps = 1e-5f;
    const float* residual = nullptr;
    long ldr = 0;
    int act = 0;
};

// C[r][c] (row pitch ldc) = epilogue( sum_k X(r,k) * Y(c,k) ), X(r,k) at
// X[r*xs_r + k*xs_k], Y(c,k) at Y[c*ys_c + k*ys_k].  Two-level batching:
// batch z = b0*nb1 + b1 adds b0*?b0 + b1*?b1 to each base pointer.
struct GemmArgs {
    const float* X = nullptr;
    const float* Y = nullptr;
    float* C = nullptr;
    long M = 0, N = 0, K = 0;
    long xs_r = 0, xs_k = 1, ys_c = 0, ys_k = 1, ldc = 0;
    int nb0 = 1, nb1 = 1;
    long xb0 = 0, xb1 = 0, yb0 = 0, yb1 = 0, cb0 = 0, cb1 = 0;
    // optional row gather (1x1 strided convolution over NHWC): row m =
    // (n*Ho + ho)*Wo + wo reads X row ((n*H + ho*sh)*W + wo*sw).
    int gather = 0, Ho = 0, Wo = 0, H = 0, W = 0, sh = 1, sw = 1;
    EpilogueArgs ep;
    // Optional inference batch-norm (+ ReLU) of the X operand, per K index, applied as the operand is
    // loaded: x'(r,k) = act((x(r,k) - mean[k]) / sqrt(var[k] + eps) * gamma[k] + beta[k]).  What a
    // pre-activation network (DenseNet) computes in front of every 1x1 convolution.  beta / mean / var go
    // together; without them the transform is a plain per-K scale, x'(r,k) = act(x(r,k) * gamma[k]) (the channel
    // gate of a squeeze-and-excitation block at batch 1).  launch_gemm returns K_EUNSUPPORTED where no kernel
    // carries the transform (see gemm.hip).
    const float* pre_gamma = nullptr;
    const float* pre_beta = nullptr;
    const float* pre_mean = nullptr;
    const float* pre_var = nullptr;
    float pre_eps = 0.f;
    int pre_relu = 0;
};
constexpr long kPreBnMaxK = 2048;  // K range of one workgroup whose folded vectors fit the kernel's LDS block

struct ConvArgs {
    const float* x = nullptr;
    const float* w = nullptr;  // [Cout][Cin][KH][KW]
    float* y = nullptr;
    int N = 0, H = 0, W = 0, Cin = 0, Cout = 0, KH = 0, KW = 0;
    int sh = 1, sw = 1, ph = 0, pw = 0;
    int x_nhwc = 1, y_nhwc = 1;  // 0 = NCHW
    // NHWC only: floats between consecutive pixels of x / y (0 = Cin / Cout).  A larger pitch
    // reads the first Cin channels of a wider tensor or writes a channel slice of one (how
    // DenseNet-style concatenation is served without a copy).
    long x_pitch = 0, y_pitch = 0;
    int groups = 1;              // 1, or Cin == Cout == groups (depthwise, NHWC, w is [C][1][KH][KW])
    EpilogueArgs ep;             // residual shares the layout of y
};

struct Workspace {
    float* ptr = nullptr;  // split-K partial sums
    size_t bytes = 0;
    const float* zeros = nullptr;  // >= 64 zero bytes, 16 B aligned: source for padded convolution taps
    // kSplitTickets counters, zero between launches: with them a K range split over workgroups is summed
    // by the workgroup that finishes a tile last, inside the same launch; without, by a second launch
    unsigned* tickets = nullptr;
};
constexpr int kSplitTickets = 1024;

void kernels_init(int device);  // caches CU count
int launch_gemm(const GemmArgs& a, const Workspace& ws, hipStream_t s);
// Bytes of split-K partial sums launch_gemm writes for this call when the workspace is large enough to
// hold them (0: the call uses no workspace); negative = the arguments are refused.
long gemm_workspace_need(const GemmArgs& a);
int launch_conv2d(const ConvArgs& a, const Workspace& ws, hipStream_t s);
// introspection for tests/bench: which path the last launch on this thread took
const char* last_kernel_name();
void set_last_kernel(const char* name);

// ---- HBM-bound operators (elementwise.hip / reduce.hip) ----
// x_pitch: NHWC only, floats between consecutive rows of x (0 = C); y is always dense.
int launch_bn_inference(const float* x, float* y, const float* g, const float* b, const float* mean,
                        const float* var, float eps, long rows, int C, int nhwc, long hw, int relu, long x_pitch,
                        hipStream_t s);
// NHWC average pooling, window k x k, zero padding counted in the divisor (torch's
// count_include_pad=True); y_pitch = floats between output pixels (0 = C).
int launch_avgpool2d(const float* x, float* y, int N, int H, int W, int C, int k, int stride, int pad, long y_pitch,
                     hipStream_t s);
// y[n][p][c] = x[n][p][c] * s[n][c], NHWC with HW pixels per image (squeeze-and-excitation gating)
int launch_scale_channels(const float* x, const float* sc, float* y, int N, long HW, int C, hipStream_t s);
// dst[r*dst_pitch + c] = src[r*src_pitch + c], r < rows, c < width
int launch_copy2d(const float* src, float* dst, long rows, int width, long src_pitch, long dst_pitch, hipStream_t s);
int launch_relu(const float* x, float* y, long n, hipStream_t s);
int launch_add(const float* a, const float* b, float* y, long n, int relu, hipStream_t s);
int launch_bias_act(const float* x, const float* bias, float* y, long rows, int C, int act, hipStream_t s);
int launch_gelu(const float* x, float* y, long n, hipStream_t s);
int launch_nchw_to_nhwc(const float* x, float* y, int N, int C, int H, int W, hipStream_t s);
int launch_nhwc_to_nchw(const float* x, float* y, int N, int C, int H, int W, hipStream_t s);
// y_pitch: NHWC only, floats between output pixels (0 = C)
int launch_maxpool2d(const float* x, float* y, int N, int H, int W, int C, int k, int stride, int pad, int nhwc,
                     long y_pitch, hipStream_t s);
int launch_global_avgpool(const float* x, float* y, int N, int HW, int C, int nhwc, const Workspace& ws,
                          hipStream_t s);
int launch_layernorm(const float* x, const float* residual, const float* gamma, const float* beta, float* y,
                     long rows, int width, float eps, hipStream_t s);
// y[row] = softmax(scale * x[row] + mask[(row / rows_per_mask) * width ...]) over `width`
int launch_softmax(const float* x, const float* mask, float* y, long rows, int width, float scale,
                   long rows_per_mask, hipStream_t s);
// out[b,q,a,:] = softmax_k(scale * Q[b,q,a,:].K[b,k,a,:] + mask[b,k]) . V[b,k,a,:]; row (b*S + t) of each
// operand is at pointer + (b*S + t)*ld, head a at column a*dh.  dh must be 64.
int launch_attention(const float* q, const float* k, const float* v, const float* mask, float* out, int B, int A, int S,
                     int dh, long ldq, long ldk, long ldv, long ldo, float scale, hipStream_t s);
int launch_embedding(const int64_t* ids, const int64_t* type_ids, const float* word, const float* pos,
                     const float* type, float* y, long tokens, int seq, int width, long vocab, int n_types,
                     hipStream_t s);
int launch_sum(const float* x, float* y, long n, hipStream_t s);  // y[0] = sum(x), two-pass deterministic
int launch_fill(float* y, float v, long n, hipStream_t s);
int launch_copy(const void* src, void* dst, size_t bytes, hipStream_t s);

// Expansion of transfer groups into the weight image.  A piece is a run of one tensor.  Raw
// (base < 0): `bytes` bytes from src to dst, both 16-byte aligned.  Packed (weight_pack.hpp): src is
// the tensor's payload and dst the tensor's place in the image; words [w_from, w_to) are expanded
// (w_from a multiple of 64; w_to a multiple of 64 or the tensor's word count), reading the codes of
// the same 2048-word block before w_from as well, which an earlier transfer group has delivered.
// w_zero_to > w_to (a multiple of 64, less than 64 words past w_to): the words [w_to, w_zero_to) -- the
// alignment gap behind the tensor's last word -- are written as zeros, as they are in the host image.
struct UnpackPiece {
    const uint8_t* src;
    uint8_t* dst;
    uint64_t bytes;
    uint64_t w_from, w_to;
    uint64_t w_zero_to;   // 0 = nothing to clear behind w_to
    const uint8_t* ext;   // the tensor's extension stream
    const uint32_t* tab;  // the tensor's block table
    int32_t base;
    uint32_t first_block;  // filled by launch_unpack
};
constexpr int kUnpackMaxPieces = 24;
struct UnpackArgs {
    UnpackPiece piece[kUnpackMaxPieces];
    int n = 0;
};
int launch_unpack(UnpackArgs& a, hipStream_t s);

}  // namespace tpk
