// HBM-bound operators for gfx950: the kernels the reference runs through
// cudnnBatchNormalizationForwardInference (include/server/cuda_server.hpp:737-771)
// and through generic cudaLaunchKernel of libtorch kernels
// (include/server/cuda_server.hpp:1226-1310): ReLU, residual add, bias add,
// GELU, max/avg pooling, LayerNorm, softmax, embedding gather, sum.
//
// Elementwise kernels move dwordx4 per lane with grid-stride loops; row
// reductions (LayerNorm, softmax) use one 64-lane wavefront per row and
// cross-lane shuffles, so a row never touches LDS.
#include "kernels.hpp"
#include "mfma_tile.hpp"

namespace tpk {

int num_cu();

static inline int grid_for(long work_items, int block) {
    long b = (work_items + block - 1) / block;
    long cap = (long)num_cu() * 16;
    if (b > cap) b = cap;
    if (b < 1) b = 1;
    return (int)b;
}
static inline bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// ---------------------------------------------------------------- batch norm
// nhwc: channel = i % C ; nchw: channel = (i / hw) % C
__global__ __launch_bounds__(256) void bn_nhwc_vec_kernel(const f32x4* __restrict__ x, f32x4* __restrict__ y,
                                                          const float* __restrict__ g, const float* __restrict__ b,
                                                          const float* __restrict__ mean,
                                                          const float* __restrict__ var, float eps, long nvec, int C4,
                                                          int relu) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += (long)gridDim.x * blockDim.x) {
        const int c = (int)(i % C4) * 4;
        f32x4 v = x[i];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float sc = g[c + j] * (1.0f / sqrtf(var[c + j] + eps));
            float o = (v[j] - mean[c + j]) * sc + b[c + j];
            if (relu) o = o > 0.f ? o : 0.f;
            v[j] = o;
        }
        y[i] = v;
    }
}
__global__ __launch_bounds__(256) void bn_scalar_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                        const float* __restrict__ g, const float* __restrict__ b,
                                                        const float* __restrict__ mean, const float* __restrict__ var,
                                                        float eps, long n, int C, long hw, int nhwc, int relu) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int c = nhwc ? (int)(i % C) : (int)((i / hw) % C);
        const float sc = g[c] * (1.0f / sqrtf(var[c] + eps));
        float o = (x[i] - mean[c]) * sc + b[c];
        if (relu) o = o > 0.f ? o : 0.f;
        y[i] = o;
    }
}
// rows of C floats at x + row*x_pitch -> dense y
__global__ __launch_bounds__(256) void bn_nhwc_pitch_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                            const float* __restrict__ g, const float* __restrict__ b,
                                                            const float* __restrict__ mean,
                                                            const float* __restrict__ var, float eps, long n4, int C4,
                                                            long x_pitch, int relu) {
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
        const long row = i / C4;
        const int c = (int)(i - row * C4) * 4;
        f32x4 v = *reinterpret_cast<const f32x4*>(x + row * x_pitch + c);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float sc = g[c + j] / sqrtf(var[c + j] + eps);
            float t = (v[j] - mean[c + j]) * sc + b[c + j];
            if (relu) t = t > 0.f ? t : 0.f;
            v[j] = t;
        }
        reinterpret_cast<f32x4*>(y)[i] = v;
    }
}
int launch_bn_inference(const float* x, float* y, const float* g, const float* b, const float* mean,
                        const float* var, float eps, long rows, int C, int nhwc, long hw, int relu, long x_pitch,
                        hipStream_t s) {
    if (!x || !y || !g || !b || !mean || !var || rows < 0 || C <= 0) return K_EINVAL;
    const long n = rows * C;  // rows = N*H*W
    if (n == 0) return 0;
    if (x_pitch != 0 && x_pitch != C) {
        if (!nhwc || x_pitch < C) return K_EINVAL;
        if (C % 4 != 0 || x_pitch % 4 != 0 || !al16(x) || !al16(y)) return K_EUNSUPPORTED;
        hipLaunchKernelGGL(bn_nhwc_pitch_kernel, dim3(grid_for(n / 4, 256)), dim3(256), 0, s, x, y, g, b, mean, var,
                           eps, n / 4, C / 4, x_pitch, relu);
        return (int)hipGetLastError();
    }
    if (nhwc && C % 4 == 0 && al16(x) && al16(y)) {
        hipLaunchKernelGGL(bn_nhwc_vec_kernel, dim3(grid_for(n / 4, 256)), dim3(256), 0, s,
                           reinterpret_cast<const f32x4*>(x), reinterpret_cast<f32x4*>(y), g, b, mean, var, eps,
                           n / 4, C / 4, relu);
    } else {
        hipLaunchKernelGGL(bn_scalar_kernel, dim3(grid_for(n, 256)), dim3(256), 0, s, x, y, g, b, mean, var, eps, n,
                           C, hw, nhwc, relu);
    }
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------- pooling window / strided copy
__global__ __launch_bounds__(256) void avgpool2d_kernel(const float* __restrict__ x, float* __restrict__ y, int H,
                                                        int W, int C, int Ho, int Wo, int k, int stride, int pad,
                                                        long y_pitch, long total) {
    const long st = (long)gridDim.x * blockDim.x;
    const float inv = 1.0f / (float)(k * k);
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += st) {
        const int c = (int)(i % C);
        long t = i / C;
        const int wo = (int)(t % Wo);
        t /= Wo;
        const int ho = (int)(t % Ho);
        const long n = t / Ho;
        float acc = 0.f;
        for (int kh = 0; kh < k; ++kh) {
            const int hi = ho * stride - pad + kh;
            if (hi < 0 || hi >= H) continue;
            for (int kw = 0; kw < k; ++kw) {
                const int wi = wo * stride - pad + kw;
                if (wi < 0 || wi >= W) continue;
                acc += x[((n * H + hi) * W + wi) * C + c];
            }
        }
        y[((n * Ho + ho) * Wo + wo) * y_pitch + c] = acc * inv;
    }
}
int launch_avgpool2d(const float* x, float* y, int N, int H, int W, int C, int k, int stride, int pad, long y_pitch,
                     hipStream_t s) {
    if (!x || !y || N < 1 || H < 1 || W < 1 || C < 1 || k < 1 || stride < 1 || pad < 0 || H + 2 * pad < k ||
        W + 2 * pad < k)
        return K_EINVAL;
    if (y_pitch == 0) y_pitch = C;
    if (y_pitch < C) return K_EINVAL;
    const int Ho = (H + 2 * pad - k) / stride + 1, Wo = (W + 2 * pad - k) / stride + 1;
    const long total = (long)N * Ho * Wo * C;
    hipLaunchKernelGGL(avgpool2d_kernel, dim3(grid_for(total, 256)), dim3(256), 0, s, x, y, H, W, C, Ho, Wo, k,
                       stride, pad, y_pitch, total);
    return (int)hipGetLastError();
}

// y[n][p][c] = x[n][p][c] * s[n][c]  (squeeze-and-excitation gating, NHWC)
__global__ __launch_bounds__(256) void scale_channels_kernel(const float* __restrict__ x, const float* __restrict__ sc,
                                                             float* __restrict__ y, long total, long hwc, int C) {
    const long st = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += st) {
        const long n = i / hwc;
        const int c = (int)(i % C);
        y[i] = x[i] * sc[n * C + c];
    }
}
int launch_scale_channels(const float* x, const float* sc, float* y, int N, long HW, int C, hipStream_t s) {
    if (!x || !sc || !y || N < 1 || HW < 1 || C < 1) return K_EINVAL;
    const long total = (long)N * HW * C;
    hipLaunchKernelGGL(scale_channels_kernel, dim3(grid_for(total, 256)), dim3(256), 0, s, x, sc, y, total, HW * C, C);
    return (int)hipGetLastError();
}

__global__ __launch_bounds__(256) void copy2d_kernel(const float* __restrict__ src, float* __restrict__ dst, long total,
                                                     int width, long src_pitch, long dst_pitch) {
    const long st = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += st) {
        const long r = i / width;
        const int c = (int)(i - r * width);
        dst[r * dst_pitch + c] = src[r * src_pitch + c];
    }
}
int launch_copy2d(const float* src, float* dst, long rows, int width, long src_pitch, long dst_pitch, hipStream_t s) {
    if (!src || !dst || rows < 0 || width < 1 || src_pitch < width || dst_pitch < width) return K_EINVAL;
    const long total = rows * width;
    if (total == 0) return 0;
    hipLaunchKernelGGL(copy2d_kernel, dim3(grid_for(total, 256)), dim3(256), 0, s, src, dst, total, width, src_pitch,
                       dst_pitch);
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------- elementwise
// mode 0: relu(a); 1: a+b; 2: relu(a+b); 3: gelu(a)
__global__ __launch_bounds__(256) void ew_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                 float* __restrict__ y, long n, int mode, int vec) {
    const long tid = (long)blockIdx.x * blockDim.x + threadIdx.x, stride = (long)gridDim.x * blockDim.x;
    if (vec) {
        const long nv = n >> 2;
        const f32x4* a4 = reinterpret_cast<const f32x4*>(a);
        const f32x4* b4 = reinterpret_cast<const f32x4*>(b);
        f32x4* y4 = reinterpret_cast<f32x4*>(y);
        for (long i = tid; i < nv; i += stride) {
            f32x4 v = a4[i];
            if (mode == 1 || mode == 2) {
                const f32x4 w = b4[i];
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] += w[j];
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (mode == 0 || mode == 2) v[j] = v[j] > 0.f ? v[j] : 0.f;
                if (mode == 3) v[j] = apply_act(v[j], ACT_GELU);
            }
            y4[i] = v;
        }
        for (long i = (nv << 2) + tid; i < n; i += stride) {
            float v = a[i];
            if (mode == 1 || mode == 2) v += b[i];
            if (mode == 0 || mode == 2) v = v > 0.f ? v : 0.f;
            if (mode == 3) v = apply_act(v, ACT_GELU);
            y[i] = v;
        }
    } else {
        for (long i = tid; i < n; i += stride) {
            float v = a[i];
            if (mode == 1 || mode == 2) v += b[i];
            if (mode == 0 || mode == 2) v = v > 0.f ? v : 0.f;
            if (mode == 3) v = apply_act(v, ACT_GELU);
            y[i] = v;
        }
    }
}
static int launch_ew(const float* a, const float* b, float* y, long n, int mode, hipStream_t s) {
    if (!a || !y || n < 0 || ((mode == 1 || mode == 2) && !b)) return K_EINVAL;
    if (n == 0) return 0;
    const int vec = al16(a) && al16(y) && (!b || al16(b));
    hipLaunchKernelGGL(ew_kernel, dim3(grid_for(vec ? (n + 3) / 4 : n, 256)), dim3(256), 0, s, a, b ? b : a, y, n,
                       mode, vec);
    return (int)hipGetLastError();
}
int launch_relu(const float* x, float* y, long n, hipStream_t s) { return launch_ew(x, nullptr, y, n, 0, s); }
int launch_add(const float* a, const float* b, float* y, long n, int relu, hipStream_t s) {
    return launch_ew(a, b, y, n, relu ? 2 : 1, s);
}
int launch_gelu(const float* x, float* y, long n, hipStream_t s) { return launch_ew(x, nullptr, y, n, 3, s); }

__global__ __launch_bounds__(256) void bias_act_kernel(const float* __restrict__ x, const float* __restrict__ bias,
                                                       float* __restrict__ y, long n, int C, int act) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        y[i] = apply_act(x[i] + bias[i % C], act);
}
int launch_bias_act(const float* x, const float* bias, float* y, long rows, int C, int act, hipStream_t s) {
    if (!x || !bias || !y || rows < 0 || C <= 0) return K_EINVAL;
    const long n = rows * C;
    if (n == 0) return 0;
    hipLaunchKernelGGL(bias_act_kernel, dim3(grid_for(n, 256)), dim3(256), 0, s, x, bias, y, n, C, act);
    return (int)hipGetLastError();
}

__global__ __launch_bounds__(256) void fill_kernel(float* __restrict__ y, float v, long n) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) y[i] = v;
}
int launch_fill(float* y, float v, long n, hipStream_t s) {
    if (!y || n < 0) return K_EINVAL;
    if (n == 0) return 0;
    hipLaunchKernelGGL(fill_kernel, dim3(grid_for(n, 256)), dim3(256), 0, s, y, v, n);
    return (int)hipGetLastError();
}

__global__ __launch_bounds__(256) void copy_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                   size_t bytes, int vec) {
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (size_t)gridDim.x * blockDim.x;
    if (vec) {
        const size_t nv = bytes >> 4;
        const f32x4* s4 = reinterpret_cast<const f32x4*>(src);
        f32x4* d4 = reinterpret_cast<f32x4*>(dst);
        for (size_t i = tid; i < nv; i += stride) d4[i] = s4[i];
        for (size_t i = (nv << 4) + tid; i < bytes; i += stride) dst[i] = src[i];
    } else {
        for (size_t i = tid; i < bytes; i += stride) dst[i] = src[i];
    }
}
int launch_copy(const void* src, void* dst, size_t bytes, hipStream_t s) {
    if (!src || !dst) return K_EINVAL;
    if (bytes == 0) return 0;
    const int vec = al16(src) && al16(dst);
    hipLaunchKernelGGL(copy_kernel, dim3(grid_for((long)(vec ? (bytes + 15) / 16 : bytes), 256)), dim3(256), 0, s,
                       static_cast<const uint8_t*>(src), static_cast<uint8_t*>(dst), bytes, vec);
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------- layout
// NCHW -> NHWC through a 32x33 LDS tile over (C, HW) per image.
__global__ __launch_bounds__(256) void transpose_kernel(const float* __restrict__ x, float* __restrict__ y, int R,
                                                        int Ccols) {
    // x: [batch][R][Ccols] -> y: [batch][Ccols][R]
    __shared__ float tile[32][33];
    const long base = (long)blockIdx.z * R * Ccols;
    const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    for (int j = ty; j < 32; j += 8) {
        const int r = r0 + j, c = c0 + tx;
        tile[j][tx] = (r < R && c < Ccols) ? x[base + (long)r * Ccols + c] : 0.f;
    }
    __syncthreads();
    for (int j = ty; j < 32; j += 8) {
        const int c = c0 + j, r = r0 + tx;
        if (r < R && c < Ccols) y[base + (long)c * R + r] = tile[tx][j];
    }
}
static int launch_transpose(const float* x, float* y, int batch, int R, int Ccols, hipStream_t s) {
    if (!x || !y || batch <= 0 || R <= 0 || Ccols <= 0) return K_EINVAL;
    dim3 grid((Ccols + 31) / 32, (R + 31) / 32, batch);
    if (grid.y > 65535 || grid.z > 65535) return K_EUNSUPPORTED;
    hipLaunchKernelGGL(transpose_kernel, grid, dim3(256), 0, s, x, y, R, Ccols);
    return (int)hipGetLastError();
}
int launch_nchw_to_nhwc(const float* x, float* y, int N, int C, int H, int W, hipStream_t s) {
    return launch_transpose(x, y, N, C, H * W, s);
}
int launch_nhwc_to_nchw(const float* x, float* y, int N, int C, int H, int W, hipStream_t s) {
    return launch_transpose(x, y, N, H * W, C, s);
}

// ---------------------------------------------------------------- pooling
__global__ __launch_bounds__(256) void maxpool_kernel(const float* __restrict__ x, float* __restrict__ y, int N, int H,
                                                      int W, int C, int Ho, int Wo, int k, int stride, int pad,
                                                      int nhwc, long y_pitch) {
    const long total = (long)N * Ho * Wo * C;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        int c, wo, ho;
        long n;
        if (nhwc) {
            c = (int)(i % C);
            long t = i / C;
            wo = (int)(t % Wo);
            t /= Wo;
            ho = (int)(t % Ho);
            n = t / Ho;
        } else {
            wo = (int)(i % Wo);
            long t = i / Wo;
            ho = (int)(t % Ho);
            t /= Ho;
            c = (int)(t % C);
            n = t / C;
        }
        float m = -INFINITY;
        for (int kh = 0; kh < k; ++kh) {
            const int hi = ho * stride - pad + kh;
            if (hi < 0 || hi >= H) continue;
            for (int kw = 0; kw < k; ++kw) {
                const int wi = wo * stride - pad + kw;
                if (wi < 0 || wi >= W) continue;
                const long xi = nhwc ? (((n * H + hi) * W + wi) * C + c) : (((n * C + c) * H + hi) * W + wi);
                m = fmaxf(m, x[xi]);
            }
        }
        y[nhwc ? (i / C) * y_pitch + c : i] = m;
    }
}
// NHWC with C % 4 == 0 and 16-byte aligned rows: a thread takes four channels of one output pixel, so the
// window is k*k 128-bit loads and the index arithmetic is done once per four results, in 32 bits.
__global__ __launch_bounds__(256) void maxpool_nhwc4_kernel(const float* __restrict__ x, float* __restrict__ y, int H,
                                                            int W, int C4, int Ho, int Wo, int k, int stride, int pad,
                                                            long y_pitch, unsigned total) {
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += gridDim.x * blockDim.x) {
        const unsigned c4 = i % (unsigned)C4;
        unsigned t = i / (unsigned)C4;
        const unsigned pix = t;  // (n * Ho + ho) * Wo + wo
        const int wo = (int)(t % (unsigned)Wo);
        t /= (unsigned)Wo;
        const int ho = (int)(t % (unsigned)Ho);
        const long n = t / (unsigned)Ho;
        float4 m = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
        for (int kh = 0; kh < k; ++kh) {
            const int hi = ho * stride - pad + kh;
            if (hi < 0 || hi >= H) continue;
            for (int kw = 0; kw < k; ++kw) {
                const int wi = wo * stride - pad + kw;
                if (wi < 0 || wi >= W) continue;
                const float4 v = *reinterpret_cast<const float4*>(x + (((n * H + hi) * W + wi) * C4 + c4) * 4);
                m.x = fmaxf(m.x, v.x), m.y = fmaxf(m.y, v.y), m.z = fmaxf(m.z, v.z), m.w = fmaxf(m.w, v.w);
            }
        }
        *reinterpret_cast<float4*>(y + (long)pix * y_pitch + c4 * 4) = m;
    }
}
int launch_maxpool2d(const float* x, float* y, int N, int H, int W, int C, int k, int stride, int pad, int nhwc,
                     long y_pitch, hipStream_t s) {
    if (!x || !y || N <= 0 || H <= 0 || W <= 0 || C <= 0 || k <= 0 || stride <= 0 || pad < 0 || pad * 2 > k)
        return K_EINVAL;
    if (y_pitch == 0) y_pitch = C;
    if (y_pitch < C || (y_pitch != C && !nhwc)) return K_EINVAL;
    const int Ho = (H + 2 * pad - k) / stride + 1, Wo = (W + 2 * pad - k) / stride + 1;
    if (Ho <= 0 || Wo <= 0) return K_EINVAL;
    const long total = (long)N * Ho * Wo * C;
    const bool vec4 = nhwc && (C & 3) == 0 && (y_pitch & 3) == 0 && total / 4 < (1L << 31) &&
                      ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
    if (vec4) {
        hipLaunchKernelGGL(maxpool_nhwc4_kernel, dim3(grid_for(total / 4, 256)), dim3(256), 0, s, x, y, H, W, C / 4, Ho,
                           Wo, k, stride, pad, y_pitch, (unsigned)(total / 4));
        return (int)hipGetLastError();
    }
    hipLaunchKernelGGL(maxpool_kernel, dim3(grid_for(total, 256)), dim3(256), 0, s, x, y, N, H, W, C, Ho, Wo, k,
                       stride, pad, nhwc, y_pitch);
    return (int)hipGetLastError();
}

// NHWC: one thread per (n, c), lanes along c (coalesced).  NCHW: one wavefront per (n, c).
__global__ __launch_bounds__(256) void avgpool_nhwc_kernel(const float* __restrict__ x, float* __restrict__ y, int N,
                                                           int HW, int C) {
    const long total = (long)N * C;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const long n = i / C;
        const int c = (int)(i - n * C);
        const float* p = x + n * HW * C + c;
        float s = 0.f;
        for (int j = 0; j < HW; ++j) s += p[(long)j * C];
        y[i] = s / (float)HW;
    }
}
__global__ __launch_bounds__(256) void avgpool_nchw_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                           long rows, int HW) {
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* p = x + row * HW;
    float s = 0.f;
    for (int j = lane; j < HW; j += 64) s += p[j];
    s = wave_sum(s);
    if (lane == 0) y[row] = s / (float)HW;
}
// NHWC maps of 16 pixels and more: the pixels of an image are cut into S slices; a workgroup sums one slice
// for 64 channels (4 pixel phases x 64 lanes, coalesced along channels), the second kernel adds
// the S partial sums in a fixed order.
__global__ __launch_bounds__(256) void avgpool_partial_kernel(const float* __restrict__ x, float* __restrict__ part,
                                                              int HW, int C, int S) {
    __shared__ float red[4][64];
    const int cx = threadIdx.x & 63, ry = threadIdx.x >> 6;
    const int c = blockIdx.x * 64 + cx, sl = blockIdx.y, n = blockIdx.z;
    const int per = (HW + S - 1) / S;
    const int p0 = sl * per, p1 = (p0 + per < HW) ? p0 + per : HW;
    float acc = 0.f;
    if (c < C) {
        const float* px = x + (long)n * HW * C + c;
#pragma unroll 8
        for (int q = p0 + ry; q < p1; q += 4) acc += px[(long)q * C];
    }
    red[ry][cx] = acc;
    __syncthreads();
    if (ry == 0 && c < C) part[((long)n * S + sl) * C + c] = (red[0][cx] + red[1][cx]) + (red[2][cx] + red[3][cx]);
}
// A workgroup adds the S partial sums of 64 channels of one image: four slice phases x 64 lanes, each thread a
// chain of at most S / 4 independent loads (kept in flight together), then the four phases in a fixed order.
// (One thread per channel walking all S slices one load after the other took 10 us for S = 64.)
__global__ __launch_bounds__(256) void avgpool_final_kernel(const float* __restrict__ part, float* __restrict__ y,
                                                            int C, int S, float inv) {
    __shared__ float red[4][64];
    const int cx = threadIdx.x & 63, ph = threadIdx.x >> 6;
    const int c = blockIdx.x * 64 + cx, n = blockIdx.y;
    float acc = 0.f;
    if (c < C) {
        const float* ps = part + (long)n * S * C + c;
#pragma unroll 8
        for (int sl = ph; sl < S; sl += 4) acc += ps[(long)sl * C];
    }
    red[ph][cx] = acc;
    __syncthreads();
    if (ph == 0 && c < C) y[(long)n * C + c] = ((red[0][cx] + red[1][cx]) + (red[2][cx] + red[3][cx])) * inv;
}
// NHWC maps of 16 to 256 pixels in one launch: a workgroup takes 64 channels of one image as 16 lanes of
// four channels (128-bit loads) x 16 pixel phases, so a thread's chain of loads is HW / 16 long, and adds the
// phases through LDS in a fixed order.
__global__ __launch_bounds__(256) void avgpool_small_kernel(const float* __restrict__ x, float* __restrict__ y, int HW,
                                                            int C, float inv) {
    __shared__ float red[16][64];
    const int cq = threadIdx.x & 15, ph = threadIdx.x >> 4;
    const int c = blockIdx.x * 64 + cq * 4, n = blockIdx.y;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    if (c < C) {  // C % 4 == 0: the four channels are in range together
        const float* px = x + (long)n * HW * C + c;
#pragma unroll 4
        for (int q = ph; q < HW; q += 16) {
            const float4 v = *reinterpret_cast<const float4*>(px + (long)q * C);
            a0 += v.x;
            a1 += v.y;
            a2 += v.z;
            a3 += v.w;
        }
    }
    red[ph][cq * 4 + 0] = a0;
    red[ph][cq * 4 + 1] = a1;
    red[ph][cq * 4 + 2] = a2;
    red[ph][cq * 4 + 3] = a3;
    __syncthreads();
    if (threadIdx.x < 64) {
        const int cc = blockIdx.x * 64 + threadIdx.x;
        if (cc < C) {
            float acc = 0.f;
#pragma unroll
            for (int p = 0; p < 16; ++p) acc += red[p][threadIdx.x];
            y[(long)n * C + cc] = acc * inv;
        }
    }
}
int launch_global_avgpool(const float* x, float* y, int N, int HW, int C, int nhwc, const Workspace& ws,
                          hipStream_t s) {
    if (!x || !y || N <= 0 || HW <= 0 || C <= 0) return K_EINVAL;
    if (nhwc && HW >= 16 && HW <= 256 && N <= 65535 && (C & 3) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
        hipLaunchKernelGGL(avgpool_small_kernel, dim3((unsigned)((C + 63) / 64), (unsigned)N), dim3(256), 0, s, x, y, HW, C,
                           1.0f / (float)HW);
        return (int)hipGetLastError();
    }
    if (nhwc && HW >= 16 && ws.ptr) {
        int S = HW >= 512 ? (HW + 63) / 64 : (HW + 7) / 8;
        if (S > 64) S = 64;
        if ((size_t)N * S * C * sizeof(float) <= ws.bytes && N <= 65535) {
            hipLaunchKernelGGL(avgpool_partial_kernel, dim3((unsigned)((C + 63) / 64), (unsigned)S, (unsigned)N),
                               dim3(256), 0, s, x, ws.ptr, HW, C, S);
            hipLaunchKernelGGL(avgpool_final_kernel, dim3((unsigned)((C + 63) / 64), (unsigned)N), dim3(256), 0, s, ws.ptr, y,
                               C, S, 1.0f / (float)HW);
            return (int)hipGetLastError();
        }
    }
    if (nhwc) {
        hipLaunchKernelGGL(avgpool_nhwc_kernel, dim3(grid_for((long)N * C, 256)), dim3(256), 0, s, x, y, N, HW, C);
    } else {
        const long rows = (long)N * C;
        hipLaunchKernelGGL(avgpool_nchw_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, x, y, rows, HW);
    }
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------- LayerNorm
// y = (v - mean) / sqrt(var + eps) * gamma + beta with v = x (+ residual);
// one wavefront per row, two-pass variance, row kept in registers up to 2048 wide.
template <int MAXV>
__global__ __launch_bounds__(256) void layernorm_kernel(const float* __restrict__ x, const float* __restrict__ res,
                                                        const float* __restrict__ gamma,
                                                        const float* __restrict__ beta, float* __restrict__ y,
                                                        long rows, int width, float eps) {
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* xr = x + row * width;
    const float* rr = res ? res + row * width : nullptr;
    float* yr = y + row * width;
    float v[MAXV];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
        const int c = lane + i * 64;
        float t = 0.f;
        if (c < width) {
            t = xr[c];
            if (rr) t += rr[c];
        }
        v[i] = t;
        s += t;
    }
    const float mean = wave_sum(s) / (float)width;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
        const int c = lane + i * 64;
        const float d = (c < width) ? v[i] - mean : 0.f;
        q += d * d;
    }
    const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)width + eps);
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
        const int c = lane + i * 64;
        if (c < width) yr[c] = (v[i] - mean) * rstd * gamma[c] + beta[c];
    }
}
// One 256-thread workgroup per row, 128-bit accesses (width % 4 == 0, width <= 1024 * MAXQ, 16 B
// aligned rows): four times the wavefronts of the wave-per-row kernel are in flight, which is
// what hides the memory latency when there are only a few thousand rows.
template <int MAXQ>
__global__ __launch_bounds__(256) void layernorm_block_kernel(const float* __restrict__ x, const float* __restrict__ res,
                                                              const float* __restrict__ gamma,
                                                              const float* __restrict__ beta, float* __restrict__ y,
                                                              int width, float eps) {
    __shared__ float red[2][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const long row = blockIdx.x;
    const float4* xr = reinterpret_cast<const float4*>(x + row * width);
    const float4* rr = res ? reinterpret_cast<const float4*>(res + row * width) : nullptr;
    const float4* gr = reinterpret_cast<const float4*>(gamma);
    const float4* br = reinterpret_cast<const float4*>(beta);
    float4* yr = reinterpret_cast<float4*>(y + row * width);
    const int nq = width >> 2;
    float4 v[MAXQ], g[MAXQ], b[MAXQ];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < MAXQ; ++i) {
        const int c = tid + i * 256;
        v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c < nq) {
            v[i] = xr[c];
            if (rr) {
                const float4 t = rr[c];
                v[i].x += t.x;
                v[i].y += t.y;
                v[i].z += t.z;
                v[i].w += t.w;
            }
            g[i] = gr[c];  // issued now, needed only after both reductions
            b[i] = br[c];
        }
        s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    }
    s = wave_sum(s);
    if (lane == 0) red[0][wave] = s;
    __syncthreads();
    const float mean = ((red[0][0] + red[0][1]) + (red[0][2] + red[0][3])) / (float)width;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < MAXQ; ++i) {
        const int c = tid + i * 256;
        if (c < nq) {
            const float dx = v[i].x - mean, dy = v[i].y - mean, dz = v[i].z - mean, dw = v[i].w - mean;
            q += (dx * dx + dy * dy) + (dz * dz + dw * dw);
        }
    }
    q = wave_sum(q);
    if (lane == 0) red[1][wave] = q;
    __syncthreads();
    const float rstd = 1.0f / sqrtf(((red[1][0] + red[1][1]) + (red[1][2] + red[1][3])) / (float)width + eps);
#pragma unroll
    for (int i = 0; i < MAXQ; ++i) {
        const int c = tid + i * 256;
        if (c < nq) {
            float4 o;
            o.x = (v[i].x - mean) * rstd * g[i].x + b[i].x;
            o.y = (v[i].y - mean) * rstd * g[i].y + b[i].y;
            o.z = (v[i].z - mean) * rstd * g[i].z + b[i].z;
            o.w = (v[i].w - mean) * rstd * g[i].w + b[i].w;
            yr[c] = o;
        }
    }
}
__global__ __launch_bounds__(256) void layernorm_wide_kernel(const float* __restrict__ x,
                                                             const float* __restrict__ res,
                                                             const float* __restrict__ gamma,
                                                             const float* __restrict__ beta, float* __restrict__ y,
                                                             long rows, int width, float eps) {
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* xr = x + row * width;
    const float* rr = res ? res + row * width : nullptr;
    float* yr = y + row * width;
    float s = 0.f;
    for (int c = lane; c < width; c += 64) s += xr[c] + (rr ? rr[c] : 0.f);
    const float mean = wave_sum(s) / (float)width;
    float q = 0.f;
    for (int c = lane; c < width; c += 64) {
        const float d = xr[c] + (rr ? rr[c] : 0.f) - mean;
        q += d * d;
    }
    const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)width + eps);
    // y may alias x or residual element-wise: each lane reads its element before writing it
    for (int c = lane; c < width; c += 64) {
        const float t = xr[c] + (rr ? rr[c] : 0.f);
        yr[c] = (t - mean) * rstd * gamma[c] + beta[c];
    }
}
int launch_layernorm(const float* x, const float* residual, const float* gamma, const float* beta, float* y,
                     long rows, int width, float eps, hipStream_t s) {
    if (!x || !gamma || !beta || !y || rows < 0 || width <= 0) return K_EINVAL;
    if (rows == 0) return 0;
    const auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    if (width % 4 == 0 && width > 256 && width <= 4096 && rows <= 0x7fffffffL && al16(x) && al16(y) && al16(gamma) &&
        al16(beta) && (!residual || al16(residual))) {
        const dim3 g1((unsigned)rows);
        if (width <= 1024)
            hipLaunchKernelGGL(layernorm_block_kernel<1>, g1, dim3(256), 0, s, x, residual, gamma, beta, y, width, eps);
        else if (width <= 2048)
            hipLaunchKernelGGL(layernorm_block_kernel<2>, g1, dim3(256), 0, s, x, residual, gamma, beta, y, width, eps);
        else
            hipLaunchKernelGGL(layernorm_block_kernel<4>, g1, dim3(256), 0, s, x, residual, gamma, beta, y, width, eps);
        return (int)hipGetLastError();
    }
    const dim3 grid((unsigned)((rows + 3) / 4));
    if (width <= 64 * 4)
        hipLaunchKernelGGL(layernorm_kernel<4>, grid, dim3(256), 0, s, x, residual, gamma, beta, y, rows, width, eps);
    else if (width <= 64 * 16)
        hipLaunchKernelGGL(layernorm_kernel<16>, grid, dim3(256), 0, s, x, residual, gamma, beta, y, rows, width, eps);
    else if (width <= 64 * 32)
        hipLaunchKernelGGL(layernorm_kernel<32>, grid, dim3(256), 0, s, x, residual, gamma, beta, y, rows, width, eps);
    else
        hipLaunchKernelGGL(layernorm_wide_kernel, grid, dim3(256), 0, s, x, residual, gamma, beta, y, rows, width,
                           eps);
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------- softmax
template <int MAXV>
__global__ __launch_bounds__(256) void softmax_kernel(const float* __restrict__ x, const float* __restrict__ mask,
                                                      float* __restrict__ y, long rows, int width, float scale,
                                                      long rows_per_mask) {
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* xr = x + row * width;
    const float* mr = mask ? mask + (row / rows_per_mask) * width : nullptr;
    float* yr = y + row * width;
    float v[MAXV];
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
        const int c = lane + i * 64;
        float t = -INFINITY;
        if (c < width) {
            t = xr[c] * scale;
            if (mr) t += mr[c];
        }
        v[i] = t;
        m = fmaxf(m, t);
    }
    m = wave_max(m);
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
        const int c = lane + i * 64;
        const float e = (c < width) ? expf(v[i] - m) : 0.f;
        v[i] = e;
        s += e;
    }
    const float inv = 1.0f / wave_sum(s);
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
        const int c = lane + i * 64;
        if (c < width) yr[c] = v[i] * inv;
    }
}
int launch_softmax(const float* x, const float* mask, float* y, long rows, int width, float scale,
                   long rows_per_mask, hipStream_t s) {
    if (!x || !y || rows < 0 || width <= 0 || (mask && rows_per_mask <= 0)) return K_EINVAL;
    if (width > 64 * 32) return K_EUNSUPPORTED;
    if (rows == 0) return 0;
    const dim3 grid((unsigned)((rows + 3) / 4));
    if (rows_per_mask <= 0) rows_per_mask = 1;
    if (width <= 64 * 2)
        hipLaunchKernelGGL(softmax_kernel<2>, grid, dim3(256), 0, s, x, mask, y, rows, width, scale, rows_per_mask);
    else if (width <= 64 * 8)
        hipLaunchKernelGGL(softmax_kernel<8>, grid, dim3(256), 0, s, x, mask, y, rows, width, scale, rows_per_mask);
    else
        hipLaunchKernelGGL(softmax_kernel<32>, grid, dim3(256), 0, s, x, mask, y, rows, width, scale, rows_per_mask);
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------- embedding
// y[tok] = word[ids[tok]] + pos[tok % seq] + type[type_ids[tok]] ; one wavefront per token
__global__ __launch_bounds__(256) void embedding_kernel(const int64_t* __restrict__ ids,
                                                        const int64_t* __restrict__ type_ids,
                                                        const float* __restrict__ word,
                                                        const float* __restrict__ pos,
                                                        const float* __restrict__ type, float* __restrict__ y,
                                                        long tokens, int seq, int width, long vocab,
                                                        int n_types) {
    const int lane = threadIdx.x & 63;
    const long tok = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tok >= tokens) return;
    long id = ids[tok];
    if (id < 0) id = 0;
    if (id >= vocab) id = vocab - 1;
    const float* wr = word + id * width;
    const float* pr = pos ? pos + (tok % seq) * width : nullptr;
    long ty = type_ids ? type_ids[tok] : 0;
    if (ty < 0) ty = 0;
    if (ty >= n_types) ty = n_types - 1;
    const float* tr = type ? type + ty * width : nullptr;
    float* yr = y + tok * width;
    // rows that start on 16 bytes go four floats at a time (the sums are the same: (word + pos) + type)
    const uintptr_t bits = reinterpret_cast<uintptr_t>(wr) | reinterpret_cast<uintptr_t>(pr) |
                           reinterpret_cast<uintptr_t>(tr) | reinterpret_cast<uintptr_t>(yr);
    if ((width & 3) == 0 && (bits & 15) == 0) {
        for (int c = lane * 4; c < width; c += 256) {
            float4 v = *reinterpret_cast<const float4*>(wr + c);
            if (pr) {
                const float4 q = *reinterpret_cast<const float4*>(pr + c);
                v.x += q.x, v.y += q.y, v.z += q.z, v.w += q.w;
            }
            if (tr) {
                const float4 q = *reinterpret_cast<const float4*>(tr + c);
                v.x += q.x, v.y += q.y, v.z += q.z, v.w += q.w;
            }
            *reinterpret_cast<float4*>(yr + c) = v;
        }
        return;
    }
    for (int c = lane; c < width; c += 64) {
        float v = wr[c];
        if (pr) v += pr[c];
        if (tr) v += tr[c];
        yr[c] = v;
    }
}
int launch_embedding(const int64_t* ids, const int64_t* type_ids, const float* word, const float* pos,
                     const float* type, float* y, long tokens, int seq, int width, long vocab, int n_types,
                     hipStream_t s) {
    if (!ids || !word || !y || tokens < 0 || seq <= 0 || width <= 0 || vocab <= 0 || n_types <= 0) return K_EINVAL;
    if (tokens == 0) return 0;
    hipLaunchKernelGGL(embedding_kernel, dim3((unsigned)((tokens + 3) / 4)), dim3(256), 0, s, ids, type_ids, word,
                       pos, type, y, tokens, seq, width, vocab, n_types);
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------- sum
// Deterministic: one workgroup, fixed per-thread strides, tree in LDS.
__global__ __launch_bounds__(1024) void sum_kernel(const float* __restrict__ x, float* __restrict__ y, long n) {
    __shared__ float part[16];
    float s = 0.f;
    for (long i = threadIdx.x; i < n; i += 1024) s += x[i];
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.f;
        for (int i = 0; i < 16; ++i) t += part[i];
        y[0] = t;
    }
}
int launch_sum(const float* x, float* y, long n, hipStream_t s) {
    if (!x || !y || n < 0) return K_EINVAL;
    hipLaunchKernelGGL(sum_kernel, dim3(1), dim3(1024), 0, s, x, y, n);
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------- weight transfer format
// One workgroup handles one 2048-word block of a tensor (8 KiB of the image): a lane takes one group
// of eight words, 6 dwords of fields and 24 bits of codes in, two 128-bit stores out.  The rank of a
// lane's first out-of-window word in the tensor's extension stream is the block-table entry plus a
// prefix sum over the lanes before it.
constexpr int kUnpackBlockBytes = 8192;
__global__ __launch_bounds__(256) void unpack_kernel(const UnpackArgs a) {
    int k = 0;
    while (k + 1 < a.n && a.piece[k + 1].first_block <= blockIdx.x) ++k;
    const UnpackPiece& pc = a.piece[k];
    const uint64_t lb = blockIdx.x - pc.first_block;
    if (pc.base < 0) {
        const uint64_t off = lb * kUnpackBlockBytes;
        if (off >= pc.bytes) return;
        const uint64_t left = pc.bytes - off;
        uint8_t* __restrict__ dst = pc.dst + off;
        const uint8_t* __restrict__ src = pc.src + off;
        const uint64_t n = left < kUnpackBlockBytes ? left : kUnpackBlockBytes;
        const uint64_t nv = n >> 4;
        for (uint64_t i = threadIdx.x; i < nv; i += 256)
            reinterpret_cast<f32x4*>(dst)[i] = reinterpret_cast<const f32x4*>(src)[i];
        for (uint64_t i = (nv << 4) + threadIdx.x; i < n; i += 256) dst[i] = src[i];
        return;
    }
    __shared__ uint32_t wave_total[4];
    const uint64_t bi = pc.w_from / 2048 + lb;
    const uint64_t word0 = bi * 2048 + (uint64_t)threadIdx.x * 8;
    const bool have = word0 < pc.w_to;  // this group has arrived
    uint32_t f[8];
    uint32_t codes = 0;
    if (have) {
        const uint64_t unit = word0 >> 6;
        const uint32_t g = (uint32_t)(word0 & 63) >> 3;
        const uint32_t* __restrict__ up = reinterpret_cast<const uint32_t*>(pc.src + unit * 216);
        const uint32_t* __restrict__ fp = up + g * 6;
        uint32_t d[6];
#pragma unroll
        for (int j = 0; j < 6; ++j) d[j] = fp[j];
        f[0] = d[0] & 0xFFFFFFu;
        f[1] = (d[0] >> 24) | ((d[1] & 0xFFFFu) << 8);
        f[2] = (d[1] >> 16) | ((d[2] & 0xFFu) << 16);
        f[3] = d[2] >> 8;
        f[4] = d[3] & 0xFFFFFFu;
        f[5] = (d[3] >> 24) | ((d[4] & 0xFFFFu) << 8);
        f[6] = (d[4] >> 16) | ((d[5] & 0xFFu) << 16);
        f[7] = d[5] >> 8;
        const uint32_t bit = 24 * g, di = bit >> 5, sh = bit & 31;
        const uint64_t two = (uint64_t)up[48 + di] | ((uint64_t)up[48 + (di < 5 ? di + 1 : 5)] << 32);
        codes = (uint32_t)(two >> sh) & 0xFFFFFFu;
    }
    uint32_t cnt = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) cnt += ((codes >> (3 * j)) & 7u) == 7u ? 1u : 0u;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t x = cnt;
#pragma unroll
    for (int dlt = 1; dlt < 64; dlt <<= 1) {
        const uint32_t y = __shfl_up(x, dlt, 64);
        if (lane >= dlt) x += y;
    }
    if (lane == 63) wave_total[wave] = x;
    __syncthreads();
    uint32_t rank = x - cnt;
    for (int w = 0; w < wave; ++w) rank += wave_total[w];
    if (!have) {
        // behind the tensor's last word: the alignment gap of the image reads as zeros
        if (word0 < pc.w_zero_to) {
            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
            u32x4* z = reinterpret_cast<u32x4*>(reinterpret_cast<uint32_t*>(pc.dst) + word0);
            z[0] = u32x4{0u, 0u, 0u, 0u};
            z[1] = u32x4{0u, 0u, 0u, 0u};
        }
        return;
    }
    if (word0 < pc.w_from) return;
    const uint8_t* __restrict__ ext = pc.ext + pc.tab[bi] + rank;
    uint32_t w[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t code = (codes >> (3 * j)) & 7u;
        uint32_t e = (uint32_t)pc.base + code;
        if (code == 7u) e = *ext++;
        w[j] = (f[j] & 0x7FFFFFu) | ((f[j] >> 23) << 31) | ((e & 0xFFu) << 23);
    }
    uint32_t* __restrict__ out = reinterpret_cast<uint32_t*>(pc.dst) + word0;
    if (word0 + 8 <= pc.w_to) {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        reinterpret_cast<u32x4*>(out)[0] = u32x4{w[0], w[1], w[2], w[3]};
        reinterpret_cast<u32x4*>(out)[1] = u32x4{w[4], w[5], w[6], w[7]};
    } else {  // last group of a tensor whose word count is not a multiple of 8
        const uint64_t words = pc.w_to - word0;
        for (uint64_t j = 0; j < words; ++j) out[j] = w[j];
        if (pc.w_zero_to > pc.w_to)
            for (uint64_t j = words; j < 8; ++j) out[j] = 0u;
    }
}
int launch_unpack(UnpackArgs& a, hipStream_t s) {
    if (a.n < 0 || a.n > kUnpackMaxPieces) return K_EINVAL;
    uint64_t blocks = 0;
    for (int k = 0; k < a.n; ++k) {
        UnpackPiece& pc = a.piece[k];
        if (!pc.src || !pc.dst || !al16(pc.src) || !al16(pc.dst)) return K_EINVAL;
        pc.first_block = (uint32_t)blocks;
        if (pc.base < 0) {
            blocks += (pc.bytes + kUnpackBlockBytes - 1) / kUnpackBlockBytes;
        } else {
            if (pc.base > 255 || !pc.tab || pc.w_to < pc.w_from || (pc.w_from & 63)) return K_EINVAL;
            if (pc.w_zero_to && (pc.w_zero_to < pc.w_to || pc.w_zero_to - pc.w_to >= 64 || (pc.w_zero_to & 63)))
                return K_EINVAL;
            if (pc.w_to > pc.w_from) blocks += (pc.w_to + 2047) / 2048 - pc.w_from / 2048;
        }
        if (blocks > 0x7FFFFFFFull) return K_EINVAL;
    }
    if (blocks == 0) return 0;
    hipLaunchKernelGGL(unpack_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a);
    return (int)hipGetLastError();
}

}  // namespace tpk
