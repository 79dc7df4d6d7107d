/* TEST INFRASTRUCTURE ONLY - never linked into, imported by or called from the product.
 *
 * CPU restatement, in plain C with fp64 accumulation, of the arithmetic the reference
 * server performs through closed third-party libraries on its hot path.  The algorithms
 * are the published definitions of those library calls; the reference call sites are:
 *   ref_gemm        cublasSgemm / cublasSgemmStridedBatched   include/server/cuda_server.hpp:502-550
 *   ref_conv2d      cudnnConvolutionForward (cross-correlation, NCHW filter [K][C][R][S])
 *                                                             include/server/cuda_server.hpp:708-735
 *   ref_bn          cudnnBatchNormalizationForwardInference   include/server/cuda_server.hpp:737-771
 *   ref_layernorm / ref_softmax / ref_gelu / ref_maxpool / ref_avgpool / ref_embedding
 *                   libtorch kernels launched by name         include/server/cuda_server.hpp:1226-1310
 *
 * Pinning (tests/test_oracle_ops.py): every function is checked against the PyTorch CPU
 * library routine of the same operation (torch.matmul, F.conv2d, F.batch_norm,
 * F.layer_norm, softmax, F.gelu, F.max_pool2d, mean, F.embedding) and against closed forms
 * (delta-kernel convolution = identity, identity batch-norm, softmax rows sum to one,
 * LayerNorm output has zero mean / unit variance).  The reference tree holds no golden
 * vectors for any of these (its tests print y.sum() without an expected value).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

/* C[r*ldc + c] = alpha * sum_k X[r*xs_r + k*xs_k] * Y[c*ys_c + k*ys_k] + beta * C[...] */
void ref_gemm(const float* X, const float* Y, float* C, long M, long N, long K, long xs_r, long xs_k, long ys_c,
              long ys_k, long ldc, float alpha, float beta) {
    for (long r = 0; r < M; ++r)
        for (long c = 0; c < N; ++c) {
            double acc = 0.0;
            for (long k = 0; k < K; ++k) acc += (double)X[r * xs_r + k * xs_k] * (double)Y[c * ys_c + k * ys_k];
            double v = (double)alpha * acc;
            if (beta != 0.f) v += (double)beta * (double)C[r * ldc + c];
            C[r * ldc + c] = (float)v;
        }
}

/* Column-major SGEMM exactly as BLAS defines it: C(m x n) = alpha*op(A)*op(B) + beta*C. */
void ref_sgemm_colmajor(int transa, int transb, int m, int n, int k, float alpha, const float* A, int lda,
                        const float* B, int ldb, float beta, float* C, int ldc) {
    for (int j = 0; j < n; ++j)
        for (int i = 0; i < m; ++i) {
            double acc = 0.0;
            for (int p = 0; p < k; ++p) {
                const double a = transa ? A[p + (long)i * lda] : A[i + (long)p * lda];
                const double b = transb ? B[j + (long)p * ldb] : B[p + (long)j * ldb];
                acc += a * b;
            }
            double v = (double)alpha * acc;
            if (beta != 0.f) v += (double)beta * (double)C[i + (long)j * ldc];
            C[i + (long)j * ldc] = (float)v;
        }
}

static long xidx(int nhwc, long n, long c, long h, long w, long C, long H, long W) {
    return nhwc ? ((n * H + h) * W + w) * C + c : ((n * C + c) * H + h) * W + w;
}

/* y[n,k,ho,wo] = sum_{c,r,s} x[n,c,ho*sh-ph+r,wo*sw-pw+s] * w[k,c,r,s]; layouts selectable */
void ref_conv2d(const float* x, const float* w, float* y, int N, int H, int W, int Cin, int Cout, int KH, int KW,
                int sh, int sw, int ph, int pw, int x_nhwc, int y_nhwc) {
    const int Ho = (H + 2 * ph - KH) / sh + 1, Wo = (W + 2 * pw - KW) / sw + 1;
    for (long n = 0; n < N; ++n)
        for (long k = 0; k < Cout; ++k)
            for (long ho = 0; ho < Ho; ++ho)
                for (long wo = 0; wo < Wo; ++wo) {
                    double acc = 0.0;
                    for (long c = 0; c < Cin; ++c)
                        for (long r = 0; r < KH; ++r) {
                            const long hi = ho * sh - ph + r;
                            if (hi < 0 || hi >= H) continue;
                            for (long s = 0; s < KW; ++s) {
                                const long wi = wo * sw - pw + s;
                                if (wi < 0 || wi >= W) continue;
                                acc += (double)x[xidx(x_nhwc, n, c, hi, wi, Cin, H, W)] *
                                       (double)w[((k * Cin + c) * KH + r) * KW + s];
                            }
                        }
                    y[xidx(y_nhwc, n, k, ho, wo, Cout, Ho, Wo)] = (float)acc;
                }
}

/* y = (x - mean) / sqrt(var + eps) * gamma + beta, per channel */
void ref_bn(const float* x, float* y, const float* gamma, const float* beta, const float* mean, const float* var,
            double eps, long rows, int C, long hw, int nhwc, int relu) {
    const long n = rows * C;
    for (long i = 0; i < n; ++i) {
        const long c = nhwc ? i % C : (i / hw) % C;
        double v = ((double)x[i] - (double)mean[c]) / sqrt((double)var[c] + eps) * (double)gamma[c] + (double)beta[c];
        if (relu && v < 0.0) v = 0.0;
        y[i] = (float)v;
    }
}

void ref_layernorm(const float* x, const float* res, const float* gamma, const float* beta, float* y, long rows,
                   int width, double eps) {
    for (long r = 0; r < rows; ++r) {
        double mean = 0.0, var = 0.0;
        for (int c = 0; c < width; ++c) mean += (double)x[r * width + c] + (res ? (double)res[r * width + c] : 0.0);
        mean /= width;
        for (int c = 0; c < width; ++c) {
            const double d = (double)x[r * width + c] + (res ? (double)res[r * width + c] : 0.0) - mean;
            var += d * d;
        }
        var /= width;
        const double rstd = 1.0 / sqrt(var + eps);
        for (int c = 0; c < width; ++c) {
            const double v = (double)x[r * width + c] + (res ? (double)res[r * width + c] : 0.0);
            y[r * width + c] = (float)((v - mean) * rstd * (double)gamma[c] + (double)beta[c]);
        }
    }
}

void ref_softmax(const float* x, const float* mask, float* y, long rows, int width, double scale,
                 long rows_per_mask) {
    for (long r = 0; r < rows; ++r) {
        const float* m = mask ? mask + (r / rows_per_mask) * width : NULL;
        double mx = -INFINITY, s = 0.0;
        for (int c = 0; c < width; ++c) {
            const double v = (double)x[r * width + c] * scale + (m ? (double)m[c] : 0.0);
            if (v > mx) mx = v;
        }
        for (int c = 0; c < width; ++c)
            s += exp((double)x[r * width + c] * scale + (m ? (double)m[c] : 0.0) - mx);
        for (int c = 0; c < width; ++c)
            y[r * width + c] = (float)(exp((double)x[r * width + c] * scale + (m ? (double)m[c] : 0.0) - mx) / s);
    }
}

void ref_gelu(const float* x, float* y, long n) {
    for (long i = 0; i < n; ++i) y[i] = (float)(0.5 * (double)x[i] * (1.0 + erf((double)x[i] / sqrt(2.0))));
}

void ref_maxpool(const float* x, float* y, int N, int H, int W, int C, int k, int stride, int pad, int nhwc) {
    const int Ho = (H + 2 * pad - k) / stride + 1, Wo = (W + 2 * pad - k) / stride + 1;
    for (long n = 0; n < N; ++n)
        for (long c = 0; c < C; ++c)
            for (long ho = 0; ho < Ho; ++ho)
                for (long wo = 0; wo < Wo; ++wo) {
                    float m = -INFINITY;
                    for (int r = 0; r < k; ++r)
                        for (int s = 0; s < k; ++s) {
                            const long hi = ho * stride - pad + r, wi = wo * stride - pad + s;
                            if (hi < 0 || hi >= H || wi < 0 || wi >= W) continue;
                            const float v = x[xidx(nhwc, n, c, hi, wi, C, H, W)];
                            if (v > m) m = v;
                        }
                    y[xidx(nhwc, n, c, ho, wo, C, Ho, Wo)] = m;
                }
}

void ref_avgpool(const float* x, float* y, int N, int HW, int C, int nhwc) {
    for (long n = 0; n < N; ++n)
        for (long c = 0; c < C; ++c) {
            double s = 0.0;
            for (long j = 0; j < HW; ++j) s += (double)(nhwc ? x[(n * HW + j) * C + c] : x[(n * C + c) * HW + j]);
            y[n * C + c] = (float)(s / HW);
        }
}

void ref_embedding(const int64_t* ids, const int64_t* type_ids, const float* word, const float* pos,
                   const float* type, float* y, long tokens, int seq, int width) {
    for (long t = 0; t < tokens; ++t)
        for (int c = 0; c < width; ++c) {
            double v = word[ids[t] * width + c];
            if (pos) v += pos[(t % seq) * width + c];
            if (type) v += type[(type_ids ? type_ids[t] : 0) * width + c];
            y[t * width + c] = (float)v;
        }
}
