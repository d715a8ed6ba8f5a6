/*
 * CPU oracle for the gputorch/gpunn convolution hot path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, in plain C, the
 * arithmetic of the reference CPU nn path so that the HIP library can be
 * checked against it and so that a CPU baseline can be timed beside the GPU.
 * Only tests, the smoke check and the cpu_baseline leg of the benchmark may
 * load it; the product library never links or calls anything in this file.
 *
 * Every function names the reference lines it follows (paths relative to the
 * reference tree).  Summation orders are kept exactly where the reference
 * fixes them (col2im, gradBias, max-pool backward, the TH fallback gemm).
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   im2col / col2im / conv fwd+bwd stride 1 with padding, and the strided conv:
 *       known answers recorded from the reference's own compiled C
 *       (tests/golden/reference_kat.json), brute force over the closed-form
 *       index map, the adjoint identity <im2col x, y> = <x, col2im y>,
 *       torch.nn.functional.conv2d + autograd on the CPU.
 *   sgemm fallback loops: float64 numpy product, exact small-integer matrices,
 *       all four transpose variants with ragged leading dimensions.
 *   sgemv / sger fallback loops (the classifier's addmv / addr): float64 numpy
 *       products, exact small-integer cases, both gemv orientations.
 *   max-pool fwd/bwd: reference known answers with overlapping windows and
 *       ties, brute force, torch max_pool2d(return_indices=True).
 *   threshold: closed form.
 *   The summation order of an external BLAS sgemm_ (the reference's USE_BLAS
 *   build, TH/generic/THBlas.c:300-317) is not fixed by the reference: the
 *   BLAS-backed variant is used only as the timed CPU baseline and is compared
 *   with the fallback loops by tolerance, never bit for bit.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

typedef void (*sgemm_fn)(const char *, const char *, const int *, const int *, const int *,
                         const float *, const float *, const int *, const float *, const int *,
                         const float *, float *, const int *);

/* Optional external BLAS (Fortran sgemm_ ABI).  NULL selects the TH fallback
 * loops, which is what the parity tests use. */
static sgemm_fn g_blas_sgemm = NULL;
typedef void (*set_threads_fn)(int);
static set_threads_fn g_blas_set_threads = NULL;
static int g_threads = 0; /* 0 = OpenMP default */

void oracle_set_blas(void *sgemm_symbol, void *set_threads_symbol)
{
    g_blas_sgemm = (sgemm_fn)sgemm_symbol;
    g_blas_set_threads = (set_threads_fn)set_threads_symbol;
}

void oracle_set_threads(int n) { g_threads = n; }

int oracle_get_threads(void)
{
#ifdef _OPENMP
    return g_threads > 0 ? g_threads : omp_get_max_threads();
#else
    return 1;
#endif
}

static int nthreads(void) { return oracle_get_threads(); }

static void blas_threads(int n)
{
    if (g_blas_set_threads) g_blas_set_threads(n);
}

/* ------------------------------------------------------------------------- */
/* Column-major C = beta*C + alpha*op(A)*op(B), the TH fallback loops:
 * TH/generic/THBlas.c:270-389.  One float accumulator per output, reduction
 * index ascending, then beta*c + alpha*sum (THBlas.c:333,349,365,381).  The
 * leading-dimension fix-ups for degenerate shapes are THBlas.c:275-298.  With
 * beta == 0 the old C is not read (BLAS semantics; the fallback would multiply
 * whatever was there by zero). */
static void sgemm_loops(char transa, char transb, long m, long n, long k, float alpha,
                        const float *a, long lda, const float *b, long ldb, float beta,
                        float *c, long ldc)
{
    int ta = (transa == 't' || transa == 'T');
    int tb = (transb == 't' || transb == 'T');
    long i, j, l;
    for (j = 0; j < n; j++) {
        for (i = 0; i < m; i++) {
            float sum = 0;
            for (l = 0; l < k; l++) {
                float av = ta ? a[i * lda + l] : a[l * lda + i];
                float bv = tb ? b[l * ldb + j] : b[j * ldb + l];
                sum += av * bv;
            }
            if (beta == 0)
                c[j * ldc + i] = alpha * sum;
            else
                c[j * ldc + i] = beta * c[j * ldc + i] + alpha * sum;
        }
    }
}

void oracle_sgemm(char transa, char transb, long m, long n, long k, float alpha,
                  const float *a, long lda, const float *b, long ldb, float beta,
                  float *c, long ldc)
{
    int ta = (transa == 't' || transa == 'T');
    int tb = (transb == 't' || transb == 'T');
    if (n == 1) ldc = m;
    if (ta) { if (m == 1) lda = k; } else { if (k == 1) lda = m; }
    if (tb) { if (k == 1) ldb = n; } else { if (n == 1) ldb = k; }

    if (g_blas_sgemm) {
        int im = (int)m, in = (int)n, ik = (int)k, ilda = (int)lda, ildb = (int)ldb, ildc = (int)ldc;
        g_blas_sgemm(&transa, &transb, &im, &in, &ik, &alpha, a, &ilda, b, &ildb, &beta, c, &ildc);
        return;
    }
    sgemm_loops(transa, transb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
}

/* ------------------------------------------------------------------------- */
/* Column-major y = beta*y + alpha*op(A)*x, the TH fallback loops:
 * TH/generic/THBlas.c:181-235.  't': one float accumulator per output, j
 * ascending, then beta*y + alpha*sum (:214-222); 'n': y scaled by beta first
 * unless beta == 1, then columns added j ascending with z = alpha*x[j]
 * (:225-234). */
void oracle_sgemv(char trans, long m, long n, float alpha, const float *a, long lda,
                  const float *x, long incx, float beta, float *y, long incy)
{
    long i, j;
    if (n == 1) lda = m;
    if (trans == 't' || trans == 'T') {
        for (i = 0; i < n; i++) {
            float sum = 0;
            const float *row_ = a + lda * i;
            for (j = 0; j < m; j++) sum += x[j * incx] * row_[j];
            y[i * incy] = beta * y[i * incy] + alpha * sum;
        }
    } else {
        if (beta != 1)
            for (i = 0; i < m; i++) y[i * incy] *= beta;
        for (j = 0; j < n; j++) {
            const float *column_ = a + lda * j;
            float z = alpha * x[j * incx];
            for (i = 0; i < m; i++) y[i * incy] += z * column_[i];
        }
    }
}

/* Column-major A += alpha * x * y^T, the TH fallback loops:
 * TH/generic/THBlas.c:237-268 (z = alpha*y[j], then column_[i] += z*x[i]). */
void oracle_sger(long m, long n, float alpha, const float *x, long incx, const float *y,
                 long incy, float *a, long lda)
{
    long i, j;
    if (n == 1) lda = m;
    for (j = 0; j < n; j++) {
        float *column_ = a + j * lda;
        float z = alpha * y[j * incy];
        for (i = 0; i < m; i++) column_[i] += z * x[i * incx];
    }
}

/* ------------------------------------------------------------------------- */
/* im2col for one image: mcw_nn/generic/SpatialConvolutionMM.c:52-96
 * (unfolded_copy: row k = (c*kH+kh)*kW+kw, memcpy of the valid span, zeros in
 * the padding), generalised to separate strides and paddings with the index
 * map of gputorch/lib/THC/gpunn-impl/SpatialConvolutionMM.cpp:10-52:
 *   col[k][ho*Wo+wo] = im[c][ho*sH-pH+kh][wo*sW-pW+kw]   or +0.0f outside. */
static void im2col_frame(const float *im, int C, int H, int W, int kH, int kW, int pH, int pW,
                         int sH, int sW, int Ho, int Wo, float *col)
{
    long k, K = (long)C * kH * kW;
    for (k = 0; k < K; k++) {
        int c = (int)(k / (kH * kW));
        int rest = (int)(k % (kH * kW));
        int kh = rest / kW, kw = rest % kW;
        float *dst = col + k * (long)Ho * Wo;
        const float *src = im + (long)c * H * W;
        int ho, wo;
        for (ho = 0; ho < Ho; ho++) {
            int iy = ho * sH - pH + kh;
            float *row = dst + (long)ho * Wo;
            if (iy < 0 || iy >= H) {
                memset(row, 0, sizeof(float) * Wo);
                continue;
            }
            if (sW == 1) {
                /* valid wo range: 0 <= wo - pW + kw < W */
                int lo = pW - kw; if (lo < 0) lo = 0;
                int hi = W + pW - kw; if (hi > Wo) hi = Wo;
                if (hi < lo) hi = lo;
                if (lo > 0) memset(row, 0, sizeof(float) * lo);
                memcpy(row + lo, src + (long)iy * W + (lo - pW + kw), sizeof(float) * (hi - lo));
                if (hi < Wo) memset(row + hi, 0, sizeof(float) * (Wo - hi));
            } else {
                for (wo = 0; wo < Wo; wo++) {
                    int ix = wo * sW - pW + kw;
                    row[wo] = (ix >= 0 && ix < W) ? src[(long)iy * W + ix] : 0.0f;
                }
            }
        }
    }
}

/* col2im for one image: mcw_nn/generic/SpatialConvolutionMM.c:6-50
 * (unfolded_acc) after the zeroing at :220.  The image starts at 0 and every
 * pixel receives its contributions in the order kh ascending, then kw
 * ascending -- the order a bit-exact device gather has to reproduce.
 * Generalised to strides/paddings like im2col_frame. */
static void col2im_frame(const float *col, int C, int H, int W, int kH, int kW, int pH, int pW,
                         int sH, int sW, int Ho, int Wo, float *im)
{
    int c, kh, kw, ho, wo;
    memset(im, 0, sizeof(float) * (size_t)C * H * W);
    for (c = 0; c < C; c++) {
        float *dst = im + (long)c * H * W;
        for (kh = 0; kh < kH; kh++) {
            for (kw = 0; kw < kW; kw++) {
                const float *src = col + (((long)c * kH + kh) * kW + kw) * Ho * Wo;
                for (ho = 0; ho < Ho; ho++) {
                    int iy = ho * sH - pH + kh;
                    if (iy < 0 || iy >= H) continue;
                    for (wo = 0; wo < Wo; wo++) {
                        int ix = wo * sW - pW + kw;
                        if (ix < 0 || ix >= W) continue;
                        dst[(long)iy * W + ix] += src[(long)ho * Wo + wo];
                    }
                }
            }
        }
    }
}

void oracle_im2col(const float *im, long B, int C, int H, int W, int kH, int kW, int pH, int pW,
                   int sH, int sW, float *col)
{
    int Ho = (H + 2 * pH - kH) / sH + 1, Wo = (W + 2 * pW - kW) / sW + 1;
    long K = (long)C * kH * kW, N = (long)Ho * Wo, b;
#pragma omp parallel for num_threads(nthreads())
    for (b = 0; b < B; b++)
        im2col_frame(im + b * (long)C * H * W, C, H, W, kH, kW, pH, pW, sH, sW, Ho, Wo, col + b * K * N);
}

void oracle_col2im(const float *col, long B, int C, int H, int W, int kH, int kW, int pH, int pW,
                   int sH, int sW, float *im)
{
    int Ho = (H + 2 * pH - kH) / sH + 1, Wo = (W + 2 * pW - kW) / sW + 1;
    long K = (long)C * kH * kW, N = (long)Ho * Wo, b;
#pragma omp parallel for num_threads(nthreads())
    for (b = 0; b < B; b++)
        col2im_frame(col + b * K * N, C, H, W, kH, kW, pH, pW, sH, sW, Ho, Wo, im + b * (long)C * H * W);
}

/* ------------------------------------------------------------------------- */
/* nn.SpatialConvolutionMM forward, batch mode:
 * mcw_nn/generic/SpatialConvolutionMM.c:120-208 (OpenMP over the batch at
 * :186) calling the frame at :98-118: unfolded_copy, bias fill of every output
 * plane (:112-113), then output2d = 1*output2d + 1*weight*finput (:115), i.e.
 * in column-major BLAS terms gemm('n','n', N, M, K, 1, finput, N, weight, K,
 * 1, output, N) (TH/generic/THTensorMath.c:458-561).
 * finput is [B, K, N] and is kept for accGradParameters (:179). */
void oracle_conv_updateOutput(const float *input, long B, int C, int H, int W,
                              const float *weight, const float *bias, int M,
                              int kH, int kW, int pH, int pW, int sH, int sW,
                              float *finput, float *output)
{
    int Ho = (H + 2 * pH - kH) / sH + 1, Wo = (W + 2 * pW - kW) / sW + 1;
    long K = (long)C * kH * kW, N = (long)Ho * Wo, b;
    blas_threads(1);
#pragma omp parallel for num_threads(nthreads())
    for (b = 0; b < B; b++) {
        float *col = finput + b * K * N;
        float *out = output + b * (long)M * N;
        long m, n;
        im2col_frame(input + b * (long)C * H * W, C, H, W, kH, kW, pH, pW, sH, sW, Ho, Wo, col);
        for (m = 0; m < M; m++)
            for (n = 0; n < N; n++) out[m * N + n] = bias[m];
        oracle_sgemm('n', 'n', N, M, K, 1.0f, col, N, weight, K, 1.0f, out, N);
    }
}

/* nn.SpatialConvolutionMM gradInput: mcw_nn/generic/SpatialConvolutionMM.c:
 * 225-282 (weight transposed at :245, OpenMP over the batch at :260) calling
 * the frame at :211-223: fgradInput = weight^T * gradOutput2d with beta 0
 * (:217), zero gradInput (:220), unfolded_acc.  Column-major:
 * gemm('n','t', N, K, M, 1, gradOutput, N, weight, K, 0, fgradInput, N). */
void oracle_conv_updateGradInput(const float *gradOutput, long B, int C, int H, int W,
                                 const float *weight, int M,
                                 int kH, int kW, int pH, int pW, int sH, int sW,
                                 float *fgradInput, float *gradInput)
{
    int Ho = (H + 2 * pH - kH) / sH + 1, Wo = (W + 2 * pW - kW) / sW + 1;
    long K = (long)C * kH * kW, N = (long)Ho * Wo, b;
    blas_threads(1);
#pragma omp parallel for num_threads(nthreads())
    for (b = 0; b < B; b++) {
        float *gcol = fgradInput + b * K * N;
        oracle_sgemm('n', 't', N, K, M, 1.0f, gradOutput + b * (long)M * N, N, weight, K, 0.0f, gcol, N);
        col2im_frame(gcol, C, H, W, kH, kW, pH, pW, sH, sW, Ho, Wo, gradInput + b * (long)C * H * W);
    }
}

/* nn.SpatialConvolutionMM accGradParameters: mcw_nn/generic/
 * SpatialConvolutionMM.c:311-346 -- a SEQUENTIAL loop over the batch (:333)
 * calling the frame at :284-309: gradWeight = 1*gradWeight + scale *
 * gradOutput2d * finput^T (:293-295; column-major gemm('t','n', K, M, N, scale,
 * finput, N, gradOutput, N, 1, gradWeight, K)), then per output plane a float
 * sum over n ascending and gradBias[m] += scale*sum (:297-305).  finput is the
 * forward's column buffer; nothing is recomputed. */
void oracle_conv_accGradParameters(const float *gradOutput, const float *finput, long B,
                                   int M, long K, long N, float scale,
                                   float *gradWeight, float *gradBias)
{
    long b, m, n;
    blas_threads(nthreads());
    for (b = 0; b < B; b++) {
        const float *go = gradOutput + b * (long)M * N;
        oracle_sgemm('t', 'n', K, M, N, scale, finput + b * K * N, N, go, N, 1.0f, gradWeight, K);
        for (m = 0; m < M; m++) {
            float sum = 0;
            for (n = 0; n < N; n++) sum += go[m * N + n];
            gradBias[m] += scale * sum;
        }
    }
    blas_threads(1);
}

/* ------------------------------------------------------------------------- */
/* nn.SpatialMaxPooling forward: mcw_nn/generic/SpatialMaxPooling.c:5-56 (frame)
 * and :58-145 (driver, OpenMP over batch :130 and planes :13).  Ho = (H-kH)/dH
 * + 1 (:94-95).  The window is scanned ky ascending, kx ascending with a strict
 * '>' against a running maximum that starts at -inf (:30-45), so the first
 * maximum wins ties.  indices is [2,B,C,Ho,Wo] stored as floats: plane 0 holds
 * ky+1, plane 1 holds kx+1 (:51-52 with the pointer arithmetic of :133-134). */
void oracle_maxpool_updateOutput(const float *input, long B, int C, int H, int W,
                                 int kH, int kW, int dH, int dW,
                                 float *output, float *indices)
{
    int Ho = (H - kH) / dH + 1, Wo = (W - kW) / dW + 1;
    long planes = B * C, p;
    float *indy = indices, *indx = indices + planes * Ho * Wo;
#pragma omp parallel for num_threads(nthreads())
    for (p = 0; p < planes; p++) {
        const float *ip = input + p * (long)H * W;
        int i, j, y, x;
        for (i = 0; i < Ho; i++) {
            for (j = 0; j < Wo; j++) {
                const float *win = ip + (long)i * dH * W + (long)j * dW;
                long maxindex = -1, t = 0;
                float maxval = -INFINITY;
                for (y = 0; y < kH; y++)
                    for (x = 0; x < kW; x++, t++) {
                        float v = win[(long)y * W + x];
                        if (v > maxval) { maxval = v; maxindex = t; }
                    }
                long o = p * (long)Ho * Wo + (long)i * Wo + j;
                output[o] = maxval;
                indy[o] = (float)((int)(maxindex / kW) + 1);
                indx[o] = (float)((maxindex % kW) + 1);
            }
        }
    }
}

/* nn.SpatialMaxPooling backward: mcw_nn/generic/SpatialMaxPooling.c:147-178
 * (frame) and :180-254 (driver: zero gradInput :203, OpenMP over batch :238 and
 * planes :155).  Within a plane the windows are visited i ascending, j
 * ascending and gradInput[argmax] += gradOutput (:165-174), which fixes the
 * float addition order when windows overlap. */
void oracle_maxpool_updateGradInput(const float *gradOutput, const float *indices, long B, int C,
                                    int H, int W, int Ho, int Wo, int dH, int dW,
                                    float *gradInput)
{
    long planes = B * C, p;
    const float *indy = indices, *indx = indices + planes * Ho * Wo;
    memset(gradInput, 0, sizeof(float) * (size_t)planes * H * W);
#pragma omp parallel for num_threads(nthreads())
    for (p = 0; p < planes; p++) {
        float *gi = gradInput + p * (long)H * W;
        long o = p * (long)Ho * Wo;
        int i, j;
        for (i = 0; i < Ho; i++)
            for (j = 0; j < Wo; j++) {
                long maxi = (long)indy[o + (long)i * Wo + j] - 1 + (long)i * dH;
                long maxj = (long)indx[o + (long)i * Wo + j] - 1 + (long)j * dW;
                gi[maxi * W + maxj] += gradOutput[o + (long)i * Wo + j];
            }
    }
}

/* ------------------------------------------------------------------------- */
/* nn.SpatialSubSampling and nn.SpatialAveragePooling.
 * forward: mcw_nn/generic/SpatialSubSampling.c:58-96 -- the output plane is
 * filled with bias[k] (:70-74), then every window adds weight[k] * sum, the sum
 * taken ky ascending, kx ascending from zero (:82-92).  SpatialAveragePooling
 * (mcw_nn/generic/SpatialAveragePooling.c:56-90) is the same loop with a zero
 * fill and no weight: it returns the window SUM, there is no division.
 * weight == NULL selects the average-pooling form. */
void oracle_subsample_updateOutput(const float *input, const float *weight, const float *bias, long B, int C,
                                   int H, int W, int kH, int kW, int dH, int dW, float *output)
{
    int Ho = (H - kH) / dH + 1, Wo = (W - kW) / dW + 1;
    long planes = B * C, p;
#pragma omp parallel for num_threads(nthreads())
    for (p = 0; p < planes; p++) {
        int k = (int)(p % C), yy, xx, ky, kx;
        const float *ip = input + p * (long)H * W;
        float *op = output + p * (long)Ho * Wo;
        float z = weight ? bias[k] : 0.0f;
        for (yy = 0; yy < Ho * Wo; yy++) op[yy] = z;
        for (yy = 0; yy < Ho; yy++)
            for (xx = 0; xx < Wo; xx++) {
                const float *win = ip + (long)yy * dH * W + (long)xx * dW;
                float sum = 0;
                for (ky = 0; ky < kH; ky++) {
                    for (kx = 0; kx < kW; kx++) sum += win[kx];
                    win += W;
                }
                if (weight) *op++ += weight[k] * sum;
                else *op++ += sum;
            }
    }
}

/* backward: SpatialSubSampling.c:151-181 / SpatialAveragePooling.c:142-171 --
 * gradInput is zeroed, then every window (yy ascending, xx ascending) adds
 * z = gradOutput * weight[k] (or gradOutput alone) to each of its pixels. */
void oracle_subsample_updateGradInput(const float *gradOutput, const float *weight, long B, int C, int H, int W,
                                      int kH, int kW, int dH, int dW, float *gradInput)
{
    int Ho = (H - kH) / dH + 1, Wo = (W - kW) / dW + 1;
    long planes = B * C, p;
#pragma omp parallel for num_threads(nthreads())
    for (p = 0; p < planes; p++) {
        int k = (int)(p % C), yy, xx, ky, kx;
        float *gi = gradInput + p * (long)H * W;
        const float *go = gradOutput + p * (long)Ho * Wo;
        for (yy = 0; yy < H * W; yy++) gi[yy] = 0.0f;
        for (yy = 0; yy < Ho; yy++)
            for (xx = 0; xx < Wo; xx++) {
                float *win = gi + (long)yy * dH * W + (long)xx * dW;
                float z = weight ? *go++ * weight[k] : *go++;
                for (ky = 0; ky < kH; ky++) {
                    for (kx = 0; kx < kW; kx++) win[kx] += z;
                    win += W;
                }
            }
    }
}

/* accGradParameters: SpatialSubSampling.c:236-270 -- per plane, image after
 * image: gradBias[k] += scale * (sum of the gradOutput plane), gradWeight[k] +=
 * scale * (sum over windows and taps of gradOutput * input), all in float. */
void oracle_subsample_accGradParameters(const float *input, const float *gradOutput, long B, int C, int H, int W,
                                        int kH, int kW, int dH, int dW, float scale, float *gradWeight,
                                        float *gradBias)
{
    int Ho = (H - kH) / dH + 1, Wo = (W - kW) / dW + 1, k;
#pragma omp parallel for num_threads(nthreads())
    for (k = 0; k < C; k++) {
        long b;
        for (b = 0; b < B; b++) {
            const float *go = gradOutput + (b * C + k) * (long)Ho * Wo;
            const float *ip = input + (b * C + k) * (long)H * W;
            float sum = 0;
            int i, yy, xx, ky, kx;
            for (i = 0; i < Ho * Wo; i++) sum += go[i];
            gradBias[k] += scale * sum;
            sum = 0;
            for (yy = 0; yy < Ho; yy++)
                for (xx = 0; xx < Wo; xx++) {
                    const float *win = ip + (long)yy * dH * W + (long)xx * dW;
                    float z = *go++;
                    for (ky = 0; ky < kH; ky++) {
                        for (kx = 0; kx < kW; kx++) sum += z * win[kx];
                        win += W;
                    }
                }
            gradWeight[k] += scale * sum;
        }
    }
}

/* ------------------------------------------------------------------------- */
/* nn.LogSoftMax: mcw_nn/generic/LogSoftMax.c:37-53 (forward) and :85-97
 * (backward).  accreal is double for float tensors; the forward sum uses
 * THExpMinusApprox (mcw_torch7_core/lib/TH/THLogAdd.c:56-86), a polynomial
 * raised to the eighth power that is exactly zero from 13 on -- not exp. */
static double exp_minus_approx(double x)
{
    if (x < 13.0) {
        double y = 1.0 + x * (0.125 + x * (0.0078125 + x * (0.00032552083 + x * 1.0172526e-5)));
        y *= y;
        y *= y;
        y *= y;
        return 1 / y;
    }
    return 0;
}

void oracle_logsoftmax_updateOutput(const float *input, long nframe, long dim, float *output)
{
    long t;
#pragma omp parallel for num_threads(nthreads())
    for (t = 0; t < nframe; t++) {
        const float *in = input + dim * t;
        float *out = output + dim * t;
        double logsum = 0;
        float maxInput = -INFINITY;
        long d;
        for (d = 0; d < dim; d++) maxInput = maxInput > in[d] ? maxInput : in[d];
        for (d = 0; d < dim; d++) logsum += exp_minus_approx(maxInput - in[d]);
        logsum = maxInput + log(logsum);
        for (d = 0; d < dim; d++) out[d] = in[d] - logsum;
    }
}

void oracle_logsoftmax_updateGradInput(const float *gradOutput, const float *output, long nframe, long dim,
                                       float *gradInput)
{
    long t;
#pragma omp parallel for num_threads(nthreads())
    for (t = 0; t < nframe; t++) {
        const float *go = gradOutput + dim * t, *out = output + dim * t;
        float *gi = gradInput + dim * t;
        double sum = 0;
        long d;
        for (d = 0; d < dim; d++) sum += go[d];
        for (d = 0; d < dim; d++) gi[d] = go[d] - exp(out[d]) * sum;
    }
}

/* ------------------------------------------------------------------------- */
/* nn.Threshold (nn.ReLU = Threshold(0,0), mcw_nn/ReLU.lua:1-5):
 * mcw_nn/generic/Threshold.c:5-32.  forward: x > threshold ? x : val;
 * backward uses the forward INPUT: x > threshold ? gradOutput : 0. */
void oracle_threshold_updateOutput(const float *input, long n, float threshold, float val, float *output)
{
    long i;
#pragma omp parallel for num_threads(nthreads())
    for (i = 0; i < n; i++) output[i] = (input[i] > threshold) ? input[i] : val;
}

void oracle_threshold_updateGradInput(const float *input, const float *gradOutput, long n,
                                      float threshold, float *gradInput)
{
    long i;
#pragma omp parallel for num_threads(nthreads())
    for (i = 0; i < n; i++) gradInput[i] = (input[i] > threshold) ? gradOutput[i] : 0.0f;
}
