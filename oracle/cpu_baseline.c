/*
 * fp32 multi-threaded CPU restatement of TurboFNO's library baseline (variant E), used ONLY as the
 * timed "cpu_baseline" leg of the benchmark and cross-checked against the fp64 oracle in tests/.
 * THIS FILE IS TEST/BENCHMARK INFRASTRUCTURE; the product path never links or calls it.
 *
 * The reference has no CPU implementation of this path; this follows the five steps of
 *   fusion_variants/1D_E_baseline/fused.cu:178-190   (FFT, truncation copy, CGEMM, zero-pad copy, FFT)
 *   fusion_variants/2D_E_baseline/fused_trunc_2D.cu:200-227 (same with a rank-2 transform)
 * with full-length transforms followed by explicit truncation / zero-padding copies, exactly as the
 * baseline does, in complex64 arithmetic, OpenMP-parallel over signals/images and GEMM columns.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <omp.h>

#define MODES 64

typedef struct { float re, im; } c32;

static c32 *make_tw(int D, int sign)
{
    c32 *tw = (c32 *)malloc(sizeof(c32) * (size_t)(D / 2 > 0 ? D / 2 : 1));
    for (int t = 0; t < D / 2; ++t) {
        double a = sign * 6.283185307179586476925286766559 * t / D;
        tw[t].re = (float)cos(a); tw[t].im = (float)sin(a);
    }
    return tw;
}

static void fft32(c32 *a, long stride, int D, const c32 *tw)
{
    for (int i = 1, j = 0; i < D; ++i) {
        int bit = D >> 1;
        for (; j & bit; bit >>= 1) j ^= bit;
        j ^= bit;
        if (i < j) { c32 t = a[i * stride]; a[i * stride] = a[j * stride]; a[j * stride] = t; }
    }
    for (int len = 2; len <= D; len <<= 1) {
        int step = D / len, half = len / 2;
        for (int i = 0; i < D; i += len)
            for (int t = 0; t < half; ++t) {
                c32 w = tw[t * step];
                c32 *pu = a + (long)(i + t) * stride, *pv = a + (long)(i + t + half) * stride;
                float vr = pv->re * w.re - pv->im * w.im, vi = pv->re * w.im + pv->im * w.re;
                float ur = pu->re, ui = pu->im;
                pu->re = ur + vr; pu->im = ui + vi;
                pv->re = ur - vr; pv->im = ui - vi;
            }
    }
}

static void cgemm32(const c32 *A, const c32 *W, c32 *C, long M, int N, int K, c32 alpha)
{
#pragma omp parallel for schedule(static)
    for (long mb = 0; mb < M; mb += 256) {
        long me = mb + 256 < M ? mb + 256 : M;
        for (int n = 0; n < N; ++n) {
            float accr[256], acci[256];
            for (long m = mb; m < me; ++m) { accr[m - mb] = 0.f; acci[m - mb] = 0.f; }
            for (int k = 0; k < K; ++k) {
                c32 w = W[k + (long)n * K];
                const c32 *a = A + (long)k * M;
                for (long m = mb; m < me; ++m) {
                    accr[m - mb] += a[m].re * w.re - a[m].im * w.im;
                    acci[m - mb] += a[m].re * w.im + a[m].im * w.re;
                }
            }
            for (long m = mb; m < me; ++m) {
                C[m + (long)n * M].re = accr[m - mb] * alpha.re - acci[m - mb] * alpha.im;
                C[m + (long)n * M].im = accr[m - mb] * alpha.im + acci[m - mb] * alpha.re;
            }
        }
    }
}

/* 1D: x[K][S][DY] -> y[N][S][DY].  work: caller-provided scratch of >= max(K,N)*S*DY complex64. */
void cpu_baseline_layer_1d(const float *x, const float *W, float *y, long S, int DY, int K, int N,
                           float alpha_re, float alpha_im, int nthreads)
{
    if (nthreads > 0) omp_set_num_threads(nthreads);
    long M = MODES * S;
    c32 *spec = (c32 *)malloc(sizeof(c32) * (size_t)((K > N ? K : N) * S * DY));
    c32 *A = (c32 *)malloc(sizeof(c32) * (size_t)(M * K));
    c32 *C = (c32 *)malloc(sizeof(c32) * (size_t)(M * N));
    c32 *twf = make_tw(DY, -1), *twb = make_tw(DY, +1);
    c32 alpha = { alpha_re, alpha_im };
    memcpy(spec, x, sizeof(c32) * (size_t)(K * S * DY));
#pragma omp parallel for schedule(static)
    for (long s = 0; s < (long)K * S; ++s) fft32(spec + s * DY, 1, DY, twf);      /* step 1: forward FFT  */
#pragma omp parallel for schedule(static)
    for (long s = 0; s < (long)K * S; ++s)                                         /* step 2: truncation   */
        memcpy(A + s * MODES, spec + s * DY, sizeof(c32) * MODES);
    cgemm32(A, (const c32 *)W, C, M, N, K, alpha);                                 /* step 3: CGEMM        */
    c32 *out = (c32 *)y;
#pragma omp parallel for schedule(static)
    for (long s = 0; s < (long)N * S; ++s) {                                       /* step 4: zero padding */
        memcpy(out + s * DY, C + s * MODES, sizeof(c32) * MODES);
        memset(out + s * DY + MODES, 0, sizeof(c32) * (size_t)(DY - MODES));
    }
#pragma omp parallel for schedule(static)
    for (long s = 0; s < (long)N * S; ++s) fft32(out + s * DY, 1, DY, twb);       /* step 5: backward FFT */
    free(spec); free(A); free(C); free(twf); free(twb);
}

static void fft2d32(c32 *img, int DX, int DY, const c32 *twx, const c32 *twy)
{
    for (int r = 0; r < DX; ++r) fft32(img + (long)r * DY, 1, DY, twy);
    for (int c = 0; c < DY; ++c) fft32(img + c, DY, DX, twx);
}

/* 2D: x[K][bs][DX][DY] -> y[N][bs][DX][DY]. */
void cpu_baseline_layer_2d(const float *x, const float *W, float *y, int bs, int DX, int DY, int K, int N,
                           float alpha_re, float alpha_im, int nthreads)
{
    if (nthreads > 0) omp_set_num_threads(nthreads);
    long img = (long)DX * DY, M = (long)bs * MODES * MODES;
    c32 *spec = (c32 *)malloc(sizeof(c32) * (size_t)((long)K * bs * img));
    c32 *A = (c32 *)malloc(sizeof(c32) * (size_t)(M * K));
    c32 *C = (c32 *)malloc(sizeof(c32) * (size_t)(M * N));
    c32 *twxf = make_tw(DX, -1), *twyf = make_tw(DY, -1), *twxb = make_tw(DX, +1), *twyb = make_tw(DY, +1);
    c32 alpha = { alpha_re, alpha_im };
    memcpy(spec, x, sizeof(c32) * (size_t)((long)K * bs * img));
#pragma omp parallel for schedule(dynamic)
    for (long i = 0; i < (long)K * bs; ++i) fft2d32(spec + i * img, DX, DY, twxf, twyf);   /* step 1 */
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)K * bs; ++i)                                                 /* step 2 */
        for (int p = 0; p < MODES; ++p)
            memcpy(A + (i * MODES + p) * MODES, spec + i * img + (long)p * DY, sizeof(c32) * MODES);
    cgemm32(A, (const c32 *)W, C, M, N, K, alpha);                                          /* step 3 */
    c32 *out = (c32 *)y;
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)N * bs; ++i) {                                               /* step 4 */
        memset(out + i * img, 0, sizeof(c32) * (size_t)img);
        for (int p = 0; p < MODES; ++p)
            memcpy(out + i * img + (long)p * DY, C + (i * MODES + p) * MODES, sizeof(c32) * MODES);
    }
#pragma omp parallel for schedule(dynamic)
    for (long i = 0; i < (long)N * bs; ++i) fft2d32(out + i * img, DX, DY, twxb, twyb);     /* step 5 */
    free(spec); free(A); free(C); free(twxf); free(twyf); free(twxb); free(twyb);
}

int cpu_baseline_max_threads(void) { return omp_get_max_threads(); }
