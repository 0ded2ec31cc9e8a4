/*
 * cpu_emitted_bench.c -- TEST / BENCHMARK INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * The CPU call sequence that the reference's RModel::Generate emits for the fp32 configurations of the
 * benchmark, restated in plain C and timed on the host cores:
 *   mlp   Gemm 64->128 + ReLU, Gemm 128->64 + ReLU, Gemm 64->8 on a batch of 256
 *         per Gemm (ROperator_Gemm.hxx:360-381): std::copy(bias broadcast to [M,N] -> Y);
 *         BLAS::sgemm_(transB, transA, n, m, k, alpha, W, ldb, X, lda, beta = 1, Y, n); the ReLU loop
 *   gemm  one large Gemm + ReLU: `--images` rows of the 4096 x 4096 x 4096 product of the benchmark (same call sequence)
 *   conv  Conv 64->128, 56x56, 3x3, stride 1, pad 1, bias, then Relu (ROperator_Conv.hxx:342-518,
 *         ROperator_Relu.hxx:54-66): inside infer the weight re-layout loop into x_f; per image Im2col
 *         (SOFIE_common.hxx:485-518), BLAS::sgemm_('N','N', m = OH*OW, n = OC, k = C*KH*KW, 1, xcol, m, x_f, k, 0,
 *         Y + off, m), BLAS::saxpy_(OC*OH*OW, 1, bias broadcast to [OC,OH,OW], 1, Y + off, 1); then the Relu loop
 *   cnn   the classifier of the batch-4096 configuration in fp32, as the reference would emit it for the float model
 *         (it has no quantized operators): Conv 1->32 3x3 + Relu, MaxPool 2x2, Conv 32->64 + Relu, MaxPool, Conv 64->128 +
 *         Relu, Flatten (a view), Gemm 12800->256 + Relu, Gemm 256->5 on 1x40x40 images. Conv and Gemm as above; the
 *         MaxPool loop of ROperator_Pool.hxx:371-416 (for every batch*channel plane, rows hmin..hmax and columns
 *         wmin..wmax in steps of the stride, the maximum over the kh x kw window cells that lie inside the plane).
 * The FLOPs of the reference run in an external Fortran BLAS chosen when it is built (CMake find_package(BLAS));
 * here sgemm_ / saxpy_ are bound at run time with dlopen from the library named on the command line
 * (--blas PATH --prefix P: symbols P"sgemm_" and P"saxpy_"), and fall back to the loops of this file (the
 * textbook column-major definition) when none is given. The thread count is whatever the library takes from
 * its environment (OMP_NUM_THREADS, MKL_NUM_THREADS, OPENBLAS_NUM_THREADS): the caller sets it.
 *
 * --dump FILE writes the inputs, weights and the result as raw floats (a test compares them with the oracle).
 * Output: one JSON line {"workload", "blas", "calls", "median_ms", "best_ms", "checksum", "selfcheck"}; selfcheck
 * is the largest |difference| between the bound sgemm_ and the bundled loops on a small product (a library that
 * binds but computes something else is rejected by the caller).
 *
 * Build: gcc -O2 -o cpu_emitted_bench cpu_emitted_bench.c -ldl -lm   (see Makefile)
 */
#define _POSIX_C_SOURCE 200809L
#include <dlfcn.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

typedef void (*sgemm_fn)(const char *, const char *, const int *, const int *, const int *, const float *, const float *,
                         const int *, const float *, const int *, const float *, float *, const int *);
typedef void (*saxpy_fn)(const int *, const float *, const float *, const int *, float *, const int *);

/* column-major SGEMM, Fortran calling convention (the bundled fallback and the self-check's truth) */
static void loop_sgemm(const char *ta, const char *tb, const int *pm, const int *pn, const int *pk, const float *palpha,
                       const float *A, const int *plda, const float *B, const int *pldb, const float *pbeta, float *C,
                       const int *pldc)
{
    const int m = *pm, n = *pn, k = *pk, lda = *plda, ldb = *pldb, ldc = *pldc;
    const int tra = (*ta == 't' || *ta == 'T'), trb = (*tb == 't' || *tb == 'T');
    const float alpha = *palpha, beta = *pbeta;
    for (int j = 0; j < n; ++j) {
        float *cj = C + (size_t)j * ldc;
        for (int i = 0; i < m; ++i) cj[i] = beta == 0.0f ? 0.0f : beta * cj[i];
        for (int l = 0; l < k; ++l) {
            const float b = alpha * (trb ? B[(size_t)l * ldb + j] : B[(size_t)j * ldb + l]);
            if (!tra) {
                const float *al = A + (size_t)l * lda;
                for (int i = 0; i < m; ++i) cj[i] += b * al[i];
            } else {
                for (int i = 0; i < m; ++i) cj[i] += b * A[(size_t)i * lda + l];
            }
        }
    }
}

static void loop_saxpy(const int *pn, const float *pa, const float *x, const int *incx, float *y, const int *incy)
{
    for (int i = 0; i < *pn; ++i) y[(size_t)i * *incy] += *pa * x[(size_t)i * *incx];
}

static sgemm_fn g_sgemm = loop_sgemm;
static saxpy_fn g_saxpy = loop_saxpy;

static double now_ms(void)
{
    struct timespec t;
    clock_gettime(CLOCK_MONOTONIC, &t);
    return t.tv_sec * 1e3 + t.tv_nsec * 1e-6;
}

/* splitmix64: the seeded inputs need no library */
static unsigned long long g_state = 0x9E3779B97F4A7C15ull;
static double uniform01(void)
{
    unsigned long long z = (g_state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (double)(z >> 11) / 9007199254740992.0;
}
static double normal01(void)
{
    double u = uniform01(), v = uniform01();
    if (u < 1e-300) u = 1e-300;
    return sqrt(-2.0 * log(u)) * cos(6.283185307179586 * v);
}

static int cmp_double(const void *a, const void *b)
{
    const double x = *(const double *)a, y = *(const double *)b;
    return (x > y) - (x < y);
}

/* ------------------------------------------------------------------ Gemm, as ROperator_Gemm<float>::Generate emits it */
static void emitted_gemm(int m, int n, int k, const float *x, const float *w, const float *bias_bcast, float *y, int relu)
{
    /* row-major Y[m,n] = X[m,k] W[k,n] + bias, computed as the column-major product Y^T = W^T X^T */
    const char transA = 'n', transB = 'n';
    const float alpha = 1.0f, beta = 1.0f;
    const int lda = k, ldb = n;
    memcpy(y, bias_bcast, (size_t)m * n * sizeof(float));                   /* std::copy(tensor_Bbcast, ...) */
    g_sgemm(&transB, &transA, &n, &m, &k, &alpha, w, &ldb, x, &lda, &beta, y, &n);
    if (relu)
        for (int id = 0; id < m * n; id++) y[id] = ((y[id] > 0) ? y[id] : 0);
}

/* ------------------------------------------------------------------ Im2col of one image, zero fill outside */
static void im2col(const float *im, int C, int H, int W, int kh, int kw, int ph, int pw, int sh, int sw, float *col)
{
    const int OH = (H + 2 * ph - kh) / sh + 1, OW = (W + 2 * pw - kw) / sw + 1;
    size_t o = 0;
    for (int c = 0; c < C; ++c)
        for (int r = 0; r < kh; ++r)
            for (int s = 0; s < kw; ++s)
                for (int oh = 0; oh < OH; ++oh) {
                    const int ih = oh * sh - ph + r;
                    if (ih < 0 || ih >= H) {
                        for (int ow = 0; ow < OW; ++ow) col[o++] = 0.0f;
                        continue;
                    }
                    const float *row = im + ((size_t)c * H + ih) * W;
                    for (int ow = 0; ow < OW; ++ow) {
                        const int iw = ow * sw - pw + s;
                        col[o++] = (iw >= 0 && iw < W) ? row[iw] : 0.0f;
                    }
                }
}

/* ------------------------------------------------------------------ Conv + Relu, as the reference emits them */
static void emitted_conv_relu(int N, int C, int H, int W, int OC, int KH, int KW, int pad, int stride, const float *x,
                              const float *w, const float *bias_bcast, float *xf, float *xcol, float *y)
{
    const int OH = (H + 2 * pad - KH) / stride + 1, OW = (W + 2 * pad - KW) / stride + 1;
    /* the weight re-layout loop sits inside infer (ROperator_Conv.hxx:342-363) */
    for (int oc = 0; oc < OC; oc++)
        for (int ic = 0; ic < C; ic++)
            for (int kh = 0; kh < KH; kh++)
                for (int kw = 0; kw < KW; kw++)
                    xf[((size_t)oc * C + ic) * KH * KW + kh * KW + kw] = w[((size_t)oc * C + ic) * KH * KW + kh * KW + kw];
    const char transA = 'N', transB = 'N';
    int m = OH * OW, n = OC, k = C * KH * KW;
    const float alpha = 1.0f, beta = 0.0f;
    for (int img = 0; img < N; img++) {
        const size_t out_offset = (size_t)img * OC * m, x_offset = (size_t)img * C * H * W;
        im2col(x + x_offset, C, H, W, KH, KW, pad, pad, stride, stride, xcol);
        g_sgemm(&transA, &transB, &m, &n, &k, &alpha, xcol, &m, xf, &k, &beta, y + out_offset, &m);
        const int size = OC * m, inc = 1;
        const float gamma = 1.0f;
        g_saxpy(&size, &gamma, bias_bcast, &inc, y + out_offset, &inc);
    }
    const size_t len = (size_t)N * OC * m;
    for (size_t id = 0; id < len; id++) y[id] = ((y[id] > 0) ? y[id] : 0);
}

/* ------------------------------------------------------------------ MaxPool, as ROperator_Pool emits it for 2-D inputs */
static void emitted_maxpool(int planes, int hsize, int wsize, int kh, int kw, int pad, int sh, int sw, const float *x, float *y)
{
    /* hmin = -pad, hmax = hsize + pad - kh + 1 (ROperator_Pool.hxx:283-305) */
    const int hmin = -pad, hmax = hsize + pad - kh + 1, wmin = -pad, wmax = wsize + pad - kw + 1;
    size_t outIndex = 0;
    for (size_t n = 0; n < (size_t)planes; n++) {
        size_t inputOffset = n * (size_t)hsize * wsize;
        for (int i = hmin; i < hmax; i += sh) {
            for (int j = wmin; j < wmax; j += sw) {
                float value = -INFINITY;
                for (int l = i; l < i + kh; l++) {
                    if (l < 0 || l >= hsize) continue;
                    for (int m = j; m < j + kw; m++) {
                        if (m < 0 || m >= wsize) continue;
                        const float xval = x[inputOffset + (size_t)l * wsize + m];
                        if (xval > value) value = xval;
                    }
                }
                y[outIndex++] = value;
            }
        }
    }
}

static float *alloc_f(size_t n)
{
    float *p = (float *)malloc(n * sizeof(float));
    if (!p) { fprintf(stderr, "cpu_emitted_bench: out of memory (%zu floats)\n", n); exit(3); }
    return p;
}

static double selfcheck(void)
{
    enum { M = 37, N = 29, K = 53 };
    float *A = alloc_f(M * K), *B = alloc_f(K * N), *C1 = alloc_f(M * N), *C2 = alloc_f(M * N);
    for (int i = 0; i < M * K; ++i) A[i] = (float)normal01();
    for (int i = 0; i < K * N; ++i) B[i] = (float)normal01();
    for (int i = 0; i < M * N; ++i) C1[i] = C2[i] = (float)normal01();
    const char nn = 'n', tt = 't';
    const int m = M, n = N, k = K, lda = K, ldb = K;
    const float alpha = 0.75f, beta = 1.0f;
    /* op(A) = A^T with A stored [K x M] col-major lda = K; op(B) = B stored [K x N] */
    g_sgemm(&tt, &nn, &m, &n, &k, &alpha, A, &lda, B, &ldb, &beta, C1, &m);
    loop_sgemm(&tt, &nn, &m, &n, &k, &alpha, A, &lda, B, &ldb, &beta, C2, &m);
    double worst = 0;
    for (int i = 0; i < M * N; ++i) worst = fmax(worst, fabs((double)C1[i] - C2[i]));
    free(A); free(B); free(C1); free(C2);
    return worst;
}

int main(int argc, char **argv)
{
    const char *workload = "mlp", *blas = NULL, *prefix = "", *dump = NULL;
    int calls = 0, images = 64;
    for (int i = 1; i < argc; ++i) {
        if (!strcmp(argv[i], "--workload") && i + 1 < argc) workload = argv[++i];
        else if (!strcmp(argv[i], "--blas") && i + 1 < argc) blas = argv[++i];
        else if (!strcmp(argv[i], "--prefix") && i + 1 < argc) prefix = argv[++i];
        else if (!strcmp(argv[i], "--calls") && i + 1 < argc) calls = atoi(argv[++i]);
        else if (!strcmp(argv[i], "--images") && i + 1 < argc) images = atoi(argv[++i]);
        else if (!strcmp(argv[i], "--dump") && i + 1 < argc) dump = argv[++i];
        else { fprintf(stderr, "usage: %s [--workload mlp|gemm|conv|cnn] [--blas PATH --prefix P] [--calls N] [--images N] [--dump FILE]\n", argv[0]); return 2; }
    }
    const char *bound = "bundled loops (no BLAS library)";
    if (blas) {
        void *h = dlopen(blas, RTLD_NOW | RTLD_GLOBAL);
        if (!h) { fprintf(stderr, "cpu_emitted_bench: dlopen(%s): %s\n", blas, dlerror()); return 4; }
        char name[128];
        snprintf(name, sizeof(name), "%ssgemm_", prefix);
        sgemm_fn sg = (sgemm_fn)dlsym(h, name);
        snprintf(name, sizeof(name), "%ssaxpy_", prefix);
        saxpy_fn sa = (saxpy_fn)dlsym(h, name);
        if (!sg || !sa) { fprintf(stderr, "cpu_emitted_bench: %s has no %ssgemm_ / %ssaxpy_\n", blas, prefix, prefix); return 5; }
        g_sgemm = sg;
        g_saxpy = sa;
        bound = blas;
    }
    const double check = selfcheck();
    double *times;
    double checksum = 0;
    if (!strcmp(workload, "mlp")) {
        /* x [256,64] N(0,1); weights Glorot-uniform; biases zero (broadcast to [M,N] at construction, :271-290) */
        const int M = 256, d[4] = {64, 128, 64, 8};
        if (calls <= 0) calls = 200;
        float *x = alloc_f((size_t)M * d[0]), *w[3], *bb[3], *h[3];
        for (int i = 0; i < M * d[0]; ++i) x[i] = (float)normal01();
        for (int l = 0; l < 3; ++l) {
            const double lim = sqrt(6.0 / (d[l] + d[l + 1]));
            w[l] = alloc_f((size_t)d[l] * d[l + 1]);
            for (int i = 0; i < d[l] * d[l + 1]; ++i) w[l][i] = (float)((2 * uniform01() - 1) * lim);
            bb[l] = (float *)calloc((size_t)M * d[l + 1], sizeof(float));
            h[l] = alloc_f((size_t)M * d[l + 1]);
        }
        times = (double *)malloc(sizeof(double) * calls);
        for (int it = -1; it < calls; ++it) {        /* one warm-up call */
            const double t0 = now_ms();
            emitted_gemm(M, d[1], d[0], x, w[0], bb[0], h[0], 1);
            emitted_gemm(M, d[2], d[1], h[0], w[1], bb[1], h[1], 1);
            emitted_gemm(M, d[3], d[2], h[1], w[2], bb[2], h[2], 0);
            if (it >= 0) times[it] = now_ms() - t0;
        }
        for (int i = 0; i < M * d[3]; ++i) checksum += h[2][i];
        if (dump) {   /* inputs, weights and result as raw floats, for the test that compares them with the oracle */
            FILE *f = fopen(dump, "wb");
            if (!f) { perror(dump); return 6; }
            fwrite(x, sizeof(float), (size_t)M * d[0], f);
            for (int l = 0; l < 3; ++l) fwrite(w[l], sizeof(float), (size_t)d[l] * d[l + 1], f);
            fwrite(h[2], sizeof(float), (size_t)M * d[3], f);
            fclose(f);
        }
    } else if (!strcmp(workload, "gemm")) {
        /* one large Gemm as ROperator_Gemm emits it: `images` rows of a [4096, 4096] x [4096, 4096] product (the rows of
           the product are independent), bias broadcast to [M, N] at construction, ReLU */
        const int M = images, N = 4096, K = 4096;
        if (calls <= 0) calls = 3;
        float *x = alloc_f((size_t)M * K), *w = alloc_f((size_t)K * N), *bb = alloc_f((size_t)M * N), *y = alloc_f((size_t)M * N);
        for (size_t i = 0; i < (size_t)M * K; ++i) x[i] = (float)normal01();
        for (size_t i = 0; i < (size_t)K * N; ++i) w[i] = (float)normal01();
        for (int n = 0; n < N; ++n) {
            const float b = (float)normal01();
            for (int m = 0; m < M; ++m) bb[(size_t)m * N + n] = b;
        }
        times = (double *)malloc(sizeof(double) * calls);
        for (int it = -1; it < calls; ++it) {
            const double t0 = now_ms();
            emitted_gemm(M, N, K, x, w, bb, y, 1);
            if (it >= 0) times[it] = now_ms() - t0;
        }
        for (size_t i = 0; i < (size_t)M * N; i += 4099) checksum += y[i];
        if (dump) {
            FILE *f = fopen(dump, "wb");
            if (!f) { perror(dump); return 6; }
            fwrite(x, sizeof(float), (size_t)M * K, f);
            fwrite(w, sizeof(float), (size_t)K * N, f);
            fwrite(bb, sizeof(float), N, f);              /* the bias row */
            fwrite(y, sizeof(float), (size_t)M * N, f);
            fclose(f);
        }
    } else if (!strcmp(workload, "conv")) {
        const int N = images, C = 64, H = 56, W = 56, OC = 128, KH = 3, KW = 3;
        if (calls <= 0) calls = 5;
        const size_t plane = (size_t)H * W;
        float *x = alloc_f((size_t)N * C * plane), *wt = alloc_f((size_t)OC * C * 9), *bias = alloc_f(OC);
        float *bb = alloc_f((size_t)OC * plane), *xf = alloc_f((size_t)OC * C * 9), *xcol = alloc_f((size_t)C * 9 * plane);
        float *y = alloc_f((size_t)N * OC * plane);
        for (size_t i = 0; i < (size_t)N * C * plane; ++i) x[i] = (float)uniform01();
        for (int i = 0; i < OC * C * 9; ++i) wt[i] = (float)(normal01() * sqrt(2.0 / 576.0));
        for (int i = 0; i < OC; ++i) bias[i] = (float)(normal01() * 0.1);
        for (int oc = 0; oc < OC; ++oc)                   /* bias broadcast to [OC,OH,OW] at construction (:284-300) */
            for (size_t p = 0; p < plane; ++p) bb[oc * plane + p] = bias[oc];
        times = (double *)malloc(sizeof(double) * calls);
        for (int it = -1; it < calls; ++it) {
            const double t0 = now_ms();
            emitted_conv_relu(N, C, H, W, OC, KH, KW, 1, 1, x, wt, bb, xf, xcol, y);
            if (it >= 0) times[it] = now_ms() - t0;
        }
        for (size_t i = 0; i < (size_t)N * OC * plane; i += 4099) checksum += y[i];
        if (dump) {
            FILE *f = fopen(dump, "wb");
            if (!f) { perror(dump); return 6; }
            fwrite(x, sizeof(float), (size_t)N * C * plane, f);
            fwrite(wt, sizeof(float), (size_t)OC * C * 9, f);
            fwrite(bias, sizeof(float), OC, f);
            fwrite(y, sizeof(float), (size_t)N * OC * plane, f);
            fclose(f);
        }
    } else if (!strcmp(workload, "cnn")) {
        /* images U[0,1]; Kaiming-normal weights; small biases, broadcast at construction as the reference does */
        const int N = images;
        const int ch[4] = {1, 32, 64, 128}, side[4] = {40, 20, 10, 10};   /* input channels / spatial size of conv l */
        if (calls <= 0) calls = 3;
        float *x = alloc_f((size_t)N * 1600);
        for (size_t i = 0; i < (size_t)N * 1600; ++i) x[i] = (float)uniform01();
        float *cw[3], *cb[3], *cbb[3], *cxf[3], *cy[3], *pool[2];
        size_t max_col = 0;
        for (int l = 0; l < 3; ++l) {
            const int C = ch[l], OC = ch[l + 1], hw = side[l] * side[l];
            cw[l] = alloc_f((size_t)OC * C * 9);
            cb[l] = alloc_f(OC);
            cbb[l] = alloc_f((size_t)OC * hw);
            cxf[l] = alloc_f((size_t)OC * C * 9);
            cy[l] = alloc_f((size_t)N * OC * hw);
            for (int i = 0; i < OC * C * 9; ++i) cw[l][i] = (float)(normal01() * sqrt(2.0 / (C * 9.0)));
            for (int i = 0; i < OC; ++i) cb[l][i] = (float)(normal01() * 0.05);
            for (int oc = 0; oc < OC; ++oc)
                for (int p = 0; p < hw; ++p) cbb[l][(size_t)oc * hw + p] = cb[l][oc];
            if ((size_t)C * 9 * hw > max_col) max_col = (size_t)C * 9 * hw;
        }
        pool[0] = alloc_f((size_t)N * 32 * 400);
        pool[1] = alloc_f((size_t)N * 64 * 100);
        float *xcol = alloc_f(max_col);
        const int K1 = 12800, N1 = 256, N2 = 5;
        float *w1 = alloc_f((size_t)K1 * N1), *w2 = alloc_f((size_t)N1 * N2), *b1 = alloc_f(N1), *b2 = alloc_f(N2);
        float *bb1 = alloc_f((size_t)N * N1), *bb2 = alloc_f((size_t)N * N2), *g1 = alloc_f((size_t)N * N1), *g2 = alloc_f((size_t)N * N2);
        for (size_t i = 0; i < (size_t)K1 * N1; ++i) w1[i] = (float)(normal01() * sqrt(2.0 / K1));
        for (int i = 0; i < N1 * N2; ++i) w2[i] = (float)(normal01() * sqrt(2.0 / N1));
        for (int i = 0; i < N1; ++i) b1[i] = (float)(normal01() * 0.05);
        for (int i = 0; i < N2; ++i) b2[i] = (float)(normal01() * 0.05);
        for (int r = 0; r < N; ++r) {
            memcpy(bb1 + (size_t)r * N1, b1, N1 * sizeof(float));
            memcpy(bb2 + (size_t)r * N2, b2, N2 * sizeof(float));
        }
        times = (double *)malloc(sizeof(double) * calls);
        for (int it = -1; it < calls; ++it) {
            const double t0 = now_ms();
            emitted_conv_relu(N, 1, 40, 40, 32, 3, 3, 1, 1, x, cw[0], cbb[0], cxf[0], xcol, cy[0]);
            emitted_maxpool(N * 32, 40, 40, 2, 2, 0, 2, 2, cy[0], pool[0]);
            emitted_conv_relu(N, 32, 20, 20, 64, 3, 3, 1, 1, pool[0], cw[1], cbb[1], cxf[1], xcol, cy[1]);
            emitted_maxpool(N * 64, 20, 20, 2, 2, 0, 2, 2, cy[1], pool[1]);
            emitted_conv_relu(N, 64, 10, 10, 128, 3, 3, 1, 1, pool[1], cw[2], cbb[2], cxf[2], xcol, cy[2]);
            emitted_gemm(N, N1, K1, cy[2], w1, bb1, g1, 1);          /* Flatten is a view of the convolution's output */
            emitted_gemm(N, N2, N1, g1, w2, bb2, g2, 0);
            if (it >= 0) times[it] = now_ms() - t0;
        }
        for (int i = 0; i < N * N2; ++i) checksum += g2[i];
        if (dump) {
            FILE *f = fopen(dump, "wb");
            if (!f) { perror(dump); return 6; }
            fwrite(x, sizeof(float), (size_t)N * 1600, f);
            for (int l = 0; l < 3; ++l) {
                fwrite(cw[l], sizeof(float), (size_t)ch[l + 1] * ch[l] * 9, f);
                fwrite(cb[l], sizeof(float), ch[l + 1], f);
            }
            fwrite(w1, sizeof(float), (size_t)K1 * N1, f);
            fwrite(b1, sizeof(float), N1, f);
            fwrite(w2, sizeof(float), (size_t)N1 * N2, f);
            fwrite(b2, sizeof(float), N2, f);
            fwrite(g2, sizeof(float), (size_t)N * N2, f);
            fclose(f);
        }
    } else {
        fprintf(stderr, "cpu_emitted_bench: unknown workload %s\n", workload);
        return 2;
    }
    qsort(times, calls, sizeof(double), cmp_double);
    printf("{\"workload\": \"%s\", \"blas\": \"%s\", \"calls\": %d, \"images\": %d, \"median_ms\": %.6f, \"best_ms\": %.6f, "
           "\"checksum\": %.6e, \"selfcheck\": %.3e}\n",
           workload, bound, calls, strcmp(workload, "mlp") ? images : 256, times[calls / 2], times[0], checksum, check);
    return 0;
}
