/*
 * CPU oracle for the Winograd 3x3 convolution path.  TEST INFRASTRUCTURE ONLY:
 * the shipped library never links, loads or calls anything in this file; it is
 * the checker the parity tests, the smoke test and the benchmark's CPU-baseline
 * leg use.
 *
 * What it restates (reference files read as text, never executed):
 *   - direct convolution ("Ground-Truth Naive Convolution"), a zero-padded 3x3
 *     stride-1 cross-correlation:
 *       layoutTest/NCHW/data/WinoTran_NCHW.py:200-228  (Conv_NCHW)
 *       layoutTest/NHWC/data/WinoTran_NHWC.py:202-229  (Conv_NHWC)
 *       layoutTest/CHWN/data/WinoTran_CHWN.py:201-228  (Conv_CHWN)
 *   - tensor/filter index conventions per layout:
 *       comparison/wrapedConv_NCHW.cuh:869   w[k][c][r][s]
 *       comparison/wrapedConv_NHWC.cuh:341   w[k][r][s][c]
 *       comparison/wrapedConv_CHWN.cuh:288   w[c][r][s][k]
 *   - the four Winograd stages (input / filter transform, per-coordinate GEMM,
 *     inverse transform) of comparison/wrapedConv_NCHW.cuh:408-452 and
 *     layoutTest/NCHW/data/WinoTran_NCHW.py:6-198, restated for F(2x2,3x3)
 *     (4x4 tiles, 16 coordinates) and, as a second mode, for the reference's own
 *     F(4x4,3x3) matrices (WinoTran_NCHW.py:22-27, 86-91, 181-186).
 *
 * Parity pins (tests/test_oracle_*.py): direct conv against a float64 library
 * correlation, brute force and closed-form cases (delta filter, all-ones, hot
 * pixel); the Winograd stages against the exact identity
 * A^T[(G g G^T).(B^T d B)]A == valid correlation on small integers (bit-exact
 * for F(2x2), whose constants are dyadic) and closed-form single-stage cases.
 *
 * Build: gcc -O2 -fopenmp -shared -fPIC (see oracle/Makefile).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

enum { L_NCHW = 0, L_NHWC = 1, L_CHWN = 2 };

/* element strides of an activation tensor, order (n, c, h, w) */
static int act_strides(int layout, long N, long C, long H, long W, long s[4]) {
    switch (layout) {
    case L_NCHW: s[0] = C * H * W; s[1] = H * W; s[2] = W; s[3] = 1; return 0;
    case L_NHWC: s[0] = H * W * C; s[1] = 1; s[2] = W * C; s[3] = C; return 0;
    case L_CHWN: s[0] = 1; s[1] = H * W * N; s[2] = W * N; s[3] = N; return 0;
    }
    return -1;
}

/* element strides of a 3x3 filter bank, order (k, c, r, s) */
static int flt_strides(int layout, long K, long C, long s[4]) {
    switch (layout) {
    case L_NCHW: s[0] = C * 9; s[1] = 9; s[2] = 3; s[3] = 1; return 0;
    case L_NHWC: s[0] = 9 * C; s[1] = 1; s[2] = 3 * C; s[3] = C; return 0;
    case L_CHWN: s[0] = 1; s[1] = 9 * K; s[2] = 3 * K; s[3] = K; return 0;
    }
    return -1;
}

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/*
 * Gold direct convolution.  x and w follow src_layout's conventions, y follows
 * dst_layout's.  y[n,k,i,j] = sum_{c,r,s} x[n,c,i+r-pad,j+s-pad] * w[k,c,r,s],
 * out-of-range x reads are 0, accumulation in double, summation order c,r,s.
 */
int oracle_direct_conv3x3(int src_layout, int dst_layout, int N, int C, int K,
                          int H, int W, int pad, const float *x, const float *w,
                          float *y) {
    long sx[4], sw[4], sy[4];
    int Ho = H + 2 * pad - 2, Wo = W + 2 * pad - 2;
    if (Ho <= 0 || Wo <= 0) return -1;
    if (act_strides(src_layout, N, C, H, W, sx)) return -1;
    if (flt_strides(src_layout, K, C, sw)) return -1;
    if (act_strides(dst_layout, N, K, Ho, Wo, sy)) return -1;
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k)
            for (int i = 0; i < Ho; ++i)
                for (int j = 0; j < Wo; ++j) {
                    double acc = 0.0;
                    for (int c = 0; c < C; ++c)
                        for (int r = 0; r < 3; ++r) {
                            int ih = i + r - pad;
                            if (ih < 0 || ih >= H) continue;
                            for (int s = 0; s < 3; ++s) {
                                int iw = j + s - pad;
                                if (iw < 0 || iw >= W) continue;
                                acc += (double)x[n * sx[0] + c * sx[1] + ih * sx[2] + iw * sx[3]] *
                                       (double)w[k * sw[0] + c * sw[1] + r * sw[2] + s * sw[3]];
                            }
                        }
                    y[n * sy[0] + k * sy[1] + i * sy[2] + j * sy[3]] = (float)acc;
                }
    return 0;
}

/* copy an activation tensor between layouts (logical permutation only) */
int oracle_permute_act(int src_layout, int dst_layout, int N, int C, int H, int W,
                       const float *src, float *dst) {
    long a[4], b[4];
    if (act_strides(src_layout, N, C, H, W, a)) return -1;
    if (act_strides(dst_layout, N, C, H, W, b)) return -1;
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; ++n)
        for (int c = 0; c < C; ++c)
            for (int h = 0; h < H; ++h)
                for (int v = 0; v < W; ++v)
                    dst[n * b[0] + c * b[1] + h * b[2] + v * b[3]] =
                        src[n * a[0] + c * a[1] + h * a[2] + v * a[3]];
    return 0;
}

int oracle_permute_flt(int src_layout, int dst_layout, int K, int C, const float *src,
                       float *dst) {
    long a[4], b[4];
    if (flt_strides(src_layout, K, C, a)) return -1;
    if (flt_strides(dst_layout, K, C, b)) return -1;
    for (int k = 0; k < K; ++k)
        for (int c = 0; c < C; ++c)
            for (int r = 0; r < 3; ++r)
                for (int s = 0; s < 3; ++s)
                    dst[k * b[0] + c * b[1] + r * b[2] + s * b[3]] =
                        src[k * a[0] + c * a[1] + r * a[2] + s * a[3]];
    return 0;
}

/*
 * Timed host baseline: the same cross-correlation with fp32 multiply-add,
 * plane-at-a-time so the inner loop runs along contiguous pixels.  Non-NCHW
 * inputs are permuted to NCHW first and the result permuted back (the permutes
 * are inside the call, as they would be for any host implementation that wants
 * unit-stride inner loops).  relu != 0 clamps negatives.
 */
int oracle_direct_conv3x3_f32(int src_layout, int dst_layout, int N, int C, int K,
                              int H, int W, int pad, const float *x, const float *w,
                              float *y, int relu) {
    int Ho = H + 2 * pad - 2, Wo = W + 2 * pad - 2;
    if (Ho <= 0 || Wo <= 0) return -1;
    const float *xc = x, *wc = w;
    float *xt = NULL, *wt = NULL, *yt = NULL, *yc = y;
    if (src_layout != L_NCHW) {
        xt = (float *)malloc(sizeof(float) * (size_t)N * C * H * W);
        wt = (float *)malloc(sizeof(float) * (size_t)K * C * 9);
        if (!xt || !wt) { free(xt); free(wt); return -2; }
        oracle_permute_act(src_layout, L_NCHW, N, C, H, W, x, xt);
        oracle_permute_flt(src_layout, L_NCHW, K, C, w, wt);
        xc = xt; wc = wt;
    }
    if (dst_layout != L_NCHW) {
        yt = (float *)malloc(sizeof(float) * (size_t)N * K * Ho * Wo);
        if (!yt) { free(xt); free(wt); return -2; }
        yc = yt;
    }
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k) {
            float *yp = yc + ((size_t)n * K + k) * Ho * Wo;
            memset(yp, 0, sizeof(float) * (size_t)Ho * Wo);
            for (int c = 0; c < C; ++c) {
                const float *xp = xc + ((size_t)n * C + c) * H * W;
                const float *wp = wc + ((size_t)k * C + c) * 9;
                for (int r = 0; r < 3; ++r)
                    for (int s = 0; s < 3; ++s) {
                        float wv = wp[r * 3 + s];
                        int i0 = pad - r > 0 ? pad - r : 0;
                        int i1 = H + pad - r < Ho ? H + pad - r : Ho;
                        int j0 = pad - s > 0 ? pad - s : 0;
                        int j1 = W + pad - s < Wo ? W + pad - s : Wo;
                        for (int i = i0; i < i1; ++i) {
                            const float *xr = xp + (size_t)(i + r - pad) * W + (s - pad);
                            float *yr = yp + (size_t)i * Wo;
                            for (int j = j0; j < j1; ++j) yr[j] += xr[j] * wv;
                        }
                    }
            }
            if (relu)
                for (int q = 0; q < Ho * Wo; ++q) yp[q] = yp[q] > 0.f ? yp[q] : 0.f;
        }
    if (yt) oracle_permute_act(L_NCHW, dst_layout, N, K, Ho, Wo, yt, y);
    free(xt); free(wt); free(yt);
    return 0;
}

/* ------------------------------------------------------------------------- */
/* Winograd minimal filtering, two tile sizes.                                */
/*   m = 2: F(2x2,3x3), t = 4, points {0, 1, -1, inf}                          */
/*   m = 4: F(4x4,3x3), t = 6, the reference's matrices                        */
/* ------------------------------------------------------------------------- */

static const double BT2[4][4] = {{1, 0, -1, 0}, {0, 1, 1, 0}, {0, -1, 1, 0}, {0, 1, 0, -1}};
static const double G2[4][3] = {{1, 0, 0}, {.5, .5, .5}, {.5, -.5, .5}, {0, 0, 1}};
static const double AT2[2][4] = {{1, 1, 1, 0}, {0, 1, -1, -1}};

static const double BT4[6][6] = {{4, 0, -5, 0, 1, 0},  {0, -4, -4, 1, 1, 0}, {0, 4, -4, -1, 1, 0},
                                 {0, -2, -1, 2, 1, 0}, {0, 2, -1, -2, 1, 0}, {0, 4, 0, -5, 0, 1}};
static const double G4[6][3] = {{1. / 4, 0, 0},
                                {-1. / 6, -1. / 6, -1. / 6},
                                {-1. / 6, 1. / 6, -1. / 6},
                                {1. / 24, 1. / 12, 1. / 6},
                                {1. / 24, -1. / 12, 1. / 6},
                                {0, 0, 1}};
static const double AT4[4][6] = {{1, 1, 1, 1, 1, 0}, {0, 1, -1, 2, -2, 0}, {0, 1, 1, 4, 4, 0}, {0, 1, -1, 8, -8, 1}};

static const double *mat_BT(int m) { return m == 2 ? &BT2[0][0] : &BT4[0][0]; }
static const double *mat_G(int m) { return m == 2 ? &G2[0][0] : &G4[0][0]; }
static const double *mat_AT(int m) { return m == 2 ? &AT2[0][0] : &AT4[0][0]; }

int oracle_wino_tiles(int m, int H, int W, int pad, int *th, int *tw) {
    int Ho = H + 2 * pad - 2, Wo = W + 2 * pad - 2;
    if ((m != 2 && m != 4) || Ho <= 0 || Wo <= 0) return -1;
    *th = (Ho + m - 1) / m;
    *tw = (Wo + m - 1) / m;
    return 0;
}

/* U[xi][c][k] = (G g G^T)[xi/t][xi%t];  fp32 result, double arithmetic rounded once */
int oracle_wino_filter_transform(int m, int layout, int K, int C, const float *w, float *U) {
    long sw[4];
    int t = m + 2;
    if ((m != 2 && m != 4) || flt_strides(layout, K, C, sw)) return -1;
    const double *G = mat_G(m);
    for (int c = 0; c < C; ++c)
        for (int k = 0; k < K; ++k) {
            double g[3][3], Gg[6][3];
            for (int r = 0; r < 3; ++r)
                for (int s = 0; s < 3; ++s)
                    g[r][s] = w[k * sw[0] + c * sw[1] + r * sw[2] + s * sw[3]];
            for (int i = 0; i < t; ++i)
                for (int s = 0; s < 3; ++s) {
                    double a = 0;
                    for (int r = 0; r < 3; ++r) a += G[i * 3 + r] * g[r][s];
                    Gg[i][s] = a;
                }
            for (int i = 0; i < t; ++i)
                for (int j = 0; j < t; ++j) {
                    double a = 0;
                    for (int s = 0; s < 3; ++s) a += Gg[i][s] * G[j * 3 + s];
                    U[((size_t)(i * t + j) * C + c) * K + k] = (float)a;
                }
        }
    return 0;
}

/* V[xi][c][p] = (B^T d B)[xi/t][xi%t], p = (n*th + ty)*tw + tx, tile origin (m*ty-pad, m*tx-pad) */
int oracle_wino_input_transform(int m, int layout, int N, int C, int H, int W, int pad,
                                const float *x, float *V) {
    long sx[4];
    int t = m + 2, th, tw;
    if (oracle_wino_tiles(m, H, W, pad, &th, &tw) || act_strides(layout, N, C, H, W, sx)) return -1;
    const double *BT = mat_BT(m);
    size_t P = (size_t)N * th * tw;
#pragma omp parallel for collapse(2) schedule(static)
    for (int c = 0; c < C; ++c)
        for (int n = 0; n < N; ++n)
            for (int ty = 0; ty < th; ++ty)
                for (int tx = 0; tx < tw; ++tx) {
                    double d[6][6], Bd[6][6];
                    for (int i = 0; i < t; ++i)
                        for (int j = 0; j < t; ++j) {
                            int ih = m * ty - pad + i, iw = m * tx - pad + j;
                            d[i][j] = (ih < 0 || ih >= H || iw < 0 || iw >= W)
                                          ? 0.0
                                          : (double)x[n * sx[0] + c * sx[1] + ih * sx[2] + iw * sx[3]];
                        }
                    for (int i = 0; i < t; ++i)
                        for (int j = 0; j < t; ++j) {
                            double a = 0;
                            for (int q = 0; q < t; ++q) a += BT[i * t + q] * d[q][j];
                            Bd[i][j] = a;
                        }
                    size_t p = ((size_t)n * th + ty) * tw + tx;
                    for (int i = 0; i < t; ++i)
                        for (int j = 0; j < t; ++j) {
                            double a = 0;
                            for (int q = 0; q < t; ++q) a += Bd[i][q] * BT[j * t + q];
                            V[((size_t)(i * t + j) * C + c) * P + p] = (float)a;
                        }
                }
    return 0;
}

/* Mo[xi][k][p] = sum_c U[xi][c][k] * V[xi][c][p], double accumulate */
int oracle_wino_gemm(int m, int C, int K, long P, const float *U, const float *V, float *Mo) {
    int t = m + 2, nxi = t * t;
#pragma omp parallel for collapse(2) schedule(static)
    for (int xi = 0; xi < nxi; ++xi)
        for (int k = 0; k < K; ++k) {
            double *acc = (double *)calloc((size_t)P, sizeof(double));
            for (int c = 0; c < C; ++c) {
                double u = U[((size_t)xi * C + c) * K + k];
                const float *v = V + ((size_t)xi * C + c) * P;
                for (long p = 0; p < P; ++p) acc[p] += u * v[p];
            }
            float *o = Mo + ((size_t)xi * K + k) * P;
            for (long p = 0; p < P; ++p) o[p] = (float)acc[p];
            free(acc);
        }
    return 0;
}

/* y (dst layout, N x K x Ho x Wo) = A^T Mo A per tile, partial edge tiles clipped */
int oracle_wino_output_transform(int m, int layout, int N, int K, int Ho, int Wo,
                                 const float *Mo, float *y) {
    long sy[4];
    int t = m + 2;
    if ((m != 2 && m != 4) || act_strides(layout, N, K, Ho, Wo, sy)) return -1;
    int th = (Ho + m - 1) / m, tw = (Wo + m - 1) / m;
    size_t P = (size_t)N * th * tw;
    const double *AT = mat_AT(m);
#pragma omp parallel for collapse(2) schedule(static)
    for (int k = 0; k < K; ++k)
        for (int n = 0; n < N; ++n)
            for (int ty = 0; ty < th; ++ty)
                for (int tx = 0; tx < tw; ++tx) {
                    size_t p = ((size_t)n * th + ty) * tw + tx;
                    double M[6][6], AM[4][6];
                    for (int i = 0; i < t; ++i)
                        for (int j = 0; j < t; ++j)
                            M[i][j] = Mo[((size_t)(i * t + j) * K + k) * P + p];
                    for (int a = 0; a < m; ++a)
                        for (int j = 0; j < t; ++j) {
                            double s = 0;
                            for (int i = 0; i < t; ++i) s += AT[a * t + i] * M[i][j];
                            AM[a][j] = s;
                        }
                    for (int a = 0; a < m; ++a)
                        for (int b = 0; b < m; ++b) {
                            int oh = m * ty + a, ow = m * tx + b;
                            if (oh >= Ho || ow >= Wo) continue;
                            double s = 0;
                            for (int j = 0; j < t; ++j) s += AM[a][j] * AT[b * t + j];
                            y[n * sy[0] + k * sy[1] + oh * sy[2] + ow * sy[3]] = (float)s;
                        }
                }
    return 0;
}

/* the four stages chained, fp32 intermediates as on the device */
int oracle_wino_conv3x3(int m, int src_layout, int dst_layout, int N, int C, int K, int H,
                        int W, int pad, const float *x, const float *w, float *y) {
    int th, tw, t = m + 2;
    if (oracle_wino_tiles(m, H, W, pad, &th, &tw)) return -1;
    size_t P = (size_t)N * th * tw, nxi = (size_t)t * t;
    float *U = (float *)malloc(sizeof(float) * nxi * C * K);
    float *V = (float *)malloc(sizeof(float) * nxi * C * P);
    float *Mo = (float *)malloc(sizeof(float) * nxi * K * P);
    int rc = -2;
    if (U && V && Mo) {
        rc = oracle_wino_filter_transform(m, src_layout, K, C, w, U);
        if (!rc) rc = oracle_wino_input_transform(m, src_layout, N, C, H, W, pad, x, V);
        if (!rc) rc = oracle_wino_gemm(m, C, K, (long)P, U, V, Mo);
        if (!rc) rc = oracle_wino_output_transform(m, dst_layout, N, K, H + 2 * pad - 2, W + 2 * pad - 2, Mo, y);
    }
    free(U); free(V); free(Mo);
    return rc;
}

/* ------------------------------------------------------------------------- */
/* error metric and reduced-precision rounding helpers                        */
/* ------------------------------------------------------------------------- */

double oracle_rel_l2(const float *got, const float *want, long n) {
    double num = 0, den = 0;
    for (long i = 0; i < n; ++i) {
        double d = (double)got[i] - (double)want[i];
        num += d * d;
        den += (double)want[i] * (double)want[i];
    }
    if (den == 0) return num == 0 ? 0.0 : INFINITY;
    return sqrt(num / den);
}

/* round-to-nearest-even fp32 -> bf16 -> fp32 */
void oracle_round_bf16(const float *src, float *dst, long n) {
    for (long i = 0; i < n; ++i) {
        uint32_t u;
        memcpy(&u, &src[i], 4);
        if ((u & 0x7f800000u) != 0x7f800000u) u += 0x7fffu + ((u >> 16) & 1u);
        u &= 0xffff0000u;
        memcpy(&dst[i], &u, 4);
    }
}

/* round-to-nearest-even fp32 -> IEEE binary16 -> fp32 (overflow -> inf, subnormals kept) */
static float f16_roundtrip(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    uint32_t sign = u & 0x80000000u, a = u & 0x7fffffffu;
    float r;
    if (a >= 0x7f800000u) return f;                 /* inf / nan unchanged */
    if (a >= 0x477ff000u) {                          /* >= 65520 rounds to inf */
        uint32_t inf = sign | 0x7f800000u;
        memcpy(&r, &inf, 4);
        return r;
    }
    if (a < 0x38800000u) {                           /* below 2^-14: spacing is 2^-24 */
        float mag;
        memcpy(&mag, &a, 4);
        /* adding 2^-1 forces rounding at 2^-24 in fp32 (RNE), then subtract it */
        volatile float t = mag + 0.5f;
        mag = t - 0.5f;
        memcpy(&a, &mag, 4);
    } else {
        a += 0xfffu + ((a >> 13) & 1u);              /* RNE at 13 dropped bits */
        a &= 0xffffe000u;
    }
    a |= sign;
    memcpy(&r, &a, 4);
    return r;
}

void oracle_round_f16(const float *src, float *dst, long n) {
    for (long i = 0; i < n; ++i) dst[i] = f16_roundtrip(src[i]);
}
