/*
 * CPU oracle for the depthwise oriented 1D convolution (fprop / dgrad / wgrad).
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may link, load or
 * call this file; it exists so that tests, the smoke check and the benchmark's
 * cpu_baseline leg have an independent statement of the reference algorithm.
 *
 * It restates the plain loops of the reference's CPU formulation
 *   models/dwoconv1d_reference/kernels/kernels.cpp:36-52   (fprop)
 *   models/dwoconv1d_reference/kernels/kernels.cpp:71-90   (dgrad)
 *   models/dwoconv1d_reference/kernels/kernels.cpp:111-126 (wgrad)
 * with the same loop order, the same fp32 sine/cosine, the same float product
 * followed by a C cast to int (truncation toward zero), the same out-of-bounds
 * rule (taps outside the image contribute nothing) and the same stride rule
 * for dgrad (a tap contributes only when both coordinates are divisible by the
 * stride).  The *_f32 functions accumulate in fp32 exactly as the reference's
 * `T sum` does; the *_f64 functions accumulate the same products in double and
 * are what tolerance-based parity tests compare against.
 *
 * Generalisation over the reference: P,Q (output extent) and H,W (input
 * extent) are both explicit so the arbitrary-size semantics of
 * models/dwoconv1d/dwoconv1d.py:154-187 (zero-pad, run, crop => P = ceil(H/stride))
 * can be checked with the same loops; with P = H/stride this is the reference.
 *
 * Pinned by tests/test_oracle_*.py against: library conv2d closed forms for
 * theta = 0 and pi/2 and the dense-2D-kernel form for any theta, impulse
 * responses, tap-table known answers, adjoint identities, and a pure-Python
 * brute force.  The reference holds no golden vectors for this path.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* kernels.cpp:37,43-44 — per-channel offsets; the product is formed in float
 * (float * int -> float) and cast to int, i.e. truncated toward zero. */
static inline void tap_offset(float sin_, float cos_, int s, int pad, int *dh, int *dw)
{
    volatile float ph = -sin_ * (float)(s - pad);
    volatile float pw = cos_ * (float)(s - pad);
    *dh = (int)ph;
    *dw = (int)pw;
}

/* mode 0: sinf/cosf (float overloads); mode 1: double sin/cos rounded to
 * float (what `float s = sin(theta_float)` yields if only the double
 * overload is visible).  Tests assert both give the same table for every
 * angle the workloads use. */
void dwo_oracle_taps(const float *theta, int C, int S, int pad, int mode, int *dh, int *dw)
{
    for (int c = 0; c < C; c++) {
        float sin_, cos_;
        if (mode == 0) {
            sin_ = sinf(theta[c]);
            cos_ = cosf(theta[c]);
        } else {
            sin_ = (float)sin((double)theta[c]);
            cos_ = (float)cos((double)theta[c]);
        }
        for (int s = 0; s < S; s++)
            tap_offset(sin_, cos_, s, pad, &dh[c * S + s], &dw[c * S + s]);
    }
}

int dwo_oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

#define IDX4(n, c, h, w, C, H, W) ((((size_t)(n) * (C) + (c)) * (H) + (h)) * (W) + (w))

#define DEFINE_FPROP(NAME, ACC, OUT)                                                            \
    void NAME(const float *x, const float *wt, const float *theta, OUT *y, int N, int C, int H, \
              int W, int P, int Q, int S, int stride, int pad, int threads)                     \
    {                                                                                           \
        (void)threads;                                                                          \
        _Pragma("omp parallel for schedule(dynamic, 1) num_threads(threads) if (threads > 1)")  \
        for (int c = 0; c < C; c++) {                                                           \
            float sin_ = sinf(theta[c]), cos_ = cosf(theta[c]);                                 \
            int dh[256], dw[256];                                                               \
            for (int s = 0; s < S; s++)                                                         \
                tap_offset(sin_, cos_, s, pad, &dh[s], &dw[s]);                                 \
            for (int n = 0; n < N; n++)                                                         \
                for (int p = 0; p < P; p++)                                                     \
                    for (int q = 0; q < Q; q++) {                                               \
                        ACC sum = 0;                                                            \
                        for (int s = 0; s < S; s++) {                                           \
                            int h = p * stride + dh[s];                                         \
                            int w = q * stride + dw[s];                                         \
                            if (h >= 0 && h < H && w >= 0 && w < W)                             \
                                sum += (ACC)x[IDX4(n, c, h, w, C, H, W)] * (ACC)wt[c * S + s];  \
                        }                                                                       \
                        y[IDX4(n, c, p, q, C, P, Q)] = (OUT)sum;                                \
                    }                                                                           \
        }                                                                                       \
    }

#define DEFINE_DGRAD(NAME, ACC, OUT)                                                             \
    void NAME(const float *dy, const float *wt, const float *theta, OUT *dx, int N, int C,       \
              int H, int W, int P, int Q, int S, int stride, int pad, int threads)               \
    {                                                                                            \
        (void)threads;                                                                           \
        _Pragma("omp parallel for schedule(dynamic, 1) num_threads(threads) if (threads > 1)")   \
        for (int c = 0; c < C; c++) {                                                            \
            float sin_ = sinf(theta[c]), cos_ = cosf(theta[c]);                                  \
            int dh[256], dw[256];                                                                \
            for (int s = 0; s < S; s++)                                                          \
                tap_offset(sin_, cos_, s, pad, &dh[s], &dw[s]);                                  \
            for (int n = 0; n < N; n++)                                                          \
                for (int h = 0; h < H; h++)                                                      \
                    for (int w = 0; w < W; w++) {                                                \
                        ACC sum = 0;                                                             \
                        for (int s = 0; s < S; s++) {                                            \
                            int pp = h - dh[s];                                                  \
                            int qq = w - dw[s];                                                  \
                            if (pp % stride != 0 || qq % stride != 0)                            \
                                continue;                                                        \
                            int p = pp / stride, q = qq / stride;                                \
                            if (p >= 0 && p < P && q >= 0 && q < Q)                              \
                                sum += (ACC)dy[IDX4(n, c, p, q, C, P, Q)] * (ACC)wt[c * S + s];  \
                        }                                                                        \
                        dx[IDX4(n, c, h, w, C, H, W)] = (OUT)sum;                                \
                    }                                                                            \
        }                                                                                        \
    }

#define DEFINE_WGRAD(NAME, ACC, OUT)                                                            \
    void NAME(const float *dy, const float *x, const float *theta, OUT *dwt, int N, int C,      \
              int H, int W, int P, int Q, int S, int stride, int pad, int threads)              \
    {                                                                                           \
        (void)threads;                                                                          \
        _Pragma("omp parallel for schedule(dynamic, 1) num_threads(threads) if (threads > 1)")  \
        for (int c = 0; c < C; c++) {                                                           \
            float sin_ = sinf(theta[c]), cos_ = cosf(theta[c]);                                 \
            for (int s = 0; s < S; s++) {                                                       \
                int dh, dw;                                                                     \
                tap_offset(sin_, cos_, s, pad, &dh, &dw);                                       \
                ACC sum = 0;                                                                    \
                for (int p = 0; p < P; p++)                                                     \
                    for (int q = 0; q < Q; q++) {                                               \
                        int h = p * stride + dh;                                                \
                        int w = q * stride + dw;                                                \
                        if (h >= 0 && h < H && w >= 0 && w < W)                                 \
                            for (int n = 0; n < N; n++)                                         \
                                sum += (ACC)x[IDX4(n, c, h, w, C, H, W)] *                      \
                                       (ACC)dy[IDX4(n, c, p, q, C, P, Q)];                      \
                    }                                                                           \
                dwt[c * S + s] = (OUT)sum;                                                      \
            }                                                                                   \
        }                                                                                       \
    }

/* fp32 accumulation: bit-for-bit the reference's arithmetic (`T sum`, T=float). */
DEFINE_FPROP(dwo_oracle_fprop_f32, float, float)
DEFINE_DGRAD(dwo_oracle_dgrad_f32, float, float)
DEFINE_WGRAD(dwo_oracle_wgrad_f32, float, float)
/* double accumulation of the same fp32 products: the tolerance oracle. */
DEFINE_FPROP(dwo_oracle_fprop_f64, double, double)
DEFINE_DGRAD(dwo_oracle_dgrad_f64, double, double)
DEFINE_WGRAD(dwo_oracle_wgrad_f64, double, double)

/* Bias gradient of models/dwoconv1d/dwoconv1d.py:66-67: db[c] = sum over n,p,q of dy. */
void dwo_oracle_bgrad_f64(const float *dy, double *db, int N, int C, int P, int Q)
{
    for (int c = 0; c < C; c++) {
        double sum = 0;
        for (int n = 0; n < N; n++)
            for (int i = 0; i < P * Q; i++)
                sum += (double)dy[((size_t)n * C + c) * P * Q + i];
        db[c] = sum;
    }
}
