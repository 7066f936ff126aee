/*
 * ddf_oracle.c - CPU restatement of the Decoupled Dynamic Filter operator.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against and the CPU baseline a benchmark reports beside them; no
 * product code path may call it.
 *
 * Each function restates, as plain gather loops, what one reference kernel
 * computes (theFoxofSky/ddfnet):
 *   forward  : grad_check.py:11-30 (loop form, stride 1) and
 *              ddf/src/cuda/ddf_mul_cuda_kernel.cu:110-163 (stride, skipped
 *              out-of-image taps); 'add' per ddf_add_cuda_kernel.cu:150-152
 *   dX       : ddf_mul_cuda_kernel.cu:222-288; add: ddf_add_cuda_kernel.cu:278-279
 *   dSF      : ddf_mul_cuda_kernel.cu:317-353; add: ddf_add_cuda_kernel.cu:338
 *   dCF      : ddf_mul_cuda_kernel.cu:379-418; add: ddf_add_cuda_kernel.cu:403
 * Sums are plain left-to-right sums in the working type (the reference's
 * Neumaier compensation is a precision aid, not part of the result's
 * definition).
 *
 * Layout: all tensors dense NCHW.  r = (k-1)/2, Ho = H/s, Wo = W/s (floor).
 * Two instantiations: _f64 (the checker) and _f32 (the timed CPU baseline).
 * Loops over (n,c) or (n,pixel) are OpenMP-parallel when built with -fopenmp.
 */
#include <stddef.h>
#include <stdint.h>

#define DDF_MUL 0
#define DDF_ADD 1

#define DEFINE_ORACLE(T, SUFFIX)                                               \
                                                                               \
    void ddf_oracle_forward_##SUFFIX(                                          \
        const T *x, const T *cf, const T *sf, T *out, int64_t N, int64_t C,    \
        int64_t H, int64_t W, int k, int d, int s, int combine) {              \
        const int64_t Ho = H / s, Wo = W / s;                                  \
        const int r = (k - 1) / 2, kk = k * k;                                 \
        _Pragma("omp parallel for schedule(static)")                           \
        for (int64_t nc = 0; nc < N * C; ++nc) {                               \
            const int64_t n = nc / C;                                          \
            const T *xp = x + nc * H * W;                                      \
            const T *cfp = cf + nc * kk;                                       \
            const T *sfp = sf + n * kk * Ho * Wo;                              \
            T *op = out + nc * Ho * Wo;                                        \
            for (int64_t y = 0; y < Ho; ++y)                                   \
                for (int64_t xo = 0; xo < Wo; ++xo) {                          \
                    T acc = 0;                                                 \
                    for (int i = 0; i < k; ++i) {                              \
                        const int64_t iy = y * s + (int64_t)(i - r) * d;       \
                        if (iy < 0 || iy >= H) continue;                       \
                        for (int j = 0; j < k; ++j) {                          \
                            const int64_t ix = xo * s + (int64_t)(j - r) * d;  \
                            if (ix < 0 || ix >= W) continue;                   \
                            const int t = i * k + j;                           \
                            const T a = cfp[t];                                \
                            const T b = sfp[(t * Ho + y) * Wo + xo];           \
                            const T w = combine == DDF_MUL ? a * b : a + b;    \
                            acc += xp[iy * W + ix] * w;                        \
                        }                                                      \
                    }                                                          \
                    op[y * Wo + xo] = acc;                                     \
                }                                                              \
        }                                                                      \
    }                                                                          \
                                                                               \
    /* dX[n,c,u,v] = sum over taps (i,j) with q = ((u-(i-r)d)/s, (v-(j-r)d)/s) \
     * integral and inside the output: dO[n,c,q] * comb(CF[n,c,i,j], SF[n,t,q]) */ \
    void ddf_oracle_backward_features_##SUFFIX(                                \
        const T *go, const T *cf, const T *sf, T *dx, int64_t N, int64_t C,    \
        int64_t H, int64_t W, int k, int d, int s, int combine) {              \
        const int64_t Ho = H / s, Wo = W / s;                                  \
        const int r = (k - 1) / 2, kk = k * k;                                 \
        _Pragma("omp parallel for schedule(static)")                           \
        for (int64_t nc = 0; nc < N * C; ++nc) {                               \
            const int64_t n = nc / C;                                          \
            const T *gp = go + nc * Ho * Wo;                                   \
            const T *cfp = cf + nc * kk;                                       \
            const T *sfp = sf + n * kk * Ho * Wo;                              \
            T *dxp = dx + nc * H * W;                                          \
            for (int64_t u = 0; u < H; ++u)                                    \
                for (int64_t v = 0; v < W; ++v) {                              \
                    T acc = 0;                                                 \
                    for (int i = 0; i < k; ++i) {                              \
                        const int64_t ty = u - (int64_t)(i - r) * d;           \
                        if (ty < 0 || ty % s != 0) continue;                   \
                        const int64_t qy = ty / s;                             \
                        if (qy >= Ho) continue;                                \
                        for (int j = 0; j < k; ++j) {                          \
                            const int64_t tx = v - (int64_t)(j - r) * d;       \
                            if (tx < 0 || tx % s != 0) continue;               \
                            const int64_t qx = tx / s;                         \
                            if (qx >= Wo) continue;                            \
                            const int t = i * k + j;                           \
                            const T a = cfp[t];                                \
                            const T b = sfp[(t * Ho + qy) * Wo + qx];          \
                            const T w = combine == DDF_MUL ? a * b : a + b;    \
                            acc += gp[qy * Wo + qx] * w;                       \
                        }                                                      \
                    }                                                          \
                    dxp[u * W + v] = acc;                                      \
                }                                                              \
        }                                                                      \
    }                                                                          \
                                                                               \
    /* dCF[n,c,i,j] = sum_{y,x} dO[n,c,y,x] * X[n,c,y*s+(i-r)d,x*s+(j-r)d]     \
     *                          * (SF[n,t,y,x] for mul, 1 for add) */          \
    void ddf_oracle_backward_channel_filter_##SUFFIX(                          \
        const T *go, const T *x, const T *sf, T *dcf, int64_t N, int64_t C,    \
        int64_t H, int64_t W, int k, int d, int s, int combine) {              \
        const int64_t Ho = H / s, Wo = W / s;                                  \
        const int r = (k - 1) / 2, kk = k * k;                                 \
        _Pragma("omp parallel for schedule(static)")                           \
        for (int64_t nc = 0; nc < N * C; ++nc) {                               \
            const int64_t n = nc / C;                                          \
            const T *gp = go + nc * Ho * Wo;                                   \
            const T *xp = x + nc * H * W;                                      \
            const T *sfp = sf + n * kk * Ho * Wo;                              \
            for (int i = 0; i < k; ++i)                                        \
                for (int j = 0; j < k; ++j) {                                  \
                    const int t = i * k + j;                                   \
                    T acc = 0;                                                 \
                    for (int64_t y = 0; y < Ho; ++y) {                         \
                        const int64_t iy = y * s + (int64_t)(i - r) * d;       \
                        if (iy < 0 || iy >= H) continue;                       \
                        for (int64_t xo = 0; xo < Wo; ++xo) {                  \
                            const int64_t ix = xo * s + (int64_t)(j - r) * d;  \
                            if (ix < 0 || ix >= W) continue;                   \
                            T term = gp[y * Wo + xo] * xp[iy * W + ix];        \
                            if (combine == DDF_MUL)                            \
                                term *= sfp[(t * Ho + y) * Wo + xo];           \
                            acc += term;                                       \
                        }                                                      \
                    }                                                          \
                    dcf[nc * kk + t] = acc;                                    \
                }                                                              \
        }                                                                      \
    }                                                                          \
                                                                               \
    /* dSF[n,t,y,x] = sum_c dO[n,c,y,x] * X[n,c,y*s+(i-r)d,x*s+(j-r)d]         \
     *                      * (CF[n,c,i,j] for mul, 1 for add) */              \
    void ddf_oracle_backward_spatial_filter_##SUFFIX(                          \
        const T *go, const T *x, const T *cf, T *dsf, int64_t N, int64_t C,    \
        int64_t H, int64_t W, int k, int d, int s, int combine) {              \
        const int64_t Ho = H / s, Wo = W / s;                                  \
        const int r = (k - 1) / 2, kk = k * k;                                 \
        _Pragma("omp parallel for schedule(static)")                           \
        for (int64_t nt = 0; nt < N * kk; ++nt) {                              \
            const int64_t n = nt / kk;                                         \
            const int t = (int)(nt % kk);                                      \
            const int i = t / k, j = t % k;                                    \
            for (int64_t y = 0; y < Ho; ++y) {                                 \
                const int64_t iy = y * s + (int64_t)(i - r) * d;               \
                for (int64_t xo = 0; xo < Wo; ++xo) {                          \
                    const int64_t ix = xo * s + (int64_t)(j - r) * d;          \
                    T acc = 0;                                                 \
                    if (iy >= 0 && iy < H && ix >= 0 && ix < W) {              \
                        for (int64_t c = 0; c < C; ++c) {                      \
                            const int64_t nc = n * C + c;                      \
                            T term = go[(nc * Ho + y) * Wo + xo] *             \
                                     x[(nc * H + iy) * W + ix];                \
                            if (combine == DDF_MUL) term *= cf[nc * kk + t];   \
                            acc += term;                                       \
                        }                                                      \
                    }                                                          \
                    dsf[(nt * Ho + y) * Wo + xo] = acc;                        \
                }                                                              \
            }                                                                  \
        }                                                                      \
    }

DEFINE_ORACLE(double, f64)
DEFINE_ORACLE(float, f32)

/* Number of OpenMP threads the loops above use (1 when built without it). */
#ifdef _OPENMP
#include <omp.h>
int ddf_oracle_num_threads(void) { return omp_get_max_threads(); }
void ddf_oracle_set_num_threads(int n) { if (n > 0) omp_set_num_threads(n); }
#else
int ddf_oracle_num_threads(void) { return 1; }
void ddf_oracle_set_num_threads(int n) { (void)n; }
#endif
