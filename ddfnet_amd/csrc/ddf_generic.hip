// Generic DDF kernels: any odd kernel size, dilation and stride, every dtype.
// One thread per result element (forward, dX, dSF) or one workgroup per
// (n, c) plane (dCF).  They read the NCHW tensors directly from global memory;
// neighbouring lanes always touch neighbouring x, so loads and stores are
// coalesced without any layout shuffle.  These are the kernels behind
// DDF_VARIANT_GENERIC (the reference's version 'o',
// ddf/src/cuda/ddf_mul_cuda_kernel.cu:85-165, :198-420) and the fallback for
// shapes the tiled family does not cover.
#include "ddf_common.h"

namespace ddf {
namespace {

constexpr int kThreads = 256;

template <typename T, bool MUL>
__global__ __launch_bounds__(kThreads) void k_forward(
    Problem p, const T *__restrict__ x, const T *__restrict__ cf,
    const T *__restrict__ sf, T *__restrict__ out, int64_t total) {
    using A = typename Acc<T>::type;
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= total) return;
    const int64_t plane = p.Ho * p.Wo;
    const int64_t nc = idx / plane;
    const int64_t pix = idx - nc * plane;
    const int64_t y = pix / p.Wo, xo = pix - y * p.Wo;
    const int64_t n = nc / p.C;
    const T *xp = x + nc * p.H * p.W;
    const T *cfp = cf + nc * p.kk;
    const T *sfp = sf + n * p.kk * plane + pix;
    A acc = 0;
    for (int i = 0; i < p.k; ++i) {
        const int64_t iy = y * p.s + (int64_t)(i - p.r) * p.d;
        if (iy < 0 || iy >= p.H) continue;
        for (int j = 0; j < p.k; ++j) {
            const int64_t ix = xo * p.s + (int64_t)(j - p.r) * p.d;
            if (ix < 0 || ix >= p.W) continue;
            const int t = i * p.k + j;
            const A w = comb<MUL, A>(ld(cfp + t), ld(sfp + t * plane));
            acc += ld(xp + iy * p.W + ix) * w;
        }
    }
    st(out + idx, acc);
}

// dX[n,c,u,v]: gather over the taps whose window centre lands on an output
// pixel q = ((u-(i-r)d)/s, (v-(j-r)d)/s).
template <typename T, bool MUL>
__global__ __launch_bounds__(kThreads) void k_backward_features(
    Problem p, const T *__restrict__ go, const T *__restrict__ cf,
    const T *__restrict__ sf, T *__restrict__ dx, int64_t total) {
    using A = typename Acc<T>::type;
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= total) return;
    const int64_t iplane = p.H * p.W, oplane = p.Ho * p.Wo;
    const int64_t nc = idx / iplane;
    const int64_t pix = idx - nc * iplane;
    const int64_t u = pix / p.W, v = pix - u * p.W;
    const int64_t n = nc / p.C;
    const T *gp = go + nc * oplane;
    const T *cfp = cf + nc * p.kk;
    const T *sfp = sf + n * p.kk * oplane;
    A acc = 0;
    for (int i = 0; i < p.k; ++i) {
        const int64_t ty = u - (int64_t)(i - p.r) * p.d;
        if (ty < 0 || ty % p.s != 0) continue;
        const int64_t qy = ty / p.s;
        if (qy >= p.Ho) continue;
        for (int j = 0; j < p.k; ++j) {
            const int64_t tx = v - (int64_t)(j - p.r) * p.d;
            if (tx < 0 || tx % p.s != 0) continue;
            const int64_t qx = tx / p.s;
            if (qx >= p.Wo) continue;
            const int t = i * p.k + j;
            const int64_t q = qy * p.Wo + qx;
            const A w = comb<MUL, A>(ld(cfp + t), ld(sfp + t * oplane + q));
            acc += ld(gp + q) * w;
        }
    }
    st(dx + idx, acc);
}

template <typename A>
__device__ __forceinline__ A wave_sum(A v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_down(v, off, kWave);
    return v;
}

// dCF[n,c,t]: one workgroup per (n,c) plane; each tap is a sum over Ho*Wo.
template <typename T, bool MUL>
__global__ __launch_bounds__(kThreads) void k_backward_channel_filter(
    Problem p, const T *__restrict__ go, const T *__restrict__ x,
    const T *__restrict__ sf, T *__restrict__ dcf) {
    using A = typename Acc<T>::type;
    __shared__ A part[kThreads / kWave];
    const int64_t nc = blockIdx.x;
    const int64_t n = nc / p.C;
    const int64_t oplane = p.Ho * p.Wo;
    const T *gp = go + nc * oplane;
    const T *xp = x + nc * p.H * p.W;
    const T *sfp = sf + n * p.kk * oplane;
    for (int t = 0; t < p.kk; ++t) {
        const int i = t / p.k, j = t - i * p.k;
        const int64_t oy = (int64_t)(i - p.r) * p.d, ox = (int64_t)(j - p.r) * p.d;
        A acc = 0;
        for (int64_t pix = threadIdx.x; pix < oplane; pix += kThreads) {
            const int64_t y = pix / p.Wo, xo = pix - y * p.Wo;
            const int64_t iy = y * p.s + oy, ix = xo * p.s + ox;
            if (iy < 0 || iy >= p.H || ix < 0 || ix >= p.W) continue;
            A term = ld(gp + pix) * ld(xp + iy * p.W + ix);
            if (MUL) term *= ld(sfp + t * oplane + pix);
            acc += term;
        }
        acc = wave_sum(acc);
        if ((threadIdx.x & (kWave - 1)) == 0) part[threadIdx.x / kWave] = acc;
        __syncthreads();
        if (threadIdx.x == 0) {
            A tot = 0;
#pragma unroll
            for (int w = 0; w < kThreads / kWave; ++w) tot += part[w];
            st(dcf + nc * p.kk + t, tot);
        }
        __syncthreads();
    }
}

// dSF[n,t,y,x]: one thread per element, serial sum over channels.
template <typename T, bool MUL>
__global__ __launch_bounds__(kThreads) void k_backward_spatial_filter(
    Problem p, const T *__restrict__ go, const T *__restrict__ x,
    const T *__restrict__ cf, T *__restrict__ dsf, int64_t total) {
    using A = typename Acc<T>::type;
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= total) return;
    const int64_t oplane = p.Ho * p.Wo, iplane = p.H * p.W;
    const int64_t nt = idx / oplane;
    const int64_t pix = idx - nt * oplane;
    const int64_t n = nt / p.kk;
    const int t = (int)(nt - n * p.kk);
    const int i = t / p.k, j = t - i * p.k;
    const int64_t y = pix / p.Wo, xo = pix - y * p.Wo;
    const int64_t iy = y * p.s + (int64_t)(i - p.r) * p.d;
    const int64_t ix = xo * p.s + (int64_t)(j - p.r) * p.d;
    A acc = 0;
    if (iy >= 0 && iy < p.H && ix >= 0 && ix < p.W) {
        const T *gp = go + n * p.C * oplane + pix;
        const T *xp = x + n * p.C * iplane + iy * p.W + ix;
        const T *cfp = cf + n * p.C * p.kk + t;
        for (int64_t c = 0; c < p.C; ++c) {
            A term = ld(gp + c * oplane) * ld(xp + c * iplane);
            if (MUL) term *= ld(cfp + c * p.kk);
            acc += term;
        }
    }
    st(dsf + idx, acc);
}

constexpr int64_t kMaxGrid = 2147483647;

}  // namespace

template <typename T>
hipError_t generic_forward(const Problem &p, const T *x, const T *cf, const T *sf,
                           T *out, hipStream_t stream) {
    const int64_t total = p.N * p.C * p.Ho * p.Wo;
    if (total == 0) return hipSuccess;
    const int64_t grid = cdiv(total, kThreads);
    if (grid > kMaxGrid) return hipErrorInvalidConfiguration;
    if (p.mul)
        hipLaunchKernelGGL((k_forward<T, true>), dim3((unsigned)grid), dim3(kThreads), 0,
                           stream, p, x, cf, sf, out, total);
    else
        hipLaunchKernelGGL((k_forward<T, false>), dim3((unsigned)grid), dim3(kThreads), 0,
                           stream, p, x, cf, sf, out, total);
    return hipGetLastError();
}

template <typename T>
hipError_t generic_backward(const Problem &p, const T *go, const T *x, const T *cf,
                            const T *sf, T *dx, T *dcf, T *dsf, unsigned need,
                            hipStream_t stream) {
    hipError_t err = hipSuccess;
    const int64_t n_dx = p.N * p.C * p.H * p.W;
    const int64_t n_dsf = p.N * p.kk * p.Ho * p.Wo;
    const int64_t n_planes = p.N * p.C;
    if ((need & DDF_NEED_DX) && n_dx > 0) {
        const int64_t grid = cdiv(n_dx, kThreads);
        if (grid > kMaxGrid) return hipErrorInvalidConfiguration;
        if (p.mul)
            hipLaunchKernelGGL((k_backward_features<T, true>), dim3((unsigned)grid),
                               dim3(kThreads), 0, stream, p, go, cf, sf, dx, n_dx);
        else
            hipLaunchKernelGGL((k_backward_features<T, false>), dim3((unsigned)grid),
                               dim3(kThreads), 0, stream, p, go, cf, sf, dx, n_dx);
        if ((err = hipGetLastError()) != hipSuccess) return err;
    }
    if ((need & DDF_NEED_DCF) && n_planes > 0) {
        if (n_planes > kMaxGrid) return hipErrorInvalidConfiguration;
        if (p.mul)
            hipLaunchKernelGGL((k_backward_channel_filter<T, true>),
                               dim3((unsigned)n_planes), dim3(kThreads), 0, stream, p, go,
                               x, sf, dcf);
        else
            hipLaunchKernelGGL((k_backward_channel_filter<T, false>),
                               dim3((unsigned)n_planes), dim3(kThreads), 0, stream, p, go,
                               x, sf, dcf);
        if ((err = hipGetLastError()) != hipSuccess) return err;
    }
    if ((need & DDF_NEED_DSF) && n_dsf > 0) {
        const int64_t grid = cdiv(n_dsf, kThreads);
        if (grid > kMaxGrid) return hipErrorInvalidConfiguration;
        if (p.mul)
            hipLaunchKernelGGL((k_backward_spatial_filter<T, true>), dim3((unsigned)grid),
                               dim3(kThreads), 0, stream, p, go, x, cf, dsf, n_dsf);
        else
            hipLaunchKernelGGL((k_backward_spatial_filter<T, false>), dim3((unsigned)grid),
                               dim3(kThreads), 0, stream, p, go, x, cf, dsf, n_dsf);
        if ((err = hipGetLastError()) != hipSuccess) return err;
    }
    return err;
}

#define INSTANTIATE(T)                                                                   \
    template hipError_t generic_forward<T>(const Problem &, const T *, const T *,        \
                                           const T *, T *, hipStream_t);                 \
    template hipError_t generic_backward<T>(const Problem &, const T *, const T *,       \
                                            const T *, const T *, T *, T *, T *,         \
                                            unsigned, hipStream_t);
INSTANTIATE(__half)
INSTANTIATE(float)
INSTANTIATE(double)

}  // namespace ddf
