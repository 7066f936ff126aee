// Filter normalisation of the two DDF branches as one kernel:
//   y[o, g, t, i] = gain[g, t] * (x[o, g, t, i] - mean_t) / (std_t + 1e-10) + offset[g, t]
// with mean_t / std_t taken over the `taps` values t of one filter (std is the
// unbiased estimate, n - 1 in the denominator).  It restates FilterNorm.forward
// of the reference (ddf/ddf.py:145-173): the spatial branch is
// (outer, groups, taps, inner) = (b, head, k*k, h*w), the channel branch is
// (b, c, k*k, 1).  One thread per filter; in the spatial case neighbouring
// threads are neighbouring pixels, so every tap plane is read and written
// with coalesced accesses.  Arithmetic is fp32 (fp64 for double tensors).
#include "ddf_common.h"

namespace ddf {
namespace {

template <typename T>
__global__ __launch_bounds__(256) void k_filter_norm(
    const T *__restrict__ x, T *__restrict__ y, int64_t filters, int64_t groups, int taps,
    int64_t inner, double gain, const T *__restrict__ gain_vec, const T *__restrict__ offset_vec) {
    using A = typename Acc<T>::type;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= filters) return;
    const int64_t og = idx / inner, i = idx - og * inner;
    const int64_t g = og % groups;
    const T *xp = x + og * taps * inner + i;
    T *yp = y + og * taps * inner + i;
    A sum = 0;
    for (int t = 0; t < taps; ++t) sum += (A)ld(xp + (int64_t)t * inner);
    const A mean = sum / (A)taps;
    A sq = 0;
    for (int t = 0; t < taps; ++t) {
        const A dlt = (A)ld(xp + (int64_t)t * inner) - mean;
        sq += dlt * dlt;
    }
    // torch.std of a single value is NaN (0 / 0); keep that
    const A sd = sqrt(sq / (A)(taps - 1));
    const A inv = (A)1 / (sd + (A)1e-10);
    for (int t = 0; t < taps; ++t) {
        const A w = gain_vec ? (A)ld(gain_vec + g * taps + t) : (A)gain;
        A v = ((A)ld(xp + (int64_t)t * inner) - mean) * inv * w;
        if (offset_vec) v += (A)ld(offset_vec + g * taps + t);
        st(yp + (int64_t)t * inner, v);
    }
}

// Gradient of the normalisation above with respect to x, recomputing mean and
// deviation from x.  With c_t = x_t - mean, inv = 1 / (sd + 1e-10),
// gy_t = dy_t * gain_t:
//   dx_t = inv * (gy_t - mean(gy)) - c_t * inv^2 * sum(gy * c) / (sd * (taps - 1))
// `terms`, when not null, receives dy_t * z_t (z the standardised value); its
// sum over (outer, inner) is the gradient of gain_vec.
template <typename T>
__global__ __launch_bounds__(256) void k_filter_norm_backward(
    const T *__restrict__ dy, const T *__restrict__ x, T *__restrict__ dx, T *__restrict__ terms,
    int64_t filters, int64_t groups, int taps, int64_t inner, double gain,
    const T *__restrict__ gain_vec) {
    using A = typename Acc<T>::type;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= filters) return;
    const int64_t og = idx / inner, i = idx - og * inner;
    const int64_t g = og % groups;
    const int64_t base = og * taps * inner + i;
    A sum = 0;
    for (int t = 0; t < taps; ++t) sum += (A)ld(x + base + (int64_t)t * inner);
    const A mean = sum / (A)taps;
    A sq = 0, s1 = 0, s2 = 0;
    for (int t = 0; t < taps; ++t) {
        const A c = (A)ld(x + base + (int64_t)t * inner) - mean;
        const A w = gain_vec ? (A)ld(gain_vec + g * taps + t) : (A)gain;
        const A gy = (A)ld(dy + base + (int64_t)t * inner) * w;
        sq += c * c;
        s1 += gy;
        s2 += gy * c;
    }
    const A sd = sqrt(sq / (A)(taps - 1));
    const A inv = (A)1 / (sd + (A)1e-10);
    const A m1 = s1 / (A)taps;
    const A k2 = inv * inv * s2 / (sd * (A)(taps - 1));
    for (int t = 0; t < taps; ++t) {
        const A c = (A)ld(x + base + (int64_t)t * inner) - mean;
        const A d = (A)ld(dy + base + (int64_t)t * inner);
        const A w = gain_vec ? (A)ld(gain_vec + g * taps + t) : (A)gain;
        st(dx + base + (int64_t)t * inner, inv * (d * w - m1) - c * k2);
        if (terms) st(terms + base + (int64_t)t * inner, d * c * inv);
    }
}

}  // namespace

template <typename T>
hipError_t filter_norm_backward(const T *dy, const T *x, T *dx, T *terms, int64_t outer,
                                int64_t groups, int taps, int64_t inner, double gain,
                                const T *gain_vec, hipStream_t stream) {
    const int64_t filters = outer * groups * inner;
    if (filters == 0 || taps == 0) return hipSuccess;
    const int64_t grid = cdiv(filters, 256);
    if (grid > 2147483647) return hipErrorInvalidConfiguration;
    hipLaunchKernelGGL((k_filter_norm_backward<T>), dim3((unsigned)grid), dim3(256), 0, stream, dy,
                       x, dx, terms, filters, groups, taps, inner, gain, gain_vec);
    return hipGetLastError();
}

template hipError_t filter_norm_backward<__half>(const __half *, const __half *, __half *, __half *,
                                                 int64_t, int64_t, int, int64_t, double,
                                                 const __half *, hipStream_t);
template hipError_t filter_norm_backward<float>(const float *, const float *, float *, float *,
                                                int64_t, int64_t, int, int64_t, double,
                                                const float *, hipStream_t);
template hipError_t filter_norm_backward<double>(const double *, const double *, double *, double *,
                                                 int64_t, int64_t, int, int64_t, double,
                                                 const double *, hipStream_t);

template <typename T>
hipError_t filter_norm(const T *x, T *y, int64_t outer, int64_t groups, int taps, int64_t inner,
                       double gain, const T *gain_vec, const T *offset_vec, hipStream_t stream) {
    const int64_t filters = outer * groups * inner;
    if (filters == 0 || taps == 0) return hipSuccess;
    const int64_t grid = cdiv(filters, 256);
    if (grid > 2147483647) return hipErrorInvalidConfiguration;
    hipLaunchKernelGGL((k_filter_norm<T>), dim3((unsigned)grid), dim3(256), 0, stream, x, y, filters,
                       groups, taps, inner, gain, gain_vec, offset_vec);
    return hipGetLastError();
}

template hipError_t filter_norm<__half>(const __half *, __half *, int64_t, int64_t, int, int64_t,
                                        double, const __half *, const __half *, hipStream_t);
template hipError_t filter_norm<float>(const float *, float *, int64_t, int64_t, int, int64_t, double,
                                       const float *, const float *, hipStream_t);
template hipError_t filter_norm<double>(const double *, double *, int64_t, int64_t, int, int64_t,
                                        double, const double *, const double *, hipStream_t);

}  // namespace ddf
