// Shared declarations of the DDF HIP library (gfx950 only, wave64).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ddf_hip.h"

namespace ddf {

constexpr int kWave = 64;

// Problem description handed to every launcher.  Ho/Wo use floor division
// (ddf/ddf.py:56 of the reference), r is the tap radius in taps.
struct Problem {
    int64_t N, C, H, W, Ho, Wo;
    int k, d, s, r, kk;
    bool mul;
};

inline Problem make_problem(int64_t N, int64_t C, int64_t H, int64_t W, int k,
                            int d, int s, int combine) {
    Problem p;
    p.N = N; p.C = C; p.H = H; p.W = W;
    p.Ho = H / s; p.Wo = W / s;
    p.k = k; p.d = d; p.s = s; p.r = (k - 1) / 2; p.kk = k * k;
    p.mul = (combine == DDF_MUL);
    return p;
}

// Accumulator type: fp16 and fp32 storage accumulate in fp32, fp64 in fp64.
template <typename T> struct Acc { using type = float; };
template <> struct Acc<double> { using type = double; };

__device__ __forceinline__ float ld(const __half *p) { return __half2float(*p); }
__device__ __forceinline__ float ld(const float *p) { return *p; }
__device__ __forceinline__ double ld(const double *p) { return *p; }
__device__ __forceinline__ void st(__half *p, float v) { *p = __float2half(v); }
__device__ __forceinline__ void st(float *p, float v) { *p = v; }
__device__ __forceinline__ void st(double *p, double v) { *p = v; }

template <bool MUL, typename A>
__device__ __forceinline__ A comb(A a, A b) { return MUL ? a * b : a + b; }

inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// The spatial filter normalisation behind the spatial-filter gradient (FilterNorm
// of the spatial branch, ddf/ddf.py:146-157 of the reference: the operator's
// spatial filter is gain * standardised(raw) over the k*k taps of a pixel).  A
// backward pass that is handed one pushes dSF through the normalisation's
// Jacobian in the pass that adds up its partial sums and writes d_raw instead;
// `applied` tells the caller whether that happened (else dSF is complete where
// the pass was told to put it, and the caller runs filter_norm_backward).
template <typename T>
struct NormTail {
    const T *raw;          // (N, k*k, Ho, Wo), before the normalisation
    T *d_raw;              // gradient with respect to raw
    T *terms;              // nullable: dSF * standardised(raw), summed by the caller into the gain_vec gradient
    const T *gain_vec;     // nullable: (groups, k*k); sample n uses group n % groups
    int groups;
    double gain;           // used when gain_vec is null
    bool applied;
};

// Launchers.  Each returns a hipError_t from the launch (hipSuccess when the
// tensor is empty and nothing was launched).  `supported` queries tell the
// API layer whether the tiled family covers a problem.
template <typename T>
hipError_t generic_forward(const Problem &p, const T *x, const T *cf, const T *sf,
                           T *out, hipStream_t st);
template <typename T>
hipError_t generic_backward(const Problem &p, const T *go, const T *x, const T *cf,
                            const T *sf, T *dx, T *dcf, T *dsf, unsigned need,
                            hipStream_t st);

// y = gain * standardised(x) + offset over the `taps` axis of an
// (outer, groups, taps, inner) tensor; gain_vec / offset_vec are (groups, taps)
// or null (then the scalar `gain` / no offset).
template <typename T>
hipError_t filter_norm(const T *x, T *y, int64_t outer, int64_t groups, int taps, int64_t inner,
                       double gain, const T *gain_vec, const T *offset_vec, hipStream_t st);

// Gradient of filter_norm with respect to x; `terms` (nullable) receives
// dy * standardised(x), whose sum over (outer, inner) is the gain_vec gradient.
template <typename T>
hipError_t filter_norm_backward(const T *dy, const T *x, T *dx, T *terms, int64_t outer,
                                int64_t groups, int taps, int64_t inner, double gain,
                                const T *gain_vec, hipStream_t st);

// The filter branches of DDFPack, one launch each (ddf_branches.hip): 1x1
// convolution (stride as the operator's) + spatial filter normalisation, and
// bottleneck MLP on the pooled features + channel filter normalisation.
// hipErrorNotSupported: kernel size or sizes not covered, nothing launched.
bool branch_kernel_size_built(int k);
template <typename T>
// pool_part (may be null): the launch also leaves the sums of the feature map over
// the pixels of each of *pool_parts parts of a plane, fp32, [(n * parts + p) * C + c]; at most
// pool_capacity floats.  hipErrorNotSupported where no kernel does that.
hipError_t spatial_branch(const T *x, const T *w, const T *bias, T *sf, int64_t N, int64_t C,
                          int64_t H, int64_t W, int head, int k, int stride, double gain,
                          const T *gain_vec, const T *offset_vec, hipStream_t st,
                          float *pool_part = nullptr, int64_t pool_capacity = 0,
                          int *pool_parts = nullptr);
// parts (may be null): the pooled vectors are scale * the sums of nparts such partial
// sums instead of `pooled`.
template <typename T>
hipError_t channel_branch(const T *pooled, const T *w1, const T *b1, const T *w2, const T *b2,
                          T *cf, int64_t N, int64_t C, int64_t mid, int k, double gain,
                          const T *gain_vec, const T *offset_vec, hipStream_t st,
                          const float *parts = nullptr, int nparts = 0, double scale = 1.0);

// All scale*scale sub-pixel branches of an up-sampling DDF in one launch,
// written into the pixel-shuffled (N, C, H*scale, W*scale) result; cf / sf are
// host arrays of scale*scale device pointers.
bool up_forward_supported(int64_t H, int64_t W, int k, int d, int scale);
template <typename T>
hipError_t up_forward(int64_t N, int64_t C, int64_t H, int64_t W, int k, int d, int scale,
                      bool mul, const T *x, const void *const *cf, const void *const *sf, T *out,
                      hipStream_t st);

// Helpers of the up-sampling backward: the gradient of the pixel shuffle (dO
// split into its scale*scale sub-pixel lattices, stored back to back) and the
// sum of `parts` equally sized tensors stored back to back.
template <typename T>
hipError_t up_split_lattices(const T *go, T *lat, int64_t planes, int64_t H, int64_t W, int scale,
                             hipStream_t st);
template <typename T>
hipError_t up_sum_parts(const T *in, T *out, int64_t count, int parts, hipStream_t st);
// For the backward pass of all branches as one batch: the branches' filters
// copied back to back (cf / sf: host arrays of `branches` device pointers), and
// afterwards dX summed from the branches' parts (parts may be null) together
// with the batch's filter gradients copied out to the branches' tensors (null
// destinations are skipped; dcf_all / dsf_all may be null).
template <typename T>
hipError_t up_gather_filters(const void *const *cf, const void *const *sf, T *cf_all, T *sf_all,
                             int64_t n_cf, int64_t n_sf, int branches, hipStream_t st);
template <typename T>
hipError_t up_finish(const T *parts, T *dx, int64_t n_x, int branches, const T *dcf_all,
                     const T *dsf_all, void *const *dcfs, void *const *dsfs, int64_t n_cf,
                     int64_t n_sf, hipStream_t st);

// Tiny planes (H*W <= 64), 3x3, stride 1: forward (backward = false: x -> out)
// and feature gradient (backward = true: dO -> dX), G = 256 / (H*W) channel
// planes per workgroup pass.
bool small_supported(const Problem &p);
template <typename T>
hipError_t small_launch(const Problem &p, bool backward, const T *x, const T *cf, const T *sf,
                        T *out, hipStream_t st);

// Row-register kernels (stride 1; rows that are a whole number of vectors):
// forward (backward = false: x -> out) or feature gradient (backward = true:
// dO -> dX).  hipErrorNotSupported when the family does not cover the problem
// or a pointer is not aligned to its vectors; nothing was launched then.
template <typename T>
hipError_t rows_launch(const Problem &p, bool backward, const T *x, const T *cf, const T *sf,
                       T *out, hipStream_t st);

// Filter gradients (dCF, dSF) on the row-register kernel; same conventions.
// With dx != nullptr the launch also writes the feature gradient (the whole
// backward pass in one kernel, 3x3 without dilation).  The workspace
// (rows_filters_workspace bytes, 256-byte aligned) holds the partial sums over
// channel splits and strips.
size_t rows_filters_workspace(const Problem &p, int dtype, unsigned need);
// The row-register kernels cover the feature gradient and, in a launch of its
// own, the filter gradients of this problem (pointer alignment assumed).
bool rows_cover_backward(const Problem &p, int dtype);
// Stride 2: the row-register kernels cover the filter gradients, and (even feature
// heights) the feature gradient asked for alone.
bool rows_cover_stride2_filters(const Problem &p, int dtype);
inline bool rows_stride2_feature_gradient(const Problem &p) { return p.s == 2 && p.H % 2 == 0; }
// x_mod != 0: the batch p.N is several groups of x_mod samples sharing one set
// of features x (x_mod samples long); everything else is indexed by the sample.
template <typename T>
hipError_t rows_filters_launch(const Problem &p, const T *go, const T *x, const T *cf, const T *sf,
                               T *dx, T *dcf, T *dsf, void *ws, unsigned need, hipStream_t st,
                               int x_mod = 0, NormTail<T> *norm = nullptr);
// The whole backward pass of such a batch on the row-register kernels, or
// hipErrorNotSupported before anything is launched (shape or alignment not
// covered).  `ws`: rows_filters_workspace(p) bytes.
template <typename T>
hipError_t rows_backward_shared_features(const Problem &p, int x_mod, const T *go, const T *x,
                                         const T *cf, const T *sf, T *dx, T *dcf, T *dsf, void *ws,
                                         unsigned need, hipStream_t st);

// Names of the kernels a forward / backward call on the tiled families would
// launch, written into buf (at most len bytes); returns snprintf's count.
int describe_forward(const Problem &p, int dtype, char *buf, int len);
int describe_backward(const Problem &p, int dtype, unsigned need, char *buf, int len);

bool tiled_forward_supported(const Problem &p, int dtype);
template <typename T>
hipError_t tiled_forward(const Problem &p, const T *x, const T *cf, const T *sf,
                         T *out, hipStream_t st);

bool tiled_backward_supported(const Problem &p, int dtype);
size_t tiled_backward_workspace(const Problem &p, int dtype, unsigned need);
template <typename T>
hipError_t tiled_backward(const Problem &p, const T *go, const T *x, const T *cf,
                          const T *sf, T *dx, T *dcf, T *dsf, void *ws,
                          unsigned need, hipStream_t st, NormTail<T> *norm = nullptr);

}  // namespace ddf
