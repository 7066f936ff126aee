// DDF forward and feature gradient for tiny planes (H*W <= 64, e.g. the 7x7
// planes of the last ResNet stage), 3x3, stride 1.
//
// A plane this small fills neither the lanes of a wavefront nor a 16-byte
// access pattern of the tile kernels.  Here a workgroup of 256 threads covers
// G = 256 / (H*W) channel planes of one sample at a time: thread t works on
// pixel t % (H*W) of channel slot t / (H*W), so the G planes it touches form one
// contiguous run of G*H*W elements in X and in the result, read and written
// with fully coalesced accesses.  All threads of a block share the sample, so
// each keeps the K*K spatial taps of its pixel in registers; the channel taps
// of the block's chunk sit in LDS.  Per channel a thread reads its K*K
// neighbours from global memory (the cache serves the overlap), U channels'
// loads in flight at a time.
//
// The feature gradient is the same walk over dO with the taps reversed:
// dX[u] = sum_t dO[u - o_t] * comb(CF[t], SF[t, u - o_t]); the spatial taps a
// thread keeps are then those of the pixels its dO values come from
// (ddf/src/cuda/ddf_mul_cuda_kernel.cu:85-165 and :198-290 of the reference).
#include <algorithm>

#include "ddf_chunks.h"

namespace ddf {
int tune_int(const char *name, int fallback);

namespace {

using chunks::kThreads;
constexpr int kMaxPlane = chunks::kSmallMaxPlane;   // G >= 4 channel planes per pass

// Up to UU channels (G apart) of one pixel; `valid` of them exist (the others
// repeat the last one and store nothing, so the loads need no branch).  `xb` /
// `ob` are wave-uniform bases and `at` the element offset of this thread's
// pixel in its first channel: every access is base + 32-bit offset.  A
// neighbour outside the plane reads the pixel itself (offset 0) and is zeroed
// afterwards.
template <typename T, int K, bool MUL, int UU, typename A>
__device__ __forceinline__ void small_channels(const T *__restrict__ xb, T *__restrict__ ob,
                                               const A *__restrict__ w, unsigned at, unsigned step,
                                               int wstep, int valid, const int (&off)[K * K],
                                               const bool (&inside)[K * K], const A (&sfr)[K * K]) {
    constexpr int KK = K * K;
    A xv[UU][KK];
#pragma unroll
    for (int u = 0; u < UU; ++u) {
        const unsigned a = at + (unsigned)min(u, valid - 1) * step;
#pragma unroll
        for (int t = 0; t < KK; ++t) xv[u][t] = (A)ld(xb + (unsigned)(a + off[t]));
    }
#pragma unroll
    for (int u = 0; u < UU; ++u) {
        const int uu = min(u, valid - 1);
        A acc = 0;
#pragma unroll
        for (int t = 0; t < KK; ++t) {
            const A x = inside[t] ? xv[u][t] : (A)0;
            acc += x * comb<MUL, A>(w[uu * wstep + t], sfr[t]);
        }
        if (u < valid) st(ob + (at + u * step), acc);
    }
}

template <typename T, int K, bool MUL, bool BWD>
__global__ __launch_bounds__(kThreads) void k_small(
    const T *__restrict__ x, const T *__restrict__ cf, const T *__restrict__ sf,
    T *__restrict__ out, int C, int H, int W, int D, int G, int cpb, int csplit, int stage) {
    using A = typename Acc<T>::type;
    constexpr int KK = K * K, RAD = K / 2, U = 4, Q = 4;
    extern __shared__ __align__(16) unsigned char small_smem[];
    A *taps = reinterpret_cast<A *>(small_smem);   // [channel][tap]

    chunks::Block blk;
    blk.init(blockIdx.x, gridDim.x, csplit, 1, cpb, C);
    const int64_t n = blk.n;
    const int c0 = blk.c0, nch = blk.nch;
    const int plane = H * W;

    // threads past the G planes idle on slot 0 / pixel 0 and store nothing
    chunks::SmallThread th;
    th.init((int)threadIdx.x, plane, G);
    const int q = th.q, pix = th.pix;
    const int y = pix / W, xx = pix - y * W;

    // neighbours: offset from the pixel, whether inside; the spatial tap that
    // goes with each (forward: of this pixel; gradient: of the neighbour)
    int off[KK];
    bool inside[KK];
    A sfr[KK];
    const T *sfn = sf + n * KK * plane;
#pragma unroll
    for (int i = 0; i < K; ++i)
#pragma unroll
        for (int j = 0; j < K; ++j) {
            const int t = i * K + j;
            const int dy = BWD ? -(i - RAD) * D : (i - RAD) * D;
            const int dx = BWD ? -(j - RAD) * D : (j - RAD) * D;
            inside[t] = y + dy >= 0 && y + dy < H && xx + dx >= 0 && xx + dx < W;
            off[t] = inside[t] ? dy * W + dx : 0;
            const A v = (A)ld(sfn + (int64_t)t * plane + pix + (BWD ? off[t] : 0));
            sfr[t] = (BWD && !inside[t]) ? (A)0 : v;
        }

    const unsigned gstep = (unsigned)(G * plane);   // G channel planes further on
    const T *xc = x + (n * C + c0) * plane;          // wave-uniform bases of the chunk
    T *oc = out + (n * C + c0) * plane;
    for (int s0 = 0; s0 < nch; s0 += stage) {
        const int ns = min(stage, nch - s0);
        if (s0 > 0) __syncthreads();
        // channel taps of this stage (contiguous), Q loads per thread in flight
        const int total = ns * KK;
        const T *src = cf + (n * C + c0 + s0) * KK;
        for (int e0 = threadIdx.x; e0 < total; e0 += Q * kThreads) {
            A v[Q];
#pragma unroll
            for (int e = 0; e < Q; ++e) v[e] = (A)ld(src + min(e0 + e * kThreads, total - 1));
#pragma unroll
            for (int e = 0; e < Q; ++e)
                if (e0 + e * kThreads < total) taps[e0 + e * kThreads] = v[e];
        }
        __syncthreads();
        // this thread's channels of the stage: q, q + G, q + 2G, ...
        const int mine = th.channels(ns, G);
        const T *xs = xc + (int64_t)s0 * plane;
        T *os = oc + (int64_t)s0 * plane;
        const A *w = taps + q * KK;
        unsigned at = (unsigned)(q * plane + pix);
#pragma unroll 1
        for (int m = 0; m < mine; m += U, at += U * gstep, w += U * G * KK)
            small_channels<T, K, MUL, U, A>(xs, os, w, at, gstep, G * KK, min(U, mine - m), off,
                                            inside, sfr);
    }
}

template <typename T, bool BWD>
hipError_t launch(const Problem &p, const T *x, const T *cf, const T *sf, T *out,
                  hipStream_t stream) {
    using A = typename Acc<T>::type;
    chunks::ChunkGeom g;
    if (!chunks::small_chunks(p.N, p.C, (int)(p.H * p.W), (int)sizeof(A),
                              tune_int("DDF_TUNE_SMALL_BLOCKS", 1024), &g))
        return hipErrorInvalidConfiguration;
    auto kern = p.mul ? k_small<T, 3, true, BWD> : k_small<T, 3, false, BWD>;
    hipLaunchKernelGGL(kern, dim3((unsigned)g.blocks), dim3(kThreads), g.lds, stream, x, cf, sf, out,
                       (int)p.C, (int)p.H, (int)p.W, p.d, g.G, g.cpb, g.csplit, g.stage);
    return hipGetLastError();
}

}  // namespace

bool small_supported(const Problem &p) {
    if (tune_int("DDF_TUNE_SMALL", 1) == 0) return false;
    if (p.k != 3 || p.s != 1 || p.d > (1 << 10)) return false;
    if (p.H * p.W > kMaxPlane || p.C > (1 << 24)) return false;   // 32-bit offsets in a chunk
    return p.N * p.C * p.H * p.W > 0;
}

template <typename T>
hipError_t small_launch(const Problem &p, bool backward, const T *x, const T *cf, const T *sf,
                        T *out, hipStream_t st) {
    return backward ? launch<T, true>(p, x, cf, sf, out, st) : launch<T, false>(p, x, cf, sf, out, st);
}

template hipError_t small_launch<__half>(const Problem &, bool, const __half *, const __half *,
                                         const __half *, __half *, hipStream_t);
template hipError_t small_launch<float>(const Problem &, bool, const float *, const float *,
                                        const float *, float *, hipStream_t);
template hipError_t small_launch<double>(const Problem &, bool, const double *, const double *,
                                         const double *, double *, hipStream_t);

}  // namespace ddf
