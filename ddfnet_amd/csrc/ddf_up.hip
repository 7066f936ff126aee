// Up-sampling DDF forward: the scale*scale filter branches of DDFUpPack in one
// launch, written straight into the pixel-shuffled result.
//
// The reference (ddf/ddf.py:257-272) runs `ddf` once per sub-pixel branch b on
// the same features, stacks the scale^2 results and pixel-shuffles them:
//   out[n, c, y*R + i, x*R + j] = ddf(X, CF_b, SF_b)[n, c, y, x],  b = i*R + j.
// Here one thread owns an input pixel (y, x) of one sample and walks over a
// chunk of channels.  It keeps the K*K spatial taps of all R*R branches in
// registers, reads the K*K neighbours of X once per channel and uses them for
// every branch, and writes R rows of R neighbouring results, so X is read once
// instead of R*R times and the result is written once, in place.  Neighbouring
// lanes are neighbouring pixels: every global access is coalesced.  The channel
// taps of the block's chunk sit in LDS in accumulator precision and are read
// with wave-uniform (broadcast) addresses.
#include <algorithm>

#include "ddf_common.h"

namespace ddf {
namespace {

constexpr int kThreads = 256;
constexpr int kStageChannels = 32;     // channels whose taps are staged in LDS at a time
constexpr int kStageBytes = 32 * 1024;  // and the LDS they may take

template <typename T>
struct UpFilters {
    const T *cf[DDF_UP_MAX_BRANCHES];
    const T *sf[DDF_UP_MAX_BRANCHES];
};

template <typename T, int R>
struct alignas((R & (R - 1)) == 0 ? sizeof(T) * R : sizeof(T)) Row {
    T e[R];
};

// Workgroups reach the 8 XCDs round-robin; renumber so that consecutive
// logical blocks (same sample and pixel block, neighbouring channel chunks,
// hence the same spatial taps) run on one XCD and share its L2.
__device__ __forceinline__ unsigned xcd_order(unsigned bid, unsigned nblocks) {
    if (nblocks % 8u != 0) return bid;
    return (bid % 8u) * (nblocks / 8u) + bid / 8u;
}

template <typename T, int K, int R, bool MUL>
__global__ __launch_bounds__(kThreads) void k_up_forward(
    UpFilters<T> f, const T *__restrict__ x, T *__restrict__ out, int C, int H, int W, int D,
    int cpb, int csplit, int pblocks, int stage, int vec_ok) {
    using A = typename Acc<T>::type;
    constexpr int KK = K * K, RR = R * R, RAD = K / 2;
    constexpr int U = KK <= 9 ? 4 : 2;              // channels whose loads are issued together
    extern __shared__ __align__(16) unsigned char up_smem[];
    A *taps = reinterpret_cast<A *>(up_smem);   // [channel][branch][tap]

    const unsigned bid = xcd_order(blockIdx.x, gridDim.x);
    const int chunk = (int)(bid % (unsigned)csplit);
    const unsigned rest = bid / (unsigned)csplit;
    const int pb = (int)(rest % (unsigned)pblocks);
    const int64_t n = rest / (unsigned)pblocks;
    const int c0 = chunk * cpb;
    const int nch = min(cpb, C - c0);
    const int plane = H * W;

    const int pix = pb * kThreads + (int)threadIdx.x;
    const bool live = pix < plane;     // idle lanes still take part in the barriers
    const int y = live ? pix / W : 0, xx = live ? pix - y * W : 0;

    A sfr[RR][KK];
#pragma unroll
    for (int b = 0; b < RR; ++b)
#pragma unroll
        for (int t = 0; t < KK; ++t)
            sfr[b][t] = live ? (A)ld(f.sf[b] + (n * KK + t) * plane + pix) : (A)0;

    // neighbours of X: offset from the pixel and whether it lies in the plane
    int off[KK];
    bool inside[KK];
#pragma unroll
    for (int i = 0; i < K; ++i)
#pragma unroll
        for (int j = 0; j < K; ++j) {
            const int iy = y + (i - RAD) * D, ix = xx + (j - RAD) * D;
            inside[i * K + j] = live && iy >= 0 && iy < H && ix >= 0 && ix < W;
            off[i * K + j] = (i - RAD) * D * W + (j - RAD) * D;
        }

    const int64_t orow = (int64_t)W * R;            // elements per result row
    const int64_t ostep = (int64_t)H * R * orow;    // and per result plane
    const T *xp = x + (n * C + c0) * plane + pix;
    T *op = out + ((n * C + c0) * H + y) * R * orow + (int64_t)xx * R;
    for (int s0 = 0; s0 < nch; s0 += stage) {
        const int ns = min(stage, nch - s0);
        if (s0 > 0) __syncthreads();                // the previous taps have been used
        // channel taps of this stage: contiguous per branch, so coalesced
#pragma unroll
        for (int b = 0; b < RR; ++b) {
            const T *src = f.cf[b] + (n * C + c0 + s0) * KK;
            for (int e = threadIdx.x; e < ns * KK; e += kThreads) {
                const int ch = e / KK, t = e - ch * KK;
                taps[(ch * RR + b) * KK + t] = (A)ld(src + e);
            }
        }
        __syncthreads();
        if (!live) continue;
        // U channels at a time: all their loads are issued before the first
        // result is needed, so a wave keeps U*K*K loads in flight
        for (int ch = 0; ch < ns; ch += U, xp += (int64_t)U * plane, op += U * ostep) {
            A xv[U][KK];
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int t = 0; t < KK; ++t)
                    xv[u][t] = (ch + u < ns && inside[t]) ? (A)ld(xp + (int64_t)u * plane + off[t])
                                                          : (A)0;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (ch + u >= ns) break;
                const A *w = taps + (ch + u) * RR * KK;
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    Row<T, R> row;
#pragma unroll
                    for (int j = 0; j < R; ++j) {
                        const int b = i * R + j;
                        A acc = 0;
#pragma unroll
                        for (int t = 0; t < KK; ++t)
                            acc += xv[u][t] * comb<MUL, A>(w[b * KK + t], sfr[b][t]);
                        st(&row.e[j], acc);
                    }
                    T *dst = op + u * ostep + i * orow;
                    if ((R == 2 || R == 4) && vec_ok) {
                        *reinterpret_cast<Row<T, R> *>(dst) = row;
                    } else {
#pragma unroll
                        for (int j = 0; j < R; ++j) dst[j] = row.e[j];
                    }
                }
            }
        }
    }
}

template <typename T, int K, int R>
hipError_t launch(bool mul, const UpFilters<T> &f, const T *x, T *out, int64_t N, int C, int H,
                  int W, int D, hipStream_t stream) {
    using A = typename Acc<T>::type;
    const int64_t pblocks = cdiv((int64_t)H * W, kThreads);
    // Split the channels only as far as it takes to fill the chip: every chunk
    // re-reads the R*R*K*K spatial taps of its pixels.
    int csplit = 1;
    while (N * pblocks * csplit < 2048 && C / (csplit * 2) >= 8) csplit *= 2;
    const int cpb = (int)cdiv(C, csplit);
    csplit = (int)cdiv(C, cpb);
    const int64_t blocks = N * pblocks * csplit;
    if (blocks > 2147483647) return hipErrorInvalidConfiguration;
    const int per_channel = R * R * K * K * (int)sizeof(A);
    const int stage = std::max(1, std::min({cpb, kStageChannels, kStageBytes / per_channel}));
    const size_t lds = (size_t)stage * per_channel;
    const int vec_ok = ((uintptr_t)out % (sizeof(T) * R)) == 0;
    auto kern = mul ? k_up_forward<T, K, R, true> : k_up_forward<T, K, R, false>;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kThreads), lds, stream, f, x, out, C, H,
                       W, D, cpb, csplit, (int)pblocks, stage, vec_ok);
    return hipGetLastError();
}

}  // namespace

bool up_forward_supported(int64_t H, int64_t W, int k, int d, int scale) {
    if (H * W > (int64_t)1 << 30) return false;   // 32-bit offsets inside a plane
    if ((int64_t)(k / 2) * d * (W + 1) > (int64_t)1 << 30) return false;
    if (k == 1 || k == 3) return scale >= 2 && scale <= 4;
    if (k == 5) return scale == 2;
    return false;
}

template <typename T>
hipError_t up_forward(int64_t N, int64_t C, int64_t H, int64_t W, int k, int d, int scale,
                      bool mul, const T *x, const void *const *cf, const void *const *sf, T *out,
                      hipStream_t stream) {
    if (N * C * H * W == 0) return hipSuccess;
    if (C > 2147483647) return hipErrorInvalidConfiguration;
    UpFilters<T> f;
    for (int b = 0; b < DDF_UP_MAX_BRANCHES; ++b) {
        f.cf[b] = b < scale * scale ? (const T *)cf[b] : nullptr;
        f.sf[b] = b < scale * scale ? (const T *)sf[b] : nullptr;
    }
#define DDF_UP_CASE(KV, RV)                                                                     \
    if (k == KV && scale == RV)                                                                 \
        return launch<T, KV, RV>(mul, f, x, out, N, (int)C, (int)H, (int)W, d, stream);
    DDF_UP_CASE(1, 2) DDF_UP_CASE(1, 3) DDF_UP_CASE(1, 4)
    DDF_UP_CASE(3, 2) DDF_UP_CASE(3, 3) DDF_UP_CASE(3, 4)
    DDF_UP_CASE(5, 2)
#undef DDF_UP_CASE
    return hipErrorInvalidConfiguration;
}

#define DDF_UP_INSTANCE(T)                                                                      \
    template hipError_t up_forward<T>(int64_t, int64_t, int64_t, int64_t, int, int, int, bool,  \
                                      const T *, const void *const *, const void *const *, T *, \
                                      hipStream_t);
DDF_UP_INSTANCE(__half)
DDF_UP_INSTANCE(float)
DDF_UP_INSTANCE(double)
#undef DDF_UP_INSTANCE

}  // namespace ddf
