// The two filter branches of DDFPack as one launch each (gfx950, inference):
//
//   spatial (ddf/ddf.py:176-180 of the reference, FilterNorm 'spatial' :145-157):
//     sf[n, g*KK + t, yo, xo] = norm_t( bias[g*KK + t] + sum_c w[g*KK + t, c] * x[n, c, yo*s, xo*s] )
//   a 1x1 convolution with the operator's stride followed by the filter
//   normalisation over the KK taps of every pixel.  It reads x once and writes
//   the normalised taps; the un-normalised taps never reach memory.
//
//   channel (ddf/ddf.py:183-192, FilterNorm 'channel' :158-170), after the global
//   average pool:
//     cf[n, c, t] = norm_t( b2[c*KK + t] + sum_m w2[c*KK + t, m] * relu(b1[m] + sum_c' w1[m, c'] * v[n, c']) )
//   the two 1x1 convolutions on the pooled (n, c) vector are small matrix
//   products; one workgroup computes the hidden vector of its sample and 64
//   (wide layers: 128) channels' filters, and normalises them in place.
//
// norm_t(u) = gain_t * (u_t - mean(u)) / (std(u) + 1e-10) + offset_t with the
// unbiased standard deviation over the KK taps, as in ddf_filter_norm.hip.
// Both kernels are bound by memory and launch latency, not by arithmetic: the
// spatial branch does KK multiply-adds per 4-byte (2-byte) load.
#include <algorithm>

#include "ddf_common.h"

namespace ddf {
int tune_int(const char *name, int fallback);

namespace {

constexpr int kChunk = 256;   // channels whose weights sit in LDS at a time (64 per wave)

// Gains, offsets and biases of the KK taps of filter group `g`, read once (all
// loads go out together; read tap by tap where they are used, every one of
// them is a round trip of its own at the end of the kernel).
template <typename T, int KK>
struct TapParams {
    float gain[KK], offset[KK], bias[KK];
    __device__ __forceinline__ void load(int64_t g, float scalar_gain, const T *gain_vec,
                                         const T *offset_vec, const T *bias_vec) {
#pragma unroll
        for (int t = 0; t < KK; ++t) {
            gain[t] = scalar_gain;
            offset[t] = 0.f;
            bias[t] = 0.f;
        }
        if (gain_vec) {
#pragma unroll
            for (int t = 0; t < KK; ++t) gain[t] = ld(gain_vec + g * KK + t);
        }
        if (offset_vec) {
#pragma unroll
            for (int t = 0; t < KK; ++t) offset[t] = ld(offset_vec + g * KK + t);
        }
        if (bias_vec) {
#pragma unroll
            for (int t = 0; t < KK; ++t) bias[t] = ld(bias_vec + g * KK + t);
        }
    }
};

// v[0..KK) + bias, standardised in place, times gain plus offset.
template <typename T, int KK>
__device__ __forceinline__ void normalise(float (&v)[KK], const TapParams<T, KK> &p) {
    float sum = 0;
#pragma unroll
    for (int t = 0; t < KK; ++t) {
        v[t] += p.bias[t];
        sum += v[t];
    }
    const float mean = sum / (float)KK;
    float sq = 0;
#pragma unroll
    for (int t = 0; t < KK; ++t) {
        v[t] -= mean;
        sq += v[t] * v[t];
    }
    const float inv = 1.f / (sqrtf(sq / (float)(KK - 1)) + 1e-10f);
#pragma unroll
    for (int t = 0; t < KK; ++t) v[t] = v[t] * inv * p.gain[t] + p.offset[t];
}

// VP storage-type values at p (aligned to VP * sizeof(T)), widened.
template <typename T, int VP>
__device__ __forceinline__ void load_pixels(const T *p, float (&v)[VP]) {
    if constexpr (VP == 1) {
        v[0] = ld(p);
    } else {
        struct alignas(VP * sizeof(T)) Pack { T e[VP]; };
        const Pack q = *reinterpret_cast<const Pack *>(p);
#pragma unroll
        for (int k = 0; k < VP; ++k) v[k] = ld(&q.e[k]);
    }
}

// grid (pixel tiles of 64 * VP, head, N); the WAVES waves of a workgroup cover
// the same result pixels (a lane owns VP consecutive pixels of a row: VP > 1
// needs stride 1 and rows that are a whole number of such vectors) and
// 1/WAVES of every channel chunk each, U channels' loads in flight at a time.
template <typename T, int KK, int WAVES, int VP>
__global__ __launch_bounds__(WAVES * kWave) void k_spatial_branch(
    const T *__restrict__ x, const T *__restrict__ w, const T *__restrict__ bias,
    T *__restrict__ sf, int C, int H, int W, int Ho, int Wo, int stride, int chunk, float gain,
    const T *__restrict__ gain_vec, const T *__restrict__ offset_vec) {
    constexpr int U = VP >= 4 ? 4 : 8;
    // weights of the chunk, [channel][tap], rows padded to 16 bytes (wide LDS reads)
    __shared__ __align__(16) float wt[kChunk][(KK + 3) / 4 * 4];
    __shared__ float red[WAVES][KK][kWave];             // per-wave sums of one pixel of the vector
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int g = blockIdx.y, heads = gridDim.y;
    const int64_t n = blockIdx.z;
    const int npix = Ho * Wo;
    const int pix = (blockIdx.x * kWave + lane) * VP;   // first of the lane's pixels
    const bool live = pix < npix;
    const int yo = live ? pix / Wo : 0, xo = live ? pix - yo * Wo : 0;
    const int64_t plane = (int64_t)H * W;
    const T *xp = x + n * C * plane + (int64_t)yo * stride * W + (int64_t)xo * stride;
    const T *wg = w + (int64_t)g * KK * C;
    const int per = chunk / WAVES;                      // channels of a chunk per wave (multiple of U)
    TapParams<T, KK> params;
    if (wave == 0) params.load(g, gain, gain_vec, offset_vec, bias);   // (wave 0 writes the taps)

    float acc[KK][VP];
#pragma unroll
    for (int t = 0; t < KK; ++t)
#pragma unroll
        for (int k = 0; k < VP; ++k) acc[t][k] = 0.f;
    for (int c0 = 0; c0 < C; c0 += chunk) {
        if (c0 > 0) __syncthreads();
        // weights of channels c0 .. c0+chunk-1 (zero past C), coalesced along a weight row
        for (int i = threadIdx.x; i < chunk; i += WAVES * kWave) {
            const int c = c0 + i;
#pragma unroll
            for (int t = 0; t < KK; ++t) wt[i][t] = c < C ? ld(wg + (int64_t)t * C + c) : 0.f;
        }
        __syncthreads();
        const int cw = c0 + wave * per;                 // this wave's channels of the chunk
        const int nc = min(per, C - cw);                // (<= 0: none left)
        for (int i0 = 0; i0 < nc; i0 += U) {
            float xv[U][VP];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int i = min(i0 + u, nc - 1);      // past the end: repeats, with zero weights
                if (live) {
                    load_pixels<T, VP>(xp + (int64_t)(cw + i) * plane, xv[u]);
                } else {
#pragma unroll
                    for (int k = 0; k < VP; ++k) xv[u][k] = 0.f;
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                // (rows past the wave's last channel belong to channels >= C: zeros)
                const float *wr = wt[wave * per + i0 + u];
#pragma unroll
                for (int t = 0; t < KK; ++t) {
                    const float wv = wr[t];
#pragma unroll
                    for (int k = 0; k < VP; ++k) acc[t][k] = fmaf(wv, xv[u][k], acc[t][k]);
                }
            }
        }
    }
    // one pixel of the vectors at a time through LDS: the waves' sums, then wave 0
    // normalises and writes that pixel's taps
#pragma unroll
    for (int k = 0; k < VP; ++k) {
        if (k > 0) __syncthreads();
#pragma unroll
        for (int t = 0; t < KK; ++t) red[wave][t][lane] = acc[t][k];
        __syncthreads();
        if (wave == 0 && live) {
            float v[KK];
#pragma unroll
            for (int t = 0; t < KK; ++t) {
                float s = 0.f;
#pragma unroll
                for (int q = 0; q < WAVES; ++q) s += red[q][t][lane];
                v[t] = s;
            }
            normalise<T, KK>(v, params);
            T *op = sf + ((n * heads + g) * KK) * (int64_t)npix + pix + k;
#pragma unroll
            for (int t = 0; t < KK; ++t) st(op + (int64_t)t * npix, v[t]);
        }
    }
}

// The same for planes with many pixels: every wave of the workgroup has its own
// 64 * VP result pixels and walks all channels, so nothing is added up across
// waves and the taps are normalised in registers.  grid (tiles of 4 * 64 * VP
// pixels, head, N).
template <typename T, int KK, int VP>
__global__ __launch_bounds__(4 * kWave) void k_spatial_branch_tiles(
    const T *__restrict__ x, const T *__restrict__ w, const T *__restrict__ bias,
    T *__restrict__ sf, int C, int H, int W, int Ho, int Wo, int stride, int chunk, float gain,
    const T *__restrict__ gain_vec, const T *__restrict__ offset_vec) {
    constexpr int U = 16;   // channels in flight per wave: what the run time hangs on
    __shared__ __align__(16) float wt[kChunk][(KK + 3) / 4 * 4];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int g = blockIdx.y, heads = gridDim.y;
    const int64_t n = blockIdx.z;
    const int npix = Ho * Wo;
    const int pix = ((blockIdx.x * 4 + wave) * kWave + lane) * VP;
    const bool live = pix < npix;
    const int yo = live ? pix / Wo : 0, xo = live ? pix - yo * Wo : 0;
    const int64_t plane = (int64_t)H * W;
    const T *xp = x + n * C * plane + (int64_t)yo * stride * W + (int64_t)xo * stride;
    const T *wg = w + (int64_t)g * KK * C;
    TapParams<T, KK> params;
    params.load(g, gain, gain_vec, offset_vec, bias);

    float acc[KK][VP];
#pragma unroll
    for (int t = 0; t < KK; ++t)
#pragma unroll
        for (int k = 0; k < VP; ++k) acc[t][k] = 0.f;
    for (int c0 = 0; c0 < C; c0 += chunk) {
        if (c0 > 0) __syncthreads();
        for (int i = threadIdx.x; i < chunk; i += 4 * kWave) {
            const int c = c0 + i;
#pragma unroll
            for (int t = 0; t < KK; ++t) wt[i][t] = c < C ? ld(wg + (int64_t)t * C + c) : 0.f;
        }
        __syncthreads();
        const int nc = min(chunk, C - c0);
        for (int i0 = 0; i0 < nc; i0 += U) {
            float xv[U][VP];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int i = min(i0 + u, nc - 1);      // past the end: repeats, with zero weights
                if (live) {
                    load_pixels<T, VP>(xp + (int64_t)(c0 + i) * plane, xv[u]);
                } else {
#pragma unroll
                    for (int k = 0; k < VP; ++k) xv[u][k] = 0.f;
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const float *wr = wt[i0 + u];           // (i0 + u < chunk: chunk is a multiple of U)
                float wv[KK];
#pragma unroll
                for (int t = 0; t < KK; ++t) wv[t] = wr[t];
#pragma unroll
                for (int t = 0; t < KK; ++t)
#pragma unroll
                    for (int k = 0; k < VP; ++k) acc[t][k] = fmaf(wv[t], xv[u][k], acc[t][k]);
            }
        }
    }
    if (!live) return;
#pragma unroll
    for (int k = 0; k < VP; ++k) {
        float v[KK];
#pragma unroll
        for (int t = 0; t < KK; ++t) v[t] = acc[t][k];
        normalise<T, KK>(v, params);
#pragma unroll
        for (int t = 0; t < KK; ++t) acc[t][k] = v[t];
    }
    // taps of the lane's VP pixels, one vector store per tap plane
    T *op = sf + ((n * heads + g) * KK) * (int64_t)npix + pix;
#pragma unroll
    for (int t = 0; t < KK; ++t) {
        if constexpr (VP == 1) {
            st(op + (int64_t)t * npix, acc[t][0]);
        } else {
            struct alignas(VP * sizeof(T)) Pack { T e[VP]; } q;
#pragma unroll
            for (int k = 0; k < VP; ++k) st(&q.e[k], acc[t][k]);
            *reinterpret_cast<Pack *>(op + (int64_t)t * npix) = q;
        }
    }
}

// Butterfly steps through the VALU's lane-permute path.  (Shuffles through the
// LDS crossbar cost a round trip each and made these kernels several times slower.)
template <int CTRL>
__device__ __forceinline__ float add_permuted(float x) {
    return x + __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), CTRL, 0xf, 0xf, true));
}
// Sum over each row of 16 lanes (the same value in every lane of the row).
__device__ __forceinline__ float row_sum(float v) {
    v = add_permuted<0xB1>(v);    // quad_perm [1,0,3,2]
    v = add_permuted<0x4E>(v);    // quad_perm [2,3,0,1]
    v = add_permuted<0x141>(v);   // row_half_mirror
    return add_permuted<0x140>(v);   // row_mirror
}

constexpr int kChannelThreads = 1024;  // sixteen waves: the rows of a block's taps are dealt out to them
constexpr int kChannelWaves = kChannelThreads / kWave;

// grid (channel blocks of BLOCK channels, groups of NS samples).  LDS: the pooled
// vectors (NS * C floats), the hidden vectors (NS * mid floats), the block's
// un-normalised taps (NS * BLOCK * KK).  Every weight a lane loads serves the NS
// samples of its workgroup (the weights are the same for all samples; re-read
// per sample they cost more L2 bandwidth than anything else here).  Every
// workgroup of a sample recomputes the hidden vector, so the blocks are large:
// smaller ones had all compute units read the same rows of w1 at once, which
// the L2 serves one after the other.
template <typename T, int KK, int BLOCK, int NS>
__global__ __launch_bounds__(kChannelThreads) void k_channel_branch(
    const T *__restrict__ pooled, const T *__restrict__ w1, const T *__restrict__ b1,
    const T *__restrict__ w2, const T *__restrict__ b2, T *__restrict__ cf, int N, int C, int mid,
    float gain, const T *__restrict__ gain_vec, const T *__restrict__ offset_vec) {
    extern __shared__ float branch_smem[];
    float *v = branch_smem;            // [NS][C]
    float *h = v + NS * C;             // [NS][mid]
    float *f = h + NS * mid;           // [NS][BLOCK * KK]
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int64_t n0 = (int64_t)blockIdx.y * NS;
    const int ns = min(NS, N - (int)n0);   // samples of this workgroup (the others: copies of the last)
    const int cb = blockIdx.x * BLOCK;
    for (int i = threadIdx.x; i < NS * C; i += kChannelThreads) {
        const int s = i / C, c = i - s * C;
        v[i] = ld(pooled + (n0 + min(s, ns - 1)) * C + c);
    }
    __syncthreads();
    // Dot products with sixteen lanes along a weight row and four rows per wave at a
    // time: each ends in a reduction over a row of 16 lanes (four lane-permute
    // additions for four results; a whole wave per row paid thirteen for one).
    const int seg = lane >> 4, sl = lane & 15;
    // hidden vectors: rows of w1
    for (int m0 = wave * 4; m0 < mid; m0 += kChannelWaves * 4) {
        const int m = min(m0 + seg, mid - 1);
        const T *row = w1 + (int64_t)m * C;
        float p[NS];
#pragma unroll
        for (int s = 0; s < NS; ++s) p[s] = 0.f;
#pragma unroll 8
        for (int c = sl; c < C; c += 16) {
            const float wv = ld(row + c);
#pragma unroll
            for (int s = 0; s < NS; ++s) p[s] = fmaf(wv, v[s * C + c], p[s]);
        }
        const float bias = b1 ? ld(b1 + m) : 0.f;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const float tot = row_sum(p[s]);
            if (sl == 0 && m0 + seg < mid) h[s * mid + m0 + seg] = fmaxf(tot + bias, 0.f);
        }
    }
    __syncthreads();
    // the block's taps: rows (cb * KK + r) of w2, RT passes of four rows in flight per wave
    constexpr int RT = NS >= 4 ? 1 : NS == 2 ? 2 : 3;
    const int rows = min(BLOCK, C - cb) * KK;
    for (int r0 = wave * 4 * RT; r0 < rows; r0 += kChannelWaves * 4 * RT) {
        float p[RT][NS];
        const T *wrow[RT];
#pragma unroll
        for (int u = 0; u < RT; ++u) {
#pragma unroll
            for (int s = 0; s < NS; ++s) p[u][s] = 0.f;
            wrow[u] = w2 + ((int64_t)cb * KK + min(r0 + 4 * u + seg, rows - 1)) * mid;
        }
#pragma unroll 2
        for (int m = sl; m < mid; m += 16) {
            float hm[NS];
#pragma unroll
            for (int s = 0; s < NS; ++s) hm[s] = h[s * mid + m];
#pragma unroll
            for (int u = 0; u < RT; ++u) {
                const float wv = ld(wrow[u] + m);
#pragma unroll
                for (int s = 0; s < NS; ++s) p[u][s] = fmaf(wv, hm[s], p[u][s]);
            }
        }
#pragma unroll
        for (int u = 0; u < RT; ++u) {
            const int r = r0 + 4 * u + seg;
            const float bias = (b2 && r < rows) ? ld(b2 + (int64_t)cb * KK + r) : 0.f;
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                const float tot = row_sum(p[u][s]);
                if (sl == 0 && r < rows) f[s * BLOCK * KK + r] = tot + bias;
            }
        }
    }
    __syncthreads();
    // one thread per (sample, channel) normalises the KK taps
    for (int i = threadIdx.x; i < NS * BLOCK; i += kChannelThreads) {
        const int s = i / BLOCK, ch = i - s * BLOCK;
        if (s >= ns || cb + ch >= C) continue;
        float u[KK];
#pragma unroll
        for (int t = 0; t < KK; ++t) u[t] = f[(s * BLOCK + ch) * KK + t];
        TapParams<T, KK> params;
        params.load(cb + ch, gain, gain_vec, offset_vec, (const T *)nullptr);   // (b2 is in f already)
        normalise<T, KK>(u, params);
        T *op = cf + ((n0 + s) * C + cb + ch) * KK;
#pragma unroll
        for (int t = 0; t < KK; ++t) st(op + t, u[t]);
    }
}

}  // namespace

bool branch_kernel_size_built(int k) { return k == 3 || k == 5; }

template <typename T>
hipError_t spatial_branch(const T *x, const T *w, const T *bias, T *sf, int64_t N, int64_t C,
                          int64_t H, int64_t W, int head, int k, int stride, double gain,
                          const T *gain_vec, const T *offset_vec, hipStream_t st) {
    const int64_t Ho = H / stride, Wo = W / stride;
    if (N == 0 || C == 0 || Ho * Wo == 0 || head == 0) return hipSuccess;
    if (N > 65535 || head > 65535 || C > (1 << 24) || H * W >= (1ll << 31)) return hipErrorNotSupported;
    const int waves = k == 3 ? 8 : 4;
    // channels staged in LDS at a time: all of them up to kChunk, a multiple of 8 per wave
    // (and so of the 16 the tile kernel keeps in flight)
    const int chunk = (int)std::min<int64_t>(kChunk, (C + 8 * waves - 1) / (8 * waves) * (8 * waves));
    // Planes with many pixels: a wave per pixel tile, as wide a vector per lane as
    // rows and alignment allow while the waves still fill the machine.
    if (stride == 1 && tune_int("DDF_TUNE_SPATIAL_TILES", 1) != 0) {
        for (int vp = 16 / (int)sizeof(T); vp >= 1; vp /= 2) {
            if (k == 5 && vp > 2) continue;   // (25 taps: the accumulators of two pixels per lane)
            if (W % vp != 0 || (((uintptr_t)x | (uintptr_t)sf) % (vp * sizeof(T))) != 0) continue;
            if (vp == 1 && sizeof(T) == 2) continue;   // (2-byte loads: the shared-pixel kernel does better)
            if ((Ho * Wo) % vp != 0 || N * head * cdiv(Ho * Wo, kWave * vp) < tune_int("DDF_TUNE_SPATIAL_TILES_MIN", 1024)) continue;
            const dim3 grid((unsigned)cdiv(Ho * Wo, 4 * kWave * vp), (unsigned)head, (unsigned)N);
#define DDF_TILES_CASE(KK_, VP_)                                                                \
    hipLaunchKernelGGL((k_spatial_branch_tiles<T, KK_, VP_>), grid, dim3(4 * kWave), 0, st, x, w, \
                       bias, sf, (int)C, (int)H, (int)W, (int)Ho, (int)Wo, stride, chunk,       \
                       (float)gain, gain_vec, offset_vec)
            if (k == 3 && vp == 8) { if constexpr (sizeof(T) == 2) DDF_TILES_CASE(9, 8); }
            else if (k == 3 && vp == 4) DDF_TILES_CASE(9, 4);
            else if (k == 3 && vp == 2) DDF_TILES_CASE(9, 2);
            else if (k == 3) DDF_TILES_CASE(9, 1);
            else if (k == 5 && vp == 2) DDF_TILES_CASE(25, 2);
            else if (k == 5) DDF_TILES_CASE(25, 1);
            else return hipErrorNotSupported;
#undef DDF_TILES_CASE
            return hipGetLastError();
        }
    }
    // Few pixels (or strided sampling): the waves of a workgroup share 64 pixels and
    // split the channels (as many waves as the LDS of the per-wave sums allows).
    const dim3 grid((unsigned)cdiv(Ho * Wo, kWave), (unsigned)head, (unsigned)N);
#define DDF_SPATIAL_CASE(KK_, WAVES_, VP_)                                                      \
    hipLaunchKernelGGL((k_spatial_branch<T, KK_, WAVES_, VP_>), grid, dim3(WAVES_ * kWave), 0, st, x, \
                       w, bias, sf, (int)C, (int)H, (int)W, (int)Ho, (int)Wo, stride, chunk,    \
                       (float)gain, gain_vec, offset_vec)
    // (vectors of pixels per lane where rows and alignment allow: fewer, wider loads)
    int vp = 1;
    // (two-byte elements; four-byte ones gain nothing from it)
    if (stride == 1 && k == 3 && sizeof(T) == 2) {
        for (int cand = tune_int("DDF_TUNE_SPATIAL_VP", 4); cand > 1; cand /= 2)
            if (W % cand == 0 && (((uintptr_t)x | (uintptr_t)sf) % (cand * sizeof(T))) == 0 &&
                N * head * cdiv(Ho * Wo, kWave * cand) >= 256) {
                vp = cand;
                break;
            }
    }
    const dim3 grid_v((unsigned)cdiv(Ho * Wo, kWave * vp), (unsigned)head, (unsigned)N);
    if (k == 3 && vp == 4) {
        hipLaunchKernelGGL((k_spatial_branch<T, 9, 8, 4>), grid_v, dim3(8 * kWave), 0, st, x, w, bias, sf,
                           (int)C, (int)H, (int)W, (int)Ho, (int)Wo, stride, chunk, (float)gain, gain_vec,
                           offset_vec);
    } else if (k == 3 && vp == 2) {
        hipLaunchKernelGGL((k_spatial_branch<T, 9, 8, 2>), grid_v, dim3(8 * kWave), 0, st, x, w, bias, sf,
                           (int)C, (int)H, (int)W, (int)Ho, (int)Wo, stride, chunk, (float)gain, gain_vec,
                           offset_vec);
    } else if (k == 3) DDF_SPATIAL_CASE(9, 8, 1);
    else if (k == 5) DDF_SPATIAL_CASE(25, 4, 1);
    else return hipErrorNotSupported;
#undef DDF_SPATIAL_CASE
    return hipGetLastError();
}

template <typename T>
hipError_t channel_branch(const T *pooled, const T *w1, const T *b1, const T *w2, const T *b2,
                          T *cf, int64_t N, int64_t C, int64_t mid, int k, double gain,
                          const T *gain_vec, const T *offset_vec, hipStream_t st) {
    if (N == 0 || C == 0) return hipSuccess;
    const int kk = k * k;
    // (wide layers: fewer, larger blocks, as every block of a sample recomputes the hidden vector)
    const int block = C >= 512 ? 128 : 64;
    // samples per workgroup: as many as keep every compute unit busy and fit the LDS
    auto lds_of = [&](int ns) { return ((size_t)C + (size_t)mid + (size_t)block * kk) * ns * sizeof(float); };
    int ns = 1;
    const int forced = tune_int("DDF_TUNE_CHANNEL_NS", 0);
    while (ns < 4 && cdiv(C, block) * cdiv(N, ns * 2) >= 256 && lds_of(ns * 2) <= 48 * 1024) ns *= 2;
    if (forced == 1 || forced == 2 || forced == 4) ns = forced;
    const size_t lds = lds_of(ns);
    if (N > 65535 * ns || mid < 1 || lds > 48 * 1024) return hipErrorNotSupported;
    const dim3 grid((unsigned)cdiv(C, block), (unsigned)cdiv(N, ns));
#define DDF_CHANNEL_LAUNCH(KK_, BLOCK_, NS_)                                                     \
    hipLaunchKernelGGL((k_channel_branch<T, KK_, BLOCK_, NS_>), grid, dim3(kChannelThreads), lds, \
                       st, pooled, w1, b1, w2, b2, cf, (int)N, (int)C, (int)mid, (float)gain,    \
                       gain_vec, offset_vec)
#define DDF_CHANNEL_CASE(KK_, BLOCK_)                                                            \
    do {                                                                                         \
        if (ns == 4) DDF_CHANNEL_LAUNCH(KK_, BLOCK_, 4);                                         \
        else if (ns == 2) DDF_CHANNEL_LAUNCH(KK_, BLOCK_, 2);                                    \
        else DDF_CHANNEL_LAUNCH(KK_, BLOCK_, 1);                                                 \
    } while (0)
    if (k == 3 && block == 64) DDF_CHANNEL_CASE(9, 64);
    else if (k == 3) DDF_CHANNEL_CASE(9, 128);
    else if (k == 5 && block == 64) DDF_CHANNEL_CASE(25, 64);
    else if (k == 5) DDF_CHANNEL_CASE(25, 128);
    else return hipErrorNotSupported;
#undef DDF_CHANNEL_LAUNCH
#undef DDF_CHANNEL_CASE
    return hipGetLastError();
}

#define DDF_INSTANTIATE_BRANCHES(T)                                                              \
    template hipError_t spatial_branch<T>(const T *, const T *, const T *, T *, int64_t, int64_t, \
                                          int64_t, int64_t, int, int, int, double, const T *,    \
                                          const T *, hipStream_t);                               \
    template hipError_t channel_branch<T>(const T *, const T *, const T *, const T *, const T *, \
                                          T *, int64_t, int64_t, int64_t, int, double, const T *, \
                                          const T *, hipStream_t);
DDF_INSTANTIATE_BRANCHES(__half)
DDF_INSTANTIATE_BRANCHES(float)
#undef DDF_INSTANTIATE_BRANCHES

}  // namespace ddf
