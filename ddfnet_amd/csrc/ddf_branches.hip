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
//   (wide layers: 128) channels' filters, and normalises them in place
//   (k_channel_branch), or, in fp16 with a hidden layer of 32 values or more,
//   sixteen samples x sixteen channels on the matrix cores (k_channel_branch_mma).
//
// norm_t(u) = gain_t * (u_t - mean(u)) / (std(u) + 1e-10) + offset_t with the
// unbiased standard deviation over the KK taps, as in ddf_filter_norm.hip.
// Both kernels are bound by memory and launch latency, not by arithmetic: the
// spatial branch does KK multiply-adds per 4-byte (2-byte) load.
#include <algorithm>
#include <type_traits>

#include "ddf_common.h"
#include "ddf_rows.h"

namespace ddf {
int tune_int(const char *name, int fallback);

namespace {
using rows::kOutside;
using rows::load_vec;
using rows::plane_rsrc;
using rows::store_vec_nt;
using rows::vec_words;

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

// ---------------------------------------------------------------------------
// Spatial branch, 3 x 3 taps, as a stream over the channels (the kernel the
// launcher prefers).  A lane owns VP neighbouring result pixels of one sample
// (stride 1: the plane is one run of pixels, so a vector may cross image rows;
// stride 2: the 2 * VP feature pixels under VP result pixels of one row come in
// as one vector) and adds up KK taps for each.  The WAVES waves of a workgroup
// cover the same pixels and a range of channels each, U at a time; their sums
// meet in LDS at the end.  Like the operator's own kernels it has
//   * every channel plane behind a buffer descriptor (an idle lane's offset and
//     the planes past the last channel read zero, no bounds branch),
//   * the loads of NST - 1 channel groups in flight while one is computed,
//   * the weights - the same for every lane - in scalar registers.
struct SpatialGeom {
    int C, W, Wo;
    int plane;      // H * W
    int npix;       // Ho * Wo
    int nvec;       // npix / VP
    int lpt;        // lanes of a workgroup's pixel tile that have a vector
    int ngroups;    // C / U
    int gpw;        // channel groups per wave
    int steps;      // gpw rounded up to a multiple of NST
};

// Sums of U (2 or 4) values per lane over each row of 16 lanes of a wave: every lane
// ends up with its row's total of value number (lane % U).  The first steps halve the
// number of values a lane carries instead of adding U full sums side by side: lane
// pairs exchange the value the other keeps (quad permutes); then the quads of a row add
// up by rotation.  (The four rows of a wave are left apart: bringing them together takes
// lane-indexed reads through the LDS unit, whose counter the kernel's scalar weight
// loads share - waiting for one drains the other's prefetch.)
template <int CTRL>
__device__ __forceinline__ float from_permuted(float x) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), CTRL, 0xf, 0xf, true));
}
template <int U>
__device__ __forceinline__ float row_sums(const float (&v)[U], int lane) {
    static_assert(U == 2 || U == 4, "two or four values per lane");
    const bool b0 = lane & 1, b1 = lane & 2;
    float k = (b0 ? v[1] : v[0]) + from_permuted<0xB1 /* quad_perm [1,0,3,2] */>(b0 ? v[0] : v[1]);
    if constexpr (U == 4) {
        const float k1 = (b0 ? v[3] : v[2]) + from_permuted<0xB1>(b0 ? v[2] : v[3]);
        k = (b1 ? k1 : k) + from_permuted<0x4E /* quad_perm [2,3,0,1] */>(b1 ? k : k1);
    } else {
        k += from_permuted<0x4E>(k);
    }
    k += from_permuted<0x124 /* row_ror:4 */>(k);
    k += from_permuted<0x128 /* row_ror:8 */>(k);
    return k;
}

// POOL: the kernel also leaves, per sample, pixel tile and channel, the sum of the
// feature map over the pixels of a quarter of the tile (the lanes of one row of 16) in
// pool_part[((n * tiles + tile) * 4 + row) * C + c] (fp32) -
// the global average pool in front of the channel branch, from the values this kernel
// has in registers anyway.  Under stride 2 (even H and W) the lane also loads the
// feature row below its own, and both columns where it otherwise takes one; those lines
// come in with their neighbours in any case.
template <typename T, int KK, int VP, int S, int WAVES, int U, int NST, bool POOL = false>
__global__ __launch_bounds__(WAVES * kWave) void k_spatial_stream(
    SpatialGeom g, const T *__restrict__ x, const T *__restrict__ w, const T *__restrict__ bias,
    T *__restrict__ sf, float gain, const T *__restrict__ gain_vec, const T *__restrict__ offset_vec,
    float *__restrict__ pool_part) {
    // feature elements a lane loads per channel (pooling under stride 2: both columns)
    constexpr int XE = S == 1 ? VP : (VP == 1 && !POOL ? 1 : 2 * VP);
    constexpr int kXB = XE * sizeof(T), NWX = vec_words(kXB);
    constexpr int kOB = VP * sizeof(T), NWO = vec_words(kOB);
    constexpr int WPU = U * sizeof(T) / 4;                     // 32-bit words of U weights
    static_assert(U * sizeof(T) % 4 == 0 && U % 2 == 0, "weights come in whole words, channels in pairs");
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int head = blockIdx.y, heads = gridDim.y;
    const int64_t n = blockIdx.z;
    const int v = blockIdx.x * g.lpt + lane;
    const bool live = lane < g.lpt && v < g.nvec;
    const int p = v * VP;                                      // first of the lane's result pixels
    int in_off = p;
    if constexpr (S == 2) {
        const int yo = p / g.Wo, xo = p - yo * g.Wo;
        in_off = 2 * yo * g.W + 2 * xo;
    }
    const uint32_t xb = live ? (uint32_t)in_off * (uint32_t)sizeof(T) : kOutside;
    const uint32_t plane_bytes = (uint32_t)g.plane * (uint32_t)sizeof(T);
    // the sample's C planes behind one descriptor; a channel is a scalar offset into it
    const __amdgpu_buffer_rsrc_t xr = plane_rsrc(x + n * g.C * (int64_t)g.plane, (uint32_t)g.C * plane_bytes);
    const char *wg = reinterpret_cast<const char *>(w + (int64_t)head * KK * g.C);
    const uint32_t row_bytes = (uint32_t)g.C * (uint32_t)sizeof(T);
    const int j0 = wave * g.gpw;                               // the wave's first channel group

    uint32_t xw[NST][U][NWX];
    uint32_t xlow[POOL && S == 2 ? NST : 1][U][NWX];           // (pooling under stride 2: the row below)
    short xh[NST][U];                                          // (single fp16 elements: as loaded)
    uint32_t ww[NST][KK][WPU];
    // channel group i of this wave's gpw consecutive ones, stage ST (consecutive: a wave's
    // weights of consecutive steps then share scalar-cache lines)
    auto issue = [&](auto st_tag, int i) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value;
        const bool have = i < g.gpw && j0 + i < g.ngroups;
        // (a group the wave does not have: every lane's offset lies outside, the loads
        // return zero - whatever weights they then meet)
        const int j = have ? j0 + i : (j0 < g.ngroups ? j0 : 0);
        const uint32_t vb = have ? xb : kOutside;
        const uint32_t cb = (uint32_t)(j * U) * plane_bytes;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if constexpr (kXB == 2) {
                xh[ST][u] = __builtin_amdgcn_raw_buffer_load_b16(xr, (int)vb, (int)(cb + (uint32_t)u * plane_bytes), 0);
            } else if constexpr (kXB == 4) {
                xw[ST][u][0] = __builtin_amdgcn_raw_buffer_load_b32(xr, (int)vb, (int)(cb + (uint32_t)u * plane_bytes), 0);
            } else if constexpr (kXB == 8) {
                const auto q = __builtin_amdgcn_raw_buffer_load_b64(xr, (int)vb, (int)(cb + (uint32_t)u * plane_bytes), 0);
                xw[ST][u][0] = q[0]; xw[ST][u][1] = q[1];
            } else {
                static_assert(kXB <= 16, "vectors of 16 bytes at most");
                const auto q = __builtin_amdgcn_raw_buffer_load_b128(xr, (int)vb, (int)(cb + (uint32_t)u * plane_bytes), 0);
#pragma unroll
                for (int k = 0; k < 4; ++k) xw[ST][u][k] = q[k];
            }
            if constexpr (POOL && S == 2) {
                if (head == 0)
                    load_vec<kXB>(xr, vb == kOutside ? kOutside : vb + (uint32_t)g.W * (uint32_t)sizeof(T) +
                                                                       cb + (uint32_t)u * plane_bytes,
                                  xlow[ST][u]);
            }
        }
    };
    // The weights of group i, stage ST.  They are requested one step ahead only (a scalar
    // load is back well within a step), so two of the NST register sets are alive at any
    // time: with all of them the pooled variants run out of scalar registers.
    auto issue_weights = [&](auto st_tag, int i) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value;
        const bool have = i < g.gpw && j0 + i < g.ngroups;
        const int j = have ? j0 + i : (j0 < g.ngroups ? j0 : 0);
        const uint32_t wb = (uint32_t)(j * U) * (uint32_t)sizeof(T);
#pragma unroll
        for (int t = 0; t < KK; ++t)
#pragma unroll
            for (int q = 0; q < WPU; ++q)
                ww[ST][t][q] = *reinterpret_cast<const uint32_t *>(wg + (wb + (uint32_t)t * row_bytes + 4u * q));
    };
    float acc[KK][VP];
#pragma unroll
    for (int t = 0; t < KK; ++t)
#pragma unroll
        for (int k = 0; k < VP; ++k) acc[t][k] = 0.f;
    // POOL: where this lane's sums of the wave's first channel group go (one partial sum
    // per row of 16 lanes: four per tile), and how many groups the wave keeps sums of (head
    // 0 of a sample does it for all heads).  Worked out here and pinned: formed inside the
    // walk they take a scalar load of a launch dimension, and the wait for it also waits
    // for the weights that were just requested for the next step.  The sums go out through
    // a buffer descriptor of the tile's 4 * C values, lanes with nothing to write at an
    // offset outside it: a store under a branch leaves the compiler unable to count the
    // loads in flight where the branch joins, and it then waits for all of them.
    // (Collecting the sums in LDS and writing them after the walk was no faster.)
    __amdgpu_buffer_rsrc_t pool_rsrc = plane_rsrc(nullptr, 0u);
    uint32_t pool_off = kOutside;
    int pool_groups = 0;
    if constexpr (POOL) {
        pool_rsrc = plane_rsrc(pool_part + ((n * gridDim.x + blockIdx.x) * 4) * g.C,
                               (uint32_t)(4 * g.C) * (uint32_t)sizeof(float));
        if (head == 0 && (lane & 15) < U)
            pool_off = (uint32_t)((lane >> 4) * g.C + j0 * U + (lane & 15)) * (uint32_t)sizeof(float);
        pool_groups = head == 0 ? min(g.gpw, g.ngroups - j0) : 0;
        asm volatile("" : "+v"(pool_off), "+s"(pool_groups));
    }
    auto compute = [&](auto st_tag, int i) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value;
        if constexpr (POOL) {
            // (No branch around the arithmetic: it would cut the step into blocks, and the
            // waits the compiler then places at their joins cost more than the sums of a
            // group the wave does not have.)
            const bool keep = i < pool_groups;
            {
                float psum[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    float ps = 0.f;
                    if constexpr (sizeof(T) == 2 && kXB == 2) {
                        ps = (float)__builtin_bit_cast(_Float16, xh[ST][u]);
                    } else if constexpr (sizeof(T) == 2) {
                        // (every word on its own, then a tree of additions: one accumulator for
                        // all words is a chain of dependent dot products, each waiting out the
                        // latency of the one before)
                        const rows::half2_t ones = {(_Float16)1, (_Float16)1};
                        float part[NWX];
#pragma unroll
                        for (int k = 0; k < NWX; ++k) {
                            part[k] = __builtin_amdgcn_fdot2(__builtin_bit_cast(rows::half2_t, xw[ST][u][k]), ones, 0.f, false);
                            if constexpr (S == 2)
                                part[k] = __builtin_amdgcn_fdot2(__builtin_bit_cast(rows::half2_t, xlow[ST][u][k]), ones, part[k], false);
                        }
                        if constexpr (NWX == 4) ps = (part[0] + part[1]) + (part[2] + part[3]);
                        else if constexpr (NWX == 2) ps = part[0] + part[1];
                        else ps = part[0];
                    } else {
#pragma unroll
                        for (int k = 0; k < NWX; ++k) {
                            ps += __uint_as_float(xw[ST][u][k]);
                            if constexpr (S == 2) ps += __uint_as_float(xlow[ST][u][k]);
                        }
                    }
                    psum[u] = ps;
                }
                const float tot = row_sums<U>(psum, lane);
                __builtin_amdgcn_raw_buffer_store_b32(
                    __float_as_uint(tot), pool_rsrc,
                    (int)(keep ? pool_off + (uint32_t)(i * U) * (uint32_t)sizeof(float) : kOutside), 0, 0);
            }
        }
        if constexpr (sizeof(T) == 2) {
            // two channels at a time: (x[c], x[c+1]) of a pixel against (w[c], w[c+1]), which is
            // one word of the weight row as it lies in memory; fp32 sums
#pragma unroll
            for (int pr = 0; pr < U / 2; ++pr)
#pragma unroll
                for (int k = 0; k < VP; ++k) {
                    constexpr uint32_t kLow = 0x05040100u, kHigh = 0x07060302u;
                    rows::half2_t xp;
                    if constexpr (kXB == 2) {
                        xp[0] = __builtin_bit_cast(_Float16, xh[ST][2 * pr]);
                        xp[1] = __builtin_bit_cast(_Float16, xh[ST][2 * pr + 1]);
                    } else {
                        const int e = S * k;
                        xp = __builtin_bit_cast(rows::half2_t,
                                                __builtin_amdgcn_perm(xw[ST][2 * pr + 1][e / 2], xw[ST][2 * pr][e / 2],
                                                                      (e & 1) ? kHigh : kLow));
                    }
#pragma unroll
                    for (int t = 0; t < KK; ++t)
                        acc[t][k] = __builtin_amdgcn_fdot2(xp, __builtin_bit_cast(rows::half2_t, ww[ST][t][pr]),
                                                           acc[t][k], false);
                }
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float xv[VP];
#pragma unroll
                for (int k = 0; k < VP; ++k) xv[k] = rows::elem<T>(xw[ST][u], S * k);
#pragma unroll
                for (int t = 0; t < KK; ++t) {
                    const float wv = rows::elem<T>(ww[ST][t], u);
#pragma unroll
                    for (int k = 0; k < VP; ++k) acc[t][k] = fmaf(wv, xv[k], acc[t][k]);
                }
            }
        }
    };
    // (in this order: the waits inside the walk count the loads that were issued later)
    issue(std::integral_constant<int, 0>{}, 0);
    issue_weights(std::integral_constant<int, 0>{}, 0);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (NST > 2) issue(std::integral_constant<int, 1>{}, 1);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (NST > 3) issue(std::integral_constant<int, 2>{}, 2);
    __builtin_amdgcn_sched_barrier(0);
    auto step = [&](auto st_tag, int i) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value;
        issue(std::integral_constant<int, (ST + NST - 1) % NST>{}, i + NST - 1);
        issue_weights(std::integral_constant<int, (ST + 1) % NST>{}, i + 1);
        __builtin_amdgcn_sched_barrier(0);
        compute(st_tag, i);
        __builtin_amdgcn_sched_barrier(0);
    };
    for (int i = 0; i < g.steps; i += NST) {
        step(std::integral_constant<int, 0>{}, i);
        if constexpr (NST > 1) step(std::integral_constant<int, 1>{}, i + 1);
        if constexpr (NST > 2) step(std::integral_constant<int, 2>{}, i + 2);
        if constexpr (NST > 3) step(std::integral_constant<int, 3>{}, i + 3);
    }

    if constexpr (WAVES > 1) {
        // the other waves' sums reach wave 0 through LDS, [wave][tap][lane][pixel]
        __shared__ __align__(16) float red[WAVES - 1][KK][kWave][VP];
        if (wave > 0) {
#pragma unroll
            for (int t = 0; t < KK; ++t)
#pragma unroll
                for (int k = 0; k < VP; ++k) red[wave - 1][t][lane][k] = acc[t][k];
        }
        __syncthreads();
        if (wave > 0) return;
        // (one wave's sums at a time: unrolled, all of them would be in registers at once)
#pragma unroll 1
        for (int q = 0; q < WAVES - 1; ++q)
#pragma unroll
            for (int t = 0; t < KK; ++t)
#pragma unroll
                for (int k = 0; k < VP; ++k) acc[t][k] += red[q][t][lane][k];
    }
    TapParams<T, KK> params;
    params.load(head, gain, gain_vec, offset_vec, bias);
#pragma unroll
    for (int k = 0; k < VP; ++k) {
        float r[KK];
#pragma unroll
        for (int t = 0; t < KK; ++t) r[t] = acc[t][k];
        normalise<T, KK>(r, params);
#pragma unroll
        for (int t = 0; t < KK; ++t) acc[t][k] = r[t];
    }
    T *on = sf + ((n * heads + head) * KK) * (int64_t)g.npix;
    const __amdgpu_buffer_rsrc_t orr = plane_rsrc(on, (uint32_t)KK * (uint32_t)g.npix * (uint32_t)sizeof(T));
    const uint32_t ob = live ? (uint32_t)p * (uint32_t)sizeof(T) : kOutside;
#pragma unroll
    for (int t = 0; t < KK; ++t) {
        uint32_t ow[NWO];
        rows::pack<T, VP, float>(acc[t], ow);
        store_vec_nt<kOB>(orr, ob + (uint32_t)t * (uint32_t)g.npix * (uint32_t)sizeof(T), ow);
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
    float gain, const T *__restrict__ gain_vec, const T *__restrict__ offset_vec,
    const float *__restrict__ parts, int nparts, float scale) {
    extern __shared__ float branch_smem[];
    float *v = branch_smem;            // [NS][C]
    float *h = v + NS * C;             // [NS][mid]
    float *f = h + NS * mid;           // [NS][BLOCK * KK]
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int64_t n0 = (int64_t)blockIdx.y * NS;
    const int ns = min(NS, N - (int)n0);   // samples of this workgroup (the others: copies of the last)
    const int cb = blockIdx.x * BLOCK;
    // the pooled vectors: given, or scale * the sum of nparts partial sums per value
    // (parts[(n * nparts + p) * C + c], what k_spatial_stream leaves)
    for (int i = threadIdx.x; i < NS * C; i += kChannelThreads) {
        const int s = i / C, c = i - s * C;
        const int64_t n = n0 + min(s, ns - 1);
        if (parts) {
            float a = 0.f;
#pragma unroll 4
            for (int q = 0; q < nparts; ++q) a += parts[(n * nparts + q) * C + c];
            v[i] = a * scale;
        } else {
            v[i] = ld(pooled + n * C + c);
        }
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


// ---- the channel branch on the matrix cores (fp16) ---------------------------
//
// Both 1x1 convolutions are matrix products with the batch as one dimension:
//   hidden[m, n] = relu(b1[m] + sum_c w1[m, c] * v[n, c])           (mid x C) . (C x N)
//   taps[r, n]   = b2[r] + sum_m w2[r, m] * hidden[m, n]            (C*KK x mid) . (mid x N)
// v_mfma_f32_16x16x32_f16 takes, per lane l of a wave, eight values of a row of A
// (row l % 16, positions 8 * (l / 16) + 0..7 of the 32 the step covers: one
// 16-byte load from a row-major weight matrix) and the eight values of column
// l % 16 of B at the same positions, and leaves D[4 * (l / 16) + 0..3][l % 16].
// A workgroup takes sixteen samples (the columns) and `block` channels:
//   * the pooled vectors go to LDS as [32 channels][sample][32], rounded to fp16
//     (what the reference's half-precision pooling returns);
//   * the hidden layer goes to LDS as [32 values][sample][32], rounded to fp16 (as
//     the reference's first convolution does);
//   * the rows of tile j of the second product are (channel c0 + i, tap j), so a
//     lane ends up with all KK taps of four channels of one sample and
//     normalises them in registers: 4 * KK contiguous values to store.
// mid is no multiple of 32 (nor of 16): the last tile of hidden values starts at
// mid - 32 (mid - 16 for the rows of the first product) and overlaps the one
// before it; the overlapping positions of its B operand are zero (they are
// counted in the tile before), so every weight that is read is a weight of the
// row it is used for.  Rows of w2 start at any even byte address: its loads are
// 16 bytes at 2-byte alignment.
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ half8_t load_half8_any(const __half *p) {
    half8_t v;
    __builtin_memcpy(&v, p, sizeof(v));
    return v;
}
__device__ __forceinline__ half8_t load_half8(const __half *p) {
    return *reinterpret_cast<const half8_t *>(p);
}
__device__ __forceinline__ half4_t load_half4(const __half *p) {
    return *reinterpret_cast<const half4_t *>(p);
}

constexpr int kMmaSamples = 16;
constexpr int kMmaStep = 32;                          // values of the summed dimension per instruction
constexpr int kMmaTile = kMmaSamples * kMmaStep;      // halves of one [sample][32] tile in LDS

template <int KK, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) void k_channel_branch_mma(
    const __half *__restrict__ pooled, const __half *__restrict__ w1, const __half *__restrict__ b1,
    const __half *__restrict__ w2, const __half *__restrict__ b2, __half *__restrict__ cf, int N, int C,
    int mid, int block, float gain, const __half *__restrict__ gain_vec,
    const __half *__restrict__ offset_vec, const float *__restrict__ parts, int nparts, float scale) {
    extern __shared__ __align__(16) _Float16 mma_smem[];
    _Float16 *pv = mma_smem;                        // [C / 32][16 samples][32]: pooled vectors
    _Float16 *hv = pv + (C / kMmaStep) * kMmaTile;  // [tiles of mid][16 samples][32]: hidden vectors
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int col = lane & 15, quad = lane >> 4;
    const int n0 = blockIdx.y * kMmaSamples;
    const int cb = blockIdx.x * block;
    const int rtiles = (mid + 15) >> 4;             // tiles of sixteen rows of w1
    const int ktiles = (mid + kMmaStep - 1) / kMmaStep;   // steps of the second product
    const int klast = mid - kMmaStep;               // where the last of them starts
    const int nk = C / kMmaStep;                    // steps of the first product

    // All waves: the pooled vectors of the sixteen samples into LDS, four channels per
    // item (given, or scale * the sum of nparts partial sums per value), and zeros in
    // the last tile of the hidden layer (its overlap with the tile before stays zero).
    auto pooled_vectors = [&]() {
        const int c4s = C >> 2;
        for (int i = threadIdx.x; i < kMmaSamples * c4s; i += WAVES * kWave) {
            const int s = i / c4s, c4 = i - s * c4s;
            const int64_t n = min(n0 + s, N - 1);
            half4_t v;
            if (parts) {
                const float4_t *src = reinterpret_cast<const float4_t *>(parts + n * nparts * C) + c4;
                float4_t a = {0.f, 0.f, 0.f, 0.f};
                // four partial sums requested together (the fence keeps the compiler from
                // taking them one round trip at a time to save registers)
                int q = 0;
                for (; q + 4 <= nparts; q += 4) {
                    const float4_t x0 = src[(int64_t)q * c4s], x1 = src[(int64_t)(q + 1) * c4s],
                                   x2 = src[(int64_t)(q + 2) * c4s], x3 = src[(int64_t)(q + 3) * c4s];
                    __builtin_amdgcn_sched_barrier(0);
                    a += (x0 + x1) + (x2 + x3);
                }
                for (; q < nparts; ++q) a += src[(int64_t)q * c4s];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = (_Float16)(a[e] * scale);
            } else {
                v = load_half4(pooled + n * C + c4 * 4);
            }
            *reinterpret_cast<half4_t *>(pv + ((c4 >> 3) * kMmaSamples + s) * kMmaStep + (c4 & 7) * 4) = v;
        }
        for (int i = threadIdx.x; i < kMmaTile / 2; i += WAVES * kWave)
            reinterpret_cast<uint32_t *>(hv + (ktiles - 1) * kMmaTile)[i] = 0u;
    };

    // The first waves compute taps (a tile of sixteen channels at a time), the others
    // the hidden layer; each kind asks for the first weights it will need before
    // anything else (they depend on nothing, and are there by the time the operand
    // from LDS is).  The two kinds run separate code, so each has the whole register
    // file for what it keeps in flight; both pass the same two barriers.
    const int tap_waves = min(min(block, C - cb) >> 4, WAVES - 1);
    if (wave >= tap_waves) {
        // ---- hidden layer: tiles of sixteen rows of w1 ----
        constexpr int kPre1 = 16;
        const int hidden_waves = WAVES - tap_waves;
        const int t0 = wave - tap_waves;
        half8_t apre[kPre1];
        auto request = [&](int t) {
            const __half *arow = w1 + (int64_t)(min(t * 16, mid - 16) + col) * C + quad * 8;
#pragma unroll
            for (int u = 0; u < kPre1; ++u) apre[u] = load_half8(arow + min(u, nk - 1) * kMmaStep);
        };
        if (t0 < rtiles) request(t0);
        pooled_vectors();
        __syncthreads();
        for (int t = t0; t < rtiles; t += hidden_waves) {
            if (t != t0) request(t);
            const int mbase = min(t * 16, mid - 16);
            const __half *arow = w1 + (int64_t)(mbase + col) * C + quad * 8;
            const _Float16 *brow = pv + col * kMmaStep + quad * 8;
            float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < kPre1; ++u) {
                if (u < nk)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        apre[u], *reinterpret_cast<const half8_t *>(brow + u * kMmaTile), acc, 0, 0, 0);
            }
            // (the matrix instruction is convergent, which rules out unrolling with a
            // remainder: chunks of a fixed number of steps, all loads of a chunk first)
            int kb = kPre1;
            auto chunk = [&](auto steps) {
                constexpr int U = decltype(steps)::value;
                half8_t a[U];
#pragma unroll
                for (int u = 0; u < U; ++u) a[u] = load_half8(arow + (kb + u) * kMmaStep);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < U; ++u)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        a[u], *reinterpret_cast<const half8_t *>(brow + (kb + u) * kMmaTile), acc, 0, 0, 0);
                kb += U;
            };
            while (nk - kb >= 16) chunk(std::integral_constant<int, 16>());
            if (nk - kb >= 8) chunk(std::integral_constant<int, 8>());
            if (nk - kb >= 4) chunk(std::integral_constant<int, 4>());
            while (kb < nk) chunk(std::integral_constant<int, 1>());
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int m = mbase + quad * 4 + e;
                if (m < t * 16) continue;    // (the last tile's overlap: those rows belong to the tile before)
                const float bias = b1 ? ld(b1 + m) : 0.f;
                const int kt = min(m / kMmaStep, ktiles - 1);
                hv[(kt * kMmaSamples + col) * kMmaStep + m - min(kt * kMmaStep, klast)] =
                    (_Float16)fmaxf(acc[e] + bias, 0.f);
            }
        }
        __syncthreads();
        return;
    }

    // ---- taps: per wave sixteen channels x KK taps x sixteen samples ----
    constexpr int kPre = KK <= 9 ? 2 : 1;           // steps of the second product requested up front
    half4_t pg[KK], po[KK], pb[KK];
    half8_t apre[kPre][KK];
    auto request = [&](int c0) {
        // gains, offsets and biases of this lane's four channels: 4 * KK contiguous values each
        const int64_t pbase = (int64_t)(c0 + quad * 4) * KK;
#pragma unroll
        for (int j = 0; j < KK; ++j) pg[j] = po[j] = pb[j] = half4_t{0, 0, 0, 0};
        if (gain_vec) {
#pragma unroll
            for (int j = 0; j < KK; ++j) pg[j] = load_half4(gain_vec + pbase + 4 * j);
        }
        if (offset_vec) {
#pragma unroll
            for (int j = 0; j < KK; ++j) po[j] = load_half4(offset_vec + pbase + 4 * j);
        }
        if (b2) {
#pragma unroll
            for (int j = 0; j < KK; ++j) pb[j] = load_half4(b2 + pbase + 4 * j);
        }
        const __half *arow = w2 + (int64_t)(c0 + col) * KK * mid + quad * 8;
#pragma unroll
        for (int u = 0; u < kPre; ++u) {
            const int kbase = min(u * kMmaStep, klast);    // (steps past the last one: the last one again, unused)
#pragma unroll
            for (int j = 0; j < KK; ++j) apre[u][j] = load_half8_any(arow + j * mid + kbase);
        }
    };
    request(cb + wave * 16);
    pooled_vectors();
    __syncthreads();
    __syncthreads();
    const int n = n0 + col;
    for (int ct = wave; ct * 16 < block && cb + ct * 16 < C; ct += tap_waves) {
        const int c0 = cb + ct * 16;
        if (ct != wave) request(c0);
        float4_t acc[KK];
#pragma unroll
        for (int j = 0; j < KK; ++j) acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
        const __half *arow = w2 + (int64_t)(c0 + col) * KK * mid + quad * 8;
        const _Float16 *brow = hv + col * kMmaStep + quad * 8;
#pragma unroll
        for (int u = 0; u < kPre; ++u) {
            if (u < ktiles) {
                const half8_t b = *reinterpret_cast<const half8_t *>(brow + u * kMmaTile);
#pragma unroll
                for (int j = 0; j < KK; ++j)
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(apre[u][j], b, acc[j], 0, 0, 0);
            }
        }
        int t = kPre;
        auto tiles = [&](auto count) {
            constexpr int U = decltype(count)::value;
            half8_t a[U][KK];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int kbase = min((t + u) * kMmaStep, klast);
#pragma unroll
                for (int j = 0; j < KK; ++j) a[u][j] = load_half8_any(arow + j * mid + kbase);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const half8_t b = *reinterpret_cast<const half8_t *>(brow + (t + u) * kMmaTile);
#pragma unroll
                for (int j = 0; j < KK; ++j)
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u][j], b, acc[j], 0, 0, 0);
            }
            t += U;
        };
        while (ktiles - t >= kPre) tiles(std::integral_constant<int, kPre>());
        if (kPre > 1 && t < ktiles) tiles(std::integral_constant<int, 1>());
        if (n >= N) continue;
        half4_t out[KK];   // channel e of the lane's four: values [e * KK, (e + 1) * KK) of the 4 * KK
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float u[KK];
            TapParams<__half, KK> params;
#pragma unroll
            for (int j = 0; j < KK; ++j) {
                const int at = e * KK + j;
                u[j] = acc[j][e];
                params.gain[j] = gain_vec ? (float)pg[at >> 2][at & 3] : gain;
                params.offset[j] = offset_vec ? (float)po[at >> 2][at & 3] : 0.f;
                params.bias[j] = b2 ? (float)pb[at >> 2][at & 3] : 0.f;
            }
            normalise<__half, KK>(u, params);
#pragma unroll
            for (int j = 0; j < KK; ++j) {
                const int at = e * KK + j;
                out[at >> 2][at & 3] = (_Float16)u[j];
            }
        }
        half4_t *op = reinterpret_cast<half4_t *>(cf + ((int64_t)n * C + c0 + quad * 4) * KK);
#pragma unroll
        for (int j = 0; j < KK; ++j) op[j] = out[j];
    }
}

}  // namespace

bool branch_kernel_size_built(int k) { return k == 3 || k == 5; }

// Launch of k_spatial_stream; hipErrorNotSupported where it does not cover the problem
// (the caller then takes the kernels above).
template <typename T>
hipError_t spatial_stream(const T *x, const T *w, const T *bias, T *sf, int64_t N, int64_t C, int64_t H,
                          int64_t W, int head, int stride, double gain, const T *gain_vec,
                          const T *offset_vec, hipStream_t st, float *pool_part = nullptr,
                          int64_t pool_capacity = 0, int *pool_parts = nullptr) {
    constexpr int KK = 9, NST = 3;
    constexpr int U = sizeof(T) == 2 ? 4 : 2;
    constexpr int esz = (int)sizeof(T);
    const int64_t Ho = H / stride, Wo = W / stride, npix = Ho * Wo;
    if (tune_int("DDF_TUNE_SPATIAL_STREAM", 1) == 0) return hipErrorNotSupported;
    if (stride != 1 && stride != 2) return hipErrorNotSupported;
    if (C % U != 0 || ((uintptr_t)w % 4) != 0) return hipErrorNotSupported;
    if (C * H * W * esz >= (1ll << 31) || KK * npix * esz >= (1ll << 31)) return hipErrorNotSupported;
    // pixels per lane: the widest vector the shapes and addresses allow ...
    const bool pool = pool_part != nullptr;
    if (pool && stride == 2 && (H % 2 != 0 || W % 2 != 0)) return hipErrorNotSupported;   // (pixels no lane covers)
    auto fits = [&](int vp) {
        if (npix % vp != 0 || ((uintptr_t)sf % (vp * esz)) != 0) return false;
        if (pool && stride == 2 && vp == 1) return ((uintptr_t)x % (2 * esz)) == 0;   // (pairs of columns)
        if (stride == 1) return ((uintptr_t)x % (vp * esz)) == 0 && (H * W) % vp == 0;
        if (vp == 1) return true;
        return Wo % vp == 0 && W % vp == 0 && (H * W) % (2 * vp) == 0 && ((uintptr_t)x % (2 * vp * esz)) == 0;
    };
    const int vp_max = (stride == 1 ? 16 : 8) / esz;
    // ... that still leaves enough waves to fill the machine: the waves of a workgroup
    // share its pixels and split the channels, at least two pipeline rounds each
    const int64_t want = tune_int("DDF_TUNE_SPATIAL_WANT", 2048);
    int vp = 0, waves = 1;
    for (int cand = vp_max; cand >= 1; cand /= 2) {
        if (!fits(cand)) continue;
        const int64_t nvec = npix / cand;
        const int64_t tiles = cdiv(nvec, kWave) * N * head;
        int wv = 1;
        // (nearly a wave per SIMD with whole channel walks: better than splitting them)
        if (tiles < tune_int("DDF_TUNE_SPATIAL_WHOLE", 768))
            while (wv < 16 && wv * 2 * cand <= 32 && tiles * wv < want && (C / U) / (wv * 2) >= 2 * NST)
                wv *= 2;
        vp = cand;
        waves = wv;
        if (tiles * wv >= want || wv == 1) break;
    }
    const int fvp = tune_int("DDF_TUNE_SPATIAL_VP", 0), fwv = tune_int("DDF_TUNE_SPATIAL_WAVES", 0);
    if (fvp > 0 && fvp <= vp_max && fits(fvp)) vp = fvp;
    if (fwv > 0) waves = fwv;
    if (vp == 0) return hipErrorNotSupported;
    if (vp * waves > 32 || (waves & (waves - 1)) != 0 || waves > 16) return hipErrorNotSupported;   // (the variants built)
    SpatialGeom g;
    g.C = (int)C; g.W = (int)W; g.Wo = (int)Wo;
    g.plane = (int)(H * W);
    g.npix = (int)npix;
    g.nvec = (int)(npix / vp);
    const int tiles = (int)cdiv(g.nvec, kWave);
    g.lpt = (int)cdiv(g.nvec, tiles);                   // (tiles of equal size)
    g.ngroups = (int)(C / U);
    g.gpw = (int)cdiv(g.ngroups, waves);
    g.steps = (int)cdiv(g.gpw, NST) * NST;
    if (N > 65535 || head > 65535) return hipErrorNotSupported;
    if (pool) {
        if (N * tiles * 4 * C > pool_capacity) return hipErrorInvalidValue;
        *pool_parts = tiles * 4;
    }
    const dim3 grid((unsigned)tiles, (unsigned)head, (unsigned)N);
#define DDF_STREAM_LAUNCH(VP_, S_, WAVES_)                                                        \
    do {                                                                                          \
        if (pool) {                                                                               \
            hipLaunchKernelGGL((k_spatial_stream<T, KK, VP_, S_, WAVES_, U, NST, true>), grid,    \
                               dim3(WAVES_ * kWave), 0, st, g, x, w, bias, sf, (float)gain,       \
                               gain_vec, offset_vec, pool_part);                                  \
            break;                                                                                \
        }                                                                                         \
        hipLaunchKernelGGL((k_spatial_stream<T, KK, VP_, S_, WAVES_, U, NST, false>), grid,       \
                           dim3(WAVES_ * kWave), 0, st, g, x, w, bias, sf, (float)gain, gain_vec, \
                           offset_vec, (float *)nullptr);                                         \
    } while (0)
#define DDF_STREAM_WAVES(VP_, S_)                                                                 \
    do {                                                                                          \
        if (waves == 1) DDF_STREAM_LAUNCH(VP_, S_, 1);                                            \
        else if (waves == 2) DDF_STREAM_LAUNCH(VP_, S_, 2);                                       \
        else if (waves == 4) DDF_STREAM_LAUNCH(VP_, S_, 4);                                       \
        else if (waves == 8 && VP_ <= 4) DDF_STREAM_LAUNCH((VP_ <= 4 ? VP_ : 1), S_, 8);          \
        else if (waves == 16 && VP_ <= 2) DDF_STREAM_LAUNCH((VP_ <= 2 ? VP_ : 1), S_, 16);        \
        else return hipErrorNotSupported;                                                         \
    } while (0)
    if (stride == 1) {
        if (vp == 8) { if constexpr (esz == 2) DDF_STREAM_WAVES(8, 1); else return hipErrorNotSupported; }
        else if (vp == 4) DDF_STREAM_WAVES(4, 1);
        else if (vp == 2) DDF_STREAM_WAVES(2, 1);
        else DDF_STREAM_WAVES(1, 1);
    } else {
        if (vp == 4) { if constexpr (esz == 2) DDF_STREAM_WAVES(4, 2); else return hipErrorNotSupported; }
        else if (vp == 2) DDF_STREAM_WAVES(2, 2);
        else DDF_STREAM_WAVES(1, 2);
    }
#undef DDF_STREAM_WAVES
#undef DDF_STREAM_LAUNCH
    return hipGetLastError();
}

template <typename T>
hipError_t spatial_branch(const T *x, const T *w, const T *bias, T *sf, int64_t N, int64_t C,
                          int64_t H, int64_t W, int head, int k, int stride, double gain,
                          const T *gain_vec, const T *offset_vec, hipStream_t st, float *pool_part,
                          int64_t pool_capacity, int *pool_parts) {
    const int64_t Ho = H / stride, Wo = W / stride;
    if (N == 0 || C == 0 || Ho * Wo == 0 || head == 0) return hipSuccess;
    if (N > 65535 || head > 65535 || C > (1 << 24) || H * W >= (1ll << 31)) return hipErrorNotSupported;
    if (k == 3) {
        const hipError_t err = spatial_stream<T>(x, w, bias, sf, N, C, H, W, head, stride, gain, gain_vec,
                                                 offset_vec, st, pool_part, pool_capacity, pool_parts);
        if (err != hipErrorNotSupported) return err;
    }
    if (pool_part) return hipErrorNotSupported;   // (only the streaming kernel pools)
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

// The matrix-core kernel where it applies (fp16, a hidden layer of at least one
// step of the matrix instruction, whole steps of channels, operands aligned for
// its vector loads); hipErrorNotSupported otherwise.
template <typename T>
hipError_t channel_branch_mma(const T *, const T *, const T *, const T *, const T *, T *, int64_t, int64_t,
                              int64_t, int, double, const T *, const T *, hipStream_t, const float *, int,
                              double) {
    return hipErrorNotSupported;
}
template <>
hipError_t channel_branch_mma<__half>(const __half *pooled, const __half *w1, const __half *b1,
                                      const __half *w2, const __half *b2, __half *cf, int64_t N, int64_t C,
                                      int64_t mid, int k, double gain, const __half *gain_vec,
                                      const __half *offset_vec, hipStream_t st, const float *parts,
                                      int nparts, double scale) {
    if (tune_int("DDF_TUNE_CHANNEL_MMA", 1) == 0) return hipErrorNotSupported;
    auto aligned = [](const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; };
    const size_t lds = (size_t)(C / kMmaStep + cdiv(mid, kMmaStep)) * kMmaTile * sizeof(__half);
    if ((k != 3 && k != 5) || mid < kMmaStep || C % kMmaStep != 0 || lds > 64 * 1024 ||
        N > (int64_t)65535 * kMmaSamples || C * k * k * mid >= ((int64_t)1 << 31))
        return hipErrorNotSupported;
    if (!aligned(w1, 16) || !aligned(cf, 8) || !aligned(b2, 8) || !aligned(gain_vec, 8) ||
        !aligned(offset_vec, 8) || !aligned(w2, 2) || (parts ? !aligned(parts, 16) : !aligned(pooled, 8)))
        return hipErrorNotSupported;
    // (25 taps: the accumulators and parameters of a tile need the registers of a wave alone on its SIMD)
    const int waves = k == 3 && tune_int("DDF_TUNE_CHANNEL_MMA_WAVES", 8) == 8 ? 8 : 4;
    int block = tune_int("DDF_TUNE_CHANNEL_MMA_BLOCK", 16);
    block = std::max(16, block / 16 * 16);
    const dim3 grid((unsigned)cdiv(C, block), (unsigned)cdiv(N, kMmaSamples));
#define DDF_MMA_LAUNCH(KK_, WAVES_)                                                                  \
    hipLaunchKernelGGL((k_channel_branch_mma<KK_, WAVES_>), grid, dim3(WAVES_ * kWave), lds, st, pooled, \
                       w1, b1, w2, b2, cf, (int)N, (int)C, (int)mid, block, (float)gain, gain_vec,      \
                       offset_vec, parts, nparts, (float)scale)
    if (k == 3 && waves == 8) DDF_MMA_LAUNCH(9, 8);
    else if (k == 3) DDF_MMA_LAUNCH(9, 4);
    else DDF_MMA_LAUNCH(25, 4);
#undef DDF_MMA_LAUNCH
    return hipGetLastError();
}

template <typename T>
hipError_t channel_branch(const T *pooled, const T *w1, const T *b1, const T *w2, const T *b2,
                          T *cf, int64_t N, int64_t C, int64_t mid, int k, double gain,
                          const T *gain_vec, const T *offset_vec, hipStream_t st, const float *parts,
                          int nparts, double scale) {
    if (N == 0 || C == 0) return hipSuccess;
    const int kk = k * k;
    if (hipError_t e = channel_branch_mma(pooled, w1, b1, w2, b2, cf, N, C, mid, k, gain, gain_vec,
                                          offset_vec, st, parts, nparts, scale);
        e != hipErrorNotSupported)
        return e;
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
                       gain_vec, offset_vec, parts, nparts, (float)scale)
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
                                          const T *, hipStream_t, float *, int64_t, int *);      \
    template hipError_t channel_branch<T>(const T *, const T *, const T *, const T *, const T *, \
                                          T *, int64_t, int64_t, int64_t, int, double, const T *, \
                                          const T *, hipStream_t, const float *, int, double);
DDF_INSTANTIATE_BRANCHES(__half)
DDF_INSTANTIATE_BRANCHES(float)
#undef DDF_INSTANTIATE_BRANCHES

}  // namespace ddf
