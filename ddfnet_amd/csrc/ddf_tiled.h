// Tiled DDF kernels for gfx950 (wave64): LDS-staged input strips, spatial-filter
// taps held in registers and reused across the channels a workgroup walks,
// wavefront butterfly reductions for the channel-filter gradient.
//
// All kernels work on full-width row strips of one (n, channel-range): a strip
// of an NCHW plane is one contiguous run in memory, so every global load and
// store is a linear, coalesced access, and only the vertical halo is re-read.
// The strip is staged in LDS with a zero border, which makes the tap loop free
// of bounds tests.  Included by one translation unit per element type.
#pragma once

#include "ddf_common.h"

namespace ddf {

// Geometry of one launch, computed on the host (ddf_tiled_host.hip).
struct TileGeom {
    int C, H, W, Ho, Wo;   // problem (per sample)
    int rows, cols;        // grid of work cells a strip is cut from
    int TH, nstrips;       // cell rows per strip
    int P, IH, tile;       // LDS tile: IH rows of pitch P elements; tile = IH * P
    int src_rows, src_cols;  // extent of the tensor staged in LDS (X or dO)
    int row0_off;          // source row of tile row 0, for strip 0 (adds strip*TH*row_step)
    int row_step;          // source rows advanced per cell row
    int col_off;           // tile column of source column 0
    int cpb, csplit, CB;   // channels per block / number of channel splits / per LDS stage
    int threads, nwaves;
    int lw_shift, lrows;   // loader: row width 1<<lw_shift, rows per pass
    unsigned cols_magic;   // ceil(2^32 / cols): q / cols for q < 65536; 0 when cols == 1
    int nblocks;           // logical blocks = N * nstrips * csplit
    int lds_bytes;
};

namespace tiled {

constexpr int kXcd = 8;

// Workgroups are handed to the 8 XCDs round-robin by hardware.  Renumber them
// so that consecutive logical blocks (same sample, neighbouring channel
// ranges: same spatial filter) share an XCD and its L2.
__device__ __forceinline__ int logical_block(int nblocks) {
    const int per = (nblocks + kXcd - 1) / kXcd;
    return (int)(blockIdx.x % kXcd) * per + (int)(blockIdx.x / kXcd);
}

// q / g.cols for q < 65536 by multiplication; cols == 1 has no 32-bit magic.
__device__ __forceinline__ int row_of(int q, const TileGeom &g) {
    return g.cols_magic ? (int)__umulhi((unsigned)q, g.cols_magic) : q;
}

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int CTRL>
__device__ __forceinline__ double dpp_move(double v) {
    const long long b = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_update_dpp(0, (int)(b & 0xffffffffll), CTRL, 0xf, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(0, (int)(b >> 32), CTRL, 0xf, 0xf, false);
    return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}

// Value held by the partner lane of butterfly stage STAGE.  Stages 0, 1, 3
// are swaps (lane^1, lane^2, lane^8); stage 2 rotates the 16-lane row by 4, so
// a lane receives from the quad next to its own: after stage 3 the two
// rotations have covered all four quads of the row.  Stages 4, 5 cross rows.
template <int STAGE, typename A>
__device__ __forceinline__ A lane_xchg(A v) {
    if constexpr (STAGE == 0) return dpp_move<0xB1>(v);        // quad_perm [1,0,3,2]
    else if constexpr (STAGE == 1) return dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
    else if constexpr (STAGE == 2) return dpp_move<0x124>(v);  // row_ror:4
    else if constexpr (STAGE == 3) return dpp_move<0x128>(v);  // row_ror:8
    else if constexpr (STAGE == 4) return __shfl_xor(v, 16, kWave);
    else return __shfl_xor(v, 32, kWave);
}

// Sum each of N per-lane values over the 64 lanes of the wavefront.  At every
// stage a lane keeps one half of its values and hands the other half to its
// partner, so the work is ~3N instructions instead of 6N.  Returns the total
// of the value whose index bfly_index() reports for this lane.
template <int N, int STAGE, typename A>
__device__ __forceinline__ A bfly_sum(const A (&v)[N], int lane) {
    if constexpr (STAGE == 6) {
        static_assert(N == 1, "at most 64 values");
        return v[0];
    } else {
        constexpr int h = N / 2, M = h + (N & 1);
        A nv[M];
        const bool up = (lane >> STAGE) & 1;
#pragma unroll
        for (int j = 0; j < h; ++j) {
            const A keep = up ? v[j + h] : v[j];
            const A send = up ? v[j] : v[j + h];
            nv[j] = keep + lane_xchg<STAGE>(send);
        }
        if constexpr (N & 1) nv[h] = v[2 * h] + lane_xchg<STAGE>(v[2 * h]);
        return bfly_sum<M, STAGE + 1, A>(nv, lane);
    }
}

template <int N, int STAGE>
__device__ __forceinline__ int bfly_index(const int (&id)[N], int lane) {
    if constexpr (STAGE == 6) {
        return id[0];
    } else {
        constexpr int h = N / 2, M = h + (N & 1);
        int nid[M];
        const bool up = (lane >> STAGE) & 1;
#pragma unroll
        for (int j = 0; j < h; ++j) nid[j] = up ? id[j + h] : id[j];
        if constexpr (N & 1) nid[h] = id[2 * h];
        return bfly_index<M, STAGE + 1>(nid, lane);
    }
}

// Lanes below this bound hold every index at least once after the reduction.
template <int N>
constexpr int bfly_writers() {
    int w = 1;
    while (w < N) w *= 2;
    return w < kWave ? w : kWave;
}

// Stage CB source planes' strips in LDS.  Thread (lrow, lcol) copies source
// element (row0 + r, lcol) for r = lrow, lrow + lrows, ...; cells outside the
// source stay at the zero written once at kernel start.
template <typename T>
__device__ __forceinline__ void stage_strips(const TileGeom &g, T *lds, const T *src_plane0,
                                             int64_t plane_stride, int ncb, int row0) {
    const int lw = 1 << g.lw_shift;
    const int lcol = threadIdx.x & (lw - 1);
    const int lrow = threadIdx.x >> g.lw_shift;
    if (lrow >= g.lrows) return;
    for (int cl = 0; cl < ncb; ++cl) {
        const T *src = src_plane0 + cl * plane_stride;
        T *dst = lds + cl * g.tile + g.col_off;
        for (int r = lrow; r < g.IH; r += g.lrows) {
            const int sr = row0 + r;
            if (sr < 0 || sr >= g.src_rows) continue;
            for (int col = lcol; col < g.src_cols; col += lw)
                dst[r * g.P + col] = src[(int64_t)sr * g.src_cols + col];
        }
    }
}

// ---------------------------------------------------------------------------
// Forward.  Work cell = output pixel; threads of the block split the strip's
// pixels, every wave walks the same channels.
// ---------------------------------------------------------------------------
template <typename T, int K, int D, int S, bool MUL, int PS>
__global__ __launch_bounds__(512) void k_forward(TileGeom g, const T *__restrict__ x,
                                                 const T *__restrict__ cf,
                                                 const T *__restrict__ sf,
                                                 T *__restrict__ out) {
    using A = typename Acc<T>::type;
    constexpr int KK = K * K, R = (K - 1) / 2;
    extern __shared__ __align__(16) unsigned char smem[];
    T *lds = reinterpret_cast<T *>(smem);

    const int b = logical_block(g.nblocks);
    if (b >= g.nblocks) return;
    const int cs = b % g.csplit;
    const int strip = (b / g.csplit) % g.nstrips;
    const int64_t n = b / (g.csplit * g.nstrips);
    const int y0 = strip * g.TH;
    const int np = min(g.TH, g.rows - y0) * g.cols;
    const int c_begin = cs * g.cpb, c_end = min(g.C, c_begin + g.cpb);
    const int64_t oplane = (int64_t)g.Ho * g.Wo, iplane = (int64_t)g.H * g.W;

    for (int i = threadIdx.x; i < g.CB * g.tile; i += g.threads) lds[i] = T(0.0f);

    int lb[PS];
    bool ok[PS];
    A sfr[PS][KK];
#pragma unroll
    for (int m = 0; m < PS; ++m) {
        const int q = threadIdx.x + m * g.threads;
        ok[m] = q < np;
        const int oy = row_of(q, g);
        const int ox = q - oy * g.cols;
        lb[m] = ok[m] ? (oy * S) * g.P + ox * S : 0;
        const T *sfp = sf + (n * KK * g.Ho + y0) * g.Wo + q;
#pragma unroll
        for (int t = 0; t < KK; ++t) sfr[m][t] = ok[m] ? (A)ld(sfp + t * oplane) : A(0);
    }
    const int row0 = y0 * S + g.row0_off;
    __syncthreads();

    for (int c0 = c_begin; c0 < c_end; c0 += g.CB) {
        const int ncb = min(g.CB, c_end - c0);
        stage_strips(g, lds, x + (n * g.C + c0) * iplane, iplane, ncb, row0);
        __syncthreads();
        for (int cl = 0; cl < ncb; ++cl) {
            const int64_t nc = n * g.C + c0 + cl;
            A w[KK];
#pragma unroll
            for (int t = 0; t < KK; ++t) w[t] = ld(cf + nc * KK + t);
            const T *tl = lds + cl * g.tile;
#pragma unroll
            for (int m = 0; m < PS; ++m) {
                if (!ok[m]) continue;
                A acc = 0;
#pragma unroll
                for (int i = 0; i < K; ++i)
#pragma unroll
                    for (int j = 0; j < K; ++j)
                        acc += (A)ld(tl + lb[m] + i * D * g.P + j * D) *
                               comb<MUL, A>(w[i * K + j], sfr[m][i * K + j]);
                st(out + (nc * g.Ho + y0) * g.Wo + threadIdx.x + m * g.threads, acc);
            }
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------------------
// Gradient with respect to the features.  Work cell (qy, qx) = the S x S block
// of input pixels (qy*S + pu, qx*S + pv).  Input pixel row u receives tap row
// i only when u - (i-R)*D is a multiple of S; with e = (i-R)*D that fixes the
// phase pu = e mod S and the output row qy + (pu - e)/S, both compile-time.
// dO is staged in LDS, the spatial filter is gathered at the neighbour
// positions once per cell and kept in registers.
// ---------------------------------------------------------------------------
template <int K, int D, int S>
struct TapMap {
    static constexpr int R = (K - 1) / 2;
    static constexpr int e(int i) { return (i - R) * D; }
    static constexpr int phase(int i) { return ((e(i) % S) + S) % S; }
    static constexpr int dq(int i) { return (phase(i) - e(i)) / S; }
    static constexpr int halo_lo = (R * D) / S;            // cells above / left
    static constexpr int halo_hi = (R * D + S - 1) / S;    // cells below / right
};

template <typename T, int K, int D, int S, bool MUL, int PS>
__global__ __launch_bounds__(512) void k_backward_features(
    TileGeom g, const T *__restrict__ go, const T *__restrict__ cf,
    const T *__restrict__ sf, T *__restrict__ dx) {
    using A = typename Acc<T>::type;
    using TM = TapMap<K, D, S>;
    constexpr int KK = K * K;
    extern __shared__ __align__(16) unsigned char smem[];
    T *lds = reinterpret_cast<T *>(smem);

    const int b = logical_block(g.nblocks);
    if (b >= g.nblocks) return;
    const int cs = b % g.csplit;
    const int strip = (b / g.csplit) % g.nstrips;
    const int64_t n = b / (g.csplit * g.nstrips);
    const int qy0 = strip * g.TH;
    const int np = min(g.TH, g.rows - qy0) * g.cols;
    const int c_begin = cs * g.cpb, c_end = min(g.C, c_begin + g.cpb);
    const int64_t oplane = (int64_t)g.Ho * g.Wo, iplane = (int64_t)g.H * g.W;

    for (int i = threadIdx.x; i < g.CB * g.tile; i += g.threads) lds[i] = T(0.0f);

    int lb[PS], cy[PS], cx[PS];
    bool ok[PS];
    A sfg[PS][KK];
#pragma unroll
    for (int m = 0; m < PS; ++m) {
        const int q = threadIdx.x + m * g.threads;
        ok[m] = q < np;
        const int ql = row_of(q, g);
        cy[m] = qy0 + ql;
        cx[m] = q - ql * g.cols;
        lb[m] = ok[m] ? ql * g.P + cx[m] : 0;
#pragma unroll
        for (int i = 0; i < K; ++i)
#pragma unroll
            for (int j = 0; j < K; ++j) {
                const int sy = cy[m] + TM::dq(i), sx = cx[m] + TM::dq(j);
                const bool in = ok[m] && sy >= 0 && sy < g.Ho && sx >= 0 && sx < g.Wo;
                sfg[m][i * K + j] =
                    in ? (A)ld(sf + ((n * KK + i * K + j) * g.Ho + sy) * g.Wo + sx) : A(0);
            }
    }
    const int row0 = qy0 + g.row0_off;
    __syncthreads();

    for (int c0 = c_begin; c0 < c_end; c0 += g.CB) {
        const int ncb = min(g.CB, c_end - c0);
        stage_strips(g, lds, go + (n * g.C + c0) * oplane, oplane, ncb, row0);
        __syncthreads();
        for (int cl = 0; cl < ncb; ++cl) {
            const int64_t nc = n * g.C + c0 + cl;
            A w[KK];
#pragma unroll
            for (int t = 0; t < KK; ++t) w[t] = ld(cf + nc * KK + t);
            const T *tl = lds + cl * g.tile;
#pragma unroll
            for (int m = 0; m < PS; ++m) {
                if (!ok[m]) continue;
                A acc[S][S];
#pragma unroll
                for (int a = 0; a < S; ++a)
#pragma unroll
                    for (int c = 0; c < S; ++c) acc[a][c] = 0;
#pragma unroll
                for (int i = 0; i < K; ++i)
#pragma unroll
                    for (int j = 0; j < K; ++j) {
                        const A gv = ld(tl + lb[m] + (TM::dq(i) + TM::halo_lo) * g.P +
                                        TM::dq(j) + TM::halo_lo);
                        acc[TM::phase(i)][TM::phase(j)] +=
                            gv * comb<MUL, A>(w[i * K + j], sfg[m][i * K + j]);
                    }
                T *dst = dx + nc * iplane;
#pragma unroll
                for (int a = 0; a < S; ++a)
#pragma unroll
                    for (int c = 0; c < S; ++c) {
                        const int u = cy[m] * S + a, v = cx[m] * S + c;
                        if (u < g.H && v < g.W) st(dst + (int64_t)u * g.W + v, acc[a][c]);
                    }
            }
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------------------
// Gradients with respect to both filters.  Work cell = output pixel, owned by
// a lane (PS pixels per lane); the waves of a block take different channels.
// Per channel a lane forms gx[t] = dO * X_t once and feeds it to both sums:
//   dSF[t, pixel] += gx[t] * CF[c, t]   (register accumulator, over channels)
//   dCF[c, t]     += gx[t] * SF[t, pixel]  (butterfly over the wave's lanes)
// Partial sums over channel splits (dSF) and strips (dCF) go to the workspace
// and are added up by k_sum_partials; no atomics, so results are reproducible.
// ---------------------------------------------------------------------------
template <typename T, int K, int D, int S, bool MUL, int PS>
__global__ __launch_bounds__(512) void k_backward_filters(
    TileGeom g, const T *__restrict__ go, const T *__restrict__ x,
    const T *__restrict__ cf, const T *__restrict__ sf, T *__restrict__ dcf,
    T *__restrict__ dsf, typename Acc<T>::type *__restrict__ ws_sf,
    typename Acc<T>::type *__restrict__ ws_cf, unsigned need) {
    using A = typename Acc<T>::type;
    constexpr int KK = K * K;
    extern __shared__ __align__(16) unsigned char smem[];
    T *lds = reinterpret_cast<T *>(smem);

    const int b = logical_block(g.nblocks);
    if (b >= g.nblocks) return;
    const int cs = b % g.csplit;
    const int strip = (b / g.csplit) % g.nstrips;
    const int64_t n = b / (g.csplit * g.nstrips);
    const int y0 = strip * g.TH;
    const int np = min(g.TH, g.rows - y0) * g.cols;
    const int c_begin = cs * g.cpb, c_end = min(g.C, c_begin + g.cpb);
    const int64_t oplane = (int64_t)g.Ho * g.Wo, iplane = (int64_t)g.H * g.W;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const bool want_cf = need & DDF_NEED_DCF, want_sf = need & DDF_NEED_DSF;

    for (int i = threadIdx.x; i < g.CB * g.tile; i += g.threads) lds[i] = T(0.0f);

    int ids[KK];
#pragma unroll
    for (int t = 0; t < KK; ++t) ids[t] = t;
    const int my_tap = bfly_index<KK, 0>(ids, lane);

    int lb[PS];
    bool ok[PS];
    A sfr[PS][KK], acc_sf[PS][KK];
#pragma unroll
    for (int m = 0; m < PS; ++m) {
        const int q = lane + m * kWave;
        ok[m] = q < np;
        const int oy = row_of(q, g);
        const int ox = q - oy * g.cols;
        lb[m] = ok[m] ? (oy * S) * g.P + ox * S : 0;
        const T *sfp = sf + (n * KK * g.Ho + y0) * g.Wo + q;
#pragma unroll
        for (int t = 0; t < KK; ++t) {
            sfr[m][t] = (MUL && ok[m]) ? (A)ld(sfp + t * oplane) : A(0);
            acc_sf[m][t] = 0;
        }
    }
    const int row0 = y0 * S + g.row0_off;
    __syncthreads();

    for (int c0 = c_begin; c0 < c_end; c0 += g.CB) {
        const int ncb = min(g.CB, c_end - c0);
        stage_strips(g, lds, x + (n * g.C + c0) * iplane, iplane, ncb, row0);
        __syncthreads();
        for (int cl = wave; cl < ncb; cl += g.nwaves) {
            const int64_t nc = n * g.C + c0 + cl;
            A w[KK];
#pragma unroll
            for (int t = 0; t < KK; ++t) w[t] = MUL ? (A)ld(cf + nc * KK + t) : A(1);
            const T *tl = lds + cl * g.tile;
            const T *gp = go + (nc * g.Ho + y0) * g.Wo + lane;
            A pcf[KK];
#pragma unroll
            for (int t = 0; t < KK; ++t) pcf[t] = 0;
#pragma unroll
            for (int m = 0; m < PS; ++m) {
                if (!ok[m]) continue;
                const A gv = ld(gp + m * kWave);
#pragma unroll
                for (int i = 0; i < K; ++i)
#pragma unroll
                    for (int j = 0; j < K; ++j) {
                        const int t = i * K + j;
                        const A gx = gv * (A)ld(tl + lb[m] + i * D * g.P + j * D);
                        if (MUL) {
                            acc_sf[m][t] += gx * w[t];
                            pcf[t] += gx * sfr[m][t];
                        } else {
                            acc_sf[m][t] += gx;
                            pcf[t] += gx;
                        }
                    }
            }
            if (want_cf) {
                const A tot = bfly_sum<KK, 0, A>(pcf, lane);
                if (lane < bfly_writers<KK>()) {
                    if (g.nstrips == 1) st(dcf + nc * KK + my_tap, tot);
                    else ws_cf[(nc * g.nstrips + strip) * KK + my_tap] = tot;
                }
            }
        }
        __syncthreads();
    }

    if (!want_sf) return;
    if (g.nwaves == 1) {
#pragma unroll
        for (int m = 0; m < PS; ++m) {
            if (!ok[m]) continue;
            const int64_t pix = (int64_t)y0 * g.Wo + lane + m * kWave;
#pragma unroll
            for (int t = 0; t < KK; ++t) {
                if (g.csplit == 1) st(dsf + (n * KK + t) * oplane + pix, acc_sf[m][t]);
                else ws_sf[((n * g.csplit + cs) * KK + t) * oplane + pix] = acc_sf[m][t];
            }
        }
        return;
    }
    // Add the waves' dSF accumulators: one slot at a time through LDS.
    A *red = reinterpret_cast<A *>(smem);
#pragma unroll
    for (int m = 0; m < PS; ++m) {
#pragma unroll
        for (int t = 0; t < KK; ++t) red[(wave * KK + t) * kWave + lane] = acc_sf[m][t];
        __syncthreads();
        const int64_t pix = (int64_t)y0 * g.Wo + lane + m * kWave;
        for (int t = wave; t < KK; t += g.nwaves) {
            A tot = 0;
            for (int wv = 0; wv < g.nwaves; ++wv) tot += red[(wv * KK + t) * kWave + lane];
            if (ok[m]) {
                if (g.csplit == 1) st(dsf + (n * KK + t) * oplane + pix, tot);
                else ws_sf[((n * g.csplit + cs) * KK + t) * oplane + pix] = tot;
            }
        }
        __syncthreads();
    }
}

// out[o, i] = sum_p part[o, p, i] for o < outer, p < parts, i < inner.
template <typename T>
__global__ __launch_bounds__(256) void k_sum_partials(
    const typename Acc<T>::type *__restrict__ part, T *__restrict__ out, int64_t outer,
    int parts, int64_t inner) {
    using A = typename Acc<T>::type;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= outer * inner) return;
    const int64_t o = idx / inner, i = idx - o * inner;
    A tot = 0;
    for (int p = 0; p < parts; ++p) tot += part[(o * parts + p) * inner + i];
    st(out + idx, tot);
}

}  // namespace tiled

// Host-side geometry (ddf_tiled_host.hip).
enum TiledKind { kKindForward = 0, kKindFeatures = 1, kKindFilters = 2 };
bool tiled_geometry(const Problem &p, int dtype, int kind, TileGeom *g, int *ps);
bool tiled_shape_instantiated(int k, int d, int s);

}  // namespace ddf
