// Filter-gradient kernel of the DDF operator for gfx950 (wave64).
//
// A block of four waves works on a full-width row strip of one sample and a
// range of its channels.  A strip of an NCHW plane is one contiguous run in
// memory, so the global side is a linear copy: 16-byte (or 8-byte) loads of
// the X and dO strips into LDS, a few channels ahead of use.  X lands in a
// zero-bordered tile, which makes the tap loop free of bounds tests.  The
// spatial-filter taps of a lane's pixels are read once into registers and
// reused for every channel the block walks; the channel-filter taps of the
// current channel are wavefront-uniform (scalar loads).
//
// Included by one translation unit per element type.
#pragma once

#include "ddf_common.h"

namespace ddf {

// Geometry of one launch, computed on the host (ddf_tiled_host.hip).
struct TileGeom {
    int C, H, W, Ho, Wo;     // problem (per sample)
    int rows, cols;          // grid of work cells a strip is cut from
    int TH, nstrips;         // cell rows per strip
    // staged source (X, or dO for the feature gradient): zero-bordered tile
    int src_rows, src_cols;  // extent of the source plane
    int P, IH, tile;         // tile: IH rows of pitch P; `tile` elements per channel
    int row0_off, col_off;   // source row of tile row 0 in strip 0; tile column of source column 0
    // result strip staged for the store (forward, feature gradient), or the
    // dO strip of the filter gradients: linear tile
    int lin_tile;            // elements per channel reserved in LDS
    int cpb, csplit;         // channels per block; number of channel splits
    int threads;
    int vec;                 // elements per global access when alignment allows (1 = scalar)
    unsigned src_magic;      // ceil(2^32 / src_cols): e / src_cols for e < 65536; 0 when src_cols == 1
    unsigned cols_magic;     // same for q / cols
    int nblocks;             // logical blocks = N * nstrips * csplit
    int lds_bytes;
};

namespace tiled {

constexpr int kXcd = 8;
// Channels staged in LDS per barrier round.
constexpr int kCB = 8;
// Channels whose channel-filter taps are fetched together (scalar loads).
constexpr int kUC = 2;
// Waves of a filter-gradient block, and channels each owns per stage.
constexpr int kFilterWaves = 4;
constexpr int kPerWave = kCB / kFilterWaves;

template <typename T, int V>
struct alignas(sizeof(T) * V) Vec {
    T e[V];
};

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

// f / d for 0 <= f < 2^22 and d >= 1, given rcp = 1.0f / d.
__device__ __forceinline__ int div_small(int f, int d, float rcp) {
    int q = (int)((float)f * rcp);
    const int r = f - q * d;
    q += (r >= d) ? 1 : 0;
    q -= (r < 0) ? 1 : 0;
    return q;
}

// Channel-filter taps of the block's channels: read once with coalesced vector
// loads into LDS as accumulator-type values (tap_pitch<KK> per channel, 16-byte
// aligned).  The per-channel reads are then wave-uniform LDS reads that never
// wait on global memory; a scalar load per channel would be a cold miss to
// HBM on the critical path of every channel.
template <int KK>
constexpr int tap_pitch() { return (KK + 3) / 4 * 4; }

template <int KK, typename T, typename A>
__device__ __forceinline__ void stage_taps(const T *__restrict__ cf, int64_t nc0, int nch,
                                           A *taps, int threads) {
    for (int i = threadIdx.x; i < nch * KK; i += threads) {
        const int c = i / KK, t = i - c * KK;
        taps[c * tap_pitch<KK>() + t] = ld(cf + nc0 * KK + i);
    }
}

template <int KK, typename A>
__device__ __forceinline__ void load_taps(const A *taps, int ci, A (&w)[KK]) {
#pragma unroll
    for (int t = 0; t < KK; ++t) w[t] = taps[ci * tap_pitch<KK>() + t];
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
// of the value whose index g_bfly_table<N> lists for this lane.
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

// Index of the value whose total bfly_sum() leaves in `lane`: the same
// keep/send choices replayed on indices, evaluated at compile time.
constexpr int bfly_index_of(int n, int lane) {
    int id[kWave] = {};
    for (int i = 0; i < n; ++i) id[i] = i;
    int cnt = n;
    for (int stage = 0; stage < 6; ++stage) {
        const int h = cnt / 2;
        const bool up = (lane >> stage) & 1;
        int nid[kWave] = {};
        for (int j = 0; j < h; ++j) nid[j] = up ? id[j + h] : id[j];
        if (cnt & 1) nid[h] = id[2 * h];
        cnt = h + (cnt & 1);
        for (int j = 0; j < cnt; ++j) id[j] = nid[j];
    }
    return id[0];
}
template <int N>
struct BflyTable {
    int tap[kWave];
    constexpr BflyTable() : tap{} {
        for (int l = 0; l < kWave; ++l) tap[l] = bfly_index_of(N, l);
    }
};
template <int N>
__device__ const BflyTable<N> g_bfly_table{};

// Lanes below this bound hold every index at least once after the reduction.
template <int N>
constexpr int bfly_writers() {
    int w = 1;
    while (w < N) w *= 2;
    return w < kWave ? w : kWave;
}

// Block -> (sample, strip, channel range), shared by the three kernels.
struct BlockWork {
    int cs, strip, row_first, nrows, np, c_begin, c_end;
    int64_t n;
    __device__ __forceinline__ bool init(const TileGeom &g) {
        const int b = logical_block(g.nblocks);
        if (b >= g.nblocks) return false;
        cs = b % g.csplit;
        const int rest = b / g.csplit;
        strip = rest % g.nstrips;
        n = rest / g.nstrips;
        row_first = strip * g.TH;
        nrows = min(g.TH, g.rows - row_first);
        np = nrows * g.cols;
        c_begin = cs * g.cpb;
        c_end = min(g.C, c_begin + g.cpb);
        return true;
    }
};

// Moves the strips of up to kCB consecutive planes from global memory to LDS
// by way of registers, V elements per access.  The strips of one stage are
// numbered as one flat list of vectors (channel-major); a thread owns vectors
// f = tid, tid + threads, ...  The first NS of them are prefetched: issue()
// starts their loads without waiting, commit() writes them to LDS later and
// moves any further vectors straight through.  Issuing stage s+1 before
// computing on stage s overlaps the fetch with the arithmetic.
//
// The destination is either a zero-bordered tile (PADDED: row pitch P, column
// offset col_off, first staged row at tile row row_shift) or a linear copy of
// the run.  Requires src_cols >= V for PADDED (one row crossing per vector).
template <typename T, int V, int NS, bool PADDED>
struct Stager {
    int nvec, run0, row_shift, dst_tile, src_cols, P, col_off, threads;
    unsigned src_magic;
    float rcp_nvec;
    int cl[NS], eoff[NS], lo[NS], col[NS];
    Vec<T, V> v[NS];

    __device__ __forceinline__ void locate(int f, int &c, int &eo, int &l, int &cc) const {
        c = div_small(f, nvec, rcp_nvec);
        const int e = (f - c * nvec) * V;
        eo = run0 + e;
        if (PADDED) {
            const int row = src_magic ? (int)__umulhi((unsigned)e, src_magic) : e;
            cc = e - row * src_cols;
            l = c * dst_tile + (row_shift + row) * P + col_off + cc;
        } else {
            cc = 0;
            l = c * dst_tile + e;
        }
    }
    // n_elems elements per channel starting at element run_start of each plane.
    __device__ __forceinline__ void init(int n_elems, int run_start, int row_shift_, int dst_tile_,
                                         int src_cols_, int P_, int col_off_, unsigned magic,
                                         int threads_) {
        nvec = n_elems / V;
        run0 = run_start;
        row_shift = row_shift_;
        dst_tile = dst_tile_;
        src_cols = src_cols_;
        P = P_;
        col_off = col_off_;
        src_magic = magic;
        threads = threads_;
        rcp_nvec = 1.0f / (float)max(nvec, 1);
#pragma unroll
        for (int j = 0; j < NS; ++j)
            locate(threadIdx.x + j * threads, cl[j], eoff[j], lo[j], col[j]);
    }
    __device__ __forceinline__ void put(T *lds, int l, int cc, const Vec<T, V> &val) const {
        if (!PADDED) {
            *reinterpret_cast<Vec<T, V> *>(lds + l) = val;
        } else {
#pragma unroll
            for (int k = 0; k < V; ++k)
                lds[l + k + ((cc + k >= src_cols) ? P - src_cols : 0)] = val.e[k];
        }
    }
    __device__ __forceinline__ void issue(const T *__restrict__ src, int64_t plane, int ncb) {
#pragma unroll
        for (int j = 0; j < NS; ++j)
            if (cl[j] < ncb)
                v[j] = *reinterpret_cast<const Vec<T, V> *>(src + cl[j] * plane + eoff[j]);
    }
    // `src`, `plane`, `ncb` as given to the matching issue().
    __device__ __forceinline__ void commit(T *lds, const T *__restrict__ src, int64_t plane,
                                           int ncb) const {
#pragma unroll
        for (int j = 0; j < NS; ++j)
            if (cl[j] < ncb) put(lds, lo[j], col[j], v[j]);
        const int total = ncb * nvec;
        for (int f = threadIdx.x + NS * threads; f < total; f += threads) {
            int c, eo, l, cc;
            locate(f, c, eo, l, cc);
            put(lds, l, cc, *reinterpret_cast<const Vec<T, V> *>(src + c * plane + eo));
        }
    }
};

// Prefetch depth: 16-byte accesses keep 3 vectors in flight per thread,
// 8-byte ones 4, scalar ones 8.
template <typename T, int V>
constexpr int stager_slots() {
    return sizeof(T) * V >= 16 ? 3 : (V > 1 ? 4 : 8);
}

template <typename T>
__device__ __forceinline__ void zero_tiles(const TileGeom &g, T *lds) {
    for (int i = threadIdx.x; i < kCB * g.tile; i += g.threads) lds[i] = T(0.0f);
}

// First staged source row, clipped, and how many rows of the strip exist.
__device__ __forceinline__ void clip_rows(const TileGeom &g, int row0, int &r_lo, int &n_rows) {
    r_lo = max(row0, 0);
    n_rows = max(min(row0 + g.IH, g.src_rows) - r_lo, 0);
}

// ---------------------------------------------------------------------------
// Gradients with respect to both filters.  Work cell = output pixel, owned by
// a lane (PS pixels per lane); the four waves of a block take different
// channels.  Per channel a lane forms gx[t] = dO * X_t once and feeds it to
// both sums:
//   dSF[t, pixel] += gx[t] * CF[c, t]   (register accumulator, over channels)
//   dCF[c, t]     += gx[t] * SF[t, pixel]  (butterfly over the wave's lanes)
// Partial sums over channel splits (dSF) and strips (dCF) go to the workspace
// and are added up by k_sum_partials; no atomics, so results are reproducible.
// LDS: kCB zero-bordered X tiles, then kCB linear dO strips.
// ---------------------------------------------------------------------------
template <typename T, int K, int D, int S, bool MUL, int PS, int V>
__global__ __launch_bounds__(kWave * kFilterWaves) void k_backward_filters(
    TileGeom g, const T *__restrict__ go, const T *__restrict__ x,
    const T *__restrict__ cf, const T *__restrict__ sf, T *__restrict__ dcf,
    T *__restrict__ dsf, typename Acc<T>::type *__restrict__ ws_sf,
    typename Acc<T>::type *__restrict__ ws_cf, unsigned need) {
    using A = typename Acc<T>::type;
    constexpr int KK = K * K;
    extern __shared__ __align__(16) unsigned char smem[];
    T *lds_in = reinterpret_cast<T *>(smem);
    T *lds_go = lds_in + kCB * g.tile;
    A *taps = reinterpret_cast<A *>(lds_go + kCB * g.lin_tile);

    BlockWork bw;
    if (!bw.init(g)) return;
    const int64_t oplane = (int64_t)g.Ho * g.Wo, iplane = (int64_t)g.H * g.W;
    const int y0 = bw.row_first;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const bool want_cf = need & DDF_NEED_DCF, want_sf = need & DDF_NEED_DSF;
    const int my_tap = g_bfly_table<KK>.tap[lane];

    int lb[PS];
    bool ok[PS];
    A sfr[PS][KK], acc_sf[PS][KK];
#pragma unroll
    for (int m = 0; m < PS; ++m) {
        const int q = lane + m * kWave;
        ok[m] = q < bw.np;
        const int oy = row_of(q, g);
        const int ox = q - oy * g.cols;
        lb[m] = ok[m] ? (oy * S) * g.P + ox * S : 0;
        const T *sfp = sf + (bw.n * KK * g.Ho + y0) * g.Wo + q;
#pragma unroll
        for (int t = 0; t < KK; ++t) {
            sfr[m][t] = (MUL && ok[m]) ? (A)ld(sfp + t * oplane) : A(0);
            acc_sf[m][t] = 0;
        }
    }

    int r_lo, n_rows;
    clip_rows(g, y0 * S + g.row0_off, r_lo, n_rows);
    Stager<T, V, stager_slots<T, V>(), true> stg;
    stg.init(n_rows * g.src_cols, r_lo * g.src_cols, r_lo - (y0 * S + g.row0_off), g.tile,
             g.src_cols, g.P, g.col_off, g.src_magic, g.threads);
    Stager<T, V, (stager_slots<T, V>() + 1) / 2, false> stg_go;
    stg_go.init(bw.np, y0 * g.Wo, 0, g.lin_tile, g.Wo, g.Wo, 0, 0u, g.threads);
    const T *xs = x + (bw.n * g.C + bw.c_begin) * iplane;
    const T *gs = go + (bw.n * g.C + bw.c_begin) * oplane;
    {
        const int ncb = min(kCB, bw.c_end - bw.c_begin);
        stg.issue(xs, iplane, ncb);
        stg_go.issue(gs, oplane, ncb);
    }
    if (MUL) stage_taps<KK>(cf, bw.n * g.C + bw.c_begin, bw.c_end - bw.c_begin, taps, g.threads);
    zero_tiles(g, lds_in);
    __syncthreads();

    for (int c0 = bw.c_begin; c0 < bw.c_end; c0 += kCB, xs += kCB * iplane, gs += kCB * oplane) {
        const int ncb = min(kCB, bw.c_end - c0);
        stg.commit(lds_in, xs, iplane, ncb);
        stg_go.commit(lds_go, gs, oplane, ncb);
        __syncthreads();
        if (c0 + kCB < bw.c_end) {
            const int nnext = min(kCB, bw.c_end - c0 - kCB);
            stg.issue(xs + kCB * iplane, iplane, nnext);
            stg_go.issue(gs + kCB * oplane, oplane, nnext);
        }
#pragma unroll
        for (int u = 0; u < kPerWave; ++u) {
            const int cl = wave + u * kFilterWaves;
            if (cl >= ncb) break;
            const int64_t nc = bw.n * g.C + c0 + cl;
            A w[KK];
            if (MUL) load_taps<KK>(taps, c0 - bw.c_begin + cl, w);
            const T *tl = lds_in + cl * g.tile;
            const T *gl = lds_go + cl * g.lin_tile + lane;
            A pcf[KK];
#pragma unroll
            for (int t = 0; t < KK; ++t) pcf[t] = 0;
#pragma unroll
            for (int m = 0; m < PS; ++m) {
                if (!ok[m]) continue;
                const A gval = ld(gl + m * kWave);
#pragma unroll
                for (int i = 0; i < K; ++i)
#pragma unroll
                    for (int j = 0; j < K; ++j) {
                        const int t = i * K + j;
                        const A gx = gval * (A)ld(tl + lb[m] + i * D * g.P + j * D);
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
                    else ws_cf[(nc * g.nstrips + bw.strip) * KK + my_tap] = tot;
                }
            }
        }
        __syncthreads();
    }

    if (!want_sf) return;
    // Add the four waves' dSF accumulators: one pixel slot at a time through LDS.
    A *red = reinterpret_cast<A *>(smem);
#pragma unroll
    for (int m = 0; m < PS; ++m) {
#pragma unroll
        for (int t = 0; t < KK; ++t) red[(wave * KK + t) * kWave + lane] = acc_sf[m][t];
        __syncthreads();
        const int64_t pix = (int64_t)y0 * g.Wo + lane + m * kWave;
        for (int t = wave; t < KK; t += kFilterWaves) {
            A tot = 0;
#pragma unroll
            for (int wv = 0; wv < kFilterWaves; ++wv) tot += red[(wv * KK + t) * kWave + lane];
            if (ok[m]) {
                if (g.csplit == 1) st(dsf + (bw.n * KK + t) * oplane + pix, tot);
                else ws_sf[((bw.n * g.csplit + bw.cs) * KK + t) * oplane + pix] = tot;
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
enum TiledKind { kKindFilters = 2 };
bool tiled_geometry(const Problem &p, int dtype, int kind, TileGeom *g, int *ps);
bool tiled_shape_instantiated(int k, int d, int s);

}  // namespace ddf
