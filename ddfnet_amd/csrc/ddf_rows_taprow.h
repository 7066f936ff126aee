// Filter gradients with the tap rows dealt out to waves (gfx950, stride 1):
// same lane layout as ddf_rows.h.
//
// K consecutive work items walk the same channels of the same strip of the
// same sample; item i handles the K taps of filter row i.  For those a wave
// needs one feature row per result row only (the one (i - K/2) * D rows away),
// K spatial taps per pixel and K accumulators per pixel, so a 5 x 5 filter
// costs a wave the registers of five taps, not of twenty-five.  The waves
// share nothing: each stores the dSF planes of its own taps and parks its own
// dCF partials in its own LDS rows, which one lane per (channel, tap) then adds
// up (see ddf_rows_filters.h).  No workgroup barrier, no atomics.  A workgroup
// is g.wpb such independent waves, one per SIMD (the K of a pixel strip mostly
// share a compute unit and its L1, where they read the same dO rows).
// Partial sums over channel splits (dSF) and strips (dCF) go to the workspace.
// Reference kernels computing the same sums:
// ddf/src/cuda/ddf_mul_cuda_kernel.cu:293-355 (spatial filter), :358-420
// (channel filter).
#pragma once

#include "ddf_rows_filters.h"

namespace ddf {
namespace rows {

// Channels whose dCF partials are parked before one lane per (channel, tap of
// the wave's row) adds them up: as many as 64 lanes serve, a power of two.
template <int K>
constexpr int taprow_flush_channels() { return K <= 4 ? 16 : 8; }

constexpr int kTaprowWaves = 4;   // independent waves per workgroup

template <int K>
constexpr int taprow_lds_bytes(int asz) {
    return kTaprowWaves * taprow_flush_channels<K>() * K * kRedPitch * asz;
}

#ifdef __HIPCC__

template <typename T, int K, int D, bool MUL, int VX, int R, bool PAD, int NST, int WPE>
__global__ __launch_bounds__(kWave * kTaprowWaves, WPE) void k_rows_taprow_filters(
    RowsGeom g, const T *__restrict__ go, const T *__restrict__ x, const T *__restrict__ cf,
    const T *__restrict__ sf, T *__restrict__ dcf, T *__restrict__ dsf,
    typename Acc<T>::type *__restrict__ ws_sf, typename Acc<T>::type *__restrict__ ws_cf,
    unsigned need, int x_mod) {
    using A = typename Acc<T>::type;
    constexpr int KK = K * K, RAD = K / 2, HX = RAD * D;
    constexpr int NW = VX * sizeof(T) / 4;
    constexpr int G = taprow_flush_channels<K>();
    using Row = ExtRow<T, VX, HX, PAD>;
    static_assert(G * K <= kWave, "one lane per (channel, tap) of a flush group");
    extern __shared__ __align__(16) unsigned char smem[];

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int item = Work::item_of(g, blockIdx.x, wave);
    if (item < 0) return;
    const int trow = item % K;   // filter row of this wave
    Work wk;
    wk.decode(g, item / K);
    const bool want_cf = need & DDF_NEED_DCF, want_sf = need & DDF_NEED_DSF;
    const int c0 = wk.c_begin;
    const int nch = wk.c_end - c0;
    const int64_t plane = (int64_t)g.H * g.W;
    const uint32_t plane_bytes = (uint32_t)plane * (uint32_t)sizeof(T);
    Lane<R, 0, VX> ln;
    ln.init(g, wk.strip, lane, (trow - RAD) * D);

    const int64_t xn = x_mod ? wk.n % x_mod : wk.n;   // (see k_rows_filters)
    const T *xs = x + (xn * g.C + c0) * plane;
    const T *gs = go + (wk.n * g.C + c0) * plane;
    uint32_t xb[R], ob[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        xb[r] = ln.xoff[r] < 0 ? kOutside : (uint32_t)ln.xoff[r] * (uint32_t)sizeof(T);
        ob[r] = ln.ooff[r] < 0 ? kOutside : (uint32_t)ln.ooff[r] * (uint32_t)sizeof(T);
    }
    const int tl = lane < K ? lane : K - 1;
    const T *cfs = cf + (wk.n * g.C + c0) * KK + trow * K;   // the wave's K taps of a channel

    // Feature rows, dO rows and channel taps of channel ci, stage ST.  A channel
    // past the last one reads zeros (empty descriptors) and so adds nothing.
    constexpr bool kScalarTaps = sizeof(T) >= 4;   // (see k_rows)
    uint32_t xw[NST][R][NW], gw[NST][R][NW];
    T cfl[NST];
    A cfu[NST][kScalarTaps && MUL ? K : 1];
    // One descriptor per tensor for the whole walk: channel ci is reached through the
    // uniform offset ci * plane_bytes, the per-lane offset stays inside one plane.
    // spatial taps of the lane's pixels (needed for dCF under 'mul' only)
    uint32_t sfw[MUL ? R : 1][K][NW];
    if constexpr (MUL) {
        const T *sfn = sf + (wk.n * KK + trow * K) * plane;
#pragma unroll
        for (int j = 0; j < K; ++j) {
            const __amdgpu_buffer_rsrc_t sr = plane_rsrc(sfn + j * plane, plane_bytes);
#pragma unroll
            for (int r = 0; r < R; ++r) load_words<NW>(sr, ob[r], sfw[r][j]);
        }
    }
    // A channel past the last one gets an empty descriptor: it reads zeros and so
    // adds nothing.  (Channels are issued in order: xs and gs run ahead plane by plane.)
    auto issue = [&](auto st_tag, int ci) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value;
        const bool live = ci < nch;
        const uint32_t bytes = live ? plane_bytes : 0u;
        const __amdgpu_buffer_rsrc_t pr = plane_rsrc(xs, bytes);
        const __amdgpu_buffer_rsrc_t gr = plane_rsrc(gs, bytes);
        xs += plane;
        gs += plane;
#pragma unroll
        for (int r = 0; r < R; ++r) load_words<NW>(pr, xb[r], xw[ST][r]);
#pragma unroll
        for (int r = 0; r < R; ++r) load_words<NW>(gr, ob[r], gw[ST][r]);
        if constexpr (MUL) {
            const int cc = live ? ci : nch - 1;
            if constexpr (kScalarTaps) {
#pragma unroll
                for (int j = 0; j < K; ++j) cfu[ST][j] = cfs[(int64_t)cc * KK + j];
            } else {
                cfl[ST] = cfs[(int64_t)cc * KK + tl];
            }
        }
    };
    static_for<0, NST - 1>([&](auto s) { issue(s, decltype(s)::value); });
    if constexpr (MUL) {
        // The taps were requested before the first channels: wait for them here, not
        // inside the walk (a wait there would drain the channel pipeline every round).
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < K; ++j)
#pragma unroll
                for (int k = 0; k < NW; ++k) asm volatile("" : "+v"(sfw[r][j][k]));
    }

    A acc_sf[R][K][VX];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int j = 0; j < K; ++j)
#pragma unroll
            for (int e = 0; e < VX; ++e) acc_sf[r][j][e] = 0;
    A *red = reinterpret_cast<A *>(smem) + (size_t)wave * (G * K * kRedPitch);

    // Where the dCF sums of the walk go: the wave's channels of dCF itself, or (more
    // than one strip per plane) of the per-strip partial sums.  Lane slot * K + j
    // serves tap j of the wave's row for channel `slot` of a flush group.
    const bool cf_direct = g.nstrips == 1;
    const uint32_t cf_pitch = cf_direct ? KK * (uint32_t)sizeof(T)                   // bytes per channel
                                        : (uint32_t)g.nstrips * KK * (uint32_t)sizeof(A);
    const __amdgpu_buffer_rsrc_t cf_out =
        cf_direct ? plane_rsrc(dcf + (wk.n * g.C + c0) * KK, (uint32_t)nch * cf_pitch)
                  : plane_rsrc(ws_cf + ((wk.n * g.C + c0) * g.nstrips + wk.strip) * KK,
                               // (the last channel's row ends with this strip's taps)
                               (uint32_t)(nch - 1) * cf_pitch + KK * (uint32_t)sizeof(A));
    const int fl_slot = lane / K, fl_tap = trow * K + (lane - fl_slot * K);
    const uint32_t cf_lane = (uint32_t)fl_slot * cf_pitch +
                             (uint32_t)fl_tap * (cf_direct ? (uint32_t)sizeof(T) : (uint32_t)sizeof(A));

    // Adds up the 64 lane partials of each (channel, tap) of a flush group of
    // `cnt` channels starting at channel `cbase` of the walk, and stores them.
    auto flush = [&](int cbase, int cnt) __attribute__((always_inline)) {
        wave_sync();
        if (lane < cnt * K) {
            const A *rowp = red + lane * kRedPitch;
            A tot[4] = {0, 0, 0, 0};
#pragma nounroll
            for (int k0 = 0; k0 < kWave / 4; k0 += 4) {
                typedef A vec4 __attribute__((ext_vector_type(4)));
                vec4 v[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) v[k] = *reinterpret_cast<const vec4 *>(rowp + 4 * (k0 + k));
#pragma unroll
                for (int k = 0; k < 4; ++k)
#pragma unroll
                    for (int q = 0; q < 4; ++q) tot[q] += v[k][q];
            }
            const A sum = (tot[0] + tot[1]) + (tot[2] + tot[3]);
            if (cf_direct) store_value<T>(cf_out, cf_lane + (uint32_t)cbase * cf_pitch, sum);
            else store_value<A>(cf_out, cf_lane + (uint32_t)cbase * cf_pitch, sum);
        }
        wave_sync();
    };

    auto compute = [&](auto st_tag, auto slot_tag) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value, SLOT = decltype(slot_tag)::value;
        if constexpr (sizeof(T) == 2 && MUL) {
            // keep the packed taps packed (see k_rows)
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int j = 0; j < K; ++j)
#pragma unroll
                    for (int k = 0; k < NW; ++k) asm volatile("" : "+v"(sfw[r][j][k]));
        }
        Row row[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
#pragma unroll
            for (int k = 0; k < NW; ++k) row[r].own[k] = xw[ST][r][k];
            row[r].sides(ln.first, ln.last);
        }
        A w[K];
        if constexpr (MUL) {
            if constexpr (kScalarTaps) {
#pragma unroll
                for (int j = 0; j < K; ++j) w[j] = cfu[ST][j];
            } else {
                const A cfa = (A)ld(&cfl[ST]);
#pragma unroll
                for (int j = 0; j < K; ++j) w[j] = lane_broadcast<A>(cfa, j);
            }
        }
        A pcf[K];
#pragma unroll
        for (int j = 0; j < K; ++j) pcf[j] = 0;
#pragma unroll
        for (int j = 0; j < K; ++j)
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int e = 0; e < VX; ++e) {
                    const A gv = elem<T>(gw[ST][r], e), xv = row[r].at(e + j * D - HX);
                    if constexpr (MUL) {
                        const A gx = gv * xv;
                        acc_sf[r][j][e] = fma_(gx, w[j], acc_sf[r][j][e]);
                        pcf[j] = fma_(gx, elem<T>(sfw[r][j], e), pcf[j]);
                    } else {
                        // (two multiply-adds instead of a product and two additions)
                        acc_sf[r][j][e] = fma_(gv, xv, acc_sf[r][j][e]);
                        pcf[j] = fma_(gv, xv, pcf[j]);
                    }
                }
        // The accumulators are not read before the walk ends: without this the compiler
        // moves every update behind the flush branch and keeps (spills) the products.
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < K; ++j)
#pragma unroll
                for (int e = 0; e < VX; ++e) asm volatile("" : "+v"(acc_sf[r][j][e]));
        // (a channel past the last one parks zeros; the flush does not read them)
#pragma unroll
        for (int j = 0; j < K; ++j) red[(SLOT * K + j) * kRedPitch + lane] = pcf[j];
    };

    // Groups of G channels, G a multiple of NST: the pipeline stage and the LDS
    // slot of every step are constants.  The walk covers whole groups; channels
    // past the last one read zeros.
    static_assert(G % NST == 0, "flush groups are whole pipeline rounds");
    for (int cb = 0; cb < nch; cb += G) {
        static_for<0, G>([&](auto s) {
            constexpr int S = decltype(s)::value;
            issue(std::integral_constant<int, (S + NST - 1) % NST>{}, cb + S + NST - 1);
            compute(std::integral_constant<int, S % NST>{}, s);
            // (one step at a time: interleaving the unrolled steps costs more registers
            // than the walk has)
            __builtin_amdgcn_sched_barrier(0);
        });
        if (want_cf) flush(cb, min(G, nch - cb));
    }

    if (!want_sf) return;
#pragma unroll
    for (int j = 0; j < K; ++j) {
        const int64_t t = trow * K + j;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (g.csplit == 1) {
                uint32_t ow[NW];
                pack<T, VX, A>(acc_sf[r][j], ow);
                store_words_nt<NW>(plane_rsrc(dsf + (wk.n * KK + t) * plane, plane_bytes), ob[r], ow);
            } else {
                // partial sums in the accumulator type, same plane shape
                constexpr int AW = VX * sizeof(A) / 4;
                constexpr int CH = AW < 4 ? AW : 4;
                const __amdgpu_buffer_rsrc_t wr =
                    plane_rsrc(ws_sf + ((wk.n * g.csplit + wk.cs) * KK + t) * plane,
                               (uint32_t)plane * (uint32_t)sizeof(A));
                const uint32_t off_a = ob[r] == kOutside ? kOutside
                                                         : ob[r] / (uint32_t)sizeof(T) * (uint32_t)sizeof(A);
                uint32_t aw[AW];
                pack<A, VX, A>(acc_sf[r][j], aw);
#pragma unroll
                for (int h = 0; h < AW; h += CH) {
                    uint32_t part[CH];
#pragma unroll
                    for (int q = 0; q < CH; ++q) part[q] = aw[h + q];
                    store_words_nt<CH>(wr, off_a + h * 4, part);
                }
            }
        }
    }
}

#endif  // __HIPCC__

}  // namespace rows

// Host-side geometry of k_rows_taprow_filters (ddf_rows_host.hip): a work item
// is a wave handling one filter row of one (sample, strip, channel range);
// g->nwork counts all K of each, g->csplit the ranges of g->cpb = g->cpw channels.
bool rows_taprow_geometry(const Problem &p, int dtype, RowsGeom *g, int *vx, int *r);

}  // namespace ddf
