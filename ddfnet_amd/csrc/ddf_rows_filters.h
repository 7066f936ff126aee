// Row-register filter-gradient kernel for gfx950 (stride 1; 3 x 3 also with
// stride 2): dCF and dSF in one walk, same lane layout and feature-row handling
// as ddf_rows.h.
//
// The kFilterWaves waves of a workgroup work on the same strip of the same
// sample and walk consecutive channel ranges of g.cpw channels each.  Per
// channel a lane forms gx[t] = dO * X_t for its R*VX pixels once and feeds it
// to both sums:
//   dSF[t, pixel] += gx[t] * CF[c, t]      register accumulators over the walk
//   dCF[c, t]      = sum over pixels of gx[t] * SF[t, pixel]
// ('add' combine: both are sums of gx[t] itself, formed by two multiply-adds
// without the product in between.)  The per-lane dCF partials
// of kFlushChannels channels are parked in LDS, lane-contiguous per (channel,
// tap); then one lane per (channel, tap) adds up the 64 lane values with
// 16-byte reads.  That costs a quarter of the vector instructions of a
// cross-lane butterfly per channel, and the LDS pipe is otherwise idle here.
// After the walk the waves add their dSF accumulators through LDS (the only
// workgroup barriers).  Partial sums over channel splits (dSF) and strips
// (dCF) go to the workspace; no atomics, so results are reproducible.
// Reference kernels computing the same sums:
// ddf/src/cuda/ddf_mul_cuda_kernel.cu:293-355 (spatial filter), :358-420
// (channel filter).
#pragma once

#include "ddf_rows.h"

namespace ddf {
namespace rows {

constexpr int kFilterWaves = 4;
constexpr int kFlushChannels = 4;   // power of two
constexpr int kRedPitch = 68;       // accumulator values per (channel, tap) row: 64 lanes + pad, 16-byte rows
constexpr int kTapChunk = 3;        // taps per round of the final dSF sum

// LDS of one workgroup of k_rows_filters, bytes.
template <int KK>
constexpr int filters_lds_bytes(int asz, int r, int vx) {
    const int flush = kFilterWaves * kFlushChannels * KK * kRedPitch * asz;
    const int final_sum = kFilterWaves * kTapChunk * r * vx * kWave * asz;
    return flush > final_sum ? flush : final_sum;
}

#ifdef __HIPCC__

// Compiler-level ordering point between LDS writes and the reads of other
// lanes of the same wavefront.  The LDS unit executes one wave's instructions
// in order, so no hardware wait is needed.
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// DX: the same walk also produces the feature gradient (as k_rows<BWD> does):
// dO then comes in with its rows above and below as well, the lane keeps a
// second set of spatial taps (those of the pixels its dO values come from),
// and every channel ends with the store of its dX rows.  One launch for the
// whole backward pass; dO, CF and SF are read once.
// S = 2 (3 x 3, one row per lane): g describes the dO plane, the lane's feature
// vectors are 2 * VX elements wide (LaneStride2).  With DX the lane of result
// row y also writes the feature gradient of feature rows 2y and 2y + 1.
// SEG (with DX): image rows are cut into segments, whose outer lanes hold dO
// values they do not own; those are kept out of the filter sums.
template <typename T, int K, int D, bool MUL, int VX, int R, bool PAD, bool DX, int NST, int WPE,
          int S = 1, bool SEG = true>
__global__ __launch_bounds__(kWave * kFilterWaves, WPE) void k_rows_filters(
    RowsGeom g, const T *__restrict__ go, const T *__restrict__ x, const T *__restrict__ cf,
    const T *__restrict__ sf, T *__restrict__ dx, T *__restrict__ dcf, T *__restrict__ dsf,
    typename Acc<T>::type *__restrict__ ws_sf, typename Acc<T>::type *__restrict__ ws_cf,
    unsigned need, int x_mod) {
    using A = typename Acc<T>::type;
    constexpr int KK = K * K, RAD = K / 2, HX = RAD * D, HY = RAD * D;
    constexpr int ROWS = R + 2 * HY;
    // dO rows a lane loads per channel, and its own first row among them (DX:
    // the whole window; with stride 2 its own row and the next)
    constexpr int GROWS = DX ? (S == 2 ? 2 : ROWS) : R;
    constexpr int GOWN = DX && S == 1 ? HY : 0;
    constexpr bool kFilters = MUL || DX;       // CF and SF values are needed at all
    // fp16 feature gradient: comb(CF, SF) of a pixel pair is formed by one packed fp16 operation
    constexpr bool kPackedComb = sizeof(T) == 2 && DX && S == 1 && VX >= 2;
    constexpr int kVB = VX * sizeof(T), kXB = S * kVB;   // bytes of a dO / filter vector, of a feature vector
    constexpr int NW = vec_words(kVB), NWX = vec_words(kXB);
    constexpr int G = kFlushChannels;
    using Row = ExtRow<T, S * VX, HX, PAD>;
    static_assert(G * KK <= kWave, "one lane per (channel, tap) of a flush group");
    static_assert(S == 1 || (S == 2 && K == 3 && D == 1 && R == 1), "stride 2: 3 x 3, one row per lane");
    extern __shared__ __align__(16) unsigned char smem[];

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    Work wk;
    if (!wk.init(g, blockIdx.x, 0)) return;   // whole workgroup leaves together
    const bool want_cf = need & DDF_NEED_DCF, want_sf = need & DDF_NEED_DSF;
    // this wave's channels inside the workgroup's range
    const int c0 = min(wk.c_begin + wave * g.cpw, wk.c_end);
    const int nch = min(g.cpw, wk.c_end - c0);
    const int c_first = min(c0, g.C - 1);   // (pointers of a wave without channels stay inside)
    const int64_t plane = (int64_t)g.H * g.W;   // dO plane
    const uint32_t plane_bytes = (uint32_t)plane * (uint32_t)sizeof(T);
    const int64_t xplane = S == 1 ? plane : (int64_t)g.Hi * g.Wi;
    const uint32_t xplane_bytes = S == 1 ? plane_bytes : (uint32_t)xplane * (uint32_t)sizeof(T);
    std::conditional_t<S == 1, Lane<R, HY, VX>, LaneStride2<VX>> ln;
    ln.init(g, wk.strip, lane);

    // x_mod != 0: the batch is several groups of x_mod samples that share one set of
    // features (the sub-pixel branches of the up-sampling operator's gradient)
    const int64_t xn = x_mod ? wk.n % x_mod : wk.n;
    const T *xs = x + (xn * g.C + c_first) * xplane;
    const T *gs = go + (wk.n * g.C + c_first) * plane;
    T *ds = DX ? dx + (wk.n * g.C + c_first) * xplane : nullptr;
    uint32_t xb[ROWS], ob[R];
#pragma unroll
    for (int rr = 0; rr < ROWS; ++rr)
        xb[rr] = ln.xoff[rr] < 0 ? kOutside : (uint32_t)ln.xoff[rr] * (uint32_t)sizeof(T);
#pragma unroll
    for (int r = 0; r < R; ++r)
        ob[r] = ln.ooff[r] < 0 ? kOutside : (uint32_t)ln.ooff[r] * (uint32_t)sizeof(T);
    // where the lane's dO rows are
    uint32_t gb[GROWS];
    if constexpr (DX && S == 2) {
        gb[0] = ob[0];
        gb[1] = ln.onext < 0 ? kOutside : (uint32_t)ln.onext * (uint32_t)sizeof(T);
    } else {
#pragma unroll
        for (int r = 0; r < GROWS; ++r) gb[r] = DX ? xb[r] : ob[r];
    }
    const int tl = lane < KK ? lane : KK - 1;
    const T *cfs = cf + (wk.n * g.C + c_first) * KK;

    // Feature rows, dO rows and channel taps of channel ci, stage ST.  A channel
    // past the wave's last one reads zeros (empty descriptors) and so adds nothing;
    // idle lanes and rows outside the image read zeros as well.
    constexpr bool kScalarTaps = sizeof(T) >= 4;   // (see k_rows)
    uint32_t xw[NST][ROWS][NWX], gw[NST][GROWS][NW];
    T cfl[NST];
    A cfu[NST][kScalarTaps && kFilters ? KK : 1];
    auto issue = [&](auto st_tag, int ci) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value;
        const uint32_t bytes = ci < nch ? plane_bytes : 0u;
        const __amdgpu_buffer_rsrc_t pr = plane_rsrc(xs + (int64_t)ci * xplane, ci < nch ? xplane_bytes : 0u);
        const __amdgpu_buffer_rsrc_t gr = plane_rsrc(gs + (int64_t)ci * plane, bytes);
        // (with dilation the window has rows no tap lands on: see row_needed)
#pragma unroll
        for (int rr = 0; rr < ROWS; ++rr)
            if (row_needed<R, K, D>(rr)) load_vec<kXB>(pr, xb[rr], xw[ST][rr]);
#pragma unroll
        for (int r = 0; r < GROWS; ++r)
            if (!DX || S == 2 || row_needed<R, K, D>(r)) load_vec<kVB>(gr, gb[r], gw[ST][r]);
        if constexpr (kFilters) {
            const int cc = ci < nch ? ci : (nch > 0 ? nch - 1 : 0);
            if constexpr (kScalarTaps) {
#pragma unroll
                for (int t = 0; t < KK; ++t) cfu[ST][t] = cfs[(int64_t)cc * KK + t];
            } else {
                cfl[ST] = cfs[(int64_t)cc * KK + tl];
            }
        }
    };
    // Spatial taps of the lane's pixels (sfw: needed for dCF under 'mul' only) and,
    // with DX, at the pixels the lane's dO values come from: slot (i, j) of sfg
    // holds tap (K-1-i, K-1-j) of the pixel (i-RAD)*D rows and (j-RAD)*D columns
    // away, zero where that pixel does not exist (see k_rows).  Both come out of
    // the same window rows of a tap's plane, each loaded once.  (Through the
    // window offsets a lane that only reads for its neighbours holds real taps in
    // sfw as well; its dO is masked below, so they enter no sum.)
    uint32_t sfw[MUL ? R : 1][KK][NW];
    uint32_t sfg[DX ? R : 1][KK][NW];
    if constexpr (DX && S == 2) {
        // Stride 2: result pixel (y, x) reaches feature pixel (2y + i - 1, 2x + j - 1)
        // through tap (i, j).  Seen from the lane's 2 x 2 VX block of feature pixels
        // (rows 2y and 2y + 1), tap row 0 belongs to the result row below and tap
        // column 0 to the result pixel to the right: slot (i, j) holds that pixel's tap.
        using SRow = ExtRow<T, VX, 1, PAD>;
        const T *sfn = sf + wk.n * KK * plane;
#pragma unroll
        for (int i = 0; i < K; ++i)
#pragma unroll
            for (int j = 0; j < K; ++j) {
                const int t = i * K + j;
                const __amdgpu_buffer_rsrc_t sr = plane_rsrc(sfn + t * plane, plane_bytes);
                uint32_t own[NW];
                if (MUL || i > 0) load_vec<kVB>(sr, gb[0], own);
                if constexpr (MUL) {
#pragma unroll
                    for (int k = 0; k < NW; ++k) sfw[0][t][k] = own[k];
                }
                SRow row;
                if (i == 0) {
                    load_vec<kVB>(sr, gb[1], row.own);
                } else {
#pragma unroll
                    for (int k = 0; k < NW; ++k) row.own[k] = own[k];
                }
                if (j == 0) {
                    row.sides(ln.first, ln.last);
                    A v[VX];
#pragma unroll
                    for (int e = 0; e < VX; ++e) v[e] = row.at(e + 1);
                    pack<T, VX, A>(v, sfg[0][t]);
                } else {
#pragma unroll
                    for (int k = 0; k < NW; ++k) sfg[0][t][k] = row.own[k];
                }
            }
    } else if constexpr (DX) {
        const T *sfn = sf + wk.n * KK * plane;
#pragma unroll
        for (int ti = 0; ti < K; ++ti)
#pragma unroll
            for (int tj = 0; tj < K; ++tj) {
                const int t = ti * K + tj, i = K - 1 - ti, j = K - 1 - tj;
                const __amdgpu_buffer_rsrc_t sr = plane_rsrc(sfn + t * plane, plane_bytes);
                uint32_t pw[ROWS][NW];
#pragma unroll
                for (int rr = 0; rr < ROWS; ++rr) {
                    const bool for_grad = rr >= i * D && rr < i * D + R;
                    const bool for_own = MUL && rr >= HY && rr < HY + R;
                    if (for_grad || for_own) load_vec<kVB>(sr, xb[rr], pw[rr]);
                }
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    if constexpr (MUL) {
#pragma unroll
                        for (int k = 0; k < NW; ++k) sfw[r][t][k] = pw[HY + r][k];
                    }
                    Row row;
#pragma unroll
                    for (int k = 0; k < NW; ++k) row.own[k] = pw[r + i * D][k];
                    row.sides(ln.first, ln.last);
                    A v[VX];
#pragma unroll
                    for (int e = 0; e < VX; ++e) v[e] = row.at(e + j * D - HX);
                    pack<T, VX, A>(v, sfg[r][i * K + j]);
                }
            }
    } else if constexpr (MUL) {
        const T *sfn = sf + wk.n * KK * plane;
#pragma unroll
        for (int t = 0; t < KK; ++t) {
            const __amdgpu_buffer_rsrc_t sr = plane_rsrc(sfn + t * plane, plane_bytes);
#pragma unroll
            for (int r = 0; r < R; ++r) load_vec<kVB>(sr, ob[r], sfw[r][t]);
        }
    }
    // first channels of the walk; then wait for the spatial taps, which were requested
    // before them: a wait inside the walk would drain the channel pipeline every round
    static_for<0, NST - 1>([&](auto s) { issue(s, decltype(s)::value); });
    if constexpr (MUL || DX) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < KK; ++t)
#pragma unroll
                for (int k = 0; k < NW; ++k) {
                    if constexpr (MUL) asm volatile("" : "+v"(sfw[r][t][k]));
                    if constexpr (DX) asm volatile("" : "+v"(sfg[r][t][k]));
                }
    }
    A acc_sf[R][KK][VX];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < KK; ++t)
#pragma unroll
            for (int e = 0; e < VX; ++e) acc_sf[r][t][e] = 0;
    A *red = reinterpret_cast<A *>(smem) + (size_t)wave * (G * KK * kRedPitch);

    // Adds up the 64 lane partials of each (channel, tap) of a flush group of
    // `cnt` channels starting at channel `cbase` of the wave, and stores them.
    auto flush = [&](int cbase, int cnt) __attribute__((always_inline)) {
        wave_sync();
        if (lane < cnt * KK) {
            const A *rowp = red + lane * kRedPitch;
            A tot[4] = {0, 0, 0, 0};
            // (four 16-byte reads in flight at a time: more would cost registers the walk needs)
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
            // lane = slot * KK + tap: consecutive lanes are consecutive elements of dCF
            const int slot = lane / KK, tap = lane - slot * KK;
            const int64_t nc = wk.n * g.C + c0 + cbase + slot;
            if (g.nstrips == 1) st(dcf + nc * KK + tap, sum);
            else ws_cf[(nc * g.nstrips + wk.strip) * KK + tap] = sum;
        }
        wave_sync();
    };

    auto compute = [&](auto st_tag, int ci) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value;
        if constexpr (sizeof(T) == 2) {
            // keep the packed taps packed (see k_rows)
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int t = 0; t < KK; ++t)
#pragma unroll
                    for (int k = 0; k < NW; ++k) {
                        if constexpr (MUL) asm volatile("" : "+v"(sfw[r][t][k]));
                        if constexpr (DX) asm volatile("" : "+v"(sfg[r][t][k]));
                    }
        }
        Row row[ROWS];
#pragma unroll
        for (int rr = 0; rr < ROWS; ++rr) {
            if (!row_needed<R, K, D>(rr)) continue;
#pragma unroll
            for (int k = 0; k < NWX; ++k) row[rr].own[k] = xw[ST][rr][k];
            row[rr].sides(ln.first, ln.last);
        }
        // dO at the lane's own pixels.  (DX loads dO through the window offsets, so a
        // lane that only reads for its neighbours - the outer lanes of a row segment -
        // holds real values here: they must not enter the filter sums twice.  Without
        // segments every lane that owns nothing reads zeros anyway.)
        A gval[R][VX];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int e = 0; e < VX; ++e) {
                const A v = elem<T>(gw[ST][GOWN + r], e);
                gval[r][e] = (DX && SEG && ob[r] == kOutside) ? A(0) : v;
            }
        // Channel taps.  fp16: tap t comes over from lane t in storage format, as a
        // wave-uniform pair (t, t); it widens inside the mixed-precision multiply-adds.
        A w[KK];
        uint32_t wpk[kPackedComb ? KK : 1];
        if constexpr (kFilters) {
            if constexpr (kScalarTaps) {
#pragma unroll
                for (int t = 0; t < KK; ++t) w[t] = cfu[ST][t];
            } else if constexpr (kPackedComb) {
                const uint32_t bits = (uint32_t)__builtin_bit_cast(unsigned short, cfl[ST]);
#pragma unroll
                for (int t = 0; t < KK; ++t) {
                    const uint32_t b = (uint32_t)__builtin_amdgcn_readlane((int)bits, t);
                    wpk[t] = b | (b << 16);
                    w[t] = (A)__builtin_bit_cast(half2_t, wpk[t])[0];
                }
            } else {
                const A cfa = (A)ld(&cfl[ST]);
#pragma unroll
                for (int t = 0; t < KK; ++t) w[t] = lane_broadcast<A>(cfa, t);
            }
        }
        A pcf[KK];
#pragma unroll
        for (int t = 0; t < KK; ++t) pcf[t] = 0;
#pragma unroll
        for (int i = 0; i < K; ++i)
#pragma unroll
            for (int j = 0; j < K; ++j) {
                const int t = i * K + j;
#pragma unroll
                for (int r = 0; r < R; ++r)
#pragma unroll
                    for (int e = 0; e < VX; ++e) {
                        const A xv = row[r + i * D].at(S * e + j * D - HX);
                        if constexpr (MUL) {
                            // (fp16: as a multiply-add the product takes both factors in
                            // storage format; a plain multiply would widen them first)
                            const A gx = sizeof(T) == 2 ? fma_(gval[r][e], xv, A(0)) : gval[r][e] * xv;
                            acc_sf[r][t][e] = fma_(gx, w[t], acc_sf[r][t][e]);
                            pcf[t] = fma_(gx, elem<T>(sfw[r][t], e), pcf[t]);
                        } else {
                            // (two multiply-adds instead of a product and two additions)
                            acc_sf[r][t][e] = fma_(gval[r][e], xv, acc_sf[r][t][e]);
                            pcf[t] = fma_(gval[r][e], xv, pcf[t]);
                        }
                    }
                // One tap at a time, so that its products die with it (left alone, the
                // scheduler forms the products of all taps first: K*K*R*VX registers).
                // The accumulators are not read before the walk ends: without the pin the
                // compiler moves every update behind the flush branch and spills the products.
#pragma unroll
                for (int r = 0; r < R; ++r)
#pragma unroll
                    for (int e = 0; e < VX; ++e) asm volatile("" : "+v"(acc_sf[r][t][e]));
                asm volatile("" : "+v"(pcf[t]));
                __builtin_amdgcn_sched_barrier(0);
            }
        if constexpr (DX && S == 2) {
            // feature gradient of the lane's two feature rows: the four parity classes
            // of a feature pixel see one, two, two and four taps
            using GRow = ExtRow<T, VX, 1, PAD>;
            GRow g0, g1;
#pragma unroll
            for (int k = 0; k < NW; ++k) { g0.own[k] = gw[ST][0][k]; g1.own[k] = gw[ST][1][k]; }
            g0.sides(ln.first, ln.last);
            g1.sides(ln.first, ln.last);
            // dO * comb(CF[i][j], SF[i][j]) with the spatial tap of slot (i, j)
            auto term = [&](A gv, int i, int j, int e, A acc) __attribute__((always_inline)) {
                const int t = i * K + j;
                const A sv = elem<T>(sfg[0][t], e);
                if constexpr (MUL) return fma_(w[t], fma_(gv, sv, A(0)), acc);
                else return fma_(gv, sv, fma_(gv, w[t], acc));
            };
            A top[2 * VX], bot[2 * VX];
#pragma unroll
            for (int e = 0; e < VX; ++e) {
                const A g00 = g0.at(e), g01 = g0.at(e + 1), g10 = g1.at(e), g11 = g1.at(e + 1);
                top[2 * e] = term(g00, 1, 1, e, A(0));
                top[2 * e + 1] = term(g00, 1, 2, e, term(g01, 1, 0, e, A(0)));
                bot[2 * e] = term(g00, 2, 1, e, term(g10, 0, 1, e, A(0)));
                bot[2 * e + 1] = term(g00, 2, 2, e, term(g01, 2, 0, e, term(g10, 0, 2, e, term(g11, 0, 0, e, A(0)))));
            }
            const __amdgpu_buffer_rsrc_t dr = plane_rsrc(ds + (int64_t)ci * xplane, ci < nch ? xplane_bytes : 0u);
            if constexpr (sizeof(T) == 2) {
#pragma unroll
                for (int e = 0; e < 2 * VX; ++e) {
                    asm volatile("" : "+v"(top[e]));
                    asm volatile("" : "+v"(bot[e]));
                }
            }
            uint32_t ow[NWX];
            pack<T, 2 * VX, A>(top, ow);
            store_vec_nt<kXB>(dr, xb[1], ow);
            pack<T, 2 * VX, A>(bot, ow);
            store_vec_nt<kXB>(dr, xb[2], ow);
        } else if constexpr (DX) {
            // feature gradient of the lane's pixels: dO at the flipped tap offsets
            Row grow[ROWS];
#pragma unroll
            for (int rr = 0; rr < ROWS; ++rr) {
                if (!row_needed<R, K, D>(rr)) continue;
#pragma unroll
                for (int k = 0; k < NW; ++k) grow[rr].own[k] = gw[ST][rr][k];
                grow[rr].sides(ln.first, ln.last);
            }
            const __amdgpu_buffer_rsrc_t dr = plane_rsrc(ds + (int64_t)ci * plane, ci < nch ? plane_bytes : 0u);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                A accx[VX];
#pragma unroll
                for (int e = 0; e < VX; ++e) accx[e] = 0;
#pragma unroll
                for (int i = 0; i < K; ++i)
#pragma unroll
                    for (int j = 0; j < K; ++j) {
                      if constexpr (kPackedComb) {
                        // fp16: the combined filter of two pixels in one packed operation
                        // (rounded to fp16 like the operands), then one multiply-add per pixel
                        const int t = i * K + j;
                        const half2_t wv = __builtin_bit_cast(half2_t, wpk[KK - 1 - t]);
#pragma unroll
                        for (int k = 0; k < NW; ++k) {
                            const half2_t sv2 = __builtin_bit_cast(half2_t, sfg[r][t][k]);
                            const half2_t cb = MUL ? wv * sv2 : wv + sv2;
#pragma unroll
                            for (int h = 0; h < 2; ++h) {
                                const int e = 2 * k + h;
                                const A gv = grow[r + i * D].at(e + j * D - HX);
                                accx[e] = fma_(gv, (A)cb[h], accx[e]);
                            }
                        }
                      } else {
#pragma unroll
                        for (int e = 0; e < VX; ++e) {
                            const int t = i * K + j;
                            const A gv = grow[r + i * D].at(e + j * D - HX);
                            const A sv = elem<T>(sfg[r][t], e);
                            if constexpr (MUL) {
                                accx[e] = fma_(w[KK - 1 - t], fma_(gv, sv, A(0)), accx[e]);
                            } else {
                                accx[e] = fma_(gv, w[KK - 1 - t], accx[e]);
                                accx[e] = fma_(gv, sv, accx[e]);
                            }
                        }
                      }
                    }
                if constexpr (sizeof(T) == 2) {
                    // round the complete fp32 sum, the same way in every unrolled copy (see k_rows)
#pragma unroll
                    for (int e = 0; e < VX; ++e) asm volatile("" : "+v"(accx[e]));
                }
                uint32_t ow[NW];
                pack<T, VX, A>(accx, ow);
                store_vec_nt<kVB>(dr, ob[r], ow);
            }
        }
        if (want_cf && ci < nch) {
            const int slot = ci & (G - 1);
#pragma unroll
            for (int t = 0; t < KK; ++t) red[(slot * KK + t) * kRedPitch + lane] = pcf[t];
            if (slot == G - 1 || ci == nch - 1) flush(ci - slot, slot + 1);
        }
    };

    // whole rounds of NST channels (see k_rows)
    auto step = [&](auto st_tag, int ci) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value;
        // (loads first, and nothing moves between steps: see k_rows)
        issue(std::integral_constant<int, (ST + NST - 1) % NST>{}, ci + NST - 1);
        __builtin_amdgcn_sched_barrier(0);
        compute(st_tag, ci);
        __builtin_amdgcn_sched_barrier(0);
    };
    for (int ci = 0; ci < nch; ci += NST) {
        step(std::integral_constant<int, 0>{}, ci);
        if constexpr (NST > 1) step(std::integral_constant<int, 1>{}, ci + 1);
        if constexpr (NST > 2) step(std::integral_constant<int, 2>{}, ci + 2);
        if constexpr (NST > 3) step(std::integral_constant<int, 3>{}, ci + 3);
    }

    if (!want_sf) return;   // (uniform over the workgroup)
    // Add the waves' dSF accumulators: kTapChunk taps per round through LDS.
    A *all = reinterpret_cast<A *>(smem);
#pragma unroll
    for (int t0 = 0; t0 < KK; t0 += kTapChunk) {
        __syncthreads();
#pragma unroll
        for (int tt = 0; tt < kTapChunk; ++tt)
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int e = 0; e < VX; ++e) {
                    const int t = t0 + tt < KK ? t0 + tt : KK - 1;   // (past the last tap: unused filler)
                    all[(((wave * kTapChunk + tt) * R + r) * VX + e) * kWave + lane] = acc_sf[r][t][e];
                }
        __syncthreads();
        // (tap, row) pairs of this round are dealt out to the waves
        for (int idx = wave; idx < kTapChunk * R; idx += kFilterWaves) {
            const int tt = idx / R, r = idx - tt * R;
            const int t = t0 + tt;
            if (t >= KK) break;
            A tot[VX];
#pragma unroll
            for (int e = 0; e < VX; ++e) {
                tot[e] = 0;
#pragma unroll
                for (int wv = 0; wv < kFilterWaves; ++wv)
                    tot[e] += all[(((wv * kTapChunk + tt) * R + r) * VX + e) * kWave + lane];
            }
            uint32_t off_r = kOutside;   // (by run-time row index, without a register array lookup)
#pragma unroll
            for (int q = 0; q < R; ++q)
                if (q == r) off_r = ob[q];
            if (g.csplit == 1) {
                uint32_t ow[NW];
                pack<T, VX, A>(tot, ow);
                store_vec_nt<kVB>(plane_rsrc(dsf + (wk.n * KK + t) * plane, plane_bytes), off_r, ow);
            } else {
                // partial sums in the accumulator type, same plane shape
                constexpr int AW = VX * sizeof(A) / 4;
                constexpr int CH = AW < 4 ? AW : 4;
                const __amdgpu_buffer_rsrc_t wr =
                    plane_rsrc(ws_sf + ((wk.n * g.csplit + wk.cs) * KK + t) * plane,
                               (uint32_t)plane * (uint32_t)sizeof(A));
                const uint32_t off_a = off_r == kOutside ? kOutside
                                                         : off_r / (uint32_t)sizeof(T) * (uint32_t)sizeof(A);
                uint32_t aw[AW];
                pack<A, VX, A>(tot, aw);
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

// Host-side geometry of k_rows_filters (ddf_rows_host.hip): a work item is a
// workgroup of rows::kFilterWaves waves (g->wpb = 1) that covers g->cpb =
// g->cpw * rows::kFilterWaves channels; g->csplit counts those ranges.
// fused: the geometry of the launch that also writes the feature gradient.
bool rows_filters_geometry(const Problem &p, int dtype, bool fused, RowsGeom *g, int *vx, int *r);
// Workspace the kernel needs (layout as the tile kernels': dSF partials over
// channel splits, then dCF partials over strips, each 256-byte aligned).
size_t rows_filters_workspace(const Problem &p, int dtype, unsigned need);

}  // namespace ddf
