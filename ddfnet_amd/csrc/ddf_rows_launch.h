// Launch code of the row-register kernels, instantiated once per element type.
#pragma once

#include <algorithm>

#include "ddf_rows_taprow.h"
#include "ddf_wave.h"

namespace ddf {
namespace rows {

constexpr int kStages = 3;   // channels in flight per wave (one computed, two loading)
// waves per SIMD the registers are budgeted for (fp16 with 16 pixels per lane needs the room)
template <typename T, int K, int VX, int R>
constexpr int waves_per_simd() {
    if (K == 5) return 2;   // 25 taps of 4 or 8 pixels in registers
    return sizeof(T) == 2 && VX * R >= 16 ? 2 : 3;
}
template <int K>
constexpr int stages() { return K == 5 ? 2 : kStages; }

template <typename T, int K, int D, int VX, int R>
hipError_t launch_kdv(const Problem &p, const RowsGeom &g, bool backward, const T *x, const T *cf,
                      const T *sf, T *out, hipStream_t st) {
    const dim3 grid(g.xcd_per * kXcd), block(kWave * g.wpb);
    const bool pad = rows_shift_in_as_is(g);
#define DDF_ROWS_CASE(MUL_, BWD_)                                                               \
    do {                                                                                        \
        if (pad)                                                                                \
            hipLaunchKernelGGL((k_rows<T, K, D, MUL_, BWD_, VX, R, true, stages<K>(),           \
                                       waves_per_simd<T, K, VX, R>()>),                         \
                               grid, block, 0, st, g, x, cf, sf, out);                          \
        else                                                                                    \
            hipLaunchKernelGGL((k_rows<T, K, D, MUL_, BWD_, VX, R, false, stages<K>(),          \
                                       waves_per_simd<T, K, VX, R>()>),                         \
                               grid, block, 0, st, g, x, cf, sf, out);                          \
    } while (0)
    if (p.mul) {
        if (backward) DDF_ROWS_CASE(true, true);
        else DDF_ROWS_CASE(true, false);
    } else {
        if (backward) DDF_ROWS_CASE(false, true);
        else DDF_ROWS_CASE(false, false);
    }
#undef DDF_ROWS_CASE
    return hipGetLastError();
}

// Stride 2: forward, or (BWD: x is dO, out is dX, even feature heights) the feature gradient.
template <typename T, int VX, bool BWD>
hipError_t launch_stride2_v(const Problem &p, const RowsGeom &g, const T *x, const T *cf,
                            const T *sf, T *out, hipStream_t st) {
    const dim3 grid(g.xcd_per * kXcd), block(kWave * g.wpb);
    const bool pad = rows_shift_in_as_is(g);
    constexpr int kWpe = sizeof(T) == 2 && VX >= 8 ? 2 : 3;
#define DDF_ROWS_CASE(MUL_, PAD_)                                                               \
    hipLaunchKernelGGL((k_rows<T, 3, 1, MUL_, BWD, VX, 1, PAD_, kStages, kWpe, 2>), grid,       \
                       block, 0, st, g, x, cf, sf, out)
    if (p.mul) {
        if (pad) DDF_ROWS_CASE(true, true);
        else DDF_ROWS_CASE(true, false);
    } else {
        if (pad) DDF_ROWS_CASE(false, true);
        else DDF_ROWS_CASE(false, false);
    }
#undef DDF_ROWS_CASE
    return hipGetLastError();
}

template <typename T, int VX, int R>
hipError_t launch_v(const Problem &p, const RowsGeom &g, bool backward, const T *x, const T *cf,
                    const T *sf, T *out, hipStream_t st) {
    if (p.k == 3 && p.d == 1) return launch_kdv<T, 3, 1, VX, R>(p, g, backward, x, cf, sf, out, st);
    if constexpr (VX >= 2 && VX * (int)sizeof(T) * R < 32) {   // (16-byte vectors, two rows: 3x3 d1 only)
        if (p.k == 3 && p.d == 2)
            return launch_kdv<T, 3, 2, VX, R>(p, g, backward, x, cf, sf, out, st);
    }
    // 25 taps: one row per lane, vectors of four pixels or more (the taps reach
    // two, with dilation four, pixels into the neighbouring lane)
    if constexpr (R == 1 && VX >= 4) {
        if (p.k == 5 && p.d == 1) return launch_kdv<T, 5, 1, VX, R>(p, g, backward, x, cf, sf, out, st);
        if (p.k == 5 && p.d == 2) return launch_kdv<T, 5, 2, VX, R>(p, g, backward, x, cf, sf, out, st);
    }
    return hipErrorNotSupported;
}

}  // namespace rows

// Forward (backward = false: x -> out) or feature gradient (backward = true:
// dO -> dX) on the row-register kernels.  hipErrorNotSupported: not covered
// (shape, or pointers not aligned to the vector the geometry wants); nothing
// was launched then.
template <typename T>
hipError_t rows_launch(const Problem &p, bool backward, const T *x, const T *cf, const T *sf,
                       T *out, hipStream_t st) {
    const int dtype = sizeof(T) == 2 ? DDF_F16 : sizeof(T) == 4 ? DDF_F32 : DDF_F64;
    RowsGeom g;
    int vx, r;
    if (!rows_geometry(p, dtype, 0, &g, &vx, &r)) return hipErrorNotSupported;
    const uintptr_t mask = (uintptr_t)(vx * sizeof(T)) - 1;
    if ((((uintptr_t)x | (uintptr_t)sf | (uintptr_t)out) & mask) != 0) return hipErrorNotSupported;
    if (p.s == 2) {
        // (feature vectors are twice as long and come in pieces of at most 16 bytes; the
        // feature gradient writes rows 2y and 2y + 1 per result row: even heights)
        const T *feat = backward ? out : x;
        if (((uintptr_t)feat & (std::min<uintptr_t>(2 * vx * sizeof(T), 16) - 1)) != 0)
            return hipErrorNotSupported;
        if (backward && !rows_stride2_feature_gradient(p)) return hipErrorNotSupported;
#define DDF_S2_CASE(VX_)                                                                       \
    return backward ? rows::launch_stride2_v<T, VX_, true>(p, g, x, cf, sf, out, st)           \
                    : rows::launch_stride2_v<T, VX_, false>(p, g, x, cf, sf, out, st)
        // (feature vectors of 16 bytes at most: vx <= 4 for fp16, 2 for fp32)
        if constexpr (sizeof(T) == 2) {
            if (vx == 4) DDF_S2_CASE(4);
        }
        if constexpr (sizeof(T) != 8) {
            if (vx == 1) DDF_S2_CASE(1);
            if (vx == 2) DDF_S2_CASE(2);
        }
#undef DDF_S2_CASE
        return hipErrorNotSupported;
    }
    if constexpr (sizeof(T) == 2) {
        if (vx == 8 && r == 1) return rows::launch_v<T, 8, 1>(p, g, backward, x, cf, sf, out, st);
        if (vx == 4 && r == 1) return rows::launch_v<T, 4, 1>(p, g, backward, x, cf, sf, out, st);
        if (vx == 2 && r == 1) return rows::launch_v<T, 2, 1>(p, g, backward, x, cf, sf, out, st);
        if (vx == 1 && r == 1) return rows::launch_v<T, 1, 1>(p, g, backward, x, cf, sf, out, st);
        if (vx == 8 && r == 2) return rows::launch_v<T, 8, 2>(p, g, backward, x, cf, sf, out, st);
        if (vx == 4 && r == 2) return rows::launch_v<T, 4, 2>(p, g, backward, x, cf, sf, out, st);
        if (vx == 2 && r == 2) return rows::launch_v<T, 2, 2>(p, g, backward, x, cf, sf, out, st);
    } else if constexpr (sizeof(T) == 4) {
        if (vx == 4 && r == 2) return rows::launch_v<T, 4, 2>(p, g, backward, x, cf, sf, out, st);
        if (vx == 2 && r == 1) return rows::launch_v<T, 2, 1>(p, g, backward, x, cf, sf, out, st);
        if (vx == 4 && r == 1) return rows::launch_v<T, 4, 1>(p, g, backward, x, cf, sf, out, st);
        if (vx == 2 && r == 2) return rows::launch_v<T, 2, 2>(p, g, backward, x, cf, sf, out, st);
        if (vx == 1 && r == 1) return rows::launch_v<T, 1, 1>(p, g, backward, x, cf, sf, out, st);
    }
    return hipErrorNotSupported;
}

namespace rows {

template <typename T, int VX, int R, bool DX>
hipError_t launch_filters_v(const Problem &p, const RowsGeom &g, const T *go, const T *x,
                            const T *cf, const T *sf, T *dx, T *dcf, T *dsf,
                            typename Acc<T>::type *ws_sf, typename Acc<T>::type *ws_cf,
                            unsigned need, int x_mod, hipStream_t st) {
    using A = typename Acc<T>::type;
    // waves per SIMD the registers are budgeted for: 'mul' keeps the spatial taps
    // as well, the fused feature gradient a second set of them
    constexpr int WPE_MUL = (DX || VX * R >= 4) ? 2 : 3, WPE_ADD = DX ? 2 : 3;
    // channels in flight per wave, a divisor of kFlushChannels (whole rounds)
    constexpr int kFilterStages = DX ? 2 : 4;
    const dim3 grid(g.xcd_per * kXcd), block(kWave * kFilterWaves);
    const int lds = filters_lds_bytes<9>((int)sizeof(A), R, VX);
    if (p.k != 3 || (p.d != 1 && p.d != 2)) return hipErrorNotSupported;
    const bool pad = rows_shift_in_as_is(g);
    // (row segments: only the launch that also writes the feature gradient tells them apart)
    const bool seg = DX && g.segs > 0;
#define DDF_ROWSF_CASE(D_, MUL_, PAD_, SEG_)                                                     \
    hipLaunchKernelGGL((k_rows_filters<T, 3, D_, MUL_, VX, R, PAD_, DX, kFilterStages,           \
                                       MUL_ ? WPE_MUL : WPE_ADD, 1, SEG_>),                      \
                       grid, block, lds, st, g, go, x, cf, sf, dx, dcf, dsf, ws_sf, ws_cf, need, x_mod)
#define DDF_ROWSF_D(D_)                                                                          \
    if (p.mul) {                                                                                 \
        if (seg) DDF_ROWSF_CASE(D_, true, true, true);                                           \
        else if (pad) DDF_ROWSF_CASE(D_, true, true, false);                                     \
        else DDF_ROWSF_CASE(D_, true, false, false);                                             \
    } else {                                                                                     \
        if (seg) DDF_ROWSF_CASE(D_, false, true, true);                                          \
        else if (pad) DDF_ROWSF_CASE(D_, false, true, false);                                    \
        else DDF_ROWSF_CASE(D_, false, false, false);                                            \
    }
    if (p.d == 1) {
        DDF_ROWSF_D(1)
    } else {
        // (dilation 2: the taps reach two pixels into the neighbouring lane; one row per lane)
        if constexpr (VX >= 2 && R == 1) { DDF_ROWSF_D(2) } else { return hipErrorNotSupported; }
    }
#undef DDF_ROWSF_D
#undef DDF_ROWSF_CASE
    return hipGetLastError();
}

// Stride 2: filter gradients and, with DX, the feature gradient in the same launch.
template <typename T, int VX, bool DX>
hipError_t launch_filters_stride2_v(const Problem &p, const RowsGeom &g, const T *go, const T *x,
                                    const T *cf, const T *sf, T *dx, T *dcf, T *dsf,
                                    typename Acc<T>::type *ws_sf, typename Acc<T>::type *ws_cf,
                                    unsigned need, hipStream_t st) {
    using A = typename Acc<T>::type;
    // (channels in flight per wave: 32-byte feature vectors of fp16 leave room for two,
    // and so does the second set of spatial taps of the feature gradient)
    constexpr int kStagesS2 = DX || (sizeof(T) == 2 && VX >= 8) ? 2 : 4, kWpe = 2;
    const dim3 grid(g.xcd_per * kXcd), block(kWave * kFilterWaves);
    const int lds = filters_lds_bytes<9>((int)sizeof(A), 1, VX);
    const bool pad = rows_shift_in_as_is(g);
#define DDF_ROWSF_CASE(MUL_, PAD_)                                                               \
    hipLaunchKernelGGL((k_rows_filters<T, 3, 1, MUL_, VX, 1, PAD_, DX, kStagesS2, kWpe, 2, false>), \
                       grid, block, lds, st, g, go, x, cf, sf, dx, dcf, dsf, ws_sf, ws_cf, need, 0)
    if (p.mul) {
        if (pad) DDF_ROWSF_CASE(true, true);
        else DDF_ROWSF_CASE(true, false);
    } else {
        if (pad) DDF_ROWSF_CASE(false, true);
        else DDF_ROWSF_CASE(false, false);
    }
#undef DDF_ROWSF_CASE
    return hipGetLastError();
}

template <typename T, int K, int D, int VX>
hipError_t launch_taprow_kdv(const Problem &p, const RowsGeom &g, const T *go, const T *x,
                             const T *cf, const T *sf, T *dcf, T *dsf,
                             typename Acc<T>::type *ws_sf, typename Acc<T>::type *ws_cf,
                             unsigned need, int x_mod, hipStream_t st) {
    using A = typename Acc<T>::type;
    constexpr int kTaprowStages = 8, kWpe = 3;   // channels in flight per wave; waves per SIMD
    const dim3 grid(g.xcd_per * kXcd), block(kWave * kTaprowWaves);
    const int lds = taprow_lds_bytes<K>((int)sizeof(A));
    const bool pad = rows_shift_in_as_is(g);
#define DDF_TAPROW_CASE(MUL_, PAD_)                                                              \
    hipLaunchKernelGGL((k_rows_taprow_filters<T, K, D, MUL_, VX, 1, PAD_, kTaprowStages, kWpe>), \
                       grid, block, lds, st, g, go, x, cf, sf, dcf, dsf, ws_sf, ws_cf, need, x_mod)
    if (p.mul) {
        if (pad) DDF_TAPROW_CASE(true, true);
        else DDF_TAPROW_CASE(true, false);
    } else {
        if (pad) DDF_TAPROW_CASE(false, true);
        else DDF_TAPROW_CASE(false, false);
    }
#undef DDF_TAPROW_CASE
    return hipGetLastError();
}

template <typename T, int VX>
hipError_t launch_taprow_v(const Problem &p, const RowsGeom &g, const T *go, const T *x,
                           const T *cf, const T *sf, T *dcf, T *dsf,
                           typename Acc<T>::type *ws_sf, typename Acc<T>::type *ws_cf,
                           unsigned need, int x_mod, hipStream_t st) {
    if (p.k == 3 && p.d == 1)
        return launch_taprow_kdv<T, 3, 1, VX>(p, g, go, x, cf, sf, dcf, dsf, ws_sf, ws_cf, need, x_mod, st);
    if (p.k == 5 && p.d == 1)
        return launch_taprow_kdv<T, 5, 1, VX>(p, g, go, x, cf, sf, dcf, dsf, ws_sf, ws_cf, need, x_mod, st);
    if constexpr (VX >= 4) {
        if (p.k == 5 && p.d == 2)
            return launch_taprow_kdv<T, 5, 2, VX>(p, g, go, x, cf, sf, dcf, dsf, ws_sf, ws_cf, need, x_mod, st);
    }
    return hipErrorNotSupported;
}

}  // namespace rows

// Filter gradients on the row-register kernel, partial sums included; with
// dx != nullptr the same launch also writes the feature gradient
// (rows_filters_geometry(..., fused = true) must cover the problem).
// hipErrorNotSupported: not covered (nothing was launched).  `ws` must hold
// rows_filters_workspace() bytes.
template <typename T>
hipError_t rows_filters_launch(const Problem &p, const T *go, const T *x, const T *cf, const T *sf,
                               T *dx, T *dcf, T *dsf, void *ws, unsigned need, hipStream_t st,
                               int x_mod, NormTail<T> *norm) {
    using A = typename Acc<T>::type;
    const int dtype = sizeof(T) == 2 ? DDF_F16 : sizeof(T) == 4 ? DDF_F32 : DDF_F64;
    const bool fused = dx != nullptr;
    RowsGeom g;
    int vx, r;
    // (5 x 5: the tap rows go to the waves of a workgroup)
    const bool taprow = !fused && rows_taprow_geometry(p, dtype, &g, &vx, &r);
    if (!taprow && !rows_filters_geometry(p, dtype, fused, &g, &vx, &r)) return hipErrorNotSupported;
    const uintptr_t mask = (uintptr_t)(vx * sizeof(T)) - 1;
    if ((((uintptr_t)x | (uintptr_t)go | (uintptr_t)sf | (uintptr_t)dsf | (uintptr_t)dx) & mask) != 0)
        return hipErrorNotSupported;
    if (p.s == 2 && (x_mod != 0 || (((uintptr_t)x | (uintptr_t)dx) &
                                    (std::min<uintptr_t>(2 * vx * sizeof(T), 16) - 1)) != 0))
        return hipErrorNotSupported;
    unsigned char *wp = static_cast<unsigned char *>(ws);
    A *ws_sf = nullptr, *ws_cf = nullptr;
    const int64_t n_sf = p.N * p.kk * p.Ho * p.Wo;
    if ((need & DDF_NEED_DSF) && g.csplit > 1) {
        ws_sf = reinterpret_cast<A *>(wp);
        wp += ((size_t)n_sf * g.csplit * sizeof(A) + 255) / 256 * 256;
    }
    if ((need & DDF_NEED_DCF) && g.nstrips > 1) ws_cf = reinterpret_cast<A *>(wp);
    hipError_t err = hipErrorNotSupported;
    if constexpr (sizeof(T) != 8) {
        if (p.s == 2) {
#define DDF_S2_CASE(VX_)                                                                          \
    err = fused ? rows::launch_filters_stride2_v<T, VX_, true>(p, g, go, x, cf, sf, dx, dcf, dsf, \
                                                               ws_sf, ws_cf, need, st)            \
                : rows::launch_filters_stride2_v<T, VX_, false>(p, g, go, x, cf, sf, dx, dcf, dsf, \
                                                                ws_sf, ws_cf, need, st)
            if (vx == 2) DDF_S2_CASE(2);
            else if (vx == 1) DDF_S2_CASE(1);
            if constexpr (sizeof(T) == 2) {
                if (vx == 4) DDF_S2_CASE(4);
            }
#undef DDF_S2_CASE
        } else if (taprow) {
            if (vx == 4)
                err = rows::launch_taprow_v<T, 4>(p, g, go, x, cf, sf, dcf, dsf, ws_sf, ws_cf, need, x_mod, st);
            else if (vx == 2)
                err = rows::launch_taprow_v<T, 2>(p, g, go, x, cf, sf, dcf, dsf, ws_sf, ws_cf, need, x_mod, st);
            if constexpr (sizeof(T) == 2) {
                if (vx == 8)
                    err = rows::launch_taprow_v<T, 8>(p, g, go, x, cf, sf, dcf, dsf, ws_sf, ws_cf, need, x_mod, st);
            }
        } else if (vx == 1) {
            if (fused)
                err = rows::launch_filters_v<T, 1, 1, true>(p, g, go, x, cf, sf, dx, dcf, dsf, ws_sf, ws_cf, need, x_mod, st);
            else
                err = rows::launch_filters_v<T, 1, 1, false>(p, g, go, x, cf, sf, dx, dcf, dsf, ws_sf, ws_cf, need, x_mod, st);
        } else if (fused) {
            if (vx == 2 && r == 2)
                err = rows::launch_filters_v<T, 2, 2, true>(p, g, go, x, cf, sf, dx, dcf, dsf, ws_sf, ws_cf, need, x_mod, st);
            else if (vx == 4 && r == 1)
                err = rows::launch_filters_v<T, 4, 1, true>(p, g, go, x, cf, sf, dx, dcf, dsf, ws_sf, ws_cf, need, x_mod, st);
        } else {
            if (vx == 4 && r == 1)
                err = rows::launch_filters_v<T, 4, 1, false>(p, g, go, x, cf, sf, dx, dcf, dsf, ws_sf, ws_cf, need, x_mod, st);
            else if (vx == 2 && r == 1)
                err = rows::launch_filters_v<T, 2, 1, false>(p, g, go, x, cf, sf, dx, dcf, dsf, ws_sf, ws_cf, need, x_mod, st);
        }
    }
    if (err != hipSuccess) return err;
    return wave::sum_filter_partials<T>(ws_sf, dsf, p.N, g.csplit, p.kk * p.Ho * p.Wo, ws_cf, dcf,
                                        p.N * p.C, g.nstrips, (int64_t)p.kk, st,
                                        (need & DDF_NEED_DSF) ? norm : nullptr);
}

template <typename T>
hipError_t rows_backward_shared_features(const Problem &p, int x_mod, const T *go, const T *x,
                                         const T *cf, const T *sf, T *dx, T *dcf, T *dsf, void *ws,
                                         unsigned need, hipStream_t st) {
    if constexpr (sizeof(T) == 8) {
        return hipErrorNotSupported;
    } else {
        const int dtype = sizeof(T) == 2 ? DDF_F16 : DDF_F32;
        const unsigned fneed = need & (DDF_NEED_DCF | DDF_NEED_DSF);
        const bool want_dx = need & DDF_NEED_DX;
        RowsGeom g;
        int vx, r;
        // every vector access 16-byte aligned, so no launch below can turn the call down
        if ((((uintptr_t)go | (uintptr_t)x | (uintptr_t)sf | (uintptr_t)dx | (uintptr_t)dsf) & 15u) != 0)
            return hipErrorNotSupported;
        if (want_dx && fneed && rows_filters_geometry(p, dtype, true, &g, &vx, &r))
            return rows_filters_launch<T>(p, go, x, cf, sf, dx, dcf, dsf, ws, fneed, st, x_mod);
        if (want_dx && !rows_geometry(p, dtype, 0, &g, &vx, &r)) return hipErrorNotSupported;
        if (fneed && !rows_taprow_geometry(p, dtype, &g, &vx, &r) &&
            !rows_filters_geometry(p, dtype, false, &g, &vx, &r))
            return hipErrorNotSupported;
        hipError_t err = hipSuccess;
        if (want_dx) {
            err = rows_launch<T>(p, true, go, cf, sf, dx, st);
            if (err != hipSuccess) return err;
        }
        if (fneed) {
            err = rows_filters_launch<T>(p, go, x, cf, sf, (T *)nullptr, dcf, dsf, ws, fneed, st, x_mod);
            if (err == hipErrorNotSupported) err = hipErrorUnknown;   // (ruled out above)
        }
        return err;
    }
}

#define DDF_INSTANTIATE_ROWS(T)                                                              \
    template hipError_t rows_filters_launch<T>(const Problem &, const T *, const T *, const T *, \
                                               const T *, T *, T *, T *, void *, unsigned,   \
                                               hipStream_t, int, NormTail<T> *);              \
    template hipError_t rows_launch<T>(const Problem &, bool, const T *, const T *, const T *, \
                                       T *, hipStream_t);                                     \
    template hipError_t rows_backward_shared_features<T>(const Problem &, int, const T *,    \
                                                         const T *, const T *, const T *, T *, \
                                                         T *, T *, void *, unsigned, hipStream_t);

}  // namespace ddf
