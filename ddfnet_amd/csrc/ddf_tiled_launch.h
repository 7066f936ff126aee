// Launch code of the tiled kernels, instantiated once per element type.
#pragma once

#include <initializer_list>

#include <type_traits>

#include "ddf_wave.h"

namespace ddf {
namespace tiled {


// Expands BODY for the (K, D, S) of the problem; BODY sees constexpr KK_, DD_, SS_.
#define DDF_DISPATCH_KDS(p, ...)                                           \
    do {                                                                   \
        const int key_ = (p).k * 100 + (p).d * 10 + (p).s;                 \
        switch (key_) {                                                    \
            case 311: { constexpr int KK_ = 3, DD_ = 1, SS_ = 1; __VA_ARGS__; } break; \
            case 312: { constexpr int KK_ = 3, DD_ = 1, SS_ = 2; __VA_ARGS__; } break; \
            case 321: { constexpr int KK_ = 3, DD_ = 2, SS_ = 1; __VA_ARGS__; } break; \
            case 322: { constexpr int KK_ = 3, DD_ = 2, SS_ = 2; __VA_ARGS__; } break; \
            case 511: { constexpr int KK_ = 5, DD_ = 1, SS_ = 1; __VA_ARGS__; } break; \
            case 512: { constexpr int KK_ = 5, DD_ = 1, SS_ = 2; __VA_ARGS__; } break; \
            case 521: { constexpr int KK_ = 5, DD_ = 2, SS_ = 1; __VA_ARGS__; } break; \
            case 522: { constexpr int KK_ = 5, DD_ = 2, SS_ = 2; __VA_ARGS__; } break; \
            default: return hipErrorNotSupported;                          \
        }                                                                  \
    } while (0)

// Largest power-of-two vector <= v to which every pointer is aligned.
template <typename T>
inline bool aligned_for(int v, std::initializer_list<const void *> ptrs) {
    for (const void *p : ptrs)
        if (reinterpret_cast<uintptr_t>(p) % (v * sizeof(T)) != 0) return false;
    return true;
}

// Instantiated (PS, NV, V) of the wave kernels: V=4 with (4,1) (4,2) (4,4)
// (8,4); V=1 with (4,4) (4,8).
#define DDF_DISPATCH_WAVE(ps, nv, v, ...)                                              \
    do {                                                                               \
        if ((v) == 4 && (ps) == 4 && (nv) == 1) { constexpr int PS_ = 4, NV_ = 1, VV_ = 4; __VA_ARGS__; } \
        else if ((v) == 4 && (ps) == 4 && (nv) == 2) { constexpr int PS_ = 4, NV_ = 2, VV_ = 4; __VA_ARGS__; } \
        else if ((v) == 4 && (ps) == 4 && (nv) == 4) { constexpr int PS_ = 4, NV_ = 4, VV_ = 4; __VA_ARGS__; } \
        else if ((v) == 4 && (ps) == 8 && (nv) == 4) { constexpr int PS_ = 8, NV_ = 4, VV_ = 4; __VA_ARGS__; } \
        else if ((v) == 1 && (ps) == 4 && (nv) == 4) { constexpr int PS_ = 4, NV_ = 4, VV_ = 1; __VA_ARGS__; } \
        else if ((v) == 1 && (ps) == 4 && (nv) == 8) { constexpr int PS_ = 4, NV_ = 8, VV_ = 1; __VA_ARGS__; } \
        else return hipErrorNotSupported;                                              \
    } while (0)

template <typename T, int K, int D, int S>
hipError_t launch_forward(const Problem &p, const WaveGeom &g, int ps, int nv, const T *x,
                          const T *cf, const T *sf, T *out, hipStream_t st) {
    const dim3 grid(g.xcd_per * wave::kXcd), block(kWave * g.wpb);
    DDF_DISPATCH_WAVE(ps, nv, g.vec, {
        if constexpr (sizeof(T) == 8 && VV_ != 1) return hipErrorNotSupported;
        else if (p.mul)
            hipLaunchKernelGGL((wave::k_forward<T, K, D, S, true, PS_, NV_, VV_>), grid, block,
                               g.lds_bytes, st, g, x, cf, sf, out);
        else
            hipLaunchKernelGGL((wave::k_forward<T, K, D, S, false, PS_, NV_, VV_>), grid, block,
                               g.lds_bytes, st, g, x, cf, sf, out);
    });
    return hipGetLastError();
}

template <typename T, int K, int D, int S>
hipError_t launch_features(const Problem &p, const WaveGeom &g, int ps, int nv, const T *go,
                           const T *cf, const T *sf, T *dx, hipStream_t st) {
    const dim3 grid(g.xcd_per * wave::kXcd), block(kWave * g.wpb);
    DDF_DISPATCH_WAVE(ps, nv, g.vec, {
        if constexpr (sizeof(T) == 8 && VV_ != 1) return hipErrorNotSupported;
        else if (p.mul)
            hipLaunchKernelGGL((wave::k_backward_features<T, K, D, S, true, PS_, NV_, VV_>), grid,
                               block, g.lds_bytes, st, g, go, cf, sf, dx);
        else
            hipLaunchKernelGGL((wave::k_backward_features<T, K, D, S, false, PS_, NV_, VV_>), grid,
                               block, g.lds_bytes, st, g, go, cf, sf, dx);
    });
    return hipGetLastError();
}

// Filter gradients: 4 pixel slots per lane for k=3, 2 for k=5 (two register
// sets per slot); V=4 with NV 1, 2, 4 and V=1 with NV 4 (and 8 for k=3).
// DX: the same launch also writes the feature gradient (3x3, stride 1).
template <typename T, int K, int D, int S, int NV, int V, bool DX>
hipError_t launch_filters_nv(const Problem &p, const WaveGeom &g, const T *go, const T *x,
                             const T *cf, const T *sf, T *dx, T *dcf, T *dsf,
                             typename Acc<T>::type *ws_sf, typename Acc<T>::type *ws_cf,
                             unsigned need, hipStream_t st) {
    constexpr int PS = K == 3 ? 4 : 2;
    const dim3 grid(g.xcd_per * wave::kXcd), block(kWave * wave::kFilterWaves);
    if (p.mul)
        hipLaunchKernelGGL((wave::k_backward_filters<T, K, D, S, true, PS, NV, V, DX>), grid,
                           block, g.lds_bytes, st, g, go, x, cf, sf, dx, dcf, dsf, ws_sf, ws_cf,
                           need);
    else
        hipLaunchKernelGGL((wave::k_backward_filters<T, K, D, S, false, PS, NV, V, DX>), grid,
                           block, g.lds_bytes, st, g, go, x, cf, sf, dx, dcf, dsf, ws_sf, ws_cf,
                           need);
    return hipGetLastError();
}

template <typename T, int K, int D, int S, bool DX>
hipError_t launch_filters(const Problem &p, const WaveGeom &g, int ps, int nv, const T *go,
                          const T *x, const T *cf, const T *sf, T *dx, T *dcf, T *dsf,
                          typename Acc<T>::type *ws_sf, typename Acc<T>::type *ws_cf,
                          unsigned need, hipStream_t st) {
    if (ps != (K == 3 ? 4 : 2)) return hipErrorNotSupported;
    if constexpr (DX && (K != 3 || S != 1)) {
        return hipErrorNotSupported;
    } else {
#define DDF_FILTERS_CASE(NV_, V_)                                                             \
    if (g.vec == V_ && nv == NV_)                                                             \
        return launch_filters_nv<T, K, D, S, NV_, V_, DX>(p, g, go, x, cf, sf, dx, dcf, dsf,  \
                                                          ws_sf, ws_cf, need, st);
        if constexpr (sizeof(T) != 8) {
            DDF_FILTERS_CASE(1, 4)
            if constexpr (!DX) {
                DDF_FILTERS_CASE(2, 4)
                DDF_FILTERS_CASE(4, 4)
            }
        }
        if constexpr (!DX) {
            DDF_FILTERS_CASE(4, 1)
            if constexpr (K == 3) { DDF_FILTERS_CASE(8, 1) }
        }
#undef DDF_FILTERS_CASE
        return hipErrorNotSupported;
    }
}

}  // namespace tiled

// A misaligned pointer sends the problem down the scalar-access geometry
// (same kernels, one element per access).
template <typename T>
bool wave_plan(const Problem &p, int kind, std::initializer_list<const void *> ptrs, WaveGeom *g,
               int *ps, int *nv) {
    const int dtype = sizeof(T) == 2 ? DDF_F16 : sizeof(T) == 4 ? DDF_F32 : DDF_F64;
    if (!wave_geometry(p, dtype, kind, 0, g, ps, nv)) return false;
    if (g->vec > 1 && !tiled::aligned_for<T>(g->vec, ptrs)) {
        // the workspace was sized for the aligned plan: the scalar plan must cut
        // the problem the same way
        const int th = g->TH, csplit = g->csplit;
        if (!wave_geometry(p, dtype, kind, 1, g, ps, nv)) return false;
        return g->TH == th && g->csplit == csplit;
    }
    return true;
}

template <typename T>
hipError_t tiled_forward(const Problem &p, const T *x, const T *cf, const T *sf, T *out,
                         hipStream_t st) {
    if constexpr (sizeof(T) != 8) {
        if (tune_int("DDF_TUNE_ROWS", 1) != 0) {
            const hipError_t err = rows_launch<T>(p, false, x, cf, sf, out, st);
            if (err != hipErrorNotSupported) return err;
        }
    }
    // (tiny planes the row-register kernels lack a vector width for: fp16 with odd rows)
    if (small_supported(p)) return small_launch<T>(p, false, x, cf, sf, out, st);
    WaveGeom g; int ps, nv;
    if (!wave_plan<T>(p, kWaveForward, {x, sf, out}, &g, &ps, &nv))
        return generic_forward<T>(p, x, cf, sf, out, st);   // e.g. pointers not 16-byte aligned
    DDF_DISPATCH_KDS(p, return tiled::launch_forward<T, KK_, DD_, SS_>(p, g, ps, nv, x, cf, sf, out, st));
    return hipErrorNotSupported;
}

template <typename T>
hipError_t tiled_backward(const Problem &p, const T *go, const T *x, const T *cf, const T *sf,
                          T *dx, T *dcf, T *dsf, void *ws, unsigned need, hipStream_t st,
                          NormTail<T> *norm) {
    using A = typename Acc<T>::type;
    const int dtype = sizeof(T) == 2 ? DDF_F16 : sizeof(T) == 4 ? DDF_F32 : DDF_F64;
    hipError_t err = hipSuccess;
    const unsigned fneed = need & (DDF_NEED_DCF | DDF_NEED_DSF);
    // One launch for all gradients where the fused kernel exists and cuts the
    // problem exactly as the workspace was sized for.
    if constexpr (sizeof(T) != 8) {
        // the row-register kernel does the whole backward pass in one launch where it covers it
        if ((need & DDF_NEED_DX) && fneed && tune_int("DDF_TUNE_ROWSF", 1) != 0) {
            err = rows_filters_launch<T>(p, go, x, cf, sf, dx, dcf, dsf, ws, fneed, st, 0, norm);
            if (err != hipErrorNotSupported) return err;
            err = hipSuccess;
        }
    }
    WaveGeom g; int ps, nv;
    bool fuse = false;
    // (where the row-register kernels cover both halves, two of their launches beat
    // the fused tile kernel)
    bool rows_both = false;
    if constexpr (sizeof(T) != 8) {
        rows_both = tune_int("DDF_TUNE_ROWS", 1) != 0 && tune_int("DDF_TUNE_ROWSF", 1) != 0 &&
                    rows_cover_backward(p, dtype);
    }
    // (stride 2: the row-register kernels do the filter gradients, the tile kernel dX)
    bool rows_filters_only = false;
    if constexpr (sizeof(T) != 8) {
        rows_filters_only = tune_int("DDF_TUNE_ROWSF", 1) != 0 && rows_cover_stride2_filters(p, dtype);
    }
    if ((need & DDF_NEED_DX) && fneed && !rows_both && !rows_filters_only &&
        tune_int("DDF_TUNE_FUSED", 1) != 0) {
        WaveGeom gp; int pps, pnv;
        fuse = wave_plan<T>(p, kWaveFused, {go, x, sf, dx}, &g, &ps, &nv) &&
               wave_geometry(p, dtype, kWaveFilters, 0, &gp, &pps, &pnv) && gp.TH == g.TH &&
               gp.csplit == g.csplit;
    }
    if ((need & DDF_NEED_DX) && !fuse) {
        bool done = false;
        if constexpr (sizeof(T) != 8) {
            if (tune_int("DDF_TUNE_ROWS", 1) != 0) {
                err = rows_launch<T>(p, true, go, cf, sf, dx, st);
                done = err != hipErrorNotSupported;
            }
        }
        if (done) {
        } else if (small_supported(p)) {
            err = small_launch<T>(p, true, go, cf, sf, dx, st);
        } else if (!wave_plan<T>(p, kWaveFeatures, {go, sf, dx}, &g, &ps, &nv)) {
            err = generic_backward<T>(p, go, x, cf, sf, dx, dcf, dsf, DDF_NEED_DX, st);
        } else {
            DDF_DISPATCH_KDS(p, err = tiled::launch_features<T, KK_, DD_, SS_>(p, g, ps, nv, go, cf, sf, dx, st));
        }
        if (err != hipSuccess) return err;
    }
    if (fneed && !fuse) {
        if constexpr (sizeof(T) != 8) {
            if (tune_int("DDF_TUNE_ROWSF", 1) != 0) {
                err = rows_filters_launch<T>(p, go, x, cf, sf, (T *)nullptr, dcf, dsf, ws, fneed, st, 0,
                                             norm);
                if (err != hipErrorNotSupported) return err;
                err = hipSuccess;
            }
        }
    }
    if (fneed) {
        if (!fuse && !wave_plan<T>(p, kWaveFilters, {go, x, sf}, &g, &ps, &nv))
            return generic_backward<T>(p, go, x, cf, sf, dx, dcf, dsf, fneed, st);
        // carve the workspace exactly as tiled_backward_workspace() sized it
        unsigned char *wp = static_cast<unsigned char *>(ws);
        A *ws_sf = nullptr, *ws_cf = nullptr;
        const int64_t n_sf = p.N * p.kk * p.Ho * p.Wo;
        if ((fneed & DDF_NEED_DSF) && g.csplit > 1) {
            ws_sf = reinterpret_cast<A *>(wp);
            wp += ((size_t)n_sf * g.csplit * sizeof(A) + 255) / 256 * 256;
        }
        if ((fneed & DDF_NEED_DCF) && g.nstrips > 1) ws_cf = reinterpret_cast<A *>(wp);
        if (fuse)
            DDF_DISPATCH_KDS(p, err = tiled::launch_filters<T, KK_, DD_, SS_, true>(
                                    p, g, ps, nv, go, x, cf, sf, dx, dcf, dsf, ws_sf, ws_cf, fneed,
                                    st));
        else
            DDF_DISPATCH_KDS(p, err = tiled::launch_filters<T, KK_, DD_, SS_, false>(
                                    p, g, ps, nv, go, x, cf, sf, dx, dcf, dsf, ws_sf, ws_cf, fneed,
                                    st));
        if (err != hipSuccess) return err;
        // dSF[n, t, pix] = sum over channel splits, dCF[nc, t] = sum over strips
        err = wave::sum_filter_partials<T>(ws_sf, dsf, p.N, g.csplit, p.kk * p.Ho * p.Wo, ws_cf, dcf,
                                           p.N * p.C, g.nstrips, (int64_t)p.kk, st,
                                           (fneed & DDF_NEED_DSF) ? norm : nullptr);
        if (err != hipSuccess) return err;
    }
    return err;
}

#define DDF_INSTANTIATE_TILED(T)                                                          \
    template hipError_t tiled_forward<T>(const Problem &, const T *, const T *, const T *, \
                                         T *, hipStream_t);                               \
    template hipError_t tiled_backward<T>(const Problem &, const T *, const T *, const T *, \
                                          const T *, T *, T *, T *, void *, unsigned,     \
                                          hipStream_t, NormTail<T> *);

}  // namespace ddf
