// Launch code of the tiled kernels, instantiated once per element type.
#pragma once

#include "ddf_tiled.h"

namespace ddf {
namespace tiled {

inline unsigned padded_grid(int nblocks) { return (unsigned)((nblocks + kXcd - 1) / kXcd * kXcd); }

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

template <typename T, int K, int D, int S, int PS>
hipError_t launch_forward(const Problem &p, const TileGeom &g, const T *x, const T *cf,
                          const T *sf, T *out, hipStream_t st) {
    const dim3 grid(padded_grid(g.nblocks)), block(g.threads);
    if (p.mul)
        hipLaunchKernelGGL((k_forward<T, K, D, S, true, PS>), grid, block, g.lds_bytes, st, g, x,
                           cf, sf, out);
    else
        hipLaunchKernelGGL((k_forward<T, K, D, S, false, PS>), grid, block, g.lds_bytes, st, g,
                           x, cf, sf, out);
    return hipGetLastError();
}

template <typename T, int K, int D, int S, int PS>
hipError_t launch_features(const Problem &p, const TileGeom &g, const T *go, const T *cf,
                           const T *sf, T *dx, hipStream_t st) {
    const dim3 grid(padded_grid(g.nblocks)), block(g.threads);
    if (p.mul)
        hipLaunchKernelGGL((k_backward_features<T, K, D, S, true, PS>), grid, block, g.lds_bytes,
                           st, g, go, cf, sf, dx);
    else
        hipLaunchKernelGGL((k_backward_features<T, K, D, S, false, PS>), grid, block,
                           g.lds_bytes, st, g, go, cf, sf, dx);
    return hipGetLastError();
}

template <typename T, int K, int D, int S, int PS>
hipError_t launch_filters(const Problem &p, const TileGeom &g, const T *go, const T *x,
                          const T *cf, const T *sf, T *dcf, T *dsf,
                          typename Acc<T>::type *ws_sf, typename Acc<T>::type *ws_cf,
                          unsigned need, hipStream_t st) {
    const dim3 grid(padded_grid(g.nblocks)), block(g.threads);
    if (p.mul)
        hipLaunchKernelGGL((k_backward_filters<T, K, D, S, true, PS>), grid, block, g.lds_bytes,
                           st, g, go, x, cf, sf, dcf, dsf, ws_sf, ws_cf, need);
    else
        hipLaunchKernelGGL((k_backward_filters<T, K, D, S, false, PS>), grid, block, g.lds_bytes,
                           st, g, go, x, cf, sf, dcf, dsf, ws_sf, ws_cf, need);
    return hipGetLastError();
}

}  // namespace tiled

template <typename T>
hipError_t tiled_forward(const Problem &p, const T *x, const T *cf, const T *sf, T *out,
                         hipStream_t st) {
    TileGeom g; int ps;
    const int dtype = sizeof(T) == 2 ? DDF_F16 : sizeof(T) == 4 ? DDF_F32 : DDF_F64;
    if (!tiled_geometry(p, dtype, kKindForward, &g, &ps)) return hipErrorNotSupported;
    DDF_DISPATCH_KDS(p, do {
        if (ps == 1) return tiled::launch_forward<T, KK_, DD_, SS_, 1>(p, g, x, cf, sf, out, st);
        return tiled::launch_forward<T, KK_, DD_, SS_, 2>(p, g, x, cf, sf, out, st);
    } while (0));
    return hipErrorNotSupported;
}

template <typename T>
hipError_t tiled_backward(const Problem &p, const T *go, const T *x, const T *cf, const T *sf,
                          T *dx, T *dcf, T *dsf, void *ws, unsigned need, hipStream_t st) {
    using A = typename Acc<T>::type;
    const int dtype = sizeof(T) == 2 ? DDF_F16 : sizeof(T) == 4 ? DDF_F32 : DDF_F64;
    hipError_t err = hipSuccess;
    if (need & DDF_NEED_DX) {
        TileGeom g; int ps;
        if (!tiled_geometry(p, dtype, kKindFeatures, &g, &ps)) return hipErrorNotSupported;
        DDF_DISPATCH_KDS(p, do {
            err = ps == 1
                ? tiled::launch_features<T, KK_, DD_, SS_, 1>(p, g, go, cf, sf, dx, st)
                : tiled::launch_features<T, KK_, DD_, SS_, 2>(p, g, go, cf, sf, dx, st);
        } while (0));
        if (err != hipSuccess) return err;
    }
    const unsigned fneed = need & (DDF_NEED_DCF | DDF_NEED_DSF);
    if (fneed) {
        TileGeom g; int ps;
        if (!tiled_geometry(p, dtype, kKindFilters, &g, &ps)) return hipErrorNotSupported;
        // carve the workspace exactly as tiled_backward_workspace() sized it
        unsigned char *wp = static_cast<unsigned char *>(ws);
        A *ws_sf = nullptr, *ws_cf = nullptr;
        const int64_t n_sf = p.N * p.kk * p.Ho * p.Wo;
        if ((fneed & DDF_NEED_DSF) && g.csplit > 1) {
            ws_sf = reinterpret_cast<A *>(wp);
            wp += ((size_t)n_sf * g.csplit * sizeof(A) + 255) / 256 * 256;
        }
        if ((fneed & DDF_NEED_DCF) && g.nstrips > 1) ws_cf = reinterpret_cast<A *>(wp);
        DDF_DISPATCH_KDS(p, do {
            if (ps == 1)
                err = tiled::launch_filters<T, KK_, DD_, SS_, 1>(p, g, go, x, cf, sf, dcf, dsf,
                                                                 ws_sf, ws_cf, fneed, st);
            else if (ps == 2)
                err = tiled::launch_filters<T, KK_, DD_, SS_, 2>(p, g, go, x, cf, sf, dcf, dsf,
                                                                 ws_sf, ws_cf, fneed, st);
            else
                err = tiled::launch_filters<T, KK_, DD_, SS_, 4>(p, g, go, x, cf, sf, dcf, dsf,
                                                                 ws_sf, ws_cf, fneed, st);
        } while (0));
        if (err != hipSuccess) return err;
        if (ws_sf) {
            // dSF[n, t, pix] = sum over channel splits
            const int64_t inner = p.kk * p.Ho * p.Wo, total = p.N * inner;
            hipLaunchKernelGGL((tiled::k_sum_partials<T>), dim3((unsigned)cdiv(total, 256)),
                               dim3(256), 0, st, ws_sf, dsf, p.N, g.csplit, inner);
            if ((err = hipGetLastError()) != hipSuccess) return err;
        }
        if (ws_cf) {
            // dCF[nc, t] = sum over strips
            const int64_t total = p.N * p.C * p.kk;
            hipLaunchKernelGGL((tiled::k_sum_partials<T>), dim3((unsigned)cdiv(total, 256)),
                               dim3(256), 0, st, ws_cf, dcf, p.N * p.C, g.nstrips,
                               (int64_t)p.kk);
            if ((err = hipGetLastError()) != hipSuccess) return err;
        }
    }
    return err;
}

#define DDF_INSTANTIATE_TILED(T)                                                          \
    template hipError_t tiled_forward<T>(const Problem &, const T *, const T *, const T *, \
                                         T *, hipStream_t);                               \
    template hipError_t tiled_backward<T>(const Problem &, const T *, const T *, const T *, \
                                          const T *, T *, T *, T *, void *, unsigned,     \
                                          hipStream_t);

}  // namespace ddf
