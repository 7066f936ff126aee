// Names of the kernels a call launches (ddf_hip_describe): the same choices as
// tiled_forward / tiled_backward in ddf_tiled_launch.h, from the geometry alone.
#include <cstdio>

#include "ddf_rows_taprow.h"
#include "ddf_wave.h"

namespace ddf {

namespace {
// The launch that adds up what a filter-gradient kernel leaves in the workspace.
// norm: the call is ddf_hip_backward_spatial_norm; the normalisation's Jacobian rides on
// that launch where there is one (and a kernel for kk taps), else it is a launch of its own.
const char *sums_name(unsigned fneed, int csplit, int nstrips, bool norm = false, int kk = 0) {
    const bool sf = (fneed & DDF_NEED_DSF) && csplit > 1, cf = (fneed & DDF_NEED_DCF) && nstrips > 1;
    if (norm && (fneed & DDF_NEED_DSF))
        return (sf || cf) && wave::norm_tail_kernel_built<float>(kk) ? " + k_sum_norm_pair"
               : sf && cf ? " + k_sum_partials_pair + k_filter_norm_backward"
               : (sf || cf) ? " + k_sum_partials + k_filter_norm_backward"
                            : " + k_filter_norm_backward";
    return sf && cf ? " + k_sum_partials_pair" : (sf || cf) ? " + k_sum_partials" : "";
}
const char *layout_name(const RowsGeom &g) {
    if (g.Hi != g.H) return g.lp > g.lpr ? "padded,stride 2" : "plain,stride 2";
    return g.segs > 0 ? "segments" : g.lp > g.lpr ? "padded" : "plain";
}
}  // namespace

// Which kernels a call would launch, in words (pointer alignment assumed).
// Mirrors the choices of tiled_forward / tiled_backward in ddf_tiled_launch.h.
int describe_forward(const Problem &p, int dtype, char *buf, int len) {
    RowsGeom rg; int vx, r;
    WaveGeom wg; int ps, nv;
    if (dtype != DDF_F64 && tune_int("DDF_TUNE_ROWS", 1) != 0 && rows_geometry(p, dtype, 0, &rg, &vx, &r))
        return snprintf(buf, len, "k_rows<VX=%d,R=%d,%s>", vx, r, layout_name(rg));
    if (small_supported(p)) return snprintf(buf, len, "k_small");
    if (wave_geometry(p, dtype, kWaveForward, 0, &wg, &ps, &nv))
        return snprintf(buf, len, "k_forward<PS=%d,NV=%d,V=%d>", ps, nv, wg.vec);
    return snprintf(buf, len, "generic_forward");
}

int describe_backward(const Problem &p, int dtype, unsigned need, char *buf, int len) {
    RowsGeom rg; int vx, r;
    WaveGeom wg, gp; int ps, nv, pps, pnv;
    const unsigned fneed = need & (DDF_NEED_DCF | DDF_NEED_DSF);
    const bool norm = need & DDF_DESCRIBE_SPATIAL_NORM;
    int n = 0;
    auto add = [&](const char *fmt, auto... args) {
        if (n < len) n += snprintf(buf + n, len - n, fmt, args...);
    };
    if (len > 0) buf[0] = 0;
    const bool tiled = wave_geometry(p, dtype, kWaveFeatures, 0, &wg, &ps, &nv) &&
                       wave_geometry(p, dtype, kWaveFilters, 0, &wg, &ps, &nv);
    const bool rows_both = dtype != DDF_F64 && tune_int("DDF_TUNE_ROWS", 1) != 0 &&
                           tune_int("DDF_TUNE_ROWSF", 1) != 0 &&
                           rows_cover_backward(p, dtype);
    if (!tiled && !rows_both) {
        add("%s", norm && (fneed & DDF_NEED_DSF) ? "generic_backward + k_filter_norm_backward" : "generic_backward");
        return n;
    }
    const bool rows_filters_only = dtype != DDF_F64 && tune_int("DDF_TUNE_ROWSF", 1) != 0 &&
                                   rows_cover_stride2_filters(p, dtype);
    const bool fuse = tiled && (need & DDF_NEED_DX) && fneed && !rows_both && !rows_filters_only &&
                      tune_int("DDF_TUNE_FUSED", 1) != 0 &&
                      wave_geometry(p, dtype, kWaveFused, 0, &wg, &ps, &nv) &&
                      wave_geometry(p, dtype, kWaveFilters, 0, &gp, &pps, &pnv) && gp.TH == wg.TH &&
                      gp.csplit == wg.csplit;
    if ((need & DDF_NEED_DX) && fneed && dtype != DDF_F64 && tune_int("DDF_TUNE_ROWSF", 1) != 0 &&
        rows_filters_geometry(p, dtype, true, &rg, &vx, &r)) {
        add("k_rows_filters<dX,VX=%d,R=%d,%s>", vx, r, layout_name(rg));
        add("%s", sums_name(fneed, rg.csplit, rg.nstrips, norm, p.kk));
        return n;
    }
    if (fuse) {
        add("%s", "k_backward_filters<DX>");
        add("%s", sums_name(fneed, wg.csplit, wg.nstrips, norm, p.kk));
        return n;
    }
    if (need & DDF_NEED_DX) {
        if (dtype != DDF_F64 && tune_int("DDF_TUNE_ROWS", 1) != 0 &&
            (p.s == 1 || rows_stride2_feature_gradient(p)) && rows_geometry(p, dtype, 0, &rg, &vx, &r))
            add("k_rows<dX,VX=%d,R=%d,%s>", vx, r, layout_name(rg));
        else if (small_supported(p)) add("%s", "k_small<dX>");
        else add("%s", "k_backward_features");
    }
    if (fneed) {
        if (n) add("%s", " + ");
        if (dtype != DDF_F64 && tune_int("DDF_TUNE_ROWSF", 1) != 0 &&
            rows_taprow_geometry(p, dtype, &rg, &vx, &r)) {
            add("k_rows_taprow_filters<VX=%d,%s>", vx, layout_name(rg));
            add("%s", sums_name(fneed, rg.csplit, rg.nstrips, norm, p.kk));
        } else if (dtype != DDF_F64 && tune_int("DDF_TUNE_ROWSF", 1) != 0 &&
            rows_filters_geometry(p, dtype, false, &rg, &vx, &r)) {
            add("k_rows_filters<VX=%d,R=%d,%s>", vx, r, layout_name(rg));
            add("%s", sums_name(fneed, rg.csplit, rg.nstrips, norm, p.kk));
        } else {
            wave_geometry(p, dtype, kWaveFilters, 0, &wg, &ps, &nv);
            add("%s", "k_backward_filters");
            add("%s", sums_name(fneed, wg.csplit, wg.nstrips, norm, p.kk));
        }
    }
    return n;
}

}  // namespace ddf
