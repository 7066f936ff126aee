// Host-side geometry of the tiled DDF kernels: strip height, LDS tile, how many
// channels a workgroup walks, and the workspace the filter gradients need.
#include <algorithm>
#include <cstdlib>

#include "ddf_tiled.h"

namespace ddf {

namespace {

constexpr int kLdsBudget = 48 * 1024;   // bytes per workgroup; leaves room for >= 3 per CU
constexpr int kMaxThreads = 512;

int env_int(const char *name, int fallback) {
    const char *v = std::getenv(name);
    return (v && *v) ? std::atoi(v) : fallback;
}

int elem_size(int dtype) { return dtype == DDF_F16 ? 2 : dtype == DDF_F32 ? 4 : 8; }
int acc_size(int dtype) { return dtype == DDF_F64 ? 8 : 4; }
int round_up(int v, int m) { return (v + m - 1) / m * m; }

}  // namespace

bool tiled_shape_instantiated(int k, int d, int s) {
    return (k == 3 || k == 5) && (d == 1 || d == 2) && (s == 1 || s == 2);
}

// Fills *g and *ps for one kernel kind; false when the tiled family does not
// cover the problem (the caller then uses the generic kernels).
bool tiled_geometry(const Problem &p, int dtype, int kind, TileGeom *g, int *ps_out) {
    if (!tiled_shape_instantiated(p.k, p.d, p.s)) return false;
    if (p.N <= 0 || p.C <= 0 || p.Ho <= 0 || p.Wo <= 0) return false;
    if (p.H > 16384 || p.W > 16384 || p.C > (1 << 24) || p.N > (1 << 24)) return false;
    const int esz = elem_size(dtype), asz = acc_size(dtype);
    const int K = p.k, D = p.d, S = p.s, R = p.r, KK = p.kk;
    const int H = (int)p.H, W = (int)p.W, Ho = (int)p.Ho, Wo = (int)p.Wo, C = (int)p.C;

    TileGeom t{};
    t.C = C; t.H = H; t.W = W; t.Ho = Ho; t.Wo = Wo;
    int halo_lo = 0, halo_hi = 0;
    if (kind == kKindFeatures) {
        halo_lo = (R * D) / S;
        halo_hi = (R * D + S - 1) / S;
        t.rows = (H + S - 1) / S; t.cols = (W + S - 1) / S;
        t.src_rows = Ho; t.src_cols = Wo;
        t.P = t.cols + halo_lo + halo_hi;
        t.col_off = halo_lo; t.row0_off = -halo_lo; t.row_step = 1;
    } else {
        t.rows = Ho; t.cols = Wo;
        t.src_rows = H; t.src_cols = W;
        t.P = std::max((Wo - 1) * S + (K - 1) * D + 1, R * D + W);
        t.col_off = R * D; t.row0_off = -R * D; t.row_step = S;
    }
    auto tile_rows = [&](int th) {
        return kind == kKindFeatures ? th + halo_lo + halo_hi : (th - 1) * S + (K - 1) * D + 1;
    };

    // Pixels (cells) one block pass can own.
    const bool per_lane = (kind == kKindFilters);
    const int max_ps = per_lane ? 4 : 2;
    const int capacity = per_lane ? kWave * max_ps : kMaxThreads * max_ps;
    if (t.cols > capacity || t.cols >= 65536) return false;
    if (tile_rows(1) * t.P * esz > kLdsBudget) return false;

    // Strip height and pixels per thread: minimise an instruction estimate per
    // strip set.  Compute costs ~2*KK (3*KK for the filter gradients) per
    // owned pixel slot, idle lanes included; staging costs ~4 per tile element;
    // the filter-gradient kernel adds one butterfly (~3*KK) per wave pass.
    const int c_comp = (per_lane ? 3 : 2) * KK, c_load = 4, c_red = 3 * KK;
    double best = 1e30;
    int best_th = 0, best_ps = 0;
    const int forced_th = env_int(per_lane ? "DDF_TUNE_TH_FILTERS" : "DDF_TUNE_TH", 0);
    const int forced_ps = env_int(per_lane ? "DDF_TUNE_PS_FILTERS" : "DDF_TUNE_PS", 0);
    for (int th = 1; th <= t.rows; ++th) {
        const int np = th * t.cols;
        if (np > capacity) break;
        if (tile_rows(th) * t.P * esz > kLdsBudget) break;
        if (forced_th && th != std::min(forced_th, t.rows)) continue;
        const int nstrips = (t.rows + th - 1) / th;
        for (int ps = 1; ps <= max_ps; ps *= 2) {
            if (forced_ps && ps != forced_ps) continue;
            const int lanes = per_lane ? kWave : kMaxThreads;
            if (np > lanes * ps) continue;
            const int slots = per_lane ? kWave * ps : round_up((np + ps - 1) / ps, kWave) * ps;
            double cost = (double)nstrips *
                          (slots * c_comp + (double)tile_rows(th) * t.P * c_load +
                           (per_lane ? c_red : 0));
            cost *= 1.0 + 0.02 * ps;  // mild preference for fewer registers
            if (cost < best) { best = cost; best_th = th; best_ps = ps; }
        }
    }
    if (best_th == 0) return false;
    t.TH = best_th;
    t.nstrips = (t.rows + t.TH - 1) / t.TH;
    t.IH = tile_rows(t.TH);
    t.tile = t.IH * t.P;
    const int ps = best_ps;
    const int np = t.TH * t.cols;

    if (per_lane) {
        t.nwaves = std::max(1, std::min(env_int("DDF_TUNE_WAVES_FILTERS", 4), C));
        t.threads = kWave * t.nwaves;
    } else {
        t.threads = round_up((np + ps - 1) / ps, kWave);
        t.nwaves = t.threads / kWave;
    }

    // Channels per block: enough blocks to fill 256 CUs several times over, but
    // long enough channel walks to amortise the spatial-filter registers.
    const int64_t base = p.N * t.nstrips;
    const int target = env_int(per_lane ? "DDF_TUNE_BLOCKS_FILTERS" : "DDF_TUNE_BLOCKS",
                               per_lane ? 1024 : 2048) * 256 / t.threads;
    int min_cpb = per_lane ? 4 * t.nwaves : 8;
    int64_t want_split = std::max<int64_t>(1, (target + base - 1) / base);
    int cpb = (int)std::max<int64_t>(min_cpb, (C + want_split - 1) / want_split);
    const int forced_cpb = env_int(per_lane ? "DDF_TUNE_CPB_FILTERS" : "DDF_TUNE_CPB", 0);
    if (forced_cpb) cpb = forced_cpb;
    if (per_lane) cpb = round_up(cpb, t.nwaves);
    cpb = std::min(cpb, per_lane ? round_up(C, t.nwaves) : C);
    t.cpb = cpb;
    t.csplit = (C + cpb - 1) / cpb;

    int cb = env_int("DDF_TUNE_CB", 8);
    if (per_lane) cb = round_up(cb, t.nwaves);
    cb = std::min(cb, cpb);
    while (cb > 1 && cb * t.tile * esz > kLdsBudget) cb = per_lane ? cb - t.nwaves : cb - 1;
    if (cb < 1 || cb * t.tile * esz > kLdsBudget) return false;
    if (per_lane && cb % t.nwaves != 0 && cb != cpb) {
        // fewer channels per stage than waves: shrink the block instead
        t.nwaves = cb; t.threads = kWave * cb;
    }
    t.CB = cb;
    t.lds_bytes = cb * t.tile * esz;
    if (per_lane) t.lds_bytes = std::max(t.lds_bytes, t.nwaves * KK * kWave * asz);
    if (t.lds_bytes > 64 * 1024) return false;

    // Loader: rows of 2^lw_shift lanes, as many rows per pass as the block has.
    int lw_shift = 0;
    while ((1 << lw_shift) < t.src_cols && (2 << lw_shift) <= t.threads) ++lw_shift;
    t.lw_shift = lw_shift;
    t.lrows = t.threads >> lw_shift;
    t.cols_magic = t.cols == 1 ? 0u : (unsigned)((0x100000000ull + t.cols - 1) / t.cols);
    const int64_t nblocks = base * t.csplit;
    if (nblocks > (1 << 30)) return false;
    t.nblocks = (int)nblocks;
    *g = t;
    *ps_out = ps;
    return true;
}

bool tiled_forward_supported(const Problem &p, int dtype) {
    TileGeom g; int ps;
    return tiled_geometry(p, dtype, kKindForward, &g, &ps);
}

bool tiled_backward_supported(const Problem &p, int dtype) {
    TileGeom g; int ps;
    return tiled_geometry(p, dtype, kKindFeatures, &g, &ps) &&
           tiled_geometry(p, dtype, kKindFilters, &g, &ps);
}

// Workspace layout: [dSF partials over channel splits][dCF partials over strips],
// each in the accumulator type and starting on a 256-byte boundary.
size_t tiled_backward_workspace(const Problem &p, int dtype, unsigned need) {
    if (!(need & (DDF_NEED_DCF | DDF_NEED_DSF))) return 0;
    TileGeom g; int ps;
    if (!tiled_geometry(p, dtype, kKindFilters, &g, &ps)) return 0;
    const size_t asz = acc_size(dtype);
    size_t bytes = 0;
    if ((need & DDF_NEED_DSF) && g.csplit > 1)
        bytes += ((size_t)p.N * g.csplit * p.kk * p.Ho * p.Wo * asz + 255) / 256 * 256;
    if ((need & DDF_NEED_DCF) && g.nstrips > 1)
        bytes += ((size_t)p.N * p.C * g.nstrips * p.kk * asz + 255) / 256 * 256;
    return bytes;
}

}  // namespace ddf
