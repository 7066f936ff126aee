// Host-side geometry of the tiled DDF kernels: strip height, LDS tile, how many
// channels a workgroup walks, and the workspace the filter gradients need.
#include <algorithm>
#include <cstdlib>

#include "ddf_rows_filters.h"
#include "ddf_wave.h"

namespace ddf {

namespace {


// Launch-geometry knobs.  A release build compiles them to their defaults: no
// environment lookups on the launch path, and a geometry that depends on the
// problem alone.  Built with -DDDF_TUNING they are read from the environment
// at every call, for experiments and for the host-side bounds model.
int env_int(const char *name, int fallback) {
#ifdef DDF_TUNING
    const char *v = std::getenv(name);
    return (v && *v) ? std::atoi(v) : fallback;
#else
    (void)name;
    return fallback;
#endif
}

int elem_size(int dtype) { return dtype == DDF_F16 ? 2 : dtype == DDF_F32 ? 4 : 8; }
int acc_size(int dtype) { return dtype == DDF_F64 ? 8 : 4; }
int round_up(int v, int m) { return (v + m - 1) / m * m; }

}  // namespace

int tune_int(const char *name, int fallback) { return env_int(name, fallback); }

size_t wave_backward_workspace(const Problem &p, int dtype, unsigned need);

bool tiled_shape_instantiated(int k, int d, int s) {
    return (k == 3 || k == 5) && (d == 1 || d == 2) && (s == 1 || s == 2);
}

// Geometry of the wavefront-per-strip kernels (forward, feature gradient).
// *ps_out / *nv_out name the instantiation: cell slots per lane and source
// vectors per lane per channel.
bool wave_geometry(const Problem &p, int dtype, int kind, int max_vec, WaveGeom *g, int *ps_out,
                   int *nv_out) {
    if (!tiled_shape_instantiated(p.k, p.d, p.s)) return false;
    if (kind == kWaveFused && (p.s != 1 || p.k != 3)) return false;
    if (p.N <= 0 || p.C <= 0 || p.Ho <= 0 || p.Wo <= 0) return false;
    if (p.H > 16384 || p.W > 16384 || p.C > (1 << 24) || p.N > (1 << 24)) return false;
    const int esz = elem_size(dtype);
    const int asz = (int)acc_size(dtype);
    const int K = p.k, D = p.d, S = p.s, R = p.r;
    const int H = (int)p.H, W = (int)p.W, Ho = (int)p.Ho, Wo = (int)p.Wo, C = (int)p.C;

    WaveGeom t{};
    t.C = C; t.H = H; t.W = W; t.Ho = Ho; t.Wo = Wo;
    int halo_lo = 0, halo_hi = 0;
    if (kind == kWaveFeatures) {
        halo_lo = (R * D) / S;
        halo_hi = (R * D + S - 1) / S;
        t.rows = (H + S - 1) / S; t.cols = (W + S - 1) / S;
        t.src_rows = Ho; t.src_cols = Wo;
        t.P = t.cols + halo_lo + halo_hi;
        t.col_off = halo_lo; t.row0_off = -halo_lo;
        t.lin_cols = W; t.lin_rpc = S; t.lin_rows = H;
    } else {
        t.rows = Ho; t.cols = Wo;
        t.src_rows = H; t.src_cols = W;
        t.P = std::max((Wo - 1) * S + (K - 1) * D + 1, R * D + W);
        t.col_off = R * D; t.row0_off = -R * D;
        t.lin_cols = Wo; t.lin_rpc = 1; t.lin_rows = Ho;
    }
    // Rows whose length is a multiple of 4 elements: widen the left border to 4
    // columns and the pitch to a multiple of 4, so that every 4-element source
    // vector lands on 4 neighbouring, 16-byte aligned tile elements.
    const bool can_widen = dtype != DDF_F64 && t.src_cols % 4 == 0 && max_vec != 1 &&
                           env_int("DDF_TUNE_VEC", 0) != 1 && env_int("DDF_TUNE_WIDE", 1) != 0;
    if (can_widen) {
        const int natural = t.col_off;
        t.col_off = round_up(natural, 4);
        t.lb_shift = t.col_off - natural;
        t.P = round_up(t.P + t.lb_shift, 4);
    }
    auto tile_rows = [&](int th) {
        return kind == kWaveFeatures ? th + halo_lo + halo_hi : (th - 1) * S + (K - 1) * D + 1;
    };

    // lanes: LW per cell row segment, 64 / LW cell rows per slot
    int lw_shift = 0;
    while ((1 << lw_shift) < std::min(t.cols, kWave)) ++lw_shift;
    const int LW = 1 << lw_shift, RS = kWave / LW;
    const int cseg = (t.cols + LW - 1) / LW;
    if (cseg > kMaxSlots) return false;
    t.lw_shift = lw_shift;

    // Every strip's source run and result run must start and end on a vector
    // boundary for V-element accesses.
    const int64_t plane_in = (int64_t)t.src_rows * t.src_cols;
    const int64_t plane_lin = (int64_t)t.lin_rows * t.lin_cols;
    auto vec_ok = [&](int v, int th) {
        if (v == 1) return true;
        if (plane_in % v || plane_lin % v || t.src_cols < v) return false;
        for (int first = 0; first < t.rows; first += th) {
            const int nrows = std::min(th, t.rows - first);
            const int row0 = (kind == kWaveFeatures ? first : first * S) + t.row0_off;
            const int r_lo = std::max(row0, 0);
            const int n_rows = std::max(std::min(row0 + tile_rows(th), t.src_rows) - r_lo, 0);
            if (((int64_t)r_lo * t.src_cols) % v || ((int64_t)n_rows * t.src_cols) % v) return false;
            const int l0 = first * t.lin_rpc;
            const int ln = std::min(nrows * t.lin_rpc, t.lin_rows - l0);
            if (((int64_t)l0 * t.lin_cols) % v || ((int64_t)ln * t.lin_cols) % v) return false;
        }
        return true;
    };
    const int forced_vec = env_int("DDF_TUNE_VEC", 0);
    const int forced_ps = env_int("DDF_TUNE_PS", 0);

    // Candidates: 4 or 8 slots per lane.  Cost ~ slots walked (idle lanes
    // included) plus the halo rows re-staged per strip.
    double best = 1e30;
    int best_ps = 0, best_th = 0, best_v = 0, best_nv = 0;
    // slots per lane: 4 or 8; the filter-gradient kernel keeps two register
    // sets per slot and is built for 4 (k=3) or 2 (k=5) only
    const bool fused = kind == kWaveFused;   // filter gradients + feature gradient in one kernel
    const bool filters = kind == kWaveFilters || fused;
    const int ps_lo = filters ? (p.kk > 9 ? 2 : 4) : 4;
    // 25 taps: the spatial-filter registers of 8 slots would leave one wave per SIMD
    const int ps_hi = filters ? ps_lo : (p.kk > 9 ? 4 : kMaxSlots);
    for (int ps = ps_lo; ps <= ps_hi; ps *= 2) {
        if (forced_ps && !filters && ps != forced_ps) continue;
        if (ps < cseg) continue;
        // cell rows per strip: as many slot rows as the lane's slots allow,
        // fewer when the source strip would not fit the staging registers
        const int forced_th = env_int("DDF_TUNE_TH", 0);
        int th = 0, v = 1, nv = 0;
        for (int srows = ps / cseg; srows >= 1 && nv == 0; --srows) {
            th = std::min(srows * RS, t.rows);
            if (forced_th) th = std::min(th, forced_th);
            v = (dtype != DDF_F64 && vec_ok(4, th)) ? 4 : 1;
            if (forced_vec) v = std::min(v, forced_vec);
            if (max_vec) v = std::min(v, max_vec);
            const int staged = std::min(tile_rows(th), t.src_rows) * t.src_cols;
            const int need_nv = (staged + v * kWave - 1) / (v * kWave);
            for (int cand : {1, 2, 4, 8})
                if (cand >= need_nv) { nv = cand; break; }
            // instantiated: V=4 with (ps 2|4: nv 1, 2, 4; ps 8: nv 4); V=1 with (ps 4: nv 4, 8; ps 2: nv 4)
            if (nv == 0) continue;   // more than 8 vectors per lane: try fewer rows
            if (v == 4) {
                if (nv == 8) nv = 0;
                else if (ps == 8) nv = 4;
            } else {
                if (ps == 8) nv = 0;
                else nv = std::max(nv, 4);
                if (ps == 2 && nv == 8) nv = 0;
            }
        }
        if (nv == 0) continue;
        const int nstrips = (t.rows + th - 1) / th;
        const int64_t lds = (int64_t)asz * (2 * round_up(tile_rows(th) * t.P, 8) + wave::kSpare) +
                            (int64_t)esz * (wave::kIdle + round_up(th * t.lin_rpc * t.lin_cols, 8)) + 4096;
        if (lds > 64 * 1024) continue;
        const int slots_used = ((th + RS - 1) / RS) * cseg;
        double cost = (double)nstrips * (slots_used * kWave * 2.0 * p.kk +
                                         (double)tile_rows(th) * t.P * 3.0 + 150.0);
        if (v == 1) cost *= 1.3;
        if (ps == 8) cost *= 1.05;  // register pressure
        if (cost < best) { best = cost; best_ps = ps; best_th = th; best_v = v; best_nv = nv; }
    }
    if (best_ps == 0) return false;
    // The fused kernel is built for strips of one 16-byte vector per lane only:
    // with longer strips its registers leave no room to prefetch, and two
    // launches are faster.
    if (fused && !(best_v == 4 && best_nv == 1)) return false;
    t.TH = best_th;
    t.nstrips = (t.rows + t.TH - 1) / t.TH;
    t.nslots = ((t.TH + RS - 1) / RS) * cseg;
    for (int m = 0; m < kMaxSlots; ++m) {
        t.slot_row[m] = m < t.nslots ? (m / cseg) * RS : 0;
        t.slot_col[m] = m < t.nslots ? (m % cseg) * LW : 0;
    }
    t.IH = tile_rows(t.TH);
    {
        // farthest element any lane (idle ones included) reads: last slot row,
        // last lane column, last tap
        const int step = kind == kWaveFeatures ? 1 : S;
        const int last_row = (t.slot_row[t.nslots - 1] + RS - 1) * step;
        const int last_col = (t.slot_col[t.nslots - 1] + LW - 1) * step;
        const int reach = kind == kWaveFeatures ? halo_lo + halo_hi : (K - 1) * D;
        const int extent = (last_row + reach) * t.P + last_col + reach + 1 + t.lb_shift;
        t.tile = round_up(std::max(t.IH * t.P, extent), 8);
    }
    t.lin_tile = round_up(t.TH * t.lin_rpc * t.lin_cols, 8);
    t.vec = best_v;
    t.wide = (can_widen && best_v == 4) ? 1 : 0;
    t.nv = best_nv;

    // Channels per wave: enough waves to fill the machine several times over,
    // long enough walks to amortise the spatial-filter registers.
    const int waves_per_block = filters ? wave::kFilterWaves : 1;
    const int64_t base = p.N * t.nstrips;
    const int target = env_int(filters ? "DDF_TUNE_WAVES_FILTERS" : "DDF_TUNE_WAVES",
                               filters ? 2048 : 4096);
    const int64_t want_split = std::max<int64_t>(1, (target + base - 1) / base);
    int cpw = (int)((C + want_split - 1) / want_split);
    cpw = std::max(cpw, std::min(C, env_int("DDF_TUNE_MIN_CPW", 4)));
    const int forced_cpw = env_int(filters ? "DDF_TUNE_CPW_FILTERS" : "DDF_TUNE_CPW", 0);
    if (forced_cpw) cpw = std::min(forced_cpw, C);
    cpw = std::max(1, std::min(cpw, wave::kTapLoads * kWave / p.kk));  // taps staged in one go
    t.cpw = cpw;
    t.cpb = cpw * waves_per_block;
    t.csplit = (C + t.cpb - 1) / t.cpb;
    // per wave: tiles, then the channel-filter taps of its channels (accumulator type)
    // per wave: tile (accumulator type), linear strip (storage type), taps
    t.lds_wave_bytes = round_up((fused ? 2 : 1) * (t.tile + wave::kSpare) * asz +
                                (t.lin_tile + wave::kIdle) * esz +
                                cpw * ((p.kk + 3) / 4 * 4) * asz, 16);
    // Forward and feature gradient: several independent waves share a workgroup
    // (workgroups are dispatched at a limited rate; waves of one start together).
    t.wpb = 1;
    if (!filters) {
        t.wpb = std::max(1, std::min(env_int("DDF_TUNE_WPB", 1), wave::kMaxWpb));
        while (t.wpb > 1 && t.lds_wave_bytes * t.wpb > 48 * 1024) --t.wpb;
    }
    t.lds_bytes = t.lds_wave_bytes * (filters ? waves_per_block : t.wpb);
    if (fused)    // the spatial-filter tiles shared by the block's waves
        t.lds_bytes += p.kk * (t.tile + wave::kSpare) * asz;
    if (filters)  // the cross-wave sum of the dSF accumulators reuses the block's LDS
        t.lds_bytes = std::max(t.lds_bytes, waves_per_block * p.kk * kWave * acc_size(dtype));
    if (t.lds_bytes > 64 * 1024) return false;
    t.src_magic = t.src_cols == 1 ? 0u : (unsigned)((0x100000000ull + t.src_cols - 1) / t.src_cols);
    const int64_t nblocks = base * t.csplit;
    if (nblocks > (1 << 30)) return false;
    // magic-number division of the block id is exact while id * divisor < 2^32
    if (nblocks * std::max(t.csplit, t.nstrips) >= (1ll << 32)) return false;
    auto magic = [](int d) { return d == 1 ? 0u : (unsigned)((0x100000000ull + d - 1) / d); };
    t.csplit_magic = magic(t.csplit);
    t.nstrips_magic = magic(t.nstrips);
    const int64_t ngroups = (nblocks + t.wpb - 1) / t.wpb;   // workgroups launched
    t.xcd_per = (unsigned)((ngroups + wave::kXcd - 1) / wave::kXcd);
    t.nblocks = (int)nblocks;
    *g = t;
    *ps_out = best_ps;
    *nv_out = best_nv;
    return true;
}

// (either family covers the problem; what one of them lacks at run time - a
// shape, an alignment - the launch code takes to the other or to the generic kernels)
bool tiled_forward_supported(const Problem &p, int dtype) {
    WaveGeom g; int ps, nv;
    RowsGeom rg; int vx, r;
    return wave_geometry(p, dtype, kWaveForward, 0, &g, &ps, &nv) ||
           (dtype != DDF_F64 && rows_geometry(p, dtype, 0, &rg, &vx, &r));
}

bool tiled_backward_supported(const Problem &p, int dtype) {
    WaveGeom w; int ps, nv;
    return (wave_geometry(p, dtype, kWaveFeatures, 0, &w, &ps, &nv) &&
            wave_geometry(p, dtype, kWaveFilters, 0, &w, &ps, &nv)) ||
           (dtype != DDF_F64 && rows_cover_backward(p, dtype));
}

// Workspace layout: [dSF partials over channel splits][dCF partials over strips],
// each in the accumulator type and starting on a 256-byte boundary.
size_t tiled_backward_workspace(const Problem &p, int dtype, unsigned need) {
    if (!(need & (DDF_NEED_DCF | DDF_NEED_DSF))) return 0;
    // whichever family runs (it depends on pointer alignment too) finds room
    return std::max(wave_backward_workspace(p, dtype, need), rows_filters_workspace(p, dtype, need));
}

size_t wave_backward_workspace(const Problem &p, int dtype, unsigned need) {
    // csplit and nstrips do not depend on the access width, so the scalar
    // fallback for misaligned pointers needs the same workspace
    WaveGeom g; int ps, nv;
    if (!wave_geometry(p, dtype, kWaveFilters, 0, &g, &ps, &nv)) return 0;
    const size_t asz = acc_size(dtype);
    size_t bytes = 0;
    if ((need & DDF_NEED_DSF) && g.csplit > 1)
        bytes += ((size_t)p.N * g.csplit * p.kk * p.Ho * p.Wo * asz + 255) / 256 * 256;
    if ((need & DDF_NEED_DCF) && g.nstrips > 1)
        bytes += ((size_t)p.N * p.C * g.nstrips * p.kk * asz + 255) / 256 * 256;
    return bytes;
}

}  // namespace ddf
