// Host-side geometry of the row-register kernels: elements per lane and row,
// rows per lane, how lanes are laid over a strip and how many channels a wave
// walks.
#include <algorithm>

#include "ddf_rows_taprow.h"

namespace ddf {

int tune_int(const char *name, int fallback);

namespace {

constexpr int kRowsStages = 3;   // channels in flight per wave of k_rows (rows::kStages)
constexpr int kMaxRowLanes = 32;  // lanes per image row before the row is cut into segments

unsigned magic_of(int d) { return d == 1 ? 0u : (unsigned)((0x100000000ull + d - 1) / d); }

// Lanes over a strip: lpr = W / vx lanes per image row, rg row groups of R rows
// per wave, strips of even height.  Where it costs no row group, every image
// row is followed by an idle lane (lane pitch lpr + 1): its loads return zero,
// which is exactly what the neighbour shift must bring in at the row ends.
void lay_out_lanes(RowsGeom *t, int H, int W, int vx, int R) {
    t->segs = t->seg_out = 0;
    t->segs_magic = 0;
    if (W / vx > kMaxRowLanes) {
        // an image row is longer than the lanes of a wave take: even segments of at
        // most 62 vectors, each with a vector of its neighbours on either side
        const int vectors = W / vx;
        t->segs = (vectors + kWave - 3) / (kWave - 2);
        t->seg_out = (vectors + t->segs - 1) / t->segs;
        t->segs_magic = magic_of(t->segs);
        t->lpr = t->lp = t->seg_out + 2;
        t->lp_magic = magic_of(t->lp);
        t->rg = 1;
        t->rps = R;
        t->nstrips = ((H + R - 1) / R) * t->segs;
        return;
    }
    t->lpr = W / vx;
    const int row_units = (H + R - 1) / R;                  // lane-sized row groups of the plane
    const int fit_plain = std::min(kWave / t->lpr, row_units);
    const int fit_padded = std::min((kWave + 1) / (t->lpr + 1), row_units);
    auto strips_with = [&](int fit) { return fit > 0 ? (row_units + fit - 1) / fit : 1 << 30; };
    const bool pad = fit_padded > 0 && strips_with(fit_padded) <= strips_with(fit_plain) &&
                     tune_int("DDF_TUNE_ROWS_PAD", 1) != 0;
    t->lp = t->lpr + (pad ? 1 : 0);
    t->lp_magic = magic_of(t->lp);
    const int rg_max = pad ? fit_padded : fit_plain;
    t->nstrips = (row_units + rg_max - 1) / rg_max;
    t->rg = (row_units + t->nstrips - 1) / t->nstrips;      // even strips
    t->rps = t->rg * R;
}

// Channels per wave of k_rows: enough waves to fill the machine (and to even out
// its SIMDs), walks long enough to amortise the spatial-filter registers.  The
// kernels walk whole rounds of `nst` channels, so the count is a multiple of
// that.  `plane`: pixels of a result plane; `min_walk`: shortest walk worth the
// prologue (0: two rounds).
bool cut_channels_forward(RowsGeom &t, int64_t N, int C, int nst, int64_t plane, int min_walk = 0) {
    const int64_t base = N * t.nstrips;
    const int target = tune_int("DDF_TUNE_ROWS_WAVES", 8192);
    const int64_t want_split = std::max<int64_t>(1, (target + base - 1) / base);
    int cpw = (int)(C / want_split);
    // Small planes (up to 32 x 32) walk more rounds where that still leaves a wave per
    // SIMD: the spatial taps a wave loads first are paid for once per walk.  Measured with
    // operands that really come from memory (fp16 and fp32, batches of 8 to 256): planes
    // up to 16 x 16 want walks of 12 channels once those leave a thousand waves (10-15 %
    // over walks of 6) and of 24 once those leave some three thousand (7-9 % more); planes
    // up to 32 x 32 want the longest of 18, 12 and 9 that leaves a thousand (6-11 % over
    // 12 at 28 x 28).  Larger planes and small batches lose by longer walks.
    auto waves_with = [&](int rnds) { return base * ((C + rnds * nst - 1) / (rnds * nst)); };
    int rounds = 2;
    if (plane <= 256) {
        if (waves_with(8) >= 2816) rounds = 8;
        else if (waves_with(4) >= 1024) rounds = 4;
    } else if (plane <= 1024) {
        if (waves_with(6) >= 1024) rounds = 6;
        else if (waves_with(4) >= 1024) rounds = 4;
        else if (waves_with(3) >= 900) rounds = 3;
    }
    const int min_cpw = tune_int("DDF_TUNE_ROWS_MIN_CPW", std::max(rounds * nst, (min_walk + nst - 1) / nst * nst));
    cpw = std::max(cpw / nst * nst, min_cpw);
    const int forced = tune_int("DDF_TUNE_ROWS_CPW", 0);
    if (forced) cpw = forced;
    t.cpw = std::max(1, std::min(cpw, C));
    t.cpb = t.cpw;
    t.csplit = (C + t.cpw - 1) / t.cpw;
    // (single-wave workgroups spread over the machine faster: what counts for the
    // smallest launches)
    t.wpb = std::max(1, std::min(tune_int("DDF_TUNE_ROWS_WPB", plane <= 256 ? 1 : 2), rows::kMaxWpb));
    const int64_t nwork = base * t.csplit;
    if (nwork > (1 << 30)) return false;
    // magic-number division of the work id is exact while id * divisor < 2^32
    if (nwork * std::max(t.csplit, t.nstrips) >= (1ll << 32)) return false;
    t.csplit_magic = magic_of(t.csplit);
    t.nstrips_magic = magic_of(t.nstrips);
    const int64_t ngroups = (nwork + t.wpb - 1) / t.wpb;
    t.xcd_per = (unsigned)((ngroups + rows::kXcd - 1) / rows::kXcd);
    t.nwork = (int)nwork;
    return true;
}

// Channels per wave of k_rows_filters: the four waves of a workgroup cover cpb =
// 4 * cpw channels; enough workgroups to fill the machine, as few channel splits
// (dSF partial sums through the workspace) as that allows.
bool cut_channels_filters(RowsGeom &t, int64_t N, int C) {
    const int64_t base = N * t.nstrips;
    const int target = tune_int("DDF_TUNE_ROWSF_WAVES", 2048);
    const int64_t want_split = std::max<int64_t>(1, (target + base * rows::kFilterWaves - 1) /
                                                        (base * rows::kFilterWaves));
    // Channels per wave for `split` channel ranges: whole rounds of the kernel's channel
    // pipeline and whole dCF flush groups.
    auto cpw_of = [&](int64_t split) {
        const int cpb = (int)((C + split - 1) / split);
        int w = (cpb + rows::kFilterWaves - 1) / rows::kFilterWaves;
        w = (w + rows::kFlushChannels - 1) / rows::kFlushChannels * rows::kFlushChannels;
        return std::max(w, tune_int("DDF_TUNE_ROWSF_MIN_CPW", 2 * rows::kFlushChannels));
    };
    // One split fewer where that turns a ragged second round of waves into a single round
    // of longer walks (rounds of `target` resident waves times channels per wave is what
    // the launch takes): 32 x 128 x 56 x 56 at stride 2 runs 1 792 waves of 16 channels
    // 5 % faster than 2 688 of 12.
    auto cost_of = [&](int w) {
        const int64_t waves = base * rows::kFilterWaves * ((C + (int64_t)w * rows::kFilterWaves - 1) / ((int64_t)w * rows::kFilterWaves));
        return ((waves + target - 1) / target) * w;
    };
    int cpw = cpw_of(want_split);
    if (want_split > 1 && cost_of(cpw_of(want_split - 1)) < cost_of(cpw)) cpw = cpw_of(want_split - 1);
    const int forced = tune_int("DDF_TUNE_ROWSF_CPW", 0);
    if (forced) cpw = std::min(forced, C);
    t.cpw = std::max(1, cpw);
    t.cpb = t.cpw * rows::kFilterWaves;
    t.csplit = (C + t.cpb - 1) / t.cpb;
    t.wpb = 1;
    const int64_t nwork = base * t.csplit;
    if (nwork > (1 << 30)) return false;
    if (nwork * std::max(t.csplit, t.nstrips) >= (1ll << 32)) return false;
    t.csplit_magic = magic_of(t.csplit);
    t.nstrips_magic = magic_of(t.nstrips);
    t.xcd_per = (unsigned)((nwork + rows::kXcd - 1) / rows::kXcd);
    t.nwork = (int)nwork;
    return true;
}

// Stride 2 (3 x 3, fp16 / fp32): lanes over the result plane, one row per lane,
// vx result pixels per lane from feature vectors of 2 * vx elements.  Rows of
// the feature plane must keep those vectors aligned (W a multiple of 2 * vx) and
// a result row must fit the lanes of a wave.  filters: the cut of
// k_rows_filters, else of k_rows.
bool stride2_geometry(const Problem &p, int dtype, bool filters, int max_vx, RowsGeom *g,
                      int *vx_out, int *r_out) {
    if (!(p.s == 2 && p.k == 3 && p.d == 1)) return false;
    if (dtype != DDF_F16 && dtype != DDF_F32) return false;
    if (p.N <= 0 || p.C <= 0 || p.Ho <= 0 || p.Wo <= 0) return false;
    if (p.H > 16384 || p.W > 16384 || p.C > (1 << 24) || p.N > (1 << 24)) return false;
    const int esz = dtype == DDF_F16 ? 2 : 4;
    const int H = (int)p.H, W = (int)p.W, Ho = (int)p.Ho, Wo = (int)p.Wo, C = (int)p.C;
    if ((int64_t)H * W * 8 >= (1ll << 31)) return false;   // byte offsets inside a plane are 32-bit
    // A lane's feature vectors are 2 * vx elements: 16 bytes at most, so that one load
    // or store instruction covers its rows without gaps.  (Vectors of 32 bytes go out as
    // two instructions that each touch every other 16 bytes: measured 7 % slower forward,
    // 9 % backward and 55 % for the feature gradient alone at 32 x 128 x 56 x 56 fp32.)
    int vx = 0;
    for (int cand = 8 / esz; cand >= 1; cand /= 2) {
        if (cand > tune_int("DDF_TUNE_ROWS_VX", 16) || cand > max_vx) continue;
        if (W % (2 * cand) != 0) continue;
        vx = cand;
        break;
    }
    if (vx == 0 || Wo / vx > kMaxRowLanes) return false;
    RowsGeom t{};
    t.C = C; t.H = Ho; t.W = Wo; t.Hi = H; t.Wi = W;
    lay_out_lanes(&t, Ho, Wo, vx, 1);
    if (filters ? !cut_channels_filters(t, p.N, C)
                : !cut_channels_forward(t, p.N, C, kRowsStages, (int64_t)Ho * Wo))
        return false;
    *g = t;
    *vx_out = vx;
    *r_out = 1;
    return true;
}

}  // namespace

// Instantiated (elements per lane and row, rows per lane) per element size.
bool rows_variant_built(int esz, int vx, int r) {
    if (esz == 2) return (r == 1 && (vx == 8 || vx == 4 || vx == 2 || vx == 1)) || (r == 2 && (vx == 8 || vx == 4 || vx == 2));
    if (esz == 4) return (r == 1 && (vx == 4 || vx == 2 || vx == 1)) || (r == 2 && (vx == 2 || vx == 4));
    return false;
}

// (stride 2: the forward pass only)
bool rows_shape_built(int k, int d, int s) {
    return (s == 1 && (k == 3 || k == 5) && (d == 1 || d == 2)) || (s == 2 && k == 3 && d == 1);
}

bool rows_geometry(const Problem &p, int dtype, int max_vx, RowsGeom *g, int *vx_out, int *r_out) {
    if (!rows_shape_built(p.k, p.d, p.s)) return false;
    if (p.s == 2) return max_vx <= 0 && stride2_geometry(p, dtype, false, 16, g, vx_out, r_out);
    if (p.N <= 0 || p.C <= 0 || p.H <= 0 || p.W <= 0) return false;
    if (p.H > 16384 || p.W > 16384 || p.C > (1 << 24) || p.N > (1 << 24)) return false;
    const int esz = dtype == DDF_F16 ? 2 : dtype == DDF_F32 ? 4 : 8;
    const int H = (int)p.H, W = (int)p.W, C = (int)p.C;
    const int hx = p.r * p.d;
    if ((int64_t)H * W * esz >= (1ll << 31)) return false;   // byte offsets inside a plane are 32-bit
    // widest vector the row length allows, at most 32 lanes per image row
    int vx = 0;
    for (int cand = 16 / esz; cand >= 1; cand /= 2) {
        if (max_vx > 0 && cand > max_vx) continue;
        if (cand > tune_int("DDF_TUNE_ROWS_VX", 16)) continue;
        if (W % cand != 0 || cand < hx) continue;
        vx = cand;
        break;
    }
    if (vx == 0) return false;
    // One row per lane keeps the registers low enough for 4-5 waves per SIMD,
    // which is what the larger planes want.  Small planes whose rows are a few
    // two-pixel vectors (14 x 14, 30 x 30) take two rows per lane: fewer strips
    // per plane, and the shorter prologue matters more there.
    // (fp16 rows of a few 4-pixel vectors as well - 28 x 28: 8-byte accesses, and half the
    // loads and neighbour shifts per pixel: 10 % faster)
    int R = ((vx == 2 || (esz == 2 && vx == 4)) && H % 2 == 0 && H * W <= 1024) ? 2 : 1;
    // Large planes stream from HBM and a lane's halo rows come in through the
    // L1 once more per row group: two rows per lane of full 16-byte vectors read
    // four rows for two instead of three for one (built for 3x3 without dilation).
    if (vx * esz == 16 && p.k == 3 && p.d == 1 && H * W >= 112 * 112) R = 2;
    R = tune_int("DDF_TUNE_ROWS_R", R);
    if (p.k == 5) {   // 25 taps: built for one row per lane and vectors of four pixels or more
        R = 1;
        if (vx < 4) return false;
    }
    if (!rows_variant_built(esz, vx, R)) return false;

    RowsGeom t{};
    t.C = C; t.H = t.Hi = H; t.W = t.Wi = W;
    lay_out_lanes(&t, H, W, vx, R);

    // (25 spatial taps per pixel to load before the walk: 32 pixel-channels per lane at least)
    if (!cut_channels_forward(t, p.N, C, p.k == 5 ? 2 : kRowsStages, (int64_t)H * W, p.k == 5 ? 32 / vx : 0))
        return false;
    *g = t;
    *vx_out = vx;
    *r_out = R;
    return true;
}

// Instantiated (elements per lane and row, rows per lane) of k_rows_filters;
// fused: of the variant that also writes the feature gradient.
bool rows_filters_variant_built(int esz, int vx, int r, bool fused) {
    if (esz != 2 && esz != 4) return false;
    if (vx == 1) return r == 1;   // odd row lengths: one pixel per lane
    if (fused) return (vx == 2 && r == 2) || (vx == 4 && r == 1);
    return r == 1 && (vx == 4 || vx == 2);
}

bool rows_filters_geometry(const Problem &p, int dtype, bool fused, RowsGeom *g, int *vx_out,
                           int *r_out) {
    // (stride 2, one launch for the whole backward pass: every feature row must be some
    // lane's 2y or 2y + 1, so the height is even; the width already is)
    if (p.s == 2)
        return (!fused || (p.H % 2 == 0 && tune_int("DDF_TUNE_ROWSF_FUSED", 1) != 0)) &&
               stride2_geometry(p, dtype, true, 16, g, vx_out, r_out);
    if (!(p.s == 1 && p.k == 3 && (p.d == 1 || p.d == 2))) return false;
    if (p.N <= 0 || p.C <= 0 || p.H <= 0 || p.W <= 0) return false;
    if (p.H > 16384 || p.W > 16384 || p.C > (1 << 24) || p.N > (1 << 24)) return false;
    const int esz = dtype == DDF_F16 ? 2 : dtype == DDF_F32 ? 4 : 8;
    const int H = (int)p.H, W = (int)p.W, C = (int)p.C;
    const int hx = p.r * p.d;
    if ((int64_t)H * W * 8 >= (1ll << 31)) return false;   // byte offsets inside a plane are 32-bit
    // One launch for the whole backward pass: dO, CF and SF are read once.  It is
    // the faster route at every plane size measured (7 x 7 to 200 x 300).
    if (fused && (H * W > tune_int("DDF_TUNE_ROWSF_FUSED_PLANE", 1 << 30) ||
                  tune_int("DDF_TUNE_ROWSF_FUSED", 1) == 0))
        return false;
    int vx = 0, R = 1;
    for (int cand = std::min(16 / esz, 4); cand >= 1; cand /= 2) {
        if (cand > tune_int("DDF_TUNE_ROWSF_VX", 16)) continue;
        if (W % cand != 0 || cand < hx) continue;
        // two rows per lane where a row is a few 2-pixel vectors (14 x 14: one strip per plane)
        const int r = (fused && cand == 2 && H % 2 == 0 && p.d == 1) ? 2 : 1;
        if (!rows_filters_variant_built(esz, cand, r, fused)) continue;
        vx = cand;
        R = r;
        break;
    }
    if (vx == 0) return false;

    RowsGeom t{};
    t.C = C; t.H = t.Hi = H; t.W = t.Wi = W;
    lay_out_lanes(&t, H, W, vx, R);

    if (!cut_channels_filters(t, p.N, C)) return false;
    *g = t;
    *vx_out = vx;
    *r_out = R;
    return true;
}

// Built: 5 x 5 filters (and, as a tuning alternative, 3 x 3 without dilation).
bool rows_taprow_shape_built(int k, int d, int s) {
    if (s != 1) return false;
    if (k == 5) return d == 1 || d == 2;
    return k == 3 && d == 1 && tune_int("DDF_TUNE_TAPROW_K3", 0) != 0;
}

bool rows_taprow_geometry(const Problem &p, int dtype, RowsGeom *g, int *vx_out, int *r_out) {
    if (!rows_taprow_shape_built(p.k, p.d, p.s)) return false;
    if (p.N <= 0 || p.C <= 0 || p.H <= 0 || p.W <= 0) return false;
    if (p.H > 16384 || p.W > 16384 || p.C > (1 << 24) || p.N > (1 << 24)) return false;
    if (dtype != DDF_F16 && dtype != DDF_F32) return false;
    const int esz = dtype == DDF_F16 ? 2 : 4;
    const int H = (int)p.H, W = (int)p.W, C = (int)p.C;
    const int hx = p.r * p.d;
    if ((int64_t)H * W * 8 >= (1ll << 31)) return false;   // byte offsets inside a plane are 32-bit
    // Widest vector that still leaves enough workgroups; below that, channel
    // splits (dSF partial sums through the workspace) make up the number.
    const int target = tune_int("DDF_TUNE_TAPROW_WAVES", 2048);
    RowsGeom t{};
    int vx = 0;
    for (int cand = 16 / esz; cand * esz >= 4; cand /= 2) {
        if (cand > tune_int("DDF_TUNE_TAPROW_VX", 16)) continue;
        if (W % cand != 0 || cand < hx || cand < 2) continue;
        RowsGeom c{};
        c.C = C; c.H = c.Hi = H; c.W = c.Wi = W;
        lay_out_lanes(&c, H, W, cand, 1);
        t = c;
        vx = cand;
        if (p.N * c.nstrips * p.k >= target) break;
    }
    if (vx == 0) return false;
    const int flush = p.k <= 4 ? rows::taprow_flush_channels<3>() : rows::taprow_flush_channels<5>();
    const int64_t base = p.N * t.nstrips;
    const int64_t want_split = std::max<int64_t>(1, (target + base * p.k - 1) / (base * p.k));
    int cpw = (int)((C + want_split - 1) / want_split);
    cpw = (cpw + flush - 1) / flush * flush;   // whole flush groups (and pipeline rounds)
    cpw = std::max(cpw, tune_int("DDF_TUNE_TAPROW_MIN_CPW", 2 * flush));
    const int forced = tune_int("DDF_TUNE_TAPROW_CPW", 0);
    if (forced) cpw = forced;
    t.cpw = std::max(1, std::min(cpw, C));
    t.cpb = t.cpw;
    t.csplit = (C + t.cpw - 1) / t.cpw;
    t.wpb = rows::kTaprowWaves;
    const int64_t nwork = base * t.csplit * p.k;   // one wave per filter row
    if (nwork > (1 << 30)) return false;
    if (nwork * std::max(t.csplit, t.nstrips) >= (1ll << 32)) return false;
    t.csplit_magic = magic_of(t.csplit);
    t.nstrips_magic = magic_of(t.nstrips);
    const int64_t ngroups = (nwork + t.wpb - 1) / t.wpb;
    t.xcd_per = (unsigned)((ngroups + rows::kXcd - 1) / rows::kXcd);
    t.nwork = (int)nwork;
    *g = t;
    *vx_out = vx;
    *r_out = 1;
    return true;
}

bool rows_cover_backward(const Problem &p, int dtype) {
    RowsGeom g; int vx, r;
    return p.s == 1 && rows_geometry(p, dtype, 0, &g, &vx, &r) &&
           (rows_taprow_geometry(p, dtype, &g, &vx, &r) ||
            rows_filters_geometry(p, dtype, false, &g, &vx, &r));
}

bool rows_cover_stride2_filters(const Problem &p, int dtype) {
    RowsGeom g; int vx, r;
    return p.s == 2 && rows_filters_geometry(p, dtype, false, &g, &vx, &r);
}

size_t rows_filters_workspace(const Problem &p, int dtype, unsigned need) {
    if (!(need & (DDF_NEED_DCF | DDF_NEED_DSF))) return 0;
    const size_t asz = dtype == DDF_F64 ? 8 : 4;
    size_t most = 0;
    // (room for either cut of the problem: which one runs also depends on pointer alignment)
    for (int cut = 0; cut < 3; ++cut) {
        RowsGeom g; int vx, r;
        if (cut == 1 && !(need & DDF_NEED_DX)) continue;
        if (cut < 2 ? !rows_filters_geometry(p, dtype, cut != 0, &g, &vx, &r)
                    : !rows_taprow_geometry(p, dtype, &g, &vx, &r))
            continue;
        size_t bytes = 0;
        if ((need & DDF_NEED_DSF) && g.csplit > 1)
            bytes += ((size_t)p.N * g.csplit * p.kk * p.Ho * p.Wo * asz + 255) / 256 * 256;
        if ((need & DDF_NEED_DCF) && g.nstrips > 1)
            bytes += ((size_t)p.N * p.C * g.nstrips * p.kk * asz + 255) / 256 * 256;
        most = std::max(most, bytes);
    }
    return most;
}

}  // namespace ddf
