// CPU model of the wave kernels' addressing.  For a list of problem shapes it asks the
// library's own host code (ddf_tiled_host.hip, compiled into this program) for the launch
// geometry and replays, lane by lane, every global and LDS address the kernels form from
// it: vector offsets of the staged strips, tile offsets, the tap reach of every cell slot,
// result strips, the block-id split, the LDS layout.  Prints one line per geometry and a
// VIOLATION line for anything out of bounds or misaligned.  Built and run by
// tests/test_geometry.py; no kernel is launched.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "ddf_tiled_host.hip"
#include "ddf_rows_host.hip"
#include "ddf_chunks.h"

using namespace ddf;

static int g_fails = 0;
#define CHECK(cond, ...)                      \
    do {                                      \
        if (!(cond)) {                        \
            if (g_fails < 10) {               \
                printf("  VIOLATION: ");      \
                printf(__VA_ARGS__);          \
                printf("\n");                 \
            }                                 \
            ++g_fails;                        \
        }                                     \
    } while (0)

static bool is_filters(int kind) { return kind == kWaveFilters || kind == kWaveFused; }

// floor(n / d) through the magic number the kernels use (0 means d == 1)
static long magic_div(long n, unsigned m) {
    return m ? (long)(((unsigned long long)(unsigned)n * m) >> 32) : n;
}

static void check_geometry(int kind, long N, long C, long H, long W, int k, int d, int s, int dtype,
                           int max_vec) {
    const Problem p = make_problem(N, C, H, W, k, d, s, 0);
    WaveGeom g;
    int ps, nv;
    if (!wave_geometry(p, dtype, kind, max_vec, &g, &ps, &nv)) {
        printf("kind %d %ldx%ldx%ldx%ld k%d d%d s%d dt%d: unsupported\n", kind, N, C, H, W, k, d, s,
               dtype);
        return;
    }
    const int esz = dtype == 0 ? 2 : dtype == 1 ? 4 : 8, asz = dtype == 2 ? 8 : 4;
    const int V = g.vec, KK = k * k, tap_pitch = (KK + 3) / 4 * 4;
    const int S = s, D = d, R = (k - 1) / 2;
    printf("kind %d %ldx%ldx%ldx%ld k%d d%d s%d dt%d: ps=%d nv=%d vec=%d wide=%d TH=%d nstrips=%d "
           "nslots=%d lw=%d P=%d IH=%d tile=%d lin_tile=%d cpw=%d cpb=%d wpb=%d csplit=%d "
           "nblocks=%d lds=%d (wave %d)\n",
           kind, N, C, H, W, k, d, s, dtype, ps, nv, V, g.wide, g.TH, g.nstrips, g.nslots,
           1 << g.lw_shift, g.P, g.IH, g.tile, g.lin_tile, g.cpw, g.cpb, g.wpb, g.csplit, g.nblocks,
           g.lds_bytes, g.lds_wave_bytes);

    CHECK(g.nslots <= ps, "nslots %d > ps %d", g.nslots, ps);
    const long tile_elems = (long)g.tile + 8;   // tile plus its spare elements
    const long plane_in = (long)g.src_rows * g.src_cols;
    const int LW = 1 << g.lw_shift;

    for (int strip = 0; strip < g.nstrips; ++strip) {
        const int row_first = strip * g.TH, nrows = std::min(g.TH, g.rows - row_first);

        // --- staged source strip: global vector offsets and tile offsets (Stager) ---
        const int row0 = (kind == kWaveFeatures ? row_first : row_first * S) + g.row0_off;
        const int r_lo = std::max(row0, 0);
        const int n_rows = std::max(std::min(row0 + g.IH, g.src_rows) - r_lo, 0);
        const int nvec = n_rows * g.src_cols / V, row_shift = r_lo - row0;
        CHECK((n_rows * g.src_cols) % V == 0, "strip %d: staged %d elements, not a multiple of V",
              strip, n_rows * g.src_cols);
        CHECK(nvec <= 64 * nv, "strip %d: %d vectors > 64 * nv (%d)", strip, nvec, 64 * nv);
        for (int lane = 0; lane < 64; ++lane)
            for (int j = 0; j < nv; ++j) {
                const int f = lane + 64 * j, e = f * V;
                if (f >= nvec) continue;
                int row = e / g.src_cols, col = e % g.src_cols;
                const long goff = (long)r_lo * g.src_cols + e;
                CHECK(goff + V <= plane_in, "strip %d: global source offset %ld + %d > plane %ld",
                      strip, goff, V, plane_in);
                CHECK((goff * esz) % (V * esz) == 0, "misaligned source vector");
                if (g.wide) {
                    const int lo0 = (row_shift + row) * g.P + g.col_off + col;
                    CHECK(V == 4, "wide commits need V = 4");
                    CHECK(lo0 % 4 == 0, "wide: tile offset %d not 16-byte aligned", lo0);
                    CHECK(col + 3 < g.src_cols, "wide: vector straddles two rows");
                }
                for (int q = 0; q < V; ++q) {
                    const int lo = (row_shift + row) * g.P + g.col_off + col;
                    CHECK(lo >= 0 && lo < g.tile, "strip %d: tile offset %d outside tile %d (row %d col %d)",
                          strip, lo, g.tile, row, col);
                    if (++col >= g.src_cols) { col = 0; ++row; }
                }
            }

        // --- cell slots: tap reach in the tile, position in the linear strip ---
        for (int lane = 0; lane < 64; ++lane) {
            const int lr = lane >> g.lw_shift, lc = lane & (LW - 1);
            for (int m = 0; m < g.nslots; ++m) {
                const int row = g.slot_row[m] + lr, col = g.slot_col[m] + lc;
                const bool ok = row < nrows && col < g.cols;
                const int step = kind == kWaveFeatures ? 1 : S;
                const int reach = kind == kWaveFeatures ? (R * D) / S + (R * D + S - 1) / S : (k - 1) * D;
                const long lb = (long)(row * step) * g.P + col * step + g.lb_shift;
                const long far = lb + (long)reach * g.P + reach;
                CHECK(far < tile_elems, "lane %d slot %d reads tile element %ld of %ld", lane, m, far,
                      tile_elems);
                if (!ok) continue;
                if (kind != kWaveFeatures) {
                    const long ob = (long)row * g.Wo + col;
                    CHECK(ob < g.lin_tile, "strip offset %ld >= lin_tile %d", ob, g.lin_tile);
                    CHECK((long)(row_first + row) * g.Wo + col < (long)g.Ho * g.Wo, "pixel outside plane");
                } else {
                    for (int a = 0; a < S; ++a)
                        for (int c = 0; c < S; ++c) {
                            const int u = (row_first + row) * S + a, v = col * S + c;
                            if (u >= g.H || v >= g.W) continue;
                            const long o = (long)(row * S + a) * g.W + v;
                            CHECK(o < g.lin_tile, "dX strip offset %ld >= lin_tile %d", o, g.lin_tile);
                        }
                }
            }
        }

        // --- result / linear strips: vector aligned, inside the plane, inside LDS ---
        CHECK(plane_in % V == 0, "source plane %ld not a multiple of V", plane_in);
        CHECK(((long)g.Ho * g.Wo) % V == 0, "output plane not a multiple of V");
        if (kind == kWaveForward) {
            const long n_out = (long)nrows * g.Wo;
            const int NG = (ps + V - 1) / V;
            CHECK(n_out % V == 0 && ((long)row_first * g.Wo) % V == 0, "output strip misaligned");
            CHECK(n_out / V <= 64 * NG, "%ld spatial-filter vectors > 64 * NG (%d)", n_out / V, 64 * NG);
            CHECK(n_out <= g.lin_tile, "output strip > lin_tile");
            CHECK((long)row_first * g.Wo + n_out <= (long)g.Ho * g.Wo, "output strip outside plane");
        }
        if (kind == kWaveFeatures) {
            const int u0 = row_first * S;
            const long n_out = (long)std::min(nrows * S, g.H - u0) * g.W;
            CHECK(n_out % V == 0 && ((long)u0 * g.W) % V == 0, "dX strip misaligned");
            CHECK((long)u0 * g.W + n_out <= (long)g.H * g.W, "dX strip outside plane");
            CHECK(n_out <= g.lin_tile, "dX strip %ld > lin_tile %d", n_out, g.lin_tile);
        }
        if (is_filters(kind)) {
            const long n_go = (long)nrows * g.Wo;
            const int NG = (ps + V - 1) / V;
            CHECK(n_go % V == 0, "dO strip misaligned");
            CHECK(n_go <= g.lin_tile, "dO strip > lin_tile");
            CHECK(n_go / V <= 64 * NG, "%ld dO vectors > 64 * NG (%d)", n_go / V, 64 * NG);
        }
    }

    // --- block id -> (sample, strip, channel split) through magic numbers ---
    const long step = g.nblocks > 200000 ? 97 : 1;
    for (long b = 0; b < g.nblocks; b += step) {
        const long rest = magic_div(b, g.csplit_magic), cs = b - rest * g.csplit;
        const long smp = magic_div(rest, g.nstrips_magic), strip = rest - smp * g.nstrips;
        CHECK(rest == b / g.csplit && cs == b % g.csplit && smp == rest / g.nstrips &&
                  strip == rest % g.nstrips,
              "block split wrong at block %ld", b);
    }
    CHECK(magic_div(g.nblocks - 1, g.csplit_magic) == (g.nblocks - 1) / g.csplit, "split of the last block");
    const long ngroups = ((long)g.nblocks + g.wpb - 1) / g.wpb;
    CHECK((long)g.xcd_per * 8 >= ngroups && (long)(g.xcd_per - 1) * 8 < ngroups, "workgroups per XCD");

    // --- LDS layout ---
    const int waves = is_filters(kind) ? 4 : g.wpb;
    const long used = (long)(g.tile + 8) * asz * (kind == kWaveFused ? 2 : 1) +
                      (long)(g.lin_tile + 64) * esz + (long)g.cpw * tap_pitch * asz;
    const long shared = kind == kWaveFused ? (long)KK * (g.tile + 8) * asz : 0;
    CHECK(used <= g.lds_wave_bytes, "a wave uses %ld bytes of LDS, has %d", used, g.lds_wave_bytes);
    CHECK(g.wpb >= 1 && g.wpb <= 4, "waves per workgroup %d", g.wpb);
    CHECK((long)g.lds_wave_bytes * waves + shared <= g.lds_bytes, "workgroup LDS");
    CHECK(g.lds_bytes <= 64 * 1024, "more than 64 KiB of LDS");
    CHECK(g.cpw * KK <= 256, "%d taps staged, at most 256", g.cpw * KK);
    CHECK((long)g.csplit * g.cpb >= C, "channels not covered");
    if (g_fails) printf("  -> %d violations\n", g_fails);
    g_fails = 0;
}

// Every work item mapped to its own (sample, strip, channel range[, tap row]), the
// channel ranges covering C, the workgroups dealt out evenly over the XCDs.
static void check_work_items(const RowsGeom &g, long N, long C, int kind, int taps) {
    const bool filters = kind == 1;
    const int per = kind == 2 ? taps : 1;   // waves (one per filter row) per (sample, strip, channel range)
    const long items = (long)N * g.nstrips * g.csplit * per;
    CHECK(items == g.nwork, "work items %d", g.nwork);
    CHECK((long)g.csplit * g.cpb >= C && (long)(g.csplit - 1) * g.cpb < C, "channel ranges");
    if (filters) CHECK(g.cpb == g.cpw * rows::kFilterWaves && g.wpb == 1, "filter workgroup shape");
    else if (kind == 2) CHECK(g.cpb == g.cpw && g.wpb == rows::kTaprowWaves, "tap-row workgroup shape");
    else CHECK(g.cpb == g.cpw && g.wpb >= 1 && g.wpb <= rows::kMaxWpb, "waves per workgroup");
    const long groups = (items + g.wpb - 1) / g.wpb;
    CHECK((long)g.xcd_per * 8 >= groups && (long)(g.xcd_per - 1) * 8 < groups, "workgroups per XCD");
    const long nblk = (long)g.xcd_per * 8;
    std::vector<char> seen(items, 0);
    const long stepb = nblk > 100000 ? 53 : 1;
    for (long blk = 0; blk < nblk; blk += stepb)
        for (int w = 0; w < g.wpb; ++w) {
            rows::Work wk;
            const int item = rows::Work::item_of(g, (int)blk, w);
            if (item < 0) continue;
            wk.decode(g, item / per);   // (as the kernels do)
            const long id = (((long)wk.n * g.nstrips + wk.strip) * g.csplit + wk.cs) * per + item % per;
            CHECK(wk.n < N && wk.strip < g.nstrips && wk.cs < g.csplit && id < items, "work item out of range");
            if (id < items) { CHECK(!seen[id], "work item %ld handed out twice", id); seen[id] = 1; }
            CHECK(wk.c_begin == wk.cs * g.cpb && wk.c_end <= C && wk.c_end > wk.c_begin, "channel range");
        }
    if (stepb == 1)
        for (long i = 0; i < items; ++i)
            if (!seen[i]) { CHECK(false, "work item %ld never handed out", i); break; }
}

// Row-register kernels (ddf_rows.h, ddf_rows_filters.h): the kernels ask rows::Lane and
// rows::Work - the very code compiled here - where a lane's vectors are, so the model runs
// that code for every lane of every strip and checks what the kernels rely on: offsets
// inside the plane and aligned to the vector (or -1: the access is given an offset outside
// the buffer descriptor), every pixel of the plane owned by exactly one lane, an idle lane
// after every image row in the padded layout, all lanes within the wavefront, every work
// item mapped to its own (sample, strip, channel range), the channel ranges covering C.
// kind 0: k_rows; 1: k_rows_filters (four waves of a workgroup split its channels);
// 2: k_rows_taprow_filters (K waves of a workgroup, wave i reads the feature rows
// (i - K/2) * D rows away: `taps` = K, `dil` = D).
template <int R, int HY, int VX>
static void replay_rows(const RowsGeom &g, long N, long C, int kind, int taps = 0, int dil = 0) {
    const bool filters = kind == 1;
    const long plane = (long)g.H * g.W;
    std::vector<int> owner(plane, 0);
    CHECK(g.lp == g.lpr || g.lp == g.lpr + 1, "lane pitch %d for %d lanes per row", g.lp, g.lpr);
    CHECK((long)(g.rg - 1) * g.lp + g.lpr <= 64, "row groups do not fit the wavefront");
    if (g.segs > 0)
        CHECK(g.seg_out >= 1 && g.seg_out <= 62 && g.lp == g.seg_out + 2 && g.rg == 1 &&
              (long)g.segs * g.seg_out * VX >= g.W && (long)(g.segs - 1) * g.seg_out * VX < g.W &&
              g.nstrips == ((g.H + R - 1) / R) * g.segs, "segments of an image row");
    else
        CHECK(g.lpr * VX == g.W, "lanes per row");
    for (int strip = 0; strip < g.nstrips; ++strip)
        for (int lane = 0; lane < 64; ++lane) {
            rows::Lane<R, HY, VX> ln;
            ln.init(g, strip, lane);
            const int grp = lane / g.lp, v = lane % g.lp;
            // first row of the lane and its vector's first column
            const int row0 = g.segs > 0 ? (strip / g.segs) * R : strip * g.rps + grp * R;
            const int col0 = g.segs > 0 ? ((strip % g.segs) * g.seg_out + lane - 1) * VX : v * VX;
            for (int rr = 0; rr < R + 2 * HY; ++rr) {
                const int off = ln.xoff[rr];
                if (off < 0) continue;
                CHECK(grp < g.rg && v < g.lpr, "idle lane %d with a live offset", lane);
                CHECK(off % VX == 0 && off + VX <= plane, "offset %d outside the plane or misaligned", off);
                const int yy = row0 - HY + rr;
                CHECK(col0 >= 0 && col0 + VX <= g.W && off == yy * g.W + col0,
                      "offset %d is not row %d column %d", off, yy, col0);
            }
            if (g.segs > 0) {
                // a lane that produces results has both neighbours' vectors in the wave
                // (or sits at an end of the image row)
                for (int r = 0; r < R; ++r)
                    if (ln.ooff[r] >= 0) CHECK(lane >= 1 && lane <= g.seg_out, "result in a halo lane %d", lane);
            }
            for (int r = 0; r < R; ++r)
                if (ln.ooff[r] >= 0)
                    for (int e = 0; e < VX; ++e) ++owner[ln.ooff[r] + e];
            if (g.lp > g.lpr && v == g.lpr)
                for (int rr = 0; rr < R + 2 * HY; ++rr) CHECK(ln.xoff[rr] < 0, "padding lane %d is live", lane);
            if (g.segs > 0) CHECK(!ln.first && !ln.last, "row ends");
            else CHECK(ln.first == (v == 0) && ln.last == (v == g.lpr - 1), "row ends");
            for (int i = 0; i < taps; ++i) {
                // the shifted window of wave i: same result rows, feature rows dy further down
                const int dy = (i - taps / 2) * dil;
                rows::Lane<R, HY, VX> sh;
                sh.init(g, strip, lane, dy);
                for (int r = 0; r < R; ++r) CHECK(sh.ooff[r] == ln.ooff[r], "result rows move with the tap row");
                for (int rr = 0; rr < R + 2 * HY; ++rr) {
                    const int off = sh.xoff[rr];
                    if (off < 0) continue;
                    const int yy = row0 - HY + rr + dy;
                    CHECK(grp < g.rg && v < g.lpr && yy >= 0 && yy < g.H && off == yy * g.W + col0,
                          "shifted offset %d is not row %d column %d", off, yy, col0);
                }
            }
        }
    for (long i = 0; i < plane; ++i)
        if (owner[i] != 1) { CHECK(false, "pixel %ld owned %d times", i, owner[i]); break; }
    check_work_items(g, N, C, kind, taps);
}

static void check_rows(long N, long C, long H, long W, int k, int d, int dtype, bool filters, bool fused = false,
                       bool taprow = false) {
    const Problem p = make_problem(N, C, H, W, k, d, 1, 0);
    RowsGeom g;
    int vx, r;
    const bool ok = taprow ? rows_taprow_geometry(p, dtype, &g, &vx, &r)
                  : filters ? rows_filters_geometry(p, dtype, fused, &g, &vx, &r)
                            : rows_geometry(p, dtype, 0, &g, &vx, &r);
    const char *name = taprow ? "-taprow" : filters ? "-filters" : "";
    if (!ok) {
        printf("kind rows%s %ldx%ldx%ldx%ld k%d d%d dt%d: unsupported\n", name, N, C, H, W, k, d, dtype);
        return;
    }
    printf("kind rows%s %ldx%ldx%ldx%ld k%d d%d dt%d: vx=%d r=%d lpr=%d lp=%d rg=%d rps=%d nstrips=%d cpw=%d cpb=%d "
           "csplit=%d wpb=%d nwork=%d\n", name, N, C, H, W, k, d, dtype, vx, r, g.lpr, g.lp,
           g.rg, g.rps, g.nstrips, g.cpw, g.cpb, g.csplit, g.wpb, g.nwork);
    if (taprow) {
        CHECK(dtype != 2 && r == 1, "tap-row kernel variant");
        CHECK((k / 2) * d <= vx, "taps reach beyond the neighbouring lane");
        const int lds = k == 3 ? rows::taprow_lds_bytes<3>(4) : rows::taprow_lds_bytes<5>(4);
        CHECK(lds <= 64 * 1024, "tap-row kernel LDS %d", lds);
#define TAPROW_CASE(VX_) if (vx == VX_) replay_rows<1, 0, VX_>(g, N, C, 2, k, d);
        TAPROW_CASE(2) TAPROW_CASE(4) TAPROW_CASE(8)
#undef TAPROW_CASE
        if (g_fails) printf("  -> %d violations\n", g_fails);
        g_fails = 0;
        return;
    }
    const int esz = dtype == 0 ? 2 : dtype == 1 ? 4 : 8;
    CHECK(vx * esz == 16 || vx * esz == 8 || vx * esz == 4 || vx * esz == 2, "vector of %d bytes", vx * esz);
    CHECK((k / 2) * d <= vx, "taps reach beyond the neighbouring lane");
    CHECK((long)H * W * 8 < (1l << 31), "plane beyond 32-bit byte offsets");
    if (filters) {
        const int lds = rows::filters_lds_bytes<9>(dtype == 2 ? 8 : 4, r, vx);
        CHECK(lds <= 64 * 1024, "filter kernel LDS %d", lds);
        CHECK(g.cpw % rows::kFlushChannels == 0, "channels per wave %d not whole flush groups", g.cpw);
    }
    const int hy = (k / 2) * d;
#define ROWS_CASE(R_, HY_, VX_) if (r == R_ && hy == HY_ && vx == VX_) { replay_rows<R_, HY_, VX_>(g, N, C, filters ? 1 : 0); done = true; }
    bool done = false;
    ROWS_CASE(1, 1, 2) ROWS_CASE(1, 1, 4) ROWS_CASE(1, 1, 8) ROWS_CASE(2, 1, 2) ROWS_CASE(2, 1, 4) ROWS_CASE(2, 1, 8)
    ROWS_CASE(1, 2, 2) ROWS_CASE(1, 2, 4) ROWS_CASE(1, 2, 8) ROWS_CASE(2, 2, 2) ROWS_CASE(2, 2, 4) ROWS_CASE(2, 2, 8)
    ROWS_CASE(1, 4, 4) ROWS_CASE(1, 4, 8) ROWS_CASE(1, 1, 1)
#undef ROWS_CASE
    CHECK(done, "no replay for r=%d hy=%d vx=%d", r, hy, vx);
    if (g_fails) printf("  -> %d violations\n", g_fails);
    g_fails = 0;
}

// Stride 2 (3 x 3) on the row-register kernels: lanes are laid out over the result plane;
// rows::LaneStride2 says where the lane's three feature vectors (2 * VX elements each) and
// its VX result pixels are.
template <int VX>
static void replay_rows_stride2(const RowsGeom &g, long N, long C, int esz, bool filters) {
    const long plane = (long)g.H * g.W, xplane = (long)g.Hi * g.Wi;
    std::vector<int> owner(plane, 0);
    CHECK(g.segs == 0 && g.lpr * VX == g.W && g.lpr <= 32, "lanes per result row");
    CHECK(g.lp == g.lpr || g.lp == g.lpr + 1, "lane pitch %d for %d lanes per row", g.lp, g.lpr);
    CHECK((long)(g.rg - 1) * g.lp + g.lpr <= 64, "row groups do not fit the wavefront");
    CHECK(g.H == g.Hi / 2 && g.W == g.Wi / 2 && g.Wi % (2 * VX) == 0, "planes %dx%d -> %dx%d", g.Hi, g.Wi, g.H, g.W);
    const int piece = 2 * VX * esz < 16 ? 2 * VX * esz : 16;   // bytes of one load instruction
    for (int strip = 0; strip < g.nstrips; ++strip)
        for (int lane = 0; lane < 64; ++lane) {
            rows::LaneStride2<VX> ln;
            ln.init(g, strip, lane);
            const int grp = lane / g.lp, v = lane % g.lp;
            const int y = strip * g.rps + grp, x0 = v * VX;
            const bool live = grp < g.rg && v < g.lpr && y < g.H;
            for (int rr = 0; rr < 3; ++rr) {
                const int yy = 2 * y - 1 + rr, off = ln.xoff[rr];
                if (!live || yy < 0) { CHECK(off < 0, "lane %d row %d should read nothing", lane, rr); continue; }
                CHECK(yy < g.Hi, "feature row %d beyond the plane", yy);
                CHECK(off == yy * g.Wi + 2 * x0 && off + 2 * VX <= xplane, "offset %d is not row %d column %d", off, yy, 2 * x0);
                CHECK(((long)off * esz) % piece == 0, "offset %d misaligned", off);
            }
            if (live) {
                CHECK(ln.ooff[0] == y * g.W + x0, "result offset");
                CHECK(ln.onext == (y + 1 < g.H ? (y + 1) * g.W + x0 : -1), "next result row");
                for (int e = 0; e < VX; ++e) ++owner[ln.ooff[0] + e];
            } else {
                CHECK(ln.ooff[0] < 0 && ln.onext < 0, "idle lane %d writes", lane);
            }
            CHECK(ln.first == (v == 0) && ln.last == (v == g.lpr - 1), "row ends");
        }
    for (long i = 0; i < plane; ++i)
        if (owner[i] != 1) { CHECK(false, "pixel %ld owned %d times", i, owner[i]); break; }
    check_work_items(g, N, C, filters ? 1 : 0, 0);
}

// fused: the cut of the launch that also writes the feature gradient (rows 2y and 2y + 1
// of the feature plane from the lane of result row y: even heights only).
static void check_rows_stride2(long N, long C, long H, long W, int dtype, bool filters, bool fused = false) {
    const Problem p = make_problem(N, C, H, W, 3, 1, 2, 0);
    RowsGeom g;
    int vx, r;
    const bool ok = filters ? rows_filters_geometry(p, dtype, fused, &g, &vx, &r) : rows_geometry(p, dtype, 0, &g, &vx, &r);
    const char *name = fused ? "-filters+dX" : filters ? "-filters" : "";
    if (!ok) {
        printf("kind rows%s stride 2 %ldx%ldx%ldx%ld dt%d: unsupported\n", name, N, C, H, W, dtype);
        return;
    }
    printf("kind rows%s stride 2 %ldx%ldx%ldx%ld dt%d: vx=%d lpr=%d lp=%d rg=%d rps=%d nstrips=%d cpw=%d cpb=%d "
           "csplit=%d wpb=%d nwork=%d\n", name, N, C, H, W, dtype, vx, g.lpr, g.lp, g.rg, g.rps, g.nstrips,
           g.cpw, g.cpb, g.csplit, g.wpb, g.nwork);
    const int esz = dtype == 0 ? 2 : 4;
    CHECK(dtype != 2 && r == 1, "stride 2 variant");
    CHECK(vx * esz == 16 || vx * esz == 8 || vx * esz == 4 || vx * esz == 2, "vector of %d bytes", vx * esz);
    if (fused) CHECK(H % 2 == 0 && g.Hi == 2 * g.H && g.Wi == 2 * g.W, "one-launch backward leaves feature rows unwritten");
    if (filters) {
        CHECK(rows::filters_lds_bytes<9>(4, 1, vx) <= 64 * 1024, "filter kernel LDS");
        CHECK(g.cpw % rows::kFlushChannels == 0, "channels per wave %d not whole flush groups", g.cpw);
    }
    if (vx == 1) replay_rows_stride2<1>(g, N, C, esz, filters);
    else if (vx == 2) replay_rows_stride2<2>(g, N, C, esz, filters);
    else if (vx == 4) replay_rows_stride2<4>(g, N, C, esz, filters);
    else if (vx == 8) replay_rows_stride2<8>(g, N, C, esz, filters);
    else CHECK(false, "no replay for vx=%d", vx);
    if (g_fails) printf("  -> %d violations\n", g_fails);
    g_fails = 0;
}

// k_small and k_up_forward (ddf_small.hip, ddf_up.hip): a workgroup takes one chunk of a
// sample's channels [and one block of 256 pixels], stages the chunk's channel taps in LDS
// `stage` channels at a time and walks the channels.  The model asks chunks::small_chunks /
// up_chunks - the launchers' own code - for the cut and replays chunks::Block and
// chunks::SmallThread - the kernels' own code - for every workgroup [and thread]: every
// (sample, pixel block, chunk) handed out exactly once, chunks covering C, LDS within the
// stage, tap indices inside the staged range, every (channel, pixel) of a chunk written once,
// element offsets inside the chunk's planes and below 2^32.
static void check_chunk_blocks(const chunks::ChunkGeom &g, long N, long C) {
    CHECK(g.cpb >= 1 && (long)g.csplit * g.cpb >= C && (long)(g.csplit - 1) * g.cpb < C, "chunks do not tile C");
    CHECK(g.blocks == N * g.pblocks * g.csplit, "block count");
    CHECK(g.stage >= 1 && g.stage <= g.cpb, "stage of %d channels for chunks of %d", g.stage, g.cpb);
    CHECK(g.lds <= 64 * 1024, "LDS %zu", g.lds);
    if (g.blocks > 400000) return;   // (the numbering is checked on the smaller cases)
    std::vector<char> seen(g.blocks, 0);
    for (long raw = 0; raw < g.blocks; ++raw) {
        chunks::Block b;
        b.init((unsigned)raw, (unsigned)g.blocks, g.csplit, g.pblocks, g.cpb, (int)C);
        CHECK(b.n >= 0 && b.n < N && b.pb >= 0 && b.pb < g.pblocks && b.chunk >= 0 && b.chunk < g.csplit, "block out of range");
        CHECK(b.c0 == b.chunk * g.cpb && b.nch >= 1 && b.c0 + b.nch <= C, "channels %d+%d of %ld", b.c0, b.nch, C);
        const long id = (b.n * g.pblocks + b.pb) * g.csplit + b.chunk;
        if (id >= 0 && id < g.blocks) { CHECK(!seen[id], "block %ld handed out twice", id); seen[id] = 1; }
    }
    for (long i = 0; i < g.blocks; ++i)
        if (!seen[i]) { CHECK(false, "block %ld never handed out", i); break; }
}

static void check_small(long N, long C, int H, int W, int dtype, long target) {
    const int plane = H * W, asz = dtype == 2 ? 8 : 4;
    chunks::ChunkGeom g;
    if (!chunks::small_chunks(N, C, plane, asz, target, &g)) {
        printf("kind small %ldx%ldx%dx%d dt%d: unsupported\n", N, C, H, W, dtype);
        return;
    }
    printf("kind small %ldx%ldx%dx%d dt%d: G=%d cpb=%d csplit=%d stage=%d blocks=%ld lds=%zu\n", N, C, H, W, dtype,
           g.G, g.cpb, g.csplit, g.stage, (long)g.blocks, g.lds);
    CHECK(g.G >= 4 && g.G * plane <= chunks::kThreads && g.pblocks == 1, "G=%d planes of %d pixels", g.G, plane);
    CHECK(g.lds == (size_t)g.stage * 9 * asz, "LDS bytes");
    check_chunk_blocks(g, N, C);
    // one chunk of every length that occurs: the full one and the last one
    const int lens[2] = {g.cpb, (int)(C - (long)(g.csplit - 1) * g.cpb)};
    for (int which = 0; which < 2; ++which) {
        const int nch = lens[which];
        CHECK((long)nch * plane < (1l << 32), "32-bit offsets inside a chunk");
        std::vector<int> owner((size_t)nch * plane, 0);
        for (int s0 = 0; s0 < nch; s0 += g.stage) {
            const int ns = std::min(g.stage, nch - s0);
            CHECK(ns * 9 <= g.stage * 9, "taps staged beyond LDS");
            for (int tid = 0; tid < chunks::kThreads; ++tid) {
                chunks::SmallThread th;
                th.init(tid, plane, g.G);
                CHECK(th.q >= 0 && th.q < g.G && th.pix >= 0 && th.pix < plane, "thread %d -> slot %d pixel %d", tid, th.q, th.pix);
                const int mine = th.channels(ns, g.G);
                CHECK(th.live || mine == 0, "idle thread %d works", tid);
                for (int m = 0; m < mine; ++m) {
                    const int ch = th.q + m * g.G;   // channel of the stage, as the kernel's `at` and `w` walk it
                    CHECK(ch < ns, "thread %d channel %d of %d", tid, ch, ns);
                    CHECK((ch + 1) * 9 <= ns * 9, "tap index beyond the staged taps");
                    if (ch < ns) ++owner[(size_t)(s0 + ch) * plane + th.pix];
                }
            }
        }
        for (size_t i = 0; i < owner.size(); ++i)
            if (owner[i] != 1) { CHECK(false, "chunk element %zu written %d times", i, owner[i]); break; }
    }
    if (g_fails) printf("  -> %d violations\n", g_fails);
    g_fails = 0;
}

static void check_up(long N, long C, long H, long W, int k, int scale, int dtype, long target, int min_chunk) {
    const int asz = dtype == 2 ? 8 : 4, taps = k * k * scale * scale;
    chunks::ChunkGeom g;
    if (!chunks::up_chunks(N, C, H * W, taps, asz, target, min_chunk, &g)) {
        printf("kind up %ldx%ldx%ldx%ld k%d x%d dt%d: unsupported\n", N, C, H, W, k, scale, dtype);
        return;
    }
    printf("kind up %ldx%ldx%ldx%ld k%d x%d dt%d: cpb=%d csplit=%d pblocks=%d stage=%d blocks=%ld lds=%zu\n", N, C, H, W,
           k, scale, dtype, g.cpb, g.csplit, g.pblocks, g.stage, (long)g.blocks, g.lds);
    CHECK((long)g.pblocks * chunks::kThreads >= H * W && (long)(g.pblocks - 1) * chunks::kThreads < H * W, "pixel blocks");
    CHECK(g.lds == (size_t)g.stage * taps * asz && g.lds <= (size_t)chunks::kUpStageBytes + (size_t)taps * asz, "LDS bytes");
    CHECK(g.stage <= chunks::kUpStageChannels, "stage");
    check_chunk_blocks(g, N, C);
    // staging of a stage's taps: element e of RR*ns*KK -> (branch, channel, tap) -> LDS slot
    const int KK = k * k, RR = scale * scale;
    for (int ns : {1, g.stage}) {
        const int per = ns * KK, total = RR * per;
        std::vector<char> slot((size_t)g.stage * RR * KK, 0);
        for (int e = 0; e < total; ++e) {
            const int b = e / per, r = e - b * per, ch = r / KK, t = r - ch * KK;
            const long at = ((long)ch * RR + b) * KK + t;
            CHECK(b < RR && ch < ns && at >= 0 && at < (long)slot.size(), "tap %d staged outside LDS", e);
            if (at >= 0 && at < (long)slot.size()) { CHECK(!slot[at], "LDS slot %ld written twice", at); slot[at] = 1; }
        }
    }
    if (g_fails) printf("  -> %d violations\n", g_fails);
    g_fails = 0;
}

int main() {
    const long shapes[][4] = {
        {96, 64, 56, 56},   {64, 256, 14, 14}, {64, 128, 28, 28},  {64, 512, 7, 7},   {64, 64, 56, 56},
        {32, 128, 56, 56},  {128, 512, 14, 14}, {1, 70, 10, 10},   {35, 1, 10, 10},   {1, 1, 50, 50},
        {2, 3, 9, 11},      {1, 5, 2, 2},      {1, 2, 1, 1},       {1, 1, 1, 64},     {1, 1, 64, 1},
        {2, 3, 20, 30},     {1, 2, 5, 200},    {1, 2, 31, 17},     {3, 65, 14, 14},   {2, 130, 7, 7},
        {2, 256, 200, 300}, {32, 256, 224, 224}, {32, 256, 112, 112}, {1, 20, 40, 40}, {2, 9, 12, 16}};
    const int kds[][3] = {{3, 1, 1}, {3, 2, 1}, {3, 1, 2}, {3, 2, 2}, {5, 1, 1}, {5, 2, 1}, {5, 1, 2}, {5, 2, 2}};
    for (auto &sh : shapes)
        for (auto &q : kds)
            for (int dtype = 0; dtype < 3; ++dtype)
                for (int kind = 0; kind < 4; ++kind)
                    for (int max_vec = 0; max_vec < 2; ++max_vec) {
                        if (sh[2] / q[2] == 0 || sh[3] / q[2] == 0) continue;
                        check_geometry(kind, sh[0], sh[1], sh[2], sh[3], q[0], q[1], q[2], dtype, max_vec);
                    }
    for (auto &sh : shapes)
        for (int d = 1; d <= 2; ++d)
            for (int dtype = 0; dtype < 3; ++dtype)
                for (int filters = 0; filters < 3; ++filters)
                    check_rows(sh[0], sh[1], sh[2], sh[3], 3, d, dtype, filters != 0, filters == 2);
    for (auto &sh : shapes)
        for (int d = 1; d <= 2; ++d)
            for (int dtype = 0; dtype < 3; ++dtype) {
                check_rows(sh[0], sh[1], sh[2], sh[3], 5, d, dtype, false);
                check_rows(sh[0], sh[1], sh[2], sh[3], 5, d, dtype, true, false, true);
                check_rows(sh[0], sh[1], sh[2], sh[3], 3, d, dtype, true, false, true);
            }
    for (auto &sh : shapes)
        for (int dtype = 0; dtype < 3; ++dtype)
            for (int filters = 0; filters < 3; ++filters)
                check_rows_stride2(sh[0], sh[1], sh[2], sh[3], dtype, filters != 0, filters == 2);
    // tiny planes (k_small): every plane size 1..64, ragged C, C below G, fp64 stages
    for (int H = 1; H <= 8; ++H)
        for (int W = 1; W <= 64 / H; W += (W < 9 ? 1 : 5))
            for (long C : {1l, 3l, 37l, 130l, 512l, 2048l})
                for (int dtype = 1; dtype < 3; ++dtype)
                    check_small(H == 7 ? 64 : 3, C, H, W, dtype, C == 130 ? 64 : 1024);
    check_small(1, 1 << 24, 8, 8, 1, 1024);
    // up-sampling forward: every (k, scale) pair that is built, ragged C, fp64 stage sizing
    const int up_pairs[][2] = {{1, 2}, {1, 3}, {1, 4}, {3, 2}, {3, 3}, {3, 4}, {5, 2}};
    for (auto &ks : up_pairs)
        for (long C : {1l, 7l, 64l, 100l, 513l})
            for (int dtype = 1; dtype < 3; ++dtype) {
                check_up(8, C, 64, 64, ks[0], ks[1], dtype, 512, 8);
                check_up(1, C, 5, 7, ks[0], ks[1], dtype, 2048, 1);
                check_up(3, C, 33, 100, ks[0], ks[1], dtype, 256, 8);
            }
    // seeded random shapes on top of the fixed list
    unsigned long long state = 0x9E3779B97F4A7C15ull;
    auto next = [&](int lo, int hi) {
        state = state * 6364136223846793005ull + 1442695040888963407ull;
        return lo + (int)((state >> 33) % (unsigned long long)(hi - lo + 1));
    };
    for (int i = 0; i < 150; ++i) {
        const long N = next(1, 130), C = next(1, 600), H = next(1, 130), W = next(1, 330);
        const int *q = kds[next(0, 7)];
        if (H / q[2] == 0 || W / q[2] == 0) continue;
        for (int kind = 0; kind < 4; ++kind)
            check_geometry(kind, N, C, H, W, q[0], q[1], q[2], next(0, 2), next(0, 1));
        check_rows(N, C, H, W / 2 * 2 + 2, 3, next(1, 2), next(0, 1), next(0, 1) != 0);
        check_rows(N, C, H, (W / 8 + 1) * 8, 3, next(1, 2), next(0, 1), next(0, 1) != 0);
        check_rows(N, C, H, (W / 8 + 1) * 8, 5, next(1, 2), next(0, 1), false);
        check_rows(N, C, H, (W / 8 + 1) * 8 * next(1, 6), 3, next(1, 2), next(0, 1), next(0, 1) != 0);
        check_rows(N, C, H, (W / 4 + 1) * 4, 5, next(1, 2), next(0, 1), true, false, true);
        check_rows_stride2(N, C, H + 1, (W / 4 + 1) * 4, next(0, 1), next(0, 1) != 0);
        check_rows_stride2(N, C, H + 1, (W / 16 + 1) * 16, next(0, 1), next(0, 1) != 0);
        check_rows_stride2(N, C, H + 1, (W / 16 + 1) * 16, next(0, 1), true, true);
    }
    return 0;
}
