// Row-register DDF kernels for gfx950: forward and feature gradient with stride 1,
// the 3 x 3 forward also with stride 2 (LaneStride2, the S = 2 instantiations).
//
// A lane owns R consecutive rows of VX neighbouring pixels (one 16-, 8-, 4- or -
// a single fp16 pixel - 2-byte vector per row) of one sample and walks a range
// of channels.  Nothing of the
// feature map goes through LDS:
//   * the R + 2*HY rows a lane needs per channel (its own and the HY = (K/2)*D
//     rows above and below) come straight from global memory as whole vectors,
//     a few channels ahead of use; the rows shared with the lanes above and
//     below are served by the cache;
//   * every plane is addressed through a buffer descriptor that covers exactly
//     that plane, so a row above or below the image, the vector of an idle lane
//     and the channels past a wave's last one are simply given an offset
//     outside the descriptor: such loads return zero and such stores are
//     dropped by the memory unit - the zero padding of the operator costs no
//     instruction and the kernels contain no bounds branch;
//   * the HX = (K/2)*D pixels left and right of a vector are the edge words of
//     the neighbouring lanes' vectors, fetched with one wavefront shift (DPP)
//     per word.  Lanes are laid out over a strip as (row group, vector) with
//     lpr = W / VX lanes per image row; where it costs no row group, an idle
//     lane (whose loads return zero) separates consecutive image rows, and the
//     shift brings in the zero padding by itself; otherwise the lanes at the
//     ends of an image row select zero;
//   * the K*K spatial-filter taps of the lane's R*VX pixels stay in registers
//     for the whole channel walk, in storage format (fp16 stays packed);
//   * the K*K channel-filter taps of a channel come in through the scalar unit
//     (fp32, fp64) or are loaded by lanes 0..K*K-1 and broadcast (fp16).
//
// The feature gradient is the same walk over dO with flipped taps,
//   dX[p] = sum_t dO[p - o_t] * comb(CF[t], SF[t, p - o_t]),
// so the only difference is the prologue: the spatial taps a lane keeps are
// those of the pixels its dO values come from (rows fetched at the tap's row
// offset, columns shifted by the same wavefront shifts, zero outside the
// image).  Reference kernels computing the same sums:
// ddf/src/cuda/ddf_mul_cuda_kernel.cu:85-165 (forward), :198-290 (feature
// gradient), ddf_mul_faster_cuda_kernel.cu:47-163.
#pragma once

#include <type_traits>

#include "ddf_common.h"

namespace ddf {

struct RowsGeom {
    int C, H, W;              // per sample, of the result plane
    int Hi, Wi;               // feature plane (stride 1: the same shape)
    int lpr, rg;              // lanes per image row, row groups per wave
    int lp;                   // lane pitch of a row group: lpr, or lpr + 1 (an idle lane after each row)
    unsigned lp_magic;        // ceil(2^32 / lp), 0 when lp == 1
    int rps, nstrips;         // rows per strip (= rg * R), strips per plane
    int cpw, cpb, csplit;     // channels per wave and per work item; channel ranges per plane
    int wpb;                  // work items (independent waves) per workgroup
    int nwork;                // N * nstrips * csplit wave-sized work items
    unsigned csplit_magic, nstrips_magic, xcd_per;
    // Image rows longer than a wave (segs > 0): a strip is one segment of one
    // row group; its wave holds seg_out vectors that it produces results for,
    // between one vector of the neighbouring segment (or of nothing, at the
    // ends of the image row) on either side, which it only reads.  rg = 1,
    // lp = lpr = seg_out + 2, nstrips = row groups * segs.
    int segs, seg_out;
    unsigned segs_magic;
};

// The vectors shifted in from the neighbouring lanes are right as they arrive
// (an idle lane or a neighbouring segment's vector sits next to every row end):
// the kernels' PAD variants.
inline bool rows_shift_in_as_is(const RowsGeom &g) { return g.lp > g.lpr || g.segs > 0; }

namespace rows {

constexpr int kXcd = 8;
constexpr int kMaxWpb = 4;

// q = n / d through the host's magic number m = ceil(2^32 / d) (0: d == 1);
// exact while n * d < 2^32.
__host__ __device__ __forceinline__ int magic_div(int n, unsigned m) {
    return m ? (int)(((unsigned long long)(unsigned)n * m) >> 32) : n;
}

// Which strip of which sample and which channel range a wave works on.
// Workgroups are handed to the 8 XCDs round-robin; they are renumbered so that
// consecutive work items (same sample, neighbouring channel ranges and strips)
// share an XCD and its L2.
struct Work {
    int cs, strip, c_begin, c_end;
    int64_t n;
    // Number of the work item of wave `wave` of workgroup `block`, -1: none.
    __host__ __device__ static __forceinline__ int item_of(const RowsGeom &g, int block, int wave) {
        const int wg = (block % kXcd) * (int)g.xcd_per + block / kXcd;
        const int b = wg * g.wpb + wave;
        return (wave >= g.wpb || b >= g.nwork) ? -1 : b;
    }
    __host__ __device__ __forceinline__ bool init(const RowsGeom &g, int block, int wave) {
        const int b = item_of(g, block, wave);
        if (b < 0) return false;
        decode(g, b);
        return true;
    }
    // b: (sample, strip, channel range) number, channel range fastest
    __host__ __device__ __forceinline__ void decode(const RowsGeom &g, int b) {
        const int rest = magic_div(b, g.csplit_magic);
        cs = b - rest * g.csplit;
        const int smp = magic_div(rest, g.nstrips_magic);
        strip = rest - smp * g.nstrips;
        n = smp;
        c_begin = cs * g.cpb;
        c_end = c_begin + g.cpb < g.C ? c_begin + g.cpb : g.C;
    }
};

// Where a lane's rows are.  Shared by the kernels and by the host-side bounds
// model, which replays it for every lane.
//   xoff[rr]: element offset inside a plane of the lane's vector in window row
//             rr (rr = 0 is HY rows above the lane's first row), or -1 when the
//             row lies outside the image or the lane is idle;
//   ooff[r]:  the same for the R result rows.
template <int R, int HY, int VX>
struct Lane {
    static constexpr int ROWS = R + 2 * HY;
    bool first, last;         // at the ends of an image row
    int xoff[ROWS];
    int ooff[R];
    // dy: the window rows (xoff) are taken dy image rows further down
    __host__ __device__ __forceinline__ void init(const RowsGeom &g, int strip, int lane, int dy = 0) {
        if (g.segs > 0) {
            // one segment of one row group: lane 0 and lane seg_out + 1 read the
            // neighbouring segments' edge vectors and produce nothing themselves
            const int grp = magic_div(strip, g.segs_magic);
            const int seg = strip - grp * g.segs;
            const int x0 = (seg * g.seg_out + lane - 1) * VX;
            const int y0 = grp * R;
            const bool reads = lane <= g.seg_out + 1 && x0 >= 0 && x0 < g.W;
            const bool owns = reads && lane >= 1 && lane <= g.seg_out;
            first = last = false;   // (the shifted-in vectors are right as they are)
#pragma unroll
            for (int rr = 0; rr < ROWS; ++rr) {
                const int yy = y0 - HY + rr + dy;
                xoff[rr] = (reads && yy >= 0 && yy < g.H) ? yy * g.W + x0 : -1;
            }
#pragma unroll
            for (int r = 0; r < R; ++r) ooff[r] = (owns && y0 + r < g.H) ? (y0 + r) * g.W + x0 : -1;
            return;
        }
        const int grp = magic_div(lane, g.lp_magic);
        const int v = lane - grp * g.lp;
        const bool live = grp < g.rg && v < g.lpr;
        const int x0 = v * VX;
        const int y0 = strip * g.rps + grp * R;
        first = v == 0;
        last = v == g.lpr - 1;
#pragma unroll
        for (int rr = 0; rr < ROWS; ++rr) {
            const int yy = y0 - HY + rr + dy;
            xoff[rr] = (live && yy >= 0 && yy < g.H) ? yy * g.W + x0 : -1;
        }
#pragma unroll
        for (int r = 0; r < R; ++r) ooff[r] = (live && y0 + r < g.H) ? (y0 + r) * g.W + x0 : -1;
    }
};

// Stride 2, 3 x 3, one result row per lane: the lane's VX result pixels of row y
// read the feature rows 2y-1 .. 2y+1, columns 2*x0-1 .. 2*x0+2*VX-1: a vector of
// 2*VX elements per row at xoff (offsets inside the feature plane) and the last
// element of the lane to the left.
template <int VX>
struct LaneStride2 {
    static constexpr int ROWS = 3;
    bool first, last;
    int xoff[ROWS];
    int ooff[1];
    int onext;   // the lane's vector one result row further down (-1: past the last row)
    __host__ __device__ __forceinline__ void init(const RowsGeom &g, int strip, int lane, int = 0) {
        const int grp = magic_div(lane, g.lp_magic);
        const int v = lane - grp * g.lp;
        const int y = strip * g.rps + grp;
        const bool live = grp < g.rg && v < g.lpr && y < g.H;
        const int x0 = v * VX;
        first = v == 0;
        last = v == g.lpr - 1;
#pragma unroll
        for (int rr = 0; rr < ROWS; ++rr) {
            const int yy = 2 * y - 1 + rr;
            xoff[rr] = (live && yy >= 0 && yy < g.Hi) ? yy * g.Wi + 2 * x0 : -1;
        }
        ooff[0] = live ? y * g.W + x0 : -1;
        onext = (live && y + 1 < g.H) ? (y + 1) * g.W + x0 : -1;
    }
};

// Window row rr (0 = HY rows above the lane's first row) is touched by some tap
// of some of the lane's R rows: rr = r + i*D.  With dilation the window has
// rows no tap lands on; they are neither loaded nor shifted.
template <int R, int K, int D>
__host__ __device__ constexpr bool row_needed(int rr) {
    for (int r = 0; r < R; ++r)
        for (int i = 0; i < K; ++i)
            if (r + i * D == rr) return true;
    return false;
}

#ifdef __HIPCC__

// Byte offset no plane reaches (planes are below 2^31 bytes): a buffer access
// at this offset is out of range whatever it is added to.
constexpr uint32_t kOutside = 0x80000000u;

// Buffer descriptor over `bytes` bytes at p (raw buffer, no stride): accesses at
// offsets >= bytes read as zero and are not written.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t plane_rsrc(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}

template <int N>
__device__ __forceinline__ void load_words(__amdgpu_buffer_rsrc_t rsrc, uint32_t off, uint32_t (&w)[N]) {
    if constexpr (N == 1) {
        w[0] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)off, 0, 0);
    } else if constexpr (N == 2) {
        const auto v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, (int)off, 0, 0);
        w[0] = v[0]; w[1] = v[1];
    } else if constexpr (N == 4) {
        const auto v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, 0);
#pragma unroll
        for (int k = 0; k < 4; ++k) w[k] = v[k];
    } else {
        static_assert(N == 8, "vectors of 4, 8, 16 or 32 bytes");
        // (an offset outside the descriptor stays outside with 16 added)
        const auto lo = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, 0);
        const auto hi = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(off + 16u), 0, 0);
#pragma unroll
        for (int k = 0; k < 4; ++k) { w[k] = lo[k]; w[4 + k] = hi[k]; }
    }
}

// f(integral_constant<int, I>) for I = 0 .. N-1, unrolled.
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// Nontemporal: results are not read again by this kernel.
template <int N>
__device__ __forceinline__ void store_words_nt(__amdgpu_buffer_rsrc_t rsrc, uint32_t off, const uint32_t (&w)[N]) {
    if constexpr (N == 1) {
        __builtin_amdgcn_raw_buffer_store_b32(w[0], rsrc, (int)off, 0, 2);
    } else if constexpr (N == 2) {
        typedef uint32_t v2 __attribute__((ext_vector_type(2)));
        v2 v = {w[0], w[1]};
        __builtin_amdgcn_raw_buffer_store_b64(v, rsrc, (int)off, 0, 2);
    } else {
        static_assert(N == 4 || N == 8, "vectors of 4, 8, 16 or 32 bytes");
        typedef uint32_t v4 __attribute__((ext_vector_type(4)));
        v4 v = {w[0], w[1], w[2], w[3]};
        __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, (int)off, 0, 2);
        if constexpr (N == 8) {
            v4 u = {w[4], w[5], w[6], w[7]};
            __builtin_amdgcn_raw_buffer_store_b128(u, rsrc, (int)(off + 16u), 0, 2);
        }
    }
}

// A lane's vector of BYTES bytes (2: one fp16 element, kept in the low half of a
// word) <-> 32-bit words.
constexpr int vec_words(int bytes) { return bytes >= 4 ? bytes / 4 : 1; }
template <int BYTES>
__device__ __forceinline__ void load_vec(__amdgpu_buffer_rsrc_t rsrc, uint32_t off,
                                         uint32_t (&w)[vec_words(BYTES)]) {
    if constexpr (BYTES == 2) w[0] = (uint32_t)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rsrc, (int)off, 0, 0);
    else load_words<BYTES / 4>(rsrc, off, w);
}
template <int BYTES>
__device__ __forceinline__ void store_vec_nt(__amdgpu_buffer_rsrc_t rsrc, uint32_t off,
                                             const uint32_t (&w)[vec_words(BYTES)]) {
    if constexpr (BYTES == 2) __builtin_amdgcn_raw_buffer_store_b16((short)w[0], rsrc, (int)off, 0, 2);
    else store_words_nt<BYTES / 4>(rsrc, off, w);
}

// One accumulator-type value, rounded to the storage type, to byte offset off
// of the buffer.
template <typename T>
__device__ __forceinline__ void store_value(__amdgpu_buffer_rsrc_t rsrc, uint32_t off,
                                            typename Acc<T>::type v) {
    if constexpr (sizeof(T) == 2) {
        const _Float16 h = (_Float16)v;
        __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(short, h), rsrc, (int)off, 0, 0);
    } else if constexpr (sizeof(T) == 4) {
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), rsrc, (int)off, 0, 0);
    } else {
        typedef uint32_t v2 __attribute__((ext_vector_type(2)));
        const v2 w = {(uint32_t)__double2loint(v), (uint32_t)__double2hiint(v)};
        __builtin_amdgcn_raw_buffer_store_b64(w, rsrc, (int)off, 0, 0);
    }
}

// Element e of a run of storage-type values held in 32-bit words, widened to
// the accumulator type.  (e is a constant wherever this is called: every loop
// around it is unrolled.)
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
template <typename T>
__device__ __forceinline__ typename Acc<T>::type elem(const uint32_t *w, int e) {
    if constexpr (sizeof(T) == 2) {
        const half2_t h = __builtin_bit_cast(half2_t, w[e / 2]);
        return (float)((e & 1) ? h[1] : h[0]);
    } else if constexpr (sizeof(T) == 4) {
        return __uint_as_float(w[e]);
    } else {
        return __hiloint2double((int)w[2 * e + 1], (int)w[2 * e]);
    }
}

// VX accumulator-type values -> storage-type words (round to nearest even).
template <typename T, int VX, typename A>
__device__ __forceinline__ void pack(const A (&v)[VX], uint32_t (&w)[vec_words(VX * sizeof(T))]) {
    if constexpr (sizeof(T) == 2 && VX == 1) {
        const _Float16 h = (_Float16)v[0];
        w[0] = (uint32_t)__builtin_bit_cast(unsigned short, h);
    } else if constexpr (sizeof(T) == 2) {
#pragma unroll
        for (int k = 0; k < VX / 2; ++k) {
            half2_t h;
            h[0] = (_Float16)v[2 * k];
            h[1] = (_Float16)v[2 * k + 1];
            w[k] = __builtin_bit_cast(uint32_t, h);
        }
    } else if constexpr (sizeof(T) == 4) {
#pragma unroll
        for (int k = 0; k < VX; ++k) w[k] = __float_as_uint(v[k]);
    } else {
#pragma unroll
        for (int k = 0; k < VX; ++k) {
            w[2 * k] = (uint32_t)__double2loint(v[k]);
            w[2 * k + 1] = (uint32_t)__double2hiint(v[k]);
        }
    }
}

// Whole-wavefront shifts of one register: lane l receives lane l-1's (from_left)
// or lane l+1's value; the lane without a source receives 0.
__device__ __forceinline__ uint32_t from_left(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x138 /* wave_shr:1 */, 0xf, 0xf, true);
}
__device__ __forceinline__ uint32_t from_right(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x130 /* wave_shl:1 */, 0xf, 0xf, true);
}

__device__ __forceinline__ float fma_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fma_(double a, double b, double c) { return __builtin_fma(a, b, c); }

// One image row as a lane sees it: its own VX elements plus HX elements of the
// lanes to its left and right (zero beyond the ends of the image row).
// PAD: an idle lane holding zeros follows every image row, so the shifted-in
// words are already right; otherwise the lanes at the row ends select zero.
template <typename T, int VX, int HX, bool PAD>
struct ExtRow {
    using A = typename Acc<T>::type;
    static constexpr int NW = vec_words(VX * sizeof(T));
    static constexpr int SW = HX == 0 ? 1 : (HX * sizeof(T) + 3) / 4;   // words taken from each neighbour
    static constexpr int kLeftFirst = (NW - SW) * 4 / (int)sizeof(T);   // neighbour element in left[0]
    static_assert(HX <= VX, "taps reach beyond the neighbouring lane");
    uint32_t own[NW], left[SW], right[SW];
    __device__ __forceinline__ void sides(bool first, bool last) {
        if constexpr (HX > 0) {
#pragma unroll
            for (int k = 0; k < SW; ++k) {
                const uint32_t l = from_left(own[NW - SW + k]);
                const uint32_t r = from_right(own[k]);
                left[k] = PAD ? l : (first ? 0u : l);
                right[k] = PAD ? r : (last ? 0u : r);
            }
        }
    }
    // element at column e relative to the lane's first pixel, e in [-HX, VX + HX)
    __device__ __forceinline__ A at(int e) const {
        if (e < 0) return elem<T>(left, VX + e - kLeftFirst);
        if (e >= VX) return elem<T>(right, e - VX);
        return elem<T>(own, e);
    }
};

template <typename A>
__device__ __forceinline__ A lane_broadcast(A v, int src_lane);
template <>
__device__ __forceinline__ float lane_broadcast<float>(float v, int src_lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src_lane));
}
template <>
__device__ __forceinline__ double lane_broadcast<double>(double v, int src_lane) {
    const int lo = __builtin_amdgcn_readlane(__double2loint(v), src_lane);
    const int hi = __builtin_amdgcn_readlane(__double2hiint(v), src_lane);
    return __hiloint2double(hi, lo);
}

// BWD = false: out = forward(x, cf, sf).  BWD = true: x is dO and out is dX.
// WPE: waves per SIMD the register allocation must leave room for.
// S = 2 (forward, 3 x 3, one row per lane): g describes the result plane, the
// lane's feature vectors are 2 * VX elements wide (LaneStride2).
template <typename T, int K, int D, bool MUL, bool BWD, int VX, int R, bool PAD, int NST, int WPE,
          int S = 1>
__global__ __launch_bounds__(kWave * kMaxWpb, WPE) void k_rows(RowsGeom g, const T *__restrict__ x,
                                                         const T *__restrict__ cf,
                                                         const T *__restrict__ sf,
                                                         T *__restrict__ out) {
    using A = typename Acc<T>::type;
    constexpr int KK = K * K, RAD = K / 2, HX = RAD * D, HY = RAD * D;
    constexpr int ROWS = R + 2 * HY;
    constexpr int kVB = VX * sizeof(T), kXB = S * kVB;   // bytes of a result / feature vector
    constexpr int NW = vec_words(kVB), NWX = vec_words(kXB);
    using Row = ExtRow<T, S * VX, HX, PAD>;
    static_assert(KK <= kWave, "one lane per channel-filter tap");
    static_assert(S == 1 || (S == 2 && K == 3 && D == 1 && R == 1), "stride 2: 3 x 3, one row per lane");
    // Stride-2 feature gradient: the lane of result row y loads dO rows y and y + 1 and
    // writes the feature rows 2y and 2y + 1 of its columns (even feature heights).
    constexpr bool S2B = S == 2 && BWD;
    constexpr int LROWS = S2B ? 2 : ROWS;                 // rows a lane loads per channel
    constexpr int kLB = S2B ? kVB : kXB, LNW = vec_words(kLB);

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    Work wk;
    if (!wk.init(g, blockIdx.x, wave) || wk.c_end <= wk.c_begin) return;
    const int nch = wk.c_end - wk.c_begin;
    const int64_t plane = (int64_t)g.H * g.W;   // result plane
    const uint32_t plane_bytes = (uint32_t)plane * (uint32_t)sizeof(T);
    const int64_t xplane = S == 1 ? plane : (int64_t)g.Hi * g.Wi;
    const uint32_t xplane_bytes = S == 1 ? plane_bytes : (uint32_t)xplane * (uint32_t)sizeof(T);
    std::conditional_t<S == 1, Lane<R, HY, VX>, LaneStride2<VX>> ln;
    ln.init(g, wk.strip, lane);

    // (the tensor read has the result plane's shape in the stride-2 gradient, and the one
    // written the feature plane's)
    const int64_t in_plane = S2B ? plane : xplane, out_plane = S2B ? xplane : plane;
    const uint32_t in_bytes = S2B ? plane_bytes : xplane_bytes, out_bytes = S2B ? xplane_bytes : plane_bytes;
    const T *xs = x + (wk.n * g.C + wk.c_begin) * in_plane;
    T *os = out + (wk.n * g.C + wk.c_begin) * out_plane;
    // byte offsets of the lane's vectors inside a plane; kOutside: reads as zero, is not written
    uint32_t xb[ROWS], ob[R];
#pragma unroll
    for (int rr = 0; rr < ROWS; ++rr)
        xb[rr] = ln.xoff[rr] < 0 ? kOutside : (uint32_t)ln.xoff[rr] * (uint32_t)sizeof(T);
#pragma unroll
    for (int r = 0; r < R; ++r)
        ob[r] = ln.ooff[r] < 0 ? kOutside : (uint32_t)ln.ooff[r] * (uint32_t)sizeof(T);
    const T *cfs = cf + (wk.n * g.C + wk.c_begin) * KK;
    constexpr bool kScalarTaps = sizeof(T) >= 4;
    constexpr bool kFlip = BWD && S == 1;       // (the stride-2 gradient names its taps itself)
    const int tl = lane < KK ? lane : KK - 1;   // lane t holds tap t of a channel (flipped for the gradient)
    const int tsel = kFlip ? KK - 1 - tl : tl;
    // where the lane's loads are
    uint32_t lb[LROWS];
    if constexpr (S2B) {
        lb[0] = ob[0];
        lb[1] = ln.onext < 0 ? kOutside : (uint32_t)ln.onext * (uint32_t)sizeof(T);
    } else {
#pragma unroll
        for (int rr = 0; rr < ROWS; ++rr) lb[rr] = xb[rr];
    }

    // Spatial taps of the lane's pixels, in storage format.  Forward: tap t at
    // the pixel itself.  Gradient: slot (i, j) holds tap (K-1-i, K-1-j) at the
    // pixel (i-RAD)*D rows and (j-RAD)*D columns away - the pixel whose result
    // that dO value belongs to - and zero where that pixel does not exist.
    uint32_t sfw[R][KK][NW];
    {
        const T *sfn = sf + wk.n * KK * plane;
        if constexpr (S2B) {
            // Result pixel (y, x) reaches feature pixel (2y + i - 1, 2x + j - 1) through tap
            // (i, j).  Seen from the lane's 2 x 2 VX block of feature pixels (rows 2y and
            // 2y + 1), tap row 0 belongs to the result row below and tap column 0 to the
            // result pixel to the right: slot (i, j) holds that pixel's tap.
            using SRow = ExtRow<T, VX, 1, PAD>;
#pragma unroll
            for (int i = 0; i < K; ++i)
#pragma unroll
                for (int j = 0; j < K; ++j) {
                    const int t = i * K + j;
                    const __amdgpu_buffer_rsrc_t sr = plane_rsrc(sfn + t * plane, plane_bytes);
                    SRow row;
                    load_vec<kVB>(sr, lb[i == 0 ? 1 : 0], row.own);
                    if (j == 0) {
                        row.sides(ln.first, ln.last);
                        A v[VX];
#pragma unroll
                        for (int e = 0; e < VX; ++e) v[e] = row.at(e + 1);
                        pack<T, VX, A>(v, sfw[0][t]);
                    } else {
#pragma unroll
                        for (int k = 0; k < NW; ++k) sfw[0][t][k] = row.own[k];
                    }
                }
        } else if constexpr (!BWD) {
#pragma unroll
            for (int t = 0; t < KK; ++t) {
                const __amdgpu_buffer_rsrc_t sr = plane_rsrc(sfn + t * plane, plane_bytes);
#pragma unroll
                for (int r = 0; r < R; ++r) load_vec<kVB>(sr, ob[r], sfw[r][t]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < K; ++i)
#pragma unroll
                for (int j = 0; j < K; ++j) {
                    const __amdgpu_buffer_rsrc_t sr =
                        plane_rsrc(sfn + ((K - 1 - i) * K + (K - 1 - j)) * plane, plane_bytes);
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        Row row;
                        load_vec<kVB>(sr, xb[r + i * D], row.own);
                        row.sides(ln.first, ln.last);
                        A v[VX];
#pragma unroll
                        for (int e = 0; e < VX; ++e) v[e] = row.at(e + j * D - HX);
                        pack<T, VX, A>(v, sfw[r][i * K + j]);
                    }
                }
        }
    }

    // feature rows and channel taps of channel ci, stage ST; a channel past the
    // wave's last one reads zeros (empty descriptor)
    uint32_t xw[NST][LROWS][LNW];
    T cfl[NST];
    A cfu[NST][kScalarTaps ? KK : 1];
    auto issue = [&](auto st_tag, int ci) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value;
        const __amdgpu_buffer_rsrc_t pr = plane_rsrc(xs + (int64_t)ci * in_plane, ci < nch ? in_bytes : 0u);
#pragma unroll
        for (int rr = 0; rr < LROWS; ++rr)
            if (S2B || row_needed<R, K, D>(rr)) load_vec<kLB>(pr, lb[rr], xw[ST][rr]);
        const int cc = ci < nch ? ci : nch - 1;   // (the taps are read through plain pointers: stay inside)
        if constexpr (kScalarTaps) {
#pragma unroll
            for (int t = 0; t < KK; ++t) cfu[ST][t] = cfs[(int64_t)cc * KK + (kFlip ? KK - 1 - t : t)];
        } else {
            cfl[ST] = cfs[(int64_t)cc * KK + tsel];
        }
    };
    issue(std::integral_constant<int, 0>{}, 0);
    if constexpr (NST > 2) issue(std::integral_constant<int, 1>{}, 1);
    if constexpr (NST > 3) issue(std::integral_constant<int, 2>{}, 2);

    // The taps were requested before the first channels.  Wait for them here:
    // a wait inside the walk would drain the channel pipeline every round.
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < KK; ++t)
#pragma unroll
            for (int k = 0; k < NW; ++k) asm volatile("" : "+v"(sfw[r][t][k]));

    // fp16, 3 x 3 without dilation: the taps of columns 0 and 1 of a filter row go through
    // the two-element dot product (fp32 accumulation), whose operands are pairs of
    // neighbouring feature pixels and, per pixel, the pair of combined filters
    // comb(CF, SF) - formed by one packed fp16 operation, i.e. rounded to fp16 like the
    // operands.  12 vector instructions per pixel and channel instead of 18.  For that
    // the spatial taps are regrouped once: sfp[r][i][e] = taps (i, 0) and (i, 1) of pixel
    // e, sfs[r][i][k] = tap (i, 2) of pixels 2k and 2k + 1.
    // (Stride 2, forward: result pixel e takes the feature pixels 2e - 1, 2e and 2e + 1.)
    constexpr bool kDot2 = sizeof(T) == 2 && K == 3 && D == 1 && VX >= 2 && (S == 1 || !BWD);
    uint32_t sfp[kDot2 ? R : 1][K][kDot2 ? VX : 1], sfs[kDot2 ? R : 1][K][NW];
    if constexpr (kDot2) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int i = 0; i < K; ++i)
#pragma unroll
                for (int k = 0; k < NW; ++k) {
                    const uint32_t a = sfw[r][i * K][k], b = sfw[r][i * K + 1][k];
                    sfp[r][i][2 * k] = (a & 0xffffu) | (b << 16);
                    sfp[r][i][2 * k + 1] = (a >> 16) | (b & 0xffff0000u);
                    sfs[r][i][k] = sfw[r][i * K + 2][k];
                }
    }

    auto compute = [&](auto st_tag, int ci) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value;
        if constexpr (kDot2) {
            // (keep the regrouped taps as they are: see below)
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int i = 0; i < K; ++i) {
#pragma unroll
                    for (int e = 0; e < VX; ++e) asm volatile("" : "+v"(sfp[r][i][e]));
#pragma unroll
                    for (int k = 0; k < NW; ++k) asm volatile("" : "+v"(sfs[r][i][k]));
                }
        } else if constexpr (sizeof(T) == 2) {
            // Keeps the packed taps packed: without this the compiler widens all
            // of them to fp32 ahead of the channel loop, twice the registers.
            // Widened at their one use per channel they fold into the
            // mixed-precision multiply-add at no cost.
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int t = 0; t < KK; ++t)
#pragma unroll
                    for (int k = 0; k < NW; ++k) asm volatile("" : "+v"(sfw[r][t][k]));
        }
        A w[KK];
        uint32_t wp[kDot2 ? K : 1], ws[kDot2 ? K : 1];   // channel taps (i, 0) | (i, 1), and (i, 2) twice
        if constexpr (kScalarTaps) {
#pragma unroll
            for (int t = 0; t < KK; ++t) w[t] = cfu[ST][t];
        } else if constexpr (kDot2) {
            const uint32_t bits = (uint32_t)__builtin_bit_cast(unsigned short, cfl[ST]);
            uint32_t b[KK];
#pragma unroll
            for (int t = 0; t < KK; ++t) b[t] = (uint32_t)__builtin_amdgcn_readlane((int)bits, t);
#pragma unroll
            for (int i = 0; i < K; ++i) {
                wp[i] = b[i * K] | (b[i * K + 1] << 16);
                ws[i] = b[i * K + 2] | (b[i * K + 2] << 16);
            }
        } else {
            const A cfa = (A)ld(&cfl[ST]);
#pragma unroll
            for (int t = 0; t < KK; ++t) w[t] = lane_broadcast<A>(cfa, t);
        }
        if constexpr (S2B) {
            // feature gradient of the lane's two feature rows: the four parity classes of a
            // feature pixel see one, two, two and four taps
            using GRow = ExtRow<T, VX, 1, PAD>;
            GRow g0, g1;
#pragma unroll
            for (int k = 0; k < NW; ++k) { g0.own[k] = xw[ST][0][k]; g1.own[k] = xw[ST][1][k]; }
            g0.sides(ln.first, ln.last);
            g1.sides(ln.first, ln.last);
            // dO * comb(CF[i][j], SF[i][j]) with the spatial tap of slot (i, j)
            auto term = [&](A gv, int i, int j, int e, A acc) __attribute__((always_inline)) {
                const int t = i * K + j;
                const A sv = elem<T>(sfw[0][t], e);
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
            const __amdgpu_buffer_rsrc_t dr = plane_rsrc(os + (int64_t)ci * out_plane, ci < nch ? out_bytes : 0u);
            if constexpr (sizeof(T) == 2) {
                // (round the complete fp32 sums, the same way in every unrolled copy: see below)
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
        } else {
        Row row[ROWS];
#pragma unroll
        for (int rr = 0; rr < ROWS; ++rr) {
            if (!row_needed<R, K, D>(rr)) continue;
#pragma unroll
            for (int k = 0; k < NWX; ++k) row[rr].own[k] = xw[ST][rr][k];
            row[rr].sides(ln.first, ln.last);
        }
        A acc[R][VX];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int e = 0; e < VX; ++e) acc[r][e] = 0;
        if constexpr (kDot2) {
            // pairs of neighbouring feature pixels (e - 1, e) of every window row: the odd e
            // are the row's own words, the even e straddle two words
            uint32_t xp[ROWS][VX];
#pragma unroll
            for (int rr = 0; rr < ROWS; ++rr) {
                if constexpr (S == 1) {
#pragma unroll
                    for (int k = 0; k < NW; ++k) {
                        const uint32_t below = k == 0 ? row[rr].left[Row::SW - 1] : row[rr].own[k - 1];
                        xp[rr][2 * k] = __builtin_amdgcn_alignbit(row[rr].own[k], below, 16);
                        xp[rr][2 * k + 1] = row[rr].own[k];
                    }
                } else {
                    // (2e - 1, 2e): the last element of word e - 1 and the first of word e
#pragma unroll
                    for (int e = 0; e < VX; ++e) {
                        const uint32_t below = e == 0 ? row[rr].left[Row::SW - 1] : row[rr].own[e - 1];
                        xp[rr][e] = __builtin_amdgcn_alignbit(row[rr].own[e], below, 16);
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < K; ++i) {
                const half2_t wpair = __builtin_bit_cast(half2_t, wp[i]);
                const half2_t wlast = __builtin_bit_cast(half2_t, ws[i]);
#pragma unroll
                for (int r = 0; r < R; ++r) {
#pragma unroll
                    for (int e = 0; e < VX; ++e) {
                        const half2_t sp = __builtin_bit_cast(half2_t, sfp[r][i][e]);
                        const half2_t cb = MUL ? wpair * sp : wpair + sp;
                        acc[r][e] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, xp[r + i][e]), cb,
                                                           acc[r][e], false);
                    }
#pragma unroll
                    for (int k = 0; k < NW; ++k) {
                        const half2_t sl = __builtin_bit_cast(half2_t, sfs[r][i][k]);
                        const half2_t cb = MUL ? wlast * sl : wlast + sl;
#pragma unroll
                        for (int h = 0; h < 2; ++h)
                            acc[r][2 * k + h] = fma_(row[r + i].at(S * (2 * k + h) + 1), (A)cb[h], acc[r][2 * k + h]);
                    }
                }
            }
        } else {
        // mul: x * sf is exact in the accumulator type for fp16 storage and goes
        // into one mixed-precision multiply; add: two multiply-adds
#pragma unroll
        for (int i = 0; i < K; ++i)
#pragma unroll
            for (int j = 0; j < K; ++j)
#pragma unroll
                for (int r = 0; r < R; ++r)
#pragma unroll
                    for (int e = 0; e < VX; ++e) {
                        const A xv = row[r + i * D].at(S * e + j * D - HX);
                        const A sv = elem<T>(sfw[r][i * K + j], e);
                        if constexpr (MUL) {
                            acc[r][e] = fma_(w[i * K + j], fma_(xv, sv, A(0)), acc[r][e]);
                        } else {
                            acc[r][e] = fma_(xv, w[i * K + j], acc[r][e]);
                            acc[r][e] = fma_(xv, sv, acc[r][e]);
                        }
                    }
        }   // (not the dot-product path)
        const __amdgpu_buffer_rsrc_t orr = plane_rsrc(os + (int64_t)ci * out_plane, ci < nch ? out_bytes : 0u);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if constexpr (sizeof(T) == 2) {
                // The sum is complete in fp32 before it is rounded to fp16.  Left
                // alone, the compiler fuses the last multiply-add with the rounding
                // in some unrolled copies of this code and not in others, and a
                // result would then depend on which copy its channel falls to.
#pragma unroll
                for (int e = 0; e < VX; ++e) asm volatile("" : "+v"(acc[r][e]));
            }
            uint32_t ow[NW];
            pack<T, VX, A>(acc[r], ow);
            store_vec_nt<kVB>(orr, ob[r], ow);
        }
        }   // (not the stride-2 gradient)
    };

    // Channel ci is computed from stage ci % NST while the loads of channel
    // ci + NST - 1 go out.  The walk is unrolled NST times so that stages are
    // compile-time register sets; it always runs whole rounds of NST channels
    // (one basic block, no tail code): a channel past the wave's last one is
    // computed from zeros and its stores are dropped.
    auto step = [&](auto st_tag, int ci) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value;
        // The loads of channel ci + NST - 1 go out before the arithmetic of channel ci,
        // and nothing moves from one step into another: left to itself the scheduler
        // sinks the loads to where their values are needed, which leaves nothing in flight.
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
}

#endif  // __HIPCC__

}  // namespace rows

// Host-side geometry (ddf_rows_host.hip).  Fills *g and names the kernel
// instantiation (*vx elements per lane and row, *r rows per lane; g->lp >
// g->lpr selects the PAD kernels); false when the family does not cover the
// problem.
bool rows_geometry(const Problem &p, int dtype, int max_vx, RowsGeom *g, int *vx, int *r);

}  // namespace ddf
