// Wavefront-per-strip DDF kernels for gfx950: forward, feature gradient, filter
// gradients (optionally with the feature gradient fused in).
//
// One 64-lane wavefront owns a full-width row strip of one sample and walks a
// range of its channels.  Lanes are laid out 2-D over the strip's work cells -
// LW = 2^k >= cols lanes per cell row, 64/LW cell rows per pass ("slot"), PS
// slots per lane - so that LDS addresses are linear in the lane id (no bank
// conflicts) and no division is needed to find a cell.
//
// Per channel the wave
//   1. copies the source strip (X, dO) from global memory with 16-byte loads, a
//      few channels ahead of use, and scatters it into a zero-bordered LDS tile
//      of accumulator-type values (the border makes the tap loop free of bounds
//      tests; fp16 is widened here, once per element),
//   2. runs the tap loop for its PS cells out of LDS, with the spatial-filter
//      taps of those cells held in registers for the whole channel walk and
//      the channel-filter taps of its channels staged once in LDS (read back as
//      wave-uniform values),
//   3. writes the results to a linear LDS copy of the result strip and stores
//      that with 16-byte accesses.
// The global side is therefore a plain linear copy in both directions, and in
// the channel walk a wave never waits for another wave: there is no workgroup
// barrier in forward and feature gradient, and only the final dSF sum over a
// block's four waves has barriers in the filter-gradient kernel.
#pragma once

#include <type_traits>

#include "ddf_common.h"

namespace ddf {

constexpr int kMaxSlots = 8;

struct WaveGeom {
    int C, H, W, Ho, Wo;      // problem (per sample)
    int rows, cols;           // grid of work cells a strip is cut from
    int lw_shift;             // lanes per cell row segment = 1 << lw_shift
    int TH, nstrips;          // cell rows per strip
    int nslots;               // slots in use (<= PS of the kernel launched)
    // staged source plane (X, or dO for the feature gradient) and its zero-bordered tile
    int src_rows, src_cols;
    int P, IH, tile;          // tile: IH rows of pitch P elements, `tile` elements reserved
    int row0_off, col_off;    // source row of tile row 0 in strip 0; tile column of source column 0
    int lb_shift;             // tile columns left of the leftmost tap (border wider than the halo)
    int wide;                 // 1: a source vector lands on 4 aligned tile elements (one 16-byte LDS write)
    // result strip (out, or dX): `lin_cols` elements per row, `lin_rpc` rows per cell row
    int lin_cols, lin_rpc, lin_rows, lin_tile;
    int cpw, csplit;          // channels per wave; number of channel ranges (of cpw * waves per block)
    int cpb;                  // channels per block (= cpw for the one-wave kernels)
    int wpb;                  // independent waves per workgroup (forward, feature gradient)
    int lds_wave_bytes;       // LDS of one wave (filter-gradient blocks hold four)
    int vec, nv;              // elements per global access; vectors per lane per channel strip
    unsigned src_magic;       // ceil(2^32 / src_cols); 0 when src_cols == 1
    unsigned csplit_magic, nstrips_magic, xcd_per;   // same for the block id split; blocks per XCD
    int nblocks;              // = N * nstrips * csplit
    int lds_bytes;
    int slot_row[kMaxSlots];  // cell row (within the strip) of lane row 0 in slot m
    int slot_col[kMaxSlots];  // cell column of lane column 0 in slot m
};

namespace wave {

constexpr int kXcd = 8;
// Most independent waves a workgroup of the forward / feature-gradient kernels holds.
constexpr int kMaxWpb = 4;
// Spare LDS elements behind each tile: idle lanes write there instead of branching.
constexpr int kSpare = 8;
// Spare elements behind each linear result strip: one per lane, where idle
// lanes put their (meaningless) results without an address conflict.
constexpr int kIdle = kWave;

template <typename T, int V>
struct alignas(sizeof(T) * V) Vec {
    T e[V];
};

// Register image of V elements that are only moved, never computed on.
template <int BYTES> struct RawBytes;
template <> struct RawBytes<2> { using type = uint16_t; };
template <> struct RawBytes<4> { using type = uint32_t; };
template <> struct RawBytes<8> { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <> struct RawBytes<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };
template <> struct RawBytes<32> { typedef uint32_t type __attribute__((ext_vector_type(8))); };
template <typename T, int V>
using Raw = typename RawBytes<sizeof(T) * V>::type;

// Compiler-level ordering point between LDS writes and the reads of other
// lanes of the same wavefront.  The LDS unit executes one wave's instructions
// in order, so no hardware wait is needed.
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Workgroups are handed to the 8 XCDs round-robin by hardware.  Renumber them
// so that consecutive logical blocks (same sample, neighbouring channel
// ranges: same spatial filter) share an XCD and its L2.
// q = n / d through the host's magic number m = ceil(2^32 / d) (0: d == 1);
// exact while n * d < 2^32, which the host checks.
__device__ __forceinline__ int magic_div(int n, unsigned m) {
    return m ? (int)__umulhi((unsigned)n, m) : n;
}

// Pins a wave-uniform value in a scalar register.  Without it the compiler
// re-reads kernel arguments from memory inside the channel loop, and the wait
// for such a read also waits for every LDS access in flight.
__device__ __forceinline__ int pin(int v) {
    v = __builtin_amdgcn_readfirstlane(v);
    asm volatile("" : "+s"(v));
    return v;
}

struct WaveWork {
    int cs, strip, row_first, nrows, c_begin, c_end;
    int64_t n;
    // `wave`: index of the calling wave among the g.wpb independent waves of
    // its workgroup (0 for kernels whose workgroup is the unit of work)
    __device__ __forceinline__ bool init(const WaveGeom &g, int wave = 0) {
        const int wg = (int)(blockIdx.x % kXcd) * (int)g.xcd_per + (int)(blockIdx.x / kXcd);
        const int b = wg * g.wpb + wave;
        if (wave >= g.wpb || b >= g.nblocks) return false;
        const int rest = magic_div(b, g.csplit_magic);
        cs = b - rest * g.csplit;
        const int smp = magic_div(rest, g.nstrips_magic);
        strip = rest - smp * g.nstrips;
        n = smp;
        row_first = strip * g.TH;
        nrows = min(g.TH, g.rows - row_first);
        c_begin = cs * g.cpb;
        c_end = min(g.C, c_begin + g.cpb);
        return true;
    }
};

// Channel-filter taps of the wave's channels.  Read once, with one coalesced
// vector load, into LDS as accumulator-type values (kTapPitch<KK> per channel,
// 16-byte aligned); the per-channel reads are then wave-uniform LDS reads that
// never wait on global memory.  (A scalar load per channel would be a cold
// miss to HBM on the critical path of every channel.)
template <int KK>
constexpr int tap_pitch() { return (KK + 3) / 4 * 4; }

// Loads of at most kTapLoads * 64 tap values start here, before anything
// waits; put() writes them to LDS later.  The host keeps cpw * KK within that.
constexpr int kTapLoads = 4;
template <int KK, typename T, typename A>
struct TapStager {
    T v[kTapLoads];
    __device__ __forceinline__ void issue(const T *__restrict__ cf, int64_t nc0, int nch,
                                          int lane) {
        const T *src = cf + nc0 * KK;
#pragma unroll
        for (int r = 0; r < kTapLoads; ++r) {
            const int i = lane + r * kWave;
            v[r] = src[min(i, nch * KK - 1)];      // clamped: no branch
        }
    }
    __device__ __forceinline__ void put(A *taps, int nch, int lane) const {
#pragma unroll
        for (int r = 0; r < kTapLoads; ++r) {
            const int i = lane + r * kWave;
            const int c = i / KK, t = i - c * KK;
            if (i < nch * KK) taps[c * tap_pitch<KK>() + t] = ld(&v[r]);
        }
    }
};

template <int KK, typename A>
__device__ __forceinline__ void load_taps(const A *taps, int ci, A (&w)[KK]) {
#pragma unroll
    for (int t = 0; t < KK; ++t) w[t] = taps[ci * tap_pitch<KK>() + t];
}

// Channels in flight per wave for a given number of vectors per channel.
// (Deeper pipelines for the narrow element types were measured and do not pay:
// the extra registers cost more occupancy than the prefetch distance gains.)
template <int NV>
constexpr int stages() { return NV <= 1 ? 4 : (NV <= 2 ? 2 : 1); }

// Source strip -> zero-bordered LDS tile, through registers.  The strip of one
// channel is a run of n_in contiguous elements; lane l owns vectors
// f = l, l + 64, ... of it.  Their tile offsets are computed once.
template <typename T, int V, int NV, int MAXST = 4>
struct Stager {
    static constexpr int NST = stages<NV>() < MAXST ? stages<NV>() : MAXST;
    int goff[NV];        // element offset of the vector inside a source plane
    int lo[NV][V];       // tile offset of each element
    Vec<T, V> v[NST][NV];

    // Lanes without a vector load plane element 0 and write to the spare cell
    // behind the tile, so that neither issue() nor commit() branches: the
    // compiler then counts outstanding loads exactly and a commit waits only
    // for its own stage.
    // init_global() is all that issue() needs; init_tile() (the costly part)
    // can run while the first loads are in flight.
    __device__ __forceinline__ void init_global(const WaveGeom &g, int row0, int lane) {
        const int r_lo = max(row0, 0);
        const int n_rows = max(min(row0 + g.IH, g.src_rows) - r_lo, 0);
        const int nvec = n_rows * g.src_cols / V;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int f = lane + j * kWave;
            goff[j] = f < nvec ? r_lo * g.src_cols + f * V : 0;
        }
    }
    __device__ __forceinline__ void init_tile(const WaveGeom &g, int row0, int lane) {
        const int r_lo = max(row0, 0);
        const int n_rows = max(min(row0 + g.IH, g.src_rows) - r_lo, 0);
        const int nvec = n_rows * g.src_cols / V;
        const int row_shift = r_lo - row0;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int f = lane + j * kWave;
            const int e = f * V;
            int row = magic_div(e, g.src_magic);
            int col = e - row * g.src_cols;
            const bool used = f < nvec;
#pragma unroll
            for (int k = 0; k < V; ++k) {
                lo[j][k] = used ? (row_shift + row) * g.P + g.col_off + col : g.tile + k;
                if (++col >= g.src_cols) { col = 0; ++row; }
            }
        }
    }
    __device__ __forceinline__ void init(const WaveGeom &g, int row0, int lane) {
        init_global(g, row0, lane);
        init_tile(g, row0, lane);
    }
    template <int ST>
    __device__ __forceinline__ void issue(const T *__restrict__ plane) {
#pragma unroll
        for (int j = 0; j < NV; ++j)
            v[ST][j] = *reinterpret_cast<const Vec<T, V> *>(plane + goff[j]);
    }
    // The tile holds accumulator-type values: fp16 is widened here, once per
    // element, instead of once per tap read; the tap reads are then aligned
    // 4-byte accesses for every storage type.
    // `wide`: the geometry guarantees that the V = 4 elements of a vector are
    // neighbours in the tile and start on a 16-byte boundary, so they go out as
    // one write; the element-wise scatter has lanes 4 elements apart, an
    // 8-way bank conflict per instruction.
    template <int ST>
    __device__ __forceinline__ void commit(typename Acc<T>::type *lds, bool wide = false) const {
        using A = typename Acc<T>::type;
        if constexpr (V == 4 && sizeof(A) == 4) {
            if (wide) {
#pragma unroll
                for (int j = 0; j < NV; ++j) {
                    Vec<A, 4> w;
#pragma unroll
                    for (int k = 0; k < 4; ++k) w.e[k] = ld(&v[ST][j].e[k]);
                    *reinterpret_cast<Raw<A, 4> *>(lds + lo[j][0]) = __builtin_bit_cast(Raw<A, 4>, w);
                }
                return;
            }
        }
#pragma unroll
        for (int j = 0; j < NV; ++j)
#pragma unroll
            for (int k = 0; k < V; ++k) lds[lo[j][k]] = ld(&v[ST][j].e[k]);
    }
};

// Linear LDS strip -> global memory, V elements per access.
template <typename T, int V>
__device__ __forceinline__ void store_strip(const T *lds, T *__restrict__ dst, int n_elems,
                                            int lane) {
    const int nvec = n_elems / V;
    for (int f = lane; f < nvec; f += kWave)
        __builtin_nontemporal_store(*reinterpret_cast<const Raw<T, V> *>(lds + f * V),
                                    reinterpret_cast<Raw<T, V> *>(dst + f * V));
}

template <typename T>
__device__ __forceinline__ void zero_tile(T *lds, int n, int lane) {
    // `n` is a multiple of 8 elements and the tile is 16-byte aligned
    constexpr int W16 = 16 / sizeof(T);
    Vec<T, W16> z;
#pragma unroll
    for (int k = 0; k < W16; ++k) z.e[k] = T(0.0f);
    for (int i = lane * W16; i < n; i += kWave * W16) *reinterpret_cast<Vec<T, W16> *>(lds + i) = z;
}

// Spatial-filter taps of a lane's cells.  A lane-per-cell gather would cost
// KK * PS four-byte load instructions per wave, and at a few channels per wave
// those loads, not the feature maps, fill the memory pipeline.  Instead the
// strip of every tap plane is read as a linear run with V-element accesses (NG
// per lane and tap), passed through a linear LDS buffer and picked up per cell.
template <typename T, int V, int NG, int KK>
struct FilterStager {
    int off[NG];   // element offset inside the strip; lanes past its end repeat vector 0
    Raw<T, V> v[KK][NG];
    __device__ __forceinline__ void init(int n_elems, int lane) {
#pragma unroll
        for (int j = 0; j < NG; ++j) {
            const int f = lane + j * kWave;
            off[j] = f < n_elems / V ? f * V : 0;
        }
    }
    // tap t of the strip starts at strip0 + t * plane
    template <int TT = 0>
    __device__ __forceinline__ void issue(const T *__restrict__ strip0, int64_t plane) {
        if constexpr (TT < KK) {
#pragma unroll
            for (int j = 0; j < NG; ++j)
                v[TT][j] = *reinterpret_cast<const Raw<T, V> *>(strip0 + TT * plane + off[j]);
            issue<TT + 1>(strip0, plane);
        }
    }
    // lds: at least n_elems elements; idx[m]: element of the lane's cell m
    template <int TT = 0, int PS, typename A>
    __device__ __forceinline__ void collect(T *lds, const int (&idx)[PS], A (&sfr)[PS][KK]) const {
        if constexpr (TT < KK) {
#pragma unroll
            for (int j = 0; j < NG; ++j)
                *reinterpret_cast<Raw<T, V> *>(lds + off[j]) = v[TT][j];
            wave_sync();
#pragma unroll
            for (int m = 0; m < PS; ++m) sfr[m][TT] = ld(lds + idx[m]);
            wave_sync();
            collect<TT + 1>(lds, idx, sfr);
        }
    }
};

// ---------------------------------------------------------------------------
// Forward: work cell = output pixel.
// ---------------------------------------------------------------------------
template <typename T, int K, int D, int S, bool MUL, int PS, int NV, int V>
__global__ __launch_bounds__(kWave * kMaxWpb) void k_forward(WaveGeom g, const T *__restrict__ x,
                                                   const T *__restrict__ cf,
                                                   const T *__restrict__ sf,
                                                   T *__restrict__ out) {
    using A = typename Acc<T>::type;
    constexpr int KK = K * K;
    constexpr bool kFlat = KK <= 9;   // tap loop without branches (see there)
    using Stg = Stager<T, V, NV>;
    constexpr int NST = Stg::NST;
    extern __shared__ __align__(16) unsigned char smem[];
    // the waves of a workgroup are independent: each has its own work and LDS
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    A *lds_in = reinterpret_cast<A *>(smem + (size_t)wave * g.lds_wave_bytes);
    T *lds_out = reinterpret_cast<T *>(lds_in + g.tile + kSpare);
    A *taps = reinterpret_cast<A *>(lds_out + g.lin_tile + kIdle);

    WaveWork ww;
    if (!ww.init(g, wave) || ww.c_end <= ww.c_begin) return;
    const int lr = lane >> g.lw_shift, lc = lane & ((1 << g.lw_shift) - 1);
    const int64_t oplane = (int64_t)g.Ho * g.Wo, iplane = (int64_t)g.H * g.W;
    const int y0 = ww.row_first;
    const int nch = ww.c_end - ww.c_begin;
    const int n_out = ww.nrows * g.Wo;
    // Every load of the prologue is issued before anything else is set up and
    // before the first wait: the feature strips of the first NST channels
    // (clamped to the last channel, so that they are unconditional), the
    // spatial filter, the channel-filter taps.  The index arithmetic below
    // then runs under one trip to memory.
    Stg stg;
    stg.init_global(g, y0 * S + g.row0_off, lane);
    const T *xs = x + (ww.n * g.C + ww.c_begin) * iplane;
    T *os = out + (ww.n * g.C + ww.c_begin) * oplane + (int64_t)y0 * g.Wo;
    stg.template issue<0>(xs);
    if constexpr (NST > 1) stg.template issue<1>(xs + (int64_t)min(1, nch - 1) * iplane);
    if constexpr (NST > 2) stg.template issue<2>(xs + (int64_t)min(2, nch - 1) * iplane);
    if constexpr (NST > 3) stg.template issue<3>(xs + (int64_t)min(3, nch - 1) * iplane);
    FilterStager<T, V, (PS + V - 1) / V, KK> fst;
    fst.init(n_out, lane);
    fst.issue(sf + (ww.n * KK * g.Ho + y0) * g.Wo, oplane);
    TapStager<KK, T, A> tst;
    tst.issue(cf, ww.n * g.C + ww.c_begin, nch, lane);

    // per slot: is the cell real, where its taps start in the tile, where its
    // result goes in the linear strip; its spatial-filter taps in registers
    bool ok[PS];
    int lb[PS], ob[PS], wb[PS];
    A sfr[PS][KK];
#pragma unroll
    for (int m = 0; m < PS; ++m) {
        const int row = g.slot_row[m] + lr, col = g.slot_col[m] + lc;
        ok[m] = m < g.nslots && row < ww.nrows && col < g.cols;
        // idle lanes keep their lane-linear tile address (inside the LDS
        // allocation): a shared dummy address would collide with the banks of
        // the working lanes and double the time of every tap read
        lb[m] = (row * S) * g.P + col * S + g.lb_shift;
        ob[m] = ok[m] ? row * g.Wo + col : 0;   // idle lanes pick up pixel 0 (unused)
        wb[m] = ok[m] ? ob[m] : g.lin_tile + lane;   // ... and write behind the strip
    }
    stg.init_tile(g, y0 * S + g.row0_off, lane);
    const int P = pin(g.P);
    const bool wide = g.wide != 0;
    zero_tile(lds_in, g.tile, lane);
    tst.put(taps, nch, lane);
    fst.collect(lds_out, ob, sfr);

    auto channel = [&](auto st_tag, int ci) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value;
        stg.template commit<ST>(lds_in, wide);
        stg.template issue<ST>(xs + (int64_t)min(ci + NST, nch - 1) * iplane);
        wave_sync();
        A w[KK];
        load_taps<KK>(taps, ci, w);
        if constexpr (kFlat) {
            // No branch in here: every slot is computed, idle lanes and idle
            // slots included (their tile addresses are valid), and the results
            // are written after all reads (a write in between would order the
            // reads of the next slot behind it).  The compiler can then overlap
            // the LDS reads of one slot with the arithmetic of another.
            A acc[PS];
#pragma unroll
            for (int m = 0; m < PS; ++m) {
                acc[m] = 0;
#pragma unroll
                for (int i = 0; i < K; ++i)
#pragma unroll
                    for (int j = 0; j < K; ++j)
                        acc[m] += (A)ld(lds_in + lb[m] + i * D * P + j * D) *
                                  comb<MUL, A>(w[i * K + j], sfr[m][i * K + j]);
            }
#pragma unroll
            for (int m = 0; m < PS; ++m) st(lds_out + wb[m], acc[m]);
        } else {
            // many taps: one slot at a time keeps the register count down
#pragma unroll
            for (int m = 0; m < PS; ++m) {
                if (m >= g.nslots) break;
                A acc = 0;
#pragma unroll
                for (int i = 0; i < K; ++i)
#pragma unroll
                    for (int j = 0; j < K; ++j)
                        acc += (A)ld(lds_in + lb[m] + i * D * P + j * D) *
                               comb<MUL, A>(w[i * K + j], sfr[m][i * K + j]);
                if (ok[m]) st(lds_out + ob[m], acc);
            }
        }
        wave_sync();
        store_strip<T, V>(lds_out, os + (int64_t)ci * oplane, n_out, lane);
        wave_sync();
    };

    auto group = [&](int c) __attribute__((always_inline)) {
        channel(std::integral_constant<int, 0>{}, c);
        if constexpr (NST > 1) channel(std::integral_constant<int, 1>{}, c + 1);
        if constexpr (NST > 2) channel(std::integral_constant<int, 2>{}, c + 2);
        if constexpr (NST > 3) channel(std::integral_constant<int, 3>{}, c + 3);
    };
    // The first group is peeled off the loop: the loop is then entered only in
    // its steady state (NST loads and NST stores in flight), and the wait the
    // compiler places before a commit covers that stage's load alone instead
    // of draining the younger loads and stores as well.
    const int nfull = nch / NST * NST;
    if (nfull > 0) {
        group(0);
        for (int c = NST; c < nfull; c += NST) group(c);
    }
    if constexpr (NST > 1) {
        // the last nch % NST channels already sit in stages 0, 1, ...
        if (nfull < nch) channel(std::integral_constant<int, 0>{}, nfull);
        if constexpr (NST > 2) {
            if (nfull + 1 < nch) channel(std::integral_constant<int, 1>{}, nfull + 1);
            if (nfull + 2 < nch) channel(std::integral_constant<int, 2>{}, nfull + 2);
        }
    }
}

// ---------------------------------------------------------------------------
// Gradient with respect to the features.  Work cell (qy, qx) = the S x S block
// of input pixels (qy*S + pu, qx*S + pv).  Input pixel row u receives tap row
// i only when u - (i-R)*D is a multiple of S; with e = (i-R)*D that fixes the
// phase pu = e mod S and the output row qy + (pu - e)/S, both compile-time.
// dO is staged in the zero-bordered tile, the spatial filter is gathered at
// the neighbour positions once per cell and kept in registers, and the S*S
// results of a cell go to the linear copy of the dX strip.
// ---------------------------------------------------------------------------
template <int K, int D, int S>
struct TapMap {
    static constexpr int R = (K - 1) / 2;
    static constexpr int e(int i) { return (i - R) * D; }
    static constexpr int phase(int i) { return ((e(i) % S) + S) % S; }
    static constexpr int dq(int i) { return (phase(i) - e(i)) / S; }
    static constexpr int halo_lo = (R * D) / S;            // cells above / left
    static constexpr int halo_hi = (R * D + S - 1) / S;    // cells below / right
};

// Spatial-filter taps at the neighbour positions of a lane's cells.  Each tap
// plane has the shape of dO, so its strip is brought in exactly like a dO strip
// (same vector offsets, same zero-bordered tile: neighbours outside the image
// read as zero) and every cell picks its neighbour out of the tile.
template <typename T, int V, int NV, int K, int D, int S>
struct NeighbourFilterStager {
    static constexpr int KK = K * K;
    using TM = TapMap<K, D, S>;
    Vec<T, V> v[KK][NV];
    template <int TT = 0>
    __device__ __forceinline__ void issue(const T *__restrict__ sf_n, int64_t plane,
                                          const int (&goff)[NV]) {
        if constexpr (TT < KK) {
#pragma unroll
            for (int j = 0; j < NV; ++j)
                v[TT][j] = *reinterpret_cast<const Vec<T, V> *>(sf_n + TT * plane + goff[j]);
            issue<TT + 1>(sf_n, plane, goff);
        }
    }
    template <int TT = 0, int PS, typename A>
    __device__ __forceinline__ void collect(A *tile, const int (&lo)[NV][V],
                                            const int (&lb)[PS], int P,
                                            A (&sfg)[PS][KK]) const {
        if constexpr (TT < KK) {
            constexpr int i = TT / K, j = TT % K;
#pragma unroll
            for (int q = 0; q < NV; ++q)
#pragma unroll
                for (int k = 0; k < V; ++k) tile[lo[q][k]] = ld(&v[TT][q].e[k]);
            wave_sync();
#pragma unroll
            for (int m = 0; m < PS; ++m)
                sfg[m][TT] = ld(tile + lb[m] + (TM::dq(i) + TM::halo_lo) * P + TM::dq(j) +
                                TM::halo_lo);
            wave_sync();
            collect<TT + 1>(tile, lo, lb, P, sfg);
        }
    }
};

template <typename T, int K, int D, int S, bool MUL, int PS, int NV, int V>
__global__ __launch_bounds__(kWave * kMaxWpb) void k_backward_features(
    WaveGeom g, const T *__restrict__ go, const T *__restrict__ cf,
    const T *__restrict__ sf, T *__restrict__ dx) {
    using A = typename Acc<T>::type;
    using TM = TapMap<K, D, S>;
    constexpr int KK = K * K;
    constexpr bool kFlat = KK <= 9 && S == 1;   // tap loop without branches (see k_forward)
    using Stg = Stager<T, V, NV>;
    constexpr int NST = Stg::NST;
    extern __shared__ __align__(16) unsigned char smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    A *lds_in = reinterpret_cast<A *>(smem + (size_t)wave * g.lds_wave_bytes);
    T *lds_out = reinterpret_cast<T *>(lds_in + g.tile + kSpare);
    A *taps = reinterpret_cast<A *>(lds_out + g.lin_tile + kIdle);

    WaveWork ww;
    if (!ww.init(g, wave) || ww.c_end <= ww.c_begin) return;
    const int lr = lane >> g.lw_shift, lc = lane & ((1 << g.lw_shift) - 1);
    const int64_t oplane = (int64_t)g.Ho * g.Wo, iplane = (int64_t)g.H * g.W;
    const int qy0 = ww.row_first;
    const int u0 = qy0 * S;                                     // first dX row of the strip
    const int n_out = min(ww.nrows * S, g.H - u0) * g.W;        // its element count
    const int nch = ww.c_end - ww.c_begin;
    // all loads of the prologue first (see k_forward), index arithmetic under them
    Stg stg;
    stg.init_global(g, qy0 + g.row0_off, lane);
    const T *gs = go + (ww.n * g.C + ww.c_begin) * oplane;
    T *ds = dx + (ww.n * g.C + ww.c_begin) * iplane + (int64_t)u0 * g.W;
    stg.template issue<0>(gs);
    if constexpr (NST > 1) stg.template issue<1>(gs + (int64_t)min(1, nch - 1) * oplane);
    if constexpr (NST > 2) stg.template issue<2>(gs + (int64_t)min(2, nch - 1) * oplane);
    if constexpr (NST > 3) stg.template issue<3>(gs + (int64_t)min(3, nch - 1) * oplane);
    // Few vectors per plane: bring the filter in through the tile.  Otherwise
    // (scalar accesses, or more registers than the taps themselves) gather it.
    constexpr bool kStageFilter = V > 1 && NV * V <= 8;
    NeighbourFilterStager<T, V, kStageFilter ? NV : 1, K, D, S> nfs;
    if constexpr (kStageFilter) nfs.issue(sf + ww.n * KK * oplane, oplane, stg.goff);
    TapStager<KK, T, A> tst;
    tst.issue(cf, ww.n * g.C + ww.c_begin, nch, lane);

    bool ok[PS];
    int lb[PS], ob[PS], cu[PS], cv[PS];
    A sfg[PS][KK];
#pragma unroll
    for (int m = 0; m < PS; ++m) {
        const int ql = g.slot_row[m] + lr, cx = g.slot_col[m] + lc;
        const int cy = qy0 + ql;
        ok[m] = m < g.nslots && ql < ww.nrows && cx < g.cols;
        lb[m] = ql * g.P + cx + g.lb_shift;   // idle lanes keep a lane-linear (bank-conflict-free) address
        ob[m] = ok[m] ? (ql * S) * g.W + cx * S : 0;
        // idle cells get coordinates outside the image: none of their results is kept
        cu[m] = ok[m] ? cy * S : g.H;
        cv[m] = cx * S;
    }
    if constexpr (!kStageFilter) {
#pragma unroll
        for (int m = 0; m < PS; ++m) {
            const int cy = qy0 + g.slot_row[m] + lr, cx = g.slot_col[m] + lc;
#pragma unroll
            for (int i = 0; i < K; ++i)
#pragma unroll
                for (int j = 0; j < K; ++j) {
                    const int sy = cy + TM::dq(i), sx = cx + TM::dq(j);
                    const bool in = ok[m] && sy >= 0 && sy < g.Ho && sx >= 0 && sx < g.Wo;
                    // out-of-range neighbours read element 0 and are zeroed: no branch
                    const A val = ld(sf + (ww.n * KK + i * K + j) * oplane +
                                     (in ? (int64_t)sy * g.Wo + sx : 0));
                    sfg[m][i * K + j] = in ? val : A(0);
                }
        }
    }
    stg.init_tile(g, qy0 + g.row0_off, lane);
    const int P = pin(g.P);
    const bool wide = g.wide != 0;
    const int idle = g.lin_tile + lane;
    zero_tile(lds_in, g.tile, lane);
    tst.put(taps, nch, lane);
    wave_sync();
    if constexpr (kStageFilter) nfs.collect(lds_in, stg.lo, lb, g.P, sfg);

    auto channel = [&](auto st_tag, int ci) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value;
        stg.template commit<ST>(lds_in, wide);
        stg.template issue<ST>(gs + (int64_t)min(ci + NST, nch - 1) * oplane);
        wave_sync();
        A w[KK];
        load_taps<KK>(taps, ci, w);
        if constexpr (kFlat) {
            // branch-free, results written after all reads (see k_forward)
            A acc[PS][S][S];
#pragma unroll
            for (int m = 0; m < PS; ++m) {
#pragma unroll
                for (int a = 0; a < S; ++a)
#pragma unroll
                    for (int c = 0; c < S; ++c) acc[m][a][c] = 0;
#pragma unroll
                for (int i = 0; i < K; ++i)
#pragma unroll
                    for (int j = 0; j < K; ++j) {
                        const A gv = ld(lds_in + lb[m] + (TM::dq(i) + TM::halo_lo) * P + TM::dq(j) +
                                        TM::halo_lo);
                        acc[m][TM::phase(i)][TM::phase(j)] +=
                            gv * comb<MUL, A>(w[i * K + j], sfg[m][i * K + j]);
                    }
            }
#pragma unroll
            for (int m = 0; m < PS; ++m)
#pragma unroll
                for (int a = 0; a < S; ++a)
#pragma unroll
                    for (int c = 0; c < S; ++c) {
                        // pixels outside the image (idle cells, odd H or W) go behind the strip
                        const bool in = cu[m] + a < g.H && cv[m] + c < g.W;
                        st(lds_out + (in ? ob[m] + a * g.W + c : idle), acc[m][a][c]);
                    }
        } else {
#pragma unroll
            for (int m = 0; m < PS; ++m) {
                if (m >= g.nslots) break;
                A acc[S][S];
#pragma unroll
                for (int a = 0; a < S; ++a)
#pragma unroll
                    for (int c = 0; c < S; ++c) acc[a][c] = 0;
#pragma unroll
                for (int i = 0; i < K; ++i)
#pragma unroll
                    for (int j = 0; j < K; ++j) {
                        const A gv = ld(lds_in + lb[m] + (TM::dq(i) + TM::halo_lo) * P +
                                        TM::dq(j) + TM::halo_lo);
                        acc[TM::phase(i)][TM::phase(j)] +=
                            gv * comb<MUL, A>(w[i * K + j], sfg[m][i * K + j]);
                    }
#pragma unroll
                for (int a = 0; a < S; ++a)
#pragma unroll
                    for (int c = 0; c < S; ++c) {
                        if (cu[m] + a < g.H && cv[m] + c < g.W)
                            st(lds_out + ob[m] + a * g.W + c, acc[a][c]);
                    }
            }
        }
        wave_sync();
        store_strip<T, V>(lds_out, ds + (int64_t)ci * iplane, n_out, lane);
        wave_sync();
    };

    auto group = [&](int c) __attribute__((always_inline)) {
        channel(std::integral_constant<int, 0>{}, c);
        if constexpr (NST > 1) channel(std::integral_constant<int, 1>{}, c + 1);
        if constexpr (NST > 2) channel(std::integral_constant<int, 2>{}, c + 2);
        if constexpr (NST > 3) channel(std::integral_constant<int, 3>{}, c + 3);
    };
    // The first group is peeled off the loop: the loop is then entered only in
    // its steady state (NST loads and NST stores in flight), and the wait the
    // compiler places before a commit covers that stage's load alone instead
    // of draining the younger loads and stores as well.
    const int nfull = nch / NST * NST;
    if (nfull > 0) {
        group(0);
        for (int c = NST; c < nfull; c += NST) group(c);
    }
    if constexpr (NST > 1) {
        if (nfull < nch) channel(std::integral_constant<int, 0>{}, nfull);
        if constexpr (NST > 2) {
            if (nfull + 1 < nch) channel(std::integral_constant<int, 1>{}, nfull + 1);
            if (nfull + 2 < nch) channel(std::integral_constant<int, 2>{}, nfull + 2);
        }
    }
}

// Linear strip (dO of the filter gradients) -> linear LDS copy, through
// registers, V elements per access; lane l owns vectors l, l + 64, ...
template <typename T, int V, int NG, int NST>
struct LinStager {
    int off[NG];   // element offset inside the strip; lanes past its end repeat vector 0
    Raw<T, V> v[NST][NG];
    __device__ __forceinline__ void init(int n_elems, int lane) {
#pragma unroll
        for (int j = 0; j < NG; ++j) {
            const int f = lane + j * kWave;
            off[j] = f < n_elems / V ? f * V : 0;
        }
    }
    template <int ST>
    __device__ __forceinline__ void issue(const T *__restrict__ strip) {
#pragma unroll
        for (int j = 0; j < NG; ++j)
            v[ST][j] = *reinterpret_cast<const Raw<T, V> *>(strip + off[j]);
    }
    template <int ST>
    __device__ __forceinline__ void commit(T *lds) const {
#pragma unroll
        for (int j = 0; j < NG; ++j)
            *reinterpret_cast<Raw<T, V> *>(lds + off[j]) = v[ST][j];
    }
};

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int CTRL>
__device__ __forceinline__ double dpp_move(double v) {
    const long long b = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_update_dpp(0, (int)(b & 0xffffffffll), CTRL, 0xf, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(0, (int)(b >> 32), CTRL, 0xf, 0xf, false);
    return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}

// Value held by the partner lane of butterfly stage STAGE.  Stages 0, 1, 3
// are swaps (lane^1, lane^2, lane^8); stage 2 rotates the 16-lane row by 4, so
// a lane receives from the quad next to its own: after stage 3 the two
// rotations have covered all four quads of the row.  Stages 4, 5 cross rows.
template <int STAGE, typename A>
__device__ __forceinline__ A lane_xchg(A v) {
    if constexpr (STAGE == 0) return dpp_move<0xB1>(v);        // quad_perm [1,0,3,2]
    else if constexpr (STAGE == 1) return dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
    else if constexpr (STAGE == 2) return dpp_move<0x124>(v);  // row_ror:4
    else if constexpr (STAGE == 3) return dpp_move<0x128>(v);  // row_ror:8
    else if constexpr (STAGE == 4) return __shfl_xor(v, 16, kWave);
    else return __shfl_xor(v, 32, kWave);
}

// Sum each of N per-lane values over the 64 lanes of the wavefront.  At every
// stage a lane keeps one half of its values and hands the other half to its
// partner, so the work is ~3N instructions instead of 6N.  Returns the total
// of the value whose index g_bfly_table<N> lists for this lane.
template <int N, int STAGE, typename A>
__device__ __forceinline__ A bfly_sum(const A (&v)[N], int lane) {
    if constexpr (STAGE == 6) {
        static_assert(N == 1, "at most 64 values");
        return v[0];
    } else {
        constexpr int h = N / 2, M = h + (N & 1);
        A nv[M];
        const bool up = (lane >> STAGE) & 1;
#pragma unroll
        for (int j = 0; j < h; ++j) {
            const A keep = up ? v[j + h] : v[j];
            const A send = up ? v[j] : v[j + h];
            nv[j] = keep + lane_xchg<STAGE>(send);
        }
        if constexpr (N & 1) nv[h] = v[2 * h] + lane_xchg<STAGE>(v[2 * h]);
        return bfly_sum<M, STAGE + 1, A>(nv, lane);
    }
}

// Index of the value whose total bfly_sum() leaves in `lane`: the same
// keep/send choices replayed on indices, evaluated at compile time.
constexpr int bfly_index_of(int n, int lane) {
    int id[kWave] = {};
    for (int i = 0; i < n; ++i) id[i] = i;
    int cnt = n;
    for (int stage = 0; stage < 6; ++stage) {
        const int h = cnt / 2;
        const bool up = (lane >> stage) & 1;
        int nid[kWave] = {};
        for (int j = 0; j < h; ++j) nid[j] = up ? id[j + h] : id[j];
        if (cnt & 1) nid[h] = id[2 * h];
        cnt = h + (cnt & 1);
        for (int j = 0; j < cnt; ++j) id[j] = nid[j];
    }
    return id[0];
}
template <int N>
struct BflyTable {
    int tap[kWave];
    constexpr BflyTable() : tap{} {
        for (int l = 0; l < kWave; ++l) tap[l] = bfly_index_of(N, l);
    }
};
template <int N>
__device__ const BflyTable<N> g_bfly_table{};

// Lanes below this bound hold every index at least once after the reduction.
template <int N>
constexpr int bfly_writers() {
    int w = 1;
    while (w < N) w *= 2;
    return w < kWave ? w : kWave;
}

// ---------------------------------------------------------------------------
// Gradients with respect to both filters.  Work cell = output pixel.  The
// kFilterWaves waves of a block work on the same strip of the same sample and
// take consecutive channel ranges of g.cpw channels each; in the channel walk
// they are as independent as the waves of the other two kernels (private LDS
// tiles, no barrier).  Per channel a lane forms gx[t] = dO * X_t once and
// feeds it to both sums:
//   dSF[t, pixel] += gx[t] * CF[c, t]      (register accumulator, over channels)
//   dCF[c, t]     += gx[t] * SF[t, pixel]  (butterfly over the wave's lanes)
// After the walk the waves add their dSF accumulators through LDS (the only
// barriers of the kernel).  Partial sums over channel splits (dSF) and strips
// (dCF) go to the workspace and are added up by k_sum_partials: no atomics, so
// results are reproducible.
// ---------------------------------------------------------------------------
constexpr int kFilterWaves = 4;

//
// With DX (stride 1 only) the same walk also produces the feature gradient:
// dO then sits in a zero-bordered tile of its own (same shape and offsets as
// the X tile), the lane gathers it at the flipped tap offsets against the
// neighbour cells' spatial filter (held in registers like the cell's own), and
// the linear strip carries the dX results out.  One launch instead of two, and
// dO, CF and SF are read once for the whole backward pass.
template <typename T, int K, int D, int S, bool MUL, int PS, int NV, int V, bool DX>
__global__ __launch_bounds__(kWave * kFilterWaves) void k_backward_filters(
    WaveGeom g, const T *__restrict__ go, const T *__restrict__ x,
    const T *__restrict__ cf, const T *__restrict__ sf, T *__restrict__ dx,
    T *__restrict__ dcf, T *__restrict__ dsf, typename Acc<T>::type *__restrict__ ws_sf,
    typename Acc<T>::type *__restrict__ ws_cf, unsigned need) {
    static_assert(!DX || S == 1, "the fused feature gradient needs stride 1");
    using A = typename Acc<T>::type;
    constexpr int KK = K * K;
    constexpr int R = (K - 1) / 2;
    constexpr bool kFilters = MUL || DX;   // CF and SF values are needed at all
    // (two channels in flight at most with DX: it stages two planes per channel
    // and holds a third set of filter registers)
    using Stg = Stager<T, V, NV, DX ? 2 : 4>;
    constexpr int NST = Stg::NST;
    constexpr int NG = (PS + V - 1) / V;
    extern __shared__ __align__(16) unsigned char smem[];
    const int lane = threadIdx.x & (kWave - 1);
    // (the wave index is the same in all lanes: say so, or everything derived from
    // it - channel range, pointers, loop bounds - is computed per lane)
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    // private LDS of this wave: X tile, [dO tile,] linear strip (dO in, or dX out), taps
    A *lds_in = reinterpret_cast<A *>(smem + (size_t)wave * g.lds_wave_bytes);
    A *lds_g = lds_in + g.tile + kSpare;
    T *lds_go = reinterpret_cast<T *>(lds_g + (DX ? g.tile + kSpare : 0));
    A *taps = reinterpret_cast<A *>(lds_go + g.lin_tile + kIdle);

    WaveWork ww;
    if (!ww.init(g)) return;   // whole block leaves together
    const int lr = lane >> g.lw_shift, lc = lane & ((1 << g.lw_shift) - 1);
    const int64_t oplane = (int64_t)g.Ho * g.Wo, iplane = (int64_t)g.H * g.W;
    const int y0 = ww.row_first;
    const bool want_cf = need & DDF_NEED_DCF, want_sf = need & DDF_NEED_DSF;
    const int my_tap = g_bfly_table<KK>.tap[lane];
    // this wave's channels inside the block's range
    const int c_begin = min(ww.c_begin + wave * g.cpw, ww.c_end);
    const int nch = min(g.cpw, ww.c_end - c_begin);
    const int nch1 = max(nch, 1);   // a wave without channels still issues (harmless) loads

    // all loads of the prologue first (see k_forward), index arithmetic under them
    Stg stg;
    stg.init_global(g, y0 * S + g.row0_off, lane);
    // dO: a bordered tile with the X tile's offsets (DX), else a linear strip
    Stg stg_g;
    LinStager<T, V, NG, NST> sgo;
    if constexpr (DX) {
#pragma unroll
        for (int j = 0; j < NV; ++j) stg_g.goff[j] = stg.goff[j];
    } else {
        sgo.init(ww.nrows * g.Wo, lane);
    }
    const int c_first = min(c_begin, g.C - 1);
    const T *xs = x + (ww.n * g.C + c_first) * iplane;
    const T *gs = go + (ww.n * g.C + c_first) * oplane + (DX ? 0 : (int64_t)y0 * g.Wo);
    auto issue_go = [&](auto st_tag, const T *plane) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value;
        if constexpr (DX) stg_g.template issue<ST>(plane);
        else sgo.template issue<ST>(plane);
    };
    stg.template issue<0>(xs);
    issue_go(std::integral_constant<int, 0>{}, gs);
    if constexpr (NST > 1) {
        stg.template issue<1>(xs + (int64_t)min(1, nch1 - 1) * iplane);
        issue_go(std::integral_constant<int, 1>{}, gs + (int64_t)min(1, nch1 - 1) * oplane);
    }
    if constexpr (NST > 2) {
        stg.template issue<2>(xs + (int64_t)min(2, nch1 - 1) * iplane);
        issue_go(std::integral_constant<int, 2>{}, gs + (int64_t)min(2, nch1 - 1) * oplane);
        stg.template issue<3>(xs + (int64_t)min(3, nch1 - 1) * iplane);
        issue_go(std::integral_constant<int, 3>{}, gs + (int64_t)min(3, nch1 - 1) * oplane);
    }
    FilterStager<T, V, NG, KK> fst;
    TapStager<KK, T, A> tst;
    // DX: the block's four waves need the same spatial filter (same sample, same
    // strip), at their cells and at the neighbour cells.  Each wave brings in
    // every fourth tap plane, laid out like a dO tile (zero border), into LDS
    // shared by the block; after one barrier every wave picks its registers
    // out of the nine tiles.
    static_assert(!DX || (V > 1 && NV * V <= 8), "fused kernel: short strips only");
    constexpr int kTapsPerWave = (KK + kFilterWaves - 1) / kFilterWaves;
    A *sf_tiles = reinterpret_cast<A *>(smem + (size_t)kFilterWaves * g.lds_wave_bytes);
    const int sf_pitch = g.tile + kSpare;
    Vec<T, V> sfv[DX ? kTapsPerWave : 1][NV];
    if (kFilters) {
        if constexpr (DX) {
#pragma unroll
            for (int q = 0; q < kTapsPerWave; ++q) {
                const int t = min(wave + q * kFilterWaves, KK - 1);   // clamped: no branch
#pragma unroll
                for (int j = 0; j < NV; ++j)
                    sfv[q][j] = *reinterpret_cast<const Vec<T, V> *>(
                        sf + (ww.n * KK + t) * oplane + stg.goff[j]);
            }
        } else {
            fst.init(ww.nrows * g.Wo, lane);
            fst.issue(sf + (ww.n * KK * g.Ho + y0) * g.Wo, oplane);
        }
        tst.issue(cf, ww.n * g.C + c_first, nch1, lane);
    }

    bool ok[PS];
    int lb[PS], ob[PS];
    A sfr[PS][KK], acc_sf[PS][KK];
    A sfg[DX ? PS : 1][KK];   // spatial filter at the neighbour cells (DX)
#pragma unroll
    for (int m = 0; m < PS; ++m) {
        const int row = g.slot_row[m] + lr, col = g.slot_col[m] + lc;
        ok[m] = m < g.nslots && row < ww.nrows && col < g.cols;
        lb[m] = (row * S) * g.P + col * S + g.lb_shift;   // lane-linear: no bank conflicts, idle lanes included
        ob[m] = ok[m] ? row * g.Wo + col : 0;
#pragma unroll
        for (int t = 0; t < KK; ++t) {
            sfr[m][t] = 0;
            acc_sf[m][t] = 0;
        }
    }
    stg.init_tile(g, y0 * S + g.row0_off, lane);
    if constexpr (DX) {
#pragma unroll
        for (int j = 0; j < NV; ++j)
#pragma unroll
            for (int k = 0; k < V; ++k) stg_g.lo[j][k] = stg.lo[j][k];
    }
    const int P = pin(g.P);
    const bool wide = g.wide != 0;
    zero_tile(lds_in, g.tile, lane);
    if constexpr (DX) zero_tile(lds_g, g.tile, lane);
    if (kFilters) {
        tst.put(taps, nch, lane);
        if constexpr (DX) {
#pragma unroll
            for (int q = 0; q < kTapsPerWave; ++q) {
                const int t = wave + q * kFilterWaves;
                if (t < KK) {
                    A *tile_t = sf_tiles + t * sf_pitch;
                    zero_tile(tile_t, g.tile, lane);
                    wave_sync();
#pragma unroll
                    for (int j = 0; j < NV; ++j)
#pragma unroll
                        for (int k = 0; k < V; ++k) tile_t[stg.lo[j][k]] = ld(&sfv[q][j].e[k]);
                }
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < K; ++i)
#pragma unroll
                for (int j = 0; j < K; ++j) {
                    const A *tile_t = sf_tiles + (i * K + j) * sf_pitch;
#pragma unroll
                    for (int m = 0; m < PS; ++m) {
                        sfr[m][i * K + j] = tile_t[lb[m] + R * D * P + R * D];
                        sfg[m][i * K + j] = tile_t[lb[m] + (2 * R - i) * D * P + (2 * R - j) * D];
                    }
                }
        } else {
            fst.collect(lds_go, ob, sfr);
        }
    }
    wave_sync();
    int wb[PS];   // where the dX value of a slot goes: idle lanes write behind the strip
#pragma unroll
    for (int m = 0; m < PS; ++m) wb[m] = ok[m] ? ob[m] : g.lin_tile + lane;
    T *ds = DX ? dx + (ww.n * g.C + c_first) * iplane + (int64_t)y0 * g.W : nullptr;
    const int n_out = ww.nrows * g.W;      // elements of the dX strip (DX: stride 1)

    auto channel = [&](auto st_tag, int ci) __attribute__((always_inline)) {
        constexpr int ST = decltype(st_tag)::value;
        stg.template commit<ST>(lds_in, wide);
        if constexpr (DX) stg_g.template commit<ST>(lds_g, wide);
        else sgo.template commit<ST>(lds_go);
        stg.template issue<ST>(xs + (int64_t)min(ci + NST, nch1 - 1) * iplane);
        issue_go(st_tag, gs + (int64_t)min(ci + NST, nch1 - 1) * oplane);
        wave_sync();
        A w[KK];
        if (kFilters) load_taps<KK>(taps, ci, w);
        A pcf[KK];
#pragma unroll
        for (int t = 0; t < KK; ++t) pcf[t] = 0;
#pragma unroll
        for (int m = 0; m < PS; ++m) {
            // (this branch also keeps the scheduler from overlapping slots, which
            // costs more registers than this kernel has)
            if (m >= g.nslots) break;
            // idle lanes read a valid dO element and are zeroed: they add nothing
            const A gread = DX ? (A)ld(lds_g + lb[m] + R * D * P + R * D) : (A)ld(lds_go + ob[m]);
            const A gval = ok[m] ? gread : A(0);
#pragma unroll
            for (int i = 0; i < K; ++i)
#pragma unroll
                for (int j = 0; j < K; ++j) {
                    const int t = i * K + j;
                    const A gx = gval * (A)ld(lds_in + lb[m] + i * D * P + j * D);
                    if (MUL) {
                        acc_sf[m][t] += gx * w[t];
                        pcf[t] += gx * sfr[m][t];
                    } else {
                        acc_sf[m][t] += gx;
                        pcf[t] += gx;
                    }
                }
            if constexpr (DX) {
                // dX of the cell: dO at the flipped tap offsets, filters of those cells
                A accx = 0;
#pragma unroll
                for (int i = 0; i < K; ++i)
#pragma unroll
                    for (int j = 0; j < K; ++j)
                        accx += (A)ld(lds_g + lb[m] + (2 * R - i) * D * P + (2 * R - j) * D) *
                                comb<MUL, A>(w[i * K + j], sfg[m][i * K + j]);
                st(lds_go + wb[m], accx);
            }
        }
        if constexpr (DX) {
            wave_sync();
            store_strip<T, V>(lds_go, ds + (int64_t)ci * iplane, n_out, lane);
        }
        if (want_cf) {
            const A tot = bfly_sum<KK, 0, A>(pcf, lane);
            if (lane < bfly_writers<KK>()) {
                const int64_t nc = ww.n * g.C + c_begin + ci;
                if (g.nstrips == 1) st(dcf + nc * KK + my_tap, tot);
                else ws_cf[(nc * g.nstrips + ww.strip) * KK + my_tap] = tot;
            }
        }
        wave_sync();
    };
    auto group = [&](int c) __attribute__((always_inline)) {
        channel(std::integral_constant<int, 0>{}, c);
        if constexpr (NST > 1) channel(std::integral_constant<int, 1>{}, c + 1);
        if constexpr (NST > 2) channel(std::integral_constant<int, 2>{}, c + 2);
        if constexpr (NST > 3) channel(std::integral_constant<int, 3>{}, c + 3);
    };
    const int nfull = nch > 0 ? nch / NST * NST : 0;
    if (nfull > 0) {
        group(0);
        for (int c = NST; c < nfull; c += NST) group(c);
    }
    if constexpr (NST > 1) {
        if (nfull < nch) channel(std::integral_constant<int, 0>{}, nfull);
        if constexpr (NST > 2) {
            if (nfull + 1 < nch) channel(std::integral_constant<int, 1>{}, nfull + 1);
            if (nfull + 2 < nch) channel(std::integral_constant<int, 2>{}, nfull + 2);
        }
    }

    if (!want_sf) return;
    // Add the waves' dSF accumulators: one pixel slot at a time through LDS.
    __syncthreads();
    A *red = reinterpret_cast<A *>(smem);
#pragma unroll
    for (int m = 0; m < PS; ++m) {
        if (m >= g.nslots) break;
#pragma unroll
        for (int t = 0; t < KK; ++t) red[(wave * KK + t) * kWave + lane] = acc_sf[m][t];
        __syncthreads();
        const int64_t pix = (int64_t)y0 * g.Wo + ob[m];
        for (int t = wave; t < KK; t += kFilterWaves) {
            A tot = 0;
#pragma unroll
            for (int wv = 0; wv < kFilterWaves; ++wv) tot += red[(wv * KK + t) * kWave + lane];
            if (ok[m]) {
                if (g.csplit == 1) st(dsf + (ww.n * KK + t) * oplane + pix, tot);
                else ws_sf[((ww.n * g.csplit + ww.cs) * KK + t) * oplane + pix] = tot;
            }
        }
        __syncthreads();
    }
}

// out[o, i] = sum_p part[o, p, i] for o < outer, p < parts, i < inner.  A
// thread adds up VEC neighbouring i (inner % VEC == 0) and keeps 8 loads in
// flight; the order of the additions is fixed, so results are reproducible.
template <typename T, int VEC>
__device__ __forceinline__ void sum_partials_block(const typename Acc<T>::type *__restrict__ part,
                                                   T *__restrict__ out, int64_t outer, int parts,
                                                   int64_t inner, unsigned block) {
    using A = typename Acc<T>::type;
    const int64_t iv = inner / VEC;
    const int64_t idx = (int64_t)block * 256 + threadIdx.x;
    if (idx >= outer * iv) return;
    const int64_t o = idx / iv, i = (idx - o * iv) * VEC;
    const A *src = part + o * parts * inner + i;
    A tot[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) tot[k] = 0;
    int p = 0;
    for (; p + 8 <= parts; p += 8) {
        Vec<A, VEC> v[8];
#pragma unroll
        for (int q = 0; q < 8; ++q)
            v[q] = *reinterpret_cast<const Vec<A, VEC> *>(src + (int64_t)(p + q) * inner);
#pragma unroll
        for (int q = 0; q < 8; ++q)
#pragma unroll
            for (int k = 0; k < VEC; ++k) tot[k] += v[q].e[k];
    }
    for (; p < parts; ++p) {
        const Vec<A, VEC> v = *reinterpret_cast<const Vec<A, VEC> *>(src + (int64_t)p * inner);
#pragma unroll
        for (int k = 0; k < VEC; ++k) tot[k] += v.e[k];
    }
#pragma unroll
    for (int k = 0; k < VEC; ++k) st(out + o * inner + i + k, tot[k]);
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void k_sum_partials(
    const typename Acc<T>::type *__restrict__ part, T *__restrict__ out, int64_t outer,
    int parts, int64_t inner) {
    sum_partials_block<T, VEC>(part, out, outer, parts, inner, blockIdx.x);
}

// dSF of a pixel = sum of its partial sums (PT: the accumulator type, or - one
// part, written by the filter kernel itself - the storage type), pushed through
// the Jacobian of the spatial filter normalisation (see k_filter_norm_backward):
// with c_t = raw_t - mean, inv = 1 / (sd + 1e-10), gy_t = dSF_t * gain_t,
//   d_raw_t = inv * (gy_t - mean(gy)) - c_t * inv^2 * sum(gy * c) / (sd * (KK - 1)).
// One thread per pixel of one sample; neighbouring threads are neighbouring
// pixels, so every tap plane is read and written with coalesced accesses.
template <typename T, typename PT, int KK>
__device__ __forceinline__ void sum_norm_block(const PT *__restrict__ part, int parts, int64_t n_samples,
                                               int64_t plane, const T *__restrict__ raw,
                                               T *__restrict__ d_raw, T *__restrict__ terms,
                                               const T *__restrict__ gain_vec, int groups,
                                               typename Acc<T>::type gain, unsigned block) {
    using A = typename Acc<T>::type;
    const int64_t idx = (int64_t)block * 256 + threadIdx.x;
    if (idx >= n_samples * plane) return;
    const int64_t n = idx / plane, pix = idx - n * plane;
    const PT *src = part + n * parts * KK * plane + pix;
    A gy[KK];
#pragma unroll
    for (int t = 0; t < KK; ++t) gy[t] = 0;
    for (int q = 0; q < parts; ++q) {
        PT v[KK];
#pragma unroll
        for (int t = 0; t < KK; ++t) v[t] = src[((int64_t)q * KK + t) * plane];
#pragma unroll
        for (int t = 0; t < KK; ++t) gy[t] += (A)v[t];
    }
    const int64_t base = n * KK * plane + pix;
    A c[KK];
    A sum = 0;
#pragma unroll
    for (int t = 0; t < KK; ++t) { c[t] = (A)ld(raw + base + t * plane); sum += c[t]; }
    const A mean = sum / (A)KK;
    const int64_t grp = n % groups;
    A sq = 0, s1 = 0, s2 = 0;
#pragma unroll
    for (int t = 0; t < KK; ++t) {
        c[t] -= mean;
        const A w = gain_vec ? (A)ld(gain_vec + grp * KK + t) : gain;
        sq += c[t] * c[t];
        s1 += gy[t] * w;
        s2 += gy[t] * w * c[t];
    }
    const A sd = sqrt(sq / (A)(KK - 1));
    const A inv = (A)1 / (sd + (A)1e-10);
    const A m1 = s1 / (A)KK;
    const A k2 = inv * inv * s2 / (sd * (A)(KK - 1));
#pragma unroll
    for (int t = 0; t < KK; ++t) {
        const A w = gain_vec ? (A)ld(gain_vec + grp * KK + t) : gain;
        st(d_raw + base + t * plane, inv * (gy[t] * w - m1) - c[t] * k2);
        if (terms) st(terms + base + t * plane, gy[t] * c[t] * inv);
    }
}

// One sum of partials: the arguments of k_sum_partials and the blocks it takes.
template <typename T>
struct SumJob {
    const typename Acc<T>::type *part;
    T *out;
    int64_t outer, inner;
    int parts;
    bool wide;         // four neighbouring elements per thread
    unsigned blocks;
};
template <typename T>
inline SumJob<T> sum_job(const typename Acc<T>::type *part, T *out, int64_t outer, int parts,
                         int64_t inner) {
    using A = typename Acc<T>::type;
    SumJob<T> j{part, out, outer, inner, parts, sizeof(A) == 4 && inner % 4 == 0, 0};
    const int64_t threads = outer * (j.wide ? inner / 4 : inner);
    j.blocks = (unsigned)((threads + 255) / 256);
    return j;
}

// Two independent sums in one launch: the first a.blocks workgroups take a,
// the others b.
template <typename T>
__global__ __launch_bounds__(256) void k_sum_partials_pair(SumJob<T> a, SumJob<T> b) {
    const bool second = blockIdx.x >= a.blocks;
    const SumJob<T> &j = second ? b : a;
    const unsigned block = second ? blockIdx.x - a.blocks : blockIdx.x;
    if (j.wide) sum_partials_block<T, 4>(j.part, j.out, j.outer, j.parts, j.inner, block);
    else sum_partials_block<T, 1>(j.part, j.out, j.outer, j.parts, j.inner, block);
}

// Launches k_sum_partials with the widest access the sizes allow (the
// workspace is 256-byte aligned).
template <typename T>
inline hipError_t sum_partials(const typename Acc<T>::type *part, T *out, int64_t outer,
                               int parts, int64_t inner, hipStream_t st) {
    const SumJob<T> j = sum_job<T>(part, out, outer, parts, inner);
    const dim3 grid(j.blocks), block(256);
    if (j.wide)
        hipLaunchKernelGGL((k_sum_partials<T, 4>), grid, block, 0, st, part, out, outer, parts, inner);
    else
        hipLaunchKernelGGL((k_sum_partials<T, 1>), grid, block, 0, st, part, out, outer, parts, inner);
    return hipGetLastError();
}

// The dSF sum with the spatial filter normalisation behind it (sum_norm_block) and,
// in the same launch, the dCF sum b (b.blocks == 0: none).  The dSF parts are
// `parts` partial sums in the accumulator type, or (part_t) one part in the
// storage type.
template <typename T, int KK>
__global__ __launch_bounds__(256) void k_sum_norm_pair(
    const typename Acc<T>::type *__restrict__ part_a, const T *__restrict__ part_t, int parts,
    int64_t n_samples, int64_t plane, const T *__restrict__ raw, T *__restrict__ d_raw,
    T *__restrict__ terms, const T *__restrict__ gain_vec, int groups,
    typename Acc<T>::type gain, unsigned norm_blocks, SumJob<T> b) {
    if (blockIdx.x >= norm_blocks) {
        const unsigned block = blockIdx.x - norm_blocks;
        if (b.wide) sum_partials_block<T, 4>(b.part, b.out, b.outer, b.parts, b.inner, block);
        else sum_partials_block<T, 1>(b.part, b.out, b.outer, b.parts, b.inner, block);
        return;
    }
    if (part_a)
        sum_norm_block<T, typename Acc<T>::type, KK>(part_a, parts, n_samples, plane, raw, d_raw,
                                                     terms, gain_vec, groups, gain, blockIdx.x);
    else
        sum_norm_block<T, T, KK>(part_t, 1, n_samples, plane, raw, d_raw, terms, gain_vec, groups,
                                 gain, blockIdx.x);
}

template <typename T>
bool norm_tail_kernel_built(int kk) { return kk == 9 || kk == 25; }

// The partial sums a filter-gradient launch leaves behind: dSF over `csplit`
// channel splits and / or dCF over `nstrips` strips (null: nothing to add), in
// one launch.  With `norm` (and a launch to be made anyway, and a kernel built
// for this tap count) the dSF part of that launch also applies the spatial
// filter normalisation's Jacobian and writes norm->d_raw: dsf is then where the
// filter kernel put a complete dSF (no partial sums), and is not written here.
template <typename T>
inline hipError_t sum_filter_partials(const typename Acc<T>::type *ws_sf, T *dsf, int64_t n,
                                      int csplit, int64_t sf_inner,
                                      const typename Acc<T>::type *ws_cf, T *dcf, int64_t nc,
                                      int nstrips, int64_t kk, hipStream_t st,
                                      NormTail<T> *norm = nullptr) {
    using A = typename Acc<T>::type;
    if (norm && dsf && (ws_sf || ws_cf) && norm_tail_kernel_built<T>((int)kk)) {
        const int64_t plane = sf_inner / kk;
        const int64_t threads = n * plane;
        const unsigned norm_blocks = (unsigned)((threads + 255) / 256);
        SumJob<T> b{};
        if (ws_cf) b = sum_job<T>(ws_cf, dcf, nc, nstrips, kk);
        const dim3 grid(norm_blocks + b.blocks), block(256);
        const A gain = (A)norm->gain;
#define DDF_SUM_NORM(KK_)                                                                         \
    hipLaunchKernelGGL((k_sum_norm_pair<T, KK_>), grid, block, 0, st, ws_sf, ws_sf ? nullptr : dsf, \
                       ws_sf ? csplit : 1, n, plane, norm->raw, norm->d_raw, norm->terms,         \
                       norm->gain_vec, norm->groups, gain, norm_blocks, b)
        if (kk == 9) DDF_SUM_NORM(9);
        else DDF_SUM_NORM(25);
#undef DDF_SUM_NORM
        norm->applied = true;
        return hipGetLastError();
    }
    if (ws_sf && ws_cf) {
        const SumJob<T> a = sum_job<T>(ws_sf, dsf, n, csplit, sf_inner);
        const SumJob<T> b = sum_job<T>(ws_cf, dcf, nc, nstrips, kk);
        hipLaunchKernelGGL((k_sum_partials_pair<T>), dim3(a.blocks + b.blocks), dim3(256), 0, st, a, b);
        return hipGetLastError();
    }
    if (ws_sf) return sum_partials<T>(ws_sf, dsf, n, csplit, sf_inner, st);
    if (ws_cf) return sum_partials<T>(ws_cf, dcf, nc, nstrips, kk, st);
    return hipSuccess;
}

}  // namespace wave

// Integer tuning knob: `fallback`, or the environment's value in a -DDDF_TUNING build.
int tune_int(const char *name, int fallback);

enum WaveKind { kWaveForward = 0, kWaveFeatures = 1, kWaveFilters = 2, kWaveFused = 3 };
// Host-side geometry (ddf_tiled_host.hip).  *ps and *nv select the kernel.
// max_vec > 0 caps the elements per global access (1 = scalar accesses).
bool wave_geometry(const Problem &p, int dtype, int kind, int max_vec, WaveGeom *g, int *ps,
                   int *nv);

}  // namespace ddf
