// Up-sampling DDF forward: the scale*scale filter branches of DDFUpPack in one
// launch, written straight into the pixel-shuffled result.
//
// The reference (ddf/ddf.py:257-272) runs `ddf` once per sub-pixel branch b on
// the same features, stacks the scale^2 results and pixel-shuffles them:
//   out[n, c, y*R + i, x*R + j] = ddf(X, CF_b, SF_b)[n, c, y, x],  b = i*R + j.
// Here one thread owns an input pixel (y, x) of one sample and walks over a
// chunk of channels.  It keeps the K*K spatial taps of all R*R branches in
// registers, reads the K*K neighbours of X once per channel and uses them for
// every branch, and writes R rows of R neighbouring results, so X is read once
// instead of R*R times and the result is written once, in place.  Neighbouring
// lanes are neighbouring pixels: every global access is coalesced.  The channel
// taps of the block's chunk sit in LDS in accumulator precision and are read
// with wave-uniform (broadcast) addresses.
#include <algorithm>
#include <atomic>

#include "ddf_chunks.h"

namespace ddf {
int tune_int(const char *name, int fallback);

namespace {

using chunks::kThreads;
constexpr int kStageChannels = chunks::kUpStageChannels;   // channels whose taps are staged in LDS at a time
constexpr int kStageBytes = chunks::kUpStageBytes;         // and the LDS they may take

template <typename T>
struct UpFilters {
    const T *cf[DDF_UP_MAX_BRANCHES];
    const T *sf[DDF_UP_MAX_BRANCHES];
};

template <typename T, int R>
struct alignas((R & (R - 1)) == 0 ? sizeof(T) * R : sizeof(T)) Row {
    T e[R];
};

// Register image of one result row, so that it leaves as a single store.
template <int BYTES> struct RowBits;
template <> struct RowBits<4> { using type = uint32_t; };
template <> struct RowBits<8> { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <> struct RowBits<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };
template <> struct RowBits<32> { typedef uint32_t type __attribute__((ext_vector_type(8))); };

// UU channels of one pixel: every load is issued before the first result is
// needed (a wave keeps UU*K*K loads in flight), then R rows of R results per
// channel are formed and stored.  A neighbour outside the plane reads the
// pixel itself (offset 0, always valid) and is zeroed afterwards, so there is
// no branch between the loads.
template <typename T, int K, int R, bool MUL, int UU, typename A>
__device__ __forceinline__ void up_channels(const T *__restrict__ xp, T *__restrict__ op,
                                            const A *__restrict__ w, int plane, int64_t orow,
                                            int64_t ostep, const int (&off)[K * K],
                                            const bool (&inside)[K * K],
                                            const A (&sfr)[R * R][K * K], int vec_ok) {
    constexpr int KK = K * K, RR = R * R;
    A xv[UU][KK];
#pragma unroll
    for (int u = 0; u < UU; ++u)
#pragma unroll
        for (int t = 0; t < KK; ++t) xv[u][t] = (A)ld(xp + (int64_t)u * plane + off[t]);
#pragma unroll
    for (int u = 0; u < UU; ++u)
#pragma unroll
        for (int t = 0; t < KK; ++t)
            if (!inside[t]) xv[u][t] = (A)0;
#pragma unroll
    for (int u = 0; u < UU; ++u) {
#pragma unroll
        for (int i = 0; i < R; ++i) {
            Row<T, R> row;
#pragma unroll
            for (int j = 0; j < R; ++j) {
                const int b = i * R + j;
                A acc = 0;
#pragma unroll
                for (int t = 0; t < KK; ++t)
                    acc += xv[u][t] * comb<MUL, A>(w[(u * RR + b) * KK + t], sfr[b][t]);
                st(&row.e[j], acc);
            }
            T *dst = op + u * ostep + i * orow;
            if constexpr (R == 2 || R == 4) {
                if (vec_ok) {   // one store of R elements
                    using Bits = typename RowBits<sizeof(T) * R>::type;
                    Bits bits = __builtin_bit_cast(Bits, row);
                    // opaque to the compiler, which would otherwise undo the
                    // packing of 2-byte results into 2-byte stores
                    if constexpr (sizeof(T) == 2) asm("" : "+v"(bits));
                    __builtin_nontemporal_store(bits, reinterpret_cast<Bits *>(dst));
                    continue;
                }
            }
#pragma unroll
            for (int j = 0; j < R; ++j) dst[j] = row.e[j];
        }
    }
}

template <typename T, int K, int R, bool MUL>
__global__ __launch_bounds__(kThreads) void k_up_forward(
    UpFilters<T> f, const T *__restrict__ x, T *__restrict__ out, int C, int H, int W, int D,
    int cpb, int csplit, int pblocks, int stage, int vec_ok) {
    using A = typename Acc<T>::type;
    constexpr int KK = K * K, RR = R * R, RAD = K / 2;
    constexpr int U = KK <= 9 ? 4 : 2;              // channels whose loads are issued together
    constexpr int Q = 4;                            // tap loads in flight per thread while staging
    extern __shared__ __align__(16) unsigned char up_smem[];
    A *taps = reinterpret_cast<A *>(up_smem);   // [channel][branch][tap]

    // (consecutive logical blocks - same sample and pixel block, neighbouring channel
    // chunks, hence the same spatial taps - run on one XCD and share its L2)
    chunks::Block blk;
    blk.init(blockIdx.x, gridDim.x, csplit, pblocks, cpb, C);
    const int pb = blk.pb;
    const int64_t n = blk.n;
    const int c0 = blk.c0, nch = blk.nch;
    const int plane = H * W;

    // Lanes past the end of the plane work on its last pixel and store nothing:
    // no branch around the loads, and they still take part in the barriers.
    const int pix_raw = pb * kThreads + (int)threadIdx.x;
    const bool live = pix_raw < plane;
    const int pix = min(pix_raw, plane - 1);
    const int y = pix / W, xx = pix - y * W;

    A sfr[RR][KK];
#pragma unroll
    for (int b = 0; b < RR; ++b)
#pragma unroll
        for (int t = 0; t < KK; ++t) sfr[b][t] = (A)ld(f.sf[b] + (n * KK + t) * plane + pix);

    // neighbours of X: offset from the pixel and whether it lies in the plane
    int off[KK];
    bool inside[KK];
#pragma unroll
    for (int i = 0; i < K; ++i)
#pragma unroll
        for (int j = 0; j < K; ++j) {
            const int iy = y + (i - RAD) * D, ix = xx + (j - RAD) * D;
            inside[i * K + j] = iy >= 0 && iy < H && ix >= 0 && ix < W;
            off[i * K + j] = inside[i * K + j] ? (i - RAD) * D * W + (j - RAD) * D : 0;
        }

    const int64_t orow = (int64_t)W * R;            // elements per result row
    const int64_t ostep = (int64_t)H * R * orow;    // and per result plane
    const T *xp = x + (n * C + c0) * plane + pix;
    T *op = out + ((n * C + c0) * H + y) * R * orow + (int64_t)xx * R;
    for (int s0 = 0; s0 < nch; s0 += stage) {
        const int ns = min(stage, nch - s0);
        if (s0 > 0) __syncthreads();                // the previous taps have been used
        // Channel taps of this stage, widened to the accumulator type.  Per
        // branch they are ns*KK contiguous elements; Q loads per thread are
        // issued before the first is written to LDS.
        const int per = ns * KK, total = RR * per;
        const int64_t cf0 = (n * C + c0 + s0) * KK;
        for (int e0 = threadIdx.x; e0 < total; e0 += Q * kThreads) {
            A v[Q];
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                const int e = min(e0 + q * kThreads, total - 1);
                const int b = e / per, r = e - b * per;
                const T *src = f.cf[0];
#pragma unroll
                for (int bb = 1; bb < RR; ++bb)
                    if (b == bb) src = f.cf[bb];
                v[q] = (A)ld(src + cf0 + r);
            }
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                const int e = e0 + q * kThreads;
                if (e < total) {
                    const int b = e / per, r = e - b * per;
                    const int ch = r / KK, t = r - ch * KK;
                    taps[(ch * RR + b) * KK + t] = v[q];
                }
            }
        }
        __syncthreads();
        if (!live) continue;
        int ch = 0;
        for (; ch + U <= ns; ch += U, xp += (int64_t)U * plane, op += U * ostep)
            up_channels<T, K, R, MUL, U, A>(xp, op, taps + ch * RR * KK, plane, orow, ostep, off,
                                            inside, sfr, vec_ok);
        for (; ch < ns; ++ch, xp += plane, op += ostep)
            up_channels<T, K, R, MUL, 1, A>(xp, op, taps + ch * RR * KK, plane, orow, ostep, off,
                                            inside, sfr, vec_ok);
    }
}

template <typename T, int K, int R>
hipError_t launch(bool mul, const UpFilters<T> &f, const T *x, T *out, int64_t N, int C, int H,
                  int W, int D, hipStream_t stream) {
    using A = typename Acc<T>::type;
    const int per_channel = R * R * K * K * (int)sizeof(A);
    // Split the channels over blocks until the chip is full once: as many
    // blocks as can be resident together (a second round of blocks would start
    // late and finish alone), and no further, because every chunk re-reads the
    // R*R*K*K spatial taps of its pixels.
    auto kern = mul ? k_up_forward<T, K, R, true> : k_up_forward<T, K, R, false>;
    static std::atomic<int> resident[2] = {{0}, {0}};     // blocks per CU, per combine
    int per_cu = resident[mul].load(std::memory_order_relaxed);
    if (per_cu == 0) {
        const size_t lds_max = (size_t)std::min(kStageChannels, kStageBytes / per_channel) * per_channel;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, kThreads, lds_max) !=
                hipSuccess || per_cu < 1) {
            (void)hipGetLastError();
            per_cu = 2;
        }
        resident[mul].store(per_cu, std::memory_order_relaxed);
    }
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
        (void)hipGetLastError();
        cus = 256;
    }
    const int64_t target = tune_int("DDF_TUNE_UP_BLOCKS", per_cu * cus);
    const int min_chunk = std::max(1, tune_int("DDF_TUNE_UP_MIN_CHUNK", 8));
    chunks::ChunkGeom g;
    if (!chunks::up_chunks(N, C, (int64_t)H * W, R * R * K * K, (int)sizeof(A), target, min_chunk, &g))
        return hipErrorInvalidConfiguration;
    const int vec_ok = ((uintptr_t)out % (sizeof(T) * R)) == 0;
    hipLaunchKernelGGL(kern, dim3((unsigned)g.blocks), dim3(kThreads), g.lds, stream, f, x, out, C, H,
                       W, D, g.cpb, g.csplit, g.pblocks, g.stage, vec_ok);
    return hipGetLastError();
}

// Gradient of the pixel shuffle: lat[b][nc][y][x] = dO[nc][y*R + i][x*R + j],
// b = i*R + j.  One thread per (nc, y, x): it reads R runs of R neighbouring
// elements and writes one element to each of the R*R lattices (neighbouring
// lanes write neighbouring elements).
template <typename T>
__global__ __launch_bounds__(kThreads) void k_up_split(const T *__restrict__ go,
                                                       T *__restrict__ lat, int64_t planes, int H,
                                                       int W, int R) {
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    const int64_t plane = (int64_t)H * W;
    if (idx >= planes * plane) return;
    const int64_t nc = idx / plane;
    const int pix = (int)(idx - nc * plane);
    const int y = pix / W, x = pix - y * W;
    const T *src = go + (nc * H * R + (int64_t)y * R) * W * R + (int64_t)x * R;
    for (int i = 0; i < R; ++i)
        for (int j = 0; j < R; ++j)
            lat[(int64_t)(i * R + j) * planes * plane + idx] = src[(int64_t)i * W * R + j];
}

// out[e] = sum over `parts` tensors of `count` elements stored back to back.
template <typename T>
__global__ __launch_bounds__(kThreads) void k_up_sum(const T *__restrict__ in,
                                                     T *__restrict__ out, int64_t count,
                                                     int parts) {
    using A = typename Acc<T>::type;
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= count) return;
    A acc = 0;
    for (int b = 0; b < parts; ++b) acc += (A)ld(in + (int64_t)b * count + idx);
    st(out + idx, acc);
}

// The branches' filters, back to back: cf_all[b] = cf of branch b (n_cf elements),
// sf_all[b] = sf of branch b (n_sf elements).
template <typename T>
__global__ __launch_bounds__(kThreads) void k_up_gather(UpFilters<T> f, T *__restrict__ cf_all,
                                                        T *__restrict__ sf_all, int64_t n_cf,
                                                        int64_t n_sf, int branches) {
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    const int64_t per = n_cf + n_sf;
    if (idx >= per * branches) return;
    const int b = (int)(idx / per);
    const int64_t e = idx - b * per;
    if (e < n_cf) cf_all[b * n_cf + e] = f.cf[b][e];
    else sf_all[b * n_sf + (e - n_cf)] = f.sf[b][e - n_cf];
}

template <typename T>
struct UpGrads {
    T *dcf[DDF_UP_MAX_BRANCHES];
    T *dsf[DDF_UP_MAX_BRANCHES];
};

// dX = sum of the branches' parts (parts != null); the branches' filter
// gradients from where the batched kernels left them back to back to the
// tensors they belong to (a null destination was not asked for).
template <typename T>
__global__ __launch_bounds__(kThreads) void k_up_finish(
    const T *__restrict__ parts, T *__restrict__ dx, int64_t n_x, int branches,
    const T *__restrict__ dcf_all, const T *__restrict__ dsf_all, UpGrads<T> g, int64_t n_cf,
    int64_t n_sf) {
    using A = typename Acc<T>::type;
    int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    const int64_t n_dx = parts ? n_x : 0;
    if (idx < n_dx) {
        A acc = 0;
        for (int b = 0; b < branches; ++b) acc += (A)ld(parts + (int64_t)b * n_x + idx);
        st(dx + idx, acc);
        return;
    }
    idx -= n_dx;
    const int64_t all_cf = dcf_all ? n_cf * branches : 0;
    if (idx < all_cf) {
        const int b = (int)(idx / n_cf);
        if (g.dcf[b]) g.dcf[b][idx - b * n_cf] = dcf_all[idx];
        return;
    }
    idx -= all_cf;
    if (dsf_all && idx < n_sf * branches) {
        const int b = (int)(idx / n_sf);
        if (g.dsf[b]) g.dsf[b][idx - b * n_sf] = dsf_all[idx];
    }
}

}  // namespace

template <typename T>
hipError_t up_gather_filters(const void *const *cf, const void *const *sf, T *cf_all, T *sf_all,
                             int64_t n_cf, int64_t n_sf, int branches, hipStream_t stream) {
    const int64_t total = (n_cf + n_sf) * branches;
    if (total == 0) return hipSuccess;
    UpFilters<T> f;
    for (int b = 0; b < DDF_UP_MAX_BRANCHES; ++b) {
        f.cf[b] = b < branches ? (const T *)cf[b] : nullptr;
        f.sf[b] = b < branches ? (const T *)sf[b] : nullptr;
    }
    const int64_t grid = cdiv(total, kThreads);
    if (grid > 2147483647) return hipErrorInvalidConfiguration;
    hipLaunchKernelGGL((k_up_gather<T>), dim3((unsigned)grid), dim3(kThreads), 0, stream, f, cf_all,
                       sf_all, n_cf, n_sf, branches);
    return hipGetLastError();
}

template <typename T>
hipError_t up_finish(const T *parts, T *dx, int64_t n_x, int branches, const T *dcf_all,
                     const T *dsf_all, void *const *dcfs, void *const *dsfs, int64_t n_cf,
                     int64_t n_sf, hipStream_t stream) {
    const int64_t total = (parts ? n_x : 0) + (dcf_all ? n_cf * branches : 0) +
                          (dsf_all ? n_sf * branches : 0);
    if (total == 0) return hipSuccess;
    UpGrads<T> g;
    for (int b = 0; b < DDF_UP_MAX_BRANCHES; ++b) {
        g.dcf[b] = (b < branches && dcfs) ? (T *)dcfs[b] : nullptr;
        g.dsf[b] = (b < branches && dsfs) ? (T *)dsfs[b] : nullptr;
    }
    const int64_t grid = cdiv(total, kThreads);
    if (grid > 2147483647) return hipErrorInvalidConfiguration;
    hipLaunchKernelGGL((k_up_finish<T>), dim3((unsigned)grid), dim3(kThreads), 0, stream, parts, dx,
                       n_x, branches, dcf_all, dsf_all, g, n_cf, n_sf);
    return hipGetLastError();
}

template <typename T>
hipError_t up_split_lattices(const T *go, T *lat, int64_t planes, int64_t H, int64_t W, int scale,
                             hipStream_t stream) {
    const int64_t total = planes * H * W;
    if (total == 0) return hipSuccess;
    const int64_t grid = cdiv(total, kThreads);
    if (grid > 2147483647) return hipErrorInvalidConfiguration;
    hipLaunchKernelGGL((k_up_split<T>), dim3((unsigned)grid), dim3(kThreads), 0, stream, go, lat,
                       planes, (int)H, (int)W, scale);
    return hipGetLastError();
}

template <typename T>
hipError_t up_sum_parts(const T *in, T *out, int64_t count, int parts, hipStream_t stream) {
    if (count == 0) return hipSuccess;
    const int64_t grid = cdiv(count, kThreads);
    if (grid > 2147483647) return hipErrorInvalidConfiguration;
    hipLaunchKernelGGL((k_up_sum<T>), dim3((unsigned)grid), dim3(kThreads), 0, stream, in, out,
                       count, parts);
    return hipGetLastError();
}

bool up_forward_supported(int64_t H, int64_t W, int k, int d, int scale) {
    if (H * W > (int64_t)1 << 30) return false;   // 32-bit offsets inside a plane
    if ((int64_t)(k / 2) * d * (W + 1) > (int64_t)1 << 30) return false;
    if (k == 1 || k == 3) return scale >= 2 && scale <= 4;
    if (k == 5) return scale == 2;
    return false;
}

template <typename T>
hipError_t up_forward(int64_t N, int64_t C, int64_t H, int64_t W, int k, int d, int scale,
                      bool mul, const T *x, const void *const *cf, const void *const *sf, T *out,
                      hipStream_t stream) {
    if (N * C * H * W == 0) return hipSuccess;
    if (C > 2147483647) return hipErrorInvalidConfiguration;
    UpFilters<T> f;
    for (int b = 0; b < DDF_UP_MAX_BRANCHES; ++b) {
        f.cf[b] = b < scale * scale ? (const T *)cf[b] : nullptr;
        f.sf[b] = b < scale * scale ? (const T *)sf[b] : nullptr;
    }
#define DDF_UP_CASE(KV, RV)                                                                     \
    if (k == KV && scale == RV)                                                                 \
        return launch<T, KV, RV>(mul, f, x, out, N, (int)C, (int)H, (int)W, d, stream);
    DDF_UP_CASE(1, 2) DDF_UP_CASE(1, 3) DDF_UP_CASE(1, 4)
    DDF_UP_CASE(3, 2) DDF_UP_CASE(3, 3) DDF_UP_CASE(3, 4)
    DDF_UP_CASE(5, 2)
#undef DDF_UP_CASE
    return hipErrorInvalidConfiguration;
}

#define DDF_UP_INSTANCE(T)                                                                      \
    template hipError_t up_forward<T>(int64_t, int64_t, int64_t, int64_t, int, int, int, bool,  \
                                      const T *, const void *const *, const void *const *, T *, \
                                      hipStream_t);                                             \
    template hipError_t up_split_lattices<T>(const T *, T *, int64_t, int64_t, int64_t, int,    \
                                             hipStream_t);                                      \
    template hipError_t up_sum_parts<T>(const T *, T *, int64_t, int, hipStream_t);             \
    template hipError_t up_gather_filters<T>(const void *const *, const void *const *, T *, T *, \
                                             int64_t, int64_t, int, hipStream_t);              \
    template hipError_t up_finish<T>(const T *, T *, int64_t, int, const T *, const T *,        \
                                     void *const *, void *const *, int64_t, int64_t, hipStream_t);
DDF_UP_INSTANCE(__half)
DDF_UP_INSTANCE(float)
DDF_UP_INSTANCE(double)
#undef DDF_UP_INSTANCE

}  // namespace ddf
