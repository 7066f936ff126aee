// Launch arithmetic of the kernels that hand a workgroup one chunk of a sample's
// channels (k_small in ddf_small.hip, k_up_forward in ddf_up.hip): the cut of
// the channels into chunks, the staging of their taps in LDS, the numbering of
// the workgroups and the thread -> (channel slot, pixel) map.  Plain host/device
// code: the kernels and their launchers call it, and the CPU bounds model
// (tests/geometry_model.cpp) replays the very same functions.
#pragma once

#include <stdint.h>

#include <algorithm>

#include "ddf_common.h"

namespace ddf {
namespace chunks {

constexpr int kThreads = 256;

// k_small: planes of at most kSmallMaxPlane pixels, G = kThreads / plane >= 4
// channel planes per pass, the taps of kSmallStageChannels channels in LDS.
constexpr int kSmallMaxPlane = 64;
constexpr int kSmallStageChannels = 128;
// k_up_forward: the taps of all scale^2 branches of at most kUpStageChannels
// channels, within kUpStageBytes of LDS.
constexpr int kUpStageChannels = 32;
constexpr int kUpStageBytes = 32 * 1024;

struct ChunkGeom {
    int cpb, csplit;   // channels per chunk, chunks per sample
    int pblocks;       // workgroups per plane (1: a workgroup covers whole planes)
    int stage;         // channels whose taps sit in LDS at a time
    int G;             // k_small: channel planes per pass
    int64_t blocks;    // N * pblocks * csplit
    size_t lds;        // bytes of LDS per workgroup
};

// Workgroups reach the 8 XCDs round-robin; renumbered so that consecutive
// logical blocks (same sample, neighbouring chunks) share an XCD and its L2.
__host__ __device__ __forceinline__ unsigned xcd_order(unsigned bid, unsigned nblocks) {
    if (nblocks % 8u != 0) return bid;
    return (bid % 8u) * (nblocks / 8u) + bid / 8u;
}

// Which sample, pixel block and channels workgroup `raw` of `nblocks` works on.
struct Block {
    int chunk, pb, c0, nch;
    int64_t n;
    __host__ __device__ __forceinline__ void init(unsigned raw, unsigned nblocks, int csplit,
                                                  int pblocks, int cpb, int C) {
        const unsigned bid = xcd_order(raw, nblocks);
        chunk = (int)(bid % (unsigned)csplit);
        const unsigned rest = bid / (unsigned)csplit;
        pb = (int)(rest % (unsigned)pblocks);
        n = rest / (unsigned)pblocks;
        c0 = chunk * cpb;
        nch = cpb < C - c0 ? cpb : C - c0;
    }
};

// k_small: thread -> channel slot q (of G) and pixel; threads past the G planes
// idle on slot 0 / pixel 0 and store nothing.
struct SmallThread {
    bool live;
    int q, pix;
    __host__ __device__ __forceinline__ void init(int tid, int plane, int G) {
        const int q_raw = tid / plane;
        live = q_raw < G;
        q = live ? q_raw : 0;
        pix = live ? tid - q_raw * plane : 0;
    }
    // channels q, q + G, q + 2G, ... of a stage of ns channels that are this thread's
    __host__ __device__ __forceinline__ int channels(int ns, int G) const {
        return live && ns > q ? (ns - q + G - 1) / G : 0;
    }
};

// About `target` workgroups (two per CU by default; more, shorter ones measured
// slower), at least 2 passes of G channels each.
inline bool small_chunks(int64_t N, int64_t C, int plane, int asz, int64_t target, ChunkGeom *g) {
    if (plane < 1 || plane > kSmallMaxPlane || N < 1 || C < 1 || C > (1 << 24)) return false;
    g->G = kThreads / plane;
    g->pblocks = 1;
    int csplit = 1;
    while (N * csplit * 2 <= target && C / (csplit * 2) >= 2 * g->G) csplit *= 2;
    g->cpb = (int)cdiv(C, csplit);
    g->csplit = (int)cdiv(C, g->cpb);
    g->blocks = N * g->csplit;
    if (g->blocks > 2147483647) return false;
    g->stage = std::min(g->cpb, kSmallStageChannels);
    g->lds = (size_t)g->stage * 9 * asz;
    return true;
}

// Channels split over workgroups until the chip is full once (`target`
// workgroups), and no further: every chunk re-reads the spatial taps of its
// pixels.  `taps`: K * K * scale * scale taps per channel.
inline bool up_chunks(int64_t N, int64_t C, int64_t plane, int taps, int asz, int64_t target,
                      int min_chunk, ChunkGeom *g) {
    if (plane < 1 || N < 1 || C < 1 || C > 2147483647) return false;
    const int per_channel = taps * asz;
    g->G = 0;
    const int64_t pblocks = cdiv(plane, kThreads);
    if (pblocks > 2147483647) return false;
    g->pblocks = (int)pblocks;
    int csplit = 1;
    while (N * pblocks * csplit * 2 <= target && C / (csplit * 2) >= min_chunk) csplit *= 2;
    g->cpb = (int)cdiv(C, csplit);
    g->csplit = (int)cdiv(C, g->cpb);
    g->blocks = N * pblocks * g->csplit;
    if (g->blocks > 2147483647) return false;
    g->stage = std::max(1, std::min({g->cpb, kUpStageChannels, kUpStageBytes / per_channel}));
    g->lds = (size_t)g->stage * per_channel;
    return true;
}

}  // namespace chunks
}  // namespace ddf
