// Launch geometry and workgroup -> work mapping, shared by host and device code.
//
// A "unit" is one (batch, query, head) triple.  `lanes_per_row` lanes of a wavefront share
// a unit: each moves `vec` channels of a value row per access, so a 64-lane wavefront works
// on 64/lanes_per_row units side by side.  A workgroup owns `tile_q` consecutive queries of
// ONE (batch, head) pair.
//
// Workgroups are dealt round-robin to the 8 XCDs of an MI355X, each with its own 4 MB L2.
// The mapping below pins a head to an XCD (or an XCD group), so that an L2 only ever
// caches the value slice value[:, :, h, :] of its heads -- 1/nh of the tensor -- and walks
// batch elements one after another.  Correctness does not depend on how the hardware deals
// workgroups; only the cache hit rate does.
#pragma once
#include <stdint.h>

#include "../../include/mxd_msda.h"

#if defined(__HIPCC__)
#define MXD_HD __host__ __device__
#else
#define MXD_HD
#endif

namespace mxd {

constexpr int kNumXcd = 8;
constexpr int kWave = 64;
constexpr int kMaxLevels = 64;
constexpr int kChunk = 16;           // samples of a unit staged per pass
constexpr int kChunkStride = 17;     // staged entries per unit incl. one pad entry (LDS banks)

// Dynamic LDS of the forward's one-workgroup-per-CU form: the whole LDS of a gfx950 CU.
constexpr int kCuLdsBytes = 160 * 1024;
constexpr int kCuWaves = 16;         // wavefronts of its workgroups
constexpr int kCuTableBytes = 2 * (kMaxLevels + 1) * 16 + 32;  // its two level tables ahead of the cached rows (multiple of 64)

constexpr int kTileThreads = 512;    // threads of the workgroups of the grad_value pass
// Pixels per tile of the grad_value pass: every thread of a workgroup keeps 32 sums, so a workgroup holds 512 pixels of
// up to 32 channels, 256 of up to 64 or 128 of up to 128 (heads of more channels take two passes over 128-pixel tiles).
// The launcher picks the size from head_dim (KArgs::tile_px_log2: 9, 8 or 7); the first backward kernel sorts its
// records by tiles of that size.
constexpr int kTilePxLog2Max = 9;

struct Work {
    int32_t b, h, q_begin, q_end;
};

// Tiles of the grad_value pass that a level contributes: its pixels [base, base + H*W), clipped
// to the value tensor, in pieces of 2^tile_px_log2.  *pixels receives the clipped pixel count.
MXD_HD inline int32_t level_tile_count(int32_t H, int32_t W, int32_t base, int32_t nk, int32_t tile_px_log2, int32_t* pixels)
{
    *pixels = 0;
    if (H <= 0 || W <= 0 || base < 0 || base >= nk) return 0;
    int64_t P = (int64_t)H * W;
    if (base + P > nk) P = nk - base;  // never address past the value tensor
    *pixels = (int32_t)P;
    return (int32_t)((P + ((int64_t)1 << tile_px_log2) - 1) >> tile_px_log2);
}

// Decode a workgroup index.  Returns false when the workgroup has nothing to do.
MXD_HD inline bool decode_block(const mxd_msda_plan& p, uint32_t bid, int32_t bs, int32_t nh, int32_t nq, Work* w)
{
    int32_t b, h, t;
    if (p.xcd_mode == 1) {
        const int32_t x = bid % kNumXcd, j = bid / kNumXcd;
        const int32_t hs = j % p.heads_per_xcd;
        const int32_t r = j / p.heads_per_xcd;
        t = r % p.ntiles;
        b = r / p.ntiles;
        h = x * p.heads_per_xcd + hs;
    } else if (p.xcd_mode == 2) {
        const int32_t x = bid % kNumXcd, j = bid / kNumXcd;
        h = x % nh;
        const int32_t part = x / nh;
        t = part + p.xcds_per_head * (j % p.tiles_per_part);
        b = j / p.tiles_per_part;
    } else {
        h = bid % nh;
        const int32_t r = bid / nh;
        t = r % p.ntiles;
        b = r / p.ntiles;
    }
    if (b >= bs || t >= p.ntiles || h >= nh) return false;
    w->b = b;
    w->h = h;
    w->q_begin = t * p.tile_q;
    const int32_t e = w->q_begin + p.tile_q;
    w->q_end = e < nq ? e : nq;
    return true;
}

}  // namespace mxd
