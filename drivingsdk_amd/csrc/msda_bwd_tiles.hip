// grad_value by tile ownership (gfx950, wave64) -- the scatter half of the backward pass.
//
//   grad_value[b, pix_c, h, :] += w_c * attn * grad_out[b, q, h, :]     for the 4 corners c
//
// (reference: kernels/multi_scale_deformable_attn/op_kernel/multi_scale_deformable_attn_grad.cpp:52-126,181-186,
//  where the same sums are issued as atomic-add DMAs.)
//
// Measured on MI355X: a global fp32 atomic is carried out at the memory side at ~20 G
// 64-byte requests/s, and an LDS fp32 atomic add retires ~0.3 lanes per clock per CU.  Either
// makes a per-sample scatter cost milliseconds.  Integer LDS atomics, plain LDS traffic and
// registers are fast, so the scatter is turned inside out:
//
//   * The pixels of every level are cut into tiles of kTilePx pixels.  A workgroup owns one
//     tile of one (batch, head); every group of 4 lanes owns 4 pixels of the tile and keeps
//     their channels in registers for the whole kernel.
//   * The backward's first kernel leaves, per sample, the pixel index of its top-left corner
//     in a level-major key array.  The owner scans the keys of its (batch, head, level) --
//     4 contiguous bytes per sample -- and rejects samples that cannot touch the tile with
//     two compares.  Survivors are compacted (ballot + prefix) so that the geometry runs on
//     dense batches of 64; per corner inside the tile an entry {query, weight} is appended to
//     that PIXEL's linked list in LDS (one integer exchange on the list head; entry storage
//     is private to the wavefront, so no allocation atomics are needed).
//   * When the entry storage fills up (or the scan ends) the workgroup meets at a barrier and
//     every lane group walks the lists of its own pixels: coalesced 16-byte loads of the
//     grad_out row of the entry's query, fma into the registers.  No atomics, no
//     read-modify-write of shared accumulators.
//   * At the end each wavefront passes its registers through LDS and writes whole rows:
//     plain stores for tiles a single workgroup owns, a few atomics per workgroup for tiles of
//     hot (coarse) levels, which are split over several workgroups by query range.
//
// Which (level, tile, query chunk) a workgroup works on is derived on the device from
// spatial_shapes / level_start_index, which never leave device memory; the host only needs
// an upper bound of the number of work items, which follows from nk, nq, nl and np.
#include "msda_device.h"

namespace mxd {

constexpr uint32_t kNil = 0xFFFFFFFFu;
constexpr int kLpp = 4;                                  // lanes per pixel row = pixels per lane group
constexpr int kScanBlocks = 8;                           // blocks of 64 keys fetched together
constexpr int kCandCap = kWave + kScanBlocks * kWave;    // accepted candidates a wavefront can hold

// Work item table, evaluated identically by every workgroup.
struct TileItem {
    int32_t level, H, W, base;   // level geometry
    int32_t p0, p1;              // pixel range of the tile, relative to the batch element
    int32_t q0, q1;              // query range
    int32_t exclusive;           // 1: no other workgroup touches this tile
};

__device__ inline bool decode_tile_item(const KArgs& a, const TileArgs& t, int32_t item, TileItem* out)
{
    int32_t first = 0;
    for (int l = 0; l < a.nl; ++l) {
        const int32_t H = a.shapes[2 * l], W = a.shapes[2 * l + 1], base = a.lsi[l];
        if (H <= 0 || W <= 0) continue;
        int64_t P = (int64_t)H * W;
        if (base < 0 || base >= a.nk) continue;
        if (base + P > a.nk) P = a.nk - base;  // never address past the value tensor
        const int32_t nt = (int32_t)((P + t.tile_px - 1) / t.tile_px);
        const int32_t tpx = (int32_t)((P + nt - 1) / nt);
        const int64_t expect = ((int64_t)a.nq * a.np) / nt;
        int32_t chunks = (int32_t)((expect + t.target - 1) / t.target);
        if (chunks < 1) chunks = 1;
        if (chunks > t.max_chunks) chunks = t.max_chunks;
        const int32_t n = nt * chunks;
        if (item < first + n) {
            const int32_t ti = (item - first) / chunks, ci = (item - first) % chunks;
            const int32_t qc = (a.nq + chunks - 1) / chunks;
            out->level = l;
            out->H = H;
            out->W = W;
            out->base = base;
            out->p0 = base + ti * tpx;
            const int64_t e = (int64_t)out->p0 + tpx;
            out->p1 = (int32_t)(e < base + P ? e : base + P);
            out->q0 = ci * qc;
            out->q1 = (out->q0 + qc) < a.nq ? (out->q0 + qc) : a.nq;
            out->exclusive = chunks == 1;
            return out->p0 < out->p1 && out->q0 < out->q1;
        }
        first += n;
    }
    return false;
}

// CH = channels a lane accumulates per pass (registers); heads with more channels are done in
// several passes over the same candidates.  VEC = elements per load of a grad_out row.
template <typename T, int CH, int VEC>
__global__ __launch_bounds__(kTilePx, 4) void msda_gradv_tiles_kernel(const KArgs a, const TileArgs t)
{
    constexpr int CHL = CH / kLpp;                      // channels per lane
    constexpr int NPC = CHL / 4;                        // 4-channel pieces per lane
    static_assert(CH % (4 * kLpp) == 0 && 4 % VEC == 0, "a lane owns whole 4-channel pieces");
    constexpr int NW = kTilePx / kWave;                 // wavefronts per workgroup
    __shared__ uint32_t heads[kTilePx];                 // list head per pixel (entry index or kNil)
    __shared__ uint32_t ent_g[NW * kTileEntCap];        // entry: byte offset of the grad_out row
    __shared__ float ent_w[NW * kTileEntCap];           //        weight
    __shared__ uint32_t ent_next[NW * kTileEntCap];     //        next entry of the same pixel
    __shared__ uint32_t cq_all[NW * kCandCap];          // accepted candidate indices, per wavefront
    __shared__ TileItem item_s;
    __shared__ int item_ok;
    __shared__ int done_count;

    Work wk;
    if (!decode_block(t.map, blockIdx.x, a.bs, a.nh, t.items_per_bh, &wk)) return;
    if (threadIdx.x == 0) {
        item_ok = decode_tile_item(a, t, wk.q_begin, &item_s) ? 1 : 0;
        done_count = 0;
    }
    heads[threadIdx.x] = kNil;
    __syncthreads();
    if (!item_ok) return;  // uniform
    const TileItem it = item_s;

    const int hd = a.hd;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;
    const int npx = it.p1 - it.p0;
    const uint32_t seg = wave * kTileEntCap;  // this wavefront's entry storage
    uint32_t* cq = cq_all + wave * kCandCap;

    const T* loc = static_cast<const T*>(a.loc);
    const T* attn = static_cast<const T*>(a.attn);
    const T* gout = static_cast<const T*>(a.grad_out);
    const i32x4 level = {it.H, it.W, it.base, 0};
    const int64_t bh_base = ((int64_t)wk.b * a.nq) * a.nh + wk.h;  // unit index = bh_base + q*nh
    const int s_first = it.level * a.np;

    // keys of this (batch, head, level), query-major then point: contiguous for a query range
    const int32_t* keys = a.keys + ((((int64_t)wk.b * a.nh + wk.h) * a.nl + it.level) * a.nq) * a.np;
    const int cand_begin = it.q0 * a.np, cand_end = it.q1 * a.np;
    // contiguous share of the candidates per wavefront, in blocks of 64
    const int nblk = (cand_end - cand_begin + kWave - 1) / kWave;
    const int blk_per_wave = (nblk + NW - 1) / NW;
    const int my_begin = cand_begin + wave * blk_per_wave * kWave;
    int my_end = my_begin + blk_per_wave * kWave;
    if (my_end > cand_end) my_end = cand_end;

    float* gimg = a.grad_value + (size_t)wk.b * (a.gbatch_bytes / 4);
    const int64_t row_pitch = (int64_t)a.nh * hd;  // floats between neighbouring pixels
    // transposition scratch of this wavefront (aliases its entry storage; used only after the last round)
    float* tr = &ent_w[seg];
    const uint32_t row_bytes = (uint32_t)(a.nh * hd * (int)sizeof(T));  // between the grad_out rows of two queries
    // grad_out of this batch element as a bound buffer: offsets >= 2^31 read as zeros
    const uint32_t gout_batch_bytes = (uint32_t)a.nq * row_bytes;
    const __amdgpu_buffer_rsrc_t gres =
        make_rsrc(reinterpret_cast<const char*>(gout) + (size_t)wk.b * gout_batch_bytes, gout_batch_bytes);
    const uint32_t ghead_off = (uint32_t)wk.h * hd * (uint32_t)sizeof(T);
    // the last entry slot of every wavefront is its dummy entry
    const uint32_t dummy = seg + kTileEntCap - 1;
    if (lane == 0) {
        ent_g[dummy] = kInvalidCorner;
        ent_w[dummy] = 0.0f;
        ent_next[dummy] = kNil;
    }

    for (int cb = 0; cb < hd; cb += CH) {
        // lane j of group g = tid/kLpp keeps, for each of the pixels g*kLpp .. g*kLpp+kLpp-1, channels
        // 4j..4j+3 of every piece of 4*kLpp channels
        float acc[kLpp][CHL];
#pragma unroll
        for (int i = 0; i < kLpp; ++i)
#pragma unroll
            for (int c = 0; c < CHL; ++c) acc[i][c] = 0.0f;

        int cursor = my_begin;   // next unscanned candidate of this wavefront (uniform)
        int32_t pre[kScanBlocks];  // keys of the blocks at `cursor`, fetched one step ahead
        auto load_keys = [&](int base) {
#pragma unroll
            for (int j = 0; j < kScanBlocks; ++j) {
                const int idx = base + j * kWave + lane;
                pre[j] = idx < my_end ? __builtin_nontemporal_load(keys + idx) : INT32_MIN;
            }
        };
        load_keys(my_begin);
        int ncq = 0;             // accepted candidates waiting in cq (uniform)
        bool counted = false;    // this wavefront has reported the end of its work
        while (true) {
            // ---- scan keys, compact accepted candidates, append list entries ---------------
            int count = 0;  // entries of this wavefront in this round (uniform)
            while (true) {
                // (1) refill the candidate queue from the keys fetched one step ahead, and put the
                // next kScanBlocks blocks of 64 keys in flight before testing the current ones
                while (cursor < my_end && ncq < kWave) {
                    int32_t key[kScanBlocks];
#pragma unroll
                    for (int j = 0; j < kScanBlocks; ++j) key[j] = pre[j];
                    load_keys(cursor + kScanBlocks * kWave);
#pragma unroll
                    for (int j = 0; j < kScanBlocks; ++j) {
                        // corners are key, key+1, key+W, key+W+1
                        const bool maybe =
                            (key[j] != INT32_MIN) && ((int64_t)key[j] + it.W + 1 >= it.p0) && (key[j] < it.p1);
                        const uint64_t mask = __ballot(maybe);
                        if (mask) {
                            if (maybe)
                                cq[ncq + __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                                                   __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0))] =
                                    cursor + j * kWave + lane;
                            ncq += __builtin_popcountll(mask);
                        }
                    }
                    cursor += kScanBlocks * kWave;
                }
                // (2) a dense batch of accepted candidates: geometry + list append
                const bool flush_tail = cursor >= my_end && ncq > 0;
                if (!(ncq >= kWave || flush_tail)) break;           // nothing left to do
                if (count + 4 * kWave > kTileEntCap - 1) break;     // entry storage full: next round
                const int take = ncq < kWave ? ncq : kWave;
                wave_lds_sync();
                int lp[4] = {-1, -1, -1, -1};
                float wv[4] = {0.f, 0.f, 0.f, 0.f};
                int q = 0;
                if (lane < take) {
                    const int idx = cq[ncq - take + lane];
                    q = idx / a.np;
                    const int p = idx - q * a.np;
                    const int64_t e = (bh_base + (int64_t)q * a.nh) * a.S_full + s_first + p;
                    const float x = to_f32(__builtin_nontemporal_load(loc + 2 * e));
                    const float y = to_f32(__builtin_nontemporal_load(loc + 2 * e + 1));
                    const float aw = to_f32(__builtin_nontemporal_load(attn + e));
                    const Sample sm = sample_geometry(x, y, level, a.nk, true);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        if (sm.cvalid[k] && sm.pix[k] >= it.p0 && sm.pix[k] < it.p1) {
                            lp[k] = sm.pix[k] - it.p0;
                            wv[k] = sm.w[k] * aw;
                        }
                    }
                }
                ncq -= take;
                wave_lds_sync();
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const bool push = lp[k] >= 0;
                    const uint64_t mask = __ballot(push);
                    if (mask) {
                        if (push) {
                            const uint32_t pos = seg + count +
                                                 __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                                                           __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
                            ent_g[pos] = (uint32_t)q * row_bytes;
                            ent_w[pos] = wv[k];
                            ent_next[pos] = atomicExch(&heads[lp[k]], pos);
                        }
                        count += __builtin_popcountll(mask);
                    }
                }
            }
            if (cursor >= my_end && ncq == 0 && !counted) {
                counted = true;
                if (lane == 0) atomicAdd(&done_count, 1);
            }
            __syncthreads();
            const bool all_done = done_count == NW;

            // ---- every group of kLpp lanes walks the lists of its kLpp pixels -----------------
            // The lanes of a group read one grad_out row with coalesced 16-byte buffer loads
            // (lane j: channels 4j..4j+3 of every 4*kLpp-channel piece).  The loop body is
            // branch-free: a list that has ended keeps "reading" the wavefront's dummy entry
            // (weight 0, out-of-range row offset, for which the buffer load returns zeros), the
            // trip count is the longest list in the wavefront.  Two entries per trip, so that the
            // row of the next entry is in flight while the fmas of the current one run.
            {
                const int grp = tid / kLpp, j = tid % kLpp;
                uint32_t piece_off[NPC];
#pragma unroll
                for (int p = 0; p < NPC; ++p) {
                    const int ch = cb + p * (kLpp * 4) + j * 4;
                    // channels past head_dim re-read channel 0; their sums are never written out
                    piece_off[p] = ghead_off + (uint32_t)(ch < hd ? ch : 0) * (uint32_t)sizeof(T);
                }
                auto fetch = [&](uint32_t& e, float (&g)[CHL], float& w) {
                    const uint32_t goff = ent_g[e];
                    w = ent_w[e];
                    const uint32_t nx = ent_next[e];
#pragma unroll
                    for (int p = 0; p < NPC; ++p) {
#pragma unroll
                        for (int c = 0; c < 4; c += VEC) {
                            float g1[VEC];
                            RowIO<T, VEC>::unpack(
                                RowIO<T, VEC>::load_raw(gres, goff + piece_off[p] + (uint32_t)(c * sizeof(T))), g1);
#pragma unroll
                            for (int v = 0; v < VEC; ++v) g[p * 4 + c + v] = g1[v];
                        }
                    }
                    e = nx == kNil ? dummy : nx;
                };
#pragma unroll
                for (int i = 0; i < kLpp; ++i) {
                    const int px = grp * kLpp + i;
                    uint32_t e = heads[px];
                    if (j == 0) heads[px] = kNil;  // same wavefront: ordered after the read above
                    e = e == kNil ? dummy : e;
                    float ga[CHL], gb[CHL], wa, wb;
                    fetch(e, ga, wa);
                    while (__ballot(e != dummy)) {
                        fetch(e, gb, wb);
#pragma unroll
                        for (int c = 0; c < CHL; ++c) acc[i][c] = __builtin_fmaf(wa, ga[c], acc[i][c]);
                        fetch(e, ga, wa);
#pragma unroll
                        for (int c = 0; c < CHL; ++c) acc[i][c] = __builtin_fmaf(wb, gb[c], acc[i][c]);
                    }
#pragma unroll
                    for (int c = 0; c < CHL; ++c) acc[i][c] = __builtin_fmaf(wa, ga[c], acc[i][c]);
                }
            }
            __syncthreads();
            if (all_done) break;
        }

        // ---- write the CH channels of this tile -------------------------------------------
        // Eight pixels at a time are parked in LDS; the whole wavefront then writes them with
        // consecutive lanes on consecutive floats (full 64-byte pieces per request).
        constexpr int TPX = 8;      // pixels per step
        constexpr int TS = CH + 1;  // padded row stride (LDS banks)
        static_assert(TPX * TS <= kTileEntCap, "transposition scratch must fit the entry storage");
        const int nch = (hd - cb) < CH ? (hd - cb) : CH;
        for (int o = 0; o < kWave / TPX; ++o) {
            wave_lds_sync();
            if ((lane / TPX) == o) {
                // the TPX lanes of this step are TPX/kLpp groups, each holding kLpp pixels
                const int gl = (lane % TPX) / kLpp, j = lane % kLpp;
#pragma unroll
                for (int i = 0; i < kLpp; ++i)
#pragma unroll
                    for (int p = 0; p < NPC; ++p)
#pragma unroll
                        for (int c = 0; c < 4; ++c)
                            tr[(gl * kLpp + i) * TS + p * (kLpp * 4) + j * 4 + c] = acc[i][p * 4 + c];
            }
            wave_lds_sync();
            const int px_base = wave * kWave + o * TPX;
            for (int i = lane; i < TPX * nch; i += kWave) {
                const int pl = i / nch, c = i - pl * nch;
                const int px = px_base + pl;
                if (px < npx) {
                    const float v = tr[pl * TS + c];
                    float* dst = gimg + (int64_t)(it.p0 + px) * row_pitch + (int64_t)wk.h * hd + cb + c;
                    if (it.exclusive && !t.accumulate)
                        *dst = v;
                    else if (it.exclusive)
                        *dst += v;
                    else
                        unsafeAtomicAdd(dst, v);
                }
            }
        }
        wave_lds_sync();
        if (cb + CH < hd) {
            // next channel pass starts from a clean state
            __syncthreads();
            if (threadIdx.x == 0) done_count = 0;
            __syncthreads();
        }
    }
}

template <typename T>
static hipError_t launch_t(const KArgs& a, const TileArgs& t, hipStream_t stream)
{
    // an octet of lanes reads a 32-channel slice of a grad_out row, 4 channels per lane: one
    // load per lane when head_dim and the pointer alignment allow it
    if (t.vec >= 4)
        hipLaunchKernelGGL((msda_gradv_tiles_kernel<T, 32, 4>), dim3(t.grid), dim3(t.block), 0, stream, a, t);
    else if (t.vec == 2)
        hipLaunchKernelGGL((msda_gradv_tiles_kernel<T, 32, 2>), dim3(t.grid), dim3(t.block), 0, stream, a, t);
    else
        hipLaunchKernelGGL((msda_gradv_tiles_kernel<T, 32, 1>), dim3(t.grid), dim3(t.block), 0, stream, a, t);
    return hipGetLastError();
}

hipError_t launch_gradv_tiles(int dtype, const KArgs& a, const TileArgs& t, hipStream_t stream)
{
    switch (dtype) {
        case MXD_DTYPE_F32: return launch_t<float>(a, t, stream);
        case MXD_DTYPE_F16: return launch_t<f16_t>(a, t, stream);
        case MXD_DTYPE_BF16: return launch_t<bf16_t>(a, t, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace mxd
