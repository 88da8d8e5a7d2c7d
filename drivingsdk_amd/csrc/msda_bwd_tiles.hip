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

constexpr int kLpp = 8;                                  // lanes per pixel row = pixels per lane group
constexpr int kScanBlocks = 4;                           // blocks of 64 keys fetched together
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

// CH = channels a lane group accumulates per pass (registers); heads with more channels are
// done in several passes over the same candidates.  VEC = elements per load of a grad_out row.
template <typename T, int CH, int VEC>
__global__ __launch_bounds__(kTilePx, 4) void msda_gradv_tiles_kernel(const KArgs a, const TileArgs t)
{
    constexpr int CHL = CH / kLpp;                      // channels per lane
    static_assert(CHL == 4 && 4 % VEC == 0, "a lane owns one 4-channel piece of a row");
    constexpr int NW = kTilePx / kWave;                 // wavefronts per workgroup
    constexpr uint32_t kDummyOfWave = kTileEntCap - 1;  // last entry slot of every wavefront
    __shared__ uint32_t heads[kTilePx];                 // list head per pixel (entry index)
    // entry: {byte offset of the grad_out row, weight for the list's pixel, weight for the
    // next pixel, next entry of the same list}
    __shared__ u32x4 ent[NW * kTileEntCap];
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
    // an empty list points at the dummy entry of the wavefront that owns the pixel
    heads[threadIdx.x] = (threadIdx.x >> 6) * kTileEntCap + kDummyOfWave;
    __syncthreads();
    if (!item_ok) return;  // uniform
    const TileItem it = item_s;

    const int hd = a.hd;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;
    const int npx = it.p1 - it.p0;
    // A tile much smaller than the workgroup is held in several copies (lists and registers),
    // each taking the samples of some queries; the copies meet in the image through atomics.
    const int npx_pad = (npx + kLpp - 1) / kLpp * kLpp;
    int copies = 1;
    while (copies < 8 && 2 * copies * npx_pad <= kTilePx) copies *= 2;
    const bool owned = it.exclusive && copies == 1;  // plain stores are enough
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
    const uint32_t row_bytes = (uint32_t)(a.nh * hd * (int)sizeof(T));  // between the grad_out rows of two queries
    // grad_out of this batch element as a bound buffer: offsets >= 2^31 read as zeros
    const uint32_t gout_batch_bytes = (uint32_t)a.nq * row_bytes;
    const __amdgpu_buffer_rsrc_t gres =
        make_rsrc(reinterpret_cast<const char*>(gout) + (size_t)wk.b * gout_batch_bytes, gout_batch_bytes);
    const uint32_t ghead_off = (uint32_t)wk.h * hd * (uint32_t)sizeof(T);
    // the dummy entry ends every list of this wavefront's pixels: weight 0, a row offset the
    // buffer range check answers with zeros (at no cost in the memory pipeline), next = itself
    const uint32_t dummy = seg + kDummyOfWave;
    if (lane == 0) ent[dummy] = u32x4{kInvalidCorner, 0u, 0u, dummy};

    // lane j of group g = tid/kLpp keeps channels 4j..4j+3 of the pixels g*kLpp .. g*kLpp+kLpp-1
    const int grp = tid / kLpp, j = tid % kLpp;

    for (int cb = 0; cb < hd; cb += CH) {
        float acc[kLpp][CHL];
#pragma unroll
        for (int i = 0; i < kLpp; ++i)
#pragma unroll
            for (int c = 0; c < CHL; ++c) acc[i][c] = 0.0f;
        // channels past head_dim re-read channel 0; their sums are never written out
        const int my_ch = cb + j * 4;
        const uint32_t lane_off = ghead_off + (uint32_t)(my_ch < hd ? my_ch : 0) * (uint32_t)sizeof(T);

        int cursor = my_begin;   // next unscanned candidate of this wavefront (uniform)
        int32_t pre[kScanBlocks];  // keys of the blocks at `cursor`, fetched one step ahead
        auto load_keys = [&](int base) {
#pragma unroll
            for (int jb = 0; jb < kScanBlocks; ++jb) {
                const int idx = base + jb * kWave + lane;
                pre[jb] = idx < my_end ? __builtin_nontemporal_load(keys + idx) : INT32_MIN;
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
                    for (int jb = 0; jb < kScanBlocks; ++jb) key[jb] = pre[jb];
                    load_keys(cursor + kScanBlocks * kWave);
#pragma unroll
                    for (int jb = 0; jb < kScanBlocks; ++jb) {
                        // corners are key, key+1, key+W, key+W+1
                        const bool maybe =
                            (key[jb] != INT32_MIN) && ((int64_t)key[jb] + it.W + 1 >= it.p0) && (key[jb] < it.p1);
                        const uint64_t mask = __ballot(maybe);
                        if (mask) {
                            if (maybe)
                                cq[ncq + __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                                                   __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0))] =
                                    cursor + jb * kWave + lane;
                            ncq += __builtin_popcountll(mask);
                        }
                    }
                    cursor += kScanBlocks * kWave;
                }
                // (2) a dense batch of accepted candidates: geometry + list append
                const bool flush_tail = cursor >= my_end && ncq > 0;
                if (!(ncq >= kWave || flush_tail)) break;                      // nothing left to do
                if (count + 4 * kWave > (int)kDummyOfWave) break;              // entry storage full: next round
                const int take = ncq < kWave ? ncq : kWave;
                wave_lds_sync();
                // A sample touches two pixel pairs (p, p+1): its upper and its lower corners.  A pair
                // whose pixels belong to the same lane group becomes ONE entry in the list of the left
                // pixel (the grad_out row is fetched once for both); otherwise each corner inside the
                // tile gets an entry of its own with no weight for the neighbour.
                int lst[4] = {-1, -1, -1, -1};   // list (pixel inside the tile) of up to 4 entries
                float w0[4] = {0.f, 0.f, 0.f, 0.f}, w1[4] = {0.f, 0.f, 0.f, 0.f};
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
                    const int copy_off = (q & (copies - 1)) * npx_pad;
#pragma unroll
                    for (int r = 0; r < 2; ++r) {
                        const int pl = sm.pix[2 * r] - it.p0;  // left pixel of the pair, relative to the tile
                        const bool in_l = sm.cvalid[2 * r] && pl >= 0 && pl < npx;
                        const bool in_r = sm.cvalid[2 * r + 1] && pl + 1 >= 0 && pl + 1 < npx;
                        const bool pair = in_l && in_r && (pl % kLpp) != kLpp - 1;
                        if (in_l) {
                            lst[2 * r] = pl + copy_off;
                            w0[2 * r] = sm.w[2 * r] * aw;
                            w1[2 * r] = pair ? sm.w[2 * r + 1] * aw : 0.0f;
                        }
                        if (in_r && !pair) {
                            lst[2 * r + 1] = pl + 1 + copy_off;
                            w0[2 * r + 1] = sm.w[2 * r + 1] * aw;
                        }
                    }
                }
                ncq -= take;
                wave_lds_sync();
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const bool push = lst[k] >= 0;
                    const uint64_t mask = __ballot(push);
                    if (mask) {
                        if (push) {
                            const uint32_t pos = seg + count +
                                                 __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                                                           __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
                            const uint32_t next = atomicExch(&heads[lst[k]], pos);
                            ent[pos] = u32x4{(uint32_t)q * row_bytes, __builtin_bit_cast(uint32_t, w0[k]),
                                             __builtin_bit_cast(uint32_t, w1[k]), next};
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
            // The lanes of a group read one grad_out row with ONE coalesced load (lane j: channels
            // 4j..4j+3): the memory pipeline's cost is per cache line touched by an instruction.
            // The loop body is branch-free: a list that has ended keeps "reading" the dummy entry.
            // Two lists are walked together, two entries of each per trip, so that four row loads
            // are in flight while the fmas of the previous ones run.
            {
                auto fetch = [&](uint32_t& e, float (&g)[CHL], float& wa, float& wb) {
                    const u32x4 en = ent[e];
                    // (a bit cast applied directly to a vector element picks up element 0: copy first)
                    const uint32_t ya = en.y, za = en.z;
                    wa = __builtin_bit_cast(float, ya);
                    wb = __builtin_bit_cast(float, za);
#pragma unroll
                    for (int c = 0; c < 4; c += VEC) {
                        float g1[VEC];
                        RowIO<T, VEC>::unpack(RowIO<T, VEC>::load_raw(gres, en.x + lane_off + (uint32_t)(c * sizeof(T))), g1);
#pragma unroll
                        for (int v = 0; v < VEC; ++v) g[c + v] = g1[v];
                    }
                    e = en.w;
                };
#pragma unroll
                for (int i = 0; i < kLpp; i += 2) {
                    const int px = grp * kLpp + i;
                    uint32_t ea = heads[px], eb = heads[px + 1];
                    if (j == 0) {  // same wavefront: ordered after the reads above
                        heads[px] = dummy;
                        heads[px + 1] = dummy;
                    }
                    float ga0[CHL], ga1[CHL], gb0[CHL], gb1[CHL];
                    float ua0, va0, ua1, va1, ub0, vb0, ub1, vb1;
                    auto fma_a = [&](const float (&g)[CHL], float u, float v) {
#pragma unroll
                        for (int c = 0; c < CHL; ++c) {
                            acc[i][c] = __builtin_fmaf(u, g[c], acc[i][c]);
                            acc[i + 1][c] = __builtin_fmaf(v, g[c], acc[i + 1][c]);
                        }
                    };
                    auto fma_b = [&](const float (&g)[CHL], float u, float v) {
#pragma unroll
                        for (int c = 0; c < CHL; ++c) {
                            acc[i + 1][c] = __builtin_fmaf(u, g[c], acc[i + 1][c]);
                            if (i + 2 < kLpp) acc[(i + 2) % kLpp][c] = __builtin_fmaf(v, g[c], acc[(i + 2) % kLpp][c]);
                        }
                    };
                    fetch(ea, ga0, ua0, va0);
                    fetch(eb, gb0, ub0, vb0);
                    while (__ballot(ea != dummy || eb != dummy)) {
                        fetch(ea, ga1, ua1, va1);
                        fetch(eb, gb1, ub1, vb1);
                        fma_a(ga0, ua0, va0);
                        fma_b(gb0, ub0, vb0);
                        fetch(ea, ga0, ua0, va0);
                        fetch(eb, gb0, ub0, vb0);
                        fma_a(ga1, ua1, va1);
                        fma_b(gb1, ub1, vb1);
                    }
                    fma_a(ga0, ua0, va0);
                    fma_b(gb0, ub0, vb0);
                }
            }
            __syncthreads();
            if (all_done) break;
        }

        // ---- write the CH channels of this tile -------------------------------------------
        const int nch = (hd - cb) < CH ? (hd - cb) : CH;
        if (owned && t.store_vec == 4) {
            // the lanes of a group hold a whole row of each of their pixels: 16-byte stores
            if (my_ch < hd) {
#pragma unroll
                for (int i = 0; i < kLpp; ++i) {
                    const int px = grp * kLpp + i;
                    if (px < npx) {
                        f32x4* dst = reinterpret_cast<f32x4*>(gimg + (int64_t)(it.p0 + px) * row_pitch +
                                                              (int64_t)wk.h * hd + my_ch);
                        f32x4 v = {acc[i][0], acc[i][1], acc[i][2], acc[i][3]};
                        if (t.accumulate) v += *dst;
                        *dst = v;
                    }
                }
            }
        } else {
            // Rows shared with other workgroups (tiles split by query range) are added with
            // atomics, which the memory side carries out per 64-byte request: pass the registers
            // through LDS (the entry storage, free after the last round) so that consecutive
            // lanes hold consecutive floats of a row.  32 pixels at a time.
            typedef uint32_t __attribute__((may_alias)) u32_alias;
            static_assert(32 * CH * 4 <= kTileEntCap * 16, "transposition scratch must fit the entry storage");
            u32x4* tr4 = &ent[seg];
            const u32_alias* tr1 = reinterpret_cast<const u32_alias*>(tr4);
            for (int half = 0; half < 2; ++half) {
                wave_lds_sync();
                if (((lane / kLpp) >> 2) == half) {
                    const int gl = (lane / kLpp) & 3;
#pragma unroll
                    for (int i = 0; i < kLpp; ++i)
                        tr4[(gl * kLpp + i) * (CH / 4) + j] =
                            u32x4{__builtin_bit_cast(uint32_t, acc[i][0]), __builtin_bit_cast(uint32_t, acc[i][1]),
                                  __builtin_bit_cast(uint32_t, acc[i][2]), __builtin_bit_cast(uint32_t, acc[i][3])};
                }
                wave_lds_sync();
                const int px_base = wave * kWave + half * 32;
#pragma unroll 4
                for (int k = 0; k < 32 * CH / kWave; ++k) {
                    const int idx = k * kWave + lane;
                    const int pl = idx / CH, c = idx % CH;
                    const int vp = px_base + pl;             // pixel slot of the workgroup
                    const int px = vp - (vp / npx_pad) * npx_pad;  // pixel of the tile (any copy)
                    if (vp < copies * npx_pad && px < npx && c < nch) {
                        const float v = __builtin_bit_cast(float, (uint32_t)tr1[idx]);
                        float* dst = gimg + (int64_t)(it.p0 + px) * row_pitch + (int64_t)wk.h * hd + cb + c;
                        if (!owned)
                            unsafeAtomicAdd(dst, v);
                        else if (t.accumulate)
                            *dst += v;
                        else
                            *dst = v;
                    }
                }
            }
            wave_lds_sync();
        }
        if (cb + CH < hd) {
            // next channel pass starts from a clean state (the dummy entry may have been
            // overwritten by the transposition)
            __syncthreads();
            if (threadIdx.x == 0) done_count = 0;
            if (lane == 0) ent[dummy] = u32x4{kInvalidCorner, 0u, 0u, dummy};
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
