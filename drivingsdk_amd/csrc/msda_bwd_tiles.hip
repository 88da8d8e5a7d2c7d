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
//     tile of one (batch, head); LANE i OWNS PIXEL i of the tile and keeps that pixel's
//     channels in registers for the whole kernel.
//   * The backward's first kernel leaves, per sample, the pixel index of its top-left corner
//     in a level-major key array.  The owner scans the keys of its (batch, head, level) --
//     4 contiguous bytes per sample -- and rejects samples that cannot touch the tile with
//     two compares.  For the rest it recomputes the geometry and, per corner inside the
//     tile, appends an entry {query, weight} to that PIXEL's linked list in LDS (one integer
//     exchange on the list head; entry storage is private to the wavefront, so no allocation
//     atomics are needed).
//   * When the entry storage fills up (or the scan ends) the workgroup meets at a barrier and
//     every lane walks its own pixel's list: fetch the grad_out row of the entry's query,
//     fma into the registers.  No atomics, no read-modify-write of shared accumulators.
//   * At the end each wavefront transposes its registers through LDS and writes whole rows:
//     plain stores for tiles a single workgroup owns, a few atomics per workgroup for tiles of
//     hot (coarse) levels, which are split over several workgroups by query range.
//
// Which (level, tile, query chunk) a workgroup works on is derived on the device from
// spatial_shapes / level_start_index, which never leave device memory; the host only needs
// an upper bound of the number of work items, which follows from nk, nq, nl and np.
#include "msda_device.h"

namespace mxd {

constexpr uint32_t kNil = 0xFFFFFFFFu;

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
__global__ __launch_bounds__(kTilePx) void msda_gradv_tiles_kernel(const KArgs a, const TileArgs t)
{
    constexpr int NW = kTilePx / kWave;                 // wavefronts per workgroup
    __shared__ uint32_t heads[kTilePx];                 // list head per pixel (entry index or kNil)
    __shared__ uint32_t ent_q[NW * kTileEntCap];        // entry: query index
    __shared__ float ent_w[NW * kTileEntCap];           //        weight
    __shared__ uint32_t ent_next[NW * kTileEntCap];     //        next entry of the same pixel
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
    float* tr = reinterpret_cast<float*>(&ent_q[seg]);

    for (int cb = 0; cb < hd; cb += CH) {
        float acc[CH];
#pragma unroll
        for (int c = 0; c < CH; ++c) acc[c] = 0.0f;

        int cursor = my_begin;   // wavefront-uniform
        bool counted = false;    // this wavefront has reported the end of its candidates
        while (true) {
            // ---- scan + append ------------------------------------------------------------
            int count = 0;  // entries of this wavefront in this round (uniform)
            while (cursor < my_end && count + 4 * kWave <= kTileEntCap) {
                const int idx = cursor + lane;
                int32_t key = INT32_MIN;
                if (idx < my_end) key = keys[idx];
                cursor += kWave;
                // corners are key, key+1, key+W, key+W+1
                const bool maybe = (key != INT32_MIN) && ((int64_t)key + it.W + 1 >= it.p0) && (key < it.p1);
                int lp[4] = {-1, -1, -1, -1};
                float wv[4] = {0.f, 0.f, 0.f, 0.f};
                int q = 0;
                if (maybe) {
                    q = idx / a.np;
                    const int p = idx - q * a.np;
                    const int64_t e = (bh_base + (int64_t)q * a.nh) * a.S_full + s_first + p;
                    const float x = to_f32(loc[2 * e]);
                    const float y = to_f32(loc[2 * e + 1]);
                    const float aw = to_f32(attn[e]);
                    const Sample sm = sample_geometry(x, y, level, a.nk, true);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        if (sm.cvalid[k] && sm.pix[k] >= it.p0 && sm.pix[k] < it.p1) {
                            lp[k] = sm.pix[k] - it.p0;
                            wv[k] = sm.w[k] * aw;
                        }
                    }
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const bool push = lp[k] >= 0;
                    const uint64_t mask = __ballot(push);
                    if (mask) {
                        if (push) {
                            const uint32_t pos = seg + count +
                                                 __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                                                           __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
                            ent_q[pos] = (uint32_t)q;
                            ent_w[pos] = wv[k];
                            ent_next[pos] = atomicExch(&heads[lp[k]], pos);
                        }
                        count += __builtin_popcountll(mask);
                    }
                }
            }
            if (cursor >= my_end && !counted) {
                counted = true;
                if (lane == 0) atomicAdd(&done_count, 1);
            }
            __syncthreads();
            const bool all_done = done_count == NW;

            // ---- every lane walks the list of its own pixel -------------------------------
            uint32_t e = heads[tid];
            heads[tid] = kNil;
            while (e != kNil) {
                const uint32_t q = ent_q[e];
                const float w = ent_w[e];
                e = ent_next[e];
                const T* gr = gout + (bh_base + (int64_t)q * a.nh) * hd + cb;
#pragma unroll
                for (int c = 0; c < CH; c += VEC) {
                    if (cb + c < hd) {
                        float g[VEC];
                        RowIO<T, VEC>::load_global(gr + c, g);
#pragma unroll
                        for (int v = 0; v < VEC; ++v) acc[c + v] = __builtin_fmaf(w, g[v], acc[c + v]);
                    }
                }
            }
            __syncthreads();
            if (all_done) break;
        }

        // ---- write the CH channels of this tile: transpose through LDS, 8 pixels at a time ----
        constexpr int TP = 8;                  // pixels per transposition step
        constexpr int TS = CH + 1;             // padded row stride (LDS banks)
        static_assert(TP * TS <= kTileEntCap, "transposition scratch must fit the entry storage");
        const int nch = (hd - cb) < CH ? (hd - cb) : CH;
        for (int half = 0; half < kWave / TP; ++half) {
            wave_lds_sync();
            if ((lane / TP) == half) {
#pragma unroll
                for (int c = 0; c < CH; ++c) tr[(lane % TP) * TS + c] = acc[c];
            }
            wave_lds_sync();
            const int px_base = wave * kWave + half * TP;
            for (int i = lane; i < TP * nch; i += kWave) {
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
    // grad_out rows are read with 16-byte loads when head_dim and the pointer allow it
    constexpr int WIDE = 16 / (int)sizeof(T);
    if (t.vec == WIDE)
        hipLaunchKernelGGL((msda_gradv_tiles_kernel<T, 32, WIDE>), dim3(t.grid), dim3(t.block), 0, stream, a, t);
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
