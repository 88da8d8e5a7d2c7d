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
//   * The pixels of every level are cut into tiles.  A workgroup (512 threads) owns one tile of
//     one (batch, head); every thread keeps 32 sums in registers for the whole kernel: a group
//     of 8 lanes owns 8 consecutive pixels of up to 32 channels (tiles of 512 pixels), 4 pixels
//     of up to 64 channels (256) or 2 pixels of up to 128 channels (128), lane j holding
//     channels 4j..4j+3 of every 32-channel block of each -- so that the records are streamed
//     and the lists built and walked once whatever head_dim is (heads of more than 128
//     channels take two passes over 128-pixel tiles).
//   * The backward's first kernel leaves its samples as pair records {pixel, query, weight,
//     weight of the pixel to the right}, sorted by tile inside the slab of each of its
//     workgroups, with a table of run starts.  The owner of a tile streams the runs of its
//     tile (dense batches of 64 records, fetched one batch ahead) and appends an entry per
//     record to the PIXEL's linked list in LDS (one integer exchange on the list head; entry
//     storage is private to the wavefront, so no allocation atomics are needed).
//   * When the entry storage fills up (or the input ends) the workgroup meets at a barrier and
//     every lane group walks the lists of its own pixels: one coalesced load of the grad_out
//     row of the entry's query per group, fma into the registers.  No atomics, no
//     read-modify-write of shared accumulators.  The walk is pipelined by hand: the entries and
//     rows of the next trip are requested before the rows of the current trip are used.
//   * At the end plain 16-byte stores for tiles a single workgroup owns; tiles of hot (coarse)
//     levels are split over several workgroups by query range and tiles much smaller than the
//     workgroup are held in several copies: those pass their registers through LDS and add
//     whole rows with a few atomics per workgroup.
//   * Slots of the workgroup that stand for no pixel take extra lists of pixels that collect
//     far more entries than the others (decided from the counts of a work item's first round),
//     so that a hot pixel's entries are walked by several lane groups side by side.
//
// Which (level, tile, query chunk) a workgroup works on is derived on the device from
// spatial_shapes / level_start_index, which never leave device memory; the host only needs
// an upper bound of the number of work items, which follows from nk, nq, nl and np.
#include "msda_device.h"

namespace mxd {


// Work item table, evaluated identically by every workgroup.
struct TileItem {
    int32_t level, H, W, base;   // level geometry
    int32_t p0, p1;              // pixel range of the tile, relative to the batch element
    int32_t w0, w1;              // range of workgroups of the first kernel whose records are taken
    int32_t tile;                // index of the tile within the (batch, head): column of the run table
    int32_t exclusive;           // 1: no other workgroup touches this tile (the item is not split by query range and the
                                 // levels tile the keys, so that no tile of another level holds the same rows)
};

// What a workgroup needs of every level, derived by one lane per level (LevelInfo::fill) so that the thread that looks up
// the work item afterwards goes through LDS values only: the level loads and the divisions behind the chunk count
// would otherwise be made one level after the other by that one thread, in front of everything the workgroup does.
struct LevelInfo {
    int32_t H[kMaxLevels], W[kMaxLevels], base[kMaxLevels];
    int32_t px[kMaxLevels];      // pixels of the level inside the value tensor
    int32_t nt[kMaxLevels];      // its tiles (before the run table's room is considered)
    int32_t chunks[kMaxLevels];  // query chunks per tile
    int32_t wpc[kMaxLevels];     // first-kernel workgroups per chunk
    __device__ void fill(const KArgs& a, int l)
    {
        const i32x4 L = load_level(a, l);
        int32_t P, w = 0;
        const int32_t n = level_tile_count(L.x, L.y, L.z, a.nk, a.tile_px_log2, &P);
        H[l] = L.x;
        W[l] = L.y;
        base[l] = L.z;
        px[l] = P;
        nt[l] = n;
        chunks[l] = n > 0 ? level_tile_chunks(a, n, &w) : 0;
        wpc[l] = w;
    }
    // levels_tile_the_keys() on the values held here
    __device__ bool tile_the_keys(const KArgs& a) const
    {
        int64_t next = 0;
        int32_t tiles = 0;
        for (int l = 0; l < a.nl; ++l) {
            if (H[l] <= 0 || W[l] <= 0 || (int64_t)base[l] != next) return false;
            const int64_t p = (int64_t)H[l] * W[l];
            next += p;
            if (next > a.nk) return false;
            tiles += (int32_t)((p + ((int64_t)1 << a.tile_px_log2) - 1) >> a.tile_px_log2);
        }
        return next == a.nk && tiles <= a.tbl_stride - 1;
    }
};

// lv_first / lv_nt: scratch of kMaxLevels entries each (first tile and tile count per level).
__device__ inline bool decode_tile_item(const KArgs& a, const TileArgs& t, const LevelInfo& lv, int32_t item, TileItem* out,
                                        int32_t* lv_first, int32_t* lv_nt)
{
    // Tiles are numbered level by level as in the first kernel; a level that does not fit the run table
    // (only possible when the levels overlap) has no tiles.
    int32_t total = 0;
    for (int l = 0; l < a.nl; ++l) {
        const int32_t nt = lv.nt[l];
        const bool fits = total + nt <= a.tbl_stride - 1;
        lv_first[l] = total;
        lv_nt[l] = fits ? nt : 0;
        if (fits) total += nt;
    }
    const bool canonical = lv.tile_the_keys(a);
    // Items are numbered from the last level to the first: the coarse levels, whose tiles are
    // split into many long-running items, start first and the short items of the fine levels
    // fill the end of the launch.
    int32_t first = 0;
    for (int l = a.nl - 1; l >= 0; --l) {
        const int32_t nt = lv_nt[l];
        if (nt == 0) continue;
        const int32_t base = lv.base[l], P = lv.px[l];
        const int32_t wpc = lv.wpc[l], chunks = lv.chunks[l];
        const int32_t n = nt * chunks;
        if (item < first + n) {
            const int32_t ti = (item - first) / chunks, ci = (item - first) % chunks;
            out->level = l;
            out->H = lv.H[l];
            out->W = lv.W[l];
            out->base = base;
            const int32_t tile_px = 1 << a.tile_px_log2;
            out->p0 = base + ti * tile_px;
            out->p1 = (out->p0 + tile_px) < (base + P) ? (out->p0 + tile_px) : (base + P);
            out->w0 = ci * wpc;
            out->w1 = (out->w0 + wpc) < a.nwg ? (out->w0 + wpc) : a.nwg;
            out->tile = lv_first[l] + ti;
            out->exclusive = chunks == 1 && canonical;
            return true;
        }
        first += n;
    }
    return false;
}

// The samples of levels whose tiles found no room in the run table, added to grad_value one sample per thread with
// atomics: share `part` of `parts` of the samples of (batch b, head h).  Only levels that overlap can have more tiles
// between them than the table holds; for such layouts the whole image was zero-filled and every tile adds with atomics
// as well.  Slow, and there so that level_start_index is honoured however it comes.  Plain operator only.
// unfit: kMaxLevels flags in LDS, filled here.
template <typename T>
__device__ inline void add_levels_without_tiles(const KArgs& a, int b, int h, int part, int parts, int32_t* unfit)
{
    __shared__ int any_unfit;
    if (threadIdx.x == 0) {
        int32_t first = 0, any = 0;
        for (int l = 0; l < a.nl; ++l) {
            const i32x4 L = load_level(a, l);
            int32_t P;
            const int32_t nt = level_tile_count(L.x, L.y, L.z, a.nk, a.tile_px_log2, &P);
            const bool fits = first + nt <= a.tbl_stride - 1;
            unfit[l] = fits ? 0 : 1;
            if (fits) first += nt;
            else if (nt > 0) any = 1;
        }
        any_unfit = any;
    }
    __syncthreads();
    if (!any_unfit) return;
    const T* loc = static_cast<const T*>(a.loc);
    const T* attn = static_cast<const T*>(a.attn);
    const T* gout = static_cast<const T*>(a.grad_out);
    float* img = a.grad_value + (size_t)b * (a.gbatch_bytes / 4) + (size_t)h * a.hd;
    const int64_t n = (int64_t)a.nq * a.S;
    for (int64_t i = (int64_t)part * blockDim.x + threadIdx.x; i < n; i += (int64_t)parts * blockDim.x) {
        const int q = (int)(i / a.S), s = (int)(i - (int64_t)q * a.S);
        const int l = (int)(((uint32_t)s * a.np_magic) >> 20);
        if (!unfit[l]) continue;
        const int64_t e = (((int64_t)b * a.nq + q) * a.nh + h) * a.S_full + s;
        const Sample sm = sample_geometry(to_f32(loc[2 * e]), to_f32(loc[2 * e + 1]), load_level(a, l), a.nk, true);
        if (!sm.valid) continue;
        const float aw = to_f32(attn[e]);
        const T* grow = gout + (((int64_t)b * a.nq + q) * a.nh + h) * a.hd;
        for (int ch = 0; ch < a.hd; ++ch) {
            const float gch = to_f32(grow[ch]) * aw;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (sm.cvalid[k]) unsafeAtomicAdd(img + (size_t)sm.pix[k] * ((size_t)a.nh * a.hd) + ch, sm.w[k] * gch);
        }
    }
}

// CHL = channels a lane accumulates per pass, 4 per 32-channel block of the row: 4, 8 or 16, for tiles of 512, 256 or
// 128 pixels (32 sums per lane either way); heads with more than 8 * CHL channels are done in several passes over the
// same records.  VEC = elements per load of a grad_out row.
template <typename T, int CHL, int VEC>
__global__ __launch_bounds__(kTileThreads, 4) void msda_gradv_tiles_kernel(const KArgs a, const TileArgs t)
{
    static_assert((CHL == 4 || CHL == 8 || CHL == 16) && 4 % VEC == 0, "a lane owns one 4-channel piece of every 32-channel block");
    constexpr int CH = kLpp * CHL;                      // channels per pass
    constexpr int NB = CHL / 4;                         // 32-channel blocks per pass
    constexpr int PPG = 32 / CHL;                       // pixels per lane group
    constexpr int kTilePx = (kTileThreads / kLpp) * PPG;  // pixels per tile = pixel slots of the workgroup
    constexpr int kTilePxLog2 = CHL == 4 ? 9 : CHL == 8 ? 8 : 7;
    static_assert((1 << kTilePxLog2) == kTilePx, "tile size");
    // lists a lane group walks together, one entry of each per trip (two trips are in flight: with 16 channels per
    // lane one list's rows take the registers that two lists' take otherwise)
    constexpr int kWalk = CHL >= 16 ? 1 : 2;
    // With 4 channels per lane a lane group also keeps the sums its pairs leave for the pixel behind its last one (the
    // first pixel of the next group) and hands them over when the rounds are done: a pair is then one list entry wherever
    // it lies in the tile, instead of two for the one pair in eight that straddles two groups.  (The wider forms have no
    // registers to spare for it.)
    constexpr bool kOverlap = CHL == 4;
    constexpr int kAccPx = PPG + (kOverlap ? 1 : 0);
    constexpr int kCarryAt = kTileEntCap - 1 - kLpp;    // entries of a wavefront's storage through which its last group hands over
    constexpr int NW = kTileThreads / kWave;            // wavefronts per workgroup
    constexpr uint32_t kDummyOfWave = kTileEntCap - 1;  // last entry slot of every wavefront
    // (a wavefront transposes the sums of half of its lane groups at a time: 4 groups x 32 sums x 8 lanes = 4 KiB)
    constexpr int kSlotPxAt = 4 * PPG * CH / 4;         // first entry behind wavefront 0's transposition scratch
    static_assert(kSlotPxAt + kTileThreads * 2 / 16 <= kCarryAt, "slot map must fit wavefront 0's entry storage");
    __shared__ uint32_t heads[kTileThreads];            // list head per pixel slot (byte offset of the entry in `ent`)
    // entry: {byte offset of the grad_out row, weight for the list's pixel, weight for the
    // next pixel, next entry of the same list}
    __shared__ u32x4 ent[NW * kTileEntCap];
    // up to 64 runs of records per wavefront at a time: first record, records before the run
    __shared__ uint32_t run_src_all[NW * kWave];
    __shared__ uint32_t run_pre_all[NW * kWave];
    __shared__ TileItem item_s;
    __shared__ int32_t lv_first[kMaxLevels], lv_nt[kMaxLevels];
    __shared__ int item_ok;
    __shared__ int done_count;
    // Pixels that collect far more entries than the others (inputs that pile samples on a few pixels) get extra
    // lists in the slots of the workgroup that no pixel of the tile uses -- when there are such slots.  The first
    // round counts entries per slot (two 16-bit counters per word); after it the same array holds, per slot,
    // {first extra slot, number of extra slots (2^k - 1)} as 9 + 4 bits.
    __shared__ uint32_t slot_info[kTileThreads / 2];
    __shared__ uint32_t spare_next, round1_total;

    if (a.tile_px_log2 != kTilePxLog2) return;  // (uniform; the launcher derives both from head_dim)
    Work wk;
    if (!decode_block(t.map, blockIdx.x, a.bs, a.nh, t.items_per_bh, &wk)) return;
    if (t.batch_major == 0) {
        // item-major, batch-minor: the long-running items (coarse levels, numbered first) of every
        // batch element start at the beginning of the launch
        const int64_t r = (int64_t)wk.b * t.items_per_bh + wk.q_begin;
        wk.b = (int32_t)(r % a.bs);
        wk.q_begin = (int32_t)(r / a.bs);
    }
    if (wk.q_begin >= t.items_per_bh - t.extra) {  // (uniform: one of the workgroups behind the work items)
        add_levels_without_tiles<T>(a, wk.b, wk.h, wk.q_begin - (t.items_per_bh - t.extra), t.extra, lv_first);
        return;
    }
    // (the per-level values live in the entry storage, which is not written before the work item is known: the kernel's
    //  static LDS is 450 bytes short of the 80 KiB that let two workgroups share a CU)
    static_assert(sizeof(LevelInfo) <= sizeof(u32x4) * kTileEntCap, "the level values must fit one wavefront's entry storage");
    LevelInfo& lv_info = *reinterpret_cast<LevelInfo*>(&ent[0]);
    if ((int)threadIdx.x < a.nl) lv_info.fill(a, (int)threadIdx.x);
    if (threadIdx.x < kTileThreads / 2) slot_info[threadIdx.x] = 0;
    // an empty list points at the dummy entry of the wavefront that owns the pixel slot (slot s belongs to lane group
    // s / PPG, i.e. to wavefront s / (8 PPG); slots past the tile size are never used)
    heads[threadIdx.x] = ((threadIdx.x / (kLpp * PPG)) % NW * kTileEntCap + kDummyOfWave) * 16u;
    __syncthreads();
    if (threadIdx.x == 0) {
        item_ok = decode_tile_item(a, t, lv_info, wk.q_begin, &item_s, lv_first, lv_nt) ? 1 : 0;
        done_count = 0;
        spare_next = 0;
        round1_total = 0;
    }
    __syncthreads();
    if (!item_ok) return;  // uniform
    const TileItem it = item_s;

    const int hd = a.hd;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    // (float32: read as a scalar -- the compiler cannot know that tid >> 6 is the same in every lane of a wavefront, and
    //  whatever depends on it, the wavefront's runs and its entry storage, is otherwise a per-lane value steered by exec
    //  masks: 7 vector registers fewer and no spill, backward at the encoder shape 262.8 -> 260.6 us, BEVFormer shape 997 ->
    //  989.  The 16-bit instantiations keep the per-lane form: with the scalar one the compiler schedules the walk's row
    //  requests right in front of their use, encoder backward 270 -> 291 us)
    const int wave = sizeof(T) == 4 ? __builtin_amdgcn_readfirstlane(tid >> 6) : tid >> 6;
    const int npx = it.p1 - it.p0;
    // A tile much smaller than the workgroup is held in several copies (lists and registers),
    // each taking the samples of some queries; the copies meet in the image through atomics.
    const int npx_pad = (npx + PPG - 1) / PPG * PPG;
    int copies = 1;
    while (copies < 8 && 2 * copies * npx_pad <= kTilePx) copies *= 2;
    const bool owned = it.exclusive && copies == 1;  // plain stores are enough
    const int copies_log2 = __builtin_ctz(copies);
    const int nused = copies * npx_pad;              // slots that stand for a pixel of the tile
    const int nspare = kTilePx - nused;              // slots free for extra lists
    const bool can_split = nspare >= PPG;
    // (owned && !can_split is what tile_stored_directly() says of this tile)
    const bool direct_t = a.sparse != 0 && a.grad_value_t != nullptr && owned && !can_split;
    typedef uint16_t __attribute__((may_alias)) u16_alias;  // halves of LDS words that are also accessed whole
    u16_alias* slot_info16 = reinterpret_cast<u16_alias*>(slot_info);
    bool first_round = true;                         // (of the first channel pass)
    const uint32_t seg = wave * kTileEntCap;  // this wavefront's entry storage
    uint32_t* run_src = run_src_all + wave * kWave;
    uint32_t* run_pre = run_pre_all + wave * kWave;

    const T* gout = static_cast<const T*>(a.grad_out);
    const int64_t bh = (int64_t)wk.b * a.nh + wk.h;
    const uint32_t* tbl = a.tbl + bh * a.nwg * a.tbl_stride + it.tile;
    // the records of this (batch, head) as a bound buffer (the layout keeps them below 4 GiB)
    typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
    const __amdgpu_buffer_rsrc_t rres = make_rsrc(a.rec + bh * a.nwg * a.rec_cap * kRecDwords,
                                                  (uint32_t)a.nwg * (uint32_t)a.rec_cap * (kRecDwords * 4u));
    // runs of this wavefront: workgroups it.w0 + wave, + NW, + 2 NW, ... of the first kernel
    const int nruns = (it.w1 - it.w0 - wave + NW - 1) / NW;  // <= 0: none

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
    // (lists are linked by byte offsets into `ent`: the walk then needs no shift per entry)
    const uint32_t dummy = (seg + kDummyOfWave) * 16u;
    auto ent_at = [&](uint32_t off) -> u32x4& { return *reinterpret_cast<u32x4*>(reinterpret_cast<unsigned char*>(ent) + off); };
    if (lane == 0) ent_at(dummy) = u32x4{kInvalidCorner, 0u, 0u, dummy};

    // lane j of group g = tid / 8 keeps channels 32k + 4j .. 32k + 4j + 3 (k < NB) of the pixels g*PPG .. g*PPG + PPG - 1
    const int grp = tid / kLpp, j = tid % kLpp;

    for (int cb = 0; cb < hd; cb += CH) {
        float acc[kAccPx][CHL];
#pragma unroll
        for (int i = 0; i < kAccPx; ++i)
#pragma unroll
            for (int c = 0; c < CHL; ++c) acc[i][c] = 0.0f;
        // channels past head_dim re-read channel 0; their sums are never written out
        const int my_ch = cb + j * 4;  // (first channel of this lane in block 0; block k: + 32 k)
        uint32_t lane_off[NB];
#pragma unroll
        for (int k = 0; k < NB; ++k)
            lane_off[k] = ghead_off + (uint32_t)(my_ch + 32 * k < hd ? my_ch + 32 * k : 0) * (uint32_t)sizeof(T);
        const int nch = (hd - cb) < CH ? (hd - cb) : CH;

        // input state of this wavefront (uniform): next group of runs, records of the current
        // group, next unread record, and the batch fetched ahead
        int rg = 0, N = 0, i0 = 0;
        u32x4 ahead = {0u, 0u, 0u, 0u};
        auto fetch_ahead = [&](int first) {
            const int i = first + lane;
            if (i < N) {
                int r = 0;
#pragma unroll
                for (int step = kWave / 2; step > 0; step >>= 1)
                    if (run_pre[r + step] <= (uint32_t)i) r += step;
                // (one 12-byte load, non-temporal: the records are read once)
                const u32x3 v = __builtin_bit_cast(
                    u32x3, __builtin_amdgcn_raw_buffer_load_b96(rres, (run_src[r] + ((uint32_t)i - run_pre[r])) * (kRecDwords * 4u), 0, 2));
                // (run r of the current group comes from workgroup it.w0 + wave + NW * (rg - 64 + r) of the first kernel;
                //  its records name queries relative to that workgroup's first one)
                ahead = u32x4{v.x, v.y, v.z, (uint32_t)(it.w0 + wave + NW * (rg - kWave + r)) * (uint32_t)a.plan.tile_q};
            }
        };
        bool counted = false;    // this wavefront has reported the end of its work
        while (true) {
            // ---- stream records, append list entries ------------------------------------------
            int count = 0;  // entries of this wavefront in this round (uniform)
            fetch_ahead(i0);  // (again after a walk: the batch fetched ahead is not kept across it)
            while (true) {
                if (i0 >= N) {
                    if (rg >= nruns) break;  // input exhausted
                    // next group of up to 64 runs: one run per lane
                    const int r = rg + lane;
                    uint32_t len = 0, src = 0;
                    if (r < nruns) {
                        const int w = it.w0 + wave + NW * r;
                        const uint32_t* row = tbl + (size_t)w * a.tbl_stride;
                        const uint32_t s = row[0];
                        len = row[1] - s;
                        src = (uint32_t)w * (uint32_t)a.rec_cap + s;
                    }
                    uint32_t inc = len;
#pragma unroll
                    for (int d = 1; d < kWave; d <<= 1) {
                        const uint32_t o = __shfl_up(inc, d, kWave);
                        if (lane >= d) inc += o;
                    }
                    wave_lds_sync();
                    run_src[lane] = src;
                    run_pre[lane] = inc - len;
                    wave_lds_sync();
                    // (read as a scalar: the loop that N bounds is then steered by scalar branches; a lane shuffle would make
                    //  N, and with it the whole input state of the wavefront, a per-lane value)
                    N = (int)__builtin_amdgcn_readlane(inc, kWave - 1);
                    rg += kWave;
                    i0 = 0;
                    fetch_ahead(0);
                    continue;
                }
                if (count + 2 * kWave > (int)kDummyOfWave) break;  // entry storage full: next round
                const bool have = i0 + lane < N;
                const u32x4 rc = ahead;
                i0 += kWave;
                fetch_ahead(i0);
                // A record is the pair (pixel, pixel + 1).  A pair whose pixels belong to the same
                // lane group becomes ONE entry in the list of the left pixel (the grad_out row is
                // fetched once for both); otherwise each pixel gets an entry of its own -- unless the
                // groups keep sums for the pixel behind their last one (kOverlap), where every pair inside
                // the tile is one entry (backward at the encoder shape 276.9 -> 269.9 us, float16 286.7 ->
                // 277.6, BEVFormer shape 1024 -> 1000).  The right pixel of the last pixel of the tile
                // belongs to the next tile: added with atomics.
                int lst[2] = {-1, -1};
                float w0[2] = {0.f, 0.f}, w1[2] = {0.f, 0.f};
                uint32_t q = 0;
                bool spill = false;
                float wb = 0.f;
                // (a record that does not belong to this tile or names no query of the batch element is dropped:
                // the run table and the records are only as good as the workspace the caller hands over)
                const uint32_t rkey = rc.x, rq0 = rc.w;
                if (have && (rkey & (uint32_t)(kTilePx - 1)) < (uint32_t)npx && rq0 + (rkey >> kTilePxLog2) < (uint32_t)a.nq) {
                    const uint32_t ya = rc.y, za = rc.z;
                    q = rq0 + (rkey >> kTilePxLog2);
                    const int pl = (int)(rkey & (uint32_t)(kTilePx - 1));
                    const float wa = __builtin_bit_cast(float, ya);
                    wb = __builtin_bit_cast(float, za);
                    const int copy_off = (int)(q & (uint32_t)(copies - 1)) * npx_pad;
                    const bool in_r = pl + 1 < npx;
                    const bool pair = in_r && (kOverlap || (pl % PPG) != PPG - 1);
                    lst[0] = pl + copy_off;
                    w0[0] = wa;
                    w1[0] = pair ? wb : 0.0f;
                    if (!pair && wb != 0.0f) {
                        if (in_r) {
                            lst[1] = pl + 1 + copy_off;
                            w0[1] = wb;
                        } else {
                            spill = true;
                        }
                    }
                }
                if (can_split && !first_round) {
                    // entries of a pixel with extra lists are dealt to them by query; a pair entry that moves
                    // to an extra list leaves its right half to the right pixel's own lists
#pragma unroll
                    for (int k = 0; k < 2; ++k) {
                        if (lst[k] >= 0) {
                            const uint32_t o = slot_info16[lst[k]];
                            const uint32_t r = (q >> copies_log2) & (o >> 9);
                            if (r != 0) {
                                if (k == 0 && w1[0] != 0.0f) {
                                    lst[1] = lst[0] + 1;
                                    w0[1] = w1[0];
                                    w1[0] = 0.0f;
                                }
                                lst[k] = nused + (int)(o & 511u) + (int)r - 1;
                            }
                        }
                    }
                }
                const bool count_slots = can_split && first_round;
#pragma unroll
                for (int k = 0; k < 2; ++k) {
                    const bool push = lst[k] >= 0;
                    const uint64_t mask = __ballot(push);
                    if (mask) {
                        if (push) {
                            const uint32_t pos = seg + count +
                                                 __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                                                           __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
                            const uint32_t next = atomicExch(&heads[lst[k]], pos * 16u);
                            ent[pos] = u32x4{q * row_bytes, __builtin_bit_cast(uint32_t, w0[k]),
                                             __builtin_bit_cast(uint32_t, w1[k]), next};
                            if (count_slots) atomicAdd(&slot_info[lst[k] >> 1], (lst[k] & 1) ? 0x10000u : 1u);
                        }
                        count += __builtin_popcountll(mask);
                    }
                }
                // pairs that reach into the next tile: one at a time, the wavefront adds the row
                uint64_t smask = __ballot(spill);
                while (smask) {
                    const int src_lane = __builtin_ctzll(smask);
                    smask &= smask - 1;
                    const uint32_t sq = __builtin_amdgcn_readlane(q, src_lane);
                    const float sw = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(uint32_t, wb), src_lane));
                    for (int ch = lane; ch < nch; ch += kWave) {
                        const float g = to_f32(gout[((int64_t)wk.b * a.nq + sq) * row_pitch + (int64_t)wk.h * hd + cb + ch]);
                        unsafeAtomicAdd(gimg + (int64_t)it.p1 * row_pitch + (int64_t)wk.h * hd + cb + ch, sw * g);
                    }
                }
            }
            if (rg >= nruns && i0 >= N && !counted) {
                counted = true;
                if (lane == 0) atomicAdd(&done_count, 1);
            }
            if (can_split && first_round && lane == 0) atomicAdd(&round1_total, (uint32_t)count);
            __syncthreads();
            const bool all_done = done_count == NW;
            if (can_split && first_round) {
                // a slot with more than 1.5 times the average gets extra lists for the rounds to come
                // (every thread replaces the counter of its own slot; neighbours share a word, not a half)
                uint32_t o = 0;
                if (!all_done && tid < nused) {
                    const uint32_t c = slot_info16[tid];
                    const float limit = __builtin_fmaxf(1.5f * (float)round1_total / (float)nused, 4.0f);
                    const uint32_t m = (uint32_t)__builtin_ceilf((float)c / limit);
                    uint32_t extra = m <= 1 ? 0u : m <= 2 ? 1u : m <= 4 ? 3u : m <= 8 ? 7u : 15u;
                    if (extra != 0) {
                        const uint32_t base = atomicAdd(&spare_next, extra);
                        while (extra != 0 && base + extra > (uint32_t)nspare) extra >>= 1;
                        if (extra != 0) o = base | (extra << 9);
                    }
                }
                slot_info16[tid] = (uint16_t)o;
                first_round = false;
            }

            // ---- every group of 8 lanes walks the lists of its PPG pixels ----------------------
            // The lanes of a group read a 32-channel block of a grad_out row with ONE coalesced load (lane j:
            // channels 4j..4j+3 of the block): the memory pipeline's cost is per cache line touched by an instruction.
            // The loop body is branch-free: a list that has ended keeps "reading" the dummy entry.
            // kWalk lists are walked together, one entry of each per trip, and two trips are in flight.
            {
                auto fetch = [&](uint32_t& e, float (&g)[CHL], float& wa, float& wb) {
                    const u32x4 en = ent_at(e);
                    // (a bit cast applied directly to a vector element picks up element 0: copy first)
                    const uint32_t ya = en.y, za = en.z;
                    wa = __builtin_bit_cast(float, ya);
                    wb = __builtin_bit_cast(float, za);
#pragma unroll
                    for (int k = 0; k < NB; ++k) {
#pragma unroll
                        for (int c = 0; c < 4; c += VEC) {
                            float g1[VEC];
                            RowIO<T, VEC>::unpack(RowIO<T, VEC>::load_raw(gres, en.x + lane_off[k] + (uint32_t)(c * sizeof(T))), g1);
#pragma unroll
                            for (int v = 0; v < VEC; ++v) g[4 * k + c + v] = g1[v];
                        }
                    }
                    e = en.w;
                };
#pragma unroll
                for (int i = 0; i < PPG; i += kWalk) {
                    const int px = grp * PPG + i;
                    uint32_t e[kWalk];
#pragma unroll
                    for (int m = 0; m < kWalk; ++m) e[m] = heads[px + m];
                    if (j == 0) {  // same wavefront: ordered after the reads above
#pragma unroll
                        for (int m = 0; m < kWalk; ++m) heads[px + m] = dummy;
                    }
                    // two sets of rows in flight: the entries and rows of the next trip are requested before the
                    // rows of this trip are used, so that a long list costs its entries' LDS latency per trip
                    // and not the latency of a row load (reads past a list's end land on the dummy entry)
                    float gA[kWalk][CHL], uA[kWalk], vA[kWalk], gB[kWalk][CHL], uB[kWalk], vB[kWalk];
                    auto use = [&](float (&g)[kWalk][CHL], float (&u)[kWalk], float (&v)[kWalk]) {
#pragma unroll
                        for (int m = 0; m < kWalk; ++m) {
#pragma unroll
                            for (int c = 0; c < CHL; ++c) {
                                acc[i + m][c] = __builtin_fmaf(u[m], g[m][c], acc[i + m][c]);
                                if (i + m + 1 < kAccPx)
                                    acc[(i + m + 1) % kAccPx][c] = __builtin_fmaf(v[m], g[m][c], acc[(i + m + 1) % kAccPx][c]);
                            }
                        }
                    };
                    auto any_left = [&]() {
                        bool t = false;
#pragma unroll
                        for (int m = 0; m < kWalk; ++m) t |= e[m] != dummy;
                        return __ballot(t) != 0;
                    };
                    if (any_left()) {
#pragma unroll
                        for (int m = 0; m < kWalk; ++m) fetch(e[m], gA[m], uA[m], vA[m]);
                        while (true) {
                            // A holds a trip that has not been used; is there anything after it?
                            bool pending = any_left();
#pragma unroll
                            for (int m = 0; m < kWalk; ++m) fetch(e[m], gB[m], uB[m], vB[m]);
                            use(gA, uA, vA);
                            if (!pending) break;  // (B holds dummy entries only)
                            pending = any_left();
#pragma unroll
                            for (int m = 0; m < kWalk; ++m) fetch(e[m], gA[m], uA[m], vA[m]);
                            use(gB, uB, vB);
                            if (!pending) break;  // (A holds dummy entries only)
                        }
                    }
                }
            }
            __syncthreads();
            if (all_done) break;
        }

        if constexpr (kOverlap) {
            // what a group collected for the first pixel of the next group: inside a wavefront from lane to lane, from
            // the last group of a wavefront to the first of the next through the entry storage (free now; the last
            // group of the workgroup has nothing to hand over: a pair never starts on the last pixel of a tile)
            const int gw = lane / kLpp;
            if (gw == kWave / kLpp - 1)
                ent[seg + kCarryAt + j] = u32x4{__builtin_bit_cast(uint32_t, acc[PPG][0]), __builtin_bit_cast(uint32_t, acc[PPG][1]),
                                                __builtin_bit_cast(uint32_t, acc[PPG][2]), __builtin_bit_cast(uint32_t, acc[PPG][3])};
            __syncthreads();
            float cin[CHL];
#pragma unroll
            for (int c = 0; c < CHL; ++c) cin[c] = __shfl_up(acc[PPG][c], kLpp, kWave);
            if (gw == 0) {
                const u32x4 o = wave > 0 ? ent[seg - kTileEntCap + kCarryAt + j] : u32x4{0u, 0u, 0u, 0u};
                const uint32_t o0 = o.x, o1 = o.y, o2 = o.z, o3 = o.w;
                cin[0] = __builtin_bit_cast(float, o0);
                cin[1] = __builtin_bit_cast(float, o1);
                cin[2] = __builtin_bit_cast(float, o2);
                cin[3] = __builtin_bit_cast(float, o3);
            }
#pragma unroll
            for (int c = 0; c < CHL; ++c) acc[0][c] += cin[c];
        }
        // ---- write the CH channels of this tile -------------------------------------------
        // (address arithmetic derived from these opaque copies stays inside this section instead of
        // occupying registers during the rounds)
        int grp_w = grp, lane_w = lane;
        asm volatile("" : "+v"(grp_w), "+v"(lane_w));
        // extra lists were handed out: their slots add to their pixels' rows through the atomics below; the map
        // from extra slot to pixel goes into wavefront 0's entry storage, behind its transposition scratch
        const bool split = spare_next != 0;  // (uniform; written before the barrier that ended the first round)
        u16_alias* slot_px = reinterpret_cast<u16_alias*>(&ent[kSlotPxAt]);
        if (split) {
            slot_px[tid] = 0xFFFFu;
            __syncthreads();
            if (tid < nused) {
                const uint32_t o = slot_info16[tid];
                for (uint32_t r = 0; r < (o >> 9); ++r)
                    if ((o & 511u) + r < (uint32_t)nspare) slot_px[(o & 511u) + r] = (uint16_t)(tid - (tid / npx_pad) * npx_pad);
            }
            __syncthreads();
        }
        if (owned && !split && t.store_vec == 4) {
            // the lanes of a group hold a whole row of each of their pixels: 16-byte stores
#pragma unroll
            for (int kb = 0; kb < NB; ++kb) {
                const int ch_w = my_ch + 32 * kb;
                if (ch_w >= hd) continue;
#pragma unroll
                for (int i = 0; i < PPG; ++i) {
                    const int px = grp_w * PPG + i;
                    if (px < npx) {
                        f32x4* dst = reinterpret_cast<f32x4*>(gimg + (int64_t)(it.p0 + px) * row_pitch +
                                                              (int64_t)wk.h * hd + ch_w);
                        f32x4 v = {acc[i][4 * kb + 0], acc[i][4 * kb + 1], acc[i][4 * kb + 2], acc[i][4 * kb + 3]};
                        if (px == 0) {
                            // the first pixel of a tile also receives, through atomics, the right
                            // halves of pairs that start on the last pixel of the previous tile
                            float* d1 = reinterpret_cast<float*>(dst);
#pragma unroll
                            for (int c = 0; c < 4; ++c) unsafeAtomicAdd(d1 + c, v[c]);
                        } else if (sizeof(T) == 2 && direct_t) {
                            // 16-bit dtypes: nobody else adds to this row, so it goes to the caller's tensor at once
                            // (the fp32 image keeps only the rows that receive atomic additions)
                            typedef T t4 __attribute__((ext_vector_type(4)));
                            const t4 r = {from_f32<T>(v[0]), from_f32<T>(v[1]), from_f32<T>(v[2]), from_f32<T>(v[3])};
                            __builtin_nontemporal_store(r, reinterpret_cast<t4*>(static_cast<T*>(a.grad_value_t) +
                                                                                 (size_t)wk.b * (a.gbatch_bytes / 4) +
                                                                                 (int64_t)(it.p0 + px) * row_pitch +
                                                                                 (int64_t)wk.h * hd + ch_w));
                        } else {
                            if (t.accumulate) v += *dst;
                            // (non-temporal: nothing reads these rows again before the kernel ends; backward 283.8 ->
                            //  281.3 us at the encoder shape)
                            __builtin_nontemporal_store(v, dst);
                        }
                    }
                }
            }
        } else {
            // Rows shared with other workgroups (tiles split by query range) are added with
            // atomics, which the memory side carries out per 64-byte request: pass the registers
            // through LDS (the entry storage, free after the last round) so that consecutive
            // lanes hold consecutive floats of a row.  Four lane groups (4 PPG pixel slots, 1024 sums) at a time.
            typedef uint32_t __attribute__((may_alias)) u32_alias;
            static_assert(4 * PPG * CH * 4 <= kTileEntCap * 16, "transposition scratch must fit the entry storage");
            u32x4* tr4 = &ent[seg];
            const u32_alias* tr1 = reinterpret_cast<const u32_alias*>(tr4);
            for (int half = 0; half < 2; ++half) {
                wave_lds_sync();
                if (((lane_w / kLpp) >> 2) == half) {
                    const int gl = (lane_w / kLpp) & 3;
#pragma unroll
                    for (int i = 0; i < PPG; ++i)
#pragma unroll
                        for (int kb = 0; kb < NB; ++kb)
                            tr4[(gl * PPG + i) * (CH / 4) + 8 * kb + j] =
                                u32x4{__builtin_bit_cast(uint32_t, acc[i][4 * kb + 0]), __builtin_bit_cast(uint32_t, acc[i][4 * kb + 1]),
                                      __builtin_bit_cast(uint32_t, acc[i][4 * kb + 2]), __builtin_bit_cast(uint32_t, acc[i][4 * kb + 3])};
                }
                wave_lds_sync();
                const int px_base = wave * (kLpp * PPG) + half * (4 * PPG);
#pragma unroll 4
                for (int k = 0; k < 4 * PPG * CH / kWave; ++k) {
                    const int idx = k * kWave + lane_w;
                    const int pl = idx / CH, c = idx % CH;
                    const int vp = px_base + pl;             // pixel slot of the workgroup
                    int px = vp - (vp / npx_pad) * npx_pad;  // pixel of the tile (any copy)
                    if (vp >= nused) px = split ? (int)slot_px[vp - nused] : npx;  // (0xFFFF: slot without a pixel)
                    if (px < npx && c < nch) {
                        const float v = __builtin_bit_cast(float, (uint32_t)tr1[idx]);
                        float* dst = gimg + (int64_t)(it.p0 + px) * row_pitch + (int64_t)wk.h * hd + cb + c;
                        if (!owned || split || px == 0)
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
            if (lane == 0) ent_at(dummy) = u32x4{kInvalidCorner, 0u, 0u, dummy};
            __syncthreads();
        }
    }
}

template <typename T>
static hipError_t launch_t(const KArgs& a, const TileArgs& t, hipStream_t stream)
{
    // an octet of lanes reads a 32-channel block of a grad_out row, 4 channels per lane: one
    // load per lane when head_dim and the pointer alignment allow it; the wider forms (tiles of 256 and 128
    // pixels) are built for that case only
    const dim3 grid(t.grid), block(t.block);
    if (a.tile_px_log2 == 8 && t.vec >= 4)
        hipLaunchKernelGGL((msda_gradv_tiles_kernel<T, 8, 4>), grid, block, 0, stream, a, t);
    else if (a.tile_px_log2 == 7 && t.vec >= 4)
        hipLaunchKernelGGL((msda_gradv_tiles_kernel<T, 16, 4>), grid, block, 0, stream, a, t);
    else if (a.tile_px_log2 != kTilePxLog2Max)
        return hipErrorInvalidConfiguration;
    else if (t.vec >= 4)
        hipLaunchKernelGGL((msda_gradv_tiles_kernel<T, 4, 4>), grid, block, 0, stream, a, t);
    else if (t.vec == 2)
        hipLaunchKernelGGL((msda_gradv_tiles_kernel<T, 4, 2>), grid, block, 0, stream, a, t);
    else
        hipLaunchKernelGGL((msda_gradv_tiles_kernel<T, 4, 1>), grid, block, 0, stream, a, t);
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
