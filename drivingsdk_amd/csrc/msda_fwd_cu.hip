// Forward kernel of multi-scale deformable attention for gfx950 (MI355X), wave64 -- the form for large problems of
// the plain operator: one workgroup of 16 wavefronts per CU, the rows of the last (coarsest) levels of its
// (batch, head) resident in the CU's LDS, and no staging memory at all.
//
//   out[b,q,h,:] = sum_{l,p} attn[b,q,h,l,p] * bilinear(value_l[b,:,h,:], loc[b,q,h,l,p])
//
// Arithmetic: reference kernels/multi_scale_deformable_attn/op_kernel/msda.h:351-539 (pixel coordinates,
// validity, weights) and kernels/multi_scale_deformable_attn/op_kernel/arch35/multi_scale_deformable_attn.cpp:36-80
// (corner predicates, accumulation); the reference overlaps its gathers with compute through a helper core and
// double buffering (op_kernel/multi_scale_deformable_attn.cpp:116-189,300-347).  Here:
//
//   * The gather is bound by the vector-memory pipeline of a CU (64 bytes per clock); rows read from LDS travel
//     through the LDS pipeline (128 bytes per clock) beside it.  A workgroup therefore owns a whole CU: it copies
//     the rows of as many levels as fit, from the last one backwards, into up to 159 KiB of LDS once and then
//     works through all queries of its share of the (batch, head).
//   * Units (b,q,h) are laid out as in the general kernel: LPR lanes share a unit, each owning 16 bytes of a row,
//     so a corner row is one coalesced load and the sum stays in fp32 registers.
//   * The geometry of a unit's samples is computed by the unit's own lanes (lane c takes samples c, c + LPR, ..
//     of a chunk of 16) and handed to the other lanes of the unit through DPP lane permutations: a copy across
//     the quads of the unit per value and group of four samples, then a quad broadcast inside the instruction
//     that uses the value (the address addition, the multiply-add).  No LDS memory and no LDS bandwidth is spent
//     on it.
//   * Per level, everything a sample needs besides its location is precomputed once per workgroup in two small
//     LDS tables (shape as integers and floats; byte offset of the level's first row, pixel and row strides and
//     the offset that stands for "outside" -- for the value tensor or for the LDS copy, whichever holds the level).
//   * Locations, weights and results go through buffer descriptors with 32-bit offsets that advance by a constant
//     per step; lanes without work carry offsets that the hardware's range check turns into zeros / dropped stores.
//   * The locations and weights of a wavefront's next chunk are requested before the gather of the current one.
#include "msda_device.h"

namespace mxd {

namespace {

// DPP controls (gfx9 encoding)
constexpr int kDppRowShl = 0x100, kDppRowShr = 0x110;
// cache policy of the results: non-temporal stores, so that they do not push value rows out of the XCD's L2 (the same
// policy on the loads of locations and weights costs 20 %: measured)
constexpr int kStreamAux = 2;

template <int CTRL>
__device__ inline uint32_t dpp_all(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
template <int CTRL, int BANKS>
__device__ inline uint32_t dpp_banks(uint32_t old, uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp((int)old, (int)v, CTRL, 0xF, BANKS, false);
}

// The value that the lanes of quad QO of every unit hold, copied to the same positions of the unit's other quads
// (a unit is LPR = 4, 8 or 16 neighbouring lanes inside a DPP row of 16).
template <int LPR, int QO>
__device__ inline uint32_t unit_view(uint32_t x)
{
    if constexpr (LPR == 4) {
        return x;
    } else if constexpr (LPR == 8) {
        // quads 0/2 of a row are the first quads of their units, quads 1/3 the second ones
        if constexpr (QO == 0) return dpp_banks<kDppRowShr + 4, 0xA>(x, x);
        else return dpp_banks<kDppRowShl + 4, 0x5>(x, x);
    } else {
        uint32_t v = x;
        if constexpr (QO != 0) v = dpp_banks<kDppRowShl + 4 * QO, 0x1>(v, x);
        if constexpr (QO > 1) v = dpp_banks<kDppRowShl + 4 * (QO - 1), 0x2>(v, x);
        if constexpr (QO < 1) v = dpp_banks<kDppRowShr + 4 * (1 - QO), 0x2>(v, x);
        if constexpr (QO > 2) v = dpp_banks<kDppRowShl + 4 * (QO - 2), 0x4>(v, x);
        if constexpr (QO < 2) v = dpp_banks<kDppRowShr + 4 * (2 - QO), 0x4>(v, x);
        if constexpr (QO < 3) v = dpp_banks<kDppRowShr + 4 * (3 - QO), 0x8>(v, x);
        return v;
    }
}

// Lane J of every quad, to all four lanes of the quad.
template <int J>
__device__ inline uint32_t quad_bcast(uint32_t v)
{
    return dpp_all<J * 0x55>(v);
}

// acc += (weight held by lane J of the quad) * v.  For float rows the broadcast rides inside the multiply-add
// (the compiler folds a DPP move into an addition but not into this one).
template <int J>
__device__ inline void fma_quad_bcast(float& acc, uint32_t w_bits, float v)
{
    if constexpr (J == 0)
        asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(acc) : "v"(w_bits), "v"(v));
    else if constexpr (J == 1)
        asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(acc) : "v"(w_bits), "v"(v));
    else if constexpr (J == 2)
        asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[2,2,2,2] row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(acc) : "v"(w_bits), "v"(v));
    else
        asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[3,3,3,3] row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(acc) : "v"(w_bits), "v"(v));
}

// What a sample needs of its level: {H, W, H as float, W as float} and {byte offset of the level's first row,
// pixel stride, row stride, offset that reads as zeros} for wherever the level's rows are read from.
struct LevelTables {
    i32x4* shape;
    u32x4* place;
};

// Geometry of one sample: byte offsets of its four corner rows (the "outside" offset for corners that must not
// be touched) and the bilinear weights times the attention weight, as bit patterns.  Same arithmetic and the same
// order of operations as sample_geometry(); the pixel offset is formed with 24-bit multiplies (plan_forward_cu()
// refuses this kernel unless the key count and the distance between neighbouring pixels are below 2^23).
__device__ inline void cu_geometry(float x, float y, float aw, bool active, const i32x4 shape, const u32x4 place,
                                   uint32_t (&off)[4], uint32_t (&wgt)[4])
{
#pragma clang fp contract(off)  // the hi/lo split below must not be re-fused by the compiler
    const int32_t H = shape.x, W = shape.y;
    const int32_t hb = shape.z, wb = shape.w;
    const float Hf = __builtin_bit_cast(float, hb), Wf = __builtin_bit_cast(float, wb);
    const float w_im = __builtin_fmaf(x, Wf, -0.5f);
    const float h_im = __builtin_fmaf(y, Hf, -0.5f);
    const bool valid = active && (h_im > -1.0f) && (w_im > -1.0f) && (h_im < Hf) && (w_im < Wf);
    const float xh = x * Wf, xl = __builtin_fmaf(x, Wf, -xh);
    const float yh = y * Hf, yl = __builtin_fmaf(y, Hf, -yh);
    const float tx = xh - 0.5f, ty = yh - 0.5f;
    float fx = __builtin_floorf(tx), fy = __builtin_floorf(ty);
    float lw = (tx - fx) + xl;
    float lh = (ty - fy) + yl;
    if (lw < 0.0f) { fx -= 1.0f; lw += 1.0f; }
    if (lw >= 1.0f) { fx += 1.0f; lw -= 1.0f; }
    if (lh < 0.0f) { fy -= 1.0f; lh += 1.0f; }
    if (lh >= 1.0f) { fy += 1.0f; lh -= 1.0f; }
    // a sample that does not count: finite fractions, a cell whose four corners are all outside, weight zero
    lw = valid ? lw : 0.0f;
    lh = valid ? lh : 0.0f;
    fx = valid ? fx : -2.0f;
    fy = valid ? fy : -2.0f;
    const float a = valid ? aw : 0.0f;
    const int32_t x0 = (int32_t)fx, y0 = (int32_t)fy;
    const bool vx0 = (uint32_t)x0 < (uint32_t)W, vx1 = (uint32_t)(x0 + 1) < (uint32_t)W;
    const bool vy0 = (uint32_t)y0 < (uint32_t)H, vy1 = (uint32_t)(y0 + 1) < (uint32_t)H;
    const float hw = 1.0f - lw, hh = 1.0f - lh;
    const float w0 = (hh * hw) * a, w1 = (hh * lw) * a, w2 = (lh * hw) * a, w3 = (lh * lw) * a;
    wgt[0] = __builtin_bit_cast(uint32_t, w0);
    wgt[1] = __builtin_bit_cast(uint32_t, w1);
    wgt[2] = __builtin_bit_cast(uint32_t, w2);
    wgt[3] = __builtin_bit_cast(uint32_t, w3);
    const uint32_t place_x = place.x, pix_stride = place.y, row_stride = place.z, outside = place.w;
    const int32_t pix = __mul24(y0, W) + x0;
    const uint32_t o00 = place_x + (uint32_t)__mul24(pix, (int32_t)pix_stride);
    const uint32_t o01 = o00 + pix_stride, o10 = o00 + row_stride, o11 = o10 + pix_stride;
    off[0] = (vy0 && vx0) ? o00 : outside;
    off[1] = (vy0 && vx1) ? o01 : outside;
    off[2] = (vy1 && vx0) ? o10 : outside;
    off[3] = (vy1 && vx1) ? o11 : outside;
}

__device__ inline __amdgpu_buffer_rsrc_t vres_touch(const KArgs& a, const Work& wk)
{
    return make_rsrc(static_cast<const char*>(a.value) + (size_t)wk.b * a.batch_bytes, a.batch_bytes);
}

}  // namespace

// SRC = kSrcFused: `loc` holds sampling offsets, `attn` logits and `ref` reference points (x, y) per (query, level);
// location = reference + offset / (W, H), weight = softmax over the unit's samples (one chunk), formed by the unit's
// lanes from the values they hold, with the arithmetic of the general kernel's fused form.
template <typename T, int VEC, int LPR, int SRC>
__global__ __launch_bounds__(1024) void msda_fwd_cu_kernel(const KArgs a)
{
    static_assert(VEC * sizeof(T) == 16, "a lane owns 16 bytes of a row");
    static_assert(LPR == 4 || LPR == 8 || LPR == 16, "a unit lies inside a DPP row");
    static_assert(SRC == kSrcPlain || SRC == kSrcFused, "the plain operator and its fused form");
    constexpr bool FUSED = SRC == kSrcFused;
    constexpr int LPR_LOG2 = LPR == 4 ? 2 : LPR == 8 ? 3 : 4;
    constexpr int U = kWave / LPR;     // units per wavefront
    constexpr int KS = kChunk / LPR;   // samples of a chunk per lane
    constexpr uint32_t ES = (uint32_t)sizeof(T);
    typedef typename RowIO<T, VEC>::raw_t raw_t;
    extern __shared__ __align__(16) unsigned char smem[];
    LevelTables tab;
    tab.shape = reinterpret_cast<i32x4*>(smem);                                       // [kMaxLevels + 1]
    tab.place = reinterpret_cast<u32x4*>(smem + (kMaxLevels + 1) * sizeof(i32x4));    // [kMaxLevels + 1]
    unsigned char* cache = smem + kCuTableBytes;

    Work wk;
    if (!decode_block(a.plan, blockIdx.x, a.bs, a.nh, a.nq, &wk)) return;  // whole workgroup leaves

    // ---- this lane's place in the workgroup, and the locations and weights of its first chunk: requested first of
    // all, so that their way from memory (they are read once and never found in a cache) overlaps the level tables and
    // the cache fill (measured at the encoder shape: forward 78.9 -> 76.2 us in float32, 68.8 -> 67.0 us in float16)
    const uint32_t row_bytes = (uint32_t)a.hd * ES;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    const int g = lane / LPR;  // unit slot of this lane
    const int c = lane % LPR;  // position inside the row
    // wavefronts 4..7 and 12..15 of the workgroup (two of the four on every SIMD) work through their chunks from the LDS
    // groups on (see `pipelined`)
    const bool flipped = a.fwd_cu_flip != 0 && ((wave >> 2) & 1) != 0;

    const __amdgpu_buffer_rsrc_t vres =
        make_rsrc(static_cast<const char*>(a.value) + (size_t)wk.b * a.batch_bytes, a.batch_bytes);
    // locations, weights and results of this batch element (plan_forward_cu() refuses this kernel unless each -- and the
    // fused form's reference points -- stays below 2 GiB, so that the 32-bit offsets below cannot wrap)
    const uint32_t unit_loc_bytes = (uint32_t)a.S_full * 2u * ES;  // locations of one (query, head)
    const uint32_t loc_batch = (uint32_t)a.nq * a.nh * unit_loc_bytes;
    const __amdgpu_buffer_rsrc_t lres = make_rsrc(static_cast<const char*>(a.loc) + (size_t)wk.b * loc_batch, loc_batch);
    const __amdgpu_buffer_rsrc_t ares =
        make_rsrc(static_cast<const char*>(a.attn) + (size_t)wk.b * (loc_batch / 2), loc_batch / 2);
    const uint32_t out_batch = (uint32_t)a.nq * a.nh * row_bytes;
    const __amdgpu_buffer_rsrc_t ores = make_rsrc(static_cast<char*>(a.out) + (size_t)wk.b * out_batch, out_batch);
    // fused form: reference points (x, y) of this batch element, one pair per (query, level)
    const uint32_t ref_level_bytes = 2u * ES;
    const uint32_t ref_batch = FUSED ? (uint32_t)a.nq * a.nl * ref_level_bytes : 0u;
    const __amdgpu_buffer_rsrc_t rres =
        make_rsrc(FUSED ? static_cast<const char*>(a.ref) + (size_t)wk.b * ref_batch : static_cast<const char*>(a.loc), ref_batch);

    // lanes past the end of the row read channel 0 and never store
    const bool chan_ok = c * VEC < a.hd;
    const uint32_t lds_choff = chan_ok ? (uint32_t)c * 16u : 0u;
    const uint32_t choff = (uint32_t)wk.h * row_bytes + lds_choff;

    // steps of this wavefront: chunks of 16 samples of its groups of U queries (groups wave, wave + nwaves, ..)
    const int ngroups = (wk.q_end - wk.q_begin + U - 1) / U;
    const int my_groups = ngroups > wave ? (ngroups - wave + nwaves - 1) / nwaves : 0;
    const int chunks = (a.S + kChunk - 1) / kChunk;
    // this lane's unit in the wavefront's first group, and what a step adds
    int q_lane = wk.q_begin + wave * U + g;
    const int q_step = nwaves * U;
    uint32_t loc_off = ((uint32_t)q_lane * a.nh + wk.h) * unit_loc_bytes + (uint32_t)c * 2u * ES;  // sample c of chunk 0
    const uint32_t loc_group_step = (uint32_t)q_step * a.nh * unit_loc_bytes;
    uint32_t out_off = ((uint32_t)q_lane * a.nh + wk.h) * row_bytes + lds_choff;
    const uint32_t out_group_step = (uint32_t)q_step * a.nh * row_bytes;
    uint32_t ref_off = (uint32_t)q_lane * a.nl * ref_level_bytes;  // reference points of this lane's unit
    const uint32_t ref_group_step = (uint32_t)q_step * a.nl * ref_level_bytes;

    // What this lane reads for chunk `ch` of its unit: the location and the weight of its KS samples of the chunk
    // (locations of the unit at byte offset `lo` of the batch element).  16-bit pairs and weights stay packed.
    struct Raw {
        uint32_t x, y, aw;  // float32: bit patterns; 16-bit types: x = the (x, y) pair, aw = the weight in the low half
        uint32_t rx, ry;    // fused form: the reference point of the sample's level, laid out like (x, y)
    };
    auto fetch = [&](uint32_t lo, uint32_t ro, int ch, Raw (&r)[KS]) {
#pragma unroll
        for (int k = 0; k < KS; ++k) {
            const uint32_t o = lo + (uint32_t)(ch * kChunk + k * LPR) * 2u * ES;
            if constexpr (FUSED) {
                const int s = ch * kChunk + k * LPR + c;
                const int lraw = (int)(((uint32_t)s * a.np_magic) >> 20);
                // (samples past the end of the list: any level's point, their weight is zero)
                const uint32_t po = ro + (uint32_t)(lraw < a.nl ? lraw : 0) * ref_level_bytes;
                if constexpr (sizeof(T) == 4) {
                    const u32x2 p = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rres, po, 0, 0));
                    r[k].rx = p.x;
                    r[k].ry = p.y;
                } else {
                    r[k].rx = __builtin_bit_cast(uint32_t, __builtin_amdgcn_raw_buffer_load_b32(rres, po, 0, 0));
                    r[k].ry = 0u;
                }
            }
            if constexpr (sizeof(T) == 4) {
                const u32x2 xy = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(lres, o, 0, 0));
                r[k].x = xy.x;
                r[k].y = xy.y;
                r[k].aw = __builtin_bit_cast(uint32_t, __builtin_amdgcn_raw_buffer_load_b32(ares, o >> 1, 0, 0));
            } else {
                r[k].x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_raw_buffer_load_b32(lres, o, 0, 0));
                r[k].y = 0u;
                r[k].aw = (uint32_t)__builtin_bit_cast(uint16_t, __builtin_amdgcn_raw_buffer_load_b16(ares, o >> 1, 0, 0));
            }
        }
    };

    Raw nxt[KS];
    if (my_groups > 0) fetch(loc_off, ref_off, 0, nxt);

    for (int i = threadIdx.x; i < a.nl; i += blockDim.x) {
        i32x4 lv = load_level(a, i);
        tab.place[i] = u32x4{(uint32_t)lv.z, 0u, 0u, 0u};  // (level_start_index, until the cache is laid out)
        const float hf = (float)lv.x, wf = (float)lv.y;
        lv.z = __builtin_bit_cast(int32_t, hf);
        lv.w = __builtin_bit_cast(int32_t, wf);
        tab.shape[i] = lv;
    }
    __syncthreads();


    // ---- level cache: rows [c_base, nk) of this (batch, head), i.e. levels c_first .. nl-1 ----------------------
    // Levels are taken from the last one backwards while level_start_index is ascending, the level lies inside the
    // value tensor and the rows from the level's start to the end of value fit; one more row of zeros stands for
    // corners outside the image.
    int c_first = a.nl, c_base = 0, c_rows = 0;
    {
        const int cap_rows = (int)(a.lds_cache_bytes / row_bytes) - 1;
        int next_b0 = a.nk;
        for (int l = a.nl - 1; l >= 0; --l) {
            const int b0 = (int)tab.place[l].x;
            const int64_t px = (int64_t)tab.shape[l].x * tab.shape[l].y;
            if (b0 < 0 || b0 >= a.nk || a.nk - b0 > cap_rows || b0 > next_b0 || tab.shape[l].x <= 0 ||
                tab.shape[l].y <= 0 || b0 + px > a.nk)
                break;
            c_first = l;
            c_base = b0;
            next_b0 = b0;
        }
        c_rows = c_first < a.nl ? a.nk - c_base : 0;
    }
    const uint32_t zero_row = (uint32_t)c_rows * row_bytes;
    __syncthreads();  // (every thread has read the level starts)
    if (threadIdx.x == 0) {
        // the empty level that samples past the end of a unit's list are given: they are gathered from LDS
        tab.shape[a.nl] = i32x4{0, 0, 0, 0};
        tab.place[a.nl] = u32x4{0u, 0u, 0u, zero_row};
    }
    for (int i = threadIdx.x; i < a.nl; i += blockDim.x) {
        const int32_t base = (int32_t)tab.place[i].x, W = tab.shape[i].y;
        if (i >= c_first)
            tab.place[i] = u32x4{(uint32_t)(base - c_base) * row_bytes, row_bytes, (uint32_t)W * row_bytes, zero_row};
        else
            tab.place[i] = u32x4{(uint32_t)base * a.pitch_bytes, a.pitch_bytes, (uint32_t)W * a.pitch_bytes, kInvalidCorner};
    }
    {
        // The rows that stay in memory, [0, c_base) of this (batch, head), are gathered out of the XCD's L2; the first
        // request for a row would otherwise travel to memory from inside the gather, where its latency holds up the
        // wavefront's later requests (loads return in order).  The workgroups of the (batch, head) -- they run on one
        // XCD -- share the rows between them and request one word of each 128 bytes here, ahead of the cache fill,
        // so that both waits overlap.
        const int wg = wk.q_begin / a.plan.tile_q;
        const int64_t lines = ((int64_t)c_base * row_bytes + 127) / 128;  // (rows are packed into lines when shorter)
        const int64_t l0 = lines * wg / a.plan.ntiles, l1 = lines * (wg + 1) / a.plan.ntiles;
        const int rows_per_line = row_bytes >= 128 ? 1 : (int)(128 / row_bytes);
        const int lines_per_row = row_bytes >= 128 ? (int)((row_bytes + 127) / 128) : 1;
        uint32_t seen = 0;
        for (int64_t i = l0 + threadIdx.x; i < l1; i += blockDim.x) {
            const int64_t row = row_bytes >= 128 ? i / lines_per_row : i * rows_per_line;
            const int64_t within = row_bytes >= 128 ? (i % lines_per_row) * 128 : 0;
            if (row < c_base)
                seen |= __builtin_bit_cast(uint32_t, __builtin_amdgcn_raw_buffer_load_b32(
                                vres_touch(a, wk), (uint32_t)(row * a.pitch_bytes + wk.h * row_bytes + within), 0, 0));
        }
        asm volatile("" ::"v"(seen));  // (the values are not used; the requests are what matters)
        const int pieces = (int)(row_bytes / 16), total = c_rows * pieces;
        const char* src = static_cast<const char*>(a.value) + (size_t)wk.b * a.batch_bytes +
                          (size_t)c_base * a.pitch_bytes + (size_t)wk.h * row_bytes;
        // twelve pieces per thread and trip, all requested before the first is stored: the fill is a matter of latency
        // (rows that no workgroup has touched yet come from memory), and a CU's LDS takes ten pieces per thread
        constexpr int kFillAhead = 12;
        // i / pieces for i < 2^16 and pieces > 1 (one piece per row: the row is the piece)
        const uint32_t pieces_magic = pieces > 1 ? (uint32_t)((0x100000000ull + pieces - 1) / pieces) : 0u;
        for (int i0 = threadIdx.x; i0 < total; i0 += kFillAhead * (int)blockDim.x) {
            u32x4 piece[kFillAhead];
#pragma unroll
            for (int j = 0; j < kFillAhead; ++j) {
                const int i = i0 + j * (int)blockDim.x;
                const int row = pieces > 1 ? (int)__umulhi((uint32_t)i, pieces_magic) : i, col = i - row * pieces;
                if (i < total) piece[j] = *reinterpret_cast<const u32x4*>(src + (size_t)row * a.pitch_bytes + col * 16);
            }
#pragma unroll
            for (int j = 0; j < kFillAhead; ++j) {
                const int i = i0 + j * (int)blockDim.x;
                if (i < total) *reinterpret_cast<u32x4*>(cache + (size_t)i * 16) = piece[j];
            }
        }
        for (int i = threadIdx.x; i < pieces; i += blockDim.x)
            *reinterpret_cast<u32x4*>(cache + (size_t)zero_row + i * 16) = u32x4{0u, 0u, 0u, 0u};
    }
    __syncthreads();
    const int s_cached = c_first * a.np;  // samples are level-major: those of the cached levels are the tail

    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;

    for (int gi = 0; gi < my_groups; ++gi) {
        for (int ch = 0; ch < chunks; ++ch) {
            // ---- one chunk: geometry, gather, weighted sum ------------------------------------------------------
            // The rows of a sample are requested kRing - 1 samples ahead of their use (a ring of kRing samples' rows in
            // registers), so that a wavefront always has requests in flight while it does arithmetic.  A group of four
            // samples is held by one quad of each unit: its values are copied to the unit's other quads (views) when the
            // group's first rows are requested; the geometry of a lane's K-th sample of the chunk is computed right
            // before the first group that needs it, between requests and their use.
            // (Samples past the end of a unit's list carry zero weights and the offset of the row of zeros.)
            constexpr int kRing = 3;
            const int c0 = ch * kChunk;
            uint32_t off[4], wgt[4];       // this lane's sample of the groups being requested
            uint32_t vo[2][4], vw[2][4];   // views of the group being requested / used, by group parity
            raw_t raw[kRing][4];           // rows of kRing samples, by sample index modulo kRing
            auto geometry = [&](auto k_c) {
                constexpr int K = decltype(k_c)::value;
                const int s = c0 + K * LPR + c;
                const bool active = q_lane < wk.q_end && s < a.S;
                // (samples past the end of the list take the empty level behind the last one: every corner outside)
                const int lraw = (int)(((uint32_t)s * a.np_magic) >> 20);
                const int l = lraw < a.nl ? lraw : a.nl;
                float x, y, aw, rx = 0.f, ry = 0.f;
                if constexpr (sizeof(T) == 4) {
                    x = __builtin_bit_cast(float, nxt[K].x);
                    y = __builtin_bit_cast(float, nxt[K].y);
                    aw = __builtin_bit_cast(float, nxt[K].aw);
                    if constexpr (FUSED) {
                        rx = __builtin_bit_cast(float, nxt[K].rx);
                        ry = __builtin_bit_cast(float, nxt[K].ry);
                    }
                } else {
                    typedef T t2 __attribute__((ext_vector_type(2)));
                    const t2 xy = __builtin_bit_cast(t2, nxt[K].x);
                    x = to_f32<T>(xy[0]);
                    y = to_f32<T>(xy[1]);
                    // (the fused form's weights are float32 by now: see the softmax below)
                    if constexpr (FUSED) aw = __builtin_bit_cast(float, nxt[K].aw);
                    else aw = to_f32<T>(__builtin_bit_cast(T, (uint16_t)nxt[K].aw));
                    if constexpr (FUSED) {
                        const t2 rp = __builtin_bit_cast(t2, nxt[K].rx);
                        rx = to_f32<T>(rp[0]);
                        ry = to_f32<T>(rp[1]);
                    }
                }
                const i32x4 shape = tab.shape[l];
                if constexpr (FUSED) {
                    // location = reference + offset / (W, H): every operation rounded on its own, as fused_location() does
                    // (the backward derives the same locations and must land on the same pixels)
#pragma clang fp contract(off)
                    // (a bit cast applied directly to a vector element picks up element 0: copy first)
                    const int32_t hb = shape.z, wb = shape.w;
                    const float Hf = __builtin_bit_cast(float, hb), Wf = __builtin_bit_cast(float, wb);
                    const float dx = x / Wf, dy = y / Hf;
                    x = rx + dx;
                    y = ry + dy;
                }
                cu_geometry(x, y, aw, active, shape, tab.place[l], off, wgt);
            };
            auto views = [&](auto g_c) {
                constexpr int G = decltype(g_c)::value, K = (4 * G) / LPR, QO = ((4 * G) % LPR) / 4;
                if constexpr ((4 * G) % LPR == 0) geometry(std::integral_constant<int, K>{});
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    vo[G & 1][j] = unit_view<LPR, QO>(off[j]);
                    vw[G & 1][j] = unit_view<LPR, QO>(wgt[j]);
                }
            };
            // (I: the sample of the chunk; R: its place in the ring of rows)
            auto load_sample = [&](auto i_c, auto r_c, auto lds_c) {
                constexpr int I = decltype(i_c)::value, R = decltype(r_c)::value, G = I / 4, J = I % 4;
                if constexpr (decltype(lds_c)::value) {
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        raw[R][k] = *reinterpret_cast<const raw_t*>(cache + (quad_bcast<J>(vo[G & 1][k]) + lds_choff));
                } else {
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        raw[R][k] = RowIO<T, VEC>::load_raw(vres, quad_bcast<J>(vo[G & 1][k]) + choff);
                }
            };
            auto use_sample = [&](auto i_c, auto r_c) {
                constexpr int I = decltype(i_c)::value, R = decltype(r_c)::value, G = I / 4, J = I % 4;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    float v[VEC];
                    RowIO<T, VEC>::unpack(raw[R][k], v);
                    if constexpr (sizeof(T) == 4) {
#pragma unroll
                        for (int e = 0; e < VEC; ++e) fma_quad_bcast<J>(acc[e], vw[G & 1][k], v[e]);
                    } else {
                        const float w = __builtin_bit_cast(float, quad_bcast<J>(vw[G & 1][k]));
#pragma unroll
                        for (int e = 0; e < VEC; ++e) acc[e] = __builtin_fmaf(w, v[e], acc[e]);
                    }
                }
            };
            // the next chunk's locations and weights: requested once this chunk's are used up, behind the chunk's last
            // rows from memory where that is later (past the wavefront's last group the offsets lie beyond the
            // workgroup's queries: nothing of it is used, and whatever lies beyond the tensor reads as zeros)
            auto fetch_next = [&]() {
                const bool wrap = ch + 1 >= chunks;
                fetch(wrap ? loc_off + loc_group_step : loc_off, wrap ? ref_off + ref_group_step : ref_off, wrap ? 0 : ch + 1, nxt);
            };
            constexpr int kLastGeometry = kChunk - LPR;  // the sample whose request computes the lane's last geometry
            // NM4 groups of four samples come from memory, the other 4 - NM4 from LDS.  FLIP: the chunk is worked through
            // from its first LDS group on, round to its memory groups (step P of the chunk takes sample (P + 4 NM4) mod
            // 16).  Half of a CU's wavefronts run flipped, two on every SIMD, so that at any moment about half of them
            // gather from memory -- the vector-memory pipeline is what they wait for -- while the other half gather
            // from LDS and keep the vector ALU busy, instead of all sixteen meeting in front of the same unit phase
            // after phase.  (The sum of a flipped wavefront's unit is formed in that order as well.)
            auto pipelined = [&](auto nm4_c, auto flip_c) {
                constexpr int NM4 = decltype(nm4_c)::value;
                constexpr bool FLIP = decltype(flip_c)::value;
                constexpr int kRot = FLIP ? 4 * NM4 : 0;  // the sample that step 0 takes
                static_assert(kRot % LPR == 0, "a flipped chunk starts with the first group of a lane's sample");
                constexpr int kLastMem = 4 * NM4 - 1;
                // after this step's request (flipped: the memory groups end the chunk, and the next chunk's first
                // geometry should not find its locations still on their way)
                constexpr int kFetchAfter = FLIP ? kLastGeometry : (kLastMem > kLastGeometry ? kLastMem : kLastGeometry);
                auto load = [&](auto p_c) {
                    constexpr int P = decltype(p_c)::value, I = (P + kRot) % kChunk;
                    if constexpr (I % 4 == 0) views(std::integral_constant<int, I / 4>{});
                    load_sample(std::integral_constant<int, I>{}, std::integral_constant<int, P % kRing>{},
                                std::integral_constant<bool, (I / 4 >= NM4)>{});
                    if constexpr (P == kFetchAfter) fetch_next();
                };
                auto step = [&](auto p_c) {
                    constexpr int P = decltype(p_c)::value, I = (P + kRot) % kChunk;
                    if constexpr (P + kRing - 1 < kChunk) load(std::integral_constant<int, P + kRing - 1>{});
                    __builtin_amdgcn_sched_barrier(0);  // requests go out before the rows of an earlier sample are waited for
                    use_sample(std::integral_constant<int, I>{}, std::integral_constant<int, P % kRing>{});
                    __builtin_amdgcn_sched_barrier(0);
                };
                load(std::integral_constant<int, 0>{});
                if constexpr (kRing > 2) load(std::integral_constant<int, 1>{});
                step(std::integral_constant<int, 0>{});
                step(std::integral_constant<int, 1>{});
                step(std::integral_constant<int, 2>{});
                step(std::integral_constant<int, 3>{});
                step(std::integral_constant<int, 4>{});
                step(std::integral_constant<int, 5>{});
                step(std::integral_constant<int, 6>{});
                step(std::integral_constant<int, 7>{});
                step(std::integral_constant<int, 8>{});
                step(std::integral_constant<int, 9>{});
                step(std::integral_constant<int, 10>{});
                step(std::integral_constant<int, 11>{});
                step(std::integral_constant<int, 12>{});
                step(std::integral_constant<int, 13>{});
                step(std::integral_constant<int, 14>{});
                step(std::integral_constant<int, 15>{});
            };
            // any other split between memory and LDS (points per level not a multiple of four): sample by sample, the
            // sample's values fetched from the lane that holds them with a run-time lane index
            auto serial = [&]() {
                auto samples_of = [&](auto k_c) {
                    constexpr int K = decltype(k_c)::value;
                    geometry(k_c);
                    if constexpr (K == KS - 1) fetch_next();
#pragma unroll 1
                    for (int cc = 0; cc < LPR; ++cc) {
                        const int s = c0 + K * LPR + cc;
                        if (s >= a.S) break;
                        const int src = ((lane & ~(LPR - 1)) | cc) * 4;
                        uint32_t o[4], w[4];
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            o[k] = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)off[k]);
                            w[k] = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)wgt[k]);
                        }
                        raw_t r[4];
                        if (s >= s_cached) {
#pragma unroll
                            for (int k = 0; k < 4; ++k) r[k] = *reinterpret_cast<const raw_t*>(cache + (o[k] + lds_choff));
                        } else {
#pragma unroll
                            for (int k = 0; k < 4; ++k) r[k] = RowIO<T, VEC>::load_raw(vres, o[k] + choff);
                        }
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            float v[VEC];
                            RowIO<T, VEC>::unpack(r[k], v);
                            const float wf = __builtin_bit_cast(float, w[k]);
#pragma unroll
                            for (int e = 0; e < VEC; ++e) acc[e] = __builtin_fmaf(wf, v[e], acc[e]);
                        }
                    }
                };
                samples_of(std::integral_constant<int, 0>{});
                if constexpr (KS >= 2) samples_of(std::integral_constant<int, 1>{});
                if constexpr (KS >= 4) {
                    samples_of(std::integral_constant<int, 2>{});
                    samples_of(std::integral_constant<int, 3>{});
                }
            };
            if constexpr (FUSED) {
                // softmax over the unit's samples (the launcher takes this form for units of one chunk only): every
                // lane holds KS logits; maximum and sum of exponentials go round the unit's lanes with DPP, and the
                // weights replace the logits as float32 bit patterns
                float lg[KS], m = -__builtin_inff();
                bool act[KS];
#pragma unroll
                for (int k = 0; k < KS; ++k) {
                    act[k] = q_lane < wk.q_end && c0 + k * LPR + c < a.S;
                    if constexpr (sizeof(T) == 4) lg[k] = __builtin_bit_cast(float, nxt[k].aw);
                    else lg[k] = to_f32<T>(__builtin_bit_cast(T, (uint16_t)nxt[k].aw));
                    if (act[k]) m = __builtin_fmaxf(m, lg[k]);
                }
                m = group_max<LPR_LOG2>(m);
                float e[KS], sum = 0.0f;
#pragma unroll
                for (int k = 0; k < KS; ++k) {
                    e[k] = act[k] ? expf(lg[k] - m) : 0.0f;
                    sum += e[k];
                }
                sum = group_sum<LPR_LOG2>(sum);
#pragma unroll
                for (int k = 0; k < KS; ++k) nxt[k].aw = __builtin_bit_cast(uint32_t, act[k] ? e[k] / sum : 0.0f);
            }
            int from_mem = s_cached - c0;  // samples of the chunk that come from memory
            from_mem = from_mem < 0 ? 0 : (from_mem > kChunk ? kChunk : from_mem);
            // (a chunk can be flipped when its first LDS group is the first group of a lane's sample)
            auto either = [&](auto nm4_c) {
                constexpr int NM4 = decltype(nm4_c)::value;
                if constexpr ((4 * NM4) % LPR == 0 && NM4 > 0 && NM4 < 4) {
                    if (flipped) {
                        pipelined(nm4_c, std::true_type{});
                        return;
                    }
                }
                pipelined(nm4_c, std::false_type{});
            };
            switch (from_mem) {
                case 0: either(std::integral_constant<int, 0>{}); break;
                case 4: either(std::integral_constant<int, 1>{}); break;
                case 8: either(std::integral_constant<int, 2>{}); break;
                case 12: either(std::integral_constant<int, 3>{}); break;
                case 16: either(std::integral_constant<int, 4>{}); break;
                default: serial(); break;
            }
        }

        // (non-temporal: results are not read again by this kernel and should not push value rows out of L2;
        //  lanes without a result carry an offset that the range check drops)
        {
            typedef T vec_t __attribute__((ext_vector_type(VEC)));
            vec_t t;
#pragma unroll
            for (int i = 0; i < VEC; ++i) t[i] = from_f32<T>(acc[i]);
            const uint32_t o = (q_lane < wk.q_end && chan_ok) ? out_off : 0xFFFFFFFFu;
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, t), ores, o, 0, kStreamAux);
        }
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;
        q_lane += q_step;
        loc_off += loc_group_step;
        out_off += out_group_step;
        ref_off += ref_group_step;
    }
}

template <typename T, int SRC>
static hipError_t launch_cu_t(const KArgs& a, hipStream_t stream)
{
    constexpr int VEC = 16 / (int)sizeof(T);
    const dim3 grid(a.plan.grid), block(a.plan.block);
    switch (a.plan.lanes_per_row) {
        case 4: hipLaunchKernelGGL((msda_fwd_cu_kernel<T, VEC, 4, SRC>), grid, block, a.plan.lds_bytes, stream, a); break;
        case 8: hipLaunchKernelGGL((msda_fwd_cu_kernel<T, VEC, 8, SRC>), grid, block, a.plan.lds_bytes, stream, a); break;
        case 16: hipLaunchKernelGGL((msda_fwd_cu_kernel<T, VEC, 16, SRC>), grid, block, a.plan.lds_bytes, stream, a); break;
        default: return hipErrorInvalidConfiguration;
    }
    return hipGetLastError();
}

template <typename T, int SRC>
static hipError_t raise_lds_t()
{
    constexpr int VEC = 16 / (int)sizeof(T);
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&msda_fwd_cu_kernel<T, VEC, 4, SRC>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kCuLdsBytes);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&msda_fwd_cu_kernel<T, VEC, 8, SRC>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kCuLdsBytes);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&msda_fwd_cu_kernel<T, VEC, 16, SRC>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kCuLdsBytes);
    return e;
}

// Opt-in to more than 64 KiB of dynamic LDS for every instantiation, on the current device.
hipError_t raise_forward_cu_lds()
{
    hipError_t e = raise_lds_t<float, kSrcPlain>();
    if (e == hipSuccess) e = raise_lds_t<f16_t, kSrcPlain>();
    if (e == hipSuccess) e = raise_lds_t<bf16_t, kSrcPlain>();
    if (e == hipSuccess) e = raise_lds_t<float, kSrcFused>();
    if (e == hipSuccess) e = raise_lds_t<f16_t, kSrcFused>();
    if (e == hipSuccess) e = raise_lds_t<bf16_t, kSrcFused>();
    return e;
}

// (the fused form when a.ref is set: reference points (x, y), units of one chunk)
hipError_t launch_forward_cu(int dtype, const KArgs& a, hipStream_t stream)
{
    const bool fused = a.ref != nullptr;
    switch (dtype) {
        case MXD_DTYPE_F32: return fused ? launch_cu_t<float, kSrcFused>(a, stream) : launch_cu_t<float, kSrcPlain>(a, stream);
        case MXD_DTYPE_F16: return fused ? launch_cu_t<f16_t, kSrcFused>(a, stream) : launch_cu_t<f16_t, kSrcPlain>(a, stream);
        case MXD_DTYPE_BF16: return fused ? launch_cu_t<bf16_t, kSrcFused>(a, stream) : launch_cu_t<bf16_t, kSrcPlain>(a, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace mxd
