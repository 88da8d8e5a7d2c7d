// Backward kernel of multi-scale deformable attention for gfx950 (MI355X), wave64 (instantiated per dtype by
// msda_bwd_f32.hip, msda_bwd_f16.hip and msda_bwd_bf16.hip).
//
// For every sample (b,q,h,l,p) with g = grad_out[b,q,h,:]:
//   grad_value[row_c] += w_c * attn * g                  (4 corner rows; left to the tile pass, or fp32 atomics)
//   d_c = dot(value[row_c], g)
//   grad_attn = sum_c w_c d_c
//   grad_x = W attn (hh (d2-d1) + lh (d4-d3)),  grad_y = H attn (hw (d3-d1) + lw (d4-d2))
// Arithmetic: reference kernels/multi_scale_deformable_attn/op_kernel/multi_scale_deformable_attn_grad.cpp:208-249
// and kernels/multi_scale_deformable_attn/op_kernel/arch35/multi_scale_deformable_attn_grad.cpp:16-145.
//
// Structure (same unit/lane layout and LDS staging as the forward kernel):
//   * geometry per lane -> LDS strip (row offsets, w_c*attn);
//   * per staged sample the lanes of a unit fetch the 4 corner rows with one buffer load
//     each and form partial dots with the register-resident grad_out row; the partial dots
//     are summed across the unit's lanes with DPP and parked in LDS;
//   * (SCATTER = true only) the scatter then walks the staged samples again with a row-contiguous lane
//     layout and issues buffer atomics (out-of-image corners carry an out-of-range offset: the load
//     yields 0, the atomic is dropped by the hardware range check);
//   * the geometry lanes turn the reduced dots into grad_attn / grad_loc and store them
//     coalesced.
//
// SCATTER = false leaves grad_value to the tile-ownership pass (msda_bwd_tiles.hip) and hands it
// the samples already sorted by tile: a sample is two "pair records" {pixel, query, weight of
// that pixel, weight of the pixel to its right} (upper and lower corners).  The workgroup first
// counts its records per tile in LDS (one geometry sweep over its sampling locations), turns
// the counts into run starts inside its own slab of the record array, publishes them as its
// row of the run table, and then -- where it computes grad_loc anyway -- drops every record
// at the next free position of its tile's run (one LDS integer atomic per record).  Records of a query
// that start on the same pixel are merged before they are counted and before they are written.  For the
// plain operator and the fused form the counting sweep already stages the first chunk of samples of the
// workgroup's first iteration for the gather, so those samples' geometry is derived once.  Its workgroups
// also zero-fill the fp32 image of grad_value between them, which the tile pass is the first to touch.
#pragma once
#include <type_traits>

#include "msda_device.h"

namespace mxd {

// RECBUF: workgroups that make several passes collect their slab of records in LDS (see `recbuf` below); an
// instantiation of its own, for the plain operator and its fused form, because the extra paths cost the others scalar
// registers (spilled ones travel through vector lanes) that they have no use for.
// FIXED != 0: the launch geometry of the common cases as compile-time constants -- rows read by 8 lanes (8 units per
// wavefront), one iteration of one chunk, the plain operator's tile form, with a unit per query (1: up to 16 samples per
// query) or two (2: up to 32): the paths for anything else and the scalar registers that steer them fall away (57
// vector registers instead of 96 and no spilled scalar ones; encoder shape 281.7 -> 276.3 us, float16 294.0 -> 286.7).
// FIXED == 3: rows of 256 bytes read by 16 lanes (4 units per wavefront), a unit per query, any number of iterations
// and chunks (heads of 128 channels in the 16-bit types: backward 380.2 -> 366.1 us in float16, 382.9 -> 369.7 in bfloat16).
template <typename T, int VEC, int NPASS, bool SCATTER, int SRC, bool RECBUF = false, int FIXED = 0>
__global__ __launch_bounds__(256) void msda_bwd_kernel(const KArgs a)
{
    static_assert(!FIXED || (!SCATTER && (SRC == kSrcPlain || (SRC == kSrcFused && FIXED == 1))),
                  "the fixed geometry is built for the tile form of the plain operator (and, one unit per query in one pass, of its fused form)");
    // 1, 2: 8 lanes per row, one pass of one chunk, one / two units per query; 3: 16 lanes per row (4 units per wavefront), a
    // unit per query, any number of iterations and chunks (rows of 256 bytes: heads of 128 channels in the 16-bit types)
    constexpr bool kOnePass = FIXED == 1 || FIXED == 2;
    static_assert(!(kOnePass && RECBUF), "a workgroup that makes one pass collects its records in its staging strips");
    static_assert(!RECBUF || (!SCATTER && (SRC == kSrcPlain || SRC == kSrcFused)), "the record buffer is built for the tile form of the operator and its fused form");
    constexpr int GSHIFT = sizeof(T) == 4 ? 0 : 1;  // value byte offset -> fp32 image byte offset
    constexpr bool FUSED = SRC == kSrcFused;
    constexpr int NC = SRC == kSrcGka ? 1 : 4;  // corner rows per sample (geometric kernel attention: one pixel)

    extern __shared__ __align__(16) unsigned char smem[];
    i32x4* lvl = reinterpret_cast<i32x4*>(smem);
    if constexpr (!SCATTER) {
        // this workgroup's share of the zero-fill of the image (every workgroup of the launch takes one, also those
        // without work): the stores ride along with this kernel instead of taking a launch of their own
        if (a.fill_n4 != 0 && a.sparse != 0 && levels_tile_the_keys(a)) {
            // only the rows that receive atomic additions in the tile pass (tiles split by query range, small tiles,
            // and the first pixel of every other tile); a row of the image is nh*hd floats, a multiple of 16 bytes here
            const int32_t tiles = a.tbl_stride - 1;  // (bound: pieces of tiles that do not exist are skipped)
            const int64_t pieces = (int64_t)a.bs * tiles * kRowParts;
            const uint32_t row4 = (uint32_t)(a.nh * a.hd) / 4;
            const f32x4 z = {0.f, 0.f, 0.f, 0.f};
            for (int64_t w = blockIdx.x; w < pieces; w += gridDim.x) {
                const int32_t b = (int32_t)(w / (tiles * kRowParts)), r = (int32_t)(w % (tiles * kRowParts));
                int32_t r0, r1;
                if (!atomic_rows_of_part(a, r / kRowParts, r % kRowParts, &r0, &r1)) continue;
                f32x4* img = reinterpret_cast<f32x4*>(a.grad_value) + ((size_t)b * a.nk + r0) * row4;
                const uint32_t n4 = (uint32_t)(r1 - r0) * row4;
                for (uint32_t i = threadIdx.x; i < n4; i += blockDim.x) __builtin_nontemporal_store(z, img + i);
            }
        } else if (a.fill_n4 != 0) {
            f32x4* img = reinterpret_cast<f32x4*>(a.grad_value);
            const uint64_t per = (a.fill_n4 + gridDim.x - 1) / gridDim.x;
            const uint64_t lo = (uint64_t)blockIdx.x * per;
            const uint64_t hi = lo + per < a.fill_n4 ? lo + per : a.fill_n4;
            const f32x4 z = {0.f, 0.f, 0.f, 0.f};
            for (uint64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) __builtin_nontemporal_store(z, img + i);
        }
    }
    // (fixed geometry: the arithmetic phases of a wavefront -- geometry and counting, gradients and records -- run at a
    //  raised priority, the gather at the default one: BEVFormer shape 988.6 -> 964.8 us, encoder shape unchanged; the
    //  other way round the encoder shape loses 7 us)
    if constexpr (FIXED != 0) __builtin_amdgcn_s_setprio(2);
    Work wk;
    if (!decode_block(a.plan, blockIdx.x, a.bs, a.nh, a.nq, &wk)) return;

    for (int i = threadIdx.x; i < a.nl; i += blockDim.x) {
        lvl[i] = load_level(a, i);
    }
    __syncthreads();

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;

    const int LPR = FIXED == 3 ? 16 : FIXED ? 8 : a.plan.lanes_per_row;
    const int lpr_log2 = FIXED == 3 ? 4 : FIXED ? 3 : __builtin_ctz(LPR);
    const int U = FIXED == 3 ? 4 : FIXED ? 8 : a.plan.units_per_wave;
    const int iters = kOnePass ? 1 : a.plan.iters;
    // 2^sp neighbouring units share a query, each taking kChunk of its samples: a pass of a wavefront covers `span`
    // samples of U >> sp queries (sp = 0: a unit is a query and goes through its samples kChunk at a time)
    const int sp = FIXED == 3 ? 0 : FIXED ? FIXED - 1 : a.unit_split_log2, sp_mask = (1 << sp) - 1, span = kChunk << sp;
    const int g = lane >> lpr_log2;
    const int c = lane & (LPR - 1);
    // lanes per row in the scatter phase: the power of two covering head_dim, within [LPR, 64]
    int span_log2 = lpr_log2;
    while ((1 << span_log2) < a.hd && span_log2 < 6) ++span_log2;

    // per-wavefront LDS strip: staged samples, then their four reduced dots
    unsigned char* strip = smem + kMaxLevels * sizeof(i32x4) +
                           (size_t)wave * U * (kChunkStride * sizeof(Entry) + kChunk * sizeof(f32x4));
    Entry* stage = reinterpret_cast<Entry*>(strip);
    f32x4* dots = reinterpret_cast<f32x4*>(strip + (size_t)U * kChunkStride * sizeof(Entry));

    const T* attn = static_cast<const T*>(a.attn);
    const T* gout = static_cast<const T*>(a.grad_out);
    T* gloc = static_cast<T*>(a.grad_loc);
    T* gattn = static_cast<T*>(a.grad_attn);
    const T* ref = static_cast<const T*>(a.ref);
    // fused form: per unit {max logit, sum of exponentials, <forward row, grad_out row>} in the pad entry that
    // ends the unit's staging strip
    auto unit_stats = [&](int u) { return reinterpret_cast<float*>(stage + u * kChunkStride + kChunk); };

    const __amdgpu_buffer_rsrc_t vres =
        make_rsrc(static_cast<const char*>(a.value) + (size_t)wk.b * a.batch_bytes, a.batch_bytes);
    const __amdgpu_buffer_rsrc_t gres =
        make_rsrc(reinterpret_cast<const char*>(a.grad_value) + (size_t)wk.b * a.gbatch_bytes, a.gbatch_bytes);
    const uint32_t head_off = (uint32_t)wk.h * a.hd * sizeof(T);
    const uint32_t ghead_off = (uint32_t)wk.h * a.hd * 4u;

    // ---- records per tile of this workgroup: count, prefix, publish -----------------------
    int32_t* tile_first = reinterpret_cast<int32_t*>(
        smem + kMaxLevels * sizeof(i32x4) +
        (size_t)a.plan.waves_per_block * a.plan.units_per_wave * (kChunkStride * sizeof(Entry) + kChunk * sizeof(f32x4)));
    int32_t* cursor = tile_first + kMaxLevels;  // [tbl_stride] counts, then next free position per tile
    uint32_t* slab = nullptr;
    const int entries = U * kChunk;
    // ---- per unit: the grad_out row in the value-load layout and, for the fused form, the softmax terms ----
    float gv[NPASS][VEC];
    // 16-bit rows: the same row as packed pairs, for dot products that multiply two pairs of 16-bit elements exactly
    // and add them to a float32 sum in one instruction (v_dot2c_f32_f16 / v_dot2c_f32_bf16)
    constexpr bool kDot2 = sizeof(T) == 2 && VEC % 2 == 0;
    constexpr int kPairs = kDot2 ? VEC / 2 : 1;
    uint32_t gpk[NPASS][kPairs];
    auto unit_prologue = [&](int q0) {
        // grad_out row of this lane's unit in the value-load layout (for the dots)
        const int qg = q0 + (g >> sp);
        const bool unit_ok = qg < wk.q_end;
        const T* grow = gout + (((int64_t)wk.b * a.nq + (unit_ok ? qg : wk.q_begin)) * a.nh + wk.h) * a.hd;
#pragma unroll
        for (int p = 0; p < NPASS; ++p) {
            const int ch = (c + p * LPR) * VEC;
            if (unit_ok && ch < a.hd) {
                RowIO<T, VEC>::load_global(grow + ch, gv[p]);
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) gv[p][e] = 0.0f;
            }
            if constexpr (kDot2) {
                typedef T t2 __attribute__((ext_vector_type(2)));
#pragma unroll
                for (int e = 0; e < kPairs; ++e)
                    gpk[p][e] = __builtin_bit_cast(uint32_t, t2{from_f32<T>(gv[p][2 * e]), from_f32<T>(gv[p][2 * e + 1])});
            }
        }

        if constexpr (FUSED) {
            // softmax backward: grad_logit_s = w_s * (grad_w_s - sum_t w_t * grad_w_t), and the sum over the
            // unit's samples equals the dot product of the forward row with the grad_out row
            const T* orow = static_cast<const T*>(a.out) +
                            (((int64_t)wk.b * a.nq + (unit_ok ? qg : wk.q_begin)) * a.nh + wk.h) * a.hd;
            float dsum = 0.0f;
#pragma unroll
            for (int p = 0; p < NPASS; ++p) {
                const int ch = (c + p * LPR) * VEC;
                if (unit_ok && ch < a.hd) {
                    float ov[VEC];
                    RowIO<T, VEC>::load_global(orow + ch, ov);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) dsum = __builtin_fmaf(ov[e], gv[p][e], dsum);
                }
            }
            for (int d = 1; d < LPR; d <<= 1) dsum += __shfl_xor(dsum, d, kWave);
            if (c == 0 && g < U) unit_stats(g)[2] = dsum;
            // softmax statistics: lanes 16u..16u+15 share unit u, each takes every 16th logit
            for (int i = lane; i < entries; i += kWave) {
                const int u = i >> 4, sl = i & (kChunk - 1), q = q0 + (u >> sp);
                const T* lg = attn + (((int64_t)wk.b * a.nq + (q < wk.q_end ? q : wk.q_begin)) * a.nh + wk.h) * a.S_full;
                float m = -__builtin_inff();
                for (int s = sl; s < a.S; s += kChunk) m = __builtin_fmaxf(m, to_f32(lg[s]));
                m = group_max<4>(m);  // (kChunk = 16 lanes = one DPP row; rows are wholly active or inactive here)
                float sum = 0.0f;
                for (int s = sl; s < a.S; s += kChunk) sum += expf(to_f32(lg[s]) - m);
                sum = group_sum<4>(sum);
                if (sl == 0) {
                    unit_stats(u)[0] = m;
                    unit_stats(u)[1] = sum;
                }
            }
            wave_lds_sync();
        }
    };
    // ---- geometry of one chunk (kChunk samples of each of the wavefront's units) ----------------
    // A lane stages entries/64 <= kLaneSamples samples per pass and meets the same samples again when
    // their dots are reduced: for the first kKeep of them (all, with up to 8 units per wavefront)
    // fractions, weight, first pixel and validity bits stay in registers until then instead of being
    // derived from the location a second time.
    // (Only for the plain operator and deformable aggregation: the other sample sources run with fewer registers
    // and more wavefronts per SIMD without it, which is worth more to them.)
    constexpr int kLaneSamples = 4, kKeep = (SRC == kSrcPlain || SRC == kSrcDagg) ? 2 : 0, kKeepRegs = kKeep > 0 ? kKeep : 1;
    constexpr int kUnroll = kKeep > 0 ? kLaneSamples : 1;  // (registers are indexed by ks: unrolled)
    float keep_lw[kKeepRegs], keep_lh[kKeepRegs], keep_aw[kKeepRegs];
    int32_t keep_pix[kKeepRegs];
    uint32_t keep_fl[kKeepRegs];  // bit 0 valid, bits 1..4 corner valid, bits 8.. level
    // The plain operator and the fused form stage the first chunk of the first iteration while the records are counted (its
    // samples' geometry is then derived once, not once for the count and once for the gather).
    constexpr bool kEarly = (SRC == kSrcPlain || SRC == kSrcFused) && !SCATTER;
    auto geometry = [&](int q0, int c0, auto counting) {
        constexpr bool COUNT = decltype(counting)::value;
        // what a lane reads for sample i of the chunk: location, weight, level
        struct Read {
            float x, y, aw;
            int l;
            bool active;
        };
        auto read_sample = [&](int i) -> Read {
            Read r{0.f, 0.f, 0.f, 0, false};
            const int u = i >> 4, sl = i & (kChunk - 1);
            const int s = c0 + ((u & sp_mask) << 4) + sl, q = q0 + (u >> sp);
            r.active = (i < entries) && (q < wk.q_end) && (s < a.S);
            if (r.active) {
                const SampleRef sr = sample_ref<SRC>(a, wk.b, q, wk.h, s);
                r.x = load_coord<SRC, T>(a.loc, 2 * sr.loc_e);
                r.y = load_coord<SRC, T>(a.loc, 2 * sr.loc_e + 1);
                if constexpr (SRC == kSrcGrid) r.aw = 1.0f;  // no weights tensor
                else r.aw = to_f32(attn[sr.w_e]);
                r.l = sr.l;
                if constexpr (FUSED) {
                    fused_location(a, ref + (((int64_t)wk.b * a.nq + q) * a.nl + r.l) * a.ref_dim, lvl[r.l], r.x, r.y);
                    r.aw = expf(r.aw - unit_stats(u)[0]) / unit_stats(u)[1];
                }
            }
            return r;
        };
        auto stage_sample = [&](auto ks_c, int i, const Read& rd) {
            constexpr int ks = decltype(ks_c)::value;  // (which registers keep the sample; i = lane + ks * 64 then)
            const int u = i >> 4, sl = i & (kChunk - 1);
            const bool active = rd.active;
            const float x = rd.x, y = rd.y, aw = rd.aw;
            const int l = rd.l;
            const bool inside = SRC != kSrcDagg || (x > 0.0f && x < 1.0f && y > 0.0f && y < 1.0f);
            const Sample sm = source_geometry<SRC>(x, y, lvl[l], a.nk, active && inside, a.grid);
            Entry en;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                en.off[k] = sm.cvalid[k] ? (uint32_t)sm.pix[k] * a.pitch_bytes : kInvalidCorner;
                if constexpr (SCATTER) en.w[k] = sm.valid ? sm.w[k] * aw : 0.0f;
            }
            // (the weights are read by the scatter of the one-kernel form only)
            if constexpr (SCATTER) stage[u * kChunkStride + sl] = en;
            else *reinterpret_cast<u32x4*>(stage[u * kChunkStride + sl].off) = u32x4{en.off[0], en.off[1], en.off[2], en.off[3]};
            if (ks < kKeep) {
                keep_lw[ks % kKeepRegs] = sm.lw;
                keep_lh[ks % kKeepRegs] = sm.lh;
                keep_aw[ks % kKeepRegs] = aw;
                keep_pix[ks % kKeepRegs] = sm.pix[0];
                keep_fl[ks % kKeepRegs] = (sm.valid ? 1u : 0u) | (sm.cvalid[0] ? 2u : 0u) | (sm.cvalid[1] ? 4u : 0u) |
                                      (sm.cvalid[2] ? 8u : 0u) | (sm.cvalid[3] ? 16u : 0u) | ((uint32_t)l << 8);
            }
            if constexpr (COUNT) {
                // the records these samples will leave, merged exactly as where they are written
                bool have[2], keep[2];
                int32_t key[2];
                float za[2] = {0.f, 0.f}, zb[2] = {0.f, 0.f};
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    have[r] = active && (sm.cvalid[2 * r] || sm.cvalid[2 * r + 1]) && tile_first[l] >= 0;
                    key[r] = sm.cvalid[2 * r] ? sm.pix[2 * r] : sm.pix[2 * r + 1];
                }
                merge_pair_records_in_quad(have, key, za, zb, keep);
#pragma unroll
                for (int r = 0; r < 2; ++r)
                    if (keep[r]) atomicAdd(&cursor[tile_first[l] + ((key[r] - lvl[l].z) >> a.tile_px_log2)], 1);
            }
        };
        if constexpr (kUnroll == kLaneSamples) {
            // two samples are read together (one trip to memory instead of two), then staged
            static_assert(kLaneSamples == 4, "written out for four samples per lane");
            {
                const Read r0 = read_sample(lane), r1 = read_sample(lane + kWave);
                if (lane < entries) stage_sample(std::integral_constant<int, 0>{}, lane, r0);
                if (lane + kWave < entries) stage_sample(std::integral_constant<int, 1>{}, lane + kWave, r1);
            }
            if (lane + 2 * kWave < entries) {
                const Read r2 = read_sample(lane + 2 * kWave), r3 = read_sample(lane + 3 * kWave);
                stage_sample(std::integral_constant<int, 2>{}, lane + 2 * kWave, r2);
                if (lane + 3 * kWave < entries) stage_sample(std::integral_constant<int, 3>{}, lane + 3 * kWave, r3);
            }
        } else {
            for (int i = lane; i < entries && i < kLaneSamples * kWave; i += kWave)
                stage_sample(std::integral_constant<int, 0>{}, i, read_sample(i));
        }
    };
    if constexpr (!SCATTER) {
        const int64_t wg_row = ((int64_t)wk.b * a.nh + wk.h) * a.nwg + wk.q_begin / a.plan.tile_q;
        slab = a.rec + wg_row * a.rec_cap * kRecDwords;
        if (threadIdx.x == 0) {
            // the run table has room for tbl_stride - 1 tiles, which is every tile when the levels do not
            // overlap; a level that does not fit (malformed shapes) is left out of grad_value: -1
            int32_t first = 0;
            for (int l = 0; l < a.nl; ++l) {
                int32_t px;
                const int32_t nt = level_tile_count(lvl[l].x, lvl[l].y, lvl[l].z, a.nk, a.tile_px_log2, &px);
                const bool fits = first + nt <= a.tbl_stride - 1;
                tile_first[l] = fits ? first : -1;
                if (fits) first += nt;
            }
        }
        for (int i = threadIdx.x; i < a.tbl_stride; i += blockDim.x) cursor[i] = 0;
        __syncthreads();
        // queries whose first `span` samples are counted here:
        const int early_units = kEarly ? (a.plan.waves_per_block * U) >> sp : 0;
        if constexpr (kEarly) {
            const int q0 = wk.q_begin + ((wave * U) >> sp);
            if (q0 < wk.q_end) {
                if constexpr (FUSED) unit_prologue(q0);  // (the weights need the softmax terms)
                geometry(q0, 0, std::true_type{});
            }
        }
        // Records are merged inside aligned groups of 4 samples of a query (merge_pair_records_in_quad), here exactly as
        // where they are written: the samples of a query are padded to a multiple of 4 lanes, and every lane of
        // the workgroup goes through every trip (the lane exchanges need their partners).
        const int S4 = (a.S + 3) & ~3;
        const int n = (wk.q_end - wk.q_begin) * S4;
        const bool all_early = kOnePass || (early_units >= wk.q_end - wk.q_begin && a.S <= span);  // nothing left to count
        for (int base = 0; base < n && !all_early; base += blockDim.x) {
            const int i = base + (int)threadIdx.x;
            const int qr = i / S4, s = i - qr * S4;
            const bool act = i < n && s < a.S && !(qr < early_units && s < span);
            int l = 0;
            Sample sm;
            sm.cvalid[0] = sm.cvalid[1] = sm.cvalid[2] = sm.cvalid[3] = false;
            sm.pix[0] = sm.pix[1] = sm.pix[2] = sm.pix[3] = 0;
            if (act) {
                const SampleRef sr = sample_ref<SRC>(a, wk.b, wk.q_begin + qr, wk.h, s);
                l = sr.l;
                float cx = load_coord<SRC, T>(a.loc, 2 * sr.loc_e), cy = load_coord<SRC, T>(a.loc, 2 * sr.loc_e + 1);
                if constexpr (FUSED)
                    fused_location(a, static_cast<const T*>(a.ref) + (((int64_t)wk.b * a.nq + wk.q_begin + qr) * a.nl + l) * a.ref_dim,
                                   lvl[l], cx, cy);
                const bool inside = SRC != kSrcDagg || (cx > 0.0f && cx < 1.0f && cy > 0.0f && cy < 1.0f);
                sm = source_geometry<SRC>(cx, cy, lvl[l], a.nk, inside, a.grid);
            }
            bool have[2], keep[2];
            int32_t key[2];
            float za[2] = {0.f, 0.f}, zb[2] = {0.f, 0.f};
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                have[r] = act && (sm.cvalid[2 * r] || sm.cvalid[2 * r + 1]) && tile_first[l] >= 0;
                key[r] = sm.cvalid[2 * r] ? sm.pix[2 * r] : sm.pix[2 * r + 1];
            }
            merge_pair_records_in_quad(have, key, za, zb, keep);
#pragma unroll
            for (int r = 0; r < 2; ++r)
                if (keep[r]) atomicAdd(&cursor[tile_first[l] + ((key[r] - lvl[l].z) >> a.tile_px_log2)], 1);
        }
        __syncthreads();
        if (wave == 0) {
            // exclusive prefix over the counts, 64 at a time
            int32_t carry = 0;
            for (int base = 0; base < a.tbl_stride; base += kWave) {
                const int i = base + lane;
                const int32_t v = i < a.tbl_stride ? cursor[i] : 0;
                int32_t inc = v;
#pragma unroll
                for (int d = 1; d < kWave; d <<= 1) {
                    const int32_t o = __shfl_up(inc, d, kWave);
                    if (lane >= d) inc += o;
                }
                if (i < a.tbl_stride) cursor[i] = carry + inc - v;
                carry += __builtin_amdgcn_readlane(inc, kWave - 1);
            }
        }
        __syncthreads();
        uint32_t* row = a.tbl + wg_row * a.tbl_stride;
        for (int i = threadIdx.x; i < a.tbl_stride; i += blockDim.x) row[i] = (uint32_t)cursor[i];
        __syncthreads();  // the cursors are advanced from here on
    }

    uint32_t choff[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
        const int ch = (c + p * LPR) * VEC;
        choff[p] = head_off + (ch < a.hd ? ch * (uint32_t)sizeof(T) : 0u);
    }

    // A workgroup that passes through one iteration of one chunk (all samples of the plain operator and of the fused
    // form staged during the count) collects its records in LDS and writes its slab in whole lines: once every
    // wavefront has gathered, the staged entries are free, and a unit's 32 records (two per sample) fit the 16 entries
    // before its pad entry (which the fused form still needs).  Record `pos` of the slab lives at record pos % 32 of
    // unit pos / 32 of the workgroup.
    const bool rec_in_lds = kOnePass || ((SRC == kSrcPlain || SRC == kSrcFused) && !SCATTER && iters == 1 && a.S <= span);
    const int u_log2 = FIXED == 3 ? 2 : FIXED ? 3 : __builtin_ctz(U);
    auto rec_lds = [&](int pos) {
        const int unit = pos >> 5;  // of the workgroup: wavefront unit >> u_log2, its unit & (U - 1)
        return reinterpret_cast<u32x4*>(smem + kMaxLevels * sizeof(i32x4) +
                                        (size_t)(unit >> u_log2) * U * (kChunkStride * sizeof(Entry) + kChunk * sizeof(f32x4)) +
                                        (size_t)(unit & (U - 1)) * (kChunkStride * sizeof(Entry))) +
               (pos & 31);
    };
    // (records take a 16-byte slot in LDS and 12 bytes in the slab)
    typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
    const __amdgpu_buffer_rsrc_t sres = make_rsrc(slab, SCATTER ? 0u : (uint32_t)a.rec_cap * (kRecDwords * 4u));
    auto store_record = [&](int pos, const u32x4 rec) {
        // (non-temporal: the records are read by the next kernel and should not push value rows out of L2)
        __builtin_amdgcn_raw_buffer_store_b96(u32x3{rec.x, rec.y, rec.z}, sres, (uint32_t)pos * (kRecDwords * 4u), 0, 2);
    };
    auto copy_records_out = [&]() {
        const int total = cursor[a.tbl_stride - 1];  // (exclusive prefix: the entry after the last tile holds the sum)
        for (int i = threadIdx.x; i < total; i += blockDim.x) store_record(i, *rec_lds(i));
    };
    // A workgroup that makes several passes (iterations, or chunks of units with more than 16 samples) and whose slab
    // is small collects its records, 12 bytes each, in a buffer of its own behind the counters and writes the slab in
    // whole lines when it is done: a pass adds a few records to every run, and stored one by one those pieces -- the
    // shorter, the smaller the tiles of the grad_value pass are -- reach memory as partial lines.
    typedef uint32_t __attribute__((may_alias)) u32_alias;
    u32_alias* recbuf = nullptr;
    if constexpr (RECBUF) {
        if (!rec_in_lds && a.rec_lds_bytes != 0)
            recbuf = reinterpret_cast<u32_alias*>(smem + ((reinterpret_cast<unsigned char*>(cursor + a.tbl_stride) - smem + 15) & ~(size_t)15));
    }

    for (int it = 0; it < iters; ++it) {
        const int q0 = wk.q_begin + (((it * a.plan.waves_per_block + wave) * U) >> sp);
        if (q0 >= wk.q_end) {
            if (rec_in_lds) {  // meets the other wavefronts at their two barriers and helps with the copy
                __syncthreads();
                __syncthreads();
                copy_records_out();
            }
            break;
        }

        if (!(kEarly && FUSED && it == 0)) unit_prologue(q0);  // (the fused form's first iteration: done before the count)

        for (int c0 = 0; c0 < (kOnePass ? 1 : a.S); c0 += span) {
            // ---- geometry (the first chunk of the first iteration was staged while records were counted) ----
            if (!(kEarly && it == 0 && c0 == 0)) geometry(q0, c0, std::false_type{});
            wave_lds_sync();

            // ---- gather and dots -------------------------------------------------------
            const int ns = (a.S - c0) < kChunk ? (a.S - c0) : kChunk;
            const Entry* mine = stage + g * kChunkStride;
            // (the reduction width is a compile-time constant inside the loop: with a run-time width its
            // uniform branches keep the row loads of the next samples from being issued early)
            auto gather_dots = [&](auto lg) {
                constexpr int LG = decltype(lg)::value;
                typedef typename RowIO<T, VEC>::raw_t raw_t;
                // the corner rows of staged sample sl (channels of row pass p)
                auto request = [&](int sl, int p, raw_t (&raw)[NC]) {
                    const u32x4 off = *reinterpret_cast<const u32x4*>(mine[sl].off);
#pragma unroll
                    for (int k = 0; k < NC; ++k) raw[k] = RowIO<T, VEC>::load_raw(vres, off[k] + choff[p]);
                };
                auto accumulate = [&](int p, const raw_t (&raw)[NC], float (&d)[4]) {
#pragma unroll
                    for (int k = 0; k < NC; ++k) {
                        if constexpr (kDot2) {
                            uint32_t words[kPairs];
                            __builtin_memcpy(words, &raw[k], sizeof(words));
#pragma unroll
                            for (int e = 0; e < kPairs; ++e) d[k] = dot2_acc<T>(words[e], gpk[p][e], d[k]);
                        } else {
                            float v[VEC];
                            RowIO<T, VEC>::unpack(raw[k], v);
#pragma unroll
                            for (int e = 0; e < VEC; ++e) d[k] = __builtin_fmaf(v[e], gv[p][e], d[k]);
                        }
                    }
                };
                auto finish = [&](int sl, const float (&d)[4]) {
                    f32x4 dsum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int k = 0; k < NC; ++k) dsum[k] = group_sum<LG>(d[k]);
                    if (c == 0) dots[g * kChunk + sl] = dsum;
                };
                // (where it measured faster: the fixed geometry, and geometric kernel attention -- step 0.807 -> 0.786 ms;
                //  the fused form, 0.440 -> 0.459 ms for forward + backward, and the grid sampler, 0.192 -> 0.200 ms, lose
                //  more to the registers than they gain)
                constexpr bool kAhead = (FIXED != 0 || SRC == kSrcGka) && NPASS <= 2;
                if constexpr (kAhead) {
                    // the rows of the next sample (of the row's second half, with two passes) are requested before the
                    // rows at hand are used: a wavefront otherwise goes through the samples of its chunk one trip to
                    // memory after the other, and spends 71 % of its life in this loop (encoder backward 268.4 ->
                    // 260.9 us, float16 277.5 -> 270.3, BEVFormer shape 998 -> 994; with three sets of rows in flight
                    // the encoder shape loses 1.5 us to the registers they take)
                    raw_t ra[NC], rb[NC];
                    constexpr int PB = NPASS - 1;  // row pass of the second set
                    float d[4] = {0.f, 0.f, 0.f, 0.f};
                    auto consume = [&](int t, auto pass, const raw_t (&raw)[NC]) {
                        constexpr int P = decltype(pass)::value;
                        accumulate(P, raw, d);
                        if (P == NPASS - 1) {
                            finish(t / NPASS, d);
                            d[0] = d[1] = d[2] = d[3] = 0.f;
                        }
                    };
                    const int nt = ns * NPASS;  // (even with two passes)
                    request(0, 0, ra);
                    for (int t = 0; t < nt; t += 2) {
                        const bool two = t + 1 < nt;
                        if (two) request((t + 1) / NPASS, PB, rb);
                        consume(t, std::integral_constant<int, 0>{}, ra);
                        if (two) {
                            if (t + 2 < nt) request((t + 2) / NPASS, 0, ra);
                            consume(t + 1, std::integral_constant<int, PB>{}, rb);
                        }
                    }
                } else {
                    for (int sl = 0; sl < ns; ++sl) {
                        float d[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int p = 0; p < NPASS; ++p) {
                            raw_t raw[NC];
                            request(sl, p, raw);
                            accumulate(p, raw, d);
                        }
                        finish(sl, d);
                    }
                }
            };
            if constexpr (FIXED != 0) __builtin_amdgcn_s_setprio(0);
            switch (lpr_log2) {
                case 2: gather_dots(std::integral_constant<int, 2>{}); break;
                case 3: gather_dots(std::integral_constant<int, 3>{}); break;
                case 4: gather_dots(std::integral_constant<int, 4>{}); break;
                case 5: gather_dots(std::integral_constant<int, 5>{}); break;
                default: gather_dots(std::integral_constant<int, 6>{}); break;
            }
            if constexpr (FIXED != 0) __builtin_amdgcn_s_setprio(2);
            wave_lds_sync();
            if (rec_in_lds) __syncthreads();  // every wavefront's staged entries have been used: the strips take records
            // ---- scatter: grad_value[row_c] += (w_c*attn) * grad_out row --------------------
            // `span` consecutive lanes own consecutive floats of one row, so every atomic
            // instruction covers 64/span rows with fully contiguous 64-byte pieces: the
            // atomics are carried out at the memory side at a fixed rate per 64-byte request,
            // whatever part of the 64 bytes a request uses.
            if constexpr (SCATTER) {
                const int nsub = kWave >> span_log2;
                const int sub = lane >> span_log2, ch0 = lane & ((1 << span_log2) - 1);
                for (int u = sub; u < U; u += nsub) {
                    const int qq = q0 + (u >> sp);
                    if (qq >= wk.q_end) break;  // later units of this lane are past the end too
                    const T* gr = gout + (((int64_t)wk.b * a.nq + qq) * a.nh + wk.h) * a.hd;
                    const Entry* ent = stage + u * kChunkStride;
                    for (int chb = 0; chb < a.hd; chb += (1 << span_log2)) {
                        const int ch = chb + ch0;
                        if (ch < a.hd) {
                            const float gg = to_f32(gr[ch]);
                            const uint32_t choff_g = ghead_off + (uint32_t)ch * 4u;
                            for (int sl = 0; sl < ns; ++sl) {
                                const u32x4 off = *reinterpret_cast<const u32x4*>(ent[sl].off);
                                const f32x4 w = *reinterpret_cast<const f32x4*>(ent[sl].w);
#pragma unroll
                                for (int k = 0; k < 4; ++k)
                                    __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(w[k] * gg, gres,
                                                                                    (off[k] << GSHIFT) + choff_g, 0, 0);
                            }
                        }
                    }
                }
            }

            // ---- grad_attn / grad_loc from the reduced dots, one sample per lane ----------
#pragma unroll kUnroll
            for (int ks = 0; ks < kLaneSamples; ++ks) {
                const int i = lane + ks * kWave;
                if (i >= entries) break;
                const int u = i >> 4, sl = i & (kChunk - 1);
                const int s = c0 + ((u & sp_mask) << 4) + sl, q = q0 + (u >> sp);
                // the sample's pair records (upper and lower corners), written after the gradients
                bool rec_have[2] = {false, false};
                int32_t rec_key[2] = {0, 0};
                float rec_wa[2] = {0.f, 0.f}, rec_wb[2] = {0.f, 0.f};
                int rec_l = 0;
                if ((q < wk.q_end) && (s < a.S)) {
                    const SampleRef sr = sample_ref<SRC>(a, wk.b, q, wk.h, s);
                    int l = sr.l;
                    float aw = 1.0f, ox = 0.f, oy = 0.f;  // (ox, oy): raw offsets of the fused form
                    Sample sm;
                    if (ks < kKeep) {
                        // the sample as the geometry pass left it
                        const uint32_t fl = keep_fl[ks % kKeepRegs];
                        l = (int)(fl >> 8);
                        aw = keep_aw[ks % kKeepRegs];
                        sm.valid = (fl & 1u) != 0;
                        sm.lw = keep_lw[ks % kKeepRegs];
                        sm.lh = keep_lh[ks % kKeepRegs];
                        sm.Wf = (float)lvl[l].y;  // (as sample_geometry sets them; only the plain operator keeps samples)
                        sm.Hf = (float)lvl[l].x;
                        float wt[4];
                        bilinear_weights(sm.lw, sm.lh, wt);
                        const int32_t Wl = lvl[l].y;
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            sm.pix[k] = keep_pix[ks % kKeepRegs] + (k & 1) + (k >> 1) * Wl;
                            sm.cvalid[k] = ((fl >> (1 + k)) & 1u) != 0;
                            sm.w[k] = sm.valid ? wt[k] : 0.0f;
                        }
                        if constexpr (FUSED) {
                            ox = load_coord<SRC, T>(a.loc, 2 * sr.loc_e);
                            oy = load_coord<SRC, T>(a.loc, 2 * sr.loc_e + 1);
                        }
                    } else {
                        float x = load_coord<SRC, T>(a.loc, 2 * sr.loc_e);
                        float y = load_coord<SRC, T>(a.loc, 2 * sr.loc_e + 1);
                        if constexpr (SRC != kSrcGrid) aw = to_f32(attn[sr.w_e]);
                        ox = x;
                        oy = y;
                        if constexpr (FUSED) {
                            fused_location(a, ref + (((int64_t)wk.b * a.nq + q) * a.nl + l) * a.ref_dim, lvl[l], x, y);
                            aw = expf(aw - unit_stats(u)[0]) / unit_stats(u)[1];
                        }
                        const bool inside = SRC != kSrcDagg || (x > 0.0f && x < 1.0f && y > 0.0f && y < 1.0f);
                        sm = source_geometry<SRC>(x, y, lvl[l], a.nk, inside, a.grid);
                    }
                    const T* rp = nullptr;
                    if constexpr (FUSED) rp = ref + (((int64_t)wk.b * a.nq + q) * a.nl + l) * a.ref_dim;
                    const f32x4 dd = dots[u * kChunk + sl];
                    float ga = 0.f, gx = 0.f, gy = 0.f;
                    if (sm.valid) {
                        const float hw = 1.0f - sm.lw, hh = 1.0f - sm.lh;
                        ga = sm.w[0] * dd[0] + sm.w[1] * dd[1] + sm.w[2] * dd[2] + sm.w[3] * dd[3];
                        gx = sm.Wf * aw * (hh * (dd[1] - dd[0]) + sm.lh * (dd[3] - dd[2]));
                        gy = sm.Hf * aw * (hw * (dd[2] - dd[0]) + sm.lw * (dd[3] - dd[1]));
                    }
                    if constexpr (FUSED) {
                        // chain rule through the softmax and through location = reference + offset * scale
                        gattn[sr.w_e] = from_f32<T>(aw * (ga - unit_stats(u)[2]));
                        float r2 = 0.0f, r3 = 0.0f;  // boxes: gradient of (w, h)
                        if (a.ref_dim == 2) {
                            gloc[2 * sr.loc_e] = from_f32<T>(gx / (float)lvl[l].y);
                            gloc[2 * sr.loc_e + 1] = from_f32<T>(gy / (float)lvl[l].x);
                        } else {
                            gloc[2 * sr.loc_e] = from_f32<T>(gx / (float)a.np * to_f32(rp[2]) * 0.5f);
                            gloc[2 * sr.loc_e + 1] = from_f32<T>(gy / (float)a.np * to_f32(rp[3]) * 0.5f);
                            r2 = gx * (ox / (float)a.np * 0.5f);
                            r3 = gy * (oy / (float)a.np * 0.5f);
                        }
                        if (a.grad_ref != nullptr) {
                            // the points of a level share the reference point: sum over them here, per head
                            // into a float32 partial image that a small kernel adds up over the heads
                            float* part = a.grad_ref + (((int64_t)wk.h * a.bs + wk.b) * a.nq + q) * (a.nl * a.ref_dim) +
                                          l * a.ref_dim;
                            if (a.np_pow2) {
                                for (int d = 1; d < a.np; d <<= 1) {
                                    gx += __shfl_xor(gx, d, kWave);
                                    gy += __shfl_xor(gy, d, kWave);
                                    r2 += __shfl_xor(r2, d, kWave);
                                    r3 += __shfl_xor(r3, d, kWave);
                                }
                                if ((s & (a.np - 1)) == 0) {
                                    part[0] = gx;
                                    part[1] = gy;
                                    if (a.ref_dim == 4) {
                                        part[2] = r2;
                                        part[3] = r3;
                                    }
                                }
                            } else {
                                unsafeAtomicAdd(part, gx);
                                unsafeAtomicAdd(part + 1, gy);
                                if (a.ref_dim == 4) {
                                    unsafeAtomicAdd(part + 2, r2);
                                    unsafeAtomicAdd(part + 3, r3);
                                }
                            }
                        }
                    } else if constexpr (SRC != kSrcGrid) __builtin_nontemporal_store(from_f32<T>(ga), gattn + sr.w_e);
                    if constexpr (FUSED) {
                    } else if constexpr (SRC == kSrcDagg) {
                        // one location serves the scales of its camera and every head: sum over the
                        // scales here (neighbouring lanes), per head into a float32 partial image that a
                        // small kernel adds up over the heads afterwards
                        float* part = reinterpret_cast<float*>(a.grad_loc) +
                                      2 * ((int64_t)wk.h * ((int64_t)a.bs * a.nq * a.np * a.cams) + sr.loc_e);
                        if (a.sc_pow2) {
                            for (int d = 1; d < a.scales; d <<= 1) {
                                gx += __shfl_xor(gx, d, kWave);
                                gy += __shfl_xor(gy, d, kWave);
                            }
                            if ((l & (a.scales - 1)) == 0) {
                                part[0] = gx;
                                part[1] = gy;
                            }
                        } else {
                            unsafeAtomicAdd(part, gx);
                            unsafeAtomicAdd(part + 1, gy);
                        }
                    } else if constexpr (SRC != kSrcGka) {  // (pixel-index locations have no gradient)
                        // (streamed out like the records: results should not push value rows out of L2)
                        __builtin_nontemporal_store(from_f32<T>(gx), gloc + 2 * sr.loc_e);
                        __builtin_nontemporal_store(from_f32<T>(gy), gloc + 2 * sr.loc_e + 1);
                    }
                    if constexpr (!SCATTER) {
                        rec_l = l;
#pragma unroll
                        for (int r = 0; r < 2; ++r) {
                            const bool vl = sm.cvalid[2 * r], vr = sm.cvalid[2 * r + 1];
                            rec_have[r] = (vl || vr) && tile_first[l] >= 0;
                            rec_key[r] = vl ? sm.pix[2 * r] : sm.pix[2 * r + 1];
                            rec_wa[r] = (vl ? sm.w[2 * r] : sm.w[2 * r + 1]) * aw;
                            rec_wb[r] = (vl && vr) ? sm.w[2 * r + 1] * aw : 0.0f;
                        }
                    }
                }
                if constexpr (!SCATTER) {
                    // pair records for the tile pass: the same decisions, lane for lane, as in the counting sweep
                    // (every lane of an aligned group of 4 takes part in the merge, with or without a record)
                    bool rec_keep[2];
                    merge_pair_records_in_quad(rec_have, rec_key, rec_wa, rec_wb, rec_keep);
#pragma unroll
                    for (int r = 0; r < 2; ++r) {
                        if (rec_keep[r]) {
                            const int32_t pos =
                                atomicAdd(&cursor[tile_first[rec_l] + ((rec_key[r] - lvl[rec_l].z) >> a.tile_px_log2)], 1);
                            const uint32_t in_tile = (uint32_t)(rec_key[r] - lvl[rec_l].z) & ((1u << a.tile_px_log2) - 1u);
                            const u32x4 rec = {in_tile | ((uint32_t)(q - wk.q_begin) << a.tile_px_log2),
                                               __builtin_bit_cast(uint32_t, rec_wa[r]), __builtin_bit_cast(uint32_t, rec_wb[r]), 0u};
                            if (rec_in_lds) {
                                *rec_lds(pos) = rec;
                            } else if (RECBUF && recbuf != nullptr) {
                                recbuf[3 * pos] = rec.x;
                                recbuf[3 * pos + 1] = rec.y;
                                recbuf[3 * pos + 2] = rec.z;
                            } else {
                                store_record(pos, rec);
                            }
                        }
                    }
                }
            }
            wave_lds_sync();
            if (rec_in_lds) {  // every wavefront's records are in the strips: the slab is written in whole lines
                __syncthreads();
                copy_records_out();
            }
        }

        // slots of levels that attention_weights carries beyond spatial_shapes: zero gradients
        const int extra = a.S_full - a.S;
        if (extra > 0) {
            for (int i = lane; i < (U >> sp) * extra; i += kWave) {
                const int u = i / extra, s = a.S + i % extra, q = q0 + u;
                if (q < wk.q_end) {
                    const int64_t e = (((int64_t)wk.b * a.nq + q) * a.nh + wk.h) * a.S_full + s;
                    gattn[e] = from_f32<T>(0.f);
                    gloc[2 * e] = from_f32<T>(0.f);
                    gloc[2 * e + 1] = from_f32<T>(0.f);
                }
            }
        }
    }
    if constexpr (RECBUF) {
        if (recbuf != nullptr) {  // (uniform over the workgroup; every wavefront leaves the loop above)
            __syncthreads();
            // the slab as it lies in the buffer: 16 bytes per lane, then the odd words
            const int words = 3 * cursor[a.tbl_stride - 1], quads = words >> 2;
            for (int i = threadIdx.x; i < quads; i += blockDim.x)
                __builtin_amdgcn_raw_buffer_store_b128(u32x4{recbuf[4 * i], recbuf[4 * i + 1], recbuf[4 * i + 2], recbuf[4 * i + 3]}, sres,
                                                       (uint32_t)i * 16u, 0, 2);
            for (int i = 4 * quads + threadIdx.x; i < words; i += blockDim.x)
                __builtin_amdgcn_raw_buffer_store_b32(recbuf[i], sres, (uint32_t)i * 4u, 0, 2);
        }
    }
}

template <typename T, int VEC, int NPASS>
inline hipError_t launch_one(const KArgs& a, bool scatter, hipStream_t stream)
{
    const dim3 grid(a.plan.grid), block(a.plan.block);
    // (the 16-lane fixed geometry is built for lanes of 16 bytes and one row pass: rows of 256 bytes; with two passes --
    //  heads of 128 float32 channels -- it changes nothing, 544 us)
    constexpr bool kWide = sizeof(T) * VEC == 16 && NPASS == 1;
    if (a.grid) {
        if (scatter)
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, NPASS, true, kSrcGrid>), grid, block, a.plan.lds_bytes, stream, a);
        else
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, NPASS, false, kSrcGrid>), grid, block, a.plan.lds_bytes, stream, a);
    } else if (a.gka) {
        if (scatter)
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, NPASS, true, kSrcGka>), grid, block, a.plan.lds_bytes, stream, a);
        else
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, NPASS, false, kSrcGka>), grid, block, a.plan.lds_bytes, stream, a);
    } else if (a.cams > 0) {
        if (scatter)
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, NPASS, true, kSrcDagg>), grid, block, a.plan.lds_bytes, stream, a);
        else
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, NPASS, false, kSrcDagg>), grid, block, a.plan.lds_bytes, stream, a);
    } else if (a.ref != nullptr) {
        if (scatter)
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, NPASS, true, kSrcFused>), grid, block, a.plan.lds_bytes, stream, a);
        else if (a.rec_lds_bytes != 0)
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, NPASS, false, kSrcFused, true>), grid, block, a.plan.lds_bytes, stream, a);
        else if (a.bwd_fixed == 1 && NPASS == 1)
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, 1, false, kSrcFused, false, 1>), grid, block, a.plan.lds_bytes, stream, a);
        else
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, NPASS, false, kSrcFused>), grid, block, a.plan.lds_bytes, stream, a);
    } else {
        if (scatter)
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, NPASS, true, kSrcPlain>), grid, block, a.plan.lds_bytes, stream, a);
        else if (a.bwd_fixed == 3 && kWide && a.rec_lds_bytes != 0)
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, kWide ? NPASS : 1, false, kSrcPlain, true, 3>), grid, block, a.plan.lds_bytes, stream, a);
        else if (a.bwd_fixed == 3 && kWide)
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, kWide ? NPASS : 1, false, kSrcPlain, false, 3>), grid, block, a.plan.lds_bytes, stream, a);
        else if (a.rec_lds_bytes != 0)
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, NPASS, false, kSrcPlain, true>), grid, block, a.plan.lds_bytes, stream, a);
        else if (a.bwd_fixed == 1 && NPASS == 1)
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, 1, false, kSrcPlain, false, 1>), grid, block, a.plan.lds_bytes, stream, a);
        else if (a.bwd_fixed == 2 && NPASS == 1)
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, 1, false, kSrcPlain, false, 2>), grid, block, a.plan.lds_bytes, stream, a);
        else
            hipLaunchKernelGGL((msda_bwd_kernel<T, VEC, NPASS, false, kSrcPlain>), grid, block, a.plan.lds_bytes, stream, a);
    }
    return hipGetLastError();
}

template <typename T>
inline hipError_t launch_dtype(const KArgs& a, bool scatter, hipStream_t stream)
{
    const int vec = a.plan.vec, np = a.plan.npass;
    if (vec == 1 && np == 1) return launch_one<T, 1, 1>(a, scatter, stream);
    if (vec == 1 && np == 2) return launch_one<T, 1, 2>(a, scatter, stream);
    if (vec == 1 && np == 4) return launch_one<T, 1, 4>(a, scatter, stream);
    if (vec == 2 && np == 1) return launch_one<T, 2, 1>(a, scatter, stream);
    if (vec == 2 && np == 2) return launch_one<T, 2, 2>(a, scatter, stream);
    if (vec == 4 && np == 1) return launch_one<T, 4, 1>(a, scatter, stream);
    if constexpr (sizeof(T) == 4) {
        if (vec == 4 && np == 2) return launch_one<T, 4, 2>(a, scatter, stream);
    }
    if constexpr (sizeof(T) == 2) {
        if (vec == 8 && np == 1) return launch_one<T, 8, 1>(a, scatter, stream);
        if (vec == 8 && np == 2) return launch_one<T, 8, 2>(a, scatter, stream);
    }
    return hipErrorInvalidConfiguration;
}


}  // namespace mxd
