// Forward kernel of multi-scale deformable attention for gfx950 (MI355X), wave64.
//
//   out[b,q,h,:] = sum_{l,p} attn[b,q,h,l,p] * bilinear(value_l[b,:,h,:], loc[b,q,h,l,p])
//
// Arithmetic: reference kernels/multi_scale_deformable_attn/op_kernel/msda.h:351-539
// (pixel coordinates, validity, weights) and
// kernels/multi_scale_deformable_attn/op_kernel/arch35/multi_scale_deformable_attn.cpp:36-80
// (corner predicates, accumulation).  The structure is this library's own:
//
//   * A wavefront works on U = 64/lanes_per_row units (b,q,h) at once; the lanes of a unit
//     each own `vec` channels, so one corner row is ONE coalesced buffer load (128 B for
//     head_dim 32 fp32) and the level/point sum stays in fp32 registers -- no reduction
//     across lanes is ever needed.
//   * Per pass, every lane first computes the geometry of one or more samples (one sample
//     per lane, not per unit): validity, floor, the 4 weights times the attention weight,
//     and the 4 row offsets.  These 32 B per sample go to the wavefront's private LDS strip
//     and are then read back, broadcast to the lanes of the owning unit.
//   * Rows are fetched with raw buffer loads bound to the batch element's value slice: a
//     corner outside the image gets an out-of-range offset and the hardware returns zeros,
//     so zero padding costs no branch and never touches memory (NaNs in unrelated pixels
//     cannot leak in).
//
// FUSED = true folds the two steps that deformable-attention modules run before the operator
// (Deformable-DETR's MSDeformAttn.forward, mmcv's MultiScaleDeformableAttention.forward) into
// the geometry stage: softmax of the nl*np attention logits of a unit (statistics per unit by
// the 16 lanes that later own its samples) and sampling location = reference point +
// offset / (W, H)  [2-d reference points]  or  + offset / np * (w, h) * 0.5  [boxes].
// The normalised locations and weights then never exist in memory.
//
// SRC = kSrcDagg is deformable aggregation (reference: mx_driving/ops/npu_deformable_aggregation.py,
// kernels/deformable_aggregation/): the same sum with a channel group as head, a (camera, scale) pair as
// level, one location per (anchor, point, camera) shared by scales and groups, weights laid out
// [.., point, camera, scale, group], and samples counted only strictly inside (0, 1) x (0, 1).
// SRC = kSrcGka: geometric kernel attention (the location is a clamped pixel index, one row per sample).
// SRC = kSrcGrid: bilinear 2-D grid sampler (one level, one head, one point, weight 1, grid coordinates).
#include "msda_device.h"

namespace mxd {

template <typename T, int VEC, int NPASS, int SRC, bool LDSC, bool AHEAD = false>
__global__ __launch_bounds__(LDSC ? 512 : 256) void msda_fwd_kernel(const KArgs a)
{
    constexpr bool FUSED = SRC == kSrcFused;
    constexpr int NC = SRC == kSrcGka ? 1 : 4;  // corner rows per sample (geometric kernel attention: one pixel)
    static_assert(!LDSC || (SRC == kSrcPlain && VEC * sizeof(T) == 16), "the level cache is built for 16-byte lanes");
    extern __shared__ __align__(16) unsigned char smem[];
    i32x4* lvl = reinterpret_cast<i32x4*>(smem);                               // [kMaxLevels]
    Entry* stage_all = reinterpret_cast<Entry*>(smem + kMaxLevels * sizeof(i32x4));

    Work wk;
    if (!decode_block(a.plan, blockIdx.x, a.bs, a.nh, a.nq, &wk)) return;      // whole workgroup leaves

    for (int i = threadIdx.x; i < a.nl; i += blockDim.x) {
        lvl[i] = load_level(a, i);
    }
    __syncthreads();

    // ---- level cache (LDSC): the rows of this (batch, head) for the last levels, as many as fit ----------
    // The gather is bound by the vector-memory pipeline (64 bytes per clock per CU); rows held in LDS are read
    // through the LDS pipeline instead, in parallel with it.  Levels are cached from the last one backwards
    // while level_start_index is ascending and the rows from that level's start to the end of value fit.
    unsigned char* cache = smem + kMaxLevels * sizeof(i32x4) +
                           (size_t)a.plan.waves_per_block * a.plan.units_per_wave * (kChunkStride * sizeof(Entry) + 2 * sizeof(float));
    const uint32_t row_bytes = (uint32_t)a.hd * sizeof(T);
    int c_first = a.nl, c_base = 0, c_rows = 0;
    if constexpr (LDSC) {
        // (every thread takes the same decision from the level table in LDS)
        const int cap_rows = (int)(a.lds_cache_bytes / row_bytes) - 1;  // one more row of zeros
        for (int l = a.nl - 1; l >= 0; --l) {
            const int b0 = lvl[l].z;
            if (b0 < 0 || b0 >= a.nk || a.nk - b0 > cap_rows || (l < a.nl - 1 && b0 > lvl[l + 1].z)) break;
            c_first = l;
            c_base = b0;
        }
        c_rows = c_first < a.nl ? a.nk - c_base : 0;
        const int pieces = (int)(row_bytes / 16), total = c_rows * pieces;
        const char* src = static_cast<const char*>(a.value) + (size_t)wk.b * a.batch_bytes +
                          (size_t)c_base * a.pitch_bytes + (size_t)wk.h * row_bytes;
        // four pieces per thread and trip, all requested before the first is stored
        for (int i0 = threadIdx.x; i0 < total; i0 += 4 * (int)blockDim.x) {
            u32x4 piece[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int i = i0 + j * (int)blockDim.x;
                const int row = i / pieces, col = i - row * pieces;
                if (i < total) piece[j] = *reinterpret_cast<const u32x4*>(src + (size_t)row * a.pitch_bytes + col * 16);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int i = i0 + j * (int)blockDim.x;
                if (i < total) *reinterpret_cast<u32x4*>(cache + (size_t)i * 16) = piece[j];
            }
        }
        for (int i = threadIdx.x; i < pieces; i += blockDim.x)
            *reinterpret_cast<u32x4*>(cache + (size_t)c_rows * row_bytes + i * 16) = u32x4{0u, 0u, 0u, 0u};
        __syncthreads();
    }

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int lpr_log2 = __builtin_ctz(a.plan.lanes_per_row);
    const int U = a.plan.units_per_wave;
    const int g = lane >> lpr_log2;                 // unit slot of this lane
    const int c = lane & (a.plan.lanes_per_row - 1);  // position inside the row
    Entry* stage = stage_all + wave * (U * kChunkStride);
    // softmax statistics of the units of this wavefront (fused form): {max, sum of exp}
    float* stats = reinterpret_cast<float*>(stage_all + a.plan.waves_per_block * (U * kChunkStride)) + wave * (2 * U);
    const T* ref = static_cast<const T*>(a.ref);

    const T* attn = static_cast<const T*>(a.attn);
    T* out = static_cast<T*>(a.out);
    const __amdgpu_buffer_rsrc_t vres =
        make_rsrc(static_cast<const char*>(a.value) + (size_t)wk.b * a.batch_bytes, a.batch_bytes);
    const uint32_t head_off = (uint32_t)wk.h * a.hd * sizeof(T);

    // channel offsets of this lane for each row pass; lanes past the end of the row read
    // channel 0 and never store
    uint32_t choff[NPASS];
    bool chan_ok[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
        const int ch = (c + p * a.plan.lanes_per_row) * VEC;
        chan_ok[p] = ch < a.hd;
        choff[p] = head_off + (chan_ok[p] ? ch * (uint32_t)sizeof(T) : 0u);
    }
    // same lane offsets inside a cached row
    uint32_t lds_choff[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p) lds_choff[p] = choff[p] - head_off;

    const int entries = U * kChunk;  // staged samples per pass

    // A sample as it is read from memory, and its way into the staging strip.
    struct RawSample {
        float x, y, aw;
        int l, u;
        bool active;
    };
    auto fetch = [&](int q0, int c0, int i) -> RawSample {
        RawSample r;
        r.u = i >> 4;
        const int sl = i & (kChunk - 1);
        const int s = c0 + sl, q = q0 + r.u;
        r.active = (i < entries) && (q < wk.q_end) && (s < a.S);
        r.x = 0.f, r.y = 0.f, r.aw = 0.f, r.l = 0;
        if (r.active) {
            const SampleRef sr = sample_ref<SRC>(a, wk.b, q, wk.h, s);
            r.x = load_coord<SRC, T>(a.loc, 2 * sr.loc_e);
            r.y = load_coord<SRC, T>(a.loc, 2 * sr.loc_e + 1);
            if constexpr (SRC == kSrcGrid) r.aw = 1.0f;  // no weights tensor
            else r.aw = to_f32(attn[sr.w_e]);
            r.l = sr.l;
            if constexpr (FUSED) {
                fused_location(a, ref + (((int64_t)wk.b * a.nq + q) * a.nl + r.l) * a.ref_dim, lvl[r.l], r.x, r.y);
                r.aw = expf(r.aw - stats[2 * r.u]) / stats[2 * r.u + 1];
            }
        }
        return r;
    };
    auto place = [&](const RawSample& r, int i) {
        const int sl = i & (kChunk - 1);
        // deformable aggregation samples only strictly inside the image (0 < x, y < 1)
        const bool inside = SRC != kSrcDagg || (r.x > 0.0f && r.x < 1.0f && r.y > 0.0f && r.y < 1.0f);
        const Sample sm = source_geometry<SRC>(r.x, r.y, lvl[r.l], a.nk, r.active && inside, a.grid);
        Entry en;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            en.off[k] = sm.cvalid[k] ? (uint32_t)sm.pix[k] * a.pitch_bytes : kInvalidCorner;
            en.w[k] = sm.valid ? sm.w[k] * r.aw : 0.0f;
            if constexpr (LDSC) {
                // cached level: byte offset of the row in the cache; the row of zeros for a corner
                // outside the image
                if (r.l >= c_first) en.off[k] = (uint32_t)(sm.cvalid[k] ? sm.pix[k] - c_base : c_rows) * row_bytes;
            }
        }
        stage[r.u * kChunkStride + sl] = en;
    };
    // AHEAD (one chunk of samples per unit, at most two samples per lane; chosen by the launcher): the samples of an
    // iteration are requested before the gather of the iteration before it, so their way from memory is covered by
    // that gather.  A template parameter, so that the other forms keep their registers.
    static_assert(!AHEAD || SRC == kSrcPlain, "look-ahead is built for the plain operator");
    constexpr bool ahead = AHEAD;
    RawSample nxt[2];
    if (ahead) {
        const int qf = wk.q_begin + wave * U;
        nxt[0] = fetch(qf, 0, lane);
        nxt[1] = fetch(qf, 0, lane + kWave);
    }
    for (int it = 0; it < a.plan.iters; ++it) {
        const int q0 = wk.q_begin + (it * a.plan.waves_per_block + wave) * U;
        if (q0 >= wk.q_end) break;  // wavefront-uniform; no workgroup barrier follows

        float acc[NPASS][VEC];
#pragma unroll
        for (int p = 0; p < NPASS; ++p)
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[p][v] = 0.0f;

        if constexpr (FUSED) {
            // softmax statistics: lanes 16u..16u+15 share unit u, each takes every 16th logit
            for (int i = lane; i < entries; i += kWave) {
                const int u = i >> 4, sl = i & (kChunk - 1), q = q0 + u;
                const T* lg = attn + (((int64_t)wk.b * a.nq + (q < wk.q_end ? q : wk.q_begin)) * a.nh + wk.h) * a.S_full;
                float m = -__builtin_inff();
                for (int s = sl; s < a.S; s += kChunk) m = __builtin_fmaxf(m, to_f32(lg[s]));
                m = group_max<4>(m);  // (kChunk = 16 lanes = one DPP row; rows are wholly active or inactive here)
                float sum = 0.0f;
                for (int s = sl; s < a.S; s += kChunk) sum += expf(to_f32(lg[s]) - m);
                sum = group_sum<4>(sum);
                if (sl == 0) {
                    stats[2 * u] = m;
                    stats[2 * u + 1] = sum;
                }
            }
            wave_lds_sync();
        }

        for (int c0 = 0; c0 < a.S; c0 += kChunk) {
            // ---- geometry: one sample per lane --------------------------------------------
            if (ahead) {
                if (lane < entries) place(nxt[0], lane);
                if (lane + kWave < entries) place(nxt[1], lane + kWave);
            } else {
                for (int i = lane; i < entries; i += kWave) place(fetch(q0, c0, i), i);
            }
            wave_lds_sync();
            if (ahead) {
                // the samples of this wavefront's next units are requested now and used after the gather
                const int qn = q0 + a.plan.waves_per_block * U;
                nxt[0] = fetch(qn, 0, lane);
                nxt[1] = fetch(qn, 0, lane + kWave);
            }

            // ---- gather + weighted sum ----------------------------------------------------
            const int ns = (a.S - c0) < kChunk ? (a.S - c0) : kChunk;
            const Entry* mine = stage + g * kChunkStride;
            // samples are level-major: those of the cached levels are the tail of the unit's list
            int n_mem = ns;
            if constexpr (LDSC) {
                n_mem = c_first * a.np - c0;
                n_mem = n_mem < 0 ? 0 : (n_mem > ns ? ns : n_mem);
            }
#pragma unroll 4
            for (int sl = 0; sl < n_mem; ++sl) {
                const u32x4 off = *reinterpret_cast<const u32x4*>(mine[sl].off);
                const f32x4 w = *reinterpret_cast<const f32x4*>(mine[sl].w);
#pragma unroll
                for (int p = 0; p < NPASS; ++p) {
                    typename RowIO<T, VEC>::raw_t raw[NC];
#pragma unroll
                    for (int k = 0; k < NC; ++k) raw[k] = RowIO<T, VEC>::load_raw(vres, off[k] + choff[p]);
#pragma unroll
                    for (int k = 0; k < NC; ++k) {
                        float v[VEC];
                        RowIO<T, VEC>::unpack(raw[k], v);
#pragma unroll
                        for (int e = 0; e < VEC; ++e) acc[p][e] = __builtin_fmaf(w[k], v[e], acc[p][e]);
                    }
                }
            }
            if constexpr (LDSC) {
#pragma unroll 4
                for (int sl = n_mem; sl < ns; ++sl) {
                    const u32x4 off = *reinterpret_cast<const u32x4*>(mine[sl].off);
                    const f32x4 w = *reinterpret_cast<const f32x4*>(mine[sl].w);
#pragma unroll
                    for (int p = 0; p < NPASS; ++p) {
                        typename RowIO<T, VEC>::raw_t raw[4];
#pragma unroll
                        for (int k = 0; k < 4; ++k)
                            raw[k] = *reinterpret_cast<const typename RowIO<T, VEC>::raw_t*>(cache + off[k] + lds_choff[p]);
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            float v[VEC];
                            RowIO<T, VEC>::unpack(raw[k], v);
#pragma unroll
                            for (int e = 0; e < VEC; ++e) acc[p][e] = __builtin_fmaf(w[k], v[e], acc[p][e]);
                        }
                    }
                }
            }
            wave_lds_sync();
        }

        const int q = q0 + g;
        if (q < wk.q_end) {
            T* orow = out + (((int64_t)wk.b * a.nq + q) * a.nh + wk.h) * a.hd;
#pragma unroll
            for (int p = 0; p < NPASS; ++p) {
                if (chan_ok[p]) RowIO<T, VEC>::store_global(orow + (c + p * a.plan.lanes_per_row) * VEC, acc[p]);
            }
        }
    }
}

template <typename T, int VEC, int NPASS>
static hipError_t launch_one(const KArgs& a, hipStream_t stream)
{
    const dim3 grid(a.plan.grid), block(a.plan.block);
    if (a.grid)
        hipLaunchKernelGGL((msda_fwd_kernel<T, VEC, NPASS, kSrcGrid, false>), grid, block, a.plan.lds_bytes, stream, a);
    else if (a.gka)
        hipLaunchKernelGGL((msda_fwd_kernel<T, VEC, NPASS, kSrcGka, false>), grid, block, a.plan.lds_bytes, stream, a);
    else if (a.cams > 0)
        hipLaunchKernelGGL((msda_fwd_kernel<T, VEC, NPASS, kSrcDagg, false>), grid, block, a.plan.lds_bytes, stream, a);
    else if (a.ref != nullptr)
        hipLaunchKernelGGL((msda_fwd_kernel<T, VEC, NPASS, kSrcFused, false>), grid, block, a.plan.lds_bytes, stream, a);
    else {
        // look-ahead form: one chunk of samples per unit and at most two samples per lane
        const bool ahead = a.fwd_ahead != 0 && a.S <= kChunk && a.plan.units_per_wave * kChunk <= 2 * kWave;
        if (a.lds_cache_bytes > 0) {
            // (more than the 64 KiB of dynamic LDS a kernel gets by default: raise_forward_lds() has opted in)
            if constexpr (VEC * sizeof(T) == 16) {
                if (ahead)
                    hipLaunchKernelGGL((msda_fwd_kernel<T, VEC, NPASS, kSrcPlain, true, true>), grid, block, a.plan.lds_bytes, stream, a);
                else
                    hipLaunchKernelGGL((msda_fwd_kernel<T, VEC, NPASS, kSrcPlain, true, false>), grid, block, a.plan.lds_bytes, stream, a);
            } else {
                return hipErrorInvalidConfiguration;
            }
        } else if (ahead)
            hipLaunchKernelGGL((msda_fwd_kernel<T, VEC, NPASS, kSrcPlain, false, true>), grid, block, a.plan.lds_bytes, stream, a);
        else
            hipLaunchKernelGGL((msda_fwd_kernel<T, VEC, NPASS, kSrcPlain, false, false>), grid, block, a.plan.lds_bytes, stream, a);
    }
    return hipGetLastError();
}

// The level-cache instantiations use up to 80 KiB of dynamic LDS: opt in, on the current device.
template <typename T, int VEC, int NPASS>
static hipError_t raise_one()
{
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&msda_fwd_kernel<T, VEC, NPASS, kSrcPlain, true, false>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&msda_fwd_kernel<T, VEC, NPASS, kSrcPlain, true, true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024);
    return e;
}

hipError_t raise_forward_lds()
{
    hipError_t e = raise_one<float, 4, 1>();
    if (e == hipSuccess) e = raise_one<f16_t, 8, 1>();
    if (e == hipSuccess) e = raise_one<bf16_t, 8, 1>();
    return e;
}

template <typename T>
static hipError_t launch_dtype(const KArgs& a, hipStream_t stream)
{
    const int vec = a.plan.vec, np = a.plan.npass;
    if (vec == 1 && np == 1) return launch_one<T, 1, 1>(a, stream);
    if (vec == 1 && np == 2) return launch_one<T, 1, 2>(a, stream);
    if (vec == 1 && np == 4) return launch_one<T, 1, 4>(a, stream);
    if (vec == 2 && np == 1) return launch_one<T, 2, 1>(a, stream);
    if (vec == 2 && np == 2) return launch_one<T, 2, 2>(a, stream);
    if (vec == 4 && np == 1) return launch_one<T, 4, 1>(a, stream);
    if constexpr (sizeof(T) == 2) {
        if (vec == 8 && np == 1) return launch_one<T, 8, 1>(a, stream);
    }
    return hipErrorInvalidConfiguration;
}

hipError_t launch_forward(int dtype, const KArgs& a, hipStream_t stream)
{
    switch (dtype) {
        case MXD_DTYPE_F32: return launch_dtype<float>(a, stream);
        case MXD_DTYPE_F16: return launch_dtype<f16_t>(a, stream);
        case MXD_DTYPE_BF16: return launch_dtype<bf16_t>(a, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace mxd
