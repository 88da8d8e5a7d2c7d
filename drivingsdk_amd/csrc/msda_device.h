// Device-side helpers shared by the forward and backward kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "msda_plan.h"

namespace mxd {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));

typedef _Float16 f16_t;
typedef __bf16 bf16_t;

// Kernel arguments (passed by value).
struct KArgs {
    const void* value;
    const int32_t* shapes;
    const int32_t* lsi;
    int32_t meta_i64;      // 1: shapes / lsi are arrays of int64 (MXD_META_I64)
    const void* loc;
    const void* attn;
    void* out;             // forward output
    // fused forward only: `loc` holds sampling offsets, `attn` holds logits (softmax over nl*np inside
    // the kernel), and the sampling location is reference point + offset / normaliser
    const void* ref;       // [bs, nq, nl, ref_dim] reference points
    int32_t ref_dim;       // 2: (x, y); 4: (x, y, w, h) boxes
    // deformable aggregation only (source = kSrcDagg): a level is a (camera, scale) pair, nl = cams*scales,
    // np = points per anchor, sample s = point*nl + level; `loc` is [bs, nq, np, cams, 2] (shared by the
    // scales of a camera and by all heads = channel groups), `attn` is [bs, nq, np, cams, scales, nh]
    int32_t cams;
    int32_t scales;
    uint32_t sc_magic;     // ceil(2^20/scales): level / scales
    int32_t lds_cache_bytes;  // forward: LDS set aside for the rows of the last (coarsest) levels, 0 = none
    int32_t fwd_ahead;        // forward: request an iteration's samples before the gather of the one before it
    int32_t fwd_cu_flip;      // forward, one workgroup per CU: half of the wavefronts take their LDS groups first
    int32_t grid_h, grid_w;  // grid sampler: the one level's shape comes with the call, not from device memory
    int32_t grid;          // grid sampler: 1 + padding mode (0 zeros, 1 border) + 2*align_corners; 0 = not a grid sampler
    int32_t gka;           // geometric kernel attention: locations are pixel indices, one pixel per sample
    int32_t sc_pow2;       // scales is a power of two that divides 16: location gradients are summed over the
                           // scales across lanes and stored once; otherwise they are added with atomics
    const void* grad_out;  // backward only from here
    float* grad_value;     // fp32 accumulation image of grad_value
    uint64_t fill_n4;      // first backward kernel, tile mode: 16-byte pieces of the image its workgroups zero-fill
                           // between them (the image is first touched by the tile pass); 0 = filled by a kernel before
    void* grad_loc;
    void* grad_attn;
    // fused form, backward: `out` holds the forward result (the softmax backward needs, per (query, head), the
    // dot product of its row with the grad_out row); grad_loc / grad_attn receive the gradients of the offsets
    // and of the logits; the reference points' gradient is summed over points here and over heads afterwards
    float* grad_ref;       // [nh][bs, nq, nl, ref_dim] float32 per-head partial sums, or nullptr: not wanted
    int32_t np_pow2;       // np is a power of two that divides 16: the point sum is taken across lanes and
                           // stored once; otherwise added with atomics into the zero-filled partial sums
    // Hand-over from the first backward kernel to the grad_value pass.  Every workgroup of the
    // first kernel (tile_q queries of one (batch, head)) owns a slab of rec_cap pair records,
    // which it fills sorted by tile; row [w] of the table holds the start of every tile's run
    // inside slab w (tbl_stride entries, the last used one being the total).
    // record (12 bytes) = {pixel within its tile | query within the workgroup << tile_px_log2, weight of that pixel,
    //                      weight of the pixel to its right}
    uint32_t* rec;         // [bs*nh][nwg][rec_cap] records of kRecDwords dwords
    uint32_t* tbl;         // [bs*nh][nwg][tbl_stride]
    int32_t nwg;           // workgroups of the first kernel per (batch, head)
    int32_t rec_cap;       // 2 * tile_q * nl * np
    int32_t tbl_stride;    // upper bound of tiles per (batch, head), plus one
    int32_t tile_px_log2;  // log2 of the pixels per tile of the grad_value pass (9, 8 or 7: see msda_plan.h)
    int32_t rec_lds_bytes; // first backward kernel: LDS behind its counters (16-byte aligned) in which a workgroup that makes
                           // several passes collects its slab before it writes it; 0 = none (records stored one by one)
    int32_t bwd_fixed;     // first backward kernel, plain operator's tile form: 1, 2 = the launch has the common geometry (rows read
                           // by 8 lanes, one iteration of one chunk, this many units per query), 3 = rows of 256 bytes read by 16
                           // lanes of 16 bytes, a unit per query: it takes the instantiation built for that geometry
    int32_t tile_target;   // pair records per work item of the tile pass aimed at when a hot tile is split by query range
    int32_t tile_max_chunks;  // most query chunks a tile is split into
    int32_t sparse;        // 1: only the rows of the image that receive atomic additions are zero-filled (and, for 16-bit
                           // dtypes, rounded afterwards): the other rows are stored once by the tile's owner
    void* grad_value_t;    // 16-bit dtypes with sparse = 1: the caller's grad_value, which receives those stores
    int32_t unit_split_log2;  // backward's first kernel: 2^this units of a wavefront share a query, each taking kChunk of
                           // its samples (unit u: query u >> this, samples ((u & (2^this - 1)) * kChunk ...); then
                           // plan.tile_q = units per workgroup >> this
    int32_t bs, nk, nh, hd, nl, np, nq;
    int32_t S;             // nl*np: samples per unit that are evaluated
    int32_t S_full;        // nl_attn*np: samples per unit that are stored
    uint32_t np_magic;     // ceil(2^20/np): s/np == (s*np_magic)>>20 while s*np < 2^20
    uint32_t pitch_bytes;  // nh*hd*sizeof(T): distance between neighbouring pixels of value
    uint32_t batch_bytes;  // nk*pitch_bytes
    uint32_t gbatch_bytes; // nk*nh*hd*4: one batch element of the fp32 grad image
    mxd_msda_plan plan;
};

// Level l as {H, W, level_start_index, 0}.
__device__ inline i32x4 load_level(const KArgs& a, int l)
{
    if (a.grid) return i32x4{a.grid_h, a.grid_w, 0, 0};
    // (int64 metadata: the low words of little-endian elements, two int32 apart)
    const int sh = a.meta_i64;
    return i32x4{a.shapes[(2 * l) << sh], a.shapes[(2 * l + 1) << sh], a.lsi[l << sh], 0};
}

// ---- tiles of the grad_value pass, as every kernel of the backward sees them ---------------------------------------
constexpr int kRecDwords = 3;  // dwords of a pair record
constexpr int kLpp = 8;        // lanes of a lane group of the tile pass (a group reads a row with one load per 32 channels)
constexpr int kRowParts = 16;  // pieces a tile's rows are cut into for the zero-fill and the rounding

// Pixels per lane group of the tile pass: 8 for tiles of 512 pixels, 4 for 256, 2 for 128 (64 groups per workgroup).
__device__ inline int32_t tile_group_px(int32_t tile_px_log2) { return 1 << (tile_px_log2 - 6); }

// Query chunks the tiles of a level with `nt` tiles are split into by the tile pass; *wpc: workgroups of the first
// kernel per chunk.
__device__ inline int32_t level_tile_chunks(const KArgs& a, int32_t nt, int32_t* wpc)
{
    // two pair records per sample, spread evenly over the tiles of the level
    // (32-bit divisions wherever the operands allow: a 64-bit one is some 150 instructions, and the workgroups of all
    //  three backward kernels go through this before they start)
    const uint64_t records = 2 * (uint64_t)a.nq * (uint64_t)a.np;
    const uint64_t expect = records <= 0xFFFFFFFFull ? (uint64_t)((uint32_t)records / (uint32_t)nt) : records / (uint64_t)nt;
    const uint32_t target = (uint32_t)a.tile_target;
    // (more chunks than the limit are cut down to it: the quotient itself is not needed then)
    uint32_t chunks;
    if (expect >= (uint64_t)target * (uint32_t)a.tile_max_chunks) chunks = (uint32_t)a.tile_max_chunks;
    else if (expect <= 0xFFFFFFFFull - target) chunks = ((uint32_t)expect + target - 1) / target;
    else chunks = (uint32_t)((expect + target - 1) / target);
    if (chunks < 1) chunks = 1;
    if (chunks > (uint32_t)a.tile_max_chunks) chunks = (uint32_t)a.tile_max_chunks;
    if (chunks > (uint32_t)a.nwg) chunks = (uint32_t)a.nwg;
    const uint32_t w = ((uint32_t)a.nwg + chunks - 1) / chunks;
    *wpc = (int32_t)w;
    return (int32_t)(((uint32_t)a.nwg + w - 1) / w);
}

// A tile of `npx` pixels whose rows its one workgroup of the tile pass stores directly: no other workgroup adds to
// them (the tile is not split by query range and is too full to be held in copies or to have slots left for extra
// lists), except to the tile's first pixel, which also receives the right halves of pairs that start on the last
// pixel of the tile before it.
__device__ inline bool tile_stored_directly(int32_t chunks, int32_t npx, int32_t tile_px_log2)
{
    const int32_t g = tile_group_px(tile_px_log2);
    return chunks == 1 && (1 << tile_px_log2) - ((npx + g - 1) / g * g) < g;
}

// Whether the levels tile the keys exactly and in order -- the first level starts at key 0, every other one where the
// one before it ends, the last one ends at key nk -- and all their tiles fit the run table.  Only then is every row of
// grad_value covered by exactly one tile, which is what lets the owner of a tile store its rows (instead of adding to
// them) and lets the rows that nobody adds to go without zeros.  level_start_index is the caller's: for any other
// layout (keys that no level covers, levels out of order or overlapping) every row is zero-filled and every tile adds
// its sums with atomics.
// (level(l): {H, W, first key} of level l, from wherever the caller holds it)
template <typename GetLevel>
__device__ inline bool levels_tile_the_keys_of(const KArgs& a, GetLevel level)
{
    int64_t next = 0;
    int32_t tiles = 0;
    for (int l = 0; l < a.nl; ++l) {
        const i32x4 L = level(l);
        if (L.x <= 0 || L.y <= 0 || (int64_t)L.z != next) return false;
        const int64_t px = (int64_t)L.x * L.y;
        next += px;
        if (next > a.nk) return false;
        tiles += (int32_t)((px + ((int64_t)1 << a.tile_px_log2) - 1) >> a.tile_px_log2);
    }
    return next == a.nk && tiles <= a.tbl_stride - 1;
}
__device__ inline bool levels_tile_the_keys(const KArgs& a)
{
    return levels_tile_the_keys_of(a, [&](int l) { return load_level(a, l); });
}

// Rows (pixels of a batch element) [*r0, *r1) of piece `part` (< kRowParts) of tile `tile` of a batch element that
// receive atomic additions in the tile pass; false when there is no such tile.  Tiles are numbered level by level as
// in the first kernel and the tile pass.
template <typename GetLevel>
__device__ inline bool atomic_rows_of_part_of(const KArgs& a, GetLevel level, int32_t tile, int32_t part, int32_t* r0, int32_t* r1)
{
    int32_t first = 0;
    for (int l = 0; l < a.nl; ++l) {
        const i32x4 L = level(l);
        int32_t P;
        const int32_t nt = level_tile_count(L.x, L.y, L.z, a.nk, a.tile_px_log2, &P);
        if (first + nt > a.tbl_stride - 1) continue;  // (a level that does not fit the run table has no tiles)
        if (tile < first + nt) {
            const int32_t ti = tile - first, tile_px = 1 << a.tile_px_log2;
            const int32_t p0 = L.z + ti * tile_px;
            const int32_t npx = (P - ti * tile_px) < tile_px ? (P - ti * tile_px) : tile_px;
            int32_t wpc;
            if (tile_stored_directly(level_tile_chunks(a, nt, &wpc), npx, a.tile_px_log2)) {
                *r0 = p0;
                *r1 = part == 0 ? p0 + 1 : p0;
            } else {
                const int per = tile_px / kRowParts;
                *r0 = p0 + (part * per < npx ? part * per : npx);
                *r1 = p0 + ((part + 1) * per < npx ? (part + 1) * per : npx);
            }
            return true;
        }
        first += nt;
    }
    return false;
}
__device__ inline bool atomic_rows_of_part(const KArgs& a, int32_t tile, int32_t part, int32_t* r0, int32_t* r1)
{
    return atomic_rows_of_part_of(a, [&](int l) { return load_level(a, l); }, tile, part, r0, r1);
}

// Where a kernel takes the location and the weight of sample s of unit (b, q, h) from.
enum : int { kSrcPlain = 0, kSrcFused = 1, kSrcDagg = 2, kSrcGka = 3, kSrcGrid = 4 };
struct SampleRef {
    int64_t loc_e;  // index of the (x, y) pair
    int64_t w_e;    // index of the weight
    int32_t l;      // level
};
template <int SRC>
__device__ inline SampleRef sample_ref(const KArgs& a, int b, int q, int h, int s)
{
    SampleRef r;
    if constexpr (SRC == kSrcDagg) {
        const int p = (int)(((uint32_t)s * a.np_magic) >> 20);  // s / nl (np_magic is built for the divisor nl here)
        r.l = s - p * a.nl;
        const int cam = (int)(((uint32_t)r.l * a.sc_magic) >> 20);
        r.loc_e = (((int64_t)b * a.nq + q) * a.np + p) * a.cams + cam;
        r.w_e = (((int64_t)b * a.nq + q) * a.S + s) * a.nh + h;
    } else {
        r.loc_e = r.w_e = (((int64_t)b * a.nq + q) * a.nh + h) * a.S_full + s;
        r.l = (int)(((uint32_t)s * a.np_magic) >> 20);
    }
    return r;
}

// Launch description of the tile-ownership grad_value kernel.
constexpr int kTileEntCap = 576;  // list entries (16 bytes) per wavefront and round
struct TileArgs {
    mxd_msda_plan map;     // only the XCD mapping fields are used: one "query" per work item
    int32_t target;        // pair records per work item aimed at when a hot tile is split by query range
    int32_t max_chunks;    // most query chunks a tile is split into
    int32_t items_per_bh;  // upper bound of work items per (batch, head), including `extra`
    int32_t extra;         // workgroups per (batch, head) behind the work items that add the samples of levels whose tiles
                           // found no room in the run table (plain operator only; they leave at once otherwise)
    int32_t vec;           // elements per load of a grad_out row
    int32_t accumulate;    // add into the existing contents of the image
    int32_t store_vec;     // 4: rows of the image are 16-byte aligned, else 1
    int32_t batch_major;   // 1: the work items of a batch element are numbered together (an XCD's L2 then holds one
                           // batch element's grad_out rows at a time); 0: item-major across batch elements
    uint32_t grid, block;
};

// One staged sample: byte offsets of its four corner rows inside the batch element's value
// slice (kInvalidCorner when the corner must not be touched) and their weights.
struct __align__(16) Entry {
    uint32_t off[4];
    float w[4];
};

// Any offset >= 2^31 is outside every buffer this library binds (slices are < 2 GiB), so the
// hardware range check turns such loads into zeros and drops such atomics.  0xC0000000
// stays out of range when shifted left by one (16-bit value offset -> fp32 grad offset) and
// when a channel offset (< 64 KiB) is added.
constexpr uint32_t kInvalidCorner = 0xC0000000u;

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes)
{
    // word3 0x00020000: raw buffer, 32-bit data format, no swizzle (gfx9 family encoding)
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

// Orders this wavefront's LDS writes before its later LDS reads (and vice versa) without a
// workgroup barrier: LDS operations of one wavefront complete in order, so it is enough to
// stop the compiler from moving them across this point.
__device__ inline void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <typename T>
__device__ inline float to_f32(T v)
{
    return (float)v;
}
template <typename T>
__device__ inline T from_f32(float v)
{
    return (T)v;
}

// acc + a.lo * b.lo + a.hi * b.hi for two packed pairs of 16-bit elements, the products and the sum in float32.
template <typename T>
__device__ inline float dot2_acc(uint32_t a, uint32_t b, float acc)
{
    static_assert(sizeof(T) == 2, "packed pairs of 16-bit elements");
    typedef T t2 __attribute__((ext_vector_type(2)));
    if constexpr (std::is_same<T, f16_t>::value)
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(t2, a), __builtin_bit_cast(t2, b), acc, false);
    else
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(t2, a), __builtin_bit_cast(t2, b), acc, false);
}

// One coordinate of a sampling location.  Geometric kernel attention carries pixel indices: they are float32 whatever
// the element type of value is (a 16-bit float cannot hold the indices of a level wider than 2048 / 256 pixels).
template <int SRC, typename T>
__device__ inline float load_coord(const void* loc, int64_t i)
{
    if constexpr (SRC == kSrcGka) return static_cast<const float*>(loc)[i];
    else return to_f32(static_cast<const T*>(loc)[i]);
}

// Fused form: sampling location from the raw offset (x, y) of a sample on level `lv` = {H, W, ..}.
// rp: the query's reference point on that level, (cx, cy) or a box (cx, cy, w, h).
//   points: location = reference + offset / (W, H)          boxes: location = centre + offset / np * (w, h) / 2
template <typename T>
__device__ inline void fused_location(const KArgs& a, const T* rp, const i32x4 lv, float& x, float& y)
{
    // every operation rounded on its own, wherever this is inlined: the backward derives the location of a
    // sample in several places (counting records, staging, gradients) and all of them must land on the same
    // pixel, as must the forward
#pragma clang fp contract(off)
    if (a.ref_dim == 2) {
        x = to_f32(rp[0]) + x / (float)lv.y;
        y = to_f32(rp[1]) + y / (float)lv.x;
    } else {
        x = to_f32(rp[0]) + x / (float)a.np * to_f32(rp[2]) * 0.5f;
        y = to_f32(rp[1]) + y / (float)a.np * to_f32(rp[3]) * 0.5f;
    }
}

// ---- row access: VEC elements of T at a byte offset of a bound buffer -> fp32 -------------
template <typename T, int VEC>
struct RowIO;

template <typename T, int VEC, int BYTES = VEC * (int)sizeof(T)>
struct RawBits;
template <typename T, int VEC>
struct RawBits<T, VEC, 16> {
    typedef u32x4 type;
    static __device__ inline type load(__amdgpu_buffer_rsrc_t r, uint32_t off)
    {
        return __builtin_bit_cast(type, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0));
    }
};
template <typename T, int VEC>
struct RawBits<T, VEC, 8> {
    typedef u32x2 type;
    static __device__ inline type load(__amdgpu_buffer_rsrc_t r, uint32_t off)
    {
        return __builtin_bit_cast(type, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0));
    }
};
template <typename T, int VEC>
struct RawBits<T, VEC, 4> {
    typedef uint32_t type;
    static __device__ inline type load(__amdgpu_buffer_rsrc_t r, uint32_t off)
    {
        return __builtin_bit_cast(type, __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0));
    }
};
template <typename T, int VEC>
struct RawBits<T, VEC, 2> {
    typedef uint16_t type;
    static __device__ inline type load(__amdgpu_buffer_rsrc_t r, uint32_t off)
    {
        return __builtin_bit_cast(type, __builtin_amdgcn_raw_buffer_load_b16(r, off, 0, 0));
    }
};

template <typename T, int VEC>
struct RowIO {
    typedef T vec_t __attribute__((ext_vector_type(VEC)));
    typedef typename RawBits<T, VEC>::type raw_t;

    static __device__ inline raw_t load_raw(__amdgpu_buffer_rsrc_t r, uint32_t off)
    {
        return RawBits<T, VEC>::load(r, off);
    }
    static __device__ inline void unpack(raw_t raw, float (&v)[VEC])
    {
        if constexpr (VEC == 1) {
            v[0] = to_f32(__builtin_bit_cast(T, raw));
        } else {
            const vec_t t = __builtin_bit_cast(vec_t, raw);
#pragma unroll
            for (int i = 0; i < VEC; ++i) v[i] = to_f32<T>(t[i]);
        }
    }
    // p must be aligned to VEC*sizeof(T)
    static __device__ inline void load_global(const T* p, float (&v)[VEC])
    {
        if constexpr (VEC == 1) {
            v[0] = to_f32(*p);
        } else {
            const vec_t t = *reinterpret_cast<const vec_t*>(p);
#pragma unroll
            for (int i = 0; i < VEC; ++i) v[i] = to_f32<T>(t[i]);
        }
    }
    static __device__ inline void store_global(T* p, const float (&v)[VEC])
    {
        // (non-temporal: results are not read again by this kernel and should not push value rows out of L2)
        if constexpr (VEC == 1) {
            __builtin_nontemporal_store(from_f32<T>(v[0]), p);
        } else {
            vec_t t;
#pragma unroll
            for (int i = 0; i < VEC; ++i) t[i] = from_f32<T>(v[i]);
            __builtin_nontemporal_store(t, reinterpret_cast<vec_t*>(p));
        }
    }
};

// ---- per-sample geometry ----------------------------------------------------------------
struct Sample {
    int32_t pix[4];  // pixel index (within the batch element) of corners (y0,x0) (y0,x1) (y1,x0) (y1,x1)
    bool cvalid[4];  // corner lies inside the level and inside [0, nk)
    float w[4];      // bilinear weights, all zero when the sample is invalid
    float lw, lh;    // fractional parts
    float Wf, Hf;
    bool valid;      // sample lies inside (-1, W) x (-1, H) in pixel space; false for NaN/Inf
};

// Bilinear corner weights from the fractions, in the corner order of Sample.
__device__ inline void bilinear_weights(float lw, float lh, float (&w)[4])
{
#pragma clang fp contract(off)
    const float hw = 1.0f - lw, hh = 1.0f - lh;
    w[0] = hh * hw;
    w[1] = hh * lw;
    w[2] = lh * hw;
    w[3] = lh * lw;
}

// level = {H, W, level_start_index, unused}
__device__ inline Sample sample_geometry(float x, float y, i32x4 level, int32_t nk, bool active)
{
#pragma clang fp contract(off)  // the hi/lo split below must not be re-fused by the compiler
    Sample s;
    const int32_t H = level.x, W = level.y, base = level.z;
    s.Wf = (float)W;
    s.Hf = (float)H;
    // Correctly rounded pixel coordinates decide validity ...
    const float w_im = __builtin_fmaf(x, s.Wf, -0.5f);
    const float h_im = __builtin_fmaf(y, s.Hf, -0.5f);
    s.valid = active && (h_im > -1.0f) && (w_im > -1.0f) && (h_im < s.Hf) && (w_im < s.Wf);
    // ... while cell index and fraction come from the exact product x*W = hi + lo, so that the
    // fraction carries an absolute error of ~2^-24 instead of half an ulp of the coordinate
    // (which at W = 150 would already be 4e-6 of a pixel).
    const float xh = x * s.Wf, xl = __builtin_fmaf(x, s.Wf, -xh);
    const float yh = y * s.Hf, yl = __builtin_fmaf(y, s.Hf, -yh);
    const float tx = xh - 0.5f, ty = yh - 0.5f;
    float fx = __builtin_floorf(tx), fy = __builtin_floorf(ty);
    s.lw = (tx - fx) + xl;
    s.lh = (ty - fy) + yl;
    if (s.lw < 0.0f) { fx -= 1.0f; s.lw += 1.0f; }
    if (s.lw >= 1.0f) { fx += 1.0f; s.lw -= 1.0f; }
    if (s.lh < 0.0f) { fy -= 1.0f; s.lh += 1.0f; }
    if (s.lh >= 1.0f) { fy += 1.0f; s.lh -= 1.0f; }
    const int32_t x0 = s.valid ? (int32_t)fx : 0;
    const int32_t y0 = s.valid ? (int32_t)fy : 0;
    // two-sided (unsigned) tests: after the fraction fix-up a cell index may sit one step
    // outside [-1, size-1] for coordinates within an ulp of a validity edge
    const bool vx0 = (uint32_t)x0 < (uint32_t)W, vx1 = (uint32_t)(x0 + 1) < (uint32_t)W;
    const bool vy0 = (uint32_t)y0 < (uint32_t)H, vy1 = (uint32_t)(y0 + 1) < (uint32_t)H;
    const int32_t p00 = base + y0 * W + x0;
    s.pix[0] = p00;
    s.pix[1] = p00 + 1;
    s.pix[2] = p00 + W;
    s.pix[3] = p00 + W + 1;
    const bool cv[4] = {vy0 && vx0, vy0 && vx1, vy1 && vx0, vy1 && vx1};
    float wt[4];
    bilinear_weights(s.lw, s.lh, wt);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        s.cvalid[k] = s.valid && cv[k] && ((uint32_t)s.pix[k] < (uint32_t)nk);
        s.w[k] = s.valid ? wt[k] : 0.0f;
    }
    return s;
}

// Geometric kernel attention (reference: mx_driving/ops/geometric_kernel_attention.py,
// kernels/geometric_kernel_attention/op_kernel/geometric_kernel_attention.cpp:150-160): the location is a
// pixel index pair (x, y), clamped to the level; the sample is that one pixel with weight 1, no interpolation.
__device__ inline Sample gka_geometry(float x, float y, i32x4 level, int32_t nk, bool active)
{
    Sample s;
    const int32_t H = level.x, W = level.y, base = level.z;
    s.Wf = (float)W;
    s.Hf = (float)H;
    s.lw = s.lh = 0.0f;
    s.valid = active && H > 0 && W > 0 && x == x && y == y;  // NaN locations contribute nothing
    int32_t xi = s.valid ? (int32_t)__builtin_fminf(__builtin_fmaxf(x, -1.0f), 2147483520.0f) : 0;
    int32_t yi = s.valid ? (int32_t)__builtin_fminf(__builtin_fmaxf(y, -1.0f), 2147483520.0f) : 0;
    xi = xi < 0 ? 0 : (xi > W - 1 ? W - 1 : xi);
    yi = yi < 0 ? 0 : (yi > H - 1 ? H - 1 : yi);
    const int32_t p = base + yi * W + xi;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        s.pix[k] = p + k;  // corners 1..3 are never valid
        s.cvalid[k] = false;
        s.w[k] = 0.0f;
    }
    s.cvalid[0] = s.valid && ((uint32_t)p < (uint32_t)nk);
    s.w[0] = s.valid ? 1.0f : 0.0f;
    return s;
}

// 2-D grid sampler, bilinear (reference: mx_driving/ops/grid_sampler2d_v2.py; the arithmetic is that of
// torch.nn.functional.grid_sample, which the reference's test uses as its golden): the location is a grid coordinate in
// [-1, 1], mapped to pixels by ((g+1)/2)*(size-1) with align_corners and ((g+1)*size-1)/2 without, clipped to
// [0, size-1] for border padding (the gradient is zero where it clips); Wf / Hf carry d(pixel)/d(grid).
__device__ inline Sample grid_geometry(float gx, float gy, i32x4 level, int32_t nk, bool active, int mode)
{
#pragma clang fp contract(off)
    Sample s;
    const int32_t H = level.x, W = level.y, base = level.z;
    const bool border = (mode - 1) & 1, align = (mode - 1) & 2;
    float ix, iy;
    if (align) {
        ix = ((gx + 1.0f) / 2.0f) * (float)(W - 1);
        iy = ((gy + 1.0f) / 2.0f) * (float)(H - 1);
        s.Wf = (float)(W - 1) / 2.0f;
        s.Hf = (float)(H - 1) / 2.0f;
    } else {
        ix = ((gx + 1.0f) * (float)W - 1.0f) / 2.0f;
        iy = ((gy + 1.0f) * (float)H - 1.0f) / 2.0f;
        s.Wf = (float)W / 2.0f;
        s.Hf = (float)H / 2.0f;
    }
    if (border) {
        if (ix <= 0.0f) { ix = 0.0f; s.Wf = 0.0f; } else if (ix >= (float)(W - 1)) { ix = (float)(W - 1); s.Wf = 0.0f; }
        if (iy <= 0.0f) { iy = 0.0f; s.Hf = 0.0f; } else if (iy >= (float)(H - 1)) { iy = (float)(H - 1); s.Hf = 0.0f; }
    }
    s.valid = active && (ix > -1.0f) && (iy > -1.0f) && (ix < (float)W) && (iy < (float)H);  // false for NaN
    const float fx = __builtin_floorf(ix), fy = __builtin_floorf(iy);
    s.lw = ix - fx;
    s.lh = iy - fy;
    const int32_t x0 = s.valid ? (int32_t)fx : 0, y0 = s.valid ? (int32_t)fy : 0;
    const bool vx0 = (uint32_t)x0 < (uint32_t)W, vx1 = (uint32_t)(x0 + 1) < (uint32_t)W;
    const bool vy0 = (uint32_t)y0 < (uint32_t)H, vy1 = (uint32_t)(y0 + 1) < (uint32_t)H;
    const int32_t p00 = base + y0 * W + x0;
    s.pix[0] = p00;
    s.pix[1] = p00 + 1;
    s.pix[2] = p00 + W;
    s.pix[3] = p00 + W + 1;
    const bool cv[4] = {vy0 && vx0, vy0 && vx1, vy1 && vx0, vy1 && vx1};
    float wt[4];
    bilinear_weights(s.lw, s.lh, wt);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        s.cvalid[k] = s.valid && cv[k] && ((uint32_t)s.pix[k] < (uint32_t)nk);
        s.w[k] = s.valid ? wt[k] : 0.0f;
    }
    return s;
}

template <int SRC>
__device__ inline Sample source_geometry(float x, float y, i32x4 level, int32_t nk, bool active, int grid_mode = 0)
{
    if constexpr (SRC == kSrcGrid) return grid_geometry(x, y, level, nk, active, grid_mode);
    if constexpr (SRC == kSrcGka) return gka_geometry(x, y, level, nk, active);
    else return sample_geometry(x, y, level, nk, active);
}

// ---- sum over the `lanes` (power of two <= 64) lanes that share a unit; every lane of the
// group ends with the total.  Uses DPP within 16-lane rows and lane swaps above.
template <int CTRL>
__device__ inline float dpp_xchg(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

template <int LANES_LOG2>
__device__ inline float group_sum(float v)
{
    // quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror
    if constexpr (LANES_LOG2 >= 1) v += dpp_xchg<0xB1>(v);
    if constexpr (LANES_LOG2 >= 2) v += dpp_xchg<0x4E>(v);
    if constexpr (LANES_LOG2 >= 3) v += dpp_xchg<0x141>(v);
    if constexpr (LANES_LOG2 >= 4) v += dpp_xchg<0x140>(v);
    if constexpr (LANES_LOG2 >= 5) v += __shfl_xor(v, 16, 64);
    if constexpr (LANES_LOG2 >= 6) v += __shfl_xor(v, 32, 64);
    return v;
}

// Pair records of one query that start on the same pixel are handed over as one record with the weights added
// up.  The points of one level of one query sit in neighbouring lanes, and on the coarse levels they often share
// their cell or sit in cells above one another, so the search is confined to the aligned group of 4 lanes this
// lane belongs to.  Every lane brings two records -- [0] for the upper corners of its sample, [1] for the lower
// ones -- and among the records with the same pixel the upper record of the lowest lane that has one keeps it
// (failing that, the lower record of the lowest lane); keep[] says which of this lane's records survive, and
// wa / wb of a surviving record carry the sums.  All four lanes of a group must make the call together; a lane
// without a record passes have = false.  `key` is a record's pixel index (>= 0); the lanes of a group belong to
// one query.
__device__ inline void merge_pair_records_in_quad(const bool (&have)[2], const int32_t (&key)[2], float (&wa)[2],
                                                  float (&wb)[2], bool (&keep)[2])
{
    const int j = (int)threadIdx.x & 3;  // lane within the group (workgroups are whole wavefronts)
    // a record that is not there gets a key no other record of the group has: equal keys then mean two records
    const int32_t k0 = have[0] ? key[0] : -1 - 2 * j, k1 = have[1] ? key[1] : -2 - 2 * j;
    bool keep0 = have[0], keep1 = have[1];
    const float wa0 = wa[0], wb0 = wb[0], wa1 = wa[1], wb1 = wb[1];
    float a0 = wa0, b0 = wb0, a1 = wa1, b1 = wb1;
    // quad_perm [1,2,3,0], [2,3,0,1], [3,0,1,2]: lane j reads lane (j + r) mod 4
    auto look = [&](auto ctrl, int r) {
        constexpr int CTRL = decltype(ctrl)::value;
        const int32_t o0 = __builtin_amdgcn_update_dpp(0, k0, CTRL, 0xF, 0xF, true);
        const int32_t o1 = __builtin_amdgcn_update_dpp(0, k1, CTRL, 0xF, 0xF, true);
        const float oa0 = dpp_xchg<CTRL>(wa0), ob0 = dpp_xchg<CTRL>(wb0);
        const float oa1 = dpp_xchg<CTRL>(wa1), ob1 = dpp_xchg<CTRL>(wb1);
        const bool lower = ((j + r) & 3) < j;  // the lane looked at comes before this one
        const bool m00 = o0 == k0, m10 = o1 == k0, m01 = o0 == k1, m11 = o1 == k1;
        // (adding 0.0f leaves a sum as it is)
        a0 += m00 ? oa0 : 0.0f;
        b0 += m00 ? ob0 : 0.0f;
        a0 += m10 ? oa1 : 0.0f;  // their lower record joins this upper one
        b0 += m10 ? ob1 : 0.0f;
        a1 += m11 ? oa1 : 0.0f;
        b1 += m11 ? ob1 : 0.0f;
        keep0 = keep0 && !(lower && m00);
        keep1 = keep1 && !m01 && !(lower && m11);  // (m01: an upper record takes it)
    };
    look(std::integral_constant<int, 0x39>{}, 1);
    look(std::integral_constant<int, 0x4E>{}, 2);
    look(std::integral_constant<int, 0x93>{}, 3);
    wa[0] = a0;
    wb[0] = b0;
    wa[1] = a1;
    wb[1] = b1;
    keep[0] = keep0;
    keep[1] = keep1;
}

// Same for the maximum (lanes of a group that is wholly inactive are not touched).
template <int LANES_LOG2>
__device__ inline float group_max(float v)
{
    static_assert(LANES_LOG2 <= 4, "within a row of 16 lanes");
    if constexpr (LANES_LOG2 >= 1) v = __builtin_fmaxf(v, dpp_xchg<0xB1>(v));
    if constexpr (LANES_LOG2 >= 2) v = __builtin_fmaxf(v, dpp_xchg<0x4E>(v));
    if constexpr (LANES_LOG2 >= 3) v = __builtin_fmaxf(v, dpp_xchg<0x141>(v));
    if constexpr (LANES_LOG2 >= 4) v = __builtin_fmaxf(v, dpp_xchg<0x140>(v));
    return v;
}

}  // namespace mxd
