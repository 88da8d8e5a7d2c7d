// C ABI entry points (include/mxd_msda.h): argument checks, launch geometry, enqueue.
// Host code only; the kernels live in msda_fwd.hip, msda_fwd_cu.hip, msda_bwd_kernel.h (with msda_bwd*.hip) and msda_bwd_tiles.hip.  Multi-scale
// deformable attention, its fused form, deformable aggregation and geometric kernel attention are the same
// three kernels with different sample sources (msda_device.h: sample_ref, source_geometry).
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "msda_device.h"

namespace mxd {
hipError_t launch_forward(int dtype, const KArgs& a, hipStream_t stream);
hipError_t launch_forward_cu(int dtype, const KArgs& a, hipStream_t stream);
hipError_t raise_forward_lds();
hipError_t raise_forward_cu_lds();
hipError_t launch_backward(int dtype, const KArgs& a, bool scatter, hipStream_t stream);
hipError_t launch_gradv_tiles(int dtype, const KArgs& a, const TileArgs& t, hipStream_t stream);
hipError_t launch_fill_zero(float* p, size_t n, hipStream_t stream);
hipError_t launch_round(int dtype, const float* src, void* dst, size_t n, hipStream_t stream);
hipError_t launch_round_rows(int dtype, const KArgs& a, hipStream_t stream);
hipError_t launch_sum_heads(int dtype, const float* part, void* dst, size_t n, int nh, hipStream_t stream);
}  // namespace mxd

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

// Splits the MXD_META_I64 flag off a dtype argument; returns 1 when it was set.
static int take_meta_flag(int* dtype)
{
    const int f = (*dtype & MXD_META_I64) ? 1 : 0;
    *dtype &= ~MXD_META_I64;
    return f;
}

int elem_size(int dtype)
{
    switch (dtype) {
        case MXD_DTYPE_F32: return 4;
        case MXD_DTYPE_F16:
        case MXD_DTYPE_BF16: return 2;
        default: return 0;
    }
}

int env_int(const char* name, int dflt)
{
    const char* v = getenv(name);
    return (v && *v) ? atoi(v) : dflt;
}

// Tuning knobs, read from the environment once per process (mxd_msda_reload_tuning() reads them again: a hook for
// tests and experiments, not to be called while other threads are inside the library).
struct Tuning {
    int xcd_mode;        // MXD_MSDA_XCD_MODE: 0 = plain workgroup mapping, -1 = by head count
    int bwd_tile_q;      // MXD_MSDA_BWD_TILE_Q: queries per workgroup of the first backward kernel, 0 = chosen here
    int bwd_atomic;      // MXD_MSDA_BWD_ATOMIC: 1 = one-kernel backward with global atomics
    int tile_target;     // MXD_MSDA_TILE_TARGET: pair records per work item of the tile pass, 0 = chosen here
    int fwd_lds;         // MXD_MSDA_FWD_LDS: bytes of the general forward's level cache, -1 = by estimate
    int fwd_iters;       // MXD_MSDA_FWD_ITERS
    int fwd_wgq;         // MXD_MSDA_FWD_WGQ: queries per workgroup of the general forward with a level cache
    int fwd_ahead;       // MXD_MSDA_FWD_AHEAD
    int fwd_cu;          // MXD_MSDA_FWD_CU: 0 = never use the one-workgroup-per-CU forward, 1 = whenever it can run,
                         // -1 = for problems large enough to pay for it
    int fwd_cu_wgs;      // MXD_MSDA_FWD_CU_WGS: its workgroups per (batch, head), 0 = chosen here
    int fwd_cu_cache;    // MXD_MSDA_FWD_CU_CACHE: most bytes of LDS its level cache takes, -1 = all the CU has (a small value
                         // makes every sample come from memory: a hook for measurements)
    int fwd_cu_flip;     // MXD_MSDA_FWD_CU_FLIP: 1 = half of its wavefronts gather from LDS first, the others from memory
                         // first; 0 = all in the same order (sums then formed in the general kernel's order, bit for bit);
                         // -1 = chosen here
    int bwd_fill_kernel; // MXD_MSDA_BWD_FILL_KERNEL: 1 = zero-fill by a kernel of its own
    int tile_order;      // MXD_MSDA_TILE_ORDER: 1 = work items of the tile pass batch-major, 0 = item-major, -1 = chosen here
    int bwd_sparse;      // MXD_MSDA_BWD_SPARSE: 0 = zero-fill (and, for 16-bit dtypes, round) the whole fp32 image of
                         // grad_value, 1 = only the rows that receive atomic additions
    int bwd_unit_split;  // MXD_MSDA_BWD_UNIT_SPLIT: 0 = a unit of the first backward kernel is always a whole query, 1 = queries
                         // of 25 to 32 samples get two units, 2 = queries of 17 to 32 samples
    int bwd_lane_bytes;  // MXD_MSDA_BWD_LANE_BYTES: most bytes of a row one lane of the first backward kernel loads
                         // (16, 8, 4), 0 = chosen here
    int tile_px_log2;    // MXD_MSDA_TILE_PX_LOG2: log2 of the pixels per tile of the grad_value pass (9, 8, 7), 0 = chosen here
    int bwd_fixed;       // MXD_MSDA_BWD_FIXED: 0 = the first backward kernel never takes the instantiation with the common launch
                         // geometry as constants (default 1: where the launch has that geometry)
    int bwd_two_pass;    // MXD_MSDA_BWD_TWO_PASS: 1 = the first backward kernel reads rows of 17 to 32 lanes of 16 bytes with 16
                         // lanes in two passes, 0 = with 32 lanes in one
    int bwd_rec_lds;     // MXD_MSDA_BWD_REC_LDS: 0 = workgroups of the first backward kernel that make several passes store
                         // their records one by one, 1 = they collect their slab in LDS wherever it fits, -1 = chosen here
};
Tuning g_tuning;
std::once_flag g_tuning_once;

void read_tuning()
{
    Tuning t;
    t.xcd_mode = env_int("MXD_MSDA_XCD_MODE", -1);
    t.bwd_tile_q = env_int("MXD_MSDA_BWD_TILE_Q", 0);
    t.bwd_atomic = env_int("MXD_MSDA_BWD_ATOMIC", 0);
    t.tile_target = env_int("MXD_MSDA_TILE_TARGET", 0);
    t.fwd_lds = env_int("MXD_MSDA_FWD_LDS", -1);
    t.fwd_iters = env_int("MXD_MSDA_FWD_ITERS", 1);
    t.fwd_wgq = env_int("MXD_MSDA_FWD_WGQ", 128);
    t.fwd_ahead = env_int("MXD_MSDA_FWD_AHEAD", 1);
    t.fwd_cu = env_int("MXD_MSDA_FWD_CU", -1);
    t.fwd_cu_wgs = env_int("MXD_MSDA_FWD_CU_WGS", 0);
    t.fwd_cu_flip = env_int("MXD_MSDA_FWD_CU_FLIP", -1);
    t.fwd_cu_cache = env_int("MXD_MSDA_FWD_CU_CACHE", -1);
    t.bwd_fill_kernel = env_int("MXD_MSDA_BWD_FILL_KERNEL", 0);
    t.tile_order = env_int("MXD_MSDA_TILE_ORDER", -1);
    t.bwd_lane_bytes = env_int("MXD_MSDA_BWD_LANE_BYTES", 0);
    t.bwd_sparse = env_int("MXD_MSDA_BWD_SPARSE", 1);
    t.bwd_unit_split = env_int("MXD_MSDA_BWD_UNIT_SPLIT", 1);
    t.tile_px_log2 = env_int("MXD_MSDA_TILE_PX_LOG2", 0);
    t.bwd_rec_lds = env_int("MXD_MSDA_BWD_REC_LDS", -1);
    t.bwd_fixed = env_int("MXD_MSDA_BWD_FIXED", 1);
    t.bwd_two_pass = env_int("MXD_MSDA_BWD_TWO_PASS", 1);
    g_tuning = t;
}

const Tuning& tuning()
{
    std::call_once(g_tuning_once, read_tuning);
    return g_tuning;
}

// Scratch of mxd_msda_backward_static(): the hand-over between the two backward kernels (and the fp32 image of
// grad_value for 16-bit dtypes) for callers that can neither allocate nor pass a workspace.  Every device that the
// library runs on holds its own copy of the array at its own address until the process ends.  In host code the name
// below is a stand-in, not a device address: g_scratch_ptr[device], resolved once per device, is what is used.
constexpr size_t kStaticScratchBytes = (size_t)MXD_MSDA_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Per-device set-up, done once per device on the first call that needs it (or by mxd_msda_init()): the forward
// kernels that use more than 64 KiB of dynamic LDS opt in, and the device address of `scratch` is looked up.
constexpr int kMaxDevices = 64;
std::atomic<int> g_device_ready[kMaxDevices];
void* g_scratch_ptr[kMaxDevices];
std::mutex g_device_mutex;

int ensure_device_ready()
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(MXD_E_LAUNCH, "hipGetDevice failed: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(MXD_E_LAUNCH, "device ordinal %d is beyond what this build keeps state for", dev);
    if (g_device_ready[dev].load(std::memory_order_acquire)) return MXD_OK;
    std::lock_guard<std::mutex> lock(g_device_mutex);
    if (g_device_ready[dev].load(std::memory_order_relaxed)) return MXD_OK;
    e = mxd::raise_forward_lds();
    if (e == hipSuccess) e = mxd::raise_forward_cu_lds();
    if (e != hipSuccess) return fail(MXD_E_LAUNCH, "raising the dynamic LDS limit failed: %s", hipGetErrorString(e));
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));  // (this device's copy of the array: the device is current)
    if (e != hipSuccess || ptr == nullptr)
        return fail(MXD_E_LAUNCH, "looking up the static scratch array failed: %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
    g_device_ready[dev].store(1, std::memory_order_release);
    return MXD_OK;
}

// The current device's copy of `scratch` (after ensure_device_ready()).
void* device_scratch()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    return g_device_ready[dev].load(std::memory_order_acquire) ? g_scratch_ptr[dev] : nullptr;
}

struct Dims {
    int64_t bs, nk, nh, hd, nl, nl_attn, nq, np;
};

int check_dims(int dtype, const Dims& d)
{
    if (elem_size(dtype) == 0) return fail(MXD_E_DTYPE, "dtype code %d is not float32(0)/float16(1)/bfloat16(2)", dtype);
    if (d.bs <= 0 || d.nk <= 0 || d.nh <= 0 || d.hd <= 0 || d.nl <= 0 || d.nq <= 0 || d.np <= 0)
        return fail(MXD_E_SHAPE, "Input Tensor can not be a empty Tensor (bs=%lld nk=%lld nh=%lld hd=%lld nl=%lld nq=%lld np=%lld)",
                    (long long)d.bs, (long long)d.nk, (long long)d.nh, (long long)d.hd, (long long)d.nl,
                    (long long)d.nq, (long long)d.np);
    if (d.hd > 256) return fail(MXD_E_SHAPE, "The number of embedding dimensions should be less than or equal to 256");
    if (d.nl > mxd::kMaxLevels) return fail(MXD_E_SHAPE, "The number of levels should be less than or equal to %d", mxd::kMaxLevels);
    if (d.nl_attn < d.nl)
        return fail(MXD_E_SHAPE, "attention_weights carries %lld levels but spatial_shapes has %lld", (long long)d.nl_attn,
                    (long long)d.nl);
    if (d.nl * d.np > 4096 || d.nl * d.np * d.np >= (1 << 20))
        return fail(MXD_E_SHAPE, "num_levels*num_points = %lld is beyond what this build indexes", (long long)(d.nl * d.np));
    if (d.nk * d.nh * d.hd * 4 >= (int64_t(1) << 31))
        return fail(MXD_E_SHAPE, "one batch element of value (num_keys*num_heads*embed_dims = %lld elements) must stay below 2 GiB at 4 bytes per element",
                    (long long)(d.nk * d.nh * d.hd));
    if (d.nq >= (int64_t(1) << 31) - 4096 || d.bs >= (1 << 24) || d.nh >= (1 << 16) ||
        d.nl_attn * d.np >= (int64_t(1) << 24))
        return fail(MXD_E_SHAPE, "a dimension is beyond what this build indexes");
    return MXD_OK;
}

// Fills the XCD mapping fields of a plan for `ntiles` work items per (batch, head); returns the grid.
int64_t fill_xcd_map(mxd_msda_plan* p, int64_t bs, int64_t nh, int64_t ntiles)
{
    p->ntiles = (int32_t)ntiles;
    const int mode_override = tuning().xcd_mode;
    if (mode_override != 0 && nh % mxd::kNumXcd == 0) {
        p->xcd_mode = 1;
        p->heads_per_xcd = (int32_t)(nh / mxd::kNumXcd);
        p->xcds_per_head = 1;
        p->tiles_per_part = (int32_t)ntiles;
        return (int64_t)mxd::kNumXcd * p->heads_per_xcd * ntiles * bs;
    }
    if (mode_override != 0 && mxd::kNumXcd % nh == 0) {
        p->xcd_mode = 2;
        p->heads_per_xcd = 1;
        p->xcds_per_head = (int32_t)(mxd::kNumXcd / nh);
        p->tiles_per_part = (int32_t)((ntiles + p->xcds_per_head - 1) / p->xcds_per_head);
        return (int64_t)mxd::kNumXcd * p->tiles_per_part * bs;
    }
    p->xcd_mode = 0;
    p->heads_per_xcd = 1;
    p->xcds_per_head = 1;
    p->tiles_per_part = (int32_t)ntiles;
    return bs * nh * ntiles;
}

// Bytes of dynamic LDS of the first backward kernel for a plan (tile mode: with the per-tile counters).
size_t backward_lds_bytes(int units_per_wave, int waves, bool tiles, int64_t tbl_stride)
{
    const size_t per_unit = mxd::kChunkStride * sizeof(mxd::Entry) + mxd::kChunk * sizeof(mxd::f32x4);
    size_t n = mxd::kMaxLevels * sizeof(mxd::i32x4) + (size_t)waves * units_per_wave * per_unit;
    if (tiles) n += (size_t)(mxd::kMaxLevels + tbl_stride) * sizeof(int32_t);
    return n;
}

// Row geometry of a problem: elements per lane, lanes per row, row passes.
// two_pass_rows: rows of 17 to 32 lanes of 16 bytes are read by 16 lanes in two passes instead (four units per
// wavefront rather than two: the first backward kernel then fills its geometry lanes and sums its dots over 16 lanes
// with DPP alone; backward at 8 heads x 128 channels in float32 587 -> 572 us, 545 with the slab collected in LDS).
void row_geometry(int es, int64_t hd, int align_bytes, int* vec_out, int* lpr_out, int* npass_out, bool two_pass_rows = false)
{
    if (align_bytes < es) align_bytes = es;
    int vec = 16 / es;
    while (vec > 1 && (hd % vec != 0 || align_bytes < vec * es)) vec >>= 1;
    const int lanes_needed = (int)((hd + vec - 1) / vec);
    int lpr = 4;
    while (lpr < lanes_needed && lpr < mxd::kWave) lpr <<= 1;
    if (two_pass_rows && vec * es == 16 && lpr == 32) lpr = 16;
    int npass = (lanes_needed + lpr - 1) / lpr;
    if (npass == 3) npass = 4;
    *vec_out = vec;
    *lpr_out = lpr;
    *npass_out = npass;
}

// Most bytes of a row that one lane of the first backward kernel loads.
int backward_lane_bytes(int dtype, const Dims& d)
{
    const int v = tuning().bwd_lane_bytes;
    if (v == 4 || v == 8 || v == 16) return v;
    // Rows of 33 to 64 bytes: 8 lanes of 8 bytes per row rather than 4 lanes of 16.  With 16 units per wavefront the
    // staging strips of a workgroup take 51 KiB of LDS, which leaves 3 wavefronts per SIMD, and a lane stages four
    // samples of which it keeps two in registers (measured, encoder shape in float16 / bfloat16: backward 322 -> 300 us;
    // BEVFormer shape in float16 1114 -> 1075 us; with rows of 256 bytes halving the lane width costs 10 %).
    const int64_t row = d.hd * elem_size(dtype);
    return (row > 32 && row <= 64) ? 8 : 16;
}

// How the backward pass is laid out for a problem size: whether grad_value goes through the
// tile-ownership pass (and then the hand-over buffers between its two kernels) or through
// global atomics, and where things live in the caller's workspace.
//   workspace = [run table][pair records][fp32 image of grad_value, 16-bit dtypes only]
// Queries per workgroup of the first backward kernel (tile pass).  Larger workgroups give the tile pass
// longer runs; with few queries they leave the chip short of workgroups, so the size steps down until the
// launch has about six workgroups per CU.  64 is the least for rows of up to 64 bytes (16 units per
// wavefront, 4 wavefronts), 32 otherwise.  MXD_MSDA_BWD_TILE_Q overrides (32/64/128/256).
static int64_t bwd_tile_q(int dtype, const Dims& d)
{
    // (units with very many samples -- deformable aggregation's 312 -- measured 1 to 2 % better with 64)
    int vec, lpr, npass;
    row_geometry(elem_size(dtype), d.hd, backward_lane_bytes(dtype, d), &vec, &lpr, &npass, tuning().bwd_two_pass != 0);
    const int64_t least = (mxd::kWave / lpr > 8 || d.nl * d.np >= 256) ? 64 : 32;
    const int v = tuning().bwd_tile_q;
    if (v == 32 || v == 64 || v == 128 || v == 256) return v < least ? least : v;
    // about 512 samples per workgroup for rows of up to 128 bytes, 1024 for longer ones (measured: 32 queries of 16
    // or of 32 samples are the optima of the encoder and the BEVFormer shapes -- with 16 samples per query all of a
    // workgroup's samples are then staged while its records are counted --, 64 queries of 16 samples that of 512-byte
    // rows; 128 queries cost 3 to 7 %)
    const int64_t samples = d.hd * elem_size(dtype) <= 128 ? 512 : 1024;
    int64_t first = 128;
    while (first > least && first * d.nl * d.np > samples) first >>= 1;
    for (int64_t tq = first; tq > least; tq >>= 1)
        if (d.bs * d.nh * ((d.nq + tq - 1) / tq) >= 6 * 256) return tq;
    // Queries of 17 to 32 samples in a workgroup that makes one pass: two neighbouring units share a query, each taking
    // 16 of its samples, so that the workgroup -- half as many queries -- stages all its samples while it counts its
    // records (their geometry is derived once) and collects its records in LDS to write its slab in whole lines, as
    // with up to 16 samples per query.
    // (it pays when the second unit has work for most of its lanes -- encoder levels, float32: 32 samples per query 544
    //  against 571 us, BEVFormer 1036 against 1094; 24 samples 2370 against 2301, 20 samples 442 against 420 --: from 25
    //  samples on; MXD_MSDA_BWD_UNIT_SPLIT=2 splits from 17 on)
    const int units = mxd::kWave / lpr * 4;
    const int64_t split_from = tuning().bwd_unit_split >= 2 ? mxd::kChunk + 1 : mxd::kChunk + mxd::kChunk / 2 + 1;
    if (tuning().bwd_unit_split && least == units && units >= 8 && d.nl * d.np >= split_from && d.nl * d.np <= 2 * mxd::kChunk)
        return least / 2;
    return least;
}
struct BwdLayout {
    bool tiles;          // false: one kernel with global atomics
    int tile_px_log2;    // log2 of the pixels per tile of the grad_value pass
    int64_t tile_q;      // queries per workgroup of the first kernel
    int64_t nwg;         // workgroups of the first kernel per (batch, head)
    int64_t rec_cap;     // pair records per workgroup slab: 2 per sample
    int64_t tbl_stride;  // tiles per (batch, head) at most, plus one
    size_t tbl_bytes, rec_bytes, image_bytes, total;
};

// Pixels per tile of the grad_value pass, as a power of two: every thread of its workgroups keeps 32 sums, so 512 pixels
// of up to 32 channels, 256 of up to 64, 128 of more (msda_plan.h).  The smaller tiles are built for rows that are read
// four elements per lane (`wide_rows`: head_dim a multiple of 4 and pointers aligned for it); other rows keep 512-pixel
// tiles and take one pass over the records per 32 channels.
int preferred_tile_px_log2(const Dims& d, bool wide_rows)
{
    if (!wide_rows || d.hd % 4 != 0) return mxd::kTilePxLog2Max;
    const int v = tuning().tile_px_log2;
    if (v >= 7 && v <= mxd::kTilePxLog2Max) return v;
    if (d.hd <= 32) return mxd::kTilePxLog2Max;
    // Maps so small that a level is a tile of 512 pixels or less keep that tile and take two or four passes: the slots
    // of the workgroup that the tile leaves free are what a pixel that collects far more entries than the others gets
    // its extra lists from, and a tile cut in two has none (geometric kernel attention at 15 x 25 pixels and 64 channels,
    // where clamping piles half of the samples on the border: 0.80 ms per step with one tile of 375 pixels and two
    // passes, 0.90 ms with tiles of 256 + 119 pixels and one).
    if (d.nk <= (int64_t)d.nl << mxd::kTilePxLog2Max) return mxd::kTilePxLog2Max;
    // (measured at 8 heads x 128 channels, encoder levels: float16 backward 588 us with tiles of 512 pixels, 431 with 256,
    //  383 with 128; float32 722, 590, 586)
    return d.hd <= 64 ? 8 : 7;
}

BwdLayout bwd_layout_for(int dtype, const Dims& d, int tile_px_log2)
{
    BwdLayout L;
    memset(&L, 0, sizeof(L));
    L.tile_px_log2 = tile_px_log2;
    L.tile_q = bwd_tile_q(dtype, d);
    L.nwg = (d.nq + L.tile_q - 1) / L.tile_q;
    L.rec_cap = 2 * L.tile_q * d.nl * d.np;
    // tiles per (batch, head) when the levels do not overlap: sum of ceil(pixels / tile) <= nk / tile + nl
    // (the kernels leave out levels that would not fit, which can only happen for overlapping levels)
    L.tbl_stride = (d.nk >> tile_px_log2) + d.nl + 1;
    const int64_t tbl = d.bs * d.nh * L.nwg * L.tbl_stride * 4;
    // dynamic LDS of the first kernel with the most units per wavefront the row can have (16-byte aligned pointers)
    int vec, lpr, npass;
    row_geometry(elem_size(dtype), d.hd, backward_lane_bytes(dtype, d), &vec, &lpr, &npass, tuning().bwd_two_pass != 0);
    const size_t lds = backward_lds_bytes(mxd::kWave / lpr, 4, true, L.tbl_stride);
    L.tiles = tuning().bwd_atomic == 0 &&
              L.tbl_stride <= 4096 &&                      // counters of the first kernel live in LDS ...
              lds <= 64 * 1024 &&                          // ... and its strips and counters fit the default limit
              tbl <= (int64_t(1) << 28) &&                 // run table of at most 256 MiB
              L.nwg * L.rec_cap * (mxd::kRecDwords * 4) < (int64_t(1) << 32) &&  // 32-bit byte offsets of the records of a (batch, head)
              d.nq * d.nh * d.hd * 4 < (int64_t(1) << 31); // grad_output rows addressed with 32-bit byte offsets
    if (L.tiles) {
        L.tbl_bytes = ((size_t)tbl + 255) & ~(size_t)255;
        L.rec_bytes = ((size_t)d.bs * d.nh * L.nwg * L.rec_cap * (mxd::kRecDwords * 4) + 255) & ~(size_t)255;
    }
    if (elem_size(dtype) == 2) L.image_bytes = (size_t)d.bs * d.nk * d.nh * d.hd * 4;
    L.total = L.tbl_bytes + L.rec_bytes + L.image_bytes;
    return L;
}

// The layout a launch uses: the tile size preferred for the rows, or 512-pixel tiles where the finer run table would
// not fit the first kernel's bookkeeping.
BwdLayout bwd_layout(int dtype, const Dims& d, bool wide_rows)
{
    const int pref = preferred_tile_px_log2(d, wide_rows);
    BwdLayout L = bwd_layout_for(dtype, d, pref);
    if (!L.tiles && pref != mxd::kTilePxLog2Max) L = bwd_layout_for(dtype, d, mxd::kTilePxLog2Max);
    return L;
}

// Workspace a caller must bring: what the launch may need whichever way its pointers are aligned.
size_t bwd_workspace_bytes(int dtype, const Dims& d)
{
    const size_t a = bwd_layout(dtype, d, true).total, b = bwd_layout(dtype, d, false).total;
    return a > b ? a : b;
}

// LDS for the slab of a workgroup of the first backward kernel that makes several passes (msda_bwd_kernel.h): 12 bytes per
// record behind the counters, when the slab is small enough to leave four workgroups to a CU and the kernel stays
// inside the default limit of dynamic LDS.  A workgroup that makes one pass of one chunk (the plain operator and the
// fused form) collects its records in its staging strips instead.  Adds the bytes to the plan.
int plan_record_buffer(mxd_msda_plan* p, const BwdLayout& L, const Dims& d, int dtype, bool plain_or_fused, int unit_split_log2)
{
    if (!L.tiles || !plain_or_fused) return 0;  // (the kernel is built with the buffer for these two sources only)
    // By default for the plain operator and its fused form, for slabs of up to 12 KiB and, with at most four units per
    // wavefront (rows of 16 lanes and more, whose staging strips are small), of up to 24 KiB (MXD_MSDA_BWD_REC_LDS=1:
    // wherever it fits).  Measured, backward: encoder levels with 2 points, float32 (12 KiB) 231 -> 216 us; 8 heads x 128
    // channels, tiles of 128 pixels (24 KiB, four units): float16 414 -> 383 us, float32 572 -> 545 us (with two units of
    // 32 lanes: 586 -> 596); geometric kernel attention (64 channels, float32, 23 KiB) 0.80 -> 0.86 ms per step -- where
    // it loses, the buffer costs the kernel a workgroup per CU, which weighs more than the partial lines.
    (void)dtype;
    const int64_t slab = L.rec_cap * (mxd::kRecDwords * 4);
    if (tuning().bwd_rec_lds < 0 && !(slab <= 12 * 1024 || p->units_per_wave <= 4)) return 0;
    const bool one_pass = plain_or_fused && p->iters == 1 && d.nl * d.np <= ((int64_t)mxd::kChunk << unit_split_log2);
    const int64_t bytes = L.rec_cap * (mxd::kRecDwords * 4);
    const int64_t total = (((int64_t)p->lds_bytes + 15) & ~(int64_t)15) + bytes;
    if (one_pass || bytes > 24 * 1024 || total > 40 * 1024 || tuning().bwd_rec_lds == 0) return 0;
    p->lds_bytes = (uint32_t)total;
    return (int)bytes;
}

// Geometry of the tile-ownership grad_value kernel (msda_bwd_tiles.hip).
int make_tile_args(const Dims& d, const BwdLayout& L, int vec, int accumulate, mxd::TileArgs* t, bool plain_operator = false)
{
    memset(t, 0, sizeof(*t));
    // pair records (counted before merging) per work item when a hot tile is split: enough items to fill the 512
    // workgroup slots of the chip about twice (measured optimum on MI355X; fewer, longer items lose to imbalance,
    // more, shorter ones to the atomics of their write-out).  Below 8192 records the write-out starts to
    // weigh more and the measured optimum falls more slowly than the problem size: geometric mean of the two
    // (0.17 M samples: 2 100, 0.5 M: 3 600, 1.3 M: 5 700 records per item).
    int64_t target = 2 * d.bs * d.nh * d.nq * d.nl * d.np / 512;
    if (target < 8192) target = (int64_t)sqrt(8192.0 * (double)(target > 32 ? target : 32));
    // (capped: 32 768 measured 0.6 to 1.7 % behind 49 152 on problems of 10 to 40 M samples, 65 536 up to 4 % behind it and
    //  100 000 up to 20 %: the launch then has too few items to fill the chip evenly)
    if (target > 49152) target = 49152;
    if (d.nl == 1) {
        // One level: its tiles all collect about the same number of records, so the launch is a whole number of
        // equal work items per tile.  Up to 512 of them run side by side in the chip's workgroup slots; a few more
        // than that make the launch last two items (measured, geometric kernel attention: 672 items 0.92 ms per
        // step, 480 items 0.81 ms, 384 items 0.87 ms).  Pick the chunk count with the least estimated duration:
        // items in flight one after another x (records per item + about 8192 records' worth of start, statistics
        // round and write-out per item).
        const int64_t nt = (d.nk + (int64_t(1) << L.tile_px_log2) - 1) >> L.tile_px_log2;
        const int64_t per_tile = 2 * d.nq * d.np / nt;
        int64_t best_c = 1;
        double best_cost = -1.0;
        for (int64_t c = 1; c <= 64 && c <= L.nwg; ++c) {
            const double items = (double)(d.bs * d.nh * nt * c);
            const double cost = (items <= 512.0 ? 1.0 : items / 512.0 + 0.5) * ((double)per_tile / (double)c + 8192.0);
            if (best_cost < 0.0 || cost < best_cost) {
                best_cost = cost;
                best_c = c;
            }
        }
        target = (per_tile + best_c - 1) / best_c;
    }
    t->target = tuning().tile_target > 0 ? tuning().tile_target : (int)target;
    if (t->target < 128) t->target = 128;
    t->max_chunks = 64;
    // work items per (batch, head): sum over levels of tiles*chunks <= 2*nl*nq*np/target + nl + sum of tiles
    const int64_t items = d.nl * ((2 * d.nq * d.np + t->target - 1) / t->target + 1) + L.tbl_stride;
    if (items >= (int64_t(1) << 24)) return fail(MXD_E_SHAPE, "backward needs %lld work items per (batch, head)", (long long)items);
    t->items_per_bh = (int32_t)items;  // (the callers add TileArgs::extra)
    t->vec = vec;
    t->accumulate = accumulate;
    t->batch_major = tuning().tile_order > 0 ? 1 : 0;
    t->map.tile_q = 1;
    t->extra = plain_operator ? 8 : 0;
    t->items_per_bh += t->extra;
    const int64_t grid = fill_xcd_map(&t->map, d.bs, d.nh, t->items_per_bh);
    if (grid >= (int64_t(1) << 31)) return fail(MXD_E_SHAPE, "backward needs %lld workgroups, beyond the launch limit", (long long)grid);
    t->grid = (uint32_t)grid;
    t->block = mxd::kTileThreads;
    return MXD_OK;
}

// Tile mode: how the fp32 image of grad_value gets its zeros and how its rows reach the caller's tensor.  Tiles that
// one workgroup of the tile pass owns store their rows once; when the rows can be written in 16-byte pieces only the
// other rows (those that receive atomic additions) are zero-filled, and for 16-bit dtypes the owner stores rounded rows
// straight into the caller's tensor, so that only those other rows go through the fp32 image and the rounding pass.
void plan_image(mxd::KArgs* a, mxd::TileArgs* t, bool half, bool accumulate, float* image, void* grad_value, int64_t hd)
{
    a->tile_target = t->target;
    a->tile_max_chunks = t->max_chunks;
    t->store_vec = (hd % 4 == 0 && (reinterpret_cast<uintptr_t>(image) & 15u) == 0) ? 4 : 1;
    a->sparse = tuning().bwd_sparse != 0 && tuning().bwd_fill_kernel == 0 && t->store_vec == 4 && !accumulate &&
                (!half || (reinterpret_cast<uintptr_t>(grad_value) & 7u) == 0);
    a->grad_value_t = (a->sparse && half) ? grad_value : nullptr;
}

// Bytes of LDS the plain forward sets aside for the rows of the last levels (0: none).  Needs 16-byte lanes.
// LDS for the forward's level cache, 0 = run without.  The cache pays when the coarsest level fits in it
// (a quarter of the samples of a 4-level pyramid then are gathered from LDS) and costs otherwise: its
// workgroups are larger and hold more LDS, which leaves fewer wavefronts per CU.  The level shapes live in
// device memory, so the decision here rests on an estimate: in a pyramid that halves from level to level
// the last one has nk*3/(4^nl - 1) pixels.  With more than 8 units per wavefront (rows of 64 bytes) the
// staging strips alone limit the wavefronts per CU, and the cache is left out.
// MXD_MSDA_FWD_LDS set in the environment overrides the estimate (0 = off, bytes = on).
int forward_cache_bytes(int vec, int es, const Dims& d, int units_per_wave)
{
    const bool forced = tuning().fwd_lds >= 0;
    const int v = forced ? tuning().fwd_lds : 40960;
    if (!(vec * es == 16 && v >= 1024 && v <= 65536)) return 0;
    if (!forced) {
        if (units_per_wave > 8) return 0;
        // Small problems lose more to the cache fill of every workgroup than the gather gains (float32, with / without:
        // 2 x 300 queries 11.3 / 6.1 us, 8 x 900 queries 37 / 34, the encoder's queries with 2 heads 18 / 14, five
        // levels with 4 points and 6.4 M samples 206 / 201; with 8 points and 12.8 M samples 406 / 421).
        if (d.bs * d.nh * d.nq * d.nl * d.np < (int64_t(1) << 23)) return 0;
        double last = (double)d.nk;
        if (d.nl > 1) last = (double)d.nk * 3.0 / ((double)(int64_t(1) << (2 * (d.nl < 16 ? d.nl : 16))) - 1.0);
        if (last * 1.1 * (double)(d.hd * es) > (double)v) return 0;
    }
    return v & ~15;
}

// Rows of the last levels that an LDS cache of `cap_rows` rows would hold, estimated for a pyramid that halves
// from level to level (the level shapes live in device memory): the last level has nk*3/(4^nl - 1) pixels.
int64_t estimated_cached_rows(const Dims& d, int64_t cap_rows)
{
    double last = (double)d.nk;
    if (d.nl > 1) last = (double)d.nk * 3.0 / ((double)(int64_t(1) << (2 * (d.nl < 16 ? d.nl : 16))) - 1.0);
    double r = last * 1.1, total = 0.0;
    for (int l = 0; l < d.nl && total + r <= (double)cap_rows; ++l) {
        total += r;
        r *= 4.0;
    }
    return (int64_t)total;
}

// The forward's one-workgroup-per-CU form (msda_fwd_cu.hip): whether a problem takes it, and its launch geometry.
// It needs 16-byte lanes, rows of at most 16 lanes and the plain operator; it pays when at least the last level fits
// the CU's LDS and the problem is large enough to keep 256 such workgroups busy well beyond their cache fill.
bool plan_forward_cu(int dtype, const Dims& d, int vec, int lpr, int npass, mxd_msda_plan* p, int* cache_bytes)
{
    const int mode = tuning().fwd_cu;
    const int es = elem_size(dtype);
    if (mode == 0 || vec * es != 16 || npass != 1 || lpr > 16) return false;
    // What the kernel's index arithmetic assumes, whatever the environment asks for: pixel indices and the distance
    // between neighbouring pixels are multiplied as 24-bit integers, and the locations, weights, results (and the
    // fused form's reference points) of one batch element are addressed with 32-bit byte offsets inside a buffer
    // descriptor.  Anything larger goes to the general kernel, which indexes with 64-bit offsets.
    const int64_t kMul24 = int64_t(1) << 23, kOff32 = int64_t(1) << 31;
    if (d.nk >= kMul24 || d.nh * d.hd * es >= kMul24 || d.nq * d.nh * d.nl_attn * d.np * 2 * es >= kOff32 ||
        d.nq * d.nh * d.hd * es >= kOff32 || d.nq * d.nl * 2 * es >= kOff32)
        return false;
    const int cap = mxd::kCuLdsBytes - mxd::kCuTableBytes;  // (two level tables come first)
    const int64_t cap_rows = cap / (d.hd * es) - 1;
    const int64_t cached = estimated_cached_rows(d, cap_rows);
    // By default (measured on MI355X, uniformly random locations, this form against the general kernel, float32 /
    // float16).  Units of up to 16 samples (one chunk): it wins where about half of the samples are gathered from LDS
    // -- the Deformable-DETR encoder shape, 79 against 86 us / 71 against 86 us; one level of 64 x 64 with 8 points,
    // 85 against 106 / 77 against 97 -- and is level or behind where fewer are (BEVFormer's levels with 4 points: 214
    // against 215 / 149 against 151; five levels: 258 against 206 / 185 against 179).  Units of more samples: it wins
    // as soon as the last level is cached -- the encoder's levels with 5, 6, 8, 12, 16 points: 0.93, 0.91, 0.79, 0.76,
    // 0.73 of the general kernel's time / 0.82, 0.78, 0.74, 0.68, 0.70; the BEVFormer shape 395 against 433 / 237
    // against 288 -- unless a (batch, head) slice of value is far beyond an XCD's 4 MiB of L2, where the general
    // kernel's larger number of wavefronts hides more of the memory latency (pyramid from 256 x 256, 11 MB in
    // float32: 1750 against 1504 us; 5.6 MB in float16: 1109 against 1147; five levels from 200 x 300, 10 MB: 441
    // against 404 / 5 MB: 287 against 308), and not where nothing is cached (one level of 100 x 150, 32 points: 153
    // against 147 / 174 against 138).  Small problems stay with the general kernel (8 x 900 queries: 59 against 37).
    if (mode < 0) {
        double last = (double)d.nk, rows = 0.0;
        if (d.nl > 1) last = (double)d.nk * 3.0 / ((double)(int64_t(1) << (2 * (d.nl < 16 ? d.nl : 16))) - 1.0);
        int levels_cached = 0;
        for (double r = last; levels_cached < d.nl && rows + r <= (double)cap_rows; r *= 4.0) {
            rows += r;
            ++levels_cached;
        }
        if (levels_cached == 0 || d.bs * d.nh * d.nq * d.nl * d.np < (int64_t(1) << 20)) return false;
        const int64_t slice = d.nk * d.hd * es;
        // (rows of 256 bytes, 16 samples per unit, one level of four cached: 0.88 to 0.93 of the general kernel's time at
        //  the encoder's levels -- head_dim 64 and 48 in float32, 128 and 96 in float16, slices of 5 MB -- but 1.18 to
        //  1.33 at slices of 8 MB and more, and 0.93 to 1.25 with 8 samples per unit)
        const bool long_rows = lpr == 16 && d.nl * d.np == mxd::kChunk && slice <= (int64_t(6) << 20);
        if (d.nl * d.np <= mxd::kChunk ? 2 * levels_cached < d.nl && !long_rows : slice > (int64_t(8) << 20)) return false;
    }
    const int U = mxd::kWave / lpr;
    const int64_t groups = (d.nq + U - 1) / U;
    // Workgroups per (batch, head): every XCD has 32 CUs, each of which runs one workgroup at a time; the launch
    // lasts (rounds of 32 workgroups per XCD) x (cache fill + the workgroup's share of the gathers).  The rows that
    // are not cached come from the XCD's 4 MiB L2: the workgroups that run side by side on an XCD should work on as
    // few (batch, head) slices as possible (workgroups of an XCD are numbered head, query range, batch element).
    int64_t best_p = 1;
    double best_cost = -1.0;
    const int64_t max_p = groups < 512 ? groups : 512;
    const double slice_bytes = (double)(d.nk - cached) * (double)(d.hd * es);
    const double launch = 3000.0, fill = (double)cached + 1000.0;   // in units of one gathered row
    for (int64_t P = 1; P <= max_p; ++P) {
        if (tuning().fwd_cu_wgs > 0 && P != tuning().fwd_cu_wgs && tuning().fwd_cu_wgs <= max_p) continue;
        const int64_t tq = U * (((d.nq + P - 1) / P + U - 1) / U);
        const int64_t nt = (d.nq + tq - 1) / tq;
        mxd_msda_plan trial;
        memset(&trial, 0, sizeof(trial));
        const int64_t grid = fill_xcd_map(&trial, d.bs, d.nh, nt);
        const double per_xcd = (double)grid / mxd::kNumXcd;
        const double rounds = ceil(per_xcd / 32.0);
        double slices = 32.0 / (double)(trial.xcd_mode == 2 ? trial.tiles_per_part : nt);  // side by side on an XCD
        if (trial.xcd_mode == 1 && slices < (double)trial.heads_per_xcd) slices = (double)trial.heads_per_xcd;
        if (trial.xcd_mode == 0) slices = slices * 8.0 < (double)d.nh ? (double)d.nh : slices * 8.0;
        if (slices < 1.0) slices = 1.0;
        // (measured at the encoder shape: two slices side by side cost 10 to 15 % also where both fit the L2 --
        //  float16, 2 x 1.2 MB -- and 15 to 25 % where they do not -- float32, 2 x 2.4 MB)
        // By default only where whole heads are pinned to an XCD, at most two of them: a head that several XCDs share
        // needs so many workgroups per (batch, head) to keep the slices side by side on an XCD few that the cache fills
        // outweigh the gain.  Measured at the encoder shape with the 16 (batch, head) pairs split as bs x heads --
        // this form against the general kernel: 2 x 8: 91 / 102 us, 1 x 16: 96 / 123, 4 x 4: 102 / 102, 8 x 2: 120 / 105
        // (152 with one round of workgroups), 16 x 1: 133 / 112 (175), 2 x 6 heads, no pinning: 106 / 94.
        // (four heads, each shared by two XCDs: with the encoder's queries and two batch elements 44.8 against 50.2 us)
        if (mode < 0 && !((trial.xcd_mode == 1 && trial.heads_per_xcd <= 2) || (trial.xcd_mode == 2 && trial.xcds_per_head <= 2)))
            continue;
        double over = ceil(slices) * slice_bytes / (4.0 * 1024 * 1024) - 0.4;
        over = over < 0.0 ? 0.0 : (over > 1.0 ? 1.0 : over);
        const double gather = (1.0 + 0.5 * over) * (double)tq * (double)(d.nl * d.np) * 4.0;
        const double cost = rounds * (launch + fill + gather);
        if (best_cost < 0.0 || cost < best_cost) {
            best_cost = cost;
            best_p = P;
        }
    }
    if (best_cost < 0.0) return false;  // (not a shape for this form)
    const int64_t tq = U * (((d.nq + best_p - 1) / best_p + U - 1) / U);
    const int64_t nt = (d.nq + tq - 1) / tq;
    memset(p, 0, sizeof(*p));
    p->vec = vec;
    p->lanes_per_row = lpr;
    p->npass = 1;
    p->units_per_wave = U;
    p->waves_per_block = mxd::kCuWaves;
    p->iters = (int32_t)((tq / U + mxd::kCuWaves - 1) / mxd::kCuWaves);
    p->tile_q = (int32_t)tq;
    const int64_t grid = fill_xcd_map(p, d.bs, d.nh, nt);
    if (grid >= (int64_t(1) << 31)) return false;
    p->grid = (uint32_t)grid;
    p->block = (uint32_t)(mxd::kCuWaves * mxd::kWave);
    p->lds_bytes = (uint32_t)mxd::kCuLdsBytes;
    *cache_bytes = cap & ~15;
    if (tuning().fwd_cu_cache >= 0 && tuning().fwd_cu_cache < *cache_bytes) {
        // (at least the row of zeros that stands for corners outside the image)
        const int least = (int)(d.hd * es + 15) & ~15;
        *cache_bytes = tuning().fwd_cu_cache < least ? least : (tuning().fwd_cu_cache & ~15);
    }
    return true;
}

// Whether half of the wavefronts of the forward's one-workgroup-per-CU form work through their chunks from the LDS
// groups on, so that memory gathers and LDS gathers of a CU's wavefronts run side by side.  Measured at the encoder
// shape (alternating launches, one box): float16 70.9 -> 69.0 us -- 16 rows of 64 bytes per load instruction keep the
// vector-memory pipeline twice as long as 8 rows of 128 bytes --, float32 78.9 -> 79.8 us: by default for 16-bit rows.
int forward_cu_flip(int dtype)
{
    const int v = tuning().fwd_cu_flip;
    return v >= 0 ? (v != 0) : (elem_size(dtype) == 2);
}

// level_cache: in/out, bytes of LDS for the forward's level cache (asked for -> granted)
// cu_form: in/out, whether the forward may take / takes the one-workgroup-per-CU form
int make_plan(int backward, int dtype, const Dims& d, int align_bytes, mxd_msda_plan* p, int* level_cache = nullptr,
              int* cu_form = nullptr)
{
    const int rc = check_dims(dtype, d);
    if (rc != MXD_OK) return rc;
    const int es = elem_size(dtype);
    int vec, lpr, npass;
    if (backward && align_bytes > backward_lane_bytes(dtype, d)) align_bytes = backward_lane_bytes(dtype, d);
    // (the forward keeps 32 lanes in one pass: at 8 heads x 128 channels in float32 two passes take 248 against 237 us)
    row_geometry(es, d.hd, align_bytes, &vec, &lpr, &npass, backward && tuning().bwd_two_pass != 0);
    if (!backward && cu_form && *cu_form && level_cache) {
        if (plan_forward_cu(dtype, d, vec, lpr, npass, p, level_cache)) return MXD_OK;
    }
    if (cu_form) *cu_form = 0;
    memset(p, 0, sizeof(*p));
    p->vec = vec;
    p->lanes_per_row = lpr;
    p->npass = npass;
    p->units_per_wave = mxd::kWave / lpr;
    p->waves_per_block = 4;
    int iters = tuning().fwd_iters;
    if (iters < 1) iters = 1;
    const BwdLayout L = bwd_layout(dtype, d, vec >= 4);
    // the tile pass wants L.tile_q queries per workgroup of the first backward kernel
    int split = 1;  // units of the backward's first kernel that share a query
    if (backward) {
        iters = L.tiles ? (int)(L.tile_q / (p->units_per_wave * p->waves_per_block)) : 1;
        if (iters < 1) {
            iters = 1;
            split = (int)(p->units_per_wave * p->waves_per_block / L.tile_q);
        }
    }
    int cache = (level_cache && *level_cache && !backward) ? forward_cache_bytes(vec, es, d, p->units_per_wave) : 0;
    if (cache > 0) {
        // 8 wavefronts share one copy of the cached rows and work through 128 queries (MXD_MSDA_FWD_WGQ; 256 and
        // 64 measure within 2 % of it); two such workgroups
        // must fit a CU (80 KiB each), else fewer wavefronts, else no cache
        int waves = 8;
        while (waves > 2 && mxd::kMaxLevels * sizeof(mxd::i32x4) + (size_t)waves * p->units_per_wave *
                                    (mxd::kChunkStride * sizeof(mxd::Entry) + 2 * sizeof(float)) + cache > 80 * 1024)
            waves >>= 1;
        if (waves > 2) {
            p->waves_per_block = waves;
            iters = tuning().fwd_wgq / (p->units_per_wave * p->waves_per_block);
            if (iters < 1) iters = 1;
        } else {
            cache = 0;
        }
    }
    p->iters = iters;
    p->tile_q = p->units_per_wave * p->waves_per_block * p->iters / split;
    const int64_t ntiles = (d.nq + p->tile_q - 1) / p->tile_q;
    p->ntiles = (int32_t)ntiles;
    const int64_t grid = fill_xcd_map(p, d.bs, d.nh, ntiles);
    if (grid >= (int64_t(1) << 31)) return fail(MXD_E_SHAPE, "problem needs %lld workgroups, beyond the launch limit", (long long)grid);
    p->grid = (uint32_t)grid;
    p->block = (uint32_t)(p->waves_per_block * mxd::kWave);
    if (backward) {
        p->lds_bytes = (uint32_t)backward_lds_bytes(p->units_per_wave, p->waves_per_block, L.tiles, L.tbl_stride);
    } else {
        p->lds_bytes = (uint32_t)(mxd::kMaxLevels * sizeof(mxd::i32x4) +
                                  (size_t)p->waves_per_block * p->units_per_wave * mxd::kChunkStride * sizeof(mxd::Entry));
        p->lds_bytes += (uint32_t)(p->waves_per_block * p->units_per_wave * 2 * sizeof(float));  // softmax statistics (fused form)
    }
    if (cache > 0) p->lds_bytes += (uint32_t)cache;
    if (level_cache) *level_cache = cache;
    return MXD_OK;
}

int ptr_align(const void* p)
{
    const uintptr_t v = reinterpret_cast<uintptr_t>(p);
    int a = 16;
    while (a > 1 && (v & (uintptr_t)(a - 1))) a >>= 1;
    return a;
}

// Units of the backward's first kernel that share a query, as a power of two (see bwd_tile_q).
int unit_split_log2(const mxd_msda_plan& p)
{
    const int units = p.units_per_wave * p.waves_per_block * p.iters;
    int s = 0;
    while (p.tile_q > 0 && (p.tile_q << (s + 1)) <= units) ++s;
    return s;
}

void fill_args(mxd::KArgs* a, int dtype, const Dims& d)
{
    const int es = elem_size(dtype);
    a->bs = (int32_t)d.bs;
    a->nk = (int32_t)d.nk;
    a->nh = (int32_t)d.nh;
    a->hd = (int32_t)d.hd;
    a->nl = (int32_t)d.nl;
    a->np = (int32_t)d.np;
    a->nq = (int32_t)d.nq;
    a->S = (int32_t)(d.nl * d.np);
    a->S_full = (int32_t)(d.nl_attn * d.np);
    a->np_magic = (uint32_t)(((1u << 20) + d.np - 1) / d.np);
    a->pitch_bytes = (uint32_t)(d.nh * d.hd * es);
    a->batch_bytes = (uint32_t)(d.nk * d.nh * d.hd * es);
    a->gbatch_bytes = (uint32_t)(d.nk * d.nh * d.hd * 4);
}

// Deformable aggregation in the terms of the kernels: channel group = head, (camera, scale) = level,
// anchor = query, points per anchor = points.
int dagg_dims(int dtype, int64_t bs, int64_t nf, int64_t C, int64_t cams, int64_t scales, int64_t A, int64_t P,
              int64_t G, Dims* d)
{
    if (G <= 0 || cams <= 0 || scales <= 0 || C <= 0)
        return fail(MXD_E_SHAPE, "Input Tensor can not be a empty Tensor (C=%lld cams=%lld scales=%lld groups=%lld)",
                    (long long)C, (long long)cams, (long long)scales, (long long)G);
    if (C % G != 0) return fail(MXD_E_SHAPE, "num_embeds (%lld) must be a multiple of num_groups (%lld)", (long long)C, (long long)G);
    *d = Dims{bs, nf, G, C / G, cams * scales, cams * scales, A, P};
    const int rc = check_dims(dtype, *d);
    if (rc != MXD_OK) return rc;
    // sample index -> (point, level) by a multiply-shift that is exact while samples * levels < 2^20
    if (d->nl * d->np * d->nl >= (1 << 20))
        return fail(MXD_E_SHAPE, "num_pts*(num_cams*num_scale)^2 = %lld is beyond what this build indexes",
                    (long long)(d->nl * d->np * d->nl));
    return MXD_OK;
}

void fill_dagg(mxd::KArgs* a, int64_t cams, int64_t scales)
{
    a->cams = (int32_t)cams;
    a->scales = (int32_t)scales;
    a->np_magic = (uint32_t)(((1u << 20) + a->nl - 1) / a->nl);  // sample / levels
    a->sc_magic = (uint32_t)(((1u << 20) + scales - 1) / scales);
    a->sc_pow2 = (scales & (scales - 1)) == 0 && scales <= 16;
}

size_t dagg_part_bytes(const Dims& d, int64_t cams)
{
    return (size_t)d.nh * d.bs * d.nq * d.np * cams * 2 * sizeof(float);
}

}  // namespace

extern "C" {

int mxd_msda_version(void) { return MXD_MSDA_VERSION; }

const char* mxd_msda_last_error(void) { return g_err; }

int mxd_msda_make_plan(int backward, int dtype, int64_t bs, int64_t nk, int64_t nh, int64_t hd, int64_t nl, int64_t nl_attn,
                  int64_t nq, int64_t np, int align_bytes, mxd_msda_plan* plan)
{
    take_meta_flag(&dtype);
    if (!plan) return fail(MXD_E_NULL, "plan is NULL");
    const Dims d{bs, nk, nh, hd, nl, nl_attn, nq, np};
    int cache = 1, cu = 1;
    return make_plan(backward != 0, dtype, d, align_bytes, plan, &cache, &cu);
}

int mxd_msda_init(void)
{
    tuning();
    return ensure_device_ready();
}

void mxd_msda_reload_tuning(void) { tuning(); read_tuning(); }

int mxd_msda_decode_block(const mxd_msda_plan* plan, uint32_t block_index, int64_t bs, int64_t nh, int64_t nq,
                          int32_t work[4])
{
    if (!plan || !work) return 0;
    mxd::Work w;
    if (!mxd::decode_block(*plan, block_index, (int32_t)bs, (int32_t)nh, (int32_t)nq, &w)) return 0;
    work[0] = w.b;
    work[1] = w.h;
    work[2] = w.q_begin;
    work[3] = w.q_end;
    return 1;
}

// kind: 0 multi-scale deformable attention, 1 geometric kernel attention, >= 2: grid sampler with mode kind - 1
static int forward_common(int kind, const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                          const void* sampling_loc, const void* attn_weight, void* output, int dtype, int64_t bs,
                          int64_t nk, int64_t nh, int64_t hd, int64_t nl, int64_t nl_attn, int64_t nq, int64_t np,
                          void* hip_stream, int64_t grid_h = 0, int64_t grid_w = 0)
{
    const int meta64 = take_meta_flag(&dtype);
    const Dims d{bs, nk, nh, hd, nl, nl_attn, nq, np};
    const int gka = kind == 1, grid = kind >= 2 ? kind - 1 : 0;
    const char* who = grid ? "mxd_grid_sampler2d_forward" : gka ? "mxd_gka_forward" : "mxd_msda_forward";
    int rc = check_dims(dtype, d);
    if (rc != MXD_OK) return rc;
    if (!value || !sampling_loc || !output || (!grid && (!spatial_shapes || !level_start_index || !attn_weight)))
        return fail(MXD_E_NULL, "%s: NULL data pointer", who);
    int align = ptr_align(value);
    if (ptr_align(output) < align) align = ptr_align(output);
    mxd::KArgs a;
    memset(&a, 0, sizeof(a));
    rc = ensure_device_ready();
    if (rc != MXD_OK) return rc;
    int cache = kind == 0;
    // (the one-workgroup-per-CU form reads a location pair with one load)
    int cu = kind == 0 && ptr_align(sampling_loc) >= 2 * elem_size(dtype);
    rc = make_plan(0, dtype, d, align, &a.plan, &cache, &cu);
    if (rc != MXD_OK) return rc;
    fill_args(&a, dtype, d);
    a.meta_i64 = meta64;
    a.value = value;
    a.shapes = spatial_shapes;
    a.lsi = level_start_index;
    a.loc = sampling_loc;
    a.attn = attn_weight;
    a.out = output;
    a.gka = gka;
    a.grid = grid;
    a.grid_h = (int32_t)grid_h;
    a.grid_w = (int32_t)grid_w;
    a.lds_cache_bytes = cache;
    a.fwd_ahead = tuning().fwd_ahead;
    a.fwd_cu_flip = forward_cu_flip(dtype);
    const hipError_t e = cu ? mxd::launch_forward_cu(dtype, a, static_cast<hipStream_t>(hip_stream))
                            : mxd::launch_forward(dtype, a, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(MXD_E_LAUNCH, "%s: launch failed: %s", who, hipGetErrorString(e));
    return MXD_OK;
}

int mxd_msda_forward(const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                     const void* sampling_loc, const void* attn_weight, void* output, int dtype, int64_t bs, int64_t nk,
                     int64_t nh, int64_t hd, int64_t nl, int64_t nl_attn, int64_t nq, int64_t np, void* hip_stream)
{
    return forward_common(0, value, spatial_shapes, level_start_index, sampling_loc, attn_weight, output, dtype, bs, nk,
                          nh, hd, nl, nl_attn, nq, np, hip_stream);
}

int mxd_gka_forward(const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                    const void* sampling_locations, const void* attn_weights, void* output, int dtype, int64_t bs,
                    int64_t nk, int64_t nh, int64_t hd, int64_t nl, int64_t nq, int64_t np, void* hip_stream)
{
    return forward_common(1, value, spatial_shapes, level_start_index, sampling_locations, attn_weights, output, dtype,
                          bs, nk, nh, hd, nl, nl, nq, np, hip_stream);
}

static int grid_mode(int interpolation_mode, int padding_mode, int align_corners)
{
    if (interpolation_mode != 0) return fail(MXD_E_SHAPE, "grid_sampler2d: only bilinear interpolation (0) is built, got %d", interpolation_mode);
    if (padding_mode != 0 && padding_mode != 1)
        return fail(MXD_E_SHAPE, "grid_sampler2d: padding_mode must be 0 (zeros) or 1 (border), got %d", padding_mode);
    return 1 + padding_mode + (align_corners ? 2 : 0);
}

int mxd_grid_sampler2d_forward(const void* input_nhwc, const void* grid, void* output_nhwc, int dtype, int64_t n,
                               int64_t c, int64_t h_in, int64_t w_in, int64_t h_out, int64_t w_out,
                               int interpolation_mode, int padding_mode, int align_corners, void* hip_stream)
{
    const int mode = grid_mode(interpolation_mode, padding_mode, align_corners);
    if (mode < 0) return mode;
    if (h_in <= 0 || w_in <= 0 || h_in * w_in >= (int64_t(1) << 31))
        return fail(MXD_E_SHAPE, "grid_sampler2d: input of %lld x %lld pixels is beyond what this build indexes", (long long)h_in, (long long)w_in);
    return forward_common(1 + mode, input_nhwc, nullptr, nullptr, grid, nullptr, output_nhwc, dtype, n, h_in * w_in, 1, c, 1,
                          1, h_out * w_out, 1, hip_stream, h_in, w_in);
}

int mxd_msda_fused_forward(const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                           const void* reference_points, int ref_dim, const void* sampling_offsets,
                           const void* attn_logits, void* output, int dtype, int64_t bs, int64_t nk, int64_t nh,
                           int64_t hd, int64_t nl, int64_t nq, int64_t np, void* hip_stream)
{
    const int meta64 = take_meta_flag(&dtype);
    const Dims d{bs, nk, nh, hd, nl, nl, nq, np};
    int rc = check_dims(dtype, d);
    if (rc != MXD_OK) return rc;
    if (!value || !spatial_shapes || !level_start_index || !reference_points || !sampling_offsets || !attn_logits || !output)
        return fail(MXD_E_NULL, "mxd_msda_fused_forward: NULL data pointer");
    if (ref_dim != 2 && ref_dim != 4)
        return fail(MXD_E_SHAPE, "Last dim of reference_points must be 2 or 4, but get %d instead.", ref_dim);
    int align = ptr_align(value);
    if (ptr_align(output) < align) align = ptr_align(output);
    mxd::KArgs a;
    memset(&a, 0, sizeof(a));
    rc = ensure_device_ready();
    if (rc != MXD_OK) return rc;
    // The one-workgroup-per-CU form takes reference points (x, y) and units of one chunk (the softmax is formed by the
    // unit's lanes from the logits they hold); it reads offset pairs and reference points with one load each.
    int cache = 0, cu = ref_dim == 2 && nl * np <= mxd::kChunk && ptr_align(sampling_offsets) >= 2 * elem_size(dtype) &&
                        ptr_align(reference_points) >= 2 * elem_size(dtype);
    if (cu) {
        cache = 1;
        rc = make_plan(0, dtype, d, align, &a.plan, &cache, &cu);
        if (rc != MXD_OK) return rc;
    }
    if (!cu) {
        cache = 0;
        rc = make_plan(0, dtype, d, align, &a.plan);
        if (rc != MXD_OK) return rc;
    }
    fill_args(&a, dtype, d);
    a.meta_i64 = meta64;
    a.value = value;
    a.shapes = spatial_shapes;
    a.lsi = level_start_index;
    a.loc = sampling_offsets;
    a.attn = attn_logits;
    a.ref = reference_points;
    a.ref_dim = ref_dim;
    a.out = output;
    a.lds_cache_bytes = cache;
    a.fwd_cu_flip = forward_cu_flip(dtype);
    const hipError_t e = cu ? mxd::launch_forward_cu(dtype, a, static_cast<hipStream_t>(hip_stream))
                            : mxd::launch_forward(dtype, a, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(MXD_E_LAUNCH, "mxd_msda_fused_forward: launch failed: %s", hipGetErrorString(e));
    return MXD_OK;
}

size_t mxd_msda_backward_workspace_bytes(int dtype, int64_t bs, int64_t nk, int64_t nh, int64_t hd, int64_t nl,
                                         int64_t nl_attn, int64_t nq, int64_t np)
{
    take_meta_flag(&dtype);
    const Dims d{bs, nk, nh, hd, nl, nl_attn, nq, np};
    if (check_dims(dtype, d) != MXD_OK) return 0;
    return bwd_workspace_bytes(dtype, d);
}

// What the fused form adds to a backward call.
struct FusedBackward {
    const void* ref;
    int ref_dim;
    const void* out;   // forward result
    void* grad_ref;    // may be nullptr
};

static size_t fused_part_bytes(const Dims& d, int ref_dim)
{
    return (((size_t)d.nh * d.bs * d.nq * d.nl * ref_dim * sizeof(float)) + 15) & ~(size_t)15;
}

static int backward_common(int kind, const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                           const void* sampling_loc, const void* attn_weight, const void* grad_output, void* grad_value,
                           void* grad_loc, void* grad_attn, void* workspace, size_t workspace_bytes, int dtype,
                           int64_t bs, int64_t nk, int64_t nh, int64_t hd, int64_t nl, int64_t nl_attn, int64_t nq,
                           int64_t np, int flags, void* hip_stream, int64_t grid_h = 0, int64_t grid_w = 0,
                           const FusedBackward* fused = nullptr)
{
    const int meta64 = take_meta_flag(&dtype);
    const Dims d{bs, nk, nh, hd, nl, nl_attn, nq, np};
    const int gka = kind == 1, grid = kind >= 2 ? kind - 1 : 0;
    const char* who = fused  ? "mxd_msda_fused_backward"
                      : grid ? "mxd_grid_sampler2d_backward"
                      : gka  ? "mxd_gka_backward"
                             : "mxd_msda_backward";
    int rc = check_dims(dtype, d);
    if (rc != MXD_OK) return rc;
    if (!value || !sampling_loc || !grad_output || !grad_value || (!grad_loc && !gka) || (!grad_attn && !grid) ||
        (!grid && (!spatial_shapes || !level_start_index || !attn_weight)))
        return fail(MXD_E_NULL, "%s: NULL data pointer", who);
    if (fused && (!fused->ref || !fused->out)) return fail(MXD_E_NULL, "%s: NULL data pointer", who);
    if (fused && fused->ref_dim != 2 && fused->ref_dim != 4)
        return fail(MXD_E_SHAPE, "Last dim of reference_points must be 2 or 4, but get %d instead.", fused->ref_dim);
    int align = ptr_align(value);
    if (ptr_align(grad_output) < align) align = ptr_align(grad_output);
    mxd::KArgs a;
    memset(&a, 0, sizeof(a));
    rc = make_plan(1, dtype, d, align, &a.plan);
    if (rc != MXD_OK) return rc;
    const BwdLayout L = bwd_layout(dtype, d, a.plan.vec >= 4);  // (as make_plan laid the first kernel's LDS out)
    const size_t part_bytes = (fused && fused->grad_ref) ? fused_part_bytes(d, fused->ref_dim) : 0;
    const size_t need = L.total + part_bytes;
    if (need > 0 && (!workspace || workspace_bytes < need))
        return fail(MXD_E_WORKSPACE, "%s: workspace of %zu bytes required, %zu given", who, need,
                    workspace ? workspace_bytes : (size_t)0);
    if (need > 0 && (reinterpret_cast<uintptr_t>(workspace) & 15u))
        return fail(MXD_E_WORKSPACE, "%s: workspace must be 16-byte aligned", who);
    const bool half = elem_size(dtype) == 2;
    if ((flags & MXD_BWD_ACCUMULATE) && half)
        return fail(MXD_E_DTYPE, "%s: MXD_BWD_ACCUMULATE is only available for float32", who);
    char* ws = static_cast<char*>(workspace);
    float* image = half ? reinterpret_cast<float*>(ws + L.tbl_bytes + L.rec_bytes) : static_cast<float*>(grad_value);
    if (reinterpret_cast<uintptr_t>(image) & 3u) return fail(MXD_E_SHAPE, "%s: grad_value is not 4-byte aligned", who);
    fill_args(&a, dtype, d);
    a.tile_px_log2 = L.tile_px_log2;
    a.unit_split_log2 = unit_split_log2(a.plan);
    a.rec_lds_bytes = plan_record_buffer(&a.plan, L, d, dtype, !gka && !grid, a.unit_split_log2);
    a.bwd_fixed = (tuning().bwd_fixed != 0 && (!fused || a.unit_split_log2 == 0) && !gka && !grid && L.tiles && a.plan.lanes_per_row == 8 &&
                   a.plan.units_per_wave == 8 && a.plan.npass == 1 && a.plan.iters == 1 && a.unit_split_log2 <= 1 &&
                   d.nl * d.np <= ((int64_t)mxd::kChunk << a.unit_split_log2) && a.rec_lds_bytes == 0)
                      ? 1 + a.unit_split_log2 : 0;
    if (tuning().bwd_fixed != 0 && !fused && !gka && !grid && L.tiles && a.plan.lanes_per_row == 16 && a.plan.units_per_wave == 4 &&
        a.plan.npass == 1 && a.plan.vec * (int)elem_size(dtype) == 16 && a.unit_split_log2 == 0)
        a.bwd_fixed = 3;
    a.meta_i64 = meta64;
    a.value = value;
    a.shapes = spatial_shapes;
    a.lsi = level_start_index;
    a.loc = sampling_loc;
    a.attn = attn_weight;
    a.grad_out = grad_output;
    a.grad_value = image;
    a.tbl = reinterpret_cast<uint32_t*>(ws);
    a.rec = reinterpret_cast<uint32_t*>(ws + L.tbl_bytes);
    a.nwg = (int32_t)L.nwg;
    a.rec_cap = (int32_t)L.rec_cap;
    a.tbl_stride = (int32_t)L.tbl_stride;
    a.grad_loc = grad_loc;
    a.grad_attn = grad_attn;
    a.gka = gka;
    a.grid = grid;
    a.grid_h = (int32_t)grid_h;
    a.grid_w = (int32_t)grid_w;
    float* part = nullptr;
    if (fused) {
        a.ref = fused->ref;
        a.ref_dim = fused->ref_dim;
        a.out = const_cast<void*>(fused->out);
        a.np_pow2 = (np & (np - 1)) == 0 && np <= 16;
        if (part_bytes > 0) part = reinterpret_cast<float*>(ws + L.total);
        a.grad_ref = part;
    }
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    const size_t n = (size_t)bs * nk * nh * hd;
    // every step that can fail for the sizes given comes before the first launch
    // (MXD_BWD_ANY_LAYOUT: the one-kernel form with global atomics, which takes level_start_index as it comes)
    const bool atomic_mode = !L.tiles || (flags & MXD_BWD_ANY_LAYOUT) != 0;
    mxd::TileArgs t;
    if (!atomic_mode) {
        rc = make_tile_args(d, L, a.plan.vec, (flags & MXD_BWD_ACCUMULATE) ? 1 : 0, &t, !fused && !gka && !grid);
        if (rc != MXD_OK) return rc;
        plan_image(&a, &t, half, (flags & MXD_BWD_ACCUMULATE) != 0, image, grad_value, hd);
    }
    hipError_t e = hipSuccess;
    // zero-fill of the image: by the first kernel's workgroups when the tile pass is the first to touch it and it
    // can be written in 16-byte pieces, by a kernel of its own otherwise
    const bool fill_inside = !atomic_mode && n % 4 == 0 && (reinterpret_cast<uintptr_t>(image) & 15u) == 0 &&
                             tuning().bwd_fill_kernel == 0;
    if (!(flags & MXD_BWD_ACCUMULATE)) {
        if (fill_inside) a.fill_n4 = n / 4;
        else e = mxd::launch_fill_zero(image, n, stream);
    }
    if (e == hipSuccess && part && !a.np_pow2) e = mxd::launch_fill_zero(part, part_bytes / sizeof(float), stream);
    if (e != hipSuccess) return fail(MXD_E_LAUNCH, "%s: zero-fill launch failed: %s", who, hipGetErrorString(e));
    e = mxd::launch_backward(dtype, a, atomic_mode, stream);
    if (e != hipSuccess) return fail(MXD_E_LAUNCH, "%s: launch failed: %s", who, hipGetErrorString(e));
    if (!atomic_mode) {
        e = mxd::launch_gradv_tiles(dtype, a, t, stream);
        if (e != hipSuccess) return fail(MXD_E_LAUNCH, "%s: tile kernel launch failed: %s", who, hipGetErrorString(e));
    }
    if (half) {
        e = a.sparse ? mxd::launch_round_rows(dtype, a, stream) : mxd::launch_round(dtype, image, grad_value, n, stream);
        if (e != hipSuccess) return fail(MXD_E_LAUNCH, "%s: rounding launch failed: %s", who, hipGetErrorString(e));
    }
    if (part) {
        e = mxd::launch_sum_heads(dtype, part, fused->grad_ref, (size_t)bs * nq * nl * fused->ref_dim, (int)nh, stream);
        if (e != hipSuccess) return fail(MXD_E_LAUNCH, "%s: head sum launch failed: %s", who, hipGetErrorString(e));
    }
    return MXD_OK;
}

size_t mxd_msda_fused_backward_workspace_bytes(int dtype, int64_t bs, int64_t nk, int64_t nh, int64_t hd,
                                               int64_t nl, int64_t nq, int64_t np, int ref_dim, int want_grad_ref)
{
    take_meta_flag(&dtype);
    const Dims d{bs, nk, nh, hd, nl, nl, nq, np};
    if (check_dims(dtype, d) != MXD_OK || (ref_dim != 2 && ref_dim != 4)) return 0;
    return bwd_workspace_bytes(dtype, d) + (want_grad_ref ? fused_part_bytes(d, ref_dim) : 0);
}

int mxd_msda_fused_backward(const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                            const void* reference_points, int ref_dim, const void* sampling_offsets,
                            const void* attn_logits, const void* output, const void* grad_output, void* grad_value,
                            void* grad_reference_points, void* grad_sampling_offsets, void* grad_attn_logits,
                            void* workspace, size_t workspace_bytes, int dtype, int64_t bs, int64_t nk, int64_t nh,
                            int64_t hd, int64_t nl, int64_t nq, int64_t np, int flags, void* hip_stream)
{
    const FusedBackward f{reference_points, ref_dim, output, grad_reference_points};
    return backward_common(0, value, spatial_shapes, level_start_index, sampling_offsets, attn_logits, grad_output,
                           grad_value, grad_sampling_offsets, grad_attn_logits, workspace, workspace_bytes, dtype, bs,
                           nk, nh, hd, nl, nl, nq, np, flags, hip_stream, 0, 0, &f);
}

int mxd_msda_backward(const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                      const void* sampling_loc, const void* attn_weight, const void* grad_output, void* grad_value,
                      void* grad_loc, void* grad_attn, void* workspace, size_t workspace_bytes, int dtype, int64_t bs,
                      int64_t nk, int64_t nh, int64_t hd, int64_t nl, int64_t nl_attn, int64_t nq, int64_t np,
                      int flags, void* hip_stream)
{
    return backward_common(0, value, spatial_shapes, level_start_index, sampling_loc, attn_weight, grad_output,
                           grad_value, grad_loc, grad_attn, workspace, workspace_bytes, dtype, bs, nk, nh, hd, nl,
                           nl_attn, nq, np, flags, hip_stream);
}

size_t mxd_msda_backward_static_limit(void) { return kStaticScratchBytes; }

int mxd_msda_backward_static(const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                             const void* sampling_loc, const void* attn_weight, const void* grad_output,
                             void* grad_value, void* grad_loc, void* grad_attn, int dtype, int64_t bs, int64_t nk,
                             int64_t nh, int64_t hd, int64_t nl, int64_t nl_attn, int64_t nq, int64_t np, int flags,
                             void* hip_stream)
{
    // (allocates nothing: the scratch is the library's own static device array; sizes beyond it are refused)
    const size_t need = mxd_msda_backward_workspace_bytes(dtype, bs, nk, nh, hd, nl, nl_attn, nq, np);
    if (need > kStaticScratchBytes)
        return fail(MXD_E_WORKSPACE,
                    "mxd_msda_backward_static: this problem needs %zu bytes of scratch, the static array holds %zu; "
                    "use mxd_msda_backward with a workspace",
                    need, kStaticScratchBytes);
    int rc = ensure_device_ready();
    if (rc != MXD_OK) return rc;
    void* ws = device_scratch();
    if (!ws) return fail(MXD_E_LAUNCH, "mxd_msda_backward_static: the static scratch array is not set up on this device");
    return backward_common(0, value, spatial_shapes, level_start_index, sampling_loc, attn_weight, grad_output,
                           grad_value, grad_loc, grad_attn, ws, kStaticScratchBytes, dtype, bs, nk, nh, hd, nl, nl_attn,
                           nq, np, flags, hip_stream);
}

size_t mxd_gka_backward_workspace_bytes(int dtype, int64_t bs, int64_t nk, int64_t nh, int64_t hd, int64_t nl,
                                        int64_t nq, int64_t np)
{
    return mxd_msda_backward_workspace_bytes(dtype, bs, nk, nh, hd, nl, nl, nq, np);
}

int mxd_gka_backward(const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                     const void* sampling_locations, const void* attn_weights, const void* grad_output,
                     void* grad_value, void* grad_attn_weights, void* workspace, size_t workspace_bytes, int dtype,
                     int64_t bs, int64_t nk, int64_t nh, int64_t hd, int64_t nl, int64_t nq, int64_t np,
                     void* hip_stream)
{
    return backward_common(1, value, spatial_shapes, level_start_index, sampling_locations, attn_weights, grad_output,
                           grad_value, nullptr, grad_attn_weights, workspace, workspace_bytes, dtype, bs, nk, nh, hd, nl,
                           nl, nq, np, 0, hip_stream);
}

size_t mxd_grid_sampler2d_backward_workspace_bytes(int dtype, int64_t n, int64_t c, int64_t h_in, int64_t w_in,
                                                   int64_t h_out, int64_t w_out)
{
    if (h_in <= 0 || w_in <= 0 || h_in * w_in >= (int64_t(1) << 31)) return 0;
    return mxd_msda_backward_workspace_bytes(dtype, n, h_in * w_in, 1, c, 1, 1, h_out * w_out, 1);
}

int mxd_grid_sampler2d_backward(const void* grad_output_nhwc, const void* input_nhwc, const void* grid,
                                void* grad_input_nhwc, void* grad_grid, void* workspace, size_t workspace_bytes,
                                int dtype, int64_t n, int64_t c, int64_t h_in, int64_t w_in, int64_t h_out,
                                int64_t w_out, int interpolation_mode, int padding_mode, int align_corners,
                                void* hip_stream)
{
    const int mode = grid_mode(interpolation_mode, padding_mode, align_corners);
    if (mode < 0) return mode;
    if (h_in <= 0 || w_in <= 0 || h_in * w_in >= (int64_t(1) << 31))
        return fail(MXD_E_SHAPE, "grid_sampler2d: input of %lld x %lld pixels is beyond what this build indexes", (long long)h_in, (long long)w_in);
    return backward_common(1 + mode, input_nhwc, nullptr, nullptr, grid, nullptr, grad_output_nhwc, grad_input_nhwc,
                           grad_grid, nullptr, workspace, workspace_bytes, dtype, n, h_in * w_in, 1, c, 1, 1,
                           h_out * w_out, 1, 0, hip_stream, h_in, w_in);
}

int mxd_dagg_forward(const void* mc_ms_feat, const int32_t* spatial_shape, const int32_t* scale_start_index,
                     const void* sampling_location, const void* weights, void* output, int dtype, int64_t bs,
                     int64_t num_feat, int64_t num_embeds, int64_t num_cams, int64_t num_scale, int64_t num_anchors,
                     int64_t num_pts, int64_t num_groups, void* hip_stream)
{
    const int meta64 = take_meta_flag(&dtype);
    Dims d;
    int rc = dagg_dims(dtype, bs, num_feat, num_embeds, num_cams, num_scale, num_anchors, num_pts, num_groups, &d);
    if (rc != MXD_OK) return rc;
    if (!mc_ms_feat || !spatial_shape || !scale_start_index || !sampling_location || !weights || !output)
        return fail(MXD_E_NULL, "mxd_dagg_forward: NULL data pointer");
    int align = ptr_align(mc_ms_feat);
    if (ptr_align(output) < align) align = ptr_align(output);
    mxd::KArgs a;
    memset(&a, 0, sizeof(a));
    rc = make_plan(0, dtype, d, align, &a.plan);
    if (rc != MXD_OK) return rc;
    fill_args(&a, dtype, d);
    a.meta_i64 = meta64;
    fill_dagg(&a, num_cams, num_scale);
    a.value = mc_ms_feat;
    a.shapes = spatial_shape;
    a.lsi = scale_start_index;
    a.loc = sampling_location;
    a.attn = weights;
    a.out = output;
    const hipError_t e = mxd::launch_forward(dtype, a, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(MXD_E_LAUNCH, "mxd_dagg_forward: launch failed: %s", hipGetErrorString(e));
    return MXD_OK;
}

size_t mxd_dagg_backward_workspace_bytes(int dtype, int64_t bs, int64_t num_feat, int64_t num_embeds, int64_t num_cams,
                                         int64_t num_scale, int64_t num_anchors, int64_t num_pts, int64_t num_groups)
{
    take_meta_flag(&dtype);
    Dims d;
    if (dagg_dims(dtype, bs, num_feat, num_embeds, num_cams, num_scale, num_anchors, num_pts, num_groups, &d) != MXD_OK)
        return 0;
    return bwd_workspace_bytes(dtype, d) + dagg_part_bytes(d, num_cams);
}

int mxd_dagg_backward(const void* mc_ms_feat, const int32_t* spatial_shape, const int32_t* scale_start_index,
                      const void* sampling_location, const void* weights, const void* grad_output,
                      void* grad_mc_ms_feat, void* grad_sampling_location, void* grad_weights, void* workspace,
                      size_t workspace_bytes, int dtype, int64_t bs, int64_t num_feat, int64_t num_embeds,
                      int64_t num_cams, int64_t num_scale, int64_t num_anchors, int64_t num_pts, int64_t num_groups,
                      void* hip_stream)
{
    const int meta64 = take_meta_flag(&dtype);
    Dims d;
    int rc = dagg_dims(dtype, bs, num_feat, num_embeds, num_cams, num_scale, num_anchors, num_pts, num_groups, &d);
    if (rc != MXD_OK) return rc;
    if (!mc_ms_feat || !spatial_shape || !scale_start_index || !sampling_location || !weights || !grad_output ||
        !grad_mc_ms_feat || !grad_sampling_location || !grad_weights)
        return fail(MXD_E_NULL, "mxd_dagg_backward: NULL data pointer");
    int align = ptr_align(mc_ms_feat);
    if (ptr_align(grad_output) < align) align = ptr_align(grad_output);
    mxd::KArgs a;
    memset(&a, 0, sizeof(a));
    rc = make_plan(1, dtype, d, align, &a.plan);
    if (rc != MXD_OK) return rc;
    const BwdLayout L = bwd_layout(dtype, d, a.plan.vec >= 4);  // (as make_plan laid the first kernel's LDS out)
    const size_t part_bytes = dagg_part_bytes(d, num_cams);
    const size_t need = L.total + part_bytes;
    if (!workspace || workspace_bytes < need)
        return fail(MXD_E_WORKSPACE, "mxd_dagg_backward: workspace of %zu bytes required, %zu given", need,
                    workspace ? workspace_bytes : (size_t)0);
    if (reinterpret_cast<uintptr_t>(workspace) & 15u)
        return fail(MXD_E_WORKSPACE, "mxd_dagg_backward: workspace must be 16-byte aligned");
    const bool half = elem_size(dtype) == 2;
    char* ws = static_cast<char*>(workspace);
    float* image = half ? reinterpret_cast<float*>(ws + L.tbl_bytes + L.rec_bytes) : static_cast<float*>(grad_mc_ms_feat);
    float* part = reinterpret_cast<float*>(ws + L.total);
    if (reinterpret_cast<uintptr_t>(image) & 3u) return fail(MXD_E_SHAPE, "mxd_dagg_backward: grad_mc_ms_feat is not 4-byte aligned");
    fill_args(&a, dtype, d);
    a.tile_px_log2 = L.tile_px_log2;
    a.unit_split_log2 = unit_split_log2(a.plan);
    a.rec_lds_bytes = plan_record_buffer(&a.plan, L, d, dtype, false, a.unit_split_log2);
    a.meta_i64 = meta64;
    fill_dagg(&a, num_cams, num_scale);
    a.value = mc_ms_feat;
    a.shapes = spatial_shape;
    a.lsi = scale_start_index;
    a.loc = sampling_location;
    a.attn = weights;
    a.grad_out = grad_output;
    a.grad_value = image;
    a.tbl = reinterpret_cast<uint32_t*>(ws);
    a.rec = reinterpret_cast<uint32_t*>(ws + L.tbl_bytes);
    a.nwg = (int32_t)L.nwg;
    a.rec_cap = (int32_t)L.rec_cap;
    a.tbl_stride = (int32_t)L.tbl_stride;
    a.grad_loc = part;  // per-head partial images, summed below
    a.grad_attn = grad_weights;
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    const size_t n = (size_t)bs * num_feat * num_embeds;
    // every step that can fail for the sizes given comes before the first launch
    const bool atomic_mode = !L.tiles;
    mxd::TileArgs t;
    if (!atomic_mode) {
        rc = make_tile_args(d, L, a.plan.vec, 0, &t);
        if (rc != MXD_OK) return rc;
        plan_image(&a, &t, half, false, image, grad_mc_ms_feat, d.hd);
    }
    hipError_t e = hipSuccess;
    if (L.tiles && n % 4 == 0 && (reinterpret_cast<uintptr_t>(image) & 15u) == 0 && tuning().bwd_fill_kernel == 0)
        a.fill_n4 = n / 4;  // zero-filled by the first kernel's workgroups
    else
        e = mxd::launch_fill_zero(image, n, stream);
    if (e == hipSuccess && !a.sc_pow2) e = mxd::launch_fill_zero(part, part_bytes / sizeof(float), stream);
    if (e != hipSuccess) return fail(MXD_E_LAUNCH, "mxd_dagg_backward: zero-fill launch failed: %s", hipGetErrorString(e));
    e = mxd::launch_backward(dtype, a, atomic_mode, stream);
    if (e != hipSuccess) return fail(MXD_E_LAUNCH, "mxd_dagg_backward: launch failed: %s", hipGetErrorString(e));
    if (!atomic_mode) {
        e = mxd::launch_gradv_tiles(dtype, a, t, stream);
        if (e != hipSuccess) return fail(MXD_E_LAUNCH, "mxd_dagg_backward: tile kernel launch failed: %s", hipGetErrorString(e));
    }
    if (half) {
        e = a.sparse ? mxd::launch_round_rows(dtype, a, stream) : mxd::launch_round(dtype, image, grad_mc_ms_feat, n, stream);
        if (e != hipSuccess) return fail(MXD_E_LAUNCH, "mxd_dagg_backward: rounding launch failed: %s", hipGetErrorString(e));
    }
    e = mxd::launch_sum_heads(dtype, part, grad_sampling_location, (size_t)bs * num_anchors * num_pts * num_cams * 2,
                              (int)num_groups, stream);
    if (e != hipSuccess) return fail(MXD_E_LAUNCH, "mxd_dagg_backward: head sum launch failed: %s", hipGetErrorString(e));
    return MXD_OK;
}

}  // extern "C"
