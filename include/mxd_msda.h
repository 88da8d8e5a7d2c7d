/*
 * mxd_msda.h -- C ABI of the MI355X (gfx950) multi-scale deformable attention library.
 *
 * This is the drop-in boundary for the reference's binding layer: the two functions
 * the reference exports from its compiled module,
 *     at::Tensor multi_scale_deformable_attn(value, value_spatial_shapes,
 *                    value_level_start_index, sampling_locations, attention_weights)
 *     std::tuple<at::Tensor, at::Tensor, at::Tensor> multi_scale_deformable_attn_backward(
 *                    ..., grad_output)
 * (include/csrc/functions.h:58-64, bound in mx_driving/csrc/pybind.cpp:110-111, implemented
 * in mx_driving/csrc/MultiScaleDeformableAttn.cpp:28-118) reduce, once tensors are
 * unwrapped, to the entry points below: plain device pointers, sizes, a dtype code and a
 * HIP stream.  No C++ or torch types cross this boundary.
 *
 * Conventions
 *   - Every data pointer is DEVICE memory, dense row-major, borrowed for the duration of
 *     the enqueued work; the library allocates and frees nothing.
 *   - Work is enqueued on `hip_stream` (a hipStream_t; NULL = the default stream) of the
 *     CURRENT device and the call returns without synchronising.
 *   - Return value: 0 on success, a negative MXD_E_* code otherwise; the message for the
 *     calling thread's last failure is returned by mxd_msda_last_error().
 *   - Thread safe.  Process-wide state: the tuning knobs (MXD_MSDA_* environment variables, read once on first
 *     use), one "set up" flag per device (the first call on a device opts its large-LDS kernels in; mxd_msda_init()
 *     does the same ahead of time), and the thread-local error message.
 *
 * Layouts (T = element type selected by `dtype`)
 *   value            T   [bs, nk, nh, hd]
 *   spatial_shapes   i32 [nl, 2]   (H, W) per level
 *   level_start_idx  i32 [nl]
 *   sampling_loc     T   [bs, nq, nh, nl_attn, np, 2]   (x, y) normalised to [0, 1]
 *   attn_weight      T   [bs, nq, nh, nl_attn, np]
 *   output           T   [bs, nq, nh*hd]
 *   grad_output      T   [bs, nq, nh*hd]
 *   grad_value       T   [bs, nk, nh, hd]
 *   grad_loc         T   like sampling_loc,   grad_attn  T  like attn_weight
 * nl_attn >= nl: only the first nl levels are sampled; the remaining slots of grad_loc and
 * grad_attn are written as zero (mx_driving/csrc/MultiScaleDeformableAttn.cpp:97-101).
 *
 * Limits (the first two are the reference's, MultiScaleDeformableAttn.cpp:46-48):
 *   hd <= 256;  nl*np <= 64 is NOT required here (any nl <= 64, any np);
 *   nk*nh*hd*4 bytes (one batch element of value, counted at 4 bytes per element) < 2 GiB.
 */
#ifndef MXD_MSDA_H
#define MXD_MSDA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MXD_MSDA_VERSION 103 /* major*10000 + minor*100 + patch */

/* dtype codes */
#define MXD_DTYPE_F32 0
#define MXD_DTYPE_F16 1
#define MXD_DTYPE_BF16 2
/* OR into `dtype`: spatial_shapes / level_start_index (spatial_shape / scale_start_index) point at int64 elements
 * instead of int32 ones.  The reference's Python layer receives these tensors as int64 and casts them to int32 on
 * every call (mx_driving/ops/multi_scale_deformable_attn.py:33-34); with this flag a binding hands them over as they
 * are and the two cast kernels are not launched.  Values must fit int32 as before. */
#define MXD_META_I64 0x100

/* error codes */
#define MXD_OK 0
#define MXD_E_DTYPE (-1)    /* unsupported dtype code                                   */
#define MXD_E_SHAPE (-2)    /* a size is non-positive or violates a documented limit    */
#define MXD_E_NULL (-3)     /* a required pointer is NULL                               */
#define MXD_E_WORKSPACE (-4) /* workspace missing or too small                          */
#define MXD_E_LAUNCH (-5)   /* the HIP runtime refused the launch                       */

/* Launch geometry chosen for a problem; filled by mxd_msda_make_plan(), read-only diagnostics.
 * Replaces the reference's host "tiling" step
 * (kernels/multi_scale_deformable_attn/op_host/multi_scale_deformable_attn.cpp:32-114,
 *  kernels/multi_scale_deformable_attn/op_host/multi_scale_deformable_attn_grad.cpp:35-87). */
typedef struct mxd_msda_plan {
    int32_t vec;             /* elements of T one lane moves per row access (1,2,4,8)   */
    int32_t lanes_per_row;   /* power of two, 4..64: lanes that share one value row     */
    int32_t npass;           /* row passes per lane when hd > lanes_per_row*vec         */
    int32_t units_per_wave;  /* (query, head) units a wavefront handles side by side    */
    int32_t waves_per_block;
    int32_t iters;           /* wave-steps each wavefront runs                          */
    int32_t tile_q;          /* queries per workgroup = units_per_wave*waves*iters (half of that where the
                                backward gives a query of 17 to 32 samples two units, 16 samples each) */
    int32_t ntiles;          /* query tiles per (batch, head)                           */
    int32_t xcd_mode;        /* 0 plain; 1 nh % 8 == 0 (heads pinned to an XCD);
                                2 8 % nh == 0 (several XCDs share a head)               */
    int32_t heads_per_xcd;   /* mode 1                                                  */
    int32_t xcds_per_head;   /* mode 2                                                  */
    int32_t tiles_per_part;  /* mode 2: tiles each of the XCDs sharing a head takes     */
    uint32_t grid;           /* workgroups                                              */
    uint32_t block;          /* threads per workgroup                                   */
    uint32_t lds_bytes;      /* dynamic LDS per workgroup                               */
} mxd_msda_plan;

/* Library version (MXD_MSDA_VERSION of the build). */
int mxd_msda_version(void);

/* Message of the calling thread's most recent failed call ("" if none). */
const char* mxd_msda_last_error(void);

/* Optional.  Does, for the CURRENT device, the one-time set-up that the compute entry points otherwise do on their
 * first call there (function attributes of the kernels that use more than 64 KiB of LDS): call it once per device
 * before capturing the library's launches in a HIP graph without a warm-up call.  Returns 0 or MXD_E_LAUNCH.
 * No counterpart in the reference (its launcher resolves its symbols lazily, include/csrc/OpApiCommon.h:117-132). */
int mxd_msda_init(void);

/* Reads the MXD_MSDA_* tuning variables from the environment again (they are otherwise read once per process).
 * A hook for tests and experiments; must not run while another thread is inside the library. */
void mxd_msda_reload_tuning(void);

/* Compute the launch geometry for a problem without touching the GPU.
 * `backward` = 0/1.  `align_bytes` = the largest power of two (<= 16) dividing every data
 * pointer that will be passed; use 16 when unknown (torch allocations are 256-byte aligned).
 * Same argument checks and limits as the compute entry points. */
int mxd_msda_make_plan(int backward, int dtype, int64_t bs, int64_t nk, int64_t nh, int64_t hd, int64_t nl,
                       int64_t nl_attn, int64_t nq, int64_t np, int align_bytes, mxd_msda_plan* plan);

/* Which slice of the problem workgroup `block_index` of a plan works on: writes
 * {batch, head, first query, one past the last query} to `work` and returns 1, or returns 0
 * when that workgroup is idle.  Host-side twin of the kernels' own decoding, for checking that
 * a plan covers every (batch, head, query) exactly once; never needed to run the operator. */
int mxd_msda_decode_block(const mxd_msda_plan* plan, uint32_t block_index, int64_t bs, int64_t nh, int64_t nq,
                          int32_t work[4]);

/* Forward.  Replaces multi_scale_deformable_attn
 * (mx_driving/csrc/MultiScaleDeformableAttn.cpp:28-66): reads T natively, accumulates in
 * fp32, rounds once at the store.  Samples outside the image, and NaN/Inf locations,
 * contribute nothing. */
int mxd_msda_forward(const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                     const void* sampling_loc, const void* attn_weight, void* output, int dtype, int64_t bs,
                     int64_t nk, int64_t nh, int64_t hd, int64_t nl, int64_t nl_attn, int64_t nq, int64_t np,
                     void* hip_stream);

/* Forward with the caller's pre-processing folded in.  No single function of the reference
 * corresponds to it: it replaces, together, the softmax over the nl*np attention logits, the
 * sampling-location arithmetic and the operator call of the deformable-attention modules the
 * reference's model recipes patch (model_examples/Deformable-DETR/Deformable-DETR_npu.patch:626-652,
 * model_examples/BEVFormer/bev_former_config.patch:404-421):
 *     attn = softmax(attn_logits[b,q,h,:])                                 [bs,nq,nh,nl*np]
 *     loc  = ref[b,q,l,:2] + off[b,q,h,l,p,:] / (W_l, H_l)                 ref_dim == 2
 *     loc  = ref[b,q,l,:2] + off[b,q,h,l,p,:] / np * ref[b,q,l,2:] * 0.5   ref_dim == 4
 *     output = mxd_msda_forward(value, ..., loc, attn)
 * reference_points [bs,nq,nl,ref_dim], sampling_offsets [bs,nq,nh,nl,np,2] and attn_logits
 * [bs,nq,nh,nl*np] have value's dtype; loc and attn are never written to memory. */
int mxd_msda_fused_forward(const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                           const void* reference_points, int ref_dim, const void* sampling_offsets,
                           const void* attn_logits, void* output, int dtype, int64_t bs, int64_t nk, int64_t nh,
                           int64_t hd, int64_t nl, int64_t nq, int64_t np, void* hip_stream);

/* Backward of mxd_msda_fused_forward: the operator's backward with the chain rule through the
 * softmax and through the location arithmetic applied inside the first kernel, so that neither
 * locations and weights nor their gradients reach memory.  `output` is the forward result (the
 * softmax backward uses, per (query, head), the dot product of its row with the grad_output row).
 * grad_sampling_offsets and grad_attn_logits have the shapes and dtype of their inputs and are
 * fully overwritten; grad_value as in mxd_msda_backward (flags: MXD_BWD_ACCUMULATE).
 * grad_reference_points [bs,nq,nl,ref_dim] may be NULL when the caller does not need it (the sum
 * over heads then is skipped); pass the same choice (want_grad_ref 0/1) to the workspace query,
 * which adds nh*bs*nq*nl*ref_dim floats of per-head partial sums to the operator's own scratch. */
size_t mxd_msda_fused_backward_workspace_bytes(int dtype, int64_t bs, int64_t nk, int64_t nh, int64_t hd,
                                               int64_t nl, int64_t nq, int64_t np, int ref_dim, int want_grad_ref);
int mxd_msda_fused_backward(const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                            const void* reference_points, int ref_dim, const void* sampling_offsets,
                            const void* attn_logits, const void* output, const void* grad_output, void* grad_value,
                            void* grad_reference_points, void* grad_sampling_offsets, void* grad_attn_logits,
                            void* workspace, size_t workspace_bytes, int dtype, int64_t bs, int64_t nk, int64_t nh,
                            int64_t hd, int64_t nl, int64_t nq, int64_t np, int flags, void* hip_stream);

/* Bytes of scratch mxd_msda_backward needs (0 if the sizes are invalid, and for float32 sizes
 * that take the one-kernel path with global atomics).  It holds the hand-over between the two
 * backward kernels -- a table of run starts and two 12-byte records per sample, written
 * sorted by tile by the first kernel and streamed by the second -- and, for fp16/bf16, an
 * fp32 image of grad_value (bs*nk*nh*hd*4) that the sums are formed in before one rounding
 * pass (the reference keeps the same fp32 buffer, MultiScaleDeformableAttn.cpp:93,103-113;
 * its launcher also allocates a workspace per call, include/csrc/OpApiCommon.h:589-595). */
size_t mxd_msda_backward_workspace_bytes(int dtype, int64_t bs, int64_t nk, int64_t nh, int64_t hd, int64_t nl,
                                         int64_t nl_attn, int64_t nq, int64_t np);

/* flags of mxd_msda_backward */
#define MXD_BWD_ACCUMULATE 1 /* fp32 only: add into the caller's grad_value instead of zero-filling it
                                first (gradient accumulation; the caller owns the initial contents) */
#define MXD_BWD_ANY_LAYOUT 2 /* take the one-kernel backward that adds to grad_value with global atomics (several
                                times slower).  level_start_index is the caller's and is honoured as it comes by every
                                form of the backward: the levels may leave keys uncovered, come in any order and
                                overlap, as for the reference's atomic-add kernel
                                (op_kernel/multi_scale_deformable_attn_grad.cpp:181-186).  One case is slow by default:
                                levels that overlap so far that they have more than num_keys/T + num_levels tiles of
                                T pixels between them (T = 512 for heads of up to 32 channels, 256 for up to 64, 128
                                beyond) -- mxd_msda_backward then adds the levels beyond that sample by sample.  The
                                fused form and the sibling operators have no such fallback: there the default form
                                leaves those levels out of grad_value, and this flag (or MXD_MSDA_BWD_ATOMIC=1 in the
                                environment) asks for the form that does not care */

/* Backward.  Replaces multi_scale_deformable_attn_backward
 * (mx_driving/csrc/MultiScaleDeformableAttn.cpp:68-118).  On `hip_stream`, in order:
 * zero-fills the fp32 accumulation image of grad_value (grad_value itself for fp32, the
 * workspace otherwise; skipped under MXD_BWD_ACCUMULATE), runs the gradient kernels, and for
 * fp16/bf16 rounds the image into grad_value.  Every element of the three outputs is written.
 * `workspace` (16-byte aligned, at least mxd_msda_backward_workspace_bytes()) is required
 * whenever that size is not 0. */
int mxd_msda_backward(const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                      const void* sampling_loc, const void* attn_weight, const void* grad_output, void* grad_value,
                      void* grad_loc, void* grad_attn, void* workspace, size_t workspace_bytes, int dtype,
                      int64_t bs, int64_t nk, int64_t nh, int64_t hd, int64_t nl, int64_t nl_attn, int64_t nq,
                      int64_t np, int flags, void* hip_stream);

/* Backward without a workspace argument and without any allocation.  No counterpart in the reference: it is for
 * callers that can neither call hipMalloc nor hand over scratch memory -- code under HIP graph capture, tight serving
 * loops, harnesses that forbid allocation.  It is mxd_msda_backward with the hand-over between its kernels (and the
 * fp32 image for 16-bit dtypes) in a static device array of MXD_MSDA_STATIC_SCRATCH_BYTES that every GPU the library
 * runs on holds until the process ends.  Problems whose mxd_msda_backward_workspace_bytes() exceeds that size are
 * refused with MXD_E_WORKSPACE.  All calls on one GPU share the array: calls that overlap in time on one GPU (other
 * streams, other threads) race; calls on one stream do not.  Nothing in the array has to survive between calls or
 * start at zero (the image is zero-filled by the call itself).  mxd_msda_backward_static_limit() returns the size. */
#define MXD_MSDA_STATIC_SCRATCH_BYTES (32u << 20)
size_t mxd_msda_backward_static_limit(void);
int mxd_msda_backward_static(const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                             const void* sampling_loc, const void* attn_weight, const void* grad_output,
                             void* grad_value, void* grad_loc, void* grad_attn, int dtype, int64_t bs, int64_t nk,
                             int64_t nh, int64_t hd, int64_t nl, int64_t nl_attn, int64_t nq, int64_t np, int flags,
                             void* hip_stream);

/* ---- deformable aggregation (Sparse4D / SparseDrive feature sampling) ------------------------
 * Replaces deformable_aggregation / deformable_aggregation_backward
 * (mx_driving/csrc/DeformableAggregation.cpp:20-82) with the same tensors:
 *   mc_ms_feat [bs, num_feat, num_embeds]        spatial_shape [num_cams, num_scale, 2] = (H, W), int32
 *   scale_start_index [num_cams, num_scale], int32
 *   sampling_location [bs, num_anchors, num_pts, num_cams, 2] = (x, y)
 *   weights [bs, num_anchors, num_pts, num_cams, num_scale, num_groups]     output [bs, num_anchors, num_embeds]
 * output[b,a,c] = sum over (pt, cam, scale) of weights[..., group(c)] * bilinear(feat of (cam, scale), location);
 * a location counts only when 0 < x < 1 and 0 < y < 1; zero padding outside the map.  The same kernels as
 * multi-scale deformable attention run it (group = head, (camera, scale) = level, anchor = query). */
int mxd_dagg_forward(const void* mc_ms_feat, const int32_t* spatial_shape, const int32_t* scale_start_index,
                     const void* sampling_location, const void* weights, void* output, int dtype, int64_t bs,
                     int64_t num_feat, int64_t num_embeds, int64_t num_cams, int64_t num_scale, int64_t num_anchors,
                     int64_t num_pts, int64_t num_groups, void* hip_stream);

/* Bytes of scratch mxd_dagg_backward needs (0 if the sizes are invalid): the hand-over between the two
 * backward kernels, the fp32 image of grad_mc_ms_feat for 16-bit dtypes, and one float32 partial image of
 * grad_sampling_location per group. */
size_t mxd_dagg_backward_workspace_bytes(int dtype, int64_t bs, int64_t num_feat, int64_t num_embeds, int64_t num_cams,
                                         int64_t num_scale, int64_t num_anchors, int64_t num_pts, int64_t num_groups);

/* Every element of the three gradients is written (the reference zero-fills them first,
 * mx_driving/ops/npu_deformable_aggregation.py:66-68). */
int mxd_dagg_backward(const void* mc_ms_feat, const int32_t* spatial_shape, const int32_t* scale_start_index,
                      const void* sampling_location, const void* weights, const void* grad_output,
                      void* grad_mc_ms_feat, void* grad_sampling_location, void* grad_weights, void* workspace,
                      size_t workspace_bytes, int dtype, int64_t bs, int64_t num_feat, int64_t num_embeds,
                      int64_t num_cams, int64_t num_scale, int64_t num_anchors, int64_t num_pts, int64_t num_groups,
                      void* hip_stream);

/* ---- geometric kernel attention --------------------------------------------------------------
 * Replaces geometric_kernel_attention_forward / _backward (mx_driving/csrc/GeometricKernelAttentionFunc.cpp:33-118)
 * with the operator's own layouts: value [bs, nk, nh, hd] (the reference's binding permutes it itself),
 * sampling_locations [bs, nq, nh, nl, np, 2] = (x, y) pixel indices as FLOAT32 whatever `dtype` is (the reference takes
 * float16/float32/int32/int64 locations, GeometricKernelAttentionFunc.cpp:40-44; a 16-bit float cannot hold the indices
 * of a level wider than 2048 pixels, so a binding converts to float32, which is exact below 2^24), clamped to the level,
 * attn_weights [bs, nq, nh, nl, np], output [bs, nq, nh*hd]:
 *   output[b,q,h,:] = sum over (l, p) of attn * value[b, start_l + y*W_l + x, h, :].
 * Gradients: grad_value and grad_attn_weights (locations are indices and have none). */
int mxd_gka_forward(const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                    const void* sampling_locations, const void* attn_weights, void* output, int dtype, int64_t bs,
                    int64_t nk, int64_t nh, int64_t hd, int64_t nl, int64_t nq, int64_t np, void* hip_stream);
size_t mxd_gka_backward_workspace_bytes(int dtype, int64_t bs, int64_t nk, int64_t nh, int64_t hd, int64_t nl,
                                        int64_t nq, int64_t np);
int mxd_gka_backward(const void* value, const int32_t* spatial_shapes, const int32_t* level_start_index,
                     const void* sampling_locations, const void* attn_weights, const void* grad_output,
                     void* grad_value, void* grad_attn_weights, void* workspace, size_t workspace_bytes, int dtype,
                     int64_t bs, int64_t nk, int64_t nh, int64_t hd, int64_t nl, int64_t nq, int64_t np,
                     void* hip_stream);

/* ---- 2-D grid sampler, bilinear ----------------------------------------------------------------
 * Replaces the aclnnGridSampler2dV2 / aclnnGridSampler2dV2Grad launches of grid_sampler2d_v2 and
 * grid_sampler2d_v2_backward (mx_driving/csrc/GridSampler2dV2.cpp:33-99), which, like these entry points, work
 * on channel-last tensors (the binding permutes NCHW <-> NHWC around them, :68-76):
 *   input_nhwc [n, h_in, w_in, c]   grid [n, h_out, w_out, 2] = (x, y) in [-1, 1]   output_nhwc [n, h_out, w_out, c]
 * with the arithmetic of torch.nn.functional.grid_sample (the reference's golden): interpolation_mode 0 (bilinear),
 * padding_mode 0 (zeros) or 1 (border), align_corners 0/1.  c <= 256. */
int mxd_grid_sampler2d_forward(const void* input_nhwc, const void* grid, void* output_nhwc, int dtype, int64_t n,
                               int64_t c, int64_t h_in, int64_t w_in, int64_t h_out, int64_t w_out,
                               int interpolation_mode, int padding_mode, int align_corners, void* hip_stream);
size_t mxd_grid_sampler2d_backward_workspace_bytes(int dtype, int64_t n, int64_t c, int64_t h_in, int64_t w_in,
                                                   int64_t h_out, int64_t w_out);
/* grad_input_nhwc [n, h_in, w_in, c] and grad_grid [n, h_out, w_out, 2]; every element is written. */
int mxd_grid_sampler2d_backward(const void* grad_output_nhwc, const void* input_nhwc, const void* grid,
                                void* grad_input_nhwc, void* grad_grid, void* workspace, size_t workspace_bytes,
                                int dtype, int64_t n, int64_t c, int64_t h_in, int64_t w_in, int64_t h_out,
                                int64_t w_out, int interpolation_mode, int padding_mode, int align_corners,
                                void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* MXD_MSDA_H */
