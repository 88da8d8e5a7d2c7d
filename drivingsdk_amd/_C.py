"""Binding layer: the two functions the reference exports from its compiled module
``mx_driving._C`` (mx_driving/_C/__init__.pyi:67-81, mx_driving/csrc/pybind.cpp:110-111),
with the checks, output allocation and dtype policy of
mx_driving/csrc/MultiScaleDeformableAttn.cpp:28-118, over the C ABI of libmxd_msda.so.

Differences from the reference binding, all widening:
  * bfloat16 is accepted next to float16/float32;
  * float16/bfloat16 are read natively by the kernels (fp32 accumulation, one rounding at
    the store) instead of being up-cast to fp32 copies first;
  * ``num_levels * num_points <= 64`` is not required.
Work is enqueued on torch's current stream of the tensors' device; nothing synchronises.
"""
import torch

from . import _lib

_FLOAT_CODES = {torch.float32: _lib.DTYPE_F32, torch.float16: _lib.DTYPE_F16, torch.bfloat16: _lib.DTYPE_BF16}


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _meta_flag(shapes):
    """The reference's Python layer casts the level metadata to int32 on every call; int64 tensors are handed to the
    library as they are instead (it reads the low words), which saves the two cast kernels."""
    return _lib.META_I64 if shapes.dtype == torch.int64 else 0


def _check_common(value, value_spatial_shapes, value_level_start_index, sampling_locations, attention_weights):
    _check(value.dtype in _FLOAT_CODES,
           f"value: float16, bfloat16 or float32 tensor expected but got a tensor with dtype: {value.dtype}")
    _check(value_spatial_shapes.dtype in (torch.int32, torch.int64),
           f"value_spatial_shapes: int32 or int64 tensor expected but got a tensor with dtype: {value_spatial_shapes.dtype}")
    _check(value_level_start_index.dtype == value_spatial_shapes.dtype,
           f"value_level_start_index: {value_spatial_shapes.dtype} tensor (as value_spatial_shapes) expected but got a "
           f"tensor with dtype: {value_level_start_index.dtype}")
    _check(sampling_locations.dtype in _FLOAT_CODES,
           "sampling_locations: float16, bfloat16 or float32 tensor expected but got a tensor with dtype: "
           f"{sampling_locations.dtype}")
    _check(attention_weights.dtype in _FLOAT_CODES,
           "attention_weights: float16, bfloat16 or float32 tensor expected but got a tensor with dtype: "
           f"{attention_weights.dtype}")
    _check(value.dim() == 4, "value: expected [bs, num_keys, num_heads, embed_dims]")
    _check(sampling_locations.dim() == 6 and sampling_locations.size(5) == 2,
           "sampling_locations: expected [bs, num_queries, num_heads, num_levels, num_points, 2]")
    _check(attention_weights.dim() == 5, "attention_weights: expected [bs, num_queries, num_heads, num_levels, num_points]")
    _check(value_spatial_shapes.dim() == 2 and value_spatial_shapes.size(1) == 2,
           "value_spatial_shapes: expected [num_levels, 2]")
    _check(value.size(3) <= 256, "The number of embedding dimensions should be less than or equal to 256")
    bs, nk, nh, hd = value.shape
    nl = value_spatial_shapes.size(0)
    _, nq, _, nl_attn, npts, _ = sampling_locations.shape
    _check(sampling_locations.size(0) == bs and sampling_locations.size(2) == nh,
           "sampling_locations: batch size / num_heads do not match value")
    _check(tuple(attention_weights.shape) == (bs, nq, nh, nl_attn, npts),
           "attention_weights: shape does not match sampling_locations")
    _check(value_level_start_index.numel() == nl, "value_level_start_index: expected [num_levels]")
    _check(nl_attn >= nl, "sampling_locations carries fewer levels than value_spatial_shapes")
    tensors = (value, value_spatial_shapes, value_level_start_index, sampling_locations, attention_weights)
    _check(all(t.is_cuda for t in tensors),
           "multi_scale_deformable_attn: all tensors must live on a GPU (this build has no CPU implementation)")
    _check(all(t.device == value.device for t in tensors), "multi_scale_deformable_attn: tensors are on different devices")
    return bs, nk, nh, hd, nl, nl_attn, nq, npts


def multi_scale_deformable_attn(value, value_spatial_shapes, value_level_start_index, sampling_locations,
                                attention_weights):
    """Forward.  Returns output ``[bs, num_queries, num_heads*embed_dims]`` in value's dtype."""
    dims = _check_common(value, value_spatial_shapes, value_level_start_index, sampling_locations, attention_weights)
    bs, nk, nh, hd, nl, nl_attn, nq, npts = dims
    lib = _lib.load()
    dt = value.dtype
    value = value.contiguous()
    shapes = value_spatial_shapes.contiguous()
    lsi = value_level_start_index.contiguous()
    loc = sampling_locations.to(dt).contiguous()
    attn = attention_weights.to(dt).contiguous()
    output = torch.empty((bs, nq, nh * hd), dtype=dt, device=value.device)
    with torch.cuda.device(value.device):
        stream = torch.cuda.current_stream().cuda_stream
        rc = lib.mxd_msda_forward(value.data_ptr(), shapes.data_ptr(), lsi.data_ptr(), loc.data_ptr(),
                                  attn.data_ptr(), output.data_ptr(), _FLOAT_CODES[dt] | _meta_flag(shapes), bs, nk, nh,
                                  hd, nl, nl_attn, nq, npts, stream)
    _check(rc == 0, _lib.last_error() if rc != 0 else "")
    return output


def multi_scale_deformable_attn_backward(value, shape, level_start_index, location_trans, attn_weight_trans,
                                         grad_output):
    """Backward.  Returns (grad_value, grad_sampling_loc, grad_attn_weight) in value's dtype."""
    _check(grad_output.dtype in _FLOAT_CODES,
           f"grad_output: float16, bfloat16 or float32 tensor expected but got a tensor with dtype: {grad_output.dtype}")
    dims = _check_common(value, shape, level_start_index, location_trans, attn_weight_trans)
    bs, nk, nh, hd, nl, nl_attn, nq, npts = dims
    _check(grad_output.is_cuda and grad_output.device == value.device, "grad_output: must be on value's device")
    _check(grad_output.numel() == bs * nq * nh * hd, "grad_output: expected [bs, num_queries, num_heads*embed_dims]")
    lib = _lib.load()
    dt = value.dtype
    value = value.contiguous()
    shapes = shape.contiguous()
    lsi = level_start_index.contiguous()
    loc = location_trans.to(dt).contiguous()
    attn = attn_weight_trans.to(dt).contiguous()
    gout = grad_output.to(dt).contiguous()
    grad_value = torch.empty_like(value)
    grad_loc = torch.empty_like(loc)
    grad_attn = torch.empty_like(attn)
    code = _FLOAT_CODES[dt] | _meta_flag(shapes)
    ws_bytes = lib.mxd_msda_backward_workspace_bytes(code, bs, nk, nh, hd, nl, nl_attn, nq, npts)
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=value.device)
    with torch.cuda.device(value.device):
        stream = torch.cuda.current_stream().cuda_stream
        rc = lib.mxd_msda_backward(value.data_ptr(), shapes.data_ptr(), lsi.data_ptr(), loc.data_ptr(), attn.data_ptr(),
                                   gout.data_ptr(), grad_value.data_ptr(), grad_loc.data_ptr(), grad_attn.data_ptr(),
                                   workspace.data_ptr(), ws_bytes, code, bs, nk,
                                   nh, hd, nl, nl_attn, nq, npts, 0, stream)
    _check(rc == 0, _lib.last_error() if rc != 0 else "")
    return grad_value, grad_loc, grad_attn


def msda_fused_forward(value, value_spatial_shapes, value_level_start_index, reference_points, sampling_offsets,
                       attention_logits):
    """Forward of the operator with the callers' softmax and sampling-location arithmetic folded into the
    kernel (``mxd_msda_fused_forward``): reference_points ``[bs, nq, nl, 2|4]``, sampling_offsets
    ``[bs, nq, nh, nl, np, 2]``, attention_logits ``[bs, nq, nh, nl*np]``.  Returns ``[bs, nq, nh*hd]``."""
    _check(value.dtype in _FLOAT_CODES,
           f"value: float16, bfloat16 or float32 tensor expected but got a tensor with dtype: {value.dtype}")
    _check(value_spatial_shapes.dtype in (torch.int32, torch.int64) and
           value_level_start_index.dtype == value_spatial_shapes.dtype,
           "value_spatial_shapes / value_level_start_index: int32 (or both int64) tensors expected")
    _check(value.dim() == 4, "value: expected [bs, num_keys, num_heads, embed_dims]")
    _check(sampling_offsets.dim() == 6 and sampling_offsets.size(5) == 2,
           "sampling_offsets: expected [bs, num_queries, num_heads, num_levels, num_points, 2]")
    bs, nk, nh, hd = value.shape
    _, nq, _, nl, npts, _ = sampling_offsets.shape
    _check(value_spatial_shapes.dim() == 2 and tuple(value_spatial_shapes.shape) == (nl, 2),
           "value_spatial_shapes: expected [num_levels, 2] with the levels of sampling_offsets")
    _check(value_level_start_index.numel() == nl, "value_level_start_index: expected [num_levels]")
    _check(sampling_offsets.size(0) == bs and sampling_offsets.size(2) == nh,
           "sampling_offsets: batch size / num_heads do not match value")
    _check(reference_points.dim() == 4 and tuple(reference_points.shape[:3]) == (bs, nq, nl),
           "reference_points: expected [bs, num_queries, num_levels, 2 or 4]")
    _check(reference_points.size(3) in (2, 4),
           f"Last dim of reference_points must be 2 or 4, but get {reference_points.size(3)} instead.")
    _check(attention_logits.numel() == bs * nq * nh * nl * npts and attention_logits.size(0) == bs,
           "attention_logits: expected [bs, num_queries, num_heads, num_levels*num_points]")
    _check(value.size(3) <= 256, "The number of embedding dimensions should be less than or equal to 256")
    tensors = (value, value_spatial_shapes, value_level_start_index, reference_points, sampling_offsets,
               attention_logits)
    _check(all(t.is_cuda for t in tensors),
           "msda_fused_forward: all tensors must live on a GPU (this build has no CPU implementation)")
    _check(all(t.device == value.device for t in tensors), "msda_fused_forward: tensors are on different devices")
    lib = _lib.load()
    dt = value.dtype
    value = value.contiguous()
    shapes, lsi = value_spatial_shapes.contiguous(), value_level_start_index.contiguous()
    ref = reference_points.to(dt).contiguous()
    off = sampling_offsets.to(dt).contiguous()
    logits = attention_logits.to(dt).contiguous()
    output = torch.empty((bs, nq, nh * hd), dtype=dt, device=value.device)
    with torch.cuda.device(value.device):
        stream = torch.cuda.current_stream().cuda_stream
        rc = lib.mxd_msda_fused_forward(value.data_ptr(), shapes.data_ptr(), lsi.data_ptr(), ref.data_ptr(),
                                        reference_points.size(3), off.data_ptr(), logits.data_ptr(),
                                        output.data_ptr(), _FLOAT_CODES[dt] | _meta_flag(shapes), bs, nk, nh, hd, nl,
                                        nq, npts, stream)
    _check(rc == 0, _lib.last_error() if rc != 0 else "")
    return output


def msda_fused_backward(value, value_spatial_shapes, value_level_start_index, reference_points, sampling_offsets,
                        attention_logits, output, grad_output, need_grad_reference_points=True):
    """Backward of ``msda_fused_forward`` (``mxd_msda_fused_backward``): the chain rule through the softmax and the
    sampling-location arithmetic runs inside the operator's first backward kernel.  ``output`` is the forward
    result.  Returns ``(grad_value, grad_reference_points or None, grad_sampling_offsets, grad_attention_logits)``,
    each with the shape and dtype of its input."""
    _check(value.dtype in _FLOAT_CODES,
           f"value: float16, bfloat16 or float32 tensor expected but got a tensor with dtype: {value.dtype}")
    _check(value.dim() == 4 and sampling_offsets.dim() == 6 and sampling_offsets.size(5) == 2,
           "msda_fused_backward: expected value [bs, nk, nh, hd] and sampling_offsets [bs, nq, nh, nl, np, 2]")
    bs, nk, nh, hd = value.shape
    _, nq, _, nl, npts, _ = sampling_offsets.shape
    _check(tuple(value_spatial_shapes.shape) == (nl, 2) and value_level_start_index.numel() == nl,
           "value_spatial_shapes / value_level_start_index: expected the levels of sampling_offsets")
    _check(value_spatial_shapes.dtype in (torch.int32, torch.int64) and
           value_level_start_index.dtype == value_spatial_shapes.dtype,
           "value_spatial_shapes / value_level_start_index: int32 (or both int64) tensors expected")
    _check(sampling_offsets.size(0) == bs and sampling_offsets.size(2) == nh,
           "sampling_offsets: batch size / num_heads do not match value")
    _check(reference_points.dim() == 4 and tuple(reference_points.shape[:3]) == (bs, nq, nl),
           "reference_points: expected [bs, num_queries, num_levels, 2 or 4]")
    ref_dim = reference_points.size(3)
    _check(ref_dim in (2, 4), f"Last dim of reference_points must be 2 or 4, but get {ref_dim} instead.")
    _check(attention_logits.numel() == bs * nq * nh * nl * npts and attention_logits.size(0) == bs,
           "attention_logits: expected [bs, num_queries, num_heads, num_levels*num_points]")
    _check(output.numel() == bs * nq * nh * hd and grad_output.numel() == bs * nq * nh * hd,
           "output / grad_output: expected [bs, num_queries, num_heads*embed_dims]")
    tensors = (value, value_spatial_shapes, value_level_start_index, reference_points, sampling_offsets,
               attention_logits, output, grad_output)
    _check(all(t.is_cuda for t in tensors),
           "msda_fused_backward: all tensors must live on a GPU (this build has no CPU implementation)")
    _check(all(t.device == value.device for t in tensors), "msda_fused_backward: tensors are on different devices")
    lib = _lib.load()
    dt = value.dtype
    value = value.contiguous()
    shapes, lsi = value_spatial_shapes.contiguous(), value_level_start_index.contiguous()
    code = _FLOAT_CODES[dt] | _meta_flag(shapes)
    ref = reference_points.to(dt).contiguous()
    off = sampling_offsets.to(dt).contiguous()
    logits = attention_logits.to(dt).contiguous()
    out = output.to(dt).contiguous()
    gout = grad_output.to(dt).contiguous()
    grad_value = torch.empty_like(value)
    grad_off = torch.empty_like(off)
    grad_logits = torch.empty_like(logits)
    grad_ref = torch.empty_like(ref) if need_grad_reference_points else None
    want = 1 if need_grad_reference_points else 0
    ws_bytes = lib.mxd_msda_fused_backward_workspace_bytes(code, bs, nk, nh, hd, nl, nq, npts, ref_dim, want)
    workspace = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=value.device)
    with torch.cuda.device(value.device):
        stream = torch.cuda.current_stream().cuda_stream
        rc = lib.mxd_msda_fused_backward(value.data_ptr(), shapes.data_ptr(), lsi.data_ptr(), ref.data_ptr(), ref_dim,
                                         off.data_ptr(), logits.data_ptr(), out.data_ptr(), gout.data_ptr(),
                                         grad_value.data_ptr(), grad_ref.data_ptr() if want else None,
                                         grad_off.data_ptr(), grad_logits.data_ptr(), workspace.data_ptr(), ws_bytes,
                                         code, bs, nk, nh, hd, nl, nq, npts, 0, stream)
    _check(rc == 0, _lib.last_error() if rc != 0 else "")
    return grad_value, grad_ref, grad_off, grad_logits


# ---- deformable aggregation (mx_driving/csrc/DeformableAggregation.cpp:20-82 of the reference) --------------

def _dagg_check(mc_ms_feat, spatial_shape, scale_start_index, sampling_location, weights, name):
    _check(mc_ms_feat.dim() == 3, f"mc_ms_feat.dim() must be 3, but got: {mc_ms_feat.dim()}")
    _check(spatial_shape.dim() == 3, f"spatial_shape.dim() must be 3, but got: {spatial_shape.dim()}")
    _check(scale_start_index.dim() == 2, f"scale_start_index.dim() must be 2, but got: {scale_start_index.dim()}")
    _check(sampling_location.dim() == 5, f"sampling_location.dim() must be 5, but got: {sampling_location.dim()}")
    _check(weights.dim() == 6, f"weights.dim() must be 6, but got: {weights.dim()}")
    _check(mc_ms_feat.dtype in _FLOAT_CODES,
           f"mc_ms_feat: float16, bfloat16 or float32 tensor expected but got a tensor with dtype: {mc_ms_feat.dtype}")
    _check(spatial_shape.dtype == torch.int32 and scale_start_index.dtype == torch.int32,
           "spatial_shape / scale_start_index: int32 tensors expected")
    bs, num_feat, num_embeds = mc_ms_feat.shape
    _, num_anchors, num_pts, num_cams, num_scale, num_groups = weights.shape
    _check(weights.size(0) == bs, "weights: batch size does not match mc_ms_feat")
    _check(tuple(spatial_shape.shape) == (num_cams, num_scale, 2), "spatial_shape: expected [num_cams, num_scale, 2]")
    _check(tuple(scale_start_index.shape) == (num_cams, num_scale), "scale_start_index: expected [num_cams, num_scale]")
    _check(tuple(sampling_location.shape) == (bs, num_anchors, num_pts, num_cams, 2),
           "sampling_location: expected [bs, num_anchors, num_pts, num_cams, 2]")
    _check(num_groups > 0 and num_embeds % num_groups == 0, "num_embeds must be a multiple of weights.sizes()[5]")
    tensors = (mc_ms_feat, spatial_shape, scale_start_index, sampling_location, weights)
    _check(all(t.is_cuda for t in tensors),
           f"{name}: all tensors must live on a GPU (this build has no CPU implementation)")
    _check(all(t.device == mc_ms_feat.device for t in tensors), f"{name}: tensors are on different devices")
    return bs, num_feat, num_embeds, num_cams, num_scale, num_anchors, num_pts, num_groups


def deformable_aggregation(mc_ms_feat, spatial_shape, scale_start_index, sampling_location, weights):
    """Forward.  Returns ``[bs, num_anchors, num_embeds]`` in mc_ms_feat's dtype."""
    dims = _dagg_check(mc_ms_feat, spatial_shape, scale_start_index, sampling_location, weights,
                       "deformable_aggregation")
    lib = _lib.load()
    dt = mc_ms_feat.dtype
    feat = mc_ms_feat.contiguous()
    ss, si = spatial_shape.contiguous(), scale_start_index.contiguous()
    loc, w = sampling_location.to(dt).contiguous(), weights.to(dt).contiguous()
    out = torch.empty((dims[0], dims[5], dims[2]), dtype=dt, device=feat.device)
    with torch.cuda.device(feat.device):
        rc = lib.mxd_dagg_forward(feat.data_ptr(), ss.data_ptr(), si.data_ptr(), loc.data_ptr(), w.data_ptr(),
                                  out.data_ptr(), _FLOAT_CODES[dt], *dims, torch.cuda.current_stream().cuda_stream)
    _check(rc == 0, _lib.last_error() if rc != 0 else "")
    return out


def deformable_aggregation_backward(mc_ms_feat, spatial_shape, scale_start_index, sampling_location, weights,
                                    grad_output, grad_mc_ms_feat=None, grad_sampling_location=None, grad_weights=None):
    """Backward.  Returns (grad_mc_ms_feat, grad_sampling_location, grad_weights).  The three optional
    tensors are the pre-allocated outputs the reference's binding takes; they are overwritten when given
    (contiguous, of the inputs' shapes and dtype) and allocated otherwise."""
    dims = _dagg_check(mc_ms_feat, spatial_shape, scale_start_index, sampling_location, weights,
                       "deformable_aggregation_backward")
    _check(grad_output.is_cuda and grad_output.device == mc_ms_feat.device, "grad_output must be on the inputs' GPU")
    _check(tuple(grad_output.shape) == (dims[0], dims[5], dims[2]), "grad_output: expected [bs, num_anchors, num_embeds]")
    lib = _lib.load()
    dt = mc_ms_feat.dtype
    feat = mc_ms_feat.contiguous()
    ss, si = spatial_shape.contiguous(), scale_start_index.contiguous()
    loc, w = sampling_location.to(dt).contiguous(), weights.to(dt).contiguous()
    go = grad_output.to(dt).contiguous()

    def out_like(given, like):
        ok = given is not None and given.is_contiguous() and given.dtype == dt and given.shape == like.shape \
            and given.device == like.device
        return given if ok else torch.empty_like(like)
    gf, gl, gw = out_like(grad_mc_ms_feat, feat), out_like(grad_sampling_location, loc), out_like(grad_weights, w)
    code = _FLOAT_CODES[dt]
    nbytes = lib.mxd_dagg_backward_workspace_bytes(code, *dims)
    workspace = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=feat.device)
    with torch.cuda.device(feat.device):
        rc = lib.mxd_dagg_backward(feat.data_ptr(), ss.data_ptr(), si.data_ptr(), loc.data_ptr(), w.data_ptr(),
                                   go.data_ptr(), gf.data_ptr(), gl.data_ptr(), gw.data_ptr(), workspace.data_ptr(),
                                   nbytes, code, *dims, torch.cuda.current_stream().cuda_stream)
    _check(rc == 0, _lib.last_error() if rc != 0 else "")
    return gf, gl, gw


# ---- geometric kernel attention (mx_driving/csrc/GeometricKernelAttentionFunc.cpp:33-118 of the reference) ------

_GKA_LOC_TYPES = (torch.float16, torch.float32, torch.int32, torch.int64)


def _gka_check(value, spatial_shapes, level_start_index, sampling_locations, attention_weights):
    _check(value.dtype in _FLOAT_CODES,
           f"value_map: float16, bfloat16 or float32 tensor expected but got a tensor with dtype: {value.dtype}")
    _check(spatial_shapes.dtype in (torch.int32, torch.int64),
           f"spatial_spatial_shapes: int32 or int64 tensor expected but got a tensor with dtype: {spatial_shapes.dtype}")
    _check(level_start_index.dtype in (torch.int32, torch.int64),
           f"level_start_index: int32 or int64 tensor expected but got a tensor with dtype: {level_start_index.dtype}")
    _check(sampling_locations.dtype in _GKA_LOC_TYPES or sampling_locations.dtype == torch.bfloat16,
           "sampling_locations: float16, float32, int32 or int64 tensor expected but got a tensor with dtype: "
           f"{sampling_locations.dtype}")
    _check(attention_weights.dtype in _FLOAT_CODES,
           f"attention_weights: float16 or float32 tensor expected but got a tensor with dtype: {attention_weights.dtype}")
    _check(value.dim() == 4 and sampling_locations.dim() == 6 and sampling_locations.size(5) == 2 and
           attention_weights.dim() == 5, "geometric_kernel_attention: expected value [bs, num_keys, num_heads, dim], "
           "sampling_locations [bs, num_queries, num_heads, num_levels, num_points, 2], attention_weights [.., num_points]")
    bs, nk, nh, hd = value.shape
    _, nq, _, nl, npts, _ = sampling_locations.shape
    _check(tuple(attention_weights.shape) == (bs, nq, nh, nl, npts) and sampling_locations.size(0) == bs and
           sampling_locations.size(2) == nh, "geometric_kernel_attention: shapes of the tensors do not match")
    _check(tuple(spatial_shapes.shape) == (nl, 2) and level_start_index.numel() == nl,
           "geometric_kernel_attention: spatial_shapes [num_levels, 2] / level_start_index [num_levels] expected")
    tensors = (value, spatial_shapes, level_start_index, sampling_locations, attention_weights)
    _check(all(t.is_cuda for t in tensors),
           "geometric_kernel_attention: all tensors must live on a GPU (this build has no CPU implementation)")
    _check(all(t.device == value.device for t in tensors), "geometric_kernel_attention: tensors are on different devices")
    return bs, nk, nh, hd, nl, nq, npts


def geometric_kernel_attention_forward(value_map, spatial_shapes, level_start_index, sampling_locations,
                                       attention_weights, output):
    """Fills ``output`` ``[bs, num_queries, num_heads*dim]`` (the reference's binding has the same out-parameter)."""
    dims = _gka_check(value_map, spatial_shapes, level_start_index, sampling_locations, attention_weights)
    lib = _lib.load()
    dt = value_map.dtype
    _check(output.is_cuda and output.is_contiguous() and output.dtype == dt and
           tuple(output.shape) == (dims[0], dims[5], dims[2] * dims[3]),
           "output: expected a contiguous [bs, num_queries, num_heads*dim] tensor of value's dtype")
    value = value_map.contiguous()
    shapes, lsi = spatial_shapes.int().contiguous(), level_start_index.int().contiguous()
    # (pixel indices travel as float32 whatever value's dtype is: exact below 2^24, where a 16-bit float is not)
    loc, attn = sampling_locations.to(torch.float32).contiguous(), attention_weights.to(dt).contiguous()
    with torch.cuda.device(value.device):
        rc = lib.mxd_gka_forward(value.data_ptr(), shapes.data_ptr(), lsi.data_ptr(), loc.data_ptr(), attn.data_ptr(),
                                 output.data_ptr(), _FLOAT_CODES[dt], *dims, torch.cuda.current_stream().cuda_stream)
    _check(rc == 0, _lib.last_error() if rc != 0 else "")


def geometric_kernel_attention_backward(value, spatial_shapes, level_start_index, sampling_locations, attn_weights,
                                        grad_output):
    """Returns (grad_value, grad_attn_weights)."""
    dims = _gka_check(value, spatial_shapes, level_start_index, sampling_locations, attn_weights)
    _check(grad_output.is_cuda and grad_output.dtype in _FLOAT_CODES, "grad_output: float tensor on the GPU expected")
    lib = _lib.load()
    dt = value.dtype
    value = value.contiguous()
    _check(grad_output.device == value.device and grad_output.numel() == dims[0] * dims[5] * dims[2] * dims[3],
           "grad_output: expected [bs, num_queries, num_heads*dim] on value's device")
    shapes, lsi = spatial_shapes.int().contiguous(), level_start_index.int().contiguous()
    loc, attn = sampling_locations.to(torch.float32).contiguous(), attn_weights.to(dt).contiguous()
    go = grad_output.to(dt).contiguous()
    gv, ga = torch.empty_like(value), torch.empty_like(attn)
    code = _FLOAT_CODES[dt]
    nbytes = lib.mxd_gka_backward_workspace_bytes(code, *dims)
    workspace = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=value.device)
    with torch.cuda.device(value.device):
        rc = lib.mxd_gka_backward(value.data_ptr(), shapes.data_ptr(), lsi.data_ptr(), loc.data_ptr(), attn.data_ptr(),
                                  go.data_ptr(), gv.data_ptr(), ga.data_ptr(), workspace.data_ptr(), nbytes, code, *dims,
                                  torch.cuda.current_stream().cuda_stream)
    _check(rc == 0, _lib.last_error() if rc != 0 else "")
    return gv, ga


# ---- 2-D grid sampler (mx_driving/csrc/GridSampler2dV2.cpp:33-99 of the reference) ------------------------------

def grid_sampler2d_v2(input, grid, interpolation_mode, padding_mode, align_corners):
    """input [N, C, H, W], grid [N, H_out, W_out, 2] -> output [N, C, H_out, W_out] (bilinear).  As in the reference's
    binding the kernel works on channel-last data: input is permuted to NHWC before and the output back after.
    An input in torch's channels_last memory format needs no copy and gets its output in that format too (torch's
    convention for memory formats); any other input gets a contiguous NCHW output as in the reference."""
    _check(input.layout == torch.strided and grid.layout == torch.strided,
           "grid_sampler2d_v2(): expected input and grid to have torch.strided layout")
    _check(input.dtype in _FLOAT_CODES and grid.dtype == input.dtype,
           f"grid_sampler2d_v2(): float tensors of one dtype expected, but got input tensor with dtype: {input.dtype} "
           f"and grid tensor with dtype: {grid.dtype}")
    _check(input.dim() == 4 and grid.dim() == 4,
           f"grid_sampler2d_v2(): input and grid must be 4D tensor, but got input with sizes {tuple(input.shape)} "
           f"and grid with sizes {tuple(grid.shape)}")
    _check(input.size(0) == grid.size(0),
           f"grid_sampler2d_v2(): input and grid must have same batch size, but got input with sizes "
           f"{tuple(input.shape)} and grid with sizes {tuple(grid.shape)}")
    _check(grid.size(-1) == 2,
           f"grid_sampler2d_v2(): grid must have size 2 in last dimension, but got grid with sizes {tuple(grid.shape)}")
    _check(input.is_cuda and grid.is_cuda and input.device == grid.device,
           "grid_sampler2d_v2(): input and grid must live on one GPU (this build has no CPU implementation)")
    n, c, h_in, w_in = input.shape
    _, h_out, w_out, _ = grid.shape
    lib = _lib.load()
    dt = input.dtype
    x = input.permute(0, 2, 3, 1).contiguous()
    g = grid.contiguous()
    out = torch.empty((n, h_out, w_out, c), dtype=dt, device=input.device)
    with torch.cuda.device(input.device):
        rc = lib.mxd_grid_sampler2d_forward(x.data_ptr(), g.data_ptr(), out.data_ptr(), _FLOAT_CODES[dt], n, c, h_in,
                                            w_in, h_out, w_out, int(interpolation_mode), int(padding_mode),
                                            int(bool(align_corners)), torch.cuda.current_stream().cuda_stream)
    _check(rc == 0, _lib.last_error() if rc != 0 else "")
    channels_last = input.is_contiguous(memory_format=torch.channels_last) and not input.is_contiguous()
    return out.permute(0, 3, 1, 2) if channels_last else out.permute(0, 3, 1, 2).contiguous()


def grid_sampler2d_v2_backward(grad_output, input_x, input_grid, interpolation_mode, padding_mode, align_corners):
    """grad_output and input_x channel-last ([N, H_out, W_out, C], [N, H, W, C]) as the reference's binding takes
    them (mx_driving/ops/grid_sampler2d_v2.py:64-70).  Returns (grad_x as an NCHW view, grad_grid)."""
    _check(grad_output.dim() == 4, f"grad_output must to be a 4D Tensor, but got: {grad_output.dim()}")
    _check(input_x.dim() == 4, f"input_x has to be a 4D Tensor, but got: {input_x.dim()}")
    _check(input_grid.dim() == 4, f"input_grid has to be a 4D Tensor, but got: {input_grid.dim()}")
    _check(all(t.is_cuda for t in (grad_output, input_x, input_grid)),
           "grid_sampler2d_v2_backward(): all tensors must live on a GPU (this build has no CPU implementation)")
    n, h_in, w_in, c = input_x.shape
    _, h_out, w_out, _ = input_grid.shape
    _check(input_grid.size(0) == n and input_grid.size(3) == 2, "input_grid: expected [N, H_out, W_out, 2]")
    _check(tuple(grad_output.shape) == (n, h_out, w_out, c), "grad_output: expected [N, H_out, W_out, C]")
    _check(grad_output.device == input_x.device and input_grid.device == input_x.device,
           "grid_sampler2d_v2_backward(): tensors are on different devices")
    lib = _lib.load()
    dt = input_x.dtype
    _check(dt in _FLOAT_CODES, f"input_x: float tensor expected but got {dt}")
    x, g, go = input_x.contiguous(), input_grid.to(dt).contiguous(), grad_output.to(dt).contiguous()
    grad_x, grad_grid = torch.empty_like(x), torch.empty_like(g)
    code = _FLOAT_CODES[dt]
    nbytes = lib.mxd_grid_sampler2d_backward_workspace_bytes(code, n, c, h_in, w_in, h_out, w_out)
    workspace = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        rc = lib.mxd_grid_sampler2d_backward(go.data_ptr(), x.data_ptr(), g.data_ptr(), grad_x.data_ptr(),
                                             grad_grid.data_ptr(), workspace.data_ptr(), nbytes, code, n, c, h_in,
                                             w_in, h_out, w_out, int(interpolation_mode), int(padding_mode),
                                             int(bool(align_corners)), torch.cuda.current_stream().cuda_stream)
    _check(rc == 0, _lib.last_error() if rc != 0 else "")
    return grad_x.permute(0, 3, 1, 2), grad_grid
