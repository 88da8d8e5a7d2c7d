"""Deformable-attention core with the module's pre-processing fused into the forward kernel.

The modules that call the operator (Deformable-DETR's ``MSDeformAttn.forward``, mmcv's
``MultiScaleDeformableAttention.forward``; in the reference's recipes:
model_examples/Deformable-DETR/Deformable-DETR_npu.patch:626-652,
model_examples/BEVFormer/bev_former_config.patch:404-421) run, between their linear layers and the operator,

    attention_weights  = softmax(attention_logits, -1).view(bs, nq, nh, nl, np)
    sampling_locations = reference_points[:, :, None, :, None, :] + sampling_offsets / offset_normalizer   # 2-d
    sampling_locations = reference_points[..., :2] + sampling_offsets / np * reference_points[..., 2:] * 0.5   # boxes
    output = multi_scale_deformable_attn(value, shapes, level_start_index, sampling_locations, attention_weights)

``multi_scale_deformable_attn_fused`` takes the module's raw tensors instead.  Its forward is ONE kernel in which
locations and weights never reach memory.  Its backward runs the operator's own backward kernels with the chain
rule through the three lines applied inside the first of them -- gradients for value, reference points, offsets
and logits; locations, weights and their gradients never reach memory either.
"""
import torch
from torch.amp import custom_bwd, custom_fwd
from torch.autograd.function import Function, once_differentiable

from .. import _C


def sampling_inputs(spatial_shapes, reference_points, sampling_offsets, attention_logits):
    """The callers' pre-processing, as plain torch ops: (sampling_locations, attention_weights)."""
    bs, nq, nh, nl, npts, _ = sampling_offsets.shape
    attn = torch.softmax(attention_logits.reshape(bs, nq, nh, nl * npts), -1).view(bs, nq, nh, nl, npts)
    if reference_points.shape[-1] == 2:
        normalizer = torch.stack([spatial_shapes[..., 1], spatial_shapes[..., 0]], -1).to(sampling_offsets.dtype)
        loc = reference_points[:, :, None, :, None, :] + sampling_offsets / normalizer[None, None, None, :, None, :]
    elif reference_points.shape[-1] == 4:
        loc = reference_points[:, :, None, :, None, :2] + \
            sampling_offsets / npts * reference_points[:, :, None, :, None, 2:] * 0.5
    else:
        raise ValueError(
            f"Last dim of reference_points must be 2 or 4, but get {reference_points.shape[-1]} instead.")
    return loc, attn


class MultiScaleDeformableAttnFusedFunction(Function):
    @staticmethod
    @custom_fwd(device_type="cuda", cast_inputs=torch.float32)
    def forward(ctx, value, value_spatial_shapes, value_level_start_index, reference_points, sampling_offsets,
                attention_logits):
        if torch.numel(value) == 0 or torch.numel(value_spatial_shapes) == 0 or torch.numel(attention_logits) == 0:
            raise Exception("Erorr! Input Tensor can not be a empty Tensor.\n")
        # (the reference casts both to int32 here; int64 metadata goes to the library as it is, other types are cast)
        if value_spatial_shapes.dtype != torch.int64 or value_level_start_index.dtype != torch.int64:
            value_spatial_shapes = value_spatial_shapes.int()
            value_level_start_index = value_level_start_index.int()
        reference_points = reference_points.type_as(value)
        sampling_offsets = sampling_offsets.type_as(value)
        attention_logits = attention_logits.type_as(value)
        output = _C.msda_fused_forward(value, value_spatial_shapes, value_level_start_index, reference_points,
                                       sampling_offsets, attention_logits)
        ctx.save_for_backward(value, value_spatial_shapes, value_level_start_index, reference_points,
                              sampling_offsets, attention_logits, output)
        return output

    @staticmethod
    @once_differentiable
    @custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        value, shapes, lsi, ref, off, logits, output = ctx.saved_tensors
        need = ctx.needs_input_grad
        grad_value, g_ref, g_off, g_log = _C.msda_fused_backward(
            value, shapes, lsi, ref, off, logits, output, grad_output, need_grad_reference_points=need[3])
        return (grad_value if need[0] else None), None, None, g_ref, (g_off if need[4] else None), \
            (g_log if need[5] else None)


multi_scale_deformable_attn_fused = MultiScaleDeformableAttnFusedFunction.apply
