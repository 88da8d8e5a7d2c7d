"""Multi-scale deformable attention: autograd Function and public aliases.

Same names, argument order, autocast policy, input coercions, saved tensors and return
structure as the reference's Python layer (mx_driving/ops/multi_scale_deformable_attn.py:18-95):
``forward(ctx, value, value_spatial_shapes, value_level_start_index, sampling_locations,
attention_weights)`` and ``backward -> (grad_value, None, None, grad_sampling_loc,
grad_attn_weight)``.  The compute sits in ``drivingsdk_amd._C`` (HIP kernels for gfx950).
"""
import warnings

import torch
from torch.amp import custom_bwd, custom_fwd
from torch.autograd.function import Function, once_differentiable

from .. import _C


class MultiScaleDeformableAttnFunction(Function):
    @staticmethod
    @custom_fwd(device_type="cuda", cast_inputs=torch.float32)
    def forward(ctx, value, value_spatial_shapes, value_level_start_index, sampling_locations, attention_weights,
                **kwargs):
        if torch.numel(value) == 0 or torch.numel(value_spatial_shapes) == 0 or torch.numel(attention_weights) == 0:
            raise Exception("Erorr! Input Tensor can not be a empty Tensor.\n")
        # (the reference casts both to int32 here; int64 metadata goes to the library as it is, other types are cast)
        if value_spatial_shapes.dtype != torch.int64 or value_level_start_index.dtype != torch.int64:
            value_spatial_shapes = value_spatial_shapes.int()
            value_level_start_index = value_level_start_index.int()
        sampling_locations = sampling_locations.type_as(value)
        attention_weights = attention_weights.type_as(value)

        output = _C.multi_scale_deformable_attn(
            value, value_spatial_shapes, value_level_start_index, sampling_locations, attention_weights)
        ctx.save_for_backward(
            value, value_spatial_shapes, value_level_start_index, sampling_locations, attention_weights)
        return output

    @staticmethod
    @once_differentiable
    @custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        value, value_spatial_shapes, value_level_start_index, sampling_locations, attention_weights = ctx.saved_tensors
        grad_value, grad_sampling_loc, grad_attn_weight = _C.multi_scale_deformable_attn_backward(
            value, value_spatial_shapes, value_level_start_index, sampling_locations, attention_weights, grad_output)
        return grad_value, None, None, grad_sampling_loc, grad_attn_weight


multi_scale_deformable_attn = MultiScaleDeformableAttnFunction.apply


def npu_multi_scale_deformable_attn_function(value, shape, offset, locations, weight):
    warnings.warn(
        "`npu_multi_scale_deformable_attn_function` will be deprecated in future. "
        "Please use `multi_scale_deformable_attn` instead.",
        DeprecationWarning,
    )
    return MultiScaleDeformableAttnFunction.apply(value, shape, offset, locations, weight)
