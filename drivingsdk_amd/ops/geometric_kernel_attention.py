"""Geometric kernel attention: autograd Function and public alias.

Same class name, argument order, saved tensors and return structure as the reference's Python layer
(mx_driving/ops/geometric_kernel_attention.py:29-57): ``forward(ctx, value, spatial_shapes, level_start_index,
sampling_locations, attention_weights)`` and ``backward -> (grad_value, None, None, None, grad_attn_weights)``.
Sampling locations are pixel indices (x, y), clamped to the level; there is no interpolation.  The compute sits in
``drivingsdk_amd._C`` (the kernels of multi-scale deformable attention with a one-pixel sample).
"""
from torch.autograd import Function

from .. import _C


class GeometricKernelAttentionFunc(Function):
    @staticmethod
    def forward(ctx, value, spatial_shapes, level_start_index, sampling_locations, attention_weights):
        ctx.save_for_backward(value, spatial_shapes, level_start_index, sampling_locations, attention_weights)
        ctx.value_size = value.size()
        batch_size, num_keys, num_heads, dim = value.size()
        num_queries = attention_weights.size(1)
        # (the reference allocates zeros for its kernel to add into; this kernel writes every element)
        output = value.new_empty(batch_size, num_queries, num_heads * dim)
        _C.geometric_kernel_attention_forward(
            value, spatial_shapes, level_start_index, sampling_locations, attention_weights, output)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        value, spatial_shapes, level_start_index, sampling_locations, attn_weights = ctx.saved_tensors
        grad_value, grad_attn_weights = _C.geometric_kernel_attention_backward(
            value, spatial_shapes, level_start_index, sampling_locations, attn_weights, grad_output)
        return grad_value, None, None, None, grad_attn_weights


geometric_kernel_attention = GeometricKernelAttentionFunc.apply
