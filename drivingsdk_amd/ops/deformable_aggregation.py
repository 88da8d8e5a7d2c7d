"""Deformable aggregation: autograd Function and public aliases.

Same class name, argument order, coercions, saved tensors and return structure as the reference's Python layer
(mx_driving/ops/npu_deformable_aggregation.py:10-88): ``forward(ctx, mc_ms_feat, spatial_shape,
scale_start_index, sampling_location, weights)`` and ``backward -> (grad_mc_ms_feat, None, None,
grad_sampling_location, grad_weights)``.  The compute sits in ``drivingsdk_amd._C`` (the HIP kernels of
multi-scale deformable attention, run with a channel group as head and a (camera, scale) pair as level).
"""
import torch
from torch.autograd import Function

from .. import _C


class AdsDeformableAggregation(Function):
    @staticmethod
    def forward(ctx, mc_ms_feat, spatial_shape, scale_start_index, sampling_location, weights):
        if torch.numel(mc_ms_feat) == 0 or torch.numel(weights) == 0:
            raise Exception("Erorr! Input Tensor can not be a empty Tensor.\n")
        mc_ms_feat = mc_ms_feat.contiguous()
        spatial_shape = spatial_shape.contiguous().int()
        scale_start_index = scale_start_index.contiguous().int()
        sampling_location = sampling_location.contiguous()
        weights = weights.contiguous()
        output = _C.deformable_aggregation(mc_ms_feat, spatial_shape, scale_start_index, sampling_location, weights)
        ctx.save_for_backward(mc_ms_feat, spatial_shape, scale_start_index, sampling_location, weights)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        mc_ms_feat, spatial_shape, scale_start_index, sampling_location, weights = ctx.saved_tensors
        if torch.numel(mc_ms_feat) == 0 or torch.numel(spatial_shape) == 0 or torch.numel(sampling_location) == 0:
            raise Exception("Erorr! Input Tensor can not be a empty Tensor.\n")
        grad_mc_ms_feat, grad_sampling_location, grad_weights = _C.deformable_aggregation_backward(
            mc_ms_feat, spatial_shape, scale_start_index, sampling_location, weights, grad_output.contiguous())
        return grad_mc_ms_feat, None, None, grad_sampling_location, grad_weights


npu_deformable_aggregation = AdsDeformableAggregation.apply
deformable_aggregation = AdsDeformableAggregation.apply
