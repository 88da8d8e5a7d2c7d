"""2-D grid sampler (bilinear): autograd Function and public alias.

Same class name, arguments, mode handling, warnings and return structure as the reference's Python layer
(mx_driving/ops/grid_sampler2d_v2.py:18-73): bilinear interpolation with zeros or border padding runs on the HIP
kernels; other interpolation modes -- and, here, more than 256 channels (128 in the reference) -- are handed to
``torch.nn.functional.grid_sample`` with a warning, exactly as the reference does for what its kernel does not cover.
"""
import warnings

import torch
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from .. import _C

MAX_CHANNELS = 256


class GridSampler2dV2Function(Function):
    @staticmethod
    def forward(ctx, input_tensor, grid_tensor, mode="bilinear", padding_mode="zeros", align_corners=False):
        if torch.numel(input_tensor) == 0 or torch.numel(grid_tensor) == 0:
            raise Exception("mx_driving.grid_sampler2d_v2(): Input tensor and grid tensor can not be empty tensor.\n")
        if input_tensor.size(1) > MAX_CHANNELS:
            warnings.warn(
                f"mx_driving.grid_sampler2d_v2(): Not support for channel of input greater than {MAX_CHANNELS}, "
                "will call torch.nn.functional.grid_sample().")
            return torch.nn.functional.grid_sample(input_tensor, grid_tensor, mode, padding_mode, align_corners)
        if mode != "bilinear":
            warnings.warn(
                f"mx_driving.grid_sampler2d_v2(): Not support '{mode}' mode, will call torch.nn.functional.grid_sample().")
            return torch.nn.functional.grid_sample(input_tensor, grid_tensor, mode, padding_mode, align_corners)
        if padding_mode != "zeros" and padding_mode != "border":
            raise ValueError(
                "nn.functional.grid_sample(): expected padding_mode to be 'zeros', 'border', "
                f"but got: '{padding_mode}'")
        ctx.interpolation = mode
        ctx.padding_mode = padding_mode
        ctx.align_corners = align_corners
        interpolation = {"bilinear": 0, "nearest": 1}.get(mode, 0)
        padding = {"zeros": 0, "border": 1, "reflection": 2}.get(padding_mode, 0)
        output = _C.grid_sampler2d_v2(input_tensor, grid_tensor, interpolation, padding, align_corners)
        ctx.save_for_backward(input_tensor, grid_tensor)
        return output

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        input_x, input_grid = ctx.saved_tensors
        nhwc_input_x = input_x.permute(0, 2, 3, 1).contiguous()
        nhwc_grad_output = grad_output.permute(0, 2, 3, 1).contiguous()
        interpolation = {"bilinear": 0, "nearest": 1}.get(ctx.interpolation, 0)
        padding = {"zeros": 0, "border": 1, "reflection": 2}.get(ctx.padding_mode, 0)
        grad_x, grad_grid = _C.grid_sampler2d_v2_backward(nhwc_grad_output, nhwc_input_x, input_grid, interpolation,
                                                          padding, ctx.align_corners)
        return grad_x, grad_grid, None, None, None


grid_sampler2d_v2 = GridSampler2dV2Function.apply
