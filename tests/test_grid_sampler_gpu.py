"""2-D grid sampler on the GPU against torch.nn.functional.grid_sample on the CPU in float64 -- the golden of the
reference's own test (tests/torch/test_grid_sampler2d_v2.py:22-26), whose shapes and modes are used here (batch sizes
shrunk), plus gradients, grids reaching outside [-1, 1], and the hand-over to torch for what the kernel does not cover."""
import warnings

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import mx_driving
from drivingsdk_amd import _lib
from util import BWD_FP32, FWD_FP32, HALF, rel_err

pytestmark = pytest.mark.gpu


def make_inputs(input_shape, grid_shape, seed=0, span=1.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.rand(input_shape, generator=g)
    grid = (2 * torch.rand(grid_shape, generator=g) - 1) * span
    go = torch.randn(input_shape[0], input_shape[1], grid_shape[1], grid_shape[2], generator=g)
    return x, grid, go


def _pixel_coords(grid, size, align):
    g = grid.double()
    return ((g + 1) / 2) * (size - 1) if align else ((g + 1) * size - 1) / 2


def check(x, grid, go, padding_mode, align, device, dtype=torch.float32, fwd_tol=FWD_FP32, bwd_tol=BWD_FP32):
    xr = x.to(dtype).double().requires_grad_()
    gr = grid.to(dtype).double().requires_grad_()
    want = F.grid_sample(xr, gr, "bilinear", padding_mode, align)
    want.backward(go.double())
    xd = x.to(device, dtype).requires_grad_()
    gd = grid.to(device, dtype).requires_grad_()
    out = mx_driving.grid_sampler2d_v2(xd, gd, "bilinear", padding_mode, align)
    assert out.shape == want.shape and out.dtype == dtype and out.is_contiguous()
    out.backward(go.to(device, dtype))
    errs = {"output": rel_err(out.detach().double().cpu().numpy(), want.detach().numpy()),
            "grad_input": rel_err(xd.grad.double().cpu().numpy(), xr.grad.numpy())}
    # the grid gradient jumps at cell edges (and, with border padding, where the coordinate starts to clip): leave
    # out samples whose float32 pixel coordinate is within 1e-4 px of an integer
    h, w = x.shape[2], x.shape[3]
    ix, iy = _pixel_coords(grid[..., 0], w, align), _pixel_coords(grid[..., 1], h, align)
    near = ((ix - ix.round()).abs() < 1e-4) | ((iy - iy.round()).abs() < 1e-4)
    assert near.float().mean() < 0.01
    keep = (~near)[..., None].numpy()
    errs["grad_grid"] = rel_err(gd.grad.double().cpu().numpy() * keep, gr.grad.numpy() * keep)
    assert errs["output"] <= fwd_tol and errs["grad_input"] <= bwd_tol and errs["grad_grid"] <= bwd_tol, errs
    return errs


@pytest.mark.parametrize("padding_mode,align", [("zeros", False), ("zeros", True), ("border", False), ("border", True)])
def test_reference_shape_all_modes(gpu_device, padding_mode, align):
    x, grid, go = make_inputs([4, 4, 64, 176], [4, 24, 176, 2], seed=1)
    print(check(x, grid, go, padding_mode, align, gpu_device))


@pytest.mark.parametrize("input_shape,grid_shape", [([2, 4, 3, 4], [2, 2, 3, 2]), ([3, 64, 64, 176], [3, 24, 176, 2]),
                                                    ([2, 128, 64, 176], [2, 24, 176, 2]), ([1, 7, 5, 9], [1, 11, 3, 2]),
                                                    ([2, 256, 8, 8], [2, 5, 5, 2])])
def test_reference_channel_counts_and_small_case(gpu_device, input_shape, grid_shape):
    x, grid, go = make_inputs(input_shape, grid_shape, seed=input_shape[1])
    print(check(x, grid, go, "zeros", False, gpu_device))


@pytest.mark.parametrize("padding_mode", ["zeros", "border"])
def test_grid_reaching_outside_the_image(gpu_device, padding_mode):
    x, grid, go = make_inputs([2, 16, 20, 30], [2, 40, 50, 2], seed=3, span=1.3)
    print(check(x, grid, go, padding_mode, False, gpu_device))
    print(check(x, grid, go, padding_mode, True, gpu_device))


def test_float16(gpu_device):
    x, grid, go = make_inputs([2, 32, 16, 24], [2, 9, 13, 2], seed=4)
    want = F.grid_sample(x.half().double(), grid.half().double(), "bilinear", "zeros", False)
    out = mx_driving.grid_sampler2d_v2(x.to(gpu_device).half(), grid.to(gpu_device).half(), "bilinear", "zeros", False)
    assert rel_err(out.double().cpu().numpy(), want.numpy()) <= HALF


def test_unsupported_modes_go_to_torch_and_errors(gpu_device):
    x, grid, _ = make_inputs([1, 4, 6, 6], [1, 3, 3, 2], seed=5)
    xd, gd = x.to(gpu_device), grid.to(gpu_device)
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        out = mx_driving.grid_sampler2d_v2(xd, gd, "nearest", "zeros", False)
        assert any("Not support 'nearest' mode" in str(i.message) for i in w)
    assert torch.equal(out, F.grid_sample(xd, gd, "nearest", "zeros", False))
    with pytest.raises(ValueError, match="expected padding_mode"):
        mx_driving.grid_sampler2d_v2(xd, gd, "bilinear", "reflection", False)
    with pytest.raises(Exception, match="can not be empty tensor"):
        mx_driving.grid_sampler2d_v2(xd[:0], gd[:0], "bilinear", "zeros", False)
    with pytest.raises(RuntimeError, match="same batch size"):
        mx_driving.grid_sampler2d_v2(xd, gd.repeat(2, 1, 1, 1), "bilinear", "zeros", False)
    lib = _lib.load()
    assert lib.mxd_grid_sampler2d_forward(None, None, None, 0, 1, 4, 6, 6, 3, 3, 0, 0, 0, None) == -3
    assert lib.mxd_grid_sampler2d_forward(None, None, None, 0, 1, 4, 6, 6, 3, 3, 1, 0, 0, None) == -2
    assert lib.mxd_grid_sampler2d_forward(None, None, None, 0, 1, 4, 6, 6, 3, 3, 0, 2, 0, None) == -2


def test_channels_last_input_keeps_its_memory_format(gpu_device):
    """A channels_last input is used in place (it is the layout the kernel works on) and the output comes back
    in the same memory format, with the same values as for a contiguous input."""
    x, grid, go = make_inputs([3, 32, 20, 30], [3, 11, 17, 2], seed=9, span=1.1)
    xd, gd = x.to(gpu_device), grid.to(gpu_device)
    plain = mx_driving.grid_sampler2d_v2(xd, gd, "bilinear", "zeros", False)
    xcl = xd.contiguous(memory_format=torch.channels_last).requires_grad_()
    out = mx_driving.grid_sampler2d_v2(xcl, gd, "bilinear", "zeros", False)
    assert plain.is_contiguous() and out.is_contiguous(memory_format=torch.channels_last) and not out.is_contiguous()
    assert torch.equal(out, plain)
    out.backward(go.to(gpu_device).contiguous(memory_format=torch.channels_last))
    xr = x.double().requires_grad_()
    F.grid_sample(xr, grid.double(), "bilinear", "zeros", False).backward(go.double())
    assert rel_err(xcl.grad.double().cpu().numpy(), xr.grad.numpy()) <= BWD_FP32


def test_largest_reference_shape_at_full_batch(gpu_device):
    """The largest shape of the reference's test at its full batch size, input [24, 128, 64, 176], grid [24, 24, 176, 2]
    (tests/torch/test_grid_sampler2d_v2.py:34-59) -- the shape bench.py times (float64 grid_sample on the CPU takes a few
    seconds at this size)."""
    x, grid, go = make_inputs([24, 128, 64, 176], [24, 24, 176, 2], seed=24)
    print(check(x, grid, go, "zeros", False, gpu_device))
