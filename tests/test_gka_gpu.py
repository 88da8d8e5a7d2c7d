"""Geometric kernel attention on the GPU against the CPU oracle.  Shapes after the reference's test
(tests/torch/test_geometric_kernel_attention.py:118-124, batch sizes shrunk; its location recipe :22-33)."""
import numpy as np
import pytest
import torch

import mx_driving
from drivingsdk_amd import _lib
from oracle import gka_oracle as gka
from util import BWD_FP32, FWD_FP32, HALF, rel_err, set_tuning

pytestmark = pytest.mark.gpu


def make_inputs(shape, hw, seed=0):
    bs, nq, hd, nh, nl, npts = shape
    g = torch.Generator().manual_seed(seed)
    sh = torch.tensor([list(hw)] * nl)
    lsi = torch.cat((sh.new_zeros((1,)), sh.prod(1).cumsum(0)[:-1]))
    nk = int(sh.prod(1).sum())
    loc = torch.rand(bs, nq, nh, nl, npts, 2, generator=g)
    loc[..., 0] = loc[..., 0] * (hw[1] + 6) - 3
    loc[..., 1] = loc[..., 1] * (hw[0] + 6) - 3
    loc = loc.long().float()                                   # as the reference test: truncated, passed as float
    value = torch.rand(bs, nk, nh, hd, generator=g) * 3
    attn = torch.rand(bs, nq, nh, nl, npts, generator=g)
    go = torch.rand(bs, nq, nh * hd, generator=g) * 10
    return value, sh, lsi, loc, attn, go


def run_gpu(value, sh, lsi, loc, attn, go, device, dtype=torch.float32, loc_dtype=None):
    v = value.to(device, dtype).requires_grad_()
    a = attn.to(device, dtype).requires_grad_()
    lo = loc.to(device, loc_dtype or dtype)
    out = mx_driving.geometric_kernel_attention(v, sh.to(device), lsi.to(device), lo, a)
    out.backward(go.to(device, dtype))
    return [t.detach().double().cpu().numpy() for t in (out, v.grad, a.grad)]


@pytest.mark.parametrize("shape,hw", [([3, 7156, 64, 4, 1, 15], (15, 25)), ([6, 1146, 64, 4, 1, 15], (6, 10)),
                                      ([2, 4, 16, 4, 2, 15], (6, 10)), ([2, 333, 32, 8, 3, 4], (20, 30))])
def test_reference_test_shapes(gpu_device, shape, hw):
    inp = make_inputs(shape, hw, seed=shape[1])
    want = (gka.forward(*inp[:5]),) + gka.backward(*inp)
    got = run_gpu(*inp, gpu_device)
    for name, g_, w_, tol in zip(("output", "grad_value", "grad_attn_weights"), got, want, (FWD_FP32, BWD_FP32, BWD_FP32)):
        assert rel_err(g_, w_) <= tol, (name, rel_err(g_, w_))


def test_integer_locations_and_float16(gpu_device):
    inp = make_inputs([2, 100, 32, 4, 2, 6], (9, 13), seed=5)
    want = gka.forward(*inp[:5])
    got = run_gpu(*inp, gpu_device, loc_dtype=torch.int64)
    assert rel_err(got[0], want) <= FWD_FP32
    value, sh, lsi, loc, attn, go = inp
    want16 = gka.forward(value.half().double(), sh, lsi, loc, attn.half().double())
    got16 = run_gpu(*inp, gpu_device, dtype=torch.float16)
    assert rel_err(got16[0], want16) <= HALF


def test_error_paths(gpu_device):
    value, sh, lsi, loc, attn, go = [t.to(gpu_device) if isinstance(t, torch.Tensor) else t
                                     for t in make_inputs([1, 5, 16, 2, 1, 3], (4, 4))]
    with pytest.raises(RuntimeError, match="sampling_locations: float16, float32, int32 or int64"):
        mx_driving.geometric_kernel_attention(value, sh, lsi, loc.double(), attn)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        mx_driving.geometric_kernel_attention(value.cpu(), sh.cpu(), lsi.cpu(), loc.cpu(), attn.cpu())
    lib = _lib.load()
    assert lib.mxd_gka_forward(None, None, None, None, None, None, 0, 1, 16, 2, 16, 1, 5, 3, None) == -3


@pytest.mark.parametrize("seed", range(8))
def test_random_small_problems(gpu_device, seed):
    rng = np.random.default_rng(700 + seed)
    shape = [int(rng.integers(1, 4)), int(rng.integers(1, 500)), int(rng.choice([1, 3, 8, 16, 32, 64, 100])),
             int(rng.integers(1, 9)), int(rng.integers(1, 4)), int(rng.integers(1, 17))]
    hw = (int(rng.integers(1, 30)), int(rng.integers(1, 30)))
    print("case", shape, hw, flush=True)
    inp = make_inputs(shape, hw, seed=seed)
    want = (gka.forward(*inp[:5]),) + gka.backward(*inp)
    got = run_gpu(*inp, gpu_device)
    for g_, w_, tol in zip(got, want, (FWD_FP32, BWD_FP32, BWD_FP32)):
        assert rel_err(g_, w_) <= tol


@pytest.mark.parametrize("dtype,loc_dtype,hw", [(torch.bfloat16, torch.float32, (3, 700)), (torch.float16, torch.float32, (2, 3000)),
                                                (torch.float16, torch.int64, (2, 3000)), (torch.bfloat16, torch.int32, (700, 3)),
                                                (torch.float16, torch.float16, (5, 40))])
def test_levels_wider_than_a_16bit_float_can_index(gpu_device, dtype, loc_dtype, hw):
    """Pixel indices beyond 256 (bfloat16) / 2048 (float16) are not representable in value's 16-bit dtype; locations
    travel to the kernels as float32 whatever value's dtype is (the reference accepts float16 values with
    float32 / int32 / int64 locations, mx_driving/csrc/GeometricKernelAttentionFunc.cpp:40-44)."""
    bs, nq, hd, nh, nl, npts = 2, 300, 16, 2, 1, 5
    g = torch.Generator().manual_seed(hw[1])
    sh = torch.tensor([list(hw)])
    lsi = torch.zeros(1, dtype=torch.int64)
    loc = torch.stack((torch.randint(-2, hw[1] + 2, (bs, nq, nh, nl, npts), generator=g),
                       torch.randint(-2, hw[0] + 2, (bs, nq, nh, nl, npts), generator=g)), -1).float()
    loc[0, 0, 0, 0, 0] = torch.tensor([hw[1] - 1.0, hw[0] - 1.0])   # the last pixel itself
    value = torch.rand(bs, hw[0] * hw[1], nh, hd, generator=g) * 3
    attn = torch.rand(bs, nq, nh, nl, npts, generator=g)
    go = torch.rand(bs, nq, nh * hd, generator=g)
    v16, a16, g16 = value.to(dtype).double(), attn.to(dtype).double(), go.to(dtype).double()
    loc_in = loc.to(loc_dtype)
    want = (gka.forward(v16, sh, lsi, loc_in.double(), a16),) + gka.backward(v16, sh, lsi, loc_in.double(), a16, g16)
    got = run_gpu(value, sh, lsi, loc_in, attn, go, gpu_device, dtype=dtype, loc_dtype=loc_dtype)
    tol = HALF if dtype == torch.float16 else 2.0 ** -8
    for name, g_, w_ in zip(("output", "grad_value", "grad_attn_weights"), got, want):
        assert rel_err(g_, w_) <= tol, (name, rel_err(g_, w_))


def test_largest_reference_shape_at_full_batch(gpu_device):
    """The largest shape of the reference's test at its full batch size, [24, 7156, 64, 4, 1, 15]
    (tests/torch/test_geometric_kernel_attention.py:112-119) -- the shape bench.py times."""
    inp = make_inputs([24, 7156, 64, 4, 1, 15], (15, 25), seed=7156)
    want = (gka.forward(*inp[:5]),) + gka.backward(*inp)
    got = run_gpu(*inp, gpu_device)
    for name, g_, w_, tol in zip(("output", "grad_value", "grad_attn_weights"), got, want, (FWD_FP32, BWD_FP32, BWD_FP32)):
        assert rel_err(g_, w_) <= tol, (name, rel_err(g_, w_))


def test_levels_that_overlap_beyond_the_run_table_take_the_atomic_form(gpu_device, monkeypatch):
    """level_start_index is the caller's.  Three levels of 513 pixels that overlap inside 600 keys have six tiles of 512
    pixels between them where the run table of the tile-mode backward has room for four (num_keys / 512 + num_levels).
    The plain operator adds such levels sample by sample; this operator documents that its default form leaves them out
    of grad_value and that MXD_MSDA_BWD_ATOMIC=1 (the one-kernel form with global atomics) takes any layout: that form
    must give the oracle's gradients, and the forward and grad_attn_weights must not depend on the form."""
    bs, nq, hd, nh, nl, npts, hw = 2, 400, 16, 3, 3, 5, (27, 19)
    g = torch.Generator().manual_seed(513)
    sh = torch.tensor([list(hw)] * nl)
    lsi = torch.tensor([0, 40, 87])
    nk = 600
    loc = torch.stack((torch.randint(-2, hw[1] + 2, (bs, nq, nh, nl, npts), generator=g),
                       torch.randint(-2, hw[0] + 2, (bs, nq, nh, nl, npts), generator=g)), -1).float()
    value = torch.rand(bs, nk, nh, hd, generator=g) * 3
    attn = torch.rand(bs, nq, nh, nl, npts, generator=g)
    go = torch.rand(bs, nq, nh * hd, generator=g) * 10
    want = (gka.forward(value, sh, lsi, loc, attn),) + gka.backward(value, sh, lsi, loc, attn, go)
    default = run_gpu(value, sh, lsi, loc, attn, go, gpu_device)
    set_tuning(monkeypatch, MXD_MSDA_BWD_ATOMIC=1)
    got = run_gpu(value, sh, lsi, loc, attn, go, gpu_device)
    for name, g_, w_, tol in zip(("output", "grad_value", "grad_attn_weights"), got, want, (FWD_FP32, BWD_FP32, BWD_FP32)):
        assert rel_err(g_, w_) <= tol, (name, rel_err(g_, w_))
    assert rel_err(default[0], want[0]) <= FWD_FP32 and rel_err(default[2], want[2]) <= BWD_FP32
