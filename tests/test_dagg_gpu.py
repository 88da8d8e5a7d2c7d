"""Deformable aggregation on the GPU against the CPU oracle (the C restatement of the reference's test goldens).
Shapes follow the reference's tests (tests/torch/test_deformable_aggregation.py:130-141: one 32x88 map,
B in {1,5,10}, C in {32,64}, groups in {8,16}, anchors 10/13/18, points 10/50/31; the gradient test adds other map
sizes) plus a Sparse4D-like multi-camera multi-scale case.  Tolerances as for multi-scale deformable attention."""
import numpy as np
import pytest
import torch

import mx_driving
import mx_driving.fused
from drivingsdk_amd import _lib
from oracle import dagg_oracle as dagg
from util import BWD_FP32, FWD_FP32, HALF, rel_err

pytestmark = pytest.mark.gpu


def make_inputs(bs, C, G, A, P, maps, seed=0, pad=False):
    """maps: [cams][scales] of (H, W).  Locations uniform in (0,1), or in (-0.1, 1.1) with pad."""
    rng = np.random.default_rng(seed)
    ss = np.array(maps, dtype=np.int32)
    cams, scales = ss.shape[:2]
    sizes = ss.reshape(-1, 2).prod(1)
    ssi = np.concatenate([[0], np.cumsum(sizes)[:-1]]).reshape(cams, scales).astype(np.int32)
    nf = int(sizes.sum())
    feat = rng.random((bs, nf, C), dtype=np.float32)
    loc = rng.random((bs, A, P, cams, 2), dtype=np.float32)
    if pad:
        loc = loc * 1.2 - 0.1
    w = rng.random((bs, A, P, cams, scales, G), dtype=np.float32)
    go = rng.standard_normal((bs, A, C)).astype(np.float32)
    return feat, ss, ssi, loc, w, go


def _edge_mask(ss, loc):
    """Locations within 2^-20 px of (not on) a cell edge at some scale: the location gradient jumps there."""
    x, y = loc[..., 0].astype(np.float64), loc[..., 1].astype(np.float64)     # [bs, A, P, cams]
    near = np.zeros(x.shape, dtype=bool)
    for cam in range(ss.shape[0]):
        for sc in range(ss.shape[1]):
            h, w = ss[cam, sc]
            for v in (x[..., cam] * w - 0.5, y[..., cam] * h - 0.5):
                d = np.abs(v - np.round(v))
                near[..., cam] |= (d > 0) & (d < 2.0 ** -20)
    return near


def run_gpu(feat, ss, ssi, loc, w, go, device, fn=None, dtype=torch.float32):
    fn = fn or mx_driving.deformable_aggregation
    f = torch.from_numpy(feat).to(device, dtype).requires_grad_()
    lo = torch.from_numpy(loc).to(device, dtype).requires_grad_()
    wt = torch.from_numpy(w).to(device, dtype).requires_grad_()
    out = fn(f, torch.from_numpy(ss).to(device), torch.from_numpy(ssi).to(device), lo, wt)
    out.backward(torch.from_numpy(go).to(device, dtype))
    return [t.detach().double().cpu().numpy() for t in (out, f.grad, lo.grad, wt.grad)]


def check(inp, device, fwd_tol=FWD_FP32, bwd_tol=BWD_FP32):
    feat, ss, ssi, loc, w, go = inp
    want_out = dagg.direct_forward(feat, ss, ssi, loc, w)
    want = (want_out,) + dagg.direct_backward(feat, ss, ssi, loc, w, go)
    got = run_gpu(*inp, device)
    keep = ~_edge_mask(ss, loc)[..., None]
    errs = {}
    for name, g, r, tol in zip(("output", "grad_mc_ms_feat", "grad_sampling_location", "grad_weights"), got, want,
                               (fwd_tol, bwd_tol, bwd_tol, bwd_tol)):
        if name == "grad_sampling_location":
            g, r = g * keep, r * keep
        errs[name] = rel_err(g, r)
        assert errs[name] <= tol, (name, errs)
    return errs


@pytest.mark.parametrize("bs,C,G,A,P", [(1, 32, 8, 10, 10), (5, 64, 16, 13, 50), (10, 32, 16, 18, 31),
                                        (1, 64, 8, 18, 50)])
def test_reference_test_shapes(gpu_device, bs, C, G, A, P):
    print(check(make_inputs(bs, C, G, A, P, [[(32, 88)]], seed=bs + C + A), gpu_device))


@pytest.mark.parametrize("hw", [(16, 22), (64, 176), (7, 5)])
def test_reference_gradient_test_map_sizes(gpu_device, hw):
    print(check(make_inputs(2, 32, 8, 13, 31, [[hw]], seed=hw[0]), gpu_device))


def test_multi_camera_multi_scale_with_padding(gpu_device):
    """6 cameras x 4 scales (a Sparse4D-like pyramid, shrunk), 13 points, 256 channels in 8 groups, locations
    partly outside (0, 1): those contribute nothing and get zero gradients."""
    maps = [[(16, 44), (8, 22), (4, 11), (2, 6)]] * 6
    inp = make_inputs(2, 256, 8, 90, 13, maps, seed=3, pad=True)
    print(check(inp, gpu_device))
    feat, ss, ssi, loc, w, go = inp
    got = run_gpu(*inp, gpu_device)
    outside = ~((loc[..., 0] > 0) & (loc[..., 0] < 1) & (loc[..., 1] > 0) & (loc[..., 1] < 1))
    assert outside.any() and np.all(got[2][outside] == 0) and np.all(got[3][outside] == 0)


def test_three_scales_use_the_atomic_location_gradient_path(gpu_device):
    """A scale count that is not a power of two: the location gradient is added with atomics."""
    maps = [[(12, 20), (6, 10), (3, 5)]] * 2
    print(check(make_inputs(2, 48, 4, 17, 5, maps, seed=4, pad=True), gpu_device))


def test_groups_need_not_be_a_multiple_of_8_and_odd_channel_counts(gpu_device):
    print(check(make_inputs(1, 30, 3, 9, 7, [[(9, 13), (5, 7)]], seed=5), gpu_device))


def test_legacy_alias_and_float16(gpu_device):
    inp = make_inputs(1, 64, 8, 13, 10, [[(32, 88)]], seed=6)
    feat, ss, ssi, loc, w, go = inp
    f16 = lambda a: a.astype(np.float16).astype(np.float32)
    want = dagg.direct_forward(f16(feat), ss, ssi, f16(loc), f16(w))
    got = run_gpu(*inp, gpu_device, fn=mx_driving.fused.npu_deformable_aggregation, dtype=torch.float16)
    assert rel_err(got[0], want) <= HALF


def test_error_paths(gpu_device):
    feat, ss, ssi, loc, w, go = make_inputs(1, 32, 8, 4, 3, [[(8, 8)]])
    t = lambda a: torch.from_numpy(a).to(gpu_device)
    with pytest.raises(RuntimeError, match=r"mc_ms_feat.dim\(\) must be 3"):
        mx_driving.deformable_aggregation(t(feat)[0], t(ss), t(ssi), t(loc), t(w))
    with pytest.raises(RuntimeError, match=r"weights.dim\(\) must be 6"):
        mx_driving.deformable_aggregation(t(feat), t(ss), t(ssi), t(loc), t(w)[..., 0])
    with pytest.raises(Exception, match="empty Tensor"):
        mx_driving.deformable_aggregation(t(feat)[:, :0], t(ss), t(ssi), t(loc), t(w))
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        mx_driving.deformable_aggregation(torch.from_numpy(feat), torch.from_numpy(ss), torch.from_numpy(ssi),
                                          torch.from_numpy(loc), torch.from_numpy(w))
    lib = _lib.load()
    assert lib.mxd_dagg_forward(None, None, None, None, None, None, 0, 1, 64, 32, 1, 1, 4, 3, 8, None) == -3
    assert lib.mxd_dagg_forward(None, None, None, None, None, None, 0, 1, 64, 30, 1, 1, 4, 3, 8, None) == -2
    assert lib.mxd_dagg_backward_workspace_bytes(0, 1, 64, 32, 1, 1, 4, 3, 8) > 0


@pytest.mark.parametrize("seed", range(10))
def test_random_small_problems(gpu_device, seed):
    rng = np.random.default_rng(500 + seed)
    cams, scales = int(rng.integers(1, 4)), int(rng.integers(1, 5))
    G = int(rng.choice([1, 2, 3, 4, 8]))
    C = G * int(rng.choice([1, 2, 4, 5, 8, 16, 32, 40]))
    maps = [[(int(rng.integers(1, 40)), int(rng.integers(1, 40))) for _ in range(scales)] for _ in range(cams)]
    bs, A, P = int(rng.integers(1, 4)), int(rng.integers(1, 200)), int(rng.integers(1, 14))
    print("case", bs, C, G, A, P, maps, flush=True)
    check(make_inputs(bs, C, G, A, P, maps, seed=seed, pad=True), gpu_device)
