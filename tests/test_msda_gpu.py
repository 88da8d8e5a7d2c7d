"""Parity of the HIP path (through the public API and the C ABI) with the CPU oracle.
Everything here needs the GPU; the library is loaded from drivingsdk_amd/lib and the tests
fail if it is missing."""
import ctypes
import os

import numpy as np
import pytest
import torch

from drivingsdk_amd import _lib, workloads
from oracle import msda_oracle as orc
from util import (BF16, BWD_FP32, FWD_FP32, HALF, check_16bit, check_close, half_tol, level_slices, oracle_all, rel_err,
                  run_gpu, set_tuning, to_device)

pytestmark = pytest.mark.gpu


def _cell_edge_mask(inp):
    """Samples whose pixel coordinate lies within 2^-20 -- or, where that is more, two float32 units in the last place
    of the coordinate -- of an integer on either axis.  The location gradient of bilinear interpolation jumps there (it
    is the slope of the cell the sample falls in; at the border of the image the sample's validity flips), so a
    float32 and a float64 evaluation may legitimately pick different sides; such samples are left out of the
    grad_sampling_locations comparison only."""
    loc = inp.sampling_locations.double()
    nl = inp.spatial_shapes.shape[0]
    hw = inp.spatial_shapes.double()
    mask = torch.zeros(loc.shape[:-1], dtype=torch.bool)
    for lvl in range(nl):
        w_im = loc[:, :, :, lvl, :, 0] * hw[lvl, 1] - 0.5
        h_im = loc[:, :, :, lvl, :, 1] * hw[lvl, 0] - 0.5
        dw, dh = (w_im - w_im.round()).abs(), (h_im - h_im.round()).abs()
        # exactly on an edge is fine: both evaluations are exact there and take the same side
        # (float32 spacing at coordinate c: 2^(floor(log2 |c|) - 23))
        ulp_w = torch.exp2(torch.floor(torch.log2(w_im.abs().clamp_min(1.0))) - 23.0)
        ulp_h = torch.exp2(torch.floor(torch.log2(h_im.abs().clamp_min(1.0))) - 23.0)
        near = ((dw > 0) & (dw < torch.maximum(2.0 * ulp_w, torch.tensor(2.0 ** -20, dtype=torch.float64)))) | \
               ((dh > 0) & (dh < torch.maximum(2.0 * ulp_h, torch.tensor(2.0 ** -20, dtype=torch.float64))))
        mask[:, :, :, lvl] = near
    return mask.numpy()


def _check_all(inp, device, fwd_tol, bwd_tol, with_grads=True):
    """HIP path against the float64 oracle on the same inputs: the max-norm figure the path's tolerances are stated in,
    and element-wise -- float32: |got - ref| <= tol * (|ref| + RMS of the element's level); 16-bit: within one unit in
    the last place of the oracle rounded to the storage type.  grad_value and the per-sample gradients are also held
    to the max-norm tolerance level by level (the coarse level collects a quarter of the samples in a few hundred rows
    and would otherwise set the scale for all of them)."""
    ref = oracle_all(inp, with_grads)
    got = run_gpu(inp, device, with_grads)
    dtype = inp.value.dtype
    errs = {}
    names = ("output", "grad_value", "grad_sampling_locations", "grad_attention_weights")
    for name, g, r, tol in zip(names, got, ref, (fwd_tol, bwd_tol, bwd_tol, bwd_tol)):
        if r is None:
            continue
        r = np.asarray(r)
        if name == "grad_sampling_locations":
            edge = _cell_edge_mask(inp)
            # (levels thousands of pixels wide have float32 coordinates spaced 2^-13 apart: up to a thousandth of the samples)
            assert edge.mean() < 2e-3 or dtype != torch.float32, "too many samples sit on a cell edge for this check to mean anything"
            keep = ~edge[..., None]
            g, r = g * keep, r * keep
            errs["cell_edge_samples"] = int(edge.sum())
        errs[name] = rel_err(g, r)
        assert errs[name] <= tol, (name, errs)
        groups = None if name == "output" else level_slices(inp, "keys" if name == "grad_value" else "samples")
        nl = inp.spatial_shapes.shape[0]
        if groups is not None and name != "grad_value":
            groups = groups[:nl]   # (extra level slots of the weights carry zeros)
        for idx in (groups or []):
            if np.abs(r[idx]).max() > 0:
                assert rel_err(g[idx], r[idx]) <= tol, (name, "level", idx, rel_err(g[idx], r[idx]))
        if dtype == torch.float32:
            check_close(g, r, tol, name, groups)
        else:
            check_16bit(g, r, dtype, name, groups, tol32=FWD_FP32 if name == "output" else BWD_FP32)
    return errs


def test_library_is_the_in_tree_build():
    lib = _lib.load()
    assert lib.mxd_msda_version() == 103
    with open("/proc/self/maps") as f:
        assert any("drivingsdk_amd/lib/libmxd_msda.so" in line for line in f)


def test_hand_computed_case_exact(gpu_device, hand_case):
    c = hand_case
    inp = workloads.MsdaInputs(c["value"].float(), c["spatial_shapes"], c["level_start_index"],
                               c["sampling_locations"].float(), c["attention_weights"].float(),
                               c["grad_output"].float())
    out, gv, gl, ga = run_gpu(inp, gpu_device)
    # every quantity of this case is exactly representable; 0.25/0.75 weights are exact too
    np.testing.assert_allclose(out, c["output"].numpy(), rtol=0, atol=1e-6)
    np.testing.assert_allclose(gv, c["grad_value"].numpy(), rtol=0, atol=1e-6)
    np.testing.assert_allclose(gl, c["grad_sampling_locations"].numpy(), rtol=0, atol=1e-5)
    np.testing.assert_allclose(ga, c["grad_attention_weights"].numpy(), rtol=0, atol=1e-6)


def test_tiny_workload_fp32_vs_fixture_and_oracle(gpu_device):
    from conftest import GOLDEN
    inp = workloads.make_inputs("tiny", with_grad_output=True)
    errs = _check_all(inp, gpu_device, FWD_FP32, BWD_FP32)
    print("tiny fp32 errors", errs)
    fx = np.load(os.path.join(GOLDEN, "tiny_expected.npz"))
    out, gv, gl, ga = run_gpu(inp, gpu_device)
    assert rel_err(out[0, fx["rows_q"]], fx["output"]) <= FWD_FP32
    assert rel_err(gv[0, fx["rows_k"]], fx["grad_value"]) <= BWD_FP32
    assert rel_err(gl[0, fx["rows_q"]], fx["grad_sampling_locations"]) <= BWD_FP32
    assert rel_err(ga[0, fx["rows_q"]], fx["grad_attention_weights"]) <= BWD_FP32


def test_detr_encoder_fp32_full_size(gpu_device):
    inp = workloads.make_inputs("detr_encoder_bwd")
    errs = _check_all(inp, gpu_device, FWD_FP32, BWD_FP32)
    print("detr_encoder fp32 errors", errs)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_bevformer_sca_forward(gpu_device, dtype):
    inp = workloads.make_inputs("bevformer_sca", dtype=dtype)
    errs = _check_all(inp, gpu_device, FWD_FP32 if dtype == torch.float32 else HALF, None, with_grads=False)
    print("bevformer_sca", dtype, errs)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_head_dim_128_forward_and_backward(gpu_device, dtype):
    inp = workloads.make_inputs("head_dim_128", dtype=dtype, with_grad_output=True)
    tol = half_tol(dtype)   # (bfloat16: its unit round-off, 2^-8)
    errs = _check_all(inp, gpu_device, tol, tol)
    print("head_dim_128", dtype, errs)


# shapes of the reference's operator test: [bs, num_queries, embed_dims, num_heads, num_levels, num_points]
REFERENCE_SHAPES = [
    [6, 9680, 32, 8, 1, 8],
    [6, 9680, 32, 8, 4, 4],
    [6, 9680, 37, 4, 5, 3],
    [1, 27216, 16, 5, 3, 1],
    [1, 1450, 64, 6, 1, 2],
    [1, 1450, 64, 8, 8, 8],
    [1, 1450, 128, 8, 8, 8],
    [1, 1450, 256, 8, 8, 8],
    [1, 1450, 147, 7, 3, 21],
    [1, 1890, 32, 7, 4, 16],
]


@pytest.mark.parametrize("shape", REFERENCE_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_reference_test_shapes_fp32(gpu_device, shape):
    inp = workloads.reference_test_inputs(shape, seed=sum(shape))
    errs = _check_all(inp, gpu_device, FWD_FP32, BWD_FP32)
    print(shape, errs)


def test_reference_fp16_case(gpu_device):
    inp = workloads.reference_test_inputs([6, 9680, 32, 8, 4, 4], dtype=torch.float16, seed=7)
    errs = _check_all(inp, gpu_device, HALF, HALF)
    print("fp16", errs)


@pytest.mark.parametrize("fill", [float("nan"), float("inf")])
def test_nan_and_inf_inputs_give_exact_zeros(gpu_device, fill):
    inp = workloads.reference_test_inputs([6, 9680, 32, 8, 4, 4], fill=fill)
    for arr in run_gpu(inp, gpu_device):
        assert np.all(arr == 0.0)


def test_zero_padding_is_exact(gpu_device):
    """Samples at and beyond the validity edges: same zero / non-zero pattern as the oracle,
    exact zeros outside, and NaNs in pixels a sample does not touch never leak."""
    # power-of-two sizes: every pixel coordinate below is exact in float32 and float64 alike,
    # so the GPU and the oracle must agree on which corners exist, not only on the numbers
    H, W = 4, 8
    shapes, lsi = workloads.level_tensors(((H, W),))
    xs = [(w + 0.5) / W for w in (-1.5, -1.0, -0.75, -0.5, 0.0, 0.5, W - 1.5, W - 1.0, W - 0.75, W - 0.5, W, W + 0.5)]
    ys = [(h + 0.5) / H for h in (-1.5, -1.0, -0.75, -0.5, 0.0, 0.5, H - 1.5, H - 1.0, H - 0.75, H - 0.5, H, H + 0.5)]
    pts = torch.tensor([(x, y) for x in xs for y in ys], dtype=torch.float32)
    nq = pts.shape[0]
    g = torch.Generator().manual_seed(5)
    value = torch.randn(1, H * W, 2, 8, generator=g)
    loc = pts.view(1, nq, 1, 1, 1, 2).expand(1, nq, 2, 1, 1, 2).contiguous()
    attn = torch.ones(1, nq, 2, 1, 1)
    gout = torch.randn(1, nq, 16, generator=g)
    inp = workloads.MsdaInputs(value, shapes, lsi, loc, attn, gout)
    ref = oracle_all(inp)
    got = run_gpu(inp, gpu_device)
    for g_, r_ in zip(got, ref):
        assert np.array_equal(g_ == 0.0, r_ == 0.0)
    assert rel_err(got[0], ref[0]) <= FWD_FP32
    # a NaN pixel poisons only the samples whose in-image corners include it
    value2 = value.clone()
    value2[0, 0] = float("nan")  # pixel (0,0)
    inp2 = inp._replace(value=value2)
    out2 = run_gpu(inp2, gpu_device, with_grads=False)[0]
    w_im = pts[:, 0].double() * W - 0.5
    h_im = pts[:, 1].double() * H - 0.5
    touches = ((w_im > -1) & (w_im < 1) & (h_im > -1) & (h_im < 1)).numpy()
    assert np.array_equal(np.isnan(out2[0]).any(-1), touches)


def test_more_attention_levels_than_spatial_shapes(gpu_device):
    """Extra level slots are ignored in the forward pass and receive zero gradients."""
    g = torch.Generator().manual_seed(11)
    shapes, lsi = workloads.level_tensors(((9, 7), (4, 6)))
    nk = int(shapes.prod(1).sum())
    value = torch.randn(2, nk, 4, 16, generator=g)
    loc = torch.rand(2, 50, 4, 3, 2, 2, generator=g)
    attn = torch.rand(2, 50, 4, 3, 2, generator=g)
    gout = torch.randn(2, 50, 64, generator=g)
    inp = workloads.MsdaInputs(value, shapes, lsi, loc, attn, gout)
    errs = _check_all(inp, gpu_device, FWD_FP32, BWD_FP32)
    got = run_gpu(inp, gpu_device)
    assert np.all(got[2][:, :, :, 2:] == 0) and np.all(got[3][:, :, :, 2:] == 0)
    print(errs)


@pytest.mark.parametrize("hd,nh,dtype", [(1, 3, torch.float32), (2, 8, torch.float16), (6, 2, torch.float32),
                                         (12, 16, torch.float32), (20, 1, torch.bfloat16), (250, 2, torch.float32),
                                         (255, 1, torch.float16), (24, 8, torch.float16), (200, 4, torch.bfloat16)])
def test_odd_head_dims_and_head_counts(gpu_device, hd, nh, dtype):
    g = torch.Generator().manual_seed(hd * 100 + nh)
    levels = ((11, 13), (5, 7), (1, 1))
    shapes, lsi = workloads.level_tensors(levels)
    nk = int(shapes.prod(1).sum())
    nq, npts, bs = 77, 5, 2
    value = torch.randn(bs, nk, nh, hd, generator=g)
    loc = torch.rand(bs, nq, nh, 3, npts, 2, generator=g) * 1.2 - 0.1
    attn = torch.rand(bs, nq, nh, 3, npts, generator=g)
    gout = torch.randn(bs, nq, nh * hd, generator=g)
    inp = workloads.MsdaInputs(*[t.to(dtype) if t.is_floating_point() else t for t in
                                 (value, shapes, lsi, loc, attn, gout)])
    tol_f, tol_b = (FWD_FP32, BWD_FP32) if dtype == torch.float32 else (half_tol(dtype), half_tol(dtype))
    errs = _check_all(inp, gpu_device, tol_f, tol_b)
    print(hd, nh, dtype, errs)


def test_unaligned_and_non_contiguous_inputs(gpu_device):
    """Views with an odd storage offset and strided layouts go through the same path."""
    import mx_driving
    inp = workloads.reference_test_inputs([2, 300, 32, 8, 2, 4], seed=3)
    ref = oracle_all(inp, with_grads=False)[0]
    d = to_device(inp, gpu_device)
    # value at a 4-byte (not 16-byte) aligned address
    buf = torch.empty(d.value.numel() + 1, device=gpu_device)
    v_off = buf[1:].view_as(d.value)
    v_off.copy_(d.value)
    assert v_off.data_ptr() % 16 == 4
    out = mx_driving.multi_scale_deformable_attn(v_off, d.spatial_shapes, d.level_start_index,
                                                 d.sampling_locations, d.attention_weights)
    assert rel_err(out.double().cpu().numpy(), ref) <= FWD_FP32
    # non-contiguous value (transposed storage) and locations
    v_nc = d.value.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    l_nc = d.sampling_locations.flip(-1).contiguous().flip(-1)
    assert not v_nc.is_contiguous()
    out = mx_driving.multi_scale_deformable_attn(v_nc, d.spatial_shapes, d.level_start_index, l_nc,
                                                 d.attention_weights)
    assert rel_err(out.double().cpu().numpy(), ref) <= FWD_FP32


def test_int64_metadata_and_mixed_float_dtypes_are_coerced(gpu_device):
    import mx_driving
    inp = workloads.reference_test_inputs([1, 200, 32, 8, 2, 4], seed=4)
    ref = oracle_all(inp, with_grads=False)[0]
    d = to_device(inp, gpu_device)
    assert d.spatial_shapes.dtype == torch.int64
    out = mx_driving.multi_scale_deformable_attn(d.value, d.spatial_shapes, d.level_start_index,
                                                 d.sampling_locations.double(), d.attention_weights.half())
    assert out.dtype == torch.float32
    # attention weights went through float16 here: compare loosely
    assert rel_err(out.double().cpu().numpy(), ref) <= HALF


def test_int64_metadata_is_read_in_place(gpu_device):
    """Level metadata as int64 (what callers hold) is handed to the library with the MXD_META_I64 flag instead of
    being cast: same results, bit for bit, as with int32 tensors -- forward, backward and the fused form."""
    from drivingsdk_amd import _C
    inp = workloads.make_inputs("detr_encoder_bwd", with_grad_output=True, scale_queries=0.03)
    d = to_device(inp, gpu_device)
    sh64, ls64 = d.spatial_shapes, d.level_start_index
    assert sh64.dtype == torch.int64 and ls64.dtype == torch.int64
    sh32, ls32 = sh64.int(), ls64.int()
    args = (d.sampling_locations, d.attention_weights)
    out64 = _C.multi_scale_deformable_attn(d.value, sh64, ls64, *args)
    out32 = _C.multi_scale_deformable_attn(d.value, sh32, ls32, *args)
    assert torch.equal(out64, out32)
    g64 = _C.multi_scale_deformable_attn_backward(d.value, sh64, ls64, *args, d.grad_output)
    g32 = _C.multi_scale_deformable_attn_backward(d.value, sh32, ls32, *args, d.grad_output)
    assert torch.equal(g64[1], g32[1]) and torch.equal(g64[2], g32[2])
    assert rel_err(g64[0].double().cpu().numpy(), g32[0].double().cpu().numpy()) <= 1e-6   # summation order varies
    bs, nq, nh, nl, npts, _ = d.sampling_locations.shape
    gen = torch.Generator().manual_seed(8)
    ref = torch.rand(bs, nq, nl, 2, generator=gen).to(gpu_device)
    off = torch.randn(bs, nq, nh, nl, npts, 2, generator=gen).to(gpu_device)
    logits = torch.randn(bs, nq, nh, nl * npts, generator=gen).to(gpu_device)
    assert torch.equal(_C.msda_fused_forward(d.value, sh64, ls64, ref, off, logits),
                       _C.msda_fused_forward(d.value, sh32, ls32, ref, off, logits))


def test_autocast_runs_in_float32(gpu_device):
    import mx_driving
    inp = workloads.reference_test_inputs([1, 200, 32, 8, 2, 4], seed=5)
    ref = oracle_all(inp, with_grads=False)[0]
    d = to_device(inp, gpu_device)
    with torch.autocast("cuda", dtype=torch.float16):
        out = mx_driving.multi_scale_deformable_attn(d.value.half(), d.spatial_shapes, d.level_start_index,
                                                     d.sampling_locations, d.attention_weights)
    assert out.dtype == torch.float32
    assert rel_err(out.double().cpu().numpy(), ref) <= HALF


def test_runs_on_a_side_stream_and_is_repeatable(gpu_device):
    import mx_driving
    inp = workloads.make_inputs("tiny", with_grad_output=True)
    d = to_device(inp, gpu_device)
    ref = oracle_all(inp)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        outs = []
        for _ in range(3):
            v = d.value.clone().requires_grad_()
            out = mx_driving.multi_scale_deformable_attn(v, d.spatial_shapes, d.level_start_index,
                                                         d.sampling_locations, d.attention_weights)
            out.backward(d.grad_output)
            outs.append((out.detach(), v.grad))
    s.synchronize()
    for out, gv in outs:
        assert torch.equal(out, outs[0][0])                       # forward is deterministic
        assert rel_err(gv.double().cpu().numpy(), ref[1]) <= BWD_FP32  # atomics: order-dependent rounding only


def test_forward_and_backward_replay_in_a_hip_graph(gpu_device):
    """The launches of one forward + backward (zero-fill kernel, both backward kernels; no memset nodes) captured
    in a HIP graph: three replays with fresh inputs copied into the captured tensors, the program's own eager
    work and synchronisations between them, each replay compared with the eager result for the same inputs."""
    from drivingsdk_amd import _C
    base = workloads.make_inputs("detr_encoder_bwd", with_grad_output=True, scale_queries=0.05)
    d = to_device(base, gpu_device)
    sh, lsi = d.spatial_shapes.int(), d.level_start_index.int()
    static = [t.clone() for t in (d.value, d.sampling_locations, d.attention_weights, d.grad_output)]

    def run(v, lo, at, go):
        out = _C.multi_scale_deformable_attn(v, sh, lsi, lo, at)
        return (out,) + tuple(_C.multi_scale_deformable_attn_backward(v, sh, lsi, lo, at, go))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            run(*static)  # warm-up outside the capture (first-use set-up of the kernels)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run(*static)
    g = torch.Generator().manual_seed(31)
    for rep in range(3):
        fresh = [torch.randn(t.shape, generator=g) * 0.5 for t in static]
        fresh[1] = torch.rand(static[1].shape, generator=g) * 1.2 - 0.1
        fresh[2] = torch.rand(static[2].shape, generator=g)
        for dst, src in zip(static, fresh):
            dst.copy_(src.to(gpu_device))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        eager = run(*[t.clone() for t in static])       # eager work between the replays
        torch.cuda.synchronize()
        for name, a_, b_, tol in zip(("output", "grad_value", "grad_loc", "grad_attn"), got, eager,
                                     (0.0, 1e-6, 0.0, 0.0)):
            err = rel_err(a_.double().cpu().numpy(), b_.double().cpu().numpy())
            assert err <= tol, (rep, name, err)   # (grad_value: summation order varies from run to run)


def test_linearity_at_full_size(gpu_device):
    """Size-independent property at the benchmark shape: linear in value and in the weights."""
    import mx_driving
    d = to_device(workloads.make_inputs("detr_encoder"), gpu_device)
    f = lambda v, a: mx_driving.multi_scale_deformable_attn(v, d.spatial_shapes, d.level_start_index,
                                                            d.sampling_locations, a)
    base = f(d.value, d.attention_weights)
    assert torch.equal(f(2 * d.value, d.attention_weights), 2 * base)       # scaling by 2 is exact
    assert torch.equal(f(d.value, 0.5 * d.attention_weights), 0.5 * base)
    other = torch.randn_like(d.value)
    lhs = f(d.value + other, d.attention_weights)
    rhs = base + f(other, d.attention_weights)
    assert rel_err(lhs.double().cpu().numpy(), rhs.double().cpu().numpy()) <= FWD_FP32


@pytest.mark.parametrize("name", ["bevformer_sca", "detr_encoder_bwd"])
def test_adjoint_identities_at_full_size(gpu_device, name):
    """Size-independent properties of the backward at the largest shapes: the forward is linear in value and in
    the attention weights, so <out, g> = <value, grad_value> = <attention_weights, grad_attention_weights> for any
    g; and along its own direction the location gradient matches a central difference of the forward (bilinear
    interpolation is piecewise linear in the location, so the difference quotient is exact except for the few
    samples whose cell the step crosses).  Sums in float64 on the device."""
    import mx_driving
    d = to_device(workloads.make_inputs(name, with_grad_output=True), gpu_device)
    value = d.value.clone().requires_grad_()
    loc = d.sampling_locations.clone().requires_grad_()
    attn = d.attention_weights.clone().requires_grad_()
    out = mx_driving.multi_scale_deformable_attn(value, d.spatial_shapes, d.level_start_index, loc, attn)
    g = d.grad_output
    out.backward(g)
    dot = lambda a, b: float((a.double() * b.double()).sum())
    lhs = dot(out.detach(), g)
    scale = float(out.detach().double().norm() * g.double().norm())
    assert abs(lhs - dot(value.detach(), value.grad)) <= 1e-6 * scale
    assert abs(lhs - dot(attn.detach(), attn.grad)) <= 1e-6 * scale
    # directional derivative with respect to the locations, along the gradient itself (a random direction would be
    # nearly orthogonal to it): steps of at most 1/64 pixel of the finest level
    direction = loc.grad / loc.grad.abs().max()
    eps = 1.0 / (64.0 * float(d.spatial_shapes.max()))
    f = lambda l: mx_driving.multi_scale_deformable_attn(d.value, d.spatial_shapes, d.level_start_index, l,
                                                         d.attention_weights)
    with torch.no_grad():
        fd = dot(f(d.sampling_locations + eps * direction) - f(d.sampling_locations - eps * direction), g) / (2 * eps)
    an = dot(loc.grad, direction)
    print(name, "directional derivative: central difference", fd, "gradient", an)
    # (the few samples that change cell inside the step, and float32 rounding of the locations, leave a per cent)
    assert abs(fd - an) <= 0.02 * abs(an), (fd, an)


def test_c_abi_direct_call_and_error_codes(gpu_device):
    """Straight through the C ABI with raw pointers (what a non-Python host would do)."""
    lib = _lib.load()
    inp = workloads.make_inputs("tiny")
    d = to_device(inp, gpu_device)
    shapes, lsi = d.spatial_shapes.int(), d.level_start_index.int()
    bs, nk, nh, hd = d.value.shape
    _, nq, _, nl, npts, _ = d.sampling_locations.shape
    out = torch.empty(bs, nq, nh * hd, device=gpu_device)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.mxd_msda_forward(d.value.data_ptr(), shapes.data_ptr(), lsi.data_ptr(), d.sampling_locations.data_ptr(),
                              d.attention_weights.data_ptr(), out.data_ptr(), 0, bs, nk, nh, hd, nl, nl, nq, npts,
                              stream)
    assert rc == 0
    torch.cuda.synchronize()
    ref = oracle_all(inp, with_grads=False)[0]
    assert rel_err(out.double().cpu().numpy(), ref) <= FWD_FP32
    # error paths never launch
    assert lib.mxd_msda_forward(None, shapes.data_ptr(), lsi.data_ptr(), d.sampling_locations.data_ptr(),
                                d.attention_weights.data_ptr(), out.data_ptr(), 0, bs, nk, nh, hd, nl, nl, nq, npts,
                                stream) == -3
    assert lib.mxd_msda_forward(d.value.data_ptr(), shapes.data_ptr(), lsi.data_ptr(),
                                d.sampling_locations.data_ptr(), d.attention_weights.data_ptr(), out.data_ptr(), 0,
                                bs, nk, nh, 257, nl, nl, nq, npts, stream) == -2
    assert "256" in _lib.last_error()
    # fp16 backward without a workspace is refused
    assert lib.mxd_msda_backward(d.value.data_ptr(), shapes.data_ptr(), lsi.data_ptr(),
                                 d.sampling_locations.data_ptr(), d.attention_weights.data_ptr(), out.data_ptr(),
                                 out.data_ptr(), out.data_ptr(), out.data_ptr(), None, 0, 1, bs, nk, nh, hd, nl, nl,
                                 nq, npts, 0, stream) == -4


def _backward_c_abi(d, flags, grad_value):
    """One raw mxd_msda_backward call (float32) on device inputs d; returns (grad_loc, grad_attn)."""
    lib = _lib.load()
    shapes, lsi = d.spatial_shapes.int().contiguous(), d.level_start_index.int().contiguous()
    bs, nk, nh, hd = d.value.shape
    _, nq, _, nl, npts, _ = d.sampling_locations.shape
    gl, ga = torch.empty_like(d.sampling_locations), torch.empty_like(d.attention_weights)
    dims = (bs, nk, nh, hd, nl, nl, nq, npts)
    nbytes = lib.mxd_msda_backward_workspace_bytes(0, *dims)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=d.value.device)
    rc = lib.mxd_msda_backward(d.value.data_ptr(), shapes.data_ptr(), lsi.data_ptr(), d.sampling_locations.data_ptr(),
                               d.attention_weights.data_ptr(), d.grad_output.data_ptr(), grad_value.data_ptr(),
                               gl.data_ptr(), ga.data_ptr(), ws.data_ptr(), nbytes, 0, *dims, flags,
                               torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    return gl, ga


@pytest.mark.parametrize("name,scale", [("tiny", 1.0), ("detr_encoder_bwd", 0.25)])
def test_backward_accumulate_flag_adds_into_grad_value(gpu_device, name, scale):
    """MXD_BWD_ACCUMULATE: the image keeps its contents and the gradient is added to it, twice in a row."""
    inp = workloads.make_inputs(name, with_grad_output=True, scale_queries=scale)
    ref_gv = oracle_all(inp)[1]
    d = to_device(inp, gpu_device)
    gv = torch.full_like(d.value, 0.5)
    _backward_c_abi(d, _lib.BWD_ACCUMULATE, gv)
    assert rel_err(gv.double().cpu().numpy(), 0.5 + ref_gv) <= BWD_FP32
    _backward_c_abi(d, _lib.BWD_ACCUMULATE, gv)
    assert rel_err(gv.double().cpu().numpy(), 0.5 + 2 * ref_gv) <= BWD_FP32
    _backward_c_abi(d, 0, gv)  # without the flag the image is overwritten
    assert rel_err(gv.double().cpu().numpy(), ref_gv) <= BWD_FP32


@pytest.mark.parametrize("env", [{"MXD_MSDA_BWD_ATOMIC": "1"}, {"MXD_MSDA_BWD_TILE_Q": "64"},
                                 {"MXD_MSDA_BWD_TILE_Q": "256"}, {"MXD_MSDA_TILE_TARGET": "128"},
                                 {"MXD_MSDA_TILE_TARGET": "1000000"}, {"MXD_MSDA_XCD_MODE": "0"},
                                 {"MXD_MSDA_BWD_FILL_KERNEL": "1"}],
                         ids=lambda e: ",".join(f"{k[9:]}={v}" for k, v in e.items()))
def test_backward_launch_variants_agree_with_the_oracle(gpu_device, monkeypatch, env):
    """The tuning knobs read at call time select other code paths (one-kernel atomic backward, other
    workgroup sizes of the first kernel, tiles split into very many or no query chunks, plain workgroup
    mapping, zero-fill by a kernel of its own); every one of them must give the same gradients."""
    set_tuning(monkeypatch, **env)
    for name, scale in (("tiny", 1.0), ("detr_encoder_bwd", 0.25)):
        inp = workloads.make_inputs(name, with_grad_output=True, scale_queries=scale)
        errs = _check_all(inp, gpu_device, FWD_FP32, BWD_FP32)
        print(env, name, errs)


@pytest.mark.parametrize("split", ["2", "0"], ids=["two-units-per-query", "one-unit-per-query"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("nl,nl_attn,npts", [(4, 4, 8), (3, 3, 7), (2, 3, 12), (1, 1, 17), (4, 5, 5)])
def test_queries_of_17_to_32_samples(gpu_device, monkeypatch, nl, nl_attn, npts, dtype, split):
    """The backward's first kernel can give a query of 17 to 32 samples two units of 16 samples each (workgroups of half
    as many queries that make one pass: by default from 25 samples on, with MXD_MSDA_BWD_UNIT_SPLIT=2 from 17 on);
    MXD_MSDA_BWD_UNIT_SPLIT=0 keeps one unit per query and two chunks.  Both against
    the oracle, with a query count that leaves the last workgroup partly filled and, in two cases, level slots in the
    weights beyond spatial_shapes (zero gradients)."""
    set_tuning(monkeypatch, MXD_MSDA_BWD_UNIT_SPLIT=split)
    levels = ((37, 52), (19, 26), (10, 13), (5, 7))[:nl]
    shapes, lsi = workloads.level_tensors(levels)
    nk = int(shapes.prod(1).sum())
    bs, nq, nh, hd = 2, 1237, 3, 32
    g = torch.Generator().manual_seed(100 * nl + npts)
    inp = workloads.MsdaInputs(torch.randn(bs, nk, nh, hd, generator=g).to(dtype), shapes, lsi,
                               (torch.rand(bs, nq, nh, nl_attn, npts, 2, generator=g) * 1.2 - 0.1).to(dtype),
                               torch.rand(bs, nq, nh, nl_attn, npts, generator=g).to(dtype),
                               torch.randn(bs, nq, nh * hd, generator=g).to(dtype))
    plan = _lib.make_plan(1, {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype], bs, nk, nh, hd, nl, nl_attn, nq, npts)
    units = plan.units_per_wave * plan.waves_per_block * plan.iters
    assert plan.tile_q * (2 if split == "2" else 1) == units
    tol = (FWD_FP32, BWD_FP32) if dtype == torch.float32 else (half_tol(dtype),) * 2
    errs = _check_all(inp, gpu_device, *tol)
    if nl_attn > nl:
        got = run_gpu(inp, gpu_device)
        assert np.all(got[2][:, :, :, nl:] == 0) and np.all(got[3][:, :, :, nl:] == 0)
    print(errs)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("nl,npts", [(4, 4), (3, 5), (1, 1), (4, 8), (2, 13)])
def test_first_backward_kernel_with_its_geometry_as_constants(gpu_device, monkeypatch, nl, npts, dtype):
    """Launches whose rows are read by 8 lanes and whose workgroups make one pass (up to 16 samples per query, or up to 32
    with two units per query) take an instantiation of the first backward kernel that has this geometry as constants;
    MXD_MSDA_BWD_FIXED=0 sends them through the general one.  Both against the oracle, and the gradients of locations and
    weights (which do not depend on the order of any sum) bit for bit against each other; the query count leaves the last
    workgroup partly filled."""
    levels = ((37, 52), (19, 26), (10, 13), (5, 7))[:nl]
    shapes, lsi = workloads.level_tensors(levels)
    nk = int(shapes.prod(1).sum())
    bs, nq, nh, hd = 2, 1237, 8, 32
    g = torch.Generator().manual_seed(7 * nl + npts)
    inp = workloads.MsdaInputs(torch.randn(bs, nk, nh, hd, generator=g).to(dtype), shapes, lsi,
                               (torch.rand(bs, nq, nh, nl, npts, 2, generator=g) * 1.2 - 0.1).to(dtype),
                               torch.rand(bs, nq, nh, nl, npts, generator=g).to(dtype),
                               torch.randn(bs, nq, nh * hd, generator=g).to(dtype))
    plan = _lib.make_plan(1, {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype], bs, nk, nh, hd, nl, nl, nq, npts)
    assert plan.lanes_per_row == 8 and plan.units_per_wave == 8 and plan.iters == 1
    tol = (FWD_FP32, BWD_FP32) if dtype == torch.float32 else (half_tol(dtype),) * 2
    got = {}
    for fixed in ("1", "0"):
        set_tuning(monkeypatch, MXD_MSDA_BWD_FIXED=fixed)
        _check_all(inp, gpu_device, *tol)
        got[fixed] = run_gpu(inp, gpu_device)
    assert np.array_equal(got["1"][2], got["0"][2]) and np.array_equal(got["1"][3], got["0"][3])


@pytest.mark.parametrize("rec_lds", ["0", "1"], ids=["records-stored-singly", "slab-in-lds"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("nl,npts", [(4, 4), (3, 5), (1, 1), (4, 8), (2, 13)])
def test_first_backward_kernel_with_rows_of_256_bytes_as_constants(gpu_device, monkeypatch, nl, npts, dtype, rec_lds):
    """Rows of 256 bytes (64 float32 channels, 128 channels of a 16-bit type) are read by 16 lanes of 16 bytes, four units
    per wavefront: such launches take an instantiation of the first backward kernel with that geometry as constants,
    whatever their number of iterations and chunks (here one to two chunks per query), with the records stored one by one
    or collected in LDS.  Against the oracle, and the gradients of locations and weights bit for bit against the general
    instantiation (MXD_MSDA_BWD_FIXED=0)."""
    levels = ((37, 52), (19, 26), (10, 13), (5, 7))[:nl]
    shapes, lsi = workloads.level_tensors(levels)
    nk = int(shapes.prod(1).sum())
    bs, nq, nh = 2, 1237, 3
    hd = 64 if dtype == torch.float32 else 128
    g = torch.Generator().manual_seed(11 * nl + npts)
    inp = workloads.MsdaInputs(torch.randn(bs, nk, nh, hd, generator=g).to(dtype), shapes, lsi,
                               (torch.rand(bs, nq, nh, nl, npts, 2, generator=g) * 1.2 - 0.1).to(dtype),
                               torch.rand(bs, nq, nh, nl, npts, generator=g).to(dtype),
                               torch.randn(bs, nq, nh * hd, generator=g).to(dtype))
    set_tuning(monkeypatch, MXD_MSDA_BWD_REC_LDS=rec_lds)
    plan = _lib.make_plan(1, {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype], bs, nk, nh, hd, nl, nl, nq, npts)
    assert plan.lanes_per_row == 16 and plan.units_per_wave == 4 and plan.npass == 1
    tol = (FWD_FP32, BWD_FP32) if dtype == torch.float32 else (half_tol(dtype),) * 2
    got = {}
    for fixed in ("1", "0"):
        set_tuning(monkeypatch, MXD_MSDA_BWD_REC_LDS=rec_lds, MXD_MSDA_BWD_FIXED=fixed)
        _check_all(inp, gpu_device, *tol)
        got[fixed] = run_gpu(inp, gpu_device)
    assert np.array_equal(got["1"][2], got["0"][2]) and np.array_equal(got["1"][3], got["0"][3])


@pytest.mark.parametrize("lds", ["0", "2048", "32768", "49152", "65536"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_forward_level_cache_sizes(gpu_device, monkeypatch, lds, dtype):
    """The forward's level cache (rows of the last levels held in LDS) is switched by an estimate of the level
    sizes; here it is forced off and on with room for no, one, several and all levels, for every dtype."""
    set_tuning(monkeypatch, MXD_MSDA_FWD_LDS=lds, MXD_MSDA_FWD_CU=0)   # (the general forward kernel's cache)
    tol = FWD_FP32 if dtype == torch.float32 else half_tol(dtype)
    for name, scale in (("tiny", 1.0), ("detr_encoder", 0.1)):
        inp = workloads.make_inputs(name, dtype=dtype, scale_queries=scale)
        want = oracle_all(inp, with_grads=False)[0]
        got = run_gpu(inp, gpu_device, with_grads=False)[0]
        assert rel_err(got, want) <= tol, (name, lds, dtype)


@pytest.mark.parametrize("env", [{"MXD_MSDA_FWD_AHEAD": "0"}, {"MXD_MSDA_FWD_AHEAD": "0", "MXD_MSDA_FWD_LDS": "0"},
                                 {"MXD_MSDA_FWD_LDS": "0"}, {"MXD_MSDA_FWD_WGQ": "64"}, {"MXD_MSDA_FWD_WGQ": "512"},
                                 {"MXD_MSDA_FWD_LDS": "0", "MXD_MSDA_FWD_ITERS": "3"},
                                 {"MXD_MSDA_FWD_CU": "1"}, {"MXD_MSDA_FWD_CU": "1", "MXD_MSDA_FWD_CU_WGS": "3"},
                                 {"MXD_MSDA_FWD_CU": "1", "MXD_MSDA_FWD_CU_WGS": "500"}],
                         ids=lambda e: ",".join(f"{k[9:]}={v}" for k, v in e.items()))
def test_forward_launch_variants_agree(gpu_device, monkeypatch, env):
    """The forward requests the samples of a wavefront's next units ahead of the gather of the current ones (with and
    without the level cache, one or several iterations per wavefront, the last one partly filled), and for large
    problems it runs as one workgroup per CU with the last levels in LDS (forced here for small ones, with few and
    with very many workgroups per (batch, head)); every such launch form must give the same output, bit for bit,
    as the form without it, and meet the oracle."""
    for name, scale in (("tiny", 1.0), ("detr_encoder", 0.13), ("bevformer_sca", 0.03)):  # (the last: 32 samples per unit)
        inp = workloads.make_inputs(name, scale_queries=scale)
        want = oracle_all(inp, with_grads=False)[0]
        base = run_gpu(inp, gpu_device, with_grads=False)[0]
        assert rel_err(base, want) <= FWD_FP32, name
        with monkeypatch.context() as m:
            set_tuning(m, **env)
            got = run_gpu(inp, gpu_device, with_grads=False)[0]
        _lib.reload_tuning()   # (the context has restored the environment)
        assert np.array_equal(np.asarray(got), np.asarray(base)), (name, env)


def test_beyond_the_reference_limits(gpu_device):
    """The reference refuses num_levels * num_points > 64; here 100 samples per (query, head) -- seven staging
    passes, the last one partly filled -- at the largest head_dim (256), forward and gradients."""
    g = torch.Generator().manual_seed(64)
    shapes, lsi = workloads.level_tensors(((9, 14), (7, 5), (4, 6), (3, 3), (2, 2)))
    nk = int(shapes.prod(1).sum())
    bs, nq, nh, hd, nl, npts = 2, 77, 3, 256, 5, 20
    inp = workloads.MsdaInputs(torch.randn(bs, nk, nh, hd, generator=g), shapes, lsi,
                               torch.rand(bs, nq, nh, nl, npts, 2, generator=g) * 1.2 - 0.1,
                               torch.rand(bs, nq, nh, nl, npts, generator=g),
                               torch.randn(bs, nq, nh * hd, generator=g))
    print(_check_all(inp, gpu_device, FWD_FP32, BWD_FP32))


def test_reference_onnx_export_shape(gpu_device):
    """The shape of the reference's ONNX export test (tests/onnx/test_wrapper_onnx_ops.py:57-65): five large levels
    whose sizes do not decrease (nk = 114400, 229 tiles per (batch, head)), 10000 queries; batch 2 of its 6."""
    g = torch.Generator().manual_seed(114400)
    shapes, lsi = workloads.level_tensors(((160, 140), (130, 120), (160, 240), (130, 120), (160, 140)))
    assert lsi.tolist() == [0, 22400, 38000, 76400, 92000]
    bs, nq, nh, hd, nl, npts = 2, 10000, 8, 32, 5, 4
    inp = workloads.MsdaInputs(torch.rand(bs, 114400, nh, hd, generator=g), shapes, lsi,
                               torch.rand(bs, nq, nh, nl, npts, 2, generator=g),
                               torch.rand(bs, nq, nh, nl, npts, generator=g),
                               torch.randn(bs, nq, nh * hd, generator=g))
    print(_check_all(inp, gpu_device, FWD_FP32, BWD_FP32))


@pytest.mark.parametrize("nq", [16, 3000])
def test_documentation_example_all_samples_in_one_pixel(gpu_device, nq):
    """The call example of the reference's documentation (docs/zh/api/context/multi_scale_deformable_attn.md:35-54):
    one 100x100 level and every sampling location equal to 0.005, so all samples of a head fall into the same cell;
    also with many queries, where one pixel list of the tile pass holds every record."""
    g = torch.Generator().manual_seed(5)
    shapes, lsi = workloads.level_tensors(((100, 100),))
    bs, nh, hd, nl, npts = 1, 4, 32, 1, 8
    inp = workloads.MsdaInputs(torch.rand(bs, 10000, nh, hd, generator=g) * 0.01, shapes, lsi,
                               torch.ones(bs, nq, nh, nl, npts, 2) * 0.005,
                               torch.rand(bs, nq, nh, nl, npts, generator=g) + 1e-5,
                               torch.ones(bs, nq, nh * hd))
    # 0.005 * 100 - 0.5 is pixel coordinate 0 to within rounding: every sample sits on a cell edge, where the
    # location gradient jumps, so that gradient is only checked for being finite
    want = oracle_all(inp)
    got = run_gpu(inp, gpu_device)
    for k, tol in ((0, FWD_FP32), (1, BWD_FP32), (3, BWD_FP32)):
        assert rel_err(got[k], want[k]) <= tol, k
    assert np.all(np.isfinite(got[2]))


@pytest.mark.parametrize("levels,hd", [(((10, 20),), 32), (((23, 31), (9, 7)), 64)], ids=["200px", "713px+63px"])
def test_hot_pixels_get_extra_lists_in_the_tile_pass(gpu_device, monkeypatch, levels, hd):
    """A tile smaller than its workgroup leaves lane groups without pixels; pixels that collect far more
    list entries than the others get extra lists there after the first round (msda_bwd_tiles.hip).  Half of the
    samples go to three spots of the first level (one of them in its last, partial tile), the others are
    uniform, and a large work-item size keeps every tile in one work item, so that the rounds after the first
    run with extra lists, pair entries among the moved ones."""
    set_tuning(monkeypatch, MXD_MSDA_TILE_TARGET=1000000)
    g = torch.Generator().manual_seed(11)
    shapes, lsi = workloads.level_tensors(levels)
    nk = int(shapes.prod(1).sum())
    bs, nq, nh, nl, npts = 2, 6000, 2, len(levels), 4
    loc = torch.rand(bs, nq, nh, nl, npts, 2, generator=g) * 1.1 - 0.05
    H, W = levels[0]
    spots = torch.tensor([[(3.3 + 0.5) / W, (4.6 + 0.5) / H], [(W - 1.4 + 0.5) / W, (H - 1.7 + 0.5) / H],
                          [(W - 5.25 + 0.5) / W, (H - 1.2 + 0.5) / H]])
    pick = torch.randint(0, 6, (bs, nq, nh, npts), generator=g)
    for k in range(3):
        loc[:, :, :, 0][pick == k] = spots[k]
    inp = workloads.MsdaInputs(torch.randn(bs, nk, nh, hd, generator=g), shapes, lsi, loc,
                               torch.rand(bs, nq, nh, nl, npts, generator=g), torch.randn(bs, nq, nh * hd, generator=g))
    errs = _check_all(inp, gpu_device, FWD_FP32, BWD_FP32)
    print(levels, errs)


@pytest.mark.parametrize("seed", range(8))
def test_random_hot_spots_many_rounds(gpu_device, monkeypatch, seed):
    """Random level shapes whose tiles are partly empty, enough samples for several rounds of the tile pass per
    work item, a random share of them on a few random spots (anywhere, also across tile and image borders), odd
    head sizes, float32 and float16; with the default work-item size for even seeds and unsplit tiles for odd ones."""
    rng = np.random.default_rng(100 + seed)
    if seed % 2:
        set_tuning(monkeypatch, MXD_MSDA_TILE_TARGET=1000000)
    nl = int(rng.integers(1, 4))
    levels = [(int(rng.integers(3, 40)), int(rng.integers(3, 40))) for _ in range(nl)]
    shapes, lsi = workloads.level_tensors(levels)
    nk = int(shapes.prod(1).sum())
    bs, nq, nh = int(rng.integers(1, 3)), int(rng.integers(2500, 7000)), int(rng.integers(1, 4))
    hd = int(rng.choice([8, 20, 32, 48, 64]))
    npts = int(rng.integers(2, 7))
    dtype = torch.float16 if seed in (2, 5) else torch.float32
    g = torch.Generator().manual_seed(200 + seed)
    loc = torch.rand(bs, nq, nh, nl, npts, 2, generator=g) * 1.2 - 0.1
    nspots = int(rng.integers(1, 6))
    spots = torch.rand(nspots, 2, generator=g) * 1.04 - 0.02
    pick = torch.randint(0, int(nspots / float(rng.uniform(0.2, 0.8))) + 1, loc.shape[:-1], generator=g)
    for k in range(nspots):
        loc[pick == k] = spots[k]
    inp = workloads.MsdaInputs(torch.randn(bs, nk, nh, hd, generator=g), shapes, lsi, loc,
                               torch.rand(bs, nq, nh, nl, npts, generator=g), torch.randn(bs, nq, nh * hd, generator=g))
    if dtype == torch.float16:
        inp = workloads.MsdaInputs(*[t.half() if t.is_floating_point() else t for t in inp])
        errs = _check_all(inp, gpu_device, HALF, HALF)
    else:
        errs = _check_all(inp, gpu_device, FWD_FP32, BWD_FP32)
    print(seed, levels, (bs, nq, nh, hd, npts), dtype, errs)


@pytest.mark.parametrize("rec_lds", [0, 1], ids=["records-one-by-one", "slab-in-LDS"])
@pytest.mark.parametrize("log2", [8, 7], ids=["tiles-of-256", "tiles-of-128"])
@pytest.mark.parametrize("seed", range(6))
def test_finer_tiles_of_the_grad_value_pass(gpu_device, monkeypatch, seed, log2, rec_lds):
    """The tile pass keeps 32 sums per thread: 512 pixels x 32 channels per workgroup, 256 x 64 or 128 x 128 (one pass
    over the records for heads of up to 64 / 128 channels, two for more).  The launcher picks the tile size from
    head_dim and the size of the maps; here both finer sizes are forced on random problems of every head size that is
    a multiple of four (more sums than channels, exactly as many, two passes), with samples piled on a few spots, tiles
    split into query chunks or not, float32 and 16-bit storage, and the first kernel's workgroups either storing their
    records one by one or collecting their slab in LDS."""
    rng = np.random.default_rng(7000 + seed)
    env = {"MXD_MSDA_TILE_PX_LOG2": log2, "MXD_MSDA_BWD_REC_LDS": rec_lds}
    if seed % 2:
        env["MXD_MSDA_TILE_TARGET"] = 1000000
    set_tuning(monkeypatch, **env)
    nl = int(rng.integers(1, 4))
    levels = [(int(rng.integers(6, 60)), int(rng.integers(6, 60))) for _ in range(nl)]
    shapes, lsi = workloads.level_tensors(levels)
    nk = int(shapes.prod(1).sum())
    bs, nq, nh = int(rng.integers(1, 3)), int(rng.integers(1500, 5000)), int(rng.integers(1, 4))
    hd = int(rng.choice([4, 20, 32, 48, 64, 100, 128, 200, 256]))
    npts = int(rng.integers(1, 7))
    dtype = (torch.float32, torch.float16, torch.bfloat16)[seed % 3]
    g = torch.Generator().manual_seed(7100 + seed)
    loc = torch.rand(bs, nq, nh, nl, npts, 2, generator=g) * 1.2 - 0.1
    nspots = int(rng.integers(1, 5))
    spots = torch.rand(nspots, 2, generator=g) * 1.04 - 0.02
    pick = torch.randint(0, 3 * nspots + 1, loc.shape[:-1], generator=g)
    for k in range(nspots):
        loc[pick == k] = spots[k]
    inp = workloads.MsdaInputs(torch.randn(bs, nk, nh, hd, generator=g), shapes, lsi, loc,
                               torch.rand(bs, nq, nh, nl, npts, generator=g), torch.randn(bs, nq, nh * hd, generator=g))
    print("case", seed, levels, (bs, nq, nh, hd, npts), dtype, env, flush=True)
    if dtype == torch.float32:
        _check_all(inp, gpu_device, FWD_FP32, BWD_FP32)
    else:
        inp = workloads.MsdaInputs(*[t.to(dtype) if t.is_floating_point() else t for t in inp])
        _check_all(inp, gpu_device, half_tol(dtype), half_tol(dtype))


def _random_case(seed):
    """A random small problem: odd sizes everywhere, locations reaching outside the image."""
    rng = np.random.default_rng(seed)
    bs, nq, nh = int(rng.integers(1, 4)), int(rng.integers(1, 700)), int(rng.integers(1, 10))
    hd = int(rng.choice([1, 2, 3, 4, 6, 8, 12, 16, 20, 24, 32, 40, 48, 64, 96, 128, 256]))
    nl, npts = int(rng.integers(1, 6)), int(rng.integers(1, 10))
    levels = [(int(rng.integers(1, 48)), int(rng.integers(1, 48))) for _ in range(nl)]
    shapes, lsi = workloads.level_tensors(levels)
    nk = int(shapes.prod(1).sum())
    g = torch.Generator().manual_seed(seed)
    value = torch.randn(bs, nk, nh, hd, generator=g)
    loc = torch.rand(bs, nq, nh, nl, npts, 2, generator=g) * 1.3 - 0.15
    attn = torch.rand(bs, nq, nh, nl, npts, generator=g)
    grad_out = torch.randn(bs, nq, nh * hd, generator=g)
    return workloads.MsdaInputs(value, shapes, lsi, loc, attn, grad_out), (bs, nq, nh, hd, levels, npts)


@pytest.mark.parametrize("seed", range(24))
def test_random_small_problems(gpu_device, seed):
    inp, desc = _random_case(1000 + seed)
    print("case", desc, flush=True)
    _check_all(inp, gpu_device, FWD_FP32, BWD_FP32)


@pytest.mark.parametrize("seed", range(12))
def test_random_small_problems_16bit(gpu_device, seed):
    """The same kind of problem in float16 (even seeds) and bfloat16 (odd seeds): the float64 oracle runs on the
    rounded inputs; the results are rounded once more, which for bfloat16 is up to 2^-8 of the largest element."""
    dtype = torch.float16 if seed % 2 == 0 else torch.bfloat16
    inp, desc = _random_case(2000 + seed)
    inp = workloads.MsdaInputs(inp.value.to(dtype), inp.spatial_shapes, inp.level_start_index,
                               inp.sampling_locations.to(dtype), inp.attention_weights.to(dtype),
                               inp.grad_output.to(dtype))
    print("case", desc, dtype, flush=True)
    tol = half_tol(dtype)
    ref = oracle_all(inp)
    got = run_gpu(inp, gpu_device)
    # 16-bit locations sit on cell edges far more often than float32 ones: the location gradient is compared away
    # from them only (the oracle and the kernel may take either side of an edge)
    lo = inp.sampling_locations.double()
    near = torch.zeros(lo.shape[:-1], dtype=torch.bool)
    for lvl, (h, w) in enumerate(inp.spatial_shapes.tolist()):
        w_im, h_im = lo[:, :, :, lvl, :, 0] * w - 0.5, lo[:, :, :, lvl, :, 1] * h - 0.5
        near[:, :, :, lvl] = ((w_im - w_im.round()).abs() < 2.0 ** -12) | ((h_im - h_im.round()).abs() < 2.0 ** -12)
    keep = (~near)[..., None].numpy()
    for name, g_, r_ in zip(("output", "grad_value", "grad_sampling_locations", "grad_attention_weights"), got, ref):
        r_ = np.asarray(r_)
        if name == "grad_sampling_locations":
            g_, r_ = g_ * keep, r_ * keep
        assert rel_err(g_, r_) <= tol, (name, rel_err(g_, r_), desc)
        # element by element: within one unit in the last place of the oracle rounded to the storage type
        groups = None if name == "output" else level_slices(inp, "keys" if name == "grad_value" else "samples")
        check_16bit(g_, r_, dtype, name, groups, tol32=FWD_FP32 if name == "output" else BWD_FP32)


@pytest.mark.parametrize("name,dtype", [("detr_encoder", torch.float32), ("detr_encoder", torch.float16),
                                        ("detr_encoder", torch.bfloat16), ("bevformer_sca", torch.float32),
                                        ("bevformer_sca", torch.float16), ("head_dim_128", torch.float16),
                                        ("head_dim_128", torch.bfloat16)])
def test_forward_cu_form_equals_the_general_form_at_full_size(gpu_device, monkeypatch, name, dtype):
    """The forward's one-workgroup-per-CU form (last levels in LDS, sample values handed across lanes by DPP; rows of 8,
    4 and 16 lanes here) at the benchmark shapes: the encoder shape takes it by default, the others are made to.  With
    every wavefront working through its chunks in the same order (MXD_MSDA_FWD_CU_FLIP=0) its sums run in the order of
    the general kernel's, so at full size the two must agree bit for bit; the general kernel is checked against the
    oracle at these sizes elsewhere."""
    from drivingsdk_amd import _C
    d = to_device(workloads.make_inputs(name, dtype=dtype), gpu_device)
    args = (d.value, d.spatial_shapes, d.level_start_index, d.sampling_locations, d.attention_weights)
    dims = (*d.value.shape, d.spatial_shapes.shape[0], d.spatial_shapes.shape[0], d.sampling_locations.shape[1],
            d.sampling_locations.shape[4])
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    if name == "detr_encoder":
        assert _lib.make_plan(0, code, *dims).block == 1024, "the encoder shape is meant to take this form by default"
    set_tuning(monkeypatch, MXD_MSDA_FWD_CU=1, MXD_MSDA_FWD_CU_FLIP=0)
    assert _lib.make_plan(0, code, *dims).block == 1024
    out_cu = _C.multi_scale_deformable_attn(*args)
    set_tuning(monkeypatch, MXD_MSDA_FWD_CU=1, MXD_MSDA_FWD_CU_FLIP=1)
    out_flipped = _C.multi_scale_deformable_attn(*args)
    set_tuning(monkeypatch, MXD_MSDA_FWD_CU=0)
    assert _lib.make_plan(0, code, *dims).block != 1024
    out_general = _C.multi_scale_deformable_attn(*args)
    assert torch.equal(out_cu, out_general)
    # Half of the wavefronts of the default build work through a chunk from its LDS groups on (MXD_MSDA_FWD_CU_FLIP=1):
    # their units' sums are formed in another order, so they agree to rounding, not bit for bit
    if dtype == torch.float32:
        check_close(out_flipped.double().cpu().numpy(), out_general.double().cpu().numpy(), FWD_FP32, "output, flipped order")
    else:
        check_16bit(out_flipped.double().cpu().numpy(), out_general.double().cpu().numpy(), dtype, "output, flipped order",
                    tol32=FWD_FP32)


@pytest.mark.parametrize("seed", range(24))
def test_random_small_problems_cu_form(gpu_device, monkeypatch, seed):
    """Random small problems forced through the one-workgroup-per-CU forward wherever it can run (16-byte lanes, rows
    of at most 16 lanes): odd point counts (the sample-by-sample path), level lists that end inside a chunk, levels
    that do and do not fit the LDS, float32 and 16-bit storage; against the oracle."""
    set_tuning(monkeypatch, MXD_MSDA_FWD_CU=1, MXD_MSDA_FWD_CU_WGS=1 + seed % 5)
    rng = np.random.default_rng(3000 + seed)
    dtype = (torch.float32, torch.float16, torch.bfloat16)[seed % 3]
    es = 4 if dtype == torch.float32 else 2
    bs, nq, nh = int(rng.integers(1, 4)), int(rng.integers(1, 900)), int(rng.integers(1, 10))
    hd = int(rng.choice([4, 8, 12, 16, 24, 32, 48, 64])) * (16 // es) // 4   # rows of 16 .. 256 bytes, multiples of 16
    nl, npts = int(rng.integers(1, 6)), int(rng.integers(1, 10))
    big = seed % 4 == 0   # a first level that cannot fit the LDS (1 350 rows of up to 256 bytes ...), small ones behind it
    levels = [(int(rng.integers(1, 48)), int(rng.integers(1, 48))) for _ in range(nl)]
    if big:
        levels[0] = (90, 150)
    shapes, lsi = workloads.level_tensors(levels)
    nk = int(shapes.prod(1).sum())
    g = torch.Generator().manual_seed(3000 + seed)
    inp = workloads.MsdaInputs(torch.randn(bs, nk, nh, hd, generator=g).to(dtype), shapes, lsi,
                               (torch.rand(bs, nq, nh, nl, npts, 2, generator=g) * 1.3 - 0.15).to(dtype),
                               torch.rand(bs, nq, nh, nl, npts, generator=g).to(dtype), None)
    print("case", (bs, nq, nh, hd, levels, npts), dtype, flush=True)
    want = oracle_all(inp, with_grads=False)[0]
    got = run_gpu(inp, gpu_device, with_grads=False)[0]
    tol = FWD_FP32 if dtype == torch.float32 else half_tol(dtype)
    assert rel_err(got, want) <= tol
    if dtype == torch.float32:
        check_close(got, want, FWD_FP32, "output")
    else:
        check_16bit(got, want, dtype, "output", tol32=FWD_FP32)
    with monkeypatch.context() as m:
        set_tuning(m, MXD_MSDA_FWD_CU=0)
        general = run_gpu(inp, gpu_device, with_grads=False)[0]
    with monkeypatch.context() as m:
        set_tuning(m, MXD_MSDA_FWD_CU=1, MXD_MSDA_FWD_CU_WGS=1 + seed % 5, MXD_MSDA_FWD_CU_FLIP=0)
        unflipped = run_gpu(inp, gpu_device, with_grads=False)[0]
    # (the same order of summation in every wavefront: bit for bit the general kernel's result)
    assert np.array_equal(np.asarray(unflipped), np.asarray(general))


def test_backward_with_more_tiles_than_the_lds_bookkeeping_holds(gpu_device):
    """One level of 2.09 M pixels and 32-byte rows (a 1080x1920 grid-sampler-like input): the per-tile counters of the
    first backward kernel would not fit the LDS next to 16 units' staging strips, so the launcher takes the
    one-kernel form with global atomics.  Gradients against the oracle."""
    g = torch.Generator().manual_seed(2090)
    levels = ((1100, 1900),)
    shapes, lsi = workloads.level_tensors(levels)
    nk = 1100 * 1900
    bs, nq, nh, hd, npts = 1, 2000, 1, 8, 4
    plan = _lib.make_plan(1, 0, bs, nk, nh, hd, 1, 1, nq, npts)
    assert plan.units_per_wave == 16
    assert plan.lds_bytes <= 64 * 1024 and plan.iters == 1      # (the atomic form: one iteration per wavefront)
    assert _lib.load().mxd_msda_backward_workspace_bytes(0, bs, nk, nh, hd, 1, 1, nq, npts) == 0
    inp = workloads.MsdaInputs(torch.randn(bs, nk, nh, hd, generator=g), shapes, lsi,
                               torch.rand(bs, nq, nh, 1, npts, 2, generator=g) * 1.02 - 0.01,
                               torch.rand(bs, nq, nh, 1, npts, generator=g), torch.randn(bs, nq, nh * hd, generator=g))
    print(_check_all(inp, gpu_device, FWD_FP32, BWD_FP32))


_LAYOUTS = {
    # name: (level shapes, level_start_index, num_keys)
    "keys_behind_the_last_level": (((40, 30), (20, 15)), (0, 1200), 1200 + 300 + 777),
    "gap_between_levels": (((40, 30), (20, 15)), (0, 1500), 1800 + 50),
    "descending_starts": (((40, 30), (20, 15)), (300, 0), 1500),
    "overlapping_levels": (((40, 30), (20, 15)), (0, 1000), 1300),
    "first_level_does_not_start_at_zero": (((40, 30), (20, 15)), (600, 1800), 2100),
}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("layout", sorted(_LAYOUTS))
@pytest.mark.parametrize("cu", ["0", "1"])
def test_level_start_indices_that_do_not_tile_the_keys(gpu_device, monkeypatch, layout, dtype, cu):
    """level_start_index is the caller's: the reference's kernels index value with it as given and add gradients with
    atomics, so levels may leave keys uncovered, come in any order or overlap (kernels/multi_scale_deformable_attn/
    op_kernel/multi_scale_deformable_attn_grad.cpp:181-186).  Rows of grad_value that no level covers are exactly zero."""
    # (the forward's form makes no difference to the backward: its runs also take the finest tiles of the grad_value pass)
    set_tuning(monkeypatch, MXD_MSDA_FWD_CU=cu, MXD_MSDA_TILE_PX_LOG2=7 if cu == "1" else 9)
    levels, starts, nk = _LAYOUTS[layout]
    shapes = torch.tensor(levels, dtype=torch.int64)
    lsi = torch.tensor(starts, dtype=torch.int64)
    bs, nq, nh, hd, npts = 2, 3100, 3, 32, 4
    g = torch.Generator().manual_seed(len(layout))
    inp = workloads.MsdaInputs(torch.randn(bs, nk, nh, hd, generator=g).to(dtype), shapes, lsi,
                               (torch.rand(bs, nq, nh, 2, npts, 2, generator=g) * 1.1 - 0.05).to(dtype),
                               torch.rand(bs, nq, nh, 2, npts, generator=g).to(dtype),
                               torch.randn(bs, nq, nh * hd, generator=g).to(dtype))
    ref = oracle_all(inp)
    got = run_gpu(inp, gpu_device)
    tol_f, tol_b = (FWD_FP32, BWD_FP32) if dtype == torch.float32 else (HALF, HALF)
    for name, g_, r_, tol in zip(("output", "grad_value", "grad_sampling_locations", "grad_attention_weights"), got, ref,
                                 (tol_f, tol_b, tol_b, tol_b)):
        if name == "grad_sampling_locations":
            keep = ~_cell_edge_mask(inp)[..., None]
            g_, r_ = g_ * keep, np.asarray(r_) * keep
        assert rel_err(g_, r_) <= tol, (name, rel_err(g_, r_))
    covered = np.zeros(nk, dtype=bool)
    for (h, w), s in zip(levels, starts):
        covered[s:s + h * w] = True
    assert not np.any(got[1][:, ~covered]), "rows of grad_value outside every level must be exactly zero"


@pytest.mark.parametrize("flags", [0, 2], ids=["default", "MXD_BWD_ANY_LAYOUT"])
def test_levels_that_overlap_beyond_the_run_table(gpu_device, flags):
    """Four levels that overlap so far that they have 17 tiles of 512 pixels between them while value has 3 422 keys
    (room for 10 in the run table).  By default the levels without room are added to grad_value sample by sample by
    workgroups of the tile pass set aside for that; with MXD_BWD_ANY_LAYOUT the backward takes the one-kernel form with
    global atomics.  Either way level_start_index is taken as it comes, as the reference's kernel takes it."""
    levels, starts, nk = ((56, 48), (10, 20), (58, 55), (58, 18)), (504, 1119, 148, 352), 3422
    bs, nq, nh, hd, npts = 2, 300, 4, 32, 5
    g = torch.Generator().manual_seed(77)
    inp = workloads.MsdaInputs(torch.randn(bs, nk, nh, hd, generator=g), torch.tensor(levels), torch.tensor(starts),
                               torch.rand(bs, nq, nh, 4, npts, 2, generator=g) * 1.2 - 0.1,
                               torch.rand(bs, nq, nh, 4, npts, generator=g), torch.randn(bs, nq, nh * hd, generator=g))
    ref = oracle_all(inp)
    d = to_device(inp, gpu_device)
    gv = torch.empty_like(d.value)
    gl, ga = _backward_c_abi(d, flags, gv)
    keep = ~_cell_edge_mask(inp)[..., None]
    assert rel_err(gv.double().cpu().numpy(), ref[1]) <= BWD_FP32
    assert rel_err(gl.double().cpu().numpy() * keep, np.asarray(ref[2]) * keep) <= BWD_FP32
    assert rel_err(ga.double().cpu().numpy(), ref[3]) <= BWD_FP32
