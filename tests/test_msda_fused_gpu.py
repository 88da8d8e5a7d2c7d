"""Fused form (softmax + sampling-location arithmetic inside the forward kernel) against the CPU oracle.
Tolerances as for the plain operator: forward 1e-5, gradients 1e-4 (float32), 2e-3 for 16-bit types."""
import numpy as np
import pytest
import torch

import drivingsdk_amd
from drivingsdk_amd import _lib, workloads
from drivingsdk_amd.ops import msda_fused
from oracle import msda_oracle as orc
from util import BF16, BWD_FP32, FWD_FP32, HALF, rel_err, set_tuning

pytestmark = pytest.mark.gpu


def make_fused_inputs(name, ref_dim=2, scale_queries=1.0, seed=77, dtype=torch.float32):
    """Module-style inputs on the pyramid of a named workload: reference points in [0,1), offsets of a few
    pixels, Gaussian logits."""
    cfg = workloads.WORKLOADS[name]
    shapes, lsi = workloads.level_tensors(cfg["levels"])
    g = torch.Generator().manual_seed(seed)
    nk = int(shapes.prod(1).sum())
    bs, nh, hd, npts, nl = cfg["bs"], cfg["nh"], cfg["hd"], cfg["np"], shapes.shape[0]
    nq = max(1, int(round((cfg["nq"] or nk) * scale_queries)))
    value = torch.randn(bs, nk, nh, hd, generator=g)
    ref = torch.rand(bs, nq, nl, ref_dim, generator=g)
    if ref_dim == 4:
        ref[..., 2:] = ref[..., 2:] * 0.3 + 0.05
    off = torch.randn(bs, nq, nh, nl, npts, 2, generator=g) * (3.0 if ref_dim == 2 else 1.5)
    logits = torch.randn(bs, nq, nh, nl * npts, generator=g) * 2.0
    grad_out = torch.randn(bs, nq, nh * hd, generator=g)
    return [t.to(dtype) for t in (value,)] + [shapes, lsi] + [t.to(dtype) for t in (ref, off, logits, grad_out)]


def _edge_masks(shapes, ref, off, logits):
    """Samples whose float32 location lies within 2^-20 px of (not on) a cell edge -- the location gradient
    jumps there -- or exactly on pixel coordinate -1, and the reference points that own such a sample."""
    loc = orc.fused_sampling_inputs(shapes, ref.float(), off.float(), logits.float())[0].double()
    near = torch.zeros(loc.shape[:-1], dtype=torch.bool)
    for lvl, (h, w) in enumerate(shapes.tolist()):
        w_im = loc[:, :, :, lvl, :, 0] * w - 0.5
        h_im = loc[:, :, :, lvl, :, 1] * h - 0.5
        dw, dh = (w_im - w_im.round()).abs(), (h_im - h_im.round()).abs()
        near[:, :, :, lvl] = ((dw > 0) & (dw < 2.0 ** -20)) | ((dh > 0) & (dh < 2.0 ** -20))
        # a pixel coordinate of exactly -1 (16-bit inputs reach it): the operator drops the sample, as the
        # reference's kernels do, where grid_sample still reports a location gradient from the weight-0 corner
        near[:, :, :, lvl] |= (w_im == -1.0) | (h_im == -1.0)
    ref_near = near.any(dim=4).any(dim=2)                     # [bs, nq, nl]
    return near.numpy(), ref_near.numpy()


def _compare(got, want, shapes, ref, off, logits, tols):
    near, ref_near = _edge_masks(shapes, ref, off, logits)
    assert near.mean() < 1e-3
    keep = {"grad_reference_points": ~ref_near[..., None], "grad_sampling_offsets": ~near[..., None]}
    names = ("output", "grad_value", "grad_reference_points", "grad_sampling_offsets", "grad_attention_logits")
    errs = {}
    for n, g_, w_, tol in zip(names, got, want, tols):
        w_ = w_.numpy()
        if n in keep:
            g_, w_ = g_ * keep[n], w_ * keep[n]
        errs[n] = rel_err(g_, w_)
        assert errs[n] <= tol, (n, errs)
    return errs


def _run(value, shapes, lsi, ref, off, logits, grad_out, device):
    v = value.to(device).requires_grad_()
    r = ref.to(device).requires_grad_()
    o = off.to(device).requires_grad_()
    z = logits.to(device).requires_grad_()
    out = drivingsdk_amd.multi_scale_deformable_attn_fused(v, shapes.to(device), lsi.to(device), r, o, z)
    out.backward(grad_out.to(device))
    return [t.detach().double().cpu().numpy() for t in (out, v.grad, r.grad, o.grad, z.grad)]


@pytest.mark.parametrize("fixed", ["1", "0"], ids=["geometry-as-constants", "general-first-kernel"])
@pytest.mark.parametrize("name,ref_dim,scale", [("tiny", 2, 1.0), ("tiny", 4, 1.0), ("detr_encoder", 2, 0.25),
                                                ("bevformer_sca", 2, 0.1)])
def test_fused_forward_and_gradients_fp32(gpu_device, monkeypatch, name, ref_dim, scale, fixed):
    """(The backward's first kernel has an instantiation with the launch geometry of up to 16 samples per query as
    constants, which the tiny and encoder shapes take by default; MXD_MSDA_BWD_FIXED=0 sends them through the general one.)"""
    set_tuning(monkeypatch, MXD_MSDA_BWD_FIXED=fixed)
    inp = make_fused_inputs(name, ref_dim, scale)
    value, shapes, lsi, ref, off, logits, grad_out = inp
    want = orc.fused_fwd_bwd(value, shapes, ref, off, logits, grad_out, loc_dtype=torch.float32)
    got = _run(*inp, gpu_device)
    print(name, ref_dim, _compare(got, want, shapes, ref, off, logits, (FWD_FP32,) + (BWD_FP32,) * 4))


def test_fused_forward_equals_the_unfused_composition(gpu_device):
    """Same inputs through torch's softmax / location arithmetic and the plain operator."""
    inp = make_fused_inputs("detr_encoder", 2, 0.25)
    value, shapes, lsi, ref, off, logits, _ = [t.to(gpu_device) for t in inp]
    fused = drivingsdk_amd.multi_scale_deformable_attn_fused(value, shapes, lsi, ref, off, logits)
    loc, attn = msda_fused.sampling_inputs(shapes, ref, off, logits)
    plain = drivingsdk_amd.multi_scale_deformable_attn(value, shapes, lsi, loc, attn)
    assert rel_err(fused.double().cpu().numpy(), plain.double().cpu().numpy()) <= FWD_FP32


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_forward_16bit(gpu_device, dtype):
    inp = make_fused_inputs("tiny", 2, 1.0, dtype=dtype)
    value, shapes, lsi, ref, off, logits, _ = inp
    want = orc.fused_fwd_bwd(value, shapes, ref, off, logits)[0]     # float64 on the rounded inputs
    out = drivingsdk_amd.multi_scale_deformable_attn_fused(*[t.to(gpu_device) for t in inp[:6]])
    assert out.dtype == dtype
    # one rounding of the float32 result to the 16-bit type: float16 within the 16-bit tolerance; a bfloat16
    # half-ulp is up to 2^-8 of the element itself, which for the largest element is all of this error measure
    tol = HALF if dtype == torch.float16 else 2.0 ** -8
    assert rel_err(out.double().cpu().numpy(), want.numpy()) <= tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("hd,nl,npts,nq", [(32, 4, 4, 1237), (32, 3, 5, 640), (16, 2, 8, 333), (64, 4, 2, 1001),
                                           (8, 1, 13, 517), (128, 4, 4, 259)])
def test_fused_forward_one_workgroup_per_cu_form(gpu_device, monkeypatch, hd, nl, npts, nq, dtype):
    """The fused forward in the form that large problems take (one workgroup per CU, coarse levels in LDS, the softmax
    formed by the unit's lanes), forced on small problems: rows of 4, 8 and 16 lanes, sample counts that are not a
    multiple of four (the sample-by-sample loop), a last group of queries that is partly filled.  Against the oracle,
    and against the general kernel's fused form (same arithmetic but for the order of the softmax sum)."""
    g = torch.Generator().manual_seed(1000 + hd + npts)
    shapes, lsi = workloads.level_tensors(((23, 31), (12, 16), (6, 8), (3, 4))[:nl])
    nk = int(shapes.prod(1).sum())
    bs, nh = 2, 3
    value = torch.randn(bs, nk, nh, hd, generator=g).to(dtype)
    ref = torch.rand(bs, nq, nl, 2, generator=g).to(dtype)
    off = (torch.randn(bs, nq, nh, nl, npts, 2, generator=g) * 2).to(dtype)
    logits = (torch.randn(bs, nq, nh, nl * npts, generator=g) * 2).to(dtype)
    want = orc.fused_fwd_bwd(value, shapes, ref, off, logits, loc_dtype=torch.float32)[0].numpy()
    args = [t.to(gpu_device) for t in (value, shapes, lsi, ref, off, logits)]
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    outs = {}
    for mode in ("1", "0"):
        set_tuning(monkeypatch, MXD_MSDA_FWD_CU=mode)
        outs[mode] = drivingsdk_amd.multi_scale_deformable_attn_fused(*args).double().cpu().numpy()
    # (the plan of the plain operator with the same sizes says which lane layout the forced form runs with)
    set_tuning(monkeypatch, MXD_MSDA_FWD_CU="1")
    eligible = hd * value.element_size() <= 256   # (rows of at most 16 lanes of 16 bytes)
    assert (_lib.make_plan(0, code, bs, nk, nh, hd, nl, nl, nq, npts).block == 1024) == eligible
    tol = FWD_FP32 if dtype == torch.float32 else HALF if dtype == torch.float16 else BF16
    assert rel_err(outs["1"], want) <= tol
    assert rel_err(outs["1"], outs["0"]) <= (2e-6 if dtype == torch.float32 else tol)


def test_fused_more_than_16_samples_per_unit_and_many_heads(gpu_device):
    """nl*np = 32 (two staging chunks, strided softmax statistics), head_dim 16 (16 units per wavefront)."""
    g = torch.Generator().manual_seed(5)
    shapes, lsi = workloads.level_tensors(((20, 30), (10, 15), (5, 8), (3, 4)))
    nk = int(shapes.prod(1).sum())
    bs, nq, nh, hd, nl, npts = 2, 333, 5, 16, 4, 8
    value = torch.randn(bs, nk, nh, hd, generator=g)
    ref = torch.rand(bs, nq, nl, 2, generator=g)
    off = torch.randn(bs, nq, nh, nl, npts, 2, generator=g) * 2
    logits = torch.randn(bs, nq, nh, nl * npts, generator=g) * 3
    grad_out = torch.randn(bs, nq, nh * hd, generator=g)
    want = orc.fused_fwd_bwd(value, shapes, ref, off, logits, grad_out, loc_dtype=torch.float32)
    got = _run(value, shapes, lsi, ref, off, logits, grad_out, gpu_device)
    _compare(got, want, shapes, ref, off, logits, (FWD_FP32,) + (BWD_FP32,) * 4)


@pytest.mark.parametrize("npts,nl,ref_dim", [(3, 3, 2), (3, 2, 4), (32, 2, 2), (1, 5, 4)])
def test_fused_gradients_other_point_counts(gpu_device, npts, nl, ref_dim):
    """Point counts that are not a power of two, or exceed one staging chunk: the reference points' gradient is
    then added up with atomics instead of across lanes."""
    g = torch.Generator().manual_seed(100 + npts)
    shapes, lsi = workloads.level_tensors(((12, 17), (6, 9), (3, 5), (2, 3), (1, 2))[:nl])
    nk = int(shapes.prod(1).sum())
    bs, nq, nh, hd = 2, 157, 3, 32
    value = torch.randn(bs, nk, nh, hd, generator=g)
    ref = torch.rand(bs, nq, nl, ref_dim, generator=g)
    if ref_dim == 4:
        ref[..., 2:] = ref[..., 2:] * 0.3 + 0.05
    off = torch.randn(bs, nq, nh, nl, npts, 2, generator=g) * 2
    logits = torch.randn(bs, nq, nh, nl * npts, generator=g) * 2
    grad_out = torch.randn(bs, nq, nh * hd, generator=g)
    want = orc.fused_fwd_bwd(value, shapes, ref, off, logits, grad_out, loc_dtype=torch.float32)
    got = _run(value, shapes, lsi, ref, off, logits, grad_out, gpu_device)
    _compare(got, want, shapes, ref, off, logits, (FWD_FP32,) + (BWD_FP32,) * 4)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("ref_dim", [2, 4])
def test_fused_gradients_16bit(gpu_device, dtype, ref_dim):
    """Gradients in 16-bit storage: float64 oracle on the rounded inputs, locations formed in float32 as the
    kernel forms them.  bfloat16 results carry one rounding of up to 2^-9 relative, which the error measure
    (largest error over largest element) can see in full."""
    inp = make_fused_inputs("tiny", ref_dim, 1.0, dtype=dtype)
    value, shapes, lsi, ref, off, logits, grad_out = inp
    want = orc.fused_fwd_bwd(value.double(), shapes, ref.double(), off.double(), logits.double(), grad_out.double(),
                             loc_dtype=torch.float32)
    got = _run(*inp, gpu_device)
    tol = HALF if dtype == torch.float16 else 2.0 ** -8
    # the logits' gradient takes the softmax backward's sum from the stored (rounded) forward result and is
    # rounded itself: two roundings
    _compare(got, want, shapes, ref, off, logits, (tol,) * 4 + (2 * tol,))


def test_fused_backward_without_reference_point_gradient(gpu_device):
    """Reference points that need no gradient: the per-head partial sums and their reduction are skipped and
    the other gradients are unchanged."""
    inp = make_fused_inputs("tiny", 2, 1.0)
    value, shapes, lsi, ref, off, logits, grad_out = inp
    full = _run(*inp, gpu_device)
    v = value.to(gpu_device).requires_grad_()
    o = off.to(gpu_device).requires_grad_()
    z = logits.to(gpu_device).requires_grad_()
    out = drivingsdk_amd.multi_scale_deformable_attn_fused(v, shapes.to(gpu_device), lsi.to(gpu_device),
                                                           ref.to(gpu_device), o, z)
    out.backward(grad_out.to(gpu_device))
    for got, want in zip((out, o.grad, z.grad), (full[0], full[3], full[4])):
        np.testing.assert_array_equal(got.detach().double().cpu().numpy(), want)
    # (grad_value is summed in an order that varies from run to run)
    assert rel_err(v.grad.double().cpu().numpy(), full[1]) <= 1e-6
    lib = _lib.load()
    with_ref = lib.mxd_msda_fused_backward_workspace_bytes(0, 1, 1360, 8, 32, 4, 1360, 4, 2, 1)
    without = lib.mxd_msda_fused_backward_workspace_bytes(0, 1, 1360, 8, 32, 4, 1360, 4, 2, 0)
    assert with_ref - without == 8 * 1360 * 4 * 2 * 4


def test_fused_error_paths(gpu_device):
    inp = make_fused_inputs("tiny", 2, 0.05)
    value, shapes, lsi, ref, off, logits, _ = [t.to(gpu_device) for t in inp]
    with pytest.raises(RuntimeError, match="must be 2 or 4"):
        drivingsdk_amd.multi_scale_deformable_attn_fused(value, shapes, lsi, ref[..., :1].repeat(1, 1, 1, 3), off, logits)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        drivingsdk_amd.multi_scale_deformable_attn_fused(value.cpu(), shapes.cpu(), lsi.cpu(), ref.cpu(), off.cpu(),
                                                         logits.cpu())
    lib = _lib.load()
    assert lib.mxd_msda_fused_forward(None, None, None, None, 2, None, None, None, 0, 1, 10, 1, 8, 1, 1, 1, None) == -3
    assert lib.mxd_msda_fused_backward(*([None] * 4), 2, *([None] * 9), 0, 0, 1, 10, 1, 8, 1, 1, 1, 0, None) == -3
    assert lib.mxd_msda_fused_backward_workspace_bytes(0, 1, 10, 1, 8, 1, 1, 1, 3, 1) == 0
