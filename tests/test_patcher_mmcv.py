"""mmcv patch of the operator, tested with fake mmcv modules as the reference does
(tests/patcher/test_patcher_mmcv.py:85-142 of the reference: class attributes, two AtomicPatches,
target paths, replacement wrappers), plus the behaviour of the wrappers themselves."""
import sys
import types

import numpy as np
import pytest
import torch

import mx_driving
from mx_driving.patcher import APPLIED, SKIPPED, AtomicPatch, MultiScaleDeformableAttention, apply_patches

BASE = "mmcv.ops.multi_scale_deform_attn.MultiScaleDeformableAttnFunction"


@pytest.fixture
def fake_mmcv(monkeypatch):
    """mmcv.ops.multi_scale_deform_attn with a Function that must never run once patched."""
    class MultiScaleDeformableAttnFunction(torch.autograd.Function):
        @staticmethod
        def forward(ctx, value, value_spatial_shapes, value_level_start_index, sampling_locations,
                    attention_weights, im2col_step):
            raise AssertionError("unpatched mmcv forward was called")

        @staticmethod
        def backward(ctx, grad_output):
            raise AssertionError("unpatched mmcv backward was called")

    mmcv = types.ModuleType("mmcv")
    ops = types.ModuleType("mmcv.ops")
    msda = types.ModuleType("mmcv.ops.multi_scale_deform_attn")
    msda.MultiScaleDeformableAttnFunction = MultiScaleDeformableAttnFunction
    mmcv.ops, ops.multi_scale_deform_attn = ops, msda
    for name, mod in (("mmcv", mmcv), ("mmcv.ops", ops), ("mmcv.ops.multi_scale_deform_attn", msda)):
        monkeypatch.setitem(sys.modules, name, mod)
    return msda


def test_patch_class_attributes():
    assert MultiScaleDeformableAttention.name == "multi_scale_deformable_attention"
    assert MultiScaleDeformableAttention.legacy_name == "msda"
    assert MultiScaleDeformableAttention.target_module == "mmcv"
    assert not hasattr(MultiScaleDeformableAttention, "precheck")


def test_patches_are_two_atomic_patches_with_wrappers():
    patches = MultiScaleDeformableAttention.patches()
    assert isinstance(patches, list) and len(patches) == 2
    assert all(isinstance(p, AtomicPatch) for p in patches)
    assert sorted(p.target for p in patches) == [BASE + ".backward", BASE + ".forward"]
    assert all(p._replacement_wrapper is not None for p in patches)


def test_skipped_without_mmcv():
    import importlib.util
    if importlib.util.find_spec("mmcv") is not None:
        pytest.skip("a real mmcv is installed")
    results = apply_patches(MultiScaleDeformableAttention.patches())
    # mmcv is not installed in this environment: nothing to patch, no exception
    assert [s for _, s in results] == [SKIPPED, SKIPPED]


def test_wrappers_adapt_the_calling_convention(fake_mmcv, monkeypatch):
    calls = {}

    def our_forward(ctx, value, shapes, lsi, loc, attn):
        calls["forward"] = (value, shapes, lsi, loc, attn)
        return "out"

    def our_backward(ctx, grad_output):
        calls["backward"] = grad_output
        return ("gv", None, None, "gl", "ga")

    monkeypatch.setattr(mx_driving.MultiScaleDeformableAttnFunction, "forward", staticmethod(our_forward))
    monkeypatch.setattr(mx_driving.MultiScaleDeformableAttnFunction, "backward", staticmethod(our_backward))
    patches = MultiScaleDeformableAttention.patches()
    assert [s for _, s in apply_patches(patches)] == [APPLIED, APPLIED]
    fn = fake_mmcv.MultiScaleDeformableAttnFunction
    # im2col_step is accepted positionally, by keyword, or not at all -- and never forwarded
    assert fn.forward("ctx", 1, 2, 3, 4, 5, 64) == "out" and calls["forward"] == (1, 2, 3, 4, 5)
    assert fn.forward("ctx", 1, 2, 3, 4, 5, im2col_step=8) == "out"
    assert fn.forward("ctx", 1, 2, 3, 4, 5) == "out"
    # six gradient slots for mmcv's six forward arguments
    assert fn.backward("ctx", "g") == ("gv", None, None, "gl", "ga", None) and calls["backward"] == "g"
    for p in patches:
        p.restore()
    with pytest.raises(AssertionError):
        fn.forward("ctx", 1, 2, 3, 4, 5, 64)


def test_atomic_patch_resolves_nested_attributes_and_reports_missing_ones(fake_mmcv):
    p = AtomicPatch("mmcv.ops.multi_scale_deform_attn.MultiScaleDeformableAttnFunction.no_such_attr", 1)
    assert p.apply() == SKIPPED and "no_such_attr" in p.reason
    p = AtomicPatch("mmcv.ops.multi_scale_deform_attn.answer", 42)
    assert p.apply() == SKIPPED
    fake_mmcv.answer = 41
    p = AtomicPatch("mmcv.ops.multi_scale_deform_attn.answer", 41, replacement_wrapper=lambda v: v + 1)
    assert p.apply() == APPLIED and fake_mmcv.answer == 42
    p.restore()
    assert fake_mmcv.answer == 41


@pytest.mark.gpu
def test_patched_mmcv_function_runs_the_hip_operator(fake_mmcv, gpu_device):
    """mmcv's call form, end to end on the GPU: apply(value, shapes, lsi, loc, attn, im2col_step)."""
    from drivingsdk_amd import workloads
    from util import BWD_FP32, FWD_FP32, oracle_all, rel_err

    patches = MultiScaleDeformableAttention.patches()
    assert [s for _, s in apply_patches(patches)] == [APPLIED, APPLIED]
    try:
        inp = workloads.make_inputs("tiny", with_grad_output=True)
        value = inp.value.to(gpu_device).requires_grad_()
        loc = inp.sampling_locations.to(gpu_device).requires_grad_()
        attn = inp.attention_weights.to(gpu_device).requires_grad_()
        out = fake_mmcv.MultiScaleDeformableAttnFunction.apply(
            value, inp.spatial_shapes.to(gpu_device), inp.level_start_index.to(gpu_device), loc, attn, 64)
        out.backward(inp.grad_output.to(gpu_device))
        ref = oracle_all(inp)
        assert rel_err(out.detach().cpu().numpy(), ref[0]) <= FWD_FP32
        assert rel_err(value.grad.cpu().numpy(), ref[1]) <= BWD_FP32
        assert rel_err(attn.grad.cpu().numpy(), ref[3]) <= BWD_FP32
    finally:
        for p in patches:
            p.restore()
