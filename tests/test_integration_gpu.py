"""The reference-side C++ binding over the C ABI (tests/integration/option_a_binding.cpp, built by
`make -C tests/integration` or __graft_entry__.build()): the form in which a PyTorch-ROCm build of the reference's
`mx_driving._C` would call libmxd_msda.so in place of its aclnn launcher
(mx_driving/csrc/MultiScaleDeformableAttn.cpp:28-118)."""
import glob
import importlib.util
import os

import numpy as np
import pytest
import torch

from drivingsdk_amd import _C, workloads
from tests.util import BWD_FP32, FWD_FP32, oracle_all, rel_err

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "integration")


def _np(t):
    return t.detach().double().cpu().numpy()


def _load():
    found = glob.glob(os.path.join(HERE, "mxd_option_a*.so"))
    if not found:
        pytest.skip("tests/integration is not built (make -C tests/integration)")
    spec = importlib.util.spec_from_file_location("mxd_option_a", found[0])
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_binding_module_imports_and_names_the_two_functions():
    """As mx_driving/csrc/pybind.cpp:110-111 registers them."""
    mod = _load()
    assert callable(mod.multi_scale_deformable_attn) and callable(mod.multi_scale_deformable_attn_backward)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("meta", [torch.int32, torch.int64])
def test_binding_matches_the_ctypes_binding_and_the_oracle(gpu_device, dtype, meta):
    mod = _load()
    inp = workloads.reference_test_inputs([2, 190, 32, 8, 3, 4], dtype=dtype, seed=5)
    dev = [t.to(gpu_device) for t in (inp.value, inp.spatial_shapes.to(meta), inp.level_start_index.to(meta),
                                      inp.sampling_locations, inp.attention_weights)]
    out = mod.multi_scale_deformable_attn(*dev)
    ours = _C.multi_scale_deformable_attn(*dev)
    assert torch.equal(out, ours)
    g = torch.Generator().manual_seed(6)
    go = torch.randn(out.shape, generator=g).to(dtype).to(gpu_device)
    grads = mod.multi_scale_deformable_attn_backward(*dev, go)
    ours_g = _C.multi_scale_deformable_attn_backward(*dev, go)
    # (grad_value is summed by workgroups whose atomic additions arrive in any order: compared with a tolerance)
    assert torch.equal(grads[1], ours_g[1]) and torch.equal(grads[2], ours_g[2])
    assert rel_err(_np(grads[0]), _np(ours_g[0])) <= (1e-6 if dtype == torch.float32 else 2e-3)
    if dtype == torch.float32:
        want = oracle_all(workloads.MsdaInputs(inp.value, inp.spatial_shapes, inp.level_start_index, inp.sampling_locations,
                                               inp.attention_weights, go.cpu()))
        assert rel_err(_np(out), want[0]) <= FWD_FP32
        for got, ref in zip(grads, want[1:]):
            assert rel_err(_np(got), ref) <= BWD_FP32


@pytest.mark.gpu
def test_binding_reports_the_library_error(gpu_device):
    mod = _load()
    inp = workloads.reference_test_inputs([1, 20, 32, 4, 2, 2], seed=7)
    dev = [t.to(gpu_device) for t in (inp.value, inp.spatial_shapes, inp.level_start_index, inp.sampling_locations,
                                      inp.attention_weights)]
    wide = torch.zeros(1, dev[0].shape[1], 1, 300, device=gpu_device)
    with pytest.raises(RuntimeError, match="embedding dimensions"):
        mod.multi_scale_deformable_attn(wide, *dev[1:])
