"""Shared helpers of the parity tests."""
import numpy as np
import torch

from oracle import msda_oracle as orc

# Tolerances of the path (relative to the largest reference magnitude of the tensor):
FWD_FP32 = 1e-5   # forward, float32
BWD_FP32 = 1e-4   # gradients, float32
HALF = 2e-3       # float16 / bfloat16, forward and gradients


def rel_err(got, ref):
    """max |got - ref| / max |ref|  (0 when both are identically zero)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.all(np.isfinite(got)), "non-finite values in the result"
    denom = np.abs(ref).max()
    num = np.abs(got - ref).max()
    return 0.0 if num == 0.0 else num / max(denom, 1e-300)


def oracle_all(inp, with_grads=True):
    """float64 direct-form oracle on the inputs exactly as stored (so for float16/bfloat16
    the rounded inputs are what is evaluated)."""
    v, sh, ls = inp.value.double(), inp.spatial_shapes, inp.level_start_index
    lo, at = inp.sampling_locations.double(), inp.attention_weights.double()
    out = orc.direct_forward(v, sh, ls, lo, at)
    if not with_grads:
        return out, None, None, None
    gv, gl, ga = orc.direct_backward(v, sh, ls, lo, at, inp.grad_output.double())
    return out, gv, gl, ga


def to_device(inp, device):
    return type(inp)(*[None if t is None else t.to(device) for t in inp])


def run_gpu(inp, device, with_grads=True):
    """Through the public API (autograd Function) on the GPU.  Returns numpy float64 arrays."""
    import mx_driving

    d = to_device(inp, device)
    value = d.value.clone().requires_grad_(with_grads)
    loc = d.sampling_locations.clone().requires_grad_(with_grads)
    attn = d.attention_weights.clone().requires_grad_(with_grads)
    out = mx_driving.multi_scale_deformable_attn(value, d.spatial_shapes, d.level_start_index, loc, attn)
    res = [out.detach().double().cpu().numpy()]
    if with_grads:
        out.backward(d.grad_output)
        res += [t.grad.double().cpu().numpy() for t in (value, loc, attn)]
        assert value.grad.dtype == value.dtype and loc.grad.dtype == loc.dtype and attn.grad.dtype == attn.dtype
    else:
        res += [None, None, None]
    torch.cuda.synchronize()
    return res


def set_tuning(monkeypatch, **env):
    """Set MXD_MSDA_* tuning variables for the rest of a test and have the library read them (it reads the
    environment once per process otherwise; conftest reads it again after the test)."""
    from drivingsdk_amd import _lib
    for k, v in env.items():
        monkeypatch.setenv(k, str(v))
    _lib.reload_tuning()
