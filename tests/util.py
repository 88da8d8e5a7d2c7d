"""Shared helpers of the parity tests."""
import numpy as np
import torch

from oracle import msda_oracle as orc

# Tolerances of the path (relative to the largest reference magnitude of the tensor):
FWD_FP32 = 1e-5   # forward, float32
BWD_FP32 = 1e-4   # gradients, float32
HALF = 2e-3       # float16, forward and gradients
# bfloat16 keeps 8 significant bits: one correct rounding of a result is off by up to 2^-8 = 3.9e-3 of the element
# (its unit round-off), and in a large tensor some element near the largest magnitude comes close to that bound.  No
# bfloat16 output, however it was computed, can promise less against an unrounded reference, so 2^-8 is the bound for
# the max-norm figure; the element-wise comparison with the ROUNDED reference (check_16bit: at most one unit in the
# last place) is the sharp statement for both 16-bit types.
BF16 = 2.0 ** -8


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


def half_tol(dtype):
    """Max-norm tolerance of a 16-bit storage type against the unrounded float64 oracle."""
    return HALF if dtype == torch.float16 else BF16


def level_slices(inp, kind):
    """Index tuples that cut a tensor of the path into its levels: 'keys' for value / grad_value ([bs, nk, nh, hd],
    rows level_start .. level_start + H*W), 'samples' for the per-sample tensors ([bs, nq, nh, nl, np(, 2)])."""
    shapes, lsi = inp.spatial_shapes.tolist(), inp.level_start_index.tolist()
    if kind == "keys":
        return [(slice(None), slice(s, s + h * w)) for (h, w), s in zip(shapes, lsi)]
    return [(slice(None), slice(None), slice(None), slice(l, l + 1)) for l in range(len(shapes))]


def check_close(got, ref, rtol, what, groups=None):
    """Element-wise |got - ref| <= rtol * |ref| + rtol * RMS(ref), the RMS taken over the element's group (a level
    when `groups` cuts the tensor into levels, else the whole tensor): a defect confined to small elements or to
    a level whose values are small cannot hide behind the largest element of the tensor."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    for idx in (groups or [()]):
        g, r = got[idx], ref[idx]
        if r.size == 0:
            continue
        rms = float(np.sqrt(np.mean(r * r)))
        excess = np.abs(g - r) - rtol * (np.abs(r) + rms)
        worst = float(excess.max())
        assert worst <= 0.0, (what, idx, "element-wise bound exceeded by", worst, "rms", rms,
                              "at", np.unravel_index(int(excess.argmax()), excess.shape))


def _ulp(x, dtype):
    """Unit in the last place of the storage dtype at the magnitudes of x (float64 array)."""
    p, emin = (11, -14) if dtype == torch.float16 else (8, -126)
    mag = np.abs(x)
    e = np.floor(np.log2(np.where(mag > 0, mag, 1.0)))
    e = np.maximum(np.where(mag > 0, e, emin), emin)
    return np.exp2(e - (p - 1))


def check_16bit(got, ref64, dtype, what, groups=None, tol32=1e-5):
    """The reference's own 16-bit test rounds its golden to the storage type and compares
    (tests/torch/test_multi_scale_deformable_attn.py:256-264).  Here: the float64 oracle (evaluated on the rounded
    inputs) rounded once to `dtype`; the kernel, which accumulates in float32 and rounds once, may land on the
    neighbouring value where the exact result sits next to a rounding boundary, so every element must be within one
    unit in the last place of the rounded reference, plus what the float32 path itself is allowed before the rounding
    (tol32 * (|ref| + RMS of the group): it matters only where the reference nearly cancels)."""
    got = np.asarray(got, dtype=np.float64)
    ref64 = np.asarray(ref64, dtype=np.float64)
    rounded = torch.from_numpy(ref64).to(dtype).double().numpy()
    for idx in (groups or [()]):
        g, r = got[idx], rounded[idx]
        if r.size == 0:
            continue
        rms = float(np.sqrt(np.mean(r * r)))
        excess = np.abs(g - r) - (_ulp(r, dtype) + tol32 * (np.abs(r) + rms))
        worst = float(excess.max())
        assert worst <= 0.0, (what, idx, "more than one unit in the last place off the rounded oracle by", worst,
                              "at", np.unravel_index(int(excess.argmax()), excess.shape))
