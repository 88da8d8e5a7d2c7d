"""TEST INFRASTRUCTURE ONLY -- CPU oracle for multi-scale deformable attention.

Two independent statements of the operator live here; neither is imported by the
shipped package (only by tests, the smoke check and the benchmark's CPU-baseline leg):

* ``msda_grid_sample`` -- the contractual oracle: the pure-PyTorch ``grid_sample``
  formulation the reference's own test uses as its golden
  (tests/torch/test_multi_scale_deformable_attn.py:35-64), with gradients from
  ``torch.autograd`` exactly as that test takes them (:68-76, :93-101).
* ``direct_forward`` / ``direct_backward`` -- ctypes wrappers over ``msda_oracle.c``
  (explicit floor / corner / validity arithmetic following the reference's SIMT
  kernels; citations in that file).  Also used as the "port" CPU baseline.

Parity pins are listed in ``msda_oracle.c`` and exercised by ``tests/test_oracle.py``.
Unpinned: ``attention_weights`` carrying more levels than ``spatial_shapes``.
"""
import ctypes
import os
import subprocess

import numpy as np
import torch
import torch.nn.functional as F

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmsda_oracle.so")
_lib = None


def build(force=False):
    """Compile msda_oracle.c with gcc (make).  Returns the path of the library."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True, capture_output=True)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        build()
        lib = ctypes.CDLL(_LIB_PATH)
        i64 = ctypes.c_int64
        ptr = ctypes.c_void_p
        for sfx in ("f32", "f64"):
            fwd = getattr(lib, f"msda_oracle_forward_{sfx}")
            fwd.restype = ctypes.c_int
            fwd.argtypes = [ptr] * 6 + [i64] * 8
            bwd = getattr(lib, f"msda_oracle_backward_{sfx}")
            bwd.restype = ctypes.c_int
            bwd.argtypes = [ptr] * 9 + [i64] * 8
        lib.msda_oracle_threads.restype = ctypes.c_int
        lib.msda_oracle_set_threads.argtypes = [ctypes.c_int]
        _lib = lib
    return _lib


def threads():
    return _load().msda_oracle_threads()


def set_threads(n):
    _load().msda_oracle_set_threads(int(n))


def _dims(value, shapes, loc):
    bs, nk, nh, hd = value.shape
    nl = shapes.shape[0]
    _, nq, _, nl_attn, npts, _ = loc.shape
    return bs, nk, nh, hd, nl, nl_attn, nq, npts


def _np(t, dtype):
    if isinstance(t, torch.Tensor):
        t = t.detach().cpu().numpy()
    return np.ascontiguousarray(t, dtype=dtype)


def direct_forward(value, shapes, lsi, loc, attn, dtype=np.float64):
    """Direct bilinear form on the CPU, arithmetic in ``dtype`` (float64 or float32)."""
    lib = _load()
    sfx = "f64" if dtype == np.float64 else "f32"
    v, lo, at = _np(value, dtype), _np(loc, dtype), _np(attn, dtype)
    sh, ls = _np(shapes, np.int32), _np(lsi, np.int32)
    bs, nk, nh, hd, nl, nl_attn, nq, npts = _dims(v, sh, lo)
    out = np.empty((bs, nq, nh * hd), dtype=dtype)
    rc = getattr(lib, f"msda_oracle_forward_{sfx}")(
        v.ctypes.data, sh.ctypes.data, ls.ctypes.data, lo.ctypes.data, at.ctypes.data, out.ctypes.data,
        bs, nk, nh, hd, nl, nl_attn, nq, npts)
    if rc != 0:
        raise ValueError("msda_oracle_forward: bad arguments")
    return out


def direct_backward(value, shapes, lsi, loc, attn, grad_out, dtype=np.float64):
    lib = _load()
    sfx = "f64" if dtype == np.float64 else "f32"
    v, lo, at, go = _np(value, dtype), _np(loc, dtype), _np(attn, dtype), _np(grad_out, dtype)
    sh, ls = _np(shapes, np.int32), _np(lsi, np.int32)
    bs, nk, nh, hd, nl, nl_attn, nq, npts = _dims(v, sh, lo)
    gv, gl, ga = np.empty_like(v), np.empty_like(lo), np.empty_like(at)
    rc = getattr(lib, f"msda_oracle_backward_{sfx}")(
        v.ctypes.data, sh.ctypes.data, ls.ctypes.data, lo.ctypes.data, at.ctypes.data, go.ctypes.data,
        gv.ctypes.data, gl.ctypes.data, ga.ctypes.data, bs, nk, nh, hd, nl, nl_attn, nq, npts)
    if rc != 0:
        raise ValueError("msda_oracle_backward: bad arguments")
    return gv, gl, ga


def msda_grid_sample(value, shapes, loc, attn):
    """grid_sample formulation (reference golden,
    tests/torch/test_multi_scale_deformable_attn.py:35-64).  Differentiable."""
    bs, _, nh, hd = value.shape
    _, nq, _, nl, npts, _ = loc.shape
    sizes = [int(h) * int(w) for h, w in shapes.tolist()]
    per_level = value.split(sizes, dim=1)
    grids = 2 * loc - 1
    sampled = []
    for lvl, (h, w) in enumerate(shapes.tolist()):
        img = per_level[lvl].flatten(2).transpose(1, 2).reshape(bs * nh, hd, int(h), int(w))
        grid = grids[:, :, :, lvl].transpose(1, 2).flatten(0, 1)  # [bs*nh, nq, np, 2]
        sampled.append(F.grid_sample(img, grid, mode="bilinear", padding_mode="zeros", align_corners=False))
    weights = attn.transpose(1, 2).reshape(bs * nh, 1, nq, nl * npts)
    out = (torch.stack(sampled, dim=-2).flatten(-2) * weights).sum(-1).view(bs, nh * hd, nq)
    return out.transpose(1, 2).contiguous()


def msda_grid_sample_fwd_bwd(value, shapes, loc, attn, grad_out=None, dtype=torch.float64):
    """Forward and (optionally) the three gradients through autograd, computed in ``dtype``
    (the reference test uses float64, :93-97).  Returns (out, gv, gl, ga) as tensors."""
    v = value.detach().to("cpu", dtype).requires_grad_(grad_out is not None)
    lo = loc.detach().to("cpu", dtype).requires_grad_(grad_out is not None)
    at = attn.detach().to("cpu", dtype).requires_grad_(grad_out is not None)
    out = msda_grid_sample(v, shapes.cpu().long(), lo, at)
    if grad_out is None:
        return out.detach(), None, None, None
    out.backward(grad_out.detach().to("cpu", dtype))
    return out.detach(), v.grad, lo.grad, at.grad


def fused_sampling_inputs(shapes, reference_points, sampling_offsets, attention_logits):
    """What deformable-attention modules compute between their linear layers and the operator
    (model_examples/Deformable-DETR/Deformable-DETR_npu.patch:626-652 of the reference; upstream
    MSDeformAttn.forward): softmax over the nl*np logits of a (batch, query, head) and
    location = reference point + offset / (W, H), or + offset / np * (w, h) / 2 for box
    reference points.  Written with explicit index arithmetic, not by calling the product's helper.
    Pinned in tests/test_oracle.py by closed forms (zero offsets, uniform logits, a hand case)."""
    bs, nq, nh, nl, npts, _ = sampling_offsets.shape
    z = attention_logits.reshape(bs, nq, nh, nl * npts)
    z = z - z.max(dim=-1, keepdim=True).values
    e = torch.exp(z)
    attn = (e / e.sum(dim=-1, keepdim=True)).reshape(bs, nq, nh, nl, npts)
    loc = []
    for lvl in range(nl):
        h, w = float(shapes[lvl, 0]), float(shapes[lvl, 1])
        ref = reference_points[:, :, lvl]                      # [bs, nq, 2 or 4]
        off = sampling_offsets[:, :, :, lvl]                   # [bs, nq, nh, np, 2]
        if reference_points.shape[-1] == 2:
            x = ref[:, :, None, None, 0] + off[..., 0] / w
            y = ref[:, :, None, None, 1] + off[..., 1] / h
        else:
            x = ref[:, :, None, None, 0] + off[..., 0] / npts * ref[:, :, None, None, 2] * 0.5
            y = ref[:, :, None, None, 1] + off[..., 1] / npts * ref[:, :, None, None, 3] * 0.5
        loc.append(torch.stack([x, y], dim=-1))
    return torch.stack(loc, dim=3), attn


def fused_fwd_bwd(value, shapes, reference_points, sampling_offsets, attention_logits, grad_out=None,
                  dtype=torch.float64, loc_dtype=None):
    """Fused form through ``msda_grid_sample`` and autograd in ``dtype``.  With ``loc_dtype`` (float32) the
    sampling locations are first formed in that type -- the same correctly rounded operations in the same order
    as the callers' torch code and the kernel, hence the same bits -- and only then widened, so that the
    comparison is not dominated by which side of a cell edge a float32 location falls on.
    Returns (out, grad_value, grad_reference_points, grad_sampling_offsets, grad_attention_logits)."""
    g = grad_out is not None
    v = value.detach().to("cpu", dtype).requires_grad_(g)
    r = reference_points.detach().to("cpu", dtype).requires_grad_(g)
    o = sampling_offsets.detach().to("cpu", dtype).requires_grad_(g)
    z = attention_logits.detach().to("cpu", dtype).requires_grad_(g)
    sh = shapes.cpu().long()
    loc, attn = fused_sampling_inputs(sh, r, o, z)
    if loc_dtype is not None:
        loc = fused_sampling_inputs(sh, r.to(loc_dtype), o.to(loc_dtype), z.to(loc_dtype))[0].to(dtype)
    out = msda_grid_sample(v, sh, loc, attn)
    if not g:
        return out.detach(), None, None, None, None
    out.backward(grad_out.detach().to("cpu", dtype))
    return out.detach(), v.grad, r.grad, o.grad, z.grad
