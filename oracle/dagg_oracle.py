"""TEST INFRASTRUCTURE ONLY -- CPU oracle for deformable aggregation.

Two independent statements:

* ``direct_forward`` / ``direct_backward`` -- ctypes wrappers over ``dagg_oracle.c``, which restates the goldens
  of the reference's tests (tests/torch/test_deformable_aggregation.py:29-126,
  tests/torch/test_deformable_aggregation_grad.py:33-181).
* ``via_msda`` -- the operator written as multi-scale deformable attention: group = head, (camera, scale) =
  level, the location of (anchor, point, camera) broadcast over scales and groups, weights permuted to
  ``[bs, anchors, groups, cams*scales, pts]`` and zeroed where the location is not strictly inside (0, 1);
  evaluated with the pinned oracle of that operator (``msda_oracle``).

Not imported by the shipped package.
"""
import ctypes
import os
import subprocess

import numpy as np
import torch

from . import msda_oracle

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdagg_oracle.so")
_lib = None


def build(force=False):
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "libdagg_oracle.so"] + (["-B"] if force else []), check=True,
                       capture_output=True)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        build()
        lib = ctypes.CDLL(_LIB_PATH)
        i64, ptr = ctypes.c_int64, ctypes.c_void_p
        for sfx in ("f32", "f64"):
            f = getattr(lib, f"dagg_oracle_forward_{sfx}")
            f.restype, f.argtypes = ctypes.c_int, [ptr] * 6 + [i64] * 8
            b = getattr(lib, f"dagg_oracle_backward_{sfx}")
            b.restype, b.argtypes = ctypes.c_int, [ptr] * 9 + [i64] * 8
        _lib = lib
    return _lib


def _np(t, dtype):
    if isinstance(t, torch.Tensor):
        t = t.detach().cpu().numpy()
    return np.ascontiguousarray(t, dtype=dtype)


def _dims(feat, ss, loc, wts):
    bs, nf, C = feat.shape
    cams, scales = ss.shape[0], ss.shape[1]
    _, A, P = loc.shape[:3]
    return bs, nf, C, cams, scales, A, P, wts.shape[5]


def direct_forward(feat, spatial_shape, scale_start_index, loc, weights, dtype=np.float64):
    lib = _load()
    sfx = "f64" if dtype == np.float64 else "f32"
    f, lo, w = _np(feat, dtype), _np(loc, dtype), _np(weights, dtype)
    ss, si = _np(spatial_shape, np.int32), _np(scale_start_index, np.int32)
    dims = _dims(f, ss, lo, w)
    out = np.empty((dims[0], dims[5], dims[2]), dtype=dtype)
    rc = getattr(lib, f"dagg_oracle_forward_{sfx}")(f.ctypes.data, ss.ctypes.data, si.ctypes.data, lo.ctypes.data,
                                                    w.ctypes.data, out.ctypes.data, *dims)
    if rc != 0:
        raise ValueError("dagg_oracle_forward: bad arguments")
    return out


def direct_backward(feat, spatial_shape, scale_start_index, loc, weights, grad_out, dtype=np.float64):
    lib = _load()
    sfx = "f64" if dtype == np.float64 else "f32"
    f, lo, w, go = _np(feat, dtype), _np(loc, dtype), _np(weights, dtype), _np(grad_out, dtype)
    ss, si = _np(spatial_shape, np.int32), _np(scale_start_index, np.int32)
    dims = _dims(f, ss, lo, w)
    gf, gl, gw = np.empty_like(f), np.empty_like(lo), np.empty_like(w)
    rc = getattr(lib, f"dagg_oracle_backward_{sfx}")(f.ctypes.data, ss.ctypes.data, si.ctypes.data, lo.ctypes.data,
                                                     w.ctypes.data, go.ctypes.data, gf.ctypes.data, gl.ctypes.data,
                                                     gw.ctypes.data, *dims)
    if rc != 0:
        raise ValueError("dagg_oracle_backward: bad arguments")
    return gf, gl, gw


def via_msda(feat, spatial_shape, scale_start_index, loc, weights, grad_out=None):
    """The operator through the multi-scale deformable attention oracle (float64).
    Returns (out, grad_feat, grad_loc, grad_weights); gradients are None without grad_out."""
    f = torch.as_tensor(np.asarray(feat), dtype=torch.float64) if not isinstance(feat, torch.Tensor) else feat.double()
    lo = torch.as_tensor(np.asarray(loc)).double() if not isinstance(loc, torch.Tensor) else loc.double()
    w = torch.as_tensor(np.asarray(weights)).double() if not isinstance(weights, torch.Tensor) else weights.double()
    ss = torch.as_tensor(np.asarray(spatial_shape)).long()
    si = torch.as_tensor(np.asarray(scale_start_index)).long()
    bs, nf, C = f.shape
    cams, scales = ss.shape[:2]
    _, A, P = lo.shape[:3]
    G = w.shape[5]
    L = cams * scales
    value = f.reshape(bs, nf, G, C // G)
    shapes, lsi = ss.reshape(L, 2), si.reshape(L)
    inside = ((lo[..., 0] > 0) & (lo[..., 0] < 1) & (lo[..., 1] > 0) & (lo[..., 1] < 1))         # [bs,A,P,cams]
    # loc_msda[b,a,g,l=(cam,scale),p,:] = loc[b,a,p,cam,:]
    lm = lo.permute(0, 1, 3, 2, 4)[:, :, None, :, None].expand(bs, A, G, cams, scales, P, 2).reshape(bs, A, G, L, P, 2)
    # attn_msda[b,a,g,l,p] = weights[b,a,p,cam,scale,g] * inside[b,a,p,cam]
    am = (w * inside[..., None, None]).permute(0, 1, 5, 3, 4, 2).reshape(bs, A, G, L, P)
    out = msda_oracle.direct_forward(value, shapes, lsi, lm, am)
    if grad_out is None:
        return out, None, None, None
    gv, gl, ga = msda_oracle.direct_backward(value, shapes, lsi, lm, am, grad_out)
    gfeat = gv.reshape(bs, nf, C)
    gl = torch.as_tensor(gl).reshape(bs, A, G, cams, scales, P, 2)
    gloc = gl.sum(dim=(2, 4)).permute(0, 1, 3, 2, 4).numpy()                                      # [bs,A,P,cams,2]
    ga = torch.as_tensor(ga).reshape(bs, A, G, cams, scales, P)
    gw = (ga.permute(0, 1, 5, 3, 4, 2) * inside[..., None, None]).numpy()
    return out, gfeat, gloc, gw
