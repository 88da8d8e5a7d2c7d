"""TEST INFRASTRUCTURE ONLY -- CPU oracle for geometric kernel attention.

Restates the golden of the reference's test (tests/torch/test_geometric_kernel_attention.py:44-93: clamp the
pixel indices to the level, flat index = level_start + x + y*W, gather the rows of value, weight and sum) in
numpy with float64 arithmetic, and its gradients in closed form (the golden takes them from autograd).
Pinned in tests/test_gka_oracle.py by a hand case and by the multi-scale deformable attention oracle evaluated at
pixel centres.  Not imported by the shipped package.
"""
import numpy as np
import torch


def _np(t, dtype=np.float64):
    if isinstance(t, torch.Tensor):
        t = t.detach().cpu().numpy()
    return np.asarray(t, dtype=dtype)


def _flat_index(shapes, lsi, loc):
    """[bs, nq, nh, nl, np] row index into value's num_keys axis."""
    shapes, lsi = _np(shapes, np.int64), _np(lsi, np.int64)
    loc = np.trunc(_np(loc)).astype(np.int64)                      # locations are integral; truncation as a cast does
    idx = np.empty(loc.shape[:-1], dtype=np.int64)
    for lvl, (h, w) in enumerate(shapes.tolist()):
        x = np.clip(loc[:, :, :, lvl, :, 0], 0, w - 1)
        y = np.clip(loc[:, :, :, lvl, :, 1], 0, h - 1)
        idx[:, :, :, lvl] = lsi[lvl] + x + y * w
    return idx


def forward(value, shapes, lsi, loc, attn):
    v, a = _np(value), _np(attn)
    bs, nk, nh, hd = v.shape
    idx = _flat_index(shapes, lsi, loc)                             # [bs, nq, nh, nl, np]
    nq = idx.shape[1]
    out = np.zeros((bs, nq, nh, hd))
    for b in range(bs):
        for h in range(nh):
            rows = v[b, :, h, :][idx[b, :, h].reshape(nq, -1)]      # [nq, nl*np, hd]
            out[b, :, h, :] = (rows * a[b, :, h].reshape(nq, -1, 1)).sum(1)
    return out.reshape(bs, nq, nh * hd)


def backward(value, shapes, lsi, loc, attn, grad_out):
    v, a, go = _np(value), _np(attn), _np(grad_out)
    bs, nk, nh, hd = v.shape
    idx = _flat_index(shapes, lsi, loc)
    nq = idx.shape[1]
    go = go.reshape(bs, nq, nh, hd)
    gv, ga = np.zeros_like(v), np.zeros_like(a)
    for b in range(bs):
        for h in range(nh):
            flat = idx[b, :, h].reshape(nq, -1)                     # [nq, S]
            rows = v[b, :, h, :][flat]                              # [nq, S, hd]
            ga[b, :, h] = (rows * go[b, :, h][:, None, :]).sum(-1).reshape(a.shape[1], *a.shape[3:])
            contrib = a[b, :, h].reshape(nq, -1, 1) * go[b, :, h][:, None, :]
            np.add.at(gv[b, :, h, :], flat.reshape(-1), contrib.reshape(-1, hd))
    return gv, ga
