"""Pins of the geometric-kernel-attention oracle (CPU only)."""
import numpy as np
import torch

from oracle import gka_oracle as gka
from oracle import msda_oracle as msda


def _case(seed=0, bs=2, nq=7, nh=3, hd=4, npts=5, shapes=((6, 10), (3, 4)), lo=-3):
    g = torch.Generator().manual_seed(seed)
    sh = torch.tensor(shapes)
    lsi = torch.cat((sh.new_zeros((1,)), sh.prod(1).cumsum(0)[:-1]))
    nk, nl = int(sh.prod(1).sum()), len(shapes)
    value = torch.randn(bs, nk, nh, hd, generator=g, dtype=torch.float64)
    loc = torch.empty(bs, nq, nh, nl, npts, 2, dtype=torch.float64)
    for lvl, (h, w) in enumerate(shapes):
        loc[:, :, :, lvl, :, 0] = torch.randint(lo, w + 3, (bs, nq, nh, npts), generator=g).double()
        loc[:, :, :, lvl, :, 1] = torch.randint(lo, h + 3, (bs, nq, nh, npts), generator=g).double()
    attn = torch.rand(bs, nq, nh, nl, npts, generator=g, dtype=torch.float64)
    go = torch.randn(bs, nq, nh * hd, generator=g, dtype=torch.float64)
    return value, sh, lsi, loc, attn, go


def test_hand_case_with_clamping():
    # one 2x3 map, value[p] = p + 1 (one head, one channel); samples (x,y): (1,0) -> pixel 1; (-5, 1) -> clamped to
    # (0,1) = pixel 3; (7, 9) -> clamped to (2,1) = pixel 5
    sh, lsi = torch.tensor([[2, 3]]), torch.tensor([0])
    value = torch.arange(1, 7, dtype=torch.float64).view(1, 6, 1, 1)
    loc = torch.tensor([[1.0, 0.0], [-5.0, 1.0], [7.0, 9.0]]).view(1, 1, 1, 1, 3, 2)
    attn = torch.tensor([0.5, 2.0, 1.0]).view(1, 1, 1, 1, 3)
    out = gka.forward(value, sh, lsi, loc, attn)
    assert out.tolist() == [[[0.5 * 2 + 2.0 * 4 + 1.0 * 6]]]
    gv, ga = gka.backward(value, sh, lsi, loc, attn, torch.tensor([[[3.0]]]))
    assert gv.reshape(-1).tolist() == [0.0, 1.5, 0.0, 6.0, 0.0, 3.0]
    assert ga.reshape(-1).tolist() == [6.0, 12.0, 18.0]


def test_equals_bilinear_sampling_at_pixel_centres():
    value, sh, lsi, loc, attn, go = _case(lo=0)
    # in-range indices only: the pixel centre (x+0.5)/W, (y+0.5)/H samples exactly that pixel
    for lvl, (h, w) in enumerate(sh.tolist()):
        loc[:, :, :, lvl, :, 0].clamp_(0, w - 1)
        loc[:, :, :, lvl, :, 1].clamp_(0, h - 1)
    norm = loc.clone()
    for lvl, (h, w) in enumerate(sh.tolist()):
        norm[:, :, :, lvl, :, 0] = (loc[:, :, :, lvl, :, 0] + 0.5) / w
        norm[:, :, :, lvl, :, 1] = (loc[:, :, :, lvl, :, 1] + 0.5) / h
    out = gka.forward(value, sh, lsi, loc, attn)
    gv, ga = gka.backward(value, sh, lsi, loc, attn, go)
    out_m = msda.direct_forward(value, sh, lsi, norm, attn)
    gv_m, _, ga_m = msda.direct_backward(value, sh, lsi, norm, attn, go)
    assert np.abs(out - out_m).max() <= 1e-12
    assert np.abs(gv - gv_m).max() <= 1e-12 and np.abs(ga - ga_m).max() <= 1e-12


def test_clamped_equals_in_range_and_gradients_are_adjoint():
    value, sh, lsi, loc, attn, go = _case(seed=3)
    clamped = loc.clone()
    for lvl, (h, w) in enumerate(sh.tolist()):
        clamped[:, :, :, lvl, :, 0].clamp_(0, w - 1)
        clamped[:, :, :, lvl, :, 1].clamp_(0, h - 1)
    assert (clamped != loc).any()
    assert np.array_equal(gka.forward(value, sh, lsi, loc, attn), gka.forward(value, sh, lsi, clamped, attn))
    # the operator is bilinear in (value, attn): <out(dv, attn), go> = <dv, grad_value>, same for attn
    gv, ga = gka.backward(value, sh, lsi, loc, attn, go)
    g = torch.Generator().manual_seed(9)
    dv = torch.randn(value.shape, generator=g, dtype=torch.float64)
    da = torch.randn(attn.shape, generator=g, dtype=torch.float64)
    lhs_v = (gka.forward(dv, sh, lsi, loc, attn) * go.numpy()).sum()
    lhs_a = (gka.forward(value, sh, lsi, loc, da) * go.numpy()).sum()
    assert abs(lhs_v - (dv.numpy() * gv).sum()) <= 1e-10 * max(1.0, abs(lhs_v))
    assert abs(lhs_a - (da.numpy() * ga).sum()) <= 1e-10 * max(1.0, abs(lhs_a))
