"""Pins of the deformable-aggregation oracle (CPU only): the C restatement of the reference's test goldens
against the same operator written through the multi-scale deformable attention oracle, a hand-computed case,
a closed form and finite differences."""
import numpy as np
import pytest
import torch

from oracle import dagg_oracle as dagg


def _case(seed=0, bs=2, C=16, G=8, A=5, P=3, pad=True):
    rng = np.random.default_rng(seed)
    ss = np.array([[[6, 5], [3, 4]], [[4, 7], [2, 3]]], dtype=np.int32)
    cams, scales = 2, 2
    sizes = ss.reshape(-1, 2).prod(1)
    ssi = np.concatenate([[0], np.cumsum(sizes)[:-1]]).reshape(cams, scales).astype(np.int32)
    nf = int(sizes.sum())
    feat = rng.standard_normal((bs, nf, C))
    loc = rng.random((bs, A, P, cams, 2)) * (1.2 if pad else 0.8) + (-0.1 if pad else 0.1)
    w = rng.random((bs, A, P, cams, scales, G))
    go = rng.standard_normal((bs, A, C))
    return feat, ss, ssi, loc, w, go


def test_two_formulations_agree():
    for seed in (0, 1, 2):
        feat, ss, ssi, loc, w, go = _case(seed)
        out = dagg.direct_forward(feat, ss, ssi, loc, w)
        gf, gl, gw = dagg.direct_backward(feat, ss, ssi, loc, w, go)
        out2, gf2, gl2, gw2 = dagg.via_msda(feat, ss, ssi, loc, w, go)
        for a, b in ((out, out2), (gf, gf2), (gl, gl2), (gw, gw2)):
            assert np.abs(a - b).max() <= 1e-12 * max(1.0, np.abs(b).max())
        # locations outside (0, 1) contribute nothing and receive nothing
        outside = ~((loc[..., 0] > 0) & (loc[..., 0] < 1) & (loc[..., 1] > 0) & (loc[..., 1] < 1))
        assert outside.any()
        assert np.all(gl[outside] == 0) and np.all(gw[outside] == 0)


def test_hand_computed_case():
    # one camera, one scale, a 2x2 map, 2 groups of one channel; value = [[1, 2], [3, 4]] and ten times that
    ss = np.array([[[2, 2]]], dtype=np.int32)
    ssi = np.array([[0]], dtype=np.int32)
    feat = np.array([[[1, 10], [2, 20], [3, 30], [4, 40]]], dtype=np.float64)   # [1, 4, 2]
    # pixel coordinates x*2-0.5, y*2-0.5: (0.5, 0.5) -> centre of the four pixels; (0.25, 0.25) -> pixel (0,0);
    # (0.875, 0.25) -> x = 1.25: between pixel 1 and the right border (weight 0.75 on pixel 1, 0.25 on padding)
    loc = np.array([[[[[0.5, 0.5]], [[0.25, 0.25]], [[0.875, 0.25]]]]], dtype=np.float64)  # [1,1,3,1,2]
    w = np.array([1.0, 2.0, 0.5, 1.0, 4.0, 0.0]).reshape(1, 1, 3, 1, 1, 2)
    out = dagg.direct_forward(feat, ss, ssi, loc, w)
    # group 0: 1*2.5 + 0.5*1 + 4*(0.75*2) = 9 ; group 1: 2*25 + 1*10 + 0 = 60
    assert np.allclose(out, [[[9.0, 60.0]]], rtol=0, atol=1e-15)
    go = np.array([[[1.0, 0.1]]])
    gf, gl, gw = dagg.direct_backward(feat, ss, ssi, loc, w, go)
    # grad_weights = grad * sampled value
    assert np.allclose(gw.reshape(3, 2), [[2.5, 2.5], [1.0, 1.0], [1.5, 1.5]], rtol=0, atol=1e-15)
    # grad_feat channel 0: 0.25*1 each from the centre sample, + 0.5 on pixel 0, + 4*0.75 on pixel 1
    assert np.allclose(gf[0, :, 0], [0.25 + 0.5, 0.25 + 3.0, 0.25, 0.25], rtol=0, atol=1e-15)
    assert np.allclose(gf[0, :, 1], [0.1 * (0.5 + 1.0), 0.1 * 0.5, 0.1 * 0.5, 0.1 * 0.5], rtol=0, atol=1e-15)
    # centre sample: d/dx = W * ((2-1)+(4-3))/2 = 2 per unit value scale, d/dy = H * ((3-1)+(4-2))/2 = 4;
    # times (w0*g0 + 10*w1*g1) = 1 + 2 = 3
    assert np.allclose(gl[0, 0, 0, 0], [2 * 3.0, 4 * 3.0], rtol=0, atol=1e-14)
    # right-border sample: d/dx = W * (0 - 2) (padding is zero), group 0 only (weight 4, grad 1); d/dy = H*0.75*(4-2)
    assert np.allclose(gl[0, 0, 2, 0], [2 * (-2.0) * 4.0, 2 * 0.75 * 2.0 * 4.0], rtol=0, atol=1e-14)


def test_constant_field_closed_form():
    feat, ss, ssi, loc, w, _ = _case(3, pad=False)
    # keep every sample at least one pixel away from the border of the coarsest map so that all corners exist
    loc = 0.3 + 0.4 * (loc - 0.1) / 0.8
    feat[:] = np.arange(1, feat.shape[2] + 1)[None, None, :]
    out = dagg.direct_forward(feat, ss, ssi, loc, w)
    G, cg = w.shape[5], feat.shape[2] // w.shape[5]
    wsum = w.sum(axis=(2, 3, 4))                                            # [bs, A, G]
    want = np.repeat(wsum, cg, axis=2) * np.arange(1, feat.shape[2] + 1)
    assert np.allclose(out, want, rtol=1e-13)


def test_gradients_by_finite_differences():
    feat, ss, ssi, loc, w, go = _case(4, pad=False)
    gf, gl, gw = dagg.direct_backward(feat, ss, ssi, loc, w, go)

    def f(feat_, loc_, w_):
        return float((dagg.direct_forward(feat_, ss, ssi, loc_, w_) * go).sum())
    eps = 1e-6
    rng = np.random.default_rng(9)
    for name, arr, grad in (("feat", feat, gf), ("loc", loc, gl), ("weights", w, gw)):
        for _ in range(6):
            idx = tuple(rng.integers(0, s) for s in arr.shape)
            ap, am = arr.copy(), arr.copy()
            ap[idx] += eps
            am[idx] -= eps
            args_p = [feat, loc, w]
            args_m = [feat, loc, w]
            k = ("feat", "loc", "weights").index(name)
            args_p[k], args_m[k] = ap, am
            fd = (f(*args_p) - f(*args_m)) / (2 * eps)
            assert abs(fd - grad[idx]) <= 2e-6 * max(1.0, abs(fd)), (name, idx, fd, grad[idx])


def test_float32_variant_tracks_float64():
    feat, ss, ssi, loc, w, go = _case(5)
    o64 = dagg.direct_forward(feat, ss, ssi, loc, w)
    o32 = dagg.direct_forward(feat, ss, ssi, loc, w, dtype=np.float32)
    assert np.abs(o32 - o64).max() <= 1e-5 * np.abs(o64).max()
