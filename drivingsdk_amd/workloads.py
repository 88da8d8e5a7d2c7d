"""Seeded synthetic inputs for multi-scale deformable attention.

The five named workloads are the shapes the benchmark and the parity tests run on
(tiny CPU-sized case, Deformable-DETR encoder, BEVFormer spatial cross attention,
head_dim 128, and the encoder shape again with a grad_output for the backward pass).
``reference_test_inputs`` rebuilds the input recipe of the reference's operator test
(tests/torch/test_multi_scale_deformable_attn.py:15-31) with a fixed seed.

Everything is generated on the CPU with ``torch.Generator().manual_seed`` so that a
GPU run and a CPU oracle run see bit-identical inputs.
"""
from collections import namedtuple

import torch

MsdaInputs = namedtuple(
    "MsdaInputs", ["value", "spatial_shapes", "level_start_index", "sampling_locations", "attention_weights",
                   "grad_output"])

_DETR_LEVELS = ((100, 150), (50, 75), (25, 38), (13, 19))
_BEV_LEVELS = ((116, 200), (58, 100), (29, 50), (15, 25))

WORKLOADS = {
    # name: (bs, nq or None (= nk), levels, nh, hd, np, location recipe, seed)
    "tiny": dict(bs=1, nq=None, levels=((32, 32), (16, 16), (8, 8), (4, 4)), nh=8, hd=32, np=4, loc="uniform_pad",
                 seed=1001),
    "detr_encoder": dict(bs=2, nq=None, levels=_DETR_LEVELS, nh=8, hd=32, np=4, loc="ref_plus_offset", seed=1002),
    "bevformer_sca": dict(bs=6, nq=9675, levels=_BEV_LEVELS, nh=8, hd=32, np=8, loc="anchor_cluster", seed=1003),
    "head_dim_128": dict(bs=1, nq=None, levels=_DETR_LEVELS, nh=8, hd=128, np=4, loc="uniform", seed=1004),
    "detr_encoder_bwd": dict(bs=2, nq=None, levels=_DETR_LEVELS, nh=8, hd=32, np=4, loc="ref_plus_offset", seed=1005),
    # the encoder's queries over its two coarse levels only, 8 points each (16 samples per query as in the encoder): every
    # row fits the LDS of a CU, so the forward's one-workgroup-per-CU form gathers nothing from memory -- the
    # measurement twin of the encoder shape with MXD_MSDA_FWD_CU_CACHE=0 (everything from memory)
    "detr_encoder_coarse": dict(bs=2, nq=19947, levels=_DETR_LEVELS[2:], nh=8, hd=32, np=8, loc="ref_plus_offset", seed=1006),
}


def level_tensors(levels):
    shapes = torch.tensor(levels, dtype=torch.int64).reshape(-1, 2)
    lsi = torch.cat((shapes.new_zeros((1,)), shapes.prod(1).cumsum(0)[:-1]))
    return shapes, lsi


def make_inputs(name, dtype=torch.float32, with_grad_output=None, scale_queries=1.0):
    """Build the named workload on the CPU.  ``scale_queries`` < 1 shrinks nq (for quick
    CPU checks of a big shape); the level pyramid is never changed."""
    cfg = WORKLOADS[name]
    g = torch.Generator().manual_seed(cfg["seed"])
    shapes, lsi = level_tensors(cfg["levels"])
    nk = int(shapes.prod(1).sum())
    bs, nh, hd, npts, nl = cfg["bs"], cfg["nh"], cfg["hd"], cfg["np"], shapes.shape[0]
    nq = cfg["nq"] if cfg["nq"] is not None else nk
    nq = max(1, int(round(nq * scale_queries)))

    value = torch.randn(bs, nk, nh, hd, generator=g)
    kind = cfg["loc"]
    if kind == "uniform_pad":
        loc = torch.rand(bs, nq, nh, nl, npts, 2, generator=g) * 1.2 - 0.1
    elif kind == "uniform":
        loc = torch.rand(bs, nq, nh, nl, npts, 2, generator=g)
    elif kind == "ref_plus_offset":
        ref = torch.rand(bs, nq, 1, 1, 1, 2, generator=g)
        loc = ref + 0.02 * torch.randn(bs, nq, nh, nl, npts, 2, generator=g)
    elif kind == "anchor_cluster":
        anchor = torch.rand(bs, nq, 1, 1, 1, 2, generator=g)
        loc = anchor + (torch.rand(bs, nq, nh, nl, npts, 2, generator=g) - 0.5) * 0.1
    else:
        raise ValueError(kind)
    logits = torch.randn(bs, nq, nh, nl * npts, generator=g)
    attn = torch.softmax(logits, dim=-1).reshape(bs, nq, nh, nl, npts)
    if with_grad_output is None:
        with_grad_output = name.endswith("_bwd")
    grad_out = torch.randn(bs, nq, nh * hd, generator=g) if with_grad_output else None
    cast = lambda t: None if t is None else t.to(dtype)
    return MsdaInputs(cast(value), shapes, lsi, cast(loc), cast(attn), cast(grad_out))


def reference_test_inputs(shape, dtype=torch.float32, seed=0, fill=None):
    """Inputs of the reference's operator test: every level is 60x40, value = U*0.01,
    locations U[0,1), weights U+1e-5 (not normalised), grad_output U*1e-3.
    ``shape`` = [bs, num_queries, embed_dims, num_heads, num_levels, num_points]."""
    bs, nq, hd, nh, nl, npts = shape
    g = torch.Generator().manual_seed(seed)
    shapes, lsi = level_tensors([(60, 40)] * nl)
    nk = int(shapes.prod(1).sum())
    value = torch.rand(bs, nk, nh, hd, generator=g) * 0.01
    loc = torch.rand(bs, nq, nh, nl, npts, 2, generator=g)
    attn = torch.rand(bs, nq, nh, nl, npts, generator=g) + 1e-5
    grad_out = torch.rand(bs, nq, nh * hd, generator=g) * 1e-3
    tensors = [value, loc, attn, grad_out]
    if fill is not None:
        tensors = [torch.full_like(t, fill) for t in tensors]
    value, loc, attn, grad_out = (t.to(dtype) for t in tensors)
    return MsdaInputs(value, shapes, lsi, loc, attn, grad_out)


def algorithmic_bytes(inputs, backward=False):
    """Compulsory HBM bytes of one call: every float input read once and every output
    written once at its storage dtype (the two tiny integer tensors are ignored)."""
    v, loc, attn = inputs.value, inputs.sampling_locations, inputs.attention_weights
    esz = v.element_size()
    bs, nq = loc.shape[0], loc.shape[1]
    out_elems = bs * nq * v.shape[2] * v.shape[3]
    ins = (v.numel() + loc.numel() + attn.numel()) * esz
    if not backward:
        return ins + out_elems * esz
    return ins + out_elems * esz + (v.numel() + loc.numel() + attn.numel()) * esz
