"""Drop-in module path of the reference SDK for the one operator this repository provides
(mx_driving/__init__.py:106-110 of the reference re-exports the same three names)."""
from drivingsdk_amd import _C  # noqa: F401
from drivingsdk_amd.ops.multi_scale_deformable_attn import (  # noqa: F401
    MultiScaleDeformableAttnFunction,
    multi_scale_deformable_attn,
    npu_multi_scale_deformable_attn_function,
)

__all__ = [
    "MultiScaleDeformableAttnFunction",
    "multi_scale_deformable_attn",
    "npu_multi_scale_deformable_attn_function",
]
