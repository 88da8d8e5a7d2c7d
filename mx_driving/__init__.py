"""Drop-in module path of the reference SDK for the one operator this repository provides
(mx_driving/__init__.py:106-110 of the reference re-exports the same three names)."""
from . import _C  # noqa: F401
from drivingsdk_amd.ops.multi_scale_deformable_attn import (  # noqa: F401
    MultiScaleDeformableAttnFunction,
    multi_scale_deformable_attn,
    npu_multi_scale_deformable_attn_function,
)

from drivingsdk_amd.ops.deformable_aggregation import (  # noqa: F401,E402  (mx_driving/__init__.py:113)
    deformable_aggregation,
    npu_deformable_aggregation,
)
from drivingsdk_amd.ops.geometric_kernel_attention import geometric_kernel_attention  # noqa: F401,E402
from drivingsdk_amd.ops.grid_sampler2d_v2 import grid_sampler2d_v2  # noqa: F401,E402

__all__ = [
    "grid_sampler2d_v2",
    "geometric_kernel_attention",
    "deformable_aggregation",
    "npu_deformable_aggregation",
    "MultiScaleDeformableAttnFunction",
    "multi_scale_deformable_attn",
    "npu_multi_scale_deformable_attn_function",
]
