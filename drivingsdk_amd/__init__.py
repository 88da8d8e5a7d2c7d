"""drivingsdk_amd -- multi-scale deformable attention for AMD Instinct MI355X (gfx950).

One operator, behind the reference SDK's own Python API:

    from drivingsdk_amd import multi_scale_deformable_attn
    out = multi_scale_deformable_attn(value, spatial_shapes, level_start_index,
                                      sampling_locations, attention_weights)

``import mx_driving`` (the alias package next to this one) exposes the same names under the
reference's module path.  The compute is hand-written HIP behind a C ABI
(include/mxd_msda.h -> drivingsdk_amd/lib/libmxd_msda.so); there is no CPU fallback.
"""
from . import _C  # noqa: F401
from .ops.multi_scale_deformable_attn import (  # noqa: F401
    MultiScaleDeformableAttnFunction,
    multi_scale_deformable_attn,
    npu_multi_scale_deformable_attn_function,
)

from .ops.deformable_aggregation import (  # noqa: F401,E402
    AdsDeformableAggregation,
    deformable_aggregation,
    npu_deformable_aggregation,
)
from .ops.geometric_kernel_attention import GeometricKernelAttentionFunc, geometric_kernel_attention  # noqa: F401,E402
from .ops.grid_sampler2d_v2 import GridSampler2dV2Function, grid_sampler2d_v2  # noqa: F401,E402
from .ops.msda_fused import (  # noqa: F401,E402
    MultiScaleDeformableAttnFusedFunction,
    multi_scale_deformable_attn_fused,
)

__all__ = [
    "GridSampler2dV2Function",
    "grid_sampler2d_v2",
    "GeometricKernelAttentionFunc",
    "geometric_kernel_attention",
    "AdsDeformableAggregation",
    "deformable_aggregation",
    "npu_deformable_aggregation",
    "MultiScaleDeformableAttnFusedFunction",
    "multi_scale_deformable_attn_fused",
    "MultiScaleDeformableAttnFunction",
    "multi_scale_deformable_attn",
    "npu_multi_scale_deformable_attn_function",
]
