"""Module path of the reference's operator file (mx_driving/ops/multi_scale_deformable_attn.py:18-95)."""
from drivingsdk_amd.ops.multi_scale_deformable_attn import (  # noqa: F401
    MultiScaleDeformableAttnFunction,
    multi_scale_deformable_attn,
    npu_multi_scale_deformable_attn_function,
)
