"""Legacy import path (mx_driving/fused.py:7-11 of the reference)."""
from drivingsdk_amd.ops.deformable_aggregation import npu_deformable_aggregation  # noqa: F401
from drivingsdk_amd.ops.multi_scale_deformable_attn import (  # noqa: F401
    multi_scale_deformable_attn,
    npu_multi_scale_deformable_attn_function,
)
