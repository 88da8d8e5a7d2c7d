"""Module path of the reference's operator file (mx_driving/ops/npu_deformable_aggregation.py:10-88)."""
from drivingsdk_amd.ops.deformable_aggregation import (  # noqa: F401
    AdsDeformableAggregation,
    deformable_aggregation,
    npu_deformable_aggregation,
)
